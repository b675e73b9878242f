#include "jpeg_codec.h"

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>

namespace xad_train {
namespace {

using Bytes = std::vector<unsigned char>;

constexpr std::size_t kMaxPixels = std::size_t(1) << 26;  // 8192 x 8192, the limit of the other readers

// Row-major position in the 8 x 8 block of the k-th coefficient of the zigzag sequence (T.81 figure A.6).
constexpr int kNatural[64] = {0,  1,  8,  16, 9,  2,  3,  10, 17, 24, 32, 25, 18, 11, 4,  5,  12, 19, 26, 33, 40, 48,
                              41, 34, 27, 20, 13, 6,  7,  14, 21, 28, 35, 42, 49, 56, 57, 50, 43, 36, 29, 22, 15, 23,
                              30, 37, 44, 51, 58, 59, 52, 45, 38, 31, 39, 46, 53, 60, 61, 54, 47, 55, 62, 63};

// The orthonormal DCT-II matrix: basis[u][x] = c(u) cos((2x + 1) u pi / 16), c(0) = sqrt(1/8), c(u) = 1/2 otherwise.
// T.81 A.3.3 in matrix form: coefficients = B samples B^T, samples = B^T coefficients B.
struct Basis {
    double at[8][8];
    Basis() {
        const double pi = std::acos(-1.0);
        for (int u = 0; u < 8; ++u)
            for (int x = 0; x < 8; ++x) at[u][x] = (u == 0 ? std::sqrt(0.125) : 0.5) * std::cos((2 * x + 1) * u * pi / 16.0);
    }
};

const Basis& basis() {
    static const Basis b;
    return b;
}

unsigned char clamp_byte(int v) { return static_cast<unsigned char>(v < 0 ? 0 : (v > 255 ? 255 : v)); }

int div_ceil(int a, int b) { return (a + b - 1) / b; }

// ---- reading -------------------------------------------------------------------

// A Huffman table as the canonical code of T.81 annex C: the codes of one length are consecutive.
struct Huffman {
    bool defined = false;
    unsigned first_code[17] = {};  // first code of each length
    int count[17] = {};            // codes of that length
    int first_symbol[17] = {};     // index of that code's symbol
    unsigned char symbol[256] = {};
    std::uint16_t fast[512] = {};  // by the next nine bits: length << 8 | symbol, 0 = longer than nine bits

    bool build(const unsigned char* counts, const unsigned char* symbols, int total) {
        unsigned code = 0;
        int index = 0;
        std::memset(fast, 0, sizeof fast);
        for (int length = 1; length <= 16; ++length) {
            first_code[length] = code;
            count[length] = counts[length - 1];
            first_symbol[length] = index;
            if (code + static_cast<unsigned>(count[length]) > (1u << length)) return false;  // more codes than the length holds
            for (int i = 0; i < count[length]; ++i, ++index, ++code) {
                symbol[index] = symbols[index];
                if (length <= 9)
                    for (unsigned pad = 0; pad < (1u << (9 - length)); ++pad)
                        fast[(code << (9 - length)) | pad] = static_cast<std::uint16_t>((length << 8) | symbols[index]);
            }
            code <<= 1;
        }
        defined = index == total;
        return defined;
    }
};

// The bits of one entropy-coded segment, most significant first.  A stuffed zero after 0xFF is dropped; at a
// marker the reader stops taking bytes, stays in front of it and hands out zeros.
class BitReader {
   public:
    BitReader(const unsigned char* begin, const unsigned char* end) : p_(begin), end_(end) {}

    unsigned bits(int n) {  // n <= 16
        if (n == 0) return 0;
        if (have_ < n) fill();
        const unsigned v = acc_ >> (32 - n);
        acc_ <<= n;
        have_ -= n;
        return v;
    }

    // Next symbol of a Huffman table, or -1 when the bits are no code of it.
    int symbol(const Huffman& h) {
        if (have_ < 16) fill();
        if (const unsigned entry = h.fast[acc_ >> 23]) {
            const int length = static_cast<int>(entry >> 8);
            acc_ <<= length;
            have_ -= length;
            return static_cast<int>(entry & 255u);
        }
        const unsigned window = acc_ >> 16;
        for (int length = 10; length <= 16; ++length) {
            const unsigned offset = (window >> (16 - length)) - h.first_code[length];
            if (offset < static_cast<unsigned>(h.count[length])) {
                acc_ <<= length;
                have_ -= length;
                return h.symbol[h.first_symbol[length] + static_cast<int>(offset)];
            }
        }
        return -1;
    }

    // A value of `size` bits in the sign convention of T.81 F.2.2.1 (figure F.12).
    int extended(int size) {
        if (size == 0) return 0;
        const int v = static_cast<int>(bits(size));
        return v < (1 << (size - 1)) ? v - (1 << size) + 1 : v;
    }

    // At a restart interval's end: drops the padding bits and steps over the restart marker.  False if
    // something else than a restart marker follows.
    bool restart() {
        acc_ = 0;
        have_ = 0;
        if (marker_ == 0) {  // the marker was not met yet: it has to be next
            while (p_ + 1 < end_ && !(p_[0] == 0xFF && p_[1] != 0 && p_[1] != 0xFF)) ++p_;
            if (p_ + 1 >= end_) return false;
            marker_ = p_[1];
        }
        if (marker_ < 0xD0 || marker_ > 0xD7) return false;
        p_ += 2;
        marker_ = 0;
        return true;
    }

    // Whether bits were handed out that the file does not hold (bits fetched ahead and never used do not count).
    bool starved() const { return phantom_ > have_; }
    const unsigned char* position() const { return p_; }

   private:
    void fill() {
        while (have_ <= 24) {
            unsigned byte = 0;
            if (marker_ == 0) {
                if (p_ >= end_) {
                    phantom_ += 8;
                } else if (*p_ != 0xFF) {
                    byte = *p_++;
                } else {
                    const unsigned char* q = p_ + 1;
                    while (q < end_ && *q == 0xFF) ++q;  // fill bytes in front of a marker
                    if (q >= end_) {
                        phantom_ += 8;
                        p_ = end_;
                    } else if (*q == 0) {
                        byte = 0xFF;
                        p_ = q + 1;
                    } else {
                        marker_ = *q;
                        p_ = q - 1;
                    }
                }
            }
            acc_ |= byte << (24 - have_);
            have_ += 8;
        }
    }

    const unsigned char* p_;
    const unsigned char* end_;
    std::uint32_t acc_ = 0;
    int have_ = 0;
    int marker_ = 0;
    int phantom_ = 0;  // bits of zeros taken in beyond the end of the file
};

struct Component {
    int id = 0, h = 1, v = 1, table = 0;
    int dc_table = 0, ac_table = 0;  // of the current scan
    int width = 0, height = 0;       // samples
    int blocks_x = 0, blocks_y = 0;  // blocks that hold samples: what a scan of this component alone covers
    int stride = 0, rows = 0;        // blocks stored: whole minimum coded units
    std::vector<short> coefficients; // rows x stride x 64, block-row-major positions
    int prediction = 0;
    short* block(int bx, int by) { return coefficients.data() + (static_cast<std::size_t>(by) * stride + bx) * 64; }
};

class Decoder {
   public:
    explicit Decoder(const Bytes& file) : file_(file) {}

    std::string run(Image& out) {
        std::size_t pos = 2;
        for (;;) {
            while (pos < file_.size() && file_[pos] != 0xFF) ++pos;  // tolerate stray bytes between segments
            while (pos < file_.size() && file_[pos] == 0xFF) ++pos;
            if (pos >= file_.size()) break;  // no end-of-image marker: take what was decoded
            const int marker = file_[pos++];
            if (marker == 0xD9) break;
            if (marker == 0xD8 || marker == 0x01 || marker == 0x00 || (marker >= 0xD0 && marker <= 0xD7)) continue;
            if (pos + 2 > file_.size()) return "JPEG: truncated file";
            const std::size_t length = (std::size_t(file_[pos]) << 8) | file_[pos + 1];
            if (length < 2 || length > file_.size() - pos) return "JPEG: segment runs past the end of the file";
            const unsigned char* data = &file_[pos + 2];
            const std::size_t size = length - 2;
            std::string err;
            switch (marker) {
                case 0xC0: case 0xC1: case 0xC2: err = frame_header(data, size, marker == 0xC2); break;
                case 0xC3: case 0xC5: case 0xC6: case 0xC7: case 0xCB: case 0xCD: case 0xCE: case 0xCF:
                    return "JPEG: lossless and hierarchical files are not supported";
                case 0xC9: case 0xCA: return "JPEG: arithmetic coding is not supported";
                case 0xC4: err = huffman_tables(data, size); break;
                case 0xDB: err = quantisation_tables(data, size); break;
                case 0xDD:
                    if (size != 2) return "JPEG: bad restart interval segment";
                    restart_interval_ = (int(data[0]) << 8) | data[1];
                    break;
                case 0xDA: {
                    const unsigned char* next = nullptr;
                    err = scan(data, size, &next);
                    if (err.empty()) {
                        pos = static_cast<std::size_t>(next - file_.data());
                        continue;
                    }
                    break;
                }
                case 0xE0: if (size >= 5 && !std::memcmp(data, "JFIF", 5)) jfif_ = true; break;
                case 0xEE:
                    if (size >= 12 && !std::memcmp(data, "Adobe", 5)) {
                        adobe_ = true;
                        adobe_transform_ = data[11];
                    }
                    break;
                case 0xDC: return "JPEG: a line count after the first scan is not supported";
                default: break;  // other application segments and comments
            }
            if (!err.empty()) return err;
            pos += length;
        }
        if (components_.empty()) return "JPEG: no frame header";
        if (scans_ == 0) return "JPEG: no scan";
        return reconstruct(out);
    }

   private:
    std::string frame_header(const unsigned char* d, std::size_t size, bool progressive) {
        if (!components_.empty()) return "JPEG: more than one frame";
        if (size < 6) return "JPEG: bad frame header";
        if (d[0] != 8) return "JPEG: only 8-bit samples are supported";
        height_ = (int(d[1]) << 8) | d[2];
        width_ = (int(d[3]) << 8) | d[4];
        const int count = d[5];
        if (width_ == 0 || height_ == 0) return "JPEG: empty image, or a line count that follows the first scan";
        if (std::size_t(width_) * std::size_t(height_) > kMaxPixels) return "JPEG: unreasonable image size";
        if (count == 4) return "JPEG: four-component (CMYK) files are not supported";
        if (count != 1 && count != 3) return "JPEG: one or three components expected";
        if (size != std::size_t(6 + 3 * count)) return "JPEG: bad frame header";
        progressive_ = progressive;
        components_.resize(count);
        h_max_ = v_max_ = 1;
        for (int i = 0; i < count; ++i) {
            Component& c = components_[i];
            c.id = d[6 + 3 * i];
            c.h = d[7 + 3 * i] >> 4;
            c.v = d[7 + 3 * i] & 15;
            c.table = d[8 + 3 * i];
            if (c.h < 1 || c.h > 4 || c.v < 1 || c.v > 4 || c.table > 3) return "JPEG: bad component description";
            h_max_ = std::max(h_max_, c.h);
            v_max_ = std::max(v_max_, c.v);
        }
        if (count == 1) components_[0].h = components_[0].v = h_max_ = v_max_ = 1;  // one component: its factors mean nothing
        mcus_x_ = div_ceil(width_, 8 * h_max_);
        mcus_y_ = div_ceil(height_, 8 * v_max_);
        for (Component& c : components_) {
            if (h_max_ % c.h || v_max_ % c.v) return "JPEG: fractional sampling ratios are not supported";
            c.width = div_ceil(width_ * c.h, h_max_);
            c.height = div_ceil(height_ * c.v, v_max_);
            c.blocks_x = div_ceil(c.width, 8);
            c.blocks_y = div_ceil(c.height, 8);
            c.stride = mcus_x_ * c.h;
            c.rows = mcus_y_ * c.v;
            c.coefficients.assign(static_cast<std::size_t>(c.stride) * c.rows * 64, 0);
        }
        return "";
    }

    std::string huffman_tables(const unsigned char* d, std::size_t size) {
        while (size > 0) {
            if (size < 17) return "JPEG: bad Huffman table segment";
            const int kind = d[0] >> 4, slot = d[0] & 15;
            if (kind > 1 || slot > 3) return "JPEG: bad Huffman table number";
            int total = 0;
            for (int i = 0; i < 16; ++i) total += d[1 + i];
            if (total > 256 || size < std::size_t(17 + total)) return "JPEG: bad Huffman table segment";
            if (!huffman_[kind][slot].build(d + 1, d + 17, total)) return "JPEG: Huffman table is not a prefix code";
            d += 17 + total;
            size -= 17 + total;
        }
        return "";
    }

    std::string quantisation_tables(const unsigned char* d, std::size_t size) {
        while (size > 0) {
            const int wide = d[0] >> 4, slot = d[0] & 15;
            if (wide > 1 || slot > 3) return "JPEG: bad quantisation table number";
            const std::size_t bytes = wide ? 128 : 64;
            if (size < 1 + bytes) return "JPEG: bad quantisation table segment";
            for (int k = 0; k < 64; ++k)
                quantiser_[slot][kNatural[k]] = wide ? (int(d[1 + 2 * k]) << 8) | d[2 + 2 * k] : d[1 + k];
            quantiser_defined_[slot] = true;
            d += 1 + bytes;
            size -= 1 + bytes;
        }
        return "";
    }

    // One scan: its header, then the entropy-coded data up to the next marker that is no restart marker.
    std::string scan(const unsigned char* d, std::size_t size, const unsigned char** next) {
        if (components_.empty()) return "JPEG: scan before the frame header";
        if (size < 1) return "JPEG: bad scan header";
        const int count = d[0];
        if (count < 1 || count > static_cast<int>(components_.size()) || size != std::size_t(4 + 2 * count))
            return "JPEG: bad scan header";
        std::vector<Component*> members;
        for (int i = 0; i < count; ++i) {
            Component* found = nullptr;
            for (Component& c : components_)
                if (c.id == d[1 + 2 * i]) found = &c;
            if (!found || std::find(members.begin(), members.end(), found) != members.end())
                return "JPEG: scan names a component the frame does not have";
            found->dc_table = d[2 + 2 * i] >> 4;
            found->ac_table = d[2 + 2 * i] & 15;
            if (found->dc_table > 3 || found->ac_table > 3) return "JPEG: bad Huffman table number";
            members.push_back(found);
        }
        int first = d[1 + 2 * count], last = d[2 + 2 * count];
        int high = d[3 + 2 * count] >> 4, low = d[3 + 2 * count] & 15;
        if (!progressive_) {
            first = 0, last = 63, high = 0, low = 0;
        } else {
            if (first > last || last > 63 || (first == 0 && last != 0) || (first != 0 && count != 1) || low > 13 || high > 13)
                return "JPEG: bad progressive scan parameters";
        }
        const bool needs_dc = first == 0 && high == 0, needs_ac = last > 0;
        for (Component* c : members) {
            if (needs_dc && !huffman_[0][c->dc_table].defined) return "JPEG: scan uses a Huffman table that was not defined";
            if (needs_ac && !huffman_[1][c->ac_table].defined) return "JPEG: scan uses a Huffman table that was not defined";
            c->prediction = 0;
        }

        BitReader reader(d + size, file_.data() + file_.size());
        int end_of_band_run = 0;
        bool corrupt = false;
        // the units of the scan: whole minimum coded units when several components are interleaved, else the
        // blocks of the one component that hold samples (T.81 A.2)
        const bool interleaved = count > 1;
        const int units_x = interleaved ? mcus_x_ : members[0]->blocks_x;
        const int units_y = interleaved ? mcus_y_ : members[0]->blocks_y;
        const long long units = static_cast<long long>(units_x) * units_y;
        int until_restart = restart_interval_;
        for (long long unit = 0; unit < units && !corrupt; ++unit) {
            const int ux = static_cast<int>(unit % units_x), uy = static_cast<int>(unit / units_x);
            for (Component* c : members) {
                const int across = interleaved ? c->h : 1, down = interleaved ? c->v : 1;
                for (int by = 0; by < down && !corrupt; ++by)
                    for (int bx = 0; bx < across && !corrupt; ++bx) {
                        short* block = c->block(ux * across + bx, uy * down + by);
                        bool ok;
                        if (!progressive_)
                            ok = sequential_block(reader, *c, block);
                        else if (first == 0)
                            ok = high == 0 ? dc_first(reader, *c, block, low) : dc_refine(reader, block, low);
                        else
                            ok = high == 0 ? ac_first(reader, *c, block, first, last, low, end_of_band_run)
                                           : ac_refine(reader, *c, block, first, last, low, end_of_band_run);
                        corrupt = !ok;
                    }
            }
            if (reader.starved()) return "JPEG: file ends inside the compressed data";
            if (restart_interval_ > 0 && --until_restart == 0 && unit + 1 < units) {
                if (!reader.restart()) return "JPEG: restart marker missing";
                until_restart = restart_interval_;
                end_of_band_run = 0;
                for (Component* c : members) c->prediction = 0;
            }
        }
        if (corrupt) return "JPEG: corrupt entropy-coded data";
        ++scans_;
        *next = reader.position();
        return "";
    }

    bool sequential_block(BitReader& r, Component& c, short* block) {
        const int size = r.symbol(huffman_[0][c.dc_table]);
        if (size < 0 || size > 15) return false;
        c.prediction += r.extended(size);
        block[0] = static_cast<short>(c.prediction);
        const Huffman& ac = huffman_[1][c.ac_table];
        for (int k = 1; k < 64;) {
            const int rs = r.symbol(ac);
            if (rs < 0) return false;
            const int run = rs >> 4, bits = rs & 15;
            if (bits == 0) {
                if (run != 15) break;  // end of block
                k += 16;
                continue;
            }
            k += run;
            if (k > 63) return false;
            block[kNatural[k++]] = static_cast<short>(r.extended(bits));
        }
        return true;
    }

    // Progressive scans, T.81 annex G.  `low` is the point transform (the scan carries the coefficients
    // divided by 2^low); a refinement scan adds one more bit to what earlier scans left.
    bool dc_first(BitReader& r, Component& c, short* block, int low) {
        const int size = r.symbol(huffman_[0][c.dc_table]);
        if (size < 0 || size > 15) return false;
        c.prediction += r.extended(size);
        block[0] = static_cast<short>(c.prediction * (1 << low));
        return true;
    }

    bool dc_refine(BitReader& r, short* block, int low) {
        if (r.bits(1)) block[0] = static_cast<short>(block[0] | (1 << low));
        return true;
    }

    bool ac_first(BitReader& r, Component& c, short* block, int first, int last, int low, int& end_of_band_run) {
        if (end_of_band_run > 0) {
            --end_of_band_run;
            return true;
        }
        const Huffman& ac = huffman_[1][c.ac_table];
        for (int k = first; k <= last;) {
            const int rs = r.symbol(ac);
            if (rs < 0) return false;
            const int run = rs >> 4, bits = rs & 15;
            if (bits == 0) {
                if (run < 15) {  // this band ends here in this block and in the next 2^run + ... - 1 blocks
                    end_of_band_run = (1 << run) - 1;
                    if (run) end_of_band_run += static_cast<int>(r.bits(run));
                    break;
                }
                k += 16;
                continue;
            }
            k += run;
            if (k > last) return false;
            block[kNatural[k++]] = static_cast<short>(r.extended(bits) * (1 << low));
        }
        return true;
    }

    // One more bit for a coefficient that is already nonzero: its magnitude grows by 2^low if the bit is set.
    static void correct(BitReader& r, short& coefficient, int low) {
        if (!r.bits(1)) return;
        const int bit = 1 << low;
        if ((coefficient & bit) == 0) coefficient = static_cast<short>(coefficient >= 0 ? coefficient + bit : coefficient - bit);
    }

    bool ac_refine(BitReader& r, Component& c, short* block, int first, int last, int low, int& end_of_band_run) {
        const Huffman& ac = huffman_[1][c.ac_table];
        int k = first;
        if (end_of_band_run == 0) {
            for (; k <= last; ++k) {
                const int rs = r.symbol(ac);
                if (rs < 0) return false;
                int run = rs >> 4;
                const int bits = rs & 15;
                int fresh = 0;  // a coefficient that becomes nonzero in this scan: plus or minus 2^low
                if (bits == 1) {
                    fresh = r.bits(1) ? (1 << low) : -(1 << low);
                } else if (bits != 0) {
                    return false;
                } else if (run != 15) {
                    end_of_band_run = 1 << run;
                    if (run) end_of_band_run += static_cast<int>(r.bits(run));
                    break;
                }
                // step over `run` coefficients that are still zero; the nonzero ones on the way get their bit
                for (; k <= last; ++k) {
                    short& coefficient = block[kNatural[k]];
                    if (coefficient != 0)
                        correct(r, coefficient, low);
                    else if (--run < 0)
                        break;
                }
                if (fresh) {
                    if (k > last) return false;
                    block[kNatural[k]] = static_cast<short>(fresh);
                }
            }
        }
        if (end_of_band_run > 0) {  // the rest of the band holds no new coefficients: only correction bits
            for (; k <= last; ++k) {
                short& coefficient = block[kNatural[k]];
                if (coefficient != 0) correct(r, coefficient, low);
            }
            --end_of_band_run;
        }
        return true;
    }

    // Samples of one component from its coefficients: dequantise, inverse transform, level shift.
    std::string samples_of(Component& c, std::vector<unsigned char>& plane) const {
        if (!quantiser_defined_[c.table]) return "JPEG: component uses a quantisation table that was not defined";
        const int* q = quantiser_[c.table];
        const Basis& b = basis();
        const int plane_width = c.stride * 8;
        plane.assign(static_cast<std::size_t>(plane_width) * c.rows * 8, 0);
        for (int by = 0; by < c.blocks_y; ++by)
            for (int bx = 0; bx < c.blocks_x; ++bx) {
                const short* block = c.block(bx, by);
                double f[64];
                int last_row = -1;
                for (int v = 0; v < 8; ++v)
                    for (int u = 0; u < 8; ++u) {
                        f[v * 8 + u] = static_cast<double>(block[v * 8 + u]) * q[v * 8 + u];
                        if (block[v * 8 + u] != 0) last_row = v;
                    }
                double half[64];  // rows transformed: half[v][x] = sum over u of f[v][u] basis[u][x]
                for (int v = 0; v <= last_row; ++v)
                    for (int x = 0; x < 8; ++x) {
                        double sum = 0.0;
                        for (int u = 0; u < 8; ++u) sum += f[v * 8 + u] * b.at[u][x];
                        half[v * 8 + x] = sum;
                    }
                unsigned char* to = plane.data() + (static_cast<std::size_t>(by) * 8) * plane_width + bx * 8;
                for (int y = 0; y < 8; ++y)
                    for (int x = 0; x < 8; ++x) {
                        double sum = 128.0;
                        for (int v = 0; v <= last_row; ++v) sum += b.at[v][y] * half[v * 8 + x];
                        to[static_cast<std::size_t>(y) * plane_width + x] = clamp_byte(static_cast<int>(std::floor(sum + 0.5)));
                    }
            }
        return "";
    }

    // The component at the frame's resolution.  A ratio of two is interpolated between the centres of the
    // component's samples (weights 3/4 and 1/4, edges repeated), in both directions at once with a single
    // rounding; any other ratio repeats samples.
    void full_resolution(const Component& c, const std::vector<unsigned char>& plane, std::vector<unsigned char>& full) const {
        const int fx = h_max_ / c.h, fy = v_max_ / c.v;
        const int plane_width = c.stride * 8;
        full.resize(static_cast<std::size_t>(width_) * height_);
        for (int y = 0; y < height_; ++y) {
            int near_row = y / fy, far_row = near_row;
            if (fy == 2) far_row = std::clamp(near_row + ((y & 1) ? 1 : -1), 0, c.height - 1);
            const unsigned char* a = plane.data() + static_cast<std::size_t>(near_row) * plane_width;
            const unsigned char* b = plane.data() + static_cast<std::size_t>(far_row) * plane_width;
            unsigned char* to = full.data() + static_cast<std::size_t>(y) * width_;
            for (int x = 0; x < width_; ++x) {
                int near_col = x / fx, far_col = near_col;
                if (fx == 2) far_col = std::clamp(near_col + ((x & 1) ? 1 : -1), 0, c.width - 1);
                const int near_sum = 3 * a[near_col] + b[near_col], far_sum = 3 * a[far_col] + b[far_col];  // times 4
                to[x] = static_cast<unsigned char>((3 * near_sum + far_sum + 8) >> 4);
            }
        }
    }

    std::string reconstruct(Image& out) {
        std::vector<std::vector<unsigned char>> full(components_.size());
        for (std::size_t i = 0; i < components_.size(); ++i) {
            std::vector<unsigned char> plane;
            if (std::string err = samples_of(components_[i], plane); !err.empty()) return err;
            full_resolution(components_[i], plane, full[i]);
            components_[i].coefficients = std::vector<short>();
        }
        out.width = width_;
        out.height = height_;
        const std::size_t pixels = static_cast<std::size_t>(width_) * height_;
        out.rgb.resize(pixels * 3);
        // three components are YCbCr when the file is a JFIF file; otherwise an Adobe segment says which, and
        // without either the component names do
        bool ycc = components_.size() == 3;
        if (ycc && !jfif_) {
            if (adobe_)
                ycc = adobe_transform_ != 0;
            else if (components_[0].id == 'R' && components_[1].id == 'G' && components_[2].id == 'B')
                ycc = false;
        }
        for (std::size_t i = 0; i < pixels; ++i) {
            int rgb[3];
            if (components_.size() == 1) {
                rgb[0] = rgb[1] = rgb[2] = full[0][i];
            } else if (!ycc) {
                for (int k = 0; k < 3; ++k) rgb[k] = full[k][i];
            } else {  // T.871 section 7
                const double luma = full[0][i], cb = full[1][i] - 128.0, cr = full[2][i] - 128.0;
                rgb[0] = static_cast<int>(std::floor(luma + 1.402 * cr + 0.5));
                rgb[1] = static_cast<int>(std::floor(luma - 0.344136286 * cb - 0.714136286 * cr + 0.5));
                rgb[2] = static_cast<int>(std::floor(luma + 1.772 * cb + 0.5));
            }
            for (int k = 0; k < 3; ++k) out.rgb[i * 3 + k] = clamp_byte(rgb[k]) / 255.0f;
        }
        return "";
    }

    const Bytes& file_;
    int width_ = 0, height_ = 0, h_max_ = 1, v_max_ = 1, mcus_x_ = 0, mcus_y_ = 0;
    bool progressive_ = false, jfif_ = false, adobe_ = false;
    int adobe_transform_ = 0;
    int restart_interval_ = 0;
    int scans_ = 0;
    std::vector<Component> components_;
    Huffman huffman_[2][4];  // [0] = DC, [1] = AC
    int quantiser_[4][64] = {};
    bool quantiser_defined_[4] = {false, false, false, false};
};

// ---- writing -------------------------------------------------------------------

// T.81 annex K.1, row-major.
constexpr int kLuminanceQuantiser[64] = {16, 11, 10, 16, 24,  40,  51,  61,  12, 12, 14, 19, 26,  58,  60,  55,
                                         14, 13, 16, 24, 40,  57,  69,  56,  14, 17, 22, 29, 51,  87,  80,  62,
                                         18, 22, 37, 56, 68,  109, 103, 77,  24, 35, 55, 64, 81,  104, 113, 92,
                                         49, 64, 78, 87, 103, 121, 120, 101, 72, 92, 95, 98, 112, 100, 103, 99};
constexpr int kChrominanceQuantiser[64] = {17, 18, 24, 47, 99, 99, 99, 99, 18, 21, 26, 66, 99, 99, 99, 99,
                                           24, 26, 56, 99, 99, 99, 99, 99, 47, 66, 99, 99, 99, 99, 99, 99,
                                           99, 99, 99, 99, 99, 99, 99, 99, 99, 99, 99, 99, 99, 99, 99, 99,
                                           99, 99, 99, 99, 99, 99, 99, 99, 99, 99, 99, 99, 99, 99, 99, 99};

// T.81 annex K.3: codes per length, then the symbols in order of increasing code.
struct CodeList {
    unsigned char counts[16];
    std::vector<unsigned char> symbols;
};

const CodeList& standard_codes(int kind, int chroma) {
    static const CodeList lists[2][2] = {
        {{{0, 1, 5, 1, 1, 1, 1, 1, 1, 0, 0, 0, 0, 0, 0, 0}, {0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11}},
         {{0, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 0, 0, 0, 0, 0}, {0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11}}},
        {{{0, 2, 1, 3, 3, 2, 4, 3, 5, 5, 4, 4, 0, 0, 1, 0x7d},
          {0x01, 0x02, 0x03, 0x00, 0x04, 0x11, 0x05, 0x12, 0x21, 0x31, 0x41, 0x06, 0x13, 0x51, 0x61, 0x07, 0x22, 0x71,
           0x14, 0x32, 0x81, 0x91, 0xa1, 0x08, 0x23, 0x42, 0xb1, 0xc1, 0x15, 0x52, 0xd1, 0xf0, 0x24, 0x33, 0x62, 0x72,
           0x82, 0x09, 0x0a, 0x16, 0x17, 0x18, 0x19, 0x1a, 0x25, 0x26, 0x27, 0x28, 0x29, 0x2a, 0x34, 0x35, 0x36, 0x37,
           0x38, 0x39, 0x3a, 0x43, 0x44, 0x45, 0x46, 0x47, 0x48, 0x49, 0x4a, 0x53, 0x54, 0x55, 0x56, 0x57, 0x58, 0x59,
           0x5a, 0x63, 0x64, 0x65, 0x66, 0x67, 0x68, 0x69, 0x6a, 0x73, 0x74, 0x75, 0x76, 0x77, 0x78, 0x79, 0x7a, 0x83,
           0x84, 0x85, 0x86, 0x87, 0x88, 0x89, 0x8a, 0x92, 0x93, 0x94, 0x95, 0x96, 0x97, 0x98, 0x99, 0x9a, 0xa2, 0xa3,
           0xa4, 0xa5, 0xa6, 0xa7, 0xa8, 0xa9, 0xaa, 0xb2, 0xb3, 0xb4, 0xb5, 0xb6, 0xb7, 0xb8, 0xb9, 0xba, 0xc2, 0xc3,
           0xc4, 0xc5, 0xc6, 0xc7, 0xc8, 0xc9, 0xca, 0xd2, 0xd3, 0xd4, 0xd5, 0xd6, 0xd7, 0xd8, 0xd9, 0xda, 0xe1, 0xe2,
           0xe3, 0xe4, 0xe5, 0xe6, 0xe7, 0xe8, 0xe9, 0xea, 0xf1, 0xf2, 0xf3, 0xf4, 0xf5, 0xf6, 0xf7, 0xf8, 0xf9, 0xfa}},
         {{0, 2, 1, 2, 4, 4, 3, 4, 7, 5, 4, 4, 0, 1, 2, 0x77},
          {0x00, 0x01, 0x02, 0x03, 0x11, 0x04, 0x05, 0x21, 0x31, 0x06, 0x12, 0x41, 0x51, 0x07, 0x61, 0x71, 0x13, 0x22,
           0x32, 0x81, 0x08, 0x14, 0x42, 0x91, 0xa1, 0xb1, 0xc1, 0x09, 0x23, 0x33, 0x52, 0xf0, 0x15, 0x62, 0x72, 0xd1,
           0x0a, 0x16, 0x24, 0x34, 0xe1, 0x25, 0xf1, 0x17, 0x18, 0x19, 0x1a, 0x26, 0x27, 0x28, 0x29, 0x2a, 0x35, 0x36,
           0x37, 0x38, 0x39, 0x3a, 0x43, 0x44, 0x45, 0x46, 0x47, 0x48, 0x49, 0x4a, 0x53, 0x54, 0x55, 0x56, 0x57, 0x58,
           0x59, 0x5a, 0x63, 0x64, 0x65, 0x66, 0x67, 0x68, 0x69, 0x6a, 0x73, 0x74, 0x75, 0x76, 0x77, 0x78, 0x79, 0x7a,
           0x82, 0x83, 0x84, 0x85, 0x86, 0x87, 0x88, 0x89, 0x8a, 0x92, 0x93, 0x94, 0x95, 0x96, 0x97, 0x98, 0x99, 0x9a,
           0xa2, 0xa3, 0xa4, 0xa5, 0xa6, 0xa7, 0xa8, 0xa9, 0xaa, 0xb2, 0xb3, 0xb4, 0xb5, 0xb6, 0xb7, 0xb8, 0xb9, 0xba,
           0xc2, 0xc3, 0xc4, 0xc5, 0xc6, 0xc7, 0xc8, 0xc9, 0xca, 0xd2, 0xd3, 0xd4, 0xd5, 0xd6, 0xd7, 0xd8, 0xd9, 0xda,
           0xe2, 0xe3, 0xe4, 0xe5, 0xe6, 0xe7, 0xe8, 0xe9, 0xea, 0xf2, 0xf3, 0xf4, 0xf5, 0xf6, 0xf7, 0xf8, 0xf9, 0xfa}}}};
    return lists[kind][chroma];
}

struct Encoding {
    unsigned code[256] = {};
    int length[256] = {};
    explicit Encoding(const CodeList& list) {
        unsigned next = 0;
        std::size_t index = 0;
        for (int bits = 1; bits <= 16; ++bits) {
            for (int i = 0; i < list.counts[bits - 1]; ++i, ++index) {
                code[list.symbols[index]] = next++;
                length[list.symbols[index]] = bits;
            }
            next <<= 1;
        }
    }
};

class BitWriter {
   public:
    explicit BitWriter(Bytes& out) : out_(out) {}
    void put(unsigned value, int bits) {
        acc_ = (acc_ << bits) | (value & ((1u << bits) - 1u));
        have_ += bits;
        while (have_ >= 8) {
            const unsigned char byte = static_cast<unsigned char>(acc_ >> (have_ - 8));
            out_.push_back(byte);
            if (byte == 0xFF) out_.push_back(0);  // so that data never looks like a marker
            have_ -= 8;
        }
    }
    void finish() {
        if (have_ > 0) put(0xFFu, 8 - have_);  // pad with ones
    }

   private:
    Bytes& out_;
    std::uint32_t acc_ = 0;
    int have_ = 0;
};

int magnitude_bits(int v) {
    int a = v < 0 ? -v : v, bits = 0;
    while (a) {
        ++bits;
        a >>= 1;
    }
    return bits;
}

void put_value(BitWriter& w, int v, int bits) {
    if (bits) w.put(static_cast<unsigned>(v < 0 ? v - 1 : v), bits);  // negative values as v - 1 in `bits` bits
}

void put_marker(Bytes& out, int marker, std::size_t payload) {
    out.push_back(0xFF);
    out.push_back(static_cast<unsigned char>(marker));
    out.push_back(static_cast<unsigned char>((payload + 2) >> 8));
    out.push_back(static_cast<unsigned char>((payload + 2) & 255));
}

// One 8 x 8 block of a plane: transform, quantise, entropy-code.
void encode_block(BitWriter& w, const float* plane, int plane_width, int x0, int y0, const int* quantiser, const Encoding& dc,
                  const Encoding& ac, int& prediction) {
    const Basis& b = basis();
    double half[64], f;
    for (int y = 0; y < 8; ++y)
        for (int u = 0; u < 8; ++u) {
            double sum = 0.0;
            for (int x = 0; x < 8; ++x) sum += (plane[static_cast<std::size_t>(y0 + y) * plane_width + x0 + x] - 128.0) * b.at[u][x];
            half[y * 8 + u] = sum;
        }
    int quantised[64];
    for (int v = 0; v < 8; ++v)
        for (int u = 0; u < 8; ++u) {
            f = 0.0;
            for (int y = 0; y < 8; ++y) f += b.at[v][y] * half[y * 8 + u];
            const double scaled = f / quantiser[v * 8 + u];
            quantised[v * 8 + u] = static_cast<int>(scaled < 0 ? -std::floor(-scaled + 0.5) : std::floor(scaled + 0.5));
        }
    const int difference = quantised[0] - prediction;
    prediction = quantised[0];
    const int size = magnitude_bits(difference);
    w.put(dc.code[size], dc.length[size]);
    put_value(w, difference, size);
    int run = 0;
    for (int k = 1; k < 64; ++k) {
        const int v = quantised[kNatural[k]];
        if (v == 0) {
            ++run;
            continue;
        }
        for (; run >= 16; run -= 16) w.put(ac.code[0xF0], ac.length[0xF0]);
        const int bits = magnitude_bits(v);
        w.put(ac.code[(run << 4) | bits], ac.length[(run << 4) | bits]);
        put_value(w, v, bits);
        run = 0;
    }
    if (run) w.put(ac.code[0], ac.length[0]);  // end of block
}

}  // namespace

std::string decode_jpeg(const Bytes& file, Image& out) {
    if (file.size() < 4 || file[0] != 0xFF || file[1] != 0xD8) return "JPEG: missing start-of-image marker";
    return Decoder(file).run(out);
}

std::string encode_jpeg(int width, int height, const Bytes& rgb8, int quality, Bytes& out) {
    if (width <= 0 || height <= 0 || width > 65535 || height > 65535) return "JPEG: image size must be within 1..65535";
    if (rgb8.size() != static_cast<std::size_t>(width) * height * 3) return "JPEG: pixel buffer does not match the size";
    quality = std::clamp(quality, 1, 100);
    const int scale = quality < 50 ? 5000 / quality : 200 - 2 * quality;
    int quantiser[2][64];
    for (int i = 0; i < 64; ++i) {
        quantiser[0][i] = std::clamp((kLuminanceQuantiser[i] * scale + 50) / 100, 1, 255);
        quantiser[1][i] = std::clamp((kChrominanceQuantiser[i] * scale + 50) / 100, 1, 255);
    }
    const int ratio = quality <= 90 ? 2 : 1;  // luminance samples per chrominance sample, each way
    const int unit = 8 * ratio;
    const int mcus_x = div_ceil(width, unit), mcus_y = div_ceil(height, unit);
    const int padded_w = mcus_x * unit, padded_h = mcus_y * unit;

    // YCbCr (T.871 section 7) at full resolution, edges repeated up to whole coding units
    std::vector<float> planes[3];
    for (auto& p : planes) p.resize(static_cast<std::size_t>(padded_w) * padded_h);
    for (int y = 0; y < padded_h; ++y)
        for (int x = 0; x < padded_w; ++x) {
            const unsigned char* px = &rgb8[(static_cast<std::size_t>(std::min(y, height - 1)) * width + std::min(x, width - 1)) * 3];
            const float r = px[0], g = px[1], b = px[2];
            const std::size_t at = static_cast<std::size_t>(y) * padded_w + x;
            planes[0][at] = 0.299f * r + 0.587f * g + 0.114f * b;
            planes[1][at] = -0.168735892f * r - 0.331264108f * g + 0.5f * b + 128.0f;
            planes[2][at] = 0.5f * r - 0.418687589f * g - 0.081312411f * b + 128.0f;
        }
    const int chroma_w = padded_w / ratio, chroma_h = padded_h / ratio;
    if (ratio == 2)
        for (int k = 1; k < 3; ++k) {
            std::vector<float> half(static_cast<std::size_t>(chroma_w) * chroma_h);
            const std::vector<float>& from = planes[k];
            for (int y = 0; y < chroma_h; ++y)
                for (int x = 0; x < chroma_w; ++x) {
                    const std::size_t at = static_cast<std::size_t>(2 * y) * padded_w + 2 * x;
                    half[static_cast<std::size_t>(y) * chroma_w + x] = 0.25f * ((from[at] + from[at + 1]) + (from[at + padded_w] + from[at + padded_w + 1]));
                }
            planes[k].swap(half);
        }

    out.clear();
    out.push_back(0xFF);
    out.push_back(0xD8);
    put_marker(out, 0xE0, 14);
    const unsigned char jfif[14] = {'J', 'F', 'I', 'F', 0, 1, 1, 0, 0, 1, 0, 1, 0, 0};  // version 1.1, aspect 1:1, no thumbnail
    out.insert(out.end(), jfif, jfif + 14);
    for (int t = 0; t < 2; ++t) {
        put_marker(out, 0xDB, 65);
        out.push_back(static_cast<unsigned char>(t));
        for (int k = 0; k < 64; ++k) out.push_back(static_cast<unsigned char>(quantiser[t][kNatural[k]]));
    }
    put_marker(out, 0xC0, 15);
    out.push_back(8);
    out.push_back(static_cast<unsigned char>(height >> 8));
    out.push_back(static_cast<unsigned char>(height & 255));
    out.push_back(static_cast<unsigned char>(width >> 8));
    out.push_back(static_cast<unsigned char>(width & 255));
    out.push_back(3);
    const unsigned char frame_components[9] = {1, static_cast<unsigned char>((ratio << 4) | ratio), 0, 2, 0x11, 1, 3, 0x11, 1};
    out.insert(out.end(), frame_components, frame_components + 9);
    for (int kind = 0; kind < 2; ++kind)
        for (int chroma = 0; chroma < 2; ++chroma) {
            const CodeList& list = standard_codes(kind, chroma);
            put_marker(out, 0xC4, 17 + list.symbols.size());
            out.push_back(static_cast<unsigned char>((kind << 4) | chroma));
            out.insert(out.end(), list.counts, list.counts + 16);
            out.insert(out.end(), list.symbols.begin(), list.symbols.end());
        }
    put_marker(out, 0xDA, 10);
    const unsigned char scan_header[10] = {3, 1, 0x00, 2, 0x11, 3, 0x11, 0, 63, 0};
    out.insert(out.end(), scan_header, scan_header + 10);

    const Encoding dc[2] = {Encoding(standard_codes(0, 0)), Encoding(standard_codes(0, 1))};
    const Encoding ac[2] = {Encoding(standard_codes(1, 0)), Encoding(standard_codes(1, 1))};
    BitWriter writer(out);
    int prediction[3] = {0, 0, 0};
    for (int my = 0; my < mcus_y; ++my)
        for (int mx = 0; mx < mcus_x; ++mx) {
            for (int by = 0; by < ratio; ++by)
                for (int bx = 0; bx < ratio; ++bx)
                    encode_block(writer, planes[0].data(), padded_w, mx * unit + bx * 8, my * unit + by * 8, quantiser[0], dc[0], ac[0],
                                 prediction[0]);
            for (int k = 1; k < 3; ++k)
                encode_block(writer, planes[k].data(), chroma_w, mx * 8, my * 8, quantiser[1], dc[1], ac[1], prediction[k]);
        }
    writer.finish();
    out.push_back(0xFF);
    out.push_back(0xD9);
    return "";
}

}  // namespace xad_train
