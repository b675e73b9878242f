#include "image_io.h"

#include <zlib.h>

#include "jpeg_codec.h"

#include <algorithm>
#include <cctype>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>

namespace xad_train {
namespace {

using Bytes = std::vector<unsigned char>;

constexpr unsigned char kPngSignature[8] = {0x89, 'P', 'N', 'G', '\r', '\n', 0x1A, '\n'};
constexpr std::size_t kMaxPixels = std::size_t(1) << 26;  // 8192 x 8192

std::string read_file(const std::string& path, Bytes& out) {
    std::unique_ptr<std::FILE, int (*)(std::FILE*)> f(std::fopen(path.c_str(), "rb"), &std::fclose);
    if (!f) return "cannot open " + path;
    unsigned char chunk[1 << 16];
    std::size_t got;
    while ((got = std::fread(chunk, 1, sizeof chunk, f.get())) > 0) out.insert(out.end(), chunk, chunk + got);
    if (std::ferror(f.get())) return "read error on " + path;
    return "";
}

std::string write_file(const std::string& path, const Bytes& data) {
    std::unique_ptr<std::FILE, int (*)(std::FILE*)> f(std::fopen(path.c_str(), "wb"), &std::fclose);
    if (!f) return "cannot create " + path;
    if (std::fwrite(data.data(), 1, data.size(), f.get()) != data.size()) return "write error on " + path;
    if (std::fflush(f.get()) != 0) return "write error on " + path;
    return "";
}

std::uint32_t be32(const unsigned char* p) {
    return (std::uint32_t(p[0]) << 24) | (std::uint32_t(p[1]) << 16) | (std::uint32_t(p[2]) << 8) | p[3];
}

void put_be32(Bytes& out, std::uint32_t v) {
    for (int shift = 24; shift >= 0; shift -= 8) out.push_back(static_cast<unsigned char>(v >> shift));
}

// ---- PNG ---------------------------------------------------------------------

int paeth(int a, int b, int c) {
    const int p = a + b - c;
    const int pa = std::abs(p - a), pb = std::abs(p - b), pc = std::abs(p - c);
    if (pa <= pb && pa <= pc) return a;
    return pb <= pc ? b : c;
}

// Undoes the per-row prediction filters in place; `raw` points at height rows of
// 1 + row_bytes bytes.  Returns false on an unknown filter type.
bool unfilter(unsigned char* raw, std::size_t height, std::size_t row_bytes, std::size_t bpp) {
    const Bytes zero_row(row_bytes, 0);
    for (std::size_t y = 0; y < height; ++y) {
        unsigned char* row = raw + y * (row_bytes + 1) + 1;
        const unsigned char* up = y ? row - (row_bytes + 1) : zero_row.data();
        const int type = row[-1];
        for (std::size_t i = 0; i < row_bytes; ++i) {
            const int a = i >= bpp ? row[i - bpp] : 0;
            const int b = up[i];
            const int c = i >= bpp ? up[i - bpp] : 0;
            int predicted;
            switch (type) {
                case 0: predicted = 0; break;
                case 1: predicted = a; break;
                case 2: predicted = b; break;
                case 3: predicted = (a + b) >> 1; break;
                case 4: predicted = paeth(a, b, c); break;
                default: return false;
            }
            row[i] = static_cast<unsigned char>(row[i] + predicted);
        }
    }
    return true;
}

std::string decode_png(const Bytes& file, Image& out) {
    std::size_t pos = 8;
    std::uint32_t width = 0, height = 0;
    int depth = 0, colour = -1, interlaced = 0;
    Bytes palette, compressed;
    bool seen_end = false;
    while (!seen_end) {
        if (pos + 12 > file.size()) return "PNG: truncated file";
        const std::uint32_t length = be32(&file[pos]);
        if (length > file.size() - pos - 12) return "PNG: chunk runs past the end of the file";
        const unsigned char* type = &file[pos + 4];
        const unsigned char* data = &file[pos + 8];
        if (be32(data + length) != crc32(0, type, length + 4)) return "PNG: chunk checksum mismatch";
        if (!std::memcmp(type, "IHDR", 4)) {
            if (length != 13) return "PNG: bad header chunk";
            width = be32(data);
            height = be32(data + 4);
            depth = data[8];
            colour = data[9];
            if (data[10] != 0 || data[11] != 0) return "PNG: unknown compression or filter method";
            interlaced = data[12];
            if (interlaced > 1) return "PNG: unknown interlace method";
        } else if (colour < 0) {
            return "PNG: first chunk is not the header";
        } else if (!std::memcmp(type, "PLTE", 4)) {
            palette.assign(data, data + length);
        } else if (!std::memcmp(type, "IDAT", 4)) {
            compressed.insert(compressed.end(), data, data + length);
        } else if (!std::memcmp(type, "IEND", 4)) {
            seen_end = true;
        } else if (!(type[0] & 0x20)) {
            return "PNG: unknown critical chunk";
        }
        pos += 12 + length;
    }
    int channels;
    switch (colour) {
        case 0: channels = 1; break;
        case 2: channels = 3; break;
        case 3: channels = 1; break;
        case 4: channels = 2; break;
        case 6: channels = 4; break;
        default: return "PNG: unknown colour type";
    }
    const bool depth_ok = colour == 0   ? (depth == 1 || depth == 2 || depth == 4 || depth == 8 || depth == 16)
                          : colour == 3 ? (depth == 1 || depth == 2 || depth == 4 || depth == 8)
                                        : (depth == 8 || depth == 16);
    if (!depth_ok) return "PNG: bit depth not allowed for this colour type";
    if (width == 0 || height == 0 || std::size_t(width) * height > kMaxPixels) return "PNG: unreasonable image size";
    if (colour == 3 && (palette.empty() || palette.size() % 3)) return "PNG: palette missing or malformed";

    // The image as one pass, or as the seven passes of Adam7: each pass is a smaller image of the pixels
    // (x0 + i dx, y0 + j dy), filtered row by row on its own.
    struct Pass { std::size_t x0, y0, dx, dy; };
    static const Pass kWhole[1] = {{0, 0, 1, 1}};
    static const Pass kAdam7[7] = {{0, 0, 8, 8}, {4, 0, 8, 8}, {0, 4, 4, 8}, {2, 0, 4, 4}, {0, 2, 2, 4}, {1, 0, 2, 2}, {0, 1, 1, 2}};
    const Pass* passes = interlaced ? kAdam7 : kWhole;
    const int pass_count = interlaced ? 7 : 1;
    const std::size_t bits_per_pixel = std::size_t(channels) * depth;
    std::size_t total = 0;
    for (int p = 0; p < pass_count; ++p) {
        const std::size_t pw = (width + passes[p].dx - 1 - passes[p].x0) / passes[p].dx;
        const std::size_t ph = (height + passes[p].dy - 1 - passes[p].y0) / passes[p].dy;
        if (pw && ph) total += ph * (1 + (pw * bits_per_pixel + 7) / 8);
    }
    Bytes raw(total);
    uLongf raw_size = raw.size();
    const int z = uncompress(raw.data(), &raw_size, compressed.data(), compressed.size());
    if (z != Z_OK || raw_size != raw.size()) return "PNG: image data does not inflate to the declared size";

    out.width = static_cast<int>(width);
    out.height = static_cast<int>(height);
    out.rgb.assign(std::size_t(width) * height * 3, 0.0f);
    const float max_sample = static_cast<float>((1u << depth) - 1);
    std::size_t offset = 0;
    for (int p = 0; p < pass_count; ++p) {
        const Pass& pass = passes[p];
        const std::size_t pw = (width + pass.dx - 1 - pass.x0) / pass.dx;
        const std::size_t ph = (height + pass.dy - 1 - pass.y0) / pass.dy;
        if (pw == 0 || ph == 0) continue;
        const std::size_t row_bytes = (pw * bits_per_pixel + 7) / 8;
        if (!unfilter(raw.data() + offset, ph, row_bytes, std::max<std::size_t>(1, bits_per_pixel / 8)))
            return "PNG: unknown row filter";
        for (std::size_t j = 0; j < ph; ++j) {
            const unsigned char* row = raw.data() + offset + j * (row_bytes + 1) + 1;
            auto sample = [&](std::size_t index) -> unsigned {
                if (depth == 8) return row[index];
                if (depth == 16) return (unsigned(row[2 * index]) << 8) | row[2 * index + 1];
                const std::size_t bit = index * depth;
                return (row[bit >> 3] >> (8 - depth - (bit & 7))) & ((1u << depth) - 1);
            };
            const std::size_t y = pass.y0 + j * pass.dy;
            for (std::size_t i = 0; i < pw; ++i) {
                float* px = &out.rgb[(y * width + pass.x0 + i * pass.dx) * 3];
                if (colour == 3) {
                    const unsigned entry = sample(i);
                    if (3 * entry + 2 >= palette.size()) return "PNG: palette index out of range";
                    for (int c = 0; c < 3; ++c) px[c] = palette[3 * entry + c] / 255.0f;
                } else if (channels <= 2) {
                    px[0] = px[1] = px[2] = sample(i * channels) / max_sample;
                } else {
                    for (int c = 0; c < 3; ++c) px[c] = sample(i * channels + c) / max_sample;
                }
            }
        }
        offset += ph * (row_bytes + 1);
    }
    return "";
}

void append_chunk(Bytes& out, const char* type, const Bytes& data) {
    put_be32(out, static_cast<std::uint32_t>(data.size()));
    const std::size_t start = out.size();
    out.insert(out.end(), type, type + 4);
    out.insert(out.end(), data.begin(), data.end());
    put_be32(out, static_cast<std::uint32_t>(crc32(0, out.data() + start, static_cast<uInt>(out.size() - start))));
}

std::string encode_png(int width, int height, const Bytes& pixels, Bytes& out) {
    const std::size_t row_bytes = std::size_t(width) * 3;
    Bytes raw;
    raw.reserve(std::size_t(height) * (row_bytes + 1));
    for (int y = 0; y < height; ++y) {
        raw.push_back(0);  // filter: none
        raw.insert(raw.end(), pixels.begin() + y * row_bytes, pixels.begin() + (y + 1) * row_bytes);
    }
    uLongf packed_size = compressBound(raw.size());
    Bytes packed(packed_size);
    if (compress2(packed.data(), &packed_size, raw.data(), raw.size(), 6) != Z_OK) return "PNG: deflate failed";
    packed.resize(packed_size);

    out.assign(kPngSignature, kPngSignature + 8);
    Bytes header;
    put_be32(header, static_cast<std::uint32_t>(width));
    put_be32(header, static_cast<std::uint32_t>(height));
    const unsigned char tail[5] = {8, 2, 0, 0, 0};  // 8 bits, RGB, deflate, adaptive filters, not interlaced
    header.insert(header.end(), tail, tail + 5);
    append_chunk(out, "IHDR", header);
    append_chunk(out, "IDAT", packed);
    append_chunk(out, "IEND", Bytes());
    return "";
}

// ---- PPM / PGM -----------------------------------------------------------------

// Next unsigned integer of a netpbm header, skipping white space and # comments.
bool next_header_number(const Bytes& file, std::size_t& pos, unsigned& value) {
    for (;;) {
        while (pos < file.size() && std::isspace(file[pos])) ++pos;
        if (pos < file.size() && file[pos] == '#') {
            while (pos < file.size() && file[pos] != '\n') ++pos;
            continue;
        }
        break;
    }
    if (pos >= file.size() || !std::isdigit(file[pos])) return false;
    unsigned long v = 0;
    while (pos < file.size() && std::isdigit(file[pos])) {
        v = v * 10 + (file[pos++] - '0');
        if (v > 1000000000ul) return false;
    }
    value = static_cast<unsigned>(v);
    return true;
}

std::string decode_netpbm(const Bytes& file, Image& out) {
    const int channels = file[1] == '6' ? 3 : 1;
    std::size_t pos = 2;
    unsigned width, height, max_value;
    if (!next_header_number(file, pos, width) || !next_header_number(file, pos, height) ||
        !next_header_number(file, pos, max_value))
        return "PPM: malformed header";
    if (pos >= file.size() || !std::isspace(file[pos])) return "PPM: malformed header";
    ++pos;  // the single white-space byte before the raster
    if (max_value == 0 || max_value > 65535) return "PPM: maximum value out of range";
    if (width == 0 || height == 0 || std::size_t(width) * height > kMaxPixels) return "PPM: unreasonable image size";
    const std::size_t sample_bytes = max_value > 255 ? 2 : 1;
    const std::size_t samples = std::size_t(width) * height * channels;
    if (file.size() - pos < samples * sample_bytes) return "PPM: raster is shorter than the header declares";
    out.width = static_cast<int>(width);
    out.height = static_cast<int>(height);
    out.rgb.resize(std::size_t(width) * height * 3);
    const unsigned char* raster = file.data() + pos;
    for (std::size_t i = 0; i < std::size_t(width) * height; ++i) {
        for (int c = 0; c < 3; ++c) {
            const std::size_t s = i * channels + (channels == 3 ? c : 0);
            const unsigned v = sample_bytes == 2 ? (unsigned(raster[2 * s]) << 8) | raster[2 * s + 1] : raster[s];
            out.rgb[i * 3 + c] = static_cast<float>(v) / static_cast<float>(max_value);
        }
    }
    return "";
}

// ---- BMP -----------------------------------------------------------------------

std::uint32_t le32(const unsigned char* p) {
    return std::uint32_t(p[0]) | (std::uint32_t(p[1]) << 8) | (std::uint32_t(p[2]) << 16) | (std::uint32_t(p[3]) << 24);
}

std::uint32_t le16(const unsigned char* p) { return std::uint32_t(p[0]) | (std::uint32_t(p[1]) << 8); }

// The field of a packed pixel that a mask selects, as a fraction of the field's largest value.
float masked_field(std::uint32_t value, std::uint32_t mask) {
    if (mask == 0) return 0.0f;
    int shift = 0;
    while (!((mask >> shift) & 1u)) ++shift;
    return static_cast<float>((value & mask) >> shift) / static_cast<float>(mask >> shift);
}

// Windows bitmaps without compression: 1, 4 or 8 bits with a colour table, 16 or 32 bits with the default or
// given channel masks, 24 bits; rows bottom-up or (negative height) top-down, padded to four bytes.
std::string decode_bmp(const Bytes& file, Image& out) {
    if (file.size() < 26) return "BMP: truncated file";
    const std::size_t data_offset = le32(&file[10]);
    const std::size_t header = le32(&file[14]);
    long long width, height;
    unsigned bits, compression = 0, colours = 0;
    std::size_t entry_bytes = 4;
    if (header == 12) {
        width = le16(&file[18]);
        height = le16(&file[20]);
        bits = le16(&file[24]);
        entry_bytes = 3;
    } else if (header >= 40 && header <= 256 && file.size() >= 14 + header) {
        width = static_cast<std::int32_t>(le32(&file[18]));
        height = static_cast<std::int32_t>(le32(&file[22]));
        bits = le16(&file[28]);
        compression = le32(&file[30]);
        colours = le32(&file[46]);
    } else {
        return "BMP: unknown header";
    }
    const bool top_down = height < 0;
    if (top_down) height = -height;
    if (width <= 0 || height <= 0 || static_cast<unsigned long long>(width) * static_cast<unsigned long long>(height) > kMaxPixels)
        return "BMP: unreasonable image size";
    if (bits != 1 && bits != 4 && bits != 8 && bits != 16 && bits != 24 && bits != 32) return "BMP: unknown bit depth";
    const bool given_masks = compression == 3 || compression == 6;
    if (compression != 0 && !(given_masks && (bits == 16 || bits == 32))) return "BMP: compressed files are not supported";
    std::uint32_t mask[3] = {0x00FF0000u, 0x0000FF00u, 0x000000FFu};
    if (bits == 16) mask[0] = 0x7C00u, mask[1] = 0x03E0u, mask[2] = 0x001Fu;
    if (given_masks) {
        if (file.size() < 66) return "BMP: truncated file";
        for (int c = 0; c < 3; ++c) mask[c] = le32(&file[54 + 4 * c]);
        if (bits == 16)
            for (std::uint32_t& m : mask) m &= 0xFFFFu;
    }
    std::size_t entries = 0;
    const unsigned char* table = nullptr;
    if (bits <= 8) {
        entries = colours ? colours : (std::size_t(1) << bits);
        if (entries > 256) return "BMP: colour table too large";
        const std::size_t table_offset = 14 + header;
        if (table_offset > file.size() || entries * entry_bytes > file.size() - table_offset) return "BMP: truncated colour table";
        table = &file[table_offset];
    }
    const std::size_t row_bytes = (static_cast<std::size_t>(width) * bits + 31) / 32 * 4;
    if (data_offset > file.size() || row_bytes * static_cast<std::size_t>(height) > file.size() - data_offset)
        return "BMP: raster is shorter than the header declares";
    out.width = static_cast<int>(width);
    out.height = static_cast<int>(height);
    out.rgb.resize(static_cast<std::size_t>(width) * height * 3);
    for (long long j = 0; j < height; ++j) {
        const unsigned char* row = &file[data_offset + static_cast<std::size_t>(j) * row_bytes];
        float* to = &out.rgb[static_cast<std::size_t>(top_down ? j : height - 1 - j) * width * 3];
        for (long long x = 0; x < width; ++x, to += 3) {
            if (bits <= 8) {
                const std::size_t bit = static_cast<std::size_t>(x) * bits;
                const std::size_t index = (row[bit >> 3] >> (8 - bits - (bit & 7))) & ((1u << bits) - 1);
                if (index >= entries) return "BMP: colour index out of range";
                for (int c = 0; c < 3; ++c) to[c] = table[index * entry_bytes + 2 - c] / 255.0f;  // stored blue, green, red
            } else if (bits == 24) {
                for (int c = 0; c < 3; ++c) to[c] = row[3 * x + 2 - c] / 255.0f;
            } else {
                const std::uint32_t value = bits == 16 ? le16(row + 2 * x) : le32(row + 4 * x);
                for (int c = 0; c < 3; ++c) to[c] = masked_field(value, mask[c]);
            }
        }
    }
    return "";
}

bool ends_with(const std::string& s, const char* suffix) {
    const std::size_t n = std::strlen(suffix);
    if (s.size() < n) return false;
    for (std::size_t i = 0; i < n; ++i)
        if (std::tolower(static_cast<unsigned char>(s[s.size() - n + i])) != suffix[i]) return false;
    return true;
}

}  // namespace

std::string load_image(const std::string& path, Image& out) {
    Bytes file;
    if (std::string err = read_file(path, file); !err.empty()) return err;
    if (file.size() >= 8 && !std::memcmp(file.data(), kPngSignature, 8)) return decode_png(file, out);
    if (file.size() >= 3 && file[0] == 'P' && (file[1] == '6' || file[1] == '5')) return decode_netpbm(file, out);
    if (file.size() >= 2 && file[0] == 0xFF && file[1] == 0xD8) return decode_jpeg(file, out);
    if (file.size() >= 2 && file[0] == 'B' && file[1] == 'M') return decode_bmp(file, out);
    return path + " is neither a PNG, a JPEG, a BMP nor a binary PPM/PGM file";
}

namespace {

// byte = (unsigned char)(clamped * 255 + 0.5), as image_utils.cpp:42-46 quantises before its encoder
std::string to_bytes(int width, int height, const float* rgb, Bytes& pixels) {
    if (width <= 0 || height <= 0 || !rgb) return "save_image: empty image";
    pixels.resize(std::size_t(width) * height * 3);
    for (std::size_t i = 0; i < pixels.size(); ++i) {
        const float v = rgb[i];
        const float clamped = v > 0.0f ? (v < 1.0f ? v : 1.0f) : 0.0f;  // NaN becomes 0
        pixels[i] = static_cast<unsigned char>(clamped * 255.0f + 0.5f);
    }
    return "";
}

}  // namespace

std::string save_image_jpeg(const std::string& path, int width, int height, const float* rgb, int quality) {
    Bytes pixels, file;
    if (std::string err = to_bytes(width, height, rgb, pixels); !err.empty()) return err;
    if (std::string err = encode_jpeg(width, height, pixels, quality, file); !err.empty()) return err;
    return write_file(path, file);
}

std::string save_image(const std::string& path, int width, int height, const float* rgb) {
    if (ends_with(path, ".jpg") || ends_with(path, ".jpeg")) return save_image_jpeg(path, width, height, rgb, kDefaultJpegQuality);
    Bytes pixels, file;
    if (std::string err = to_bytes(width, height, rgb, pixels); !err.empty()) return err;
    if (ends_with(path, ".png")) {
        if (std::string err = encode_png(width, height, pixels, file); !err.empty()) return err;
    } else if (ends_with(path, ".ppm")) {
        char header[64];
        const int n = std::snprintf(header, sizeof header, "P6\n%d %d\n255\n", width, height);
        file.assign(header, header + n);
        file.insert(file.end(), pixels.begin(), pixels.end());
    } else {
        return "save_image: " + path + " must end in .jpg, .jpeg, .png or .ppm";
    }
    return write_file(path, file);
}

void test_pattern(int width, int height, float* rgb) {
    for (int y = 0; y < height; ++y) {
        for (int x = 0; x < width; ++x) {
            const float r = static_cast<float>(x) / width;
            const float g = static_cast<float>(y) / height;
            float* px = rgb + (std::size_t(y) * width + x) * 3;
            px[0] = r;
            px[1] = g;
            px[2] = 0.5f * (r + g);
        }
    }
}

}  // namespace xad_train
