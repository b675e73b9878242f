#include "checkpoint.h"

#include <zlib.h>

#include <cstdio>
#include <cstring>
#include <memory>

namespace xad_train {
namespace {

constexpr char kMagic[8] = {'X', 'A', 'D', 'S', 'P', 'L', 'T', '1'};
constexpr std::uint32_t kVersion = 1;

using File = std::unique_ptr<std::FILE, int (*)(std::FILE*)>;

struct Writer {
    std::FILE* f;
    std::uint32_t crc = 0;
    bool ok = true;
    void put(const void* data, std::size_t bytes) {
        if (!ok || bytes == 0) return;
        crc = static_cast<std::uint32_t>(crc32(crc, static_cast<const Bytef*>(data), static_cast<uInt>(bytes)));
        ok = std::fwrite(data, 1, bytes, f) == bytes;
    }
};

struct Reader {
    std::FILE* f;
    std::uint32_t crc = 0;
    bool ok = true;
    void get(void* data, std::size_t bytes) {
        if (!ok || bytes == 0) return;
        ok = std::fread(data, 1, bytes, f) == bytes;
        if (ok) crc = static_cast<std::uint32_t>(crc32(crc, static_cast<const Bytef*>(data), static_cast<uInt>(bytes)));
    }
};

}  // namespace

std::string write_checkpoint(const std::string& path, const CheckpointState& state) {
    const std::size_t g = static_cast<std::size_t>(state.header.num_gaussians);
    if (state.params.size() != 9 * g || state.m.size() != 9 * g || state.v.size() != 9 * g || state.depth.size() != g)
        return "checkpoint: state arrays do not match the Gaussian count";
    CheckpointHeader header = state.header;
    std::memcpy(header.magic, kMagic, sizeof kMagic);
    header.version = kVersion;
    header.header_bytes = sizeof(CheckpointHeader);
    const std::string tmp = path + ".tmp";
    {
        File f(std::fopen(tmp.c_str(), "wb"), &std::fclose);
        if (!f) return "checkpoint: cannot create " + tmp;
        Writer w{f.get()};
        w.put(&header, sizeof header);
        // the element count stays far below the 4 GiB a single zlib call accepts: G <= 2^31 / 36
        w.put(state.params.data(), state.params.size() * sizeof(float));
        w.put(state.m.data(), state.m.size() * sizeof(float));
        w.put(state.v.data(), state.v.size() * sizeof(float));
        w.put(state.depth.data(), state.depth.size() * sizeof(float));
        const std::uint32_t crc = w.crc;
        if (w.ok) w.ok = std::fwrite(&crc, 1, sizeof crc, f.get()) == sizeof crc;
        if (w.ok) w.ok = std::fflush(f.get()) == 0;
        if (!w.ok) {
            f.reset();
            std::remove(tmp.c_str());
            return "checkpoint: write error on " + tmp;
        }
    }
    if (std::rename(tmp.c_str(), path.c_str()) != 0) {
        std::remove(tmp.c_str());
        return "checkpoint: cannot rename " + tmp + " to " + path;
    }
    return "";
}

std::string read_checkpoint(const std::string& path, CheckpointState& state) {
    File f(std::fopen(path.c_str(), "rb"), &std::fclose);
    if (!f) return "checkpoint: cannot open " + path;
    Reader r{f.get()};
    CheckpointHeader& h = state.header;
    r.get(&h, sizeof h);
    if (!r.ok) return "checkpoint: " + path + " is shorter than a header";
    if (std::memcmp(h.magic, kMagic, sizeof kMagic) != 0) return "checkpoint: " + path + " is not a splatting checkpoint";
    if (h.version != kVersion || h.header_bytes != sizeof(CheckpointHeader))
        return "checkpoint: " + path + " has an unknown format version";
    if (h.num_gaussians <= 0 || h.num_gaussians > (1 << 26) || h.width <= 0 || h.height <= 0 || h.iteration < 0)
        return "checkpoint: " + path + " has a damaged header";
    const std::size_t g = static_cast<std::size_t>(h.num_gaussians);
    {
        // the header fixes the length of the file: check it before sizing anything by the header
        const long at = std::ftell(f.get());
        if (at < 0 || std::fseek(f.get(), 0, SEEK_END) != 0) return "checkpoint: cannot seek in " + path;
        const long length = std::ftell(f.get());
        if (std::fseek(f.get(), at, SEEK_SET) != 0) return "checkpoint: cannot seek in " + path;
        const unsigned long long expected = sizeof(CheckpointHeader) + 4ull * 28ull * g + 4ull;
        if (length < 0 || static_cast<unsigned long long>(length) < expected) return "checkpoint: " + path + " is truncated";
        if (static_cast<unsigned long long>(length) > expected) return "checkpoint: " + path + " has trailing bytes";
    }
    state.params.resize(9 * g);
    state.m.resize(9 * g);
    state.v.resize(9 * g);
    state.depth.resize(g);
    r.get(state.params.data(), state.params.size() * sizeof(float));
    r.get(state.m.data(), state.m.size() * sizeof(float));
    r.get(state.v.data(), state.v.size() * sizeof(float));
    r.get(state.depth.data(), state.depth.size() * sizeof(float));
    if (!r.ok) return "checkpoint: " + path + " is truncated";
    std::uint32_t stored = 0;
    if (std::fread(&stored, 1, sizeof stored, f.get()) != sizeof stored) return "checkpoint: " + path + " is truncated";
    if (stored != r.crc) return "checkpoint: " + path + " fails its checksum";
    if (std::fgetc(f.get()) != EOF) return "checkpoint: " + path + " has trailing bytes";
    return "";
}

}  // namespace xad_train
