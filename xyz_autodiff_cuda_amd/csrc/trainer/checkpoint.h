#pragma once
// Training-state files of the splatting trainer (host side).
//
// Layout, little endian:
//   Header (fixed size, below) | params 9G f32 | m 9G f32 | v 9G f32 | depth G f32 | crc32 u32
// The CRC-32 covers every byte before it.  xyz-autodiff-cuda has no such file:
// its GaussianCollection only copies the state between device and host
// (examples/mini-gaussian-splatting/gaussian_parameters.cu:68-116).

#include <cstdint>
#include <string>
#include <vector>

namespace xad_train {

struct CheckpointHeader {
    char magic[8];  // "XADSPLT1"
    std::uint32_t version;
    std::uint32_t header_bytes;
    std::int32_t width, height, num_gaussians, iteration;
    float lr_center, lr_scale, lr_rotation, lr_color, lr_opacity;
    float beta1, beta2, epsilon;
    std::uint64_t seed;
};
static_assert(sizeof(CheckpointHeader) == 72, "checkpoint header layout is part of the file format");

struct CheckpointState {
    CheckpointHeader header;
    std::vector<float> params, m, v, depth;  // 9G, 9G, 9G, G
};

// Both return "" or the reason for failure.  write_checkpoint writes to
// `path`.tmp and renames it over `path`.
std::string write_checkpoint(const std::string& path, const CheckpointState& state);
std::string read_checkpoint(const std::string& path, CheckpointState& state);

}  // namespace xad_train
