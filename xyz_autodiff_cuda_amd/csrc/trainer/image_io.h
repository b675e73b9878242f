#pragma once
// Image files for the splatting trainer: float RGB in [0, 1], rows top to
// bottom, three interleaved values per pixel.
//
// Plays the part of load_image / save_image_jpeg / create_test_image of
// xyz-autodiff-cuda (examples/mini-gaussian-splatting/image_utils.cpp:12-79),
// which go through the stb single-header libraries.  Here PNG, JPEG and binary
// PPM/PGM are read and written directly (DEFLATE and CRC-32 from the system's
// zlib; the JPEG codec is jpeg_codec.cpp).

#include <string>
#include <vector>

namespace xad_train {

struct Image {
    int width = 0;
    int height = 0;
    std::vector<float> rgb;  // height x width x 3
};

// Reads a PNG (any bit depth and colour type, interlaced or not), a JPEG
// (Huffman-coded, sequential or progressive, grey or colour), an uncompressed
// BMP or a binary PPM/PGM (P6/P5), told apart by their first bytes.  Grey becomes R = G = B, alpha is
// dropped, samples are divided by their maximum value (image_utils.cpp:27-30
// divides bytes by 255).  Returns "" or the reason for failure.
std::string load_image(const std::string& path, Image& out);

// The quality save_image_jpeg has by default in the reference (image_utils.h:21).
constexpr int kDefaultJpegQuality = 90;

// Writes 8-bit RGB as JPEG (at kDefaultJpegQuality), PNG or PPM by the path's
// extension (.jpg / .jpeg / .png / .ppm).  Values are clamped to [0, 1] and
// rounded as the reference does before its JPEG encoder:
// byte = (unsigned char)(clamped * 255 + 0.5) (image_utils.cpp:42-46).
std::string save_image(const std::string& path, int width, int height, const float* rgb);

// save_image_jpeg of the reference (image_utils.cpp:38-56): a JPEG of the given quality (1..100) whatever the extension.
std::string save_image_jpeg(const std::string& path, int width, int height, const float* rgb, int quality);

// r = x / width, g = y / height, b = (r + g) / 2 (image_utils.cpp:58-77).
void test_pattern(int width, int height, float* rgb);

}  // namespace xad_train
