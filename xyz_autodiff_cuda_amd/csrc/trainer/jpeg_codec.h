#pragma once
// JPEG files (ITU-T T.81 with the JFIF conventions of T.871) for the splatting
// trainer, written from the standard.
//
// The trainer of xyz-autodiff-cuda reads its target through stb_image and writes
// every snapshot as a JPEG of quality 90 through stb_image_write
// (examples/mini-gaussian-splatting/image_utils.cpp:12-56,
// gaussian_splatting_training.cu:84-108, :124); this file gives the trainer here
// the same two formats without those libraries.
//
// Reading: Huffman-coded baseline, extended sequential and progressive files of
// 8-bit samples, grey or three components (YCbCr, or RGB when an Adobe marker or
// the component names say so), any integral sampling ratios, restart intervals.
// Arithmetic coding, lossless and hierarchical modes, 12-bit samples and four
// components are refused with a message.  The inverse transform is the exact
// one (floating point, rounded once); chroma sampled at half the rate is
// interpolated with the 3:1 triangle weights of centred chroma samples, other
// ratios are replicated; a decoded byte can differ by one or two levels from
// what another conforming decoder gives, as the standard allows.
//
// Writing: baseline, YCbCr, the tables of annex K scaled by the quality as the
// Independent JPEG Group's software scales them, chroma at half the rate in both
// directions up to quality 90 and at the full rate above it (the policy of the
// writer the reference calls).

#include <string>
#include <vector>

#include "image_io.h"

namespace xad_train {

// Returns "" or the reason for failure.
std::string decode_jpeg(const std::vector<unsigned char>& file, Image& out);

// rgb8: height x width x 3 bytes.  quality 1..100.
std::string encode_jpeg(int width, int height, const std::vector<unsigned char>& rgb8, int quality,
                        std::vector<unsigned char>& out);

}  // namespace xad_train
