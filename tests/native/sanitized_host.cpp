// The host side of the build under AddressSanitizer and UndefinedBehaviorSanitizer: one program,
// compiled by g++ alone with -fsanitize=address,undefined -fno-sanitize-recover=all, that runs
//   1. every known-answer case of the operator API and the benchmark graph, host build of the templates;
//   2. every gradient-tester call of the reference's tests, host build;
//   3. the trainer's command-line parser on well- and ill-formed command lines;
//   4. the image and checkpoint readers (hand-written PNG/PPM framing over zlib; they take files from
//      outside) on a corpus of valid files and on a bounded number of random mutations of them.
// A finding of either sanitizer aborts the program; the test checks the exit status and the summary line.
// The reference reads images through stb (examples/mini-gaussian-splatting/image_utils.cpp:12-37) and has
// no such tier.
#include <dirent.h>
#include <sys/stat.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "../../include/xad_capi.h"
#include "../../xyz_autodiff_cuda_amd/csrc/chain.cuh"
#include "../../xyz_autodiff_cuda_amd/csrc/trainer/checkpoint.h"
#include "../../xyz_autodiff_cuda_amd/csrc/trainer/image_io.h"
#include "api_cases.cuh"
#include "tester_suite.cuh"

namespace xad {
char* last_error_buffer() {  // what capi_common.hip provides inside the library
    static thread_local char buffer[512] = {0};
    return buffer;
}
}  // namespace xad

namespace {

std::vector<unsigned char> slurp(const std::string& path) {
    std::vector<unsigned char> bytes;
    if (FILE* f = std::fopen(path.c_str(), "rb")) {
        int c;
        while ((c = std::fgetc(f)) != EOF) bytes.push_back(static_cast<unsigned char>(c));
        std::fclose(f);
    }
    return bytes;
}

bool spit(const std::string& path, const std::vector<unsigned char>& bytes) {
    FILE* f = std::fopen(path.c_str(), "wb");
    if (!f) return false;
    const bool ok = std::fwrite(bytes.data(), 1, bytes.size(), f) == bytes.size();
    return std::fclose(f) == 0 && ok;
}

int api_cases() {
    int ran = 0;
    for (int id = 0; id < 64; ++id) {
        double out[xad_test::kCaseCapacity] = {0};
        const int n = xad_test::run_case(id, out);
        if (n < 0) continue;  // no such case
        if (n > xad_test::kCaseCapacity) return -1;
        ++ran;
    }
    // the benchmark graph, float and double, over a spread of inputs including the ends of the ranges
    std::mt19937 rng(7);
    std::uniform_real_distribution<double> s(-2.0, 1.0), angle(-3.2, 3.2), p(-6.0, 6.0);
    double sink = 0.0;
    for (int i = 0; i < 20000; ++i) {
        const double sx = s(rng), sy = s(rng), th = angle(rng), o = p(rng), px = p(rng), py = p(rng);
        const auto a = xad_chain::forward_backward<double>(sx, sy, th, o, px, py);
        const auto b = xad_chain::forward_backward<float>(float(sx), float(sy), float(th), float(o), float(px), float(py));
        sink += a.w + a.d_sx + b.w + b.d_theta;
    }
    const auto edge = xad_chain::forward_backward<float>(-2.f, 1.f, 3.1415927f, -80.f, 1e3f, -1e3f);
    sink += edge.w;
    return std::isfinite(sink) ? ran : -1;
}

int config_cases() {
    const std::vector<std::vector<const char*>> lines = {
        {"prog", "0.01", "0.005", "0.02", "0.01", "0.01", "--target", "t.png"},
        {"prog", "0.01", "0.005", "0.02", "0.01", "0.01", "--target", "t.png", "--max-iterations", "10", "--save-interval", "5",
         "--num-gaussians", "77", "--no-save-images", "--beta1", "0.8", "--beta2", "0.99", "--epsilon", "1e-6", "--seed", "18446744073709551615",
         "--output-dir", "o", "--checkpoint", "c.ckpt", "--checkpoint-interval", "3", "--resume", "r.ckpt"},
        {"prog"},
        {"prog", "--help"},
        {"prog", "0.01", "0.005", "0.02", "0.01"},
        {"prog", "x", "y", "z", "", "nan", "--target", "t.png"},
        {"prog", "0.01", "0.005", "0.02", "0.01", "0.01", "--target"},
        {"prog", "0.01", "0.005", "0.02", "0.01", "0.01", "--bogus", "1"},
        {"prog", "0.01", "0.005", "0.02", "0.01", "0.01", "--target", "t.png", "--max-iterations", "99999999999999999999"},
        {"prog", "0.01", "0.005", "0.02", "0.01", "0.01", "--target", "t.png", "--num-gaussians", "-5"},
        {"prog", "1e400", "-1", "0", "inf", "0.01", "--target", "t.png", "--beta1", "2"},
    };
    int accepted = 0;
    for (const auto& line : lines) {
        xad_training_config config;
        xad_training_config_defaults(&config);
        const int st = xad_training_config_parse(static_cast<int>(line.size()), line.data(), &config);
        if (st == XAD_OK && xad_training_config_validate(&config) == XAD_OK) ++accepted;
    }
    // a path longer than the fixed field must be refused, not copied
    std::string longer(5000, 'a');
    const char* argv[] = {"prog", "0.01", "0.005", "0.02", "0.01", "0.01", "--target", longer.c_str()};
    xad_training_config config;
    xad_training_config_defaults(&config);
    if (xad_training_config_parse(8, argv, &config) == XAD_OK) return -1;
    if (std::strlen(xad_training_usage()) < 100) return -1;
    return accepted;
}

struct Tally {
    long accepted = 0, rejected = 0;
};

bool try_file(const std::string& path, Tally& tally) {
    xad_train::Image image;
    const std::string err = xad_train::load_image(path, image);
    if (err.empty()) {
        ++tally.accepted;
        if (image.width <= 0 || image.height <= 0 ||
            static_cast<std::size_t>(image.width) * image.height * 3 != image.rgb.size())
            return false;
        for (float v : image.rgb)
            if (!(v >= 0.f && v <= 1.f)) return false;
    } else {
        ++tally.rejected;
    }
    xad_train::CheckpointState state;
    if (xad_train::read_checkpoint(path, state).empty()) {
        const std::size_t g = static_cast<std::size_t>(state.header.num_gaussians);
        if (state.params.size() != 9 * g || state.m.size() != 9 * g || state.v.size() != 9 * g || state.depth.size() != g) return false;
    }
    return true;
}

}  // namespace

// argv: corpus directory (valid image files; a checkpoint is added here), scratch directory, mutations
int main(int argc, char** argv) {
    if (argc != 4) return 2;
    const std::string corpus_dir = argv[1], scratch = argv[2];
    const int mutations = std::atoi(argv[3]);

    const int cases = api_cases();
    if (cases <= 0) { std::printf("api cases failed\n"); return 1; }

    std::vector<char> text(1 << 16);
    unsigned self_checks = 0;
    const int tester_calls = xad_suite::export_suite(text.data(), text.size(), &self_checks);
    if (tester_calls <= 0) { std::printf("tester suite failed: %s\n", text.data()); return 1; }

    const int configs = config_cases();
    if (configs < 0) { std::printf("config cases failed\n"); return 1; }

    {   // a valid checkpoint joins the corpus; it must round-trip, and survive being written as an image target
        xad_train::CheckpointState st{};
        std::memcpy(st.header.magic, "XADSPLT1", 8);
        st.header.width = 32; st.header.height = 16; st.header.num_gaussians = 5; st.header.iteration = 7;
        st.params.assign(45, 1.f); st.m.assign(45, 2.f); st.v.assign(45, 3.f); st.depth.assign(5, 0.5f);
        const std::string err = xad_train::write_checkpoint(corpus_dir + "/state.ckpt", st);
        if (!err.empty()) { std::printf("%s\n", err.c_str()); return 1; }
        xad_train::CheckpointState back;
        if (!xad_train::read_checkpoint(corpus_dir + "/state.ckpt", back).empty() || back.m[3] != 2.f || back.header.iteration != 7) {
            std::printf("checkpoint round trip failed\n");
            return 1;
        }
        std::vector<float> rgb(24 * 10 * 3);
        xad_train::test_pattern(24, 10, rgb.data());
        if (!xad_train::save_image(corpus_dir + "/pattern.png", 24, 10, rgb.data()).empty() ||
            !xad_train::save_image(corpus_dir + "/pattern.ppm", 24, 10, rgb.data()).empty() ||
            !xad_train::save_image(corpus_dir + "/pattern.jpg", 24, 10, rgb.data()).empty() ||
            !xad_train::save_image_jpeg(corpus_dir + "/pattern_q100.jpg", 24, 10, rgb.data(), 100).empty()) {
            std::printf("save_image failed\n");
            return 1;
        }
    }

    std::vector<std::vector<unsigned char>> corpus;
    Tally clean;
    if (DIR* d = opendir(corpus_dir.c_str())) {
        while (dirent* e = readdir(d)) {
            const std::string name = e->d_name;
            if (name == "." || name == "..") continue;
            const std::string path = corpus_dir + "/" + name;
            if (!try_file(path, clean)) { std::printf("inconsistent result for %s\n", name.c_str()); return 1; }
            corpus.push_back(slurp(path));
        }
        closedir(d);
    }
    if (corpus.size() < 3 || clean.accepted < 2) { std::printf("corpus too small\n"); return 1; }

    std::mt19937 rng(1);
    Tally mutated;
    const std::string tmp = scratch + "/mutated.bin";
    for (int it = 0; it < mutations; ++it) {
        std::vector<unsigned char> bytes = corpus[rng() % corpus.size()];
        if (bytes.empty()) continue;
        const int edits = 1 + static_cast<int>(rng() % 4);
        for (int k = 0; k < edits && !bytes.empty(); ++k) {
            switch (rng() % 5) {
                case 0: bytes[rng() % bytes.size()] = static_cast<unsigned char>(rng()); break;
                case 1: bytes[rng() % bytes.size()] ^= static_cast<unsigned char>(1u << (rng() % 8)); break;
                case 2: if (bytes.size() > 10) bytes.resize(bytes.size() - 1 - rng() % 8); break;
                case 3: bytes.insert(bytes.begin() + static_cast<long>(rng() % bytes.size()), static_cast<unsigned char>(rng())); break;
                case 4: {  // a big-endian length or size field set to an extreme
                    const std::size_t at = rng() % bytes.size();
                    const unsigned char extreme[4] = {0xff, 0x7f, 0x00, 0x80};
                    for (std::size_t b = 0; b < 4 && at + b < bytes.size(); ++b) bytes[at + b] = extreme[(rng() + b) % 4];
                } break;
            }
        }
        if (!spit(tmp, bytes)) { std::printf("cannot write %s\n", tmp.c_str()); return 1; }
        if (!try_file(tmp, mutated)) { std::printf("inconsistent result for mutation %d\n", it); return 1; }
    }
    std::remove(tmp.c_str());
    std::printf("sanitized host tier ok: %d api cases, %d tester calls, %d command lines accepted, corpus %zu files, "
                "%ld mutations accepted, %ld rejected\n",
                cases, tester_calls, configs, corpus.size(), mutated.accepted, mutated.rejected);
    return 0;
}
