// Command line of the splatting trainer: the arguments, defaults, checks and
// messages of TrainingConfigParser in xyz-autodiff-cuda
// (examples/mini-gaussian-splatting/training_config.cpp:29-146), returned as
// status codes and error text instead of exceptions, plus the options this
// build adds (seed, output directory, image format, checkpoints).
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include "../common.cuh"

namespace {

const char kUsage[] =
    "Usage: %s <lr_center> <lr_scale> <lr_rotation> <lr_color> <lr_opacity> [OPTIONS]\n"
    "\n"
    "Required Arguments:\n"
    "  lr_center      Learning rate for Gaussian center positions\n"
    "  lr_scale       Learning rate for Gaussian scale parameters\n"
    "  lr_rotation    Learning rate for Gaussian rotation parameters\n"
    "  lr_color       Learning rate for Gaussian color parameters\n"
    "  lr_opacity     Learning rate for Gaussian opacity parameters\n"
    "\n"
    "Options:\n"
    "  --target PATH              Target image file path, JPEG, PNG or PPM (required)\n"
    "  --max-iterations N         Maximum training iterations (default: 500)\n"
    "  --save-interval N          Save image every N iterations (default: 25)\n"
    "  --num-gaussians N          Number of Gaussians to use (default: 1000)\n"
    "  --no-save-images           Disable saving intermediate images\n"
    "  --beta1 VALUE              Adam optimizer beta1 parameter (default: 0.9)\n"
    "  --beta2 VALUE              Adam optimizer beta2 parameter (default: 0.999)\n"
    "  --epsilon VALUE            Adam optimizer epsilon parameter (default: 1e-8)\n"
    "  --seed N                   Seed of the initial Gaussians (default: 0)\n"
    "  --output-dir DIR           Where images are written (default: output)\n"
    "  --image-format FORMAT      jpg, png or ppm: the format of those images (default: jpg)\n"
    "  --checkpoint PATH          Write the training state to PATH at the end\n"
    "  --checkpoint-interval N    ... and every N iterations\n"
    "  --resume PATH              Continue from the checkpoint at PATH\n"
    "  --help                     Show this help message\n"
    "\n"
    "Example:\n"
    "  %s 0.01 0.005 0.02 0.01 0.01 --target data/target.png --max-iterations 1000 --save-interval 50\n";

bool copy_path(char (&dst)[1024], const char* src) {
    if (std::strlen(src) >= sizeof dst) return false;
    std::strcpy(dst, src);
    return true;
}

}  // namespace

extern "C" const char* xad_training_usage(void) { return kUsage; }

extern "C" void xad_training_config_defaults(xad_training_config* c) {
    if (!c) return;
    std::memset(c, 0, sizeof *c);
    c->lr_center = c->lr_scale = c->lr_rotation = c->lr_color = c->lr_opacity = 0.01f;
    c->max_iterations = 500;
    c->save_interval = 25;
    c->num_gaussians = 1000;
    c->save_images = 1;
    c->beta1 = 0.9f;
    c->beta2 = 0.999f;
    c->epsilon = 1e-8f;
    c->seed = 0;
    c->checkpoint_interval = 0;
    std::strcpy(c->output_dir, "output");
    std::strcpy(c->image_format, "jpg");
}

extern "C" int xad_training_config_validate(const xad_training_config* c) {
    XAD_REQUIRE(c, "config must not be null");
    XAD_REQUIRE(c->lr_center > 0 && c->lr_scale > 0 && c->lr_rotation > 0 && c->lr_color > 0 && c->lr_opacity > 0,
                "All learning rates must be positive");
    XAD_REQUIRE(c->max_iterations > 0, "Max iterations must be positive");
    XAD_REQUIRE(c->save_interval > 0, "Save interval must be positive");
    XAD_REQUIRE(c->num_gaussians > 0, "Number of Gaussians must be positive");
    XAD_REQUIRE(c->target_image_path[0] != '\0', "Target image path must be specified with --target");
    XAD_REQUIRE(c->beta1 > 0 && c->beta1 < 1, "Beta1 must be in range (0, 1)");
    XAD_REQUIRE(c->beta2 > 0 && c->beta2 < 1, "Beta2 must be in range (0, 1)");
    XAD_REQUIRE(c->epsilon > 0, "Epsilon must be positive");
    XAD_REQUIRE(c->checkpoint_interval >= 0, "Checkpoint interval must not be negative");
    XAD_REQUIRE(c->checkpoint_interval == 0 || c->checkpoint_path[0] != '\0',
                "A checkpoint interval needs a checkpoint path (--checkpoint)");
    XAD_REQUIRE(c->output_dir[0] != '\0', "Output directory must not be empty");
    XAD_REQUIRE(!std::strcmp(c->image_format, "jpg") || !std::strcmp(c->image_format, "png") || !std::strcmp(c->image_format, "ppm"),
                "Image format must be jpg, png or ppm");
    return XAD_OK;
}

extern "C" int xad_training_config_parse(int argc, const char* const* argv, xad_training_config* c) {
    XAD_REQUIRE(c && argv, "config and argv must not be null");
    xad_training_config_defaults(c);
    for (int i = 1; i < argc; ++i)
        if (!std::strcmp(argv[i], "--help")) return XAD_HELP_REQUESTED;
    XAD_REQUIRE(argc >= 6, "Insufficient arguments");
    int at = 1;
    c->lr_center = static_cast<float>(std::atof(argv[at++]));
    c->lr_scale = static_cast<float>(std::atof(argv[at++]));
    c->lr_rotation = static_cast<float>(std::atof(argv[at++]));
    c->lr_color = static_cast<float>(std::atof(argv[at++]));
    c->lr_opacity = static_cast<float>(std::atof(argv[at++]));
    while (at < argc) {
        const std::string arg = argv[at];
        const bool has_value = at + 1 < argc;
        bool path_ok = true;
        if (arg == "--target" && has_value) {
            path_ok = copy_path(c->target_image_path, argv[++at]);
        } else if (arg == "--max-iterations" && has_value) {
            c->max_iterations = std::atoi(argv[++at]);
        } else if (arg == "--save-interval" && has_value) {
            c->save_interval = std::atoi(argv[++at]);
        } else if (arg == "--num-gaussians" && has_value) {
            c->num_gaussians = std::atoi(argv[++at]);
        } else if (arg == "--no-save-images") {
            c->save_images = 0;
        } else if (arg == "--beta1" && has_value) {
            c->beta1 = static_cast<float>(std::atof(argv[++at]));
        } else if (arg == "--beta2" && has_value) {
            c->beta2 = static_cast<float>(std::atof(argv[++at]));
        } else if (arg == "--epsilon" && has_value) {
            c->epsilon = static_cast<float>(std::atof(argv[++at]));
        } else if (arg == "--seed" && has_value) {
            c->seed = std::strtoull(argv[++at], nullptr, 10);
        } else if (arg == "--output-dir" && has_value) {
            path_ok = copy_path(c->output_dir, argv[++at]);
        } else if (arg == "--image-format" && has_value) {
            const char* format = argv[++at];
            XAD_REQUIRE(std::strlen(format) < sizeof c->image_format, "Image format must be jpg, png or ppm");
            std::strcpy(c->image_format, format);
        } else if (arg == "--checkpoint" && has_value) {
            path_ok = copy_path(c->checkpoint_path, argv[++at]);
        } else if (arg == "--checkpoint-interval" && has_value) {
            c->checkpoint_interval = std::atoi(argv[++at]);
        } else if (arg == "--resume" && has_value) {
            path_ok = copy_path(c->resume_path, argv[++at]);
        } else {
            return xad::fail(XAD_ERR_INVALID_ARGUMENT, "Invalid argument: %s", arg.c_str());
        }
        XAD_REQUIRE(path_ok, "Invalid argument: path after %s is too long", arg.c_str());
        ++at;
    }
    return xad_training_config_validate(c);
}
