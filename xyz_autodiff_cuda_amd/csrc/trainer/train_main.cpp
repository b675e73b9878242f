// xad_splat_train: fits 2D Gaussians to a target image.
//
// The program of examples/mini-gaussian-splatting/gaussian_splatting_training.cu
// in xyz-autodiff-cuda (main, :183-232, and GaussianSplattingTrainer::train,
// :110-181) on top of the C ABI of libxad_hip.so: same command line, same
// progress lines, image schedule and image names (JPEG snapshots unless
// --image-format says otherwise), and optional checkpoints.
#include <sys/stat.h>

#include <chrono>
#include <cstdio>
#include <string>
#include <vector>

#include "../../../include/xad_capi.h"

namespace {

int fail(const char* what) {
    std::fprintf(stderr, "%s: %s\n", what, xad_last_error());
    return 1;
}

bool save_rendering(xad_trainer* trainer, const xad_training_config& config, int width, int height, int iteration,
                    std::vector<float>& scratch) {
    if (xad_trainer_download_image(trainer, scratch.data()) != XAD_OK) return false;
    char name[64];
    std::snprintf(name, sizeof name, "/iteration_%06d.%s", iteration, config.image_format);  // gaussian_splatting_training.cu:106
    const std::string path = std::string(config.output_dir) + name;
    if (xad_image_save(path.c_str(), width, height, scratch.data()) != XAD_OK) return false;
    std::printf("Saved image: %s\n", path.c_str());
    return true;
}

}  // namespace

int main(int argc, char** argv) {
    std::printf("Gaussian Splatting Training with HIP Automatic Differentiation\n");
    std::printf("===============================================================\n");

    xad_training_config config;
    const int parsed = xad_training_config_parse(argc, argv, &config);
    if (parsed == XAD_HELP_REQUESTED) {
        std::printf(xad_training_usage(), argv[0], argv[0]);
        return 0;
    }
    if (parsed != XAD_OK) {
        std::fprintf(stderr, xad_training_usage(), argv[0], argv[0]);
        std::fprintf(stderr, "Failed to parse arguments: %s\n", xad_last_error());
        return 1;
    }

    int width = 0, height = 0;
    float* loaded = nullptr;
    std::vector<float> target;
    std::printf("Loading target image: %s\n", config.target_image_path);
    if (xad_image_load(config.target_image_path, &width, &height, &loaded) == XAD_OK) {
        target.assign(loaded, loaded + static_cast<std::size_t>(width) * height * 3);
        xad_image_free(loaded);
    } else {
        // gaussian_splatting_training.cu:47-50: fall back to the 256 x 256 test pattern
        std::printf("Failed to load image (%s), creating test image instead...\n", xad_last_error());
        width = height = 256;
        target.resize(static_cast<std::size_t>(width) * height * 3);
        xad_image_test_pattern(width, height, target.data());
    }
    std::printf("Target image: %dx%d (3 channels)\n", width, height);

    xad_trainer* trainer = nullptr;
    if (xad_trainer_create(&config, width, height, target.data(), &trainer) != XAD_OK) return fail("Failed to set up training");
    if (config.resume_path[0]) {
        if (xad_trainer_load_checkpoint(trainer, config.resume_path) != XAD_OK) return fail("Failed to resume");
        std::printf("Resumed from %s at iteration %d\n", config.resume_path, xad_trainer_iteration(trainer));
    }

    std::printf("\n=== Starting Gaussian Splatting Training ===\n");
    std::printf("Target image: %dx%d\nGaussians: %d\n", width, height, config.num_gaussians);
    std::printf("Learning rates: center %g, scale %g, rotation %g, color %g, opacity %g\n", config.lr_center, config.lr_scale,
                config.lr_rotation, config.lr_color, config.lr_opacity);
    std::printf("Adam: beta1 %g, beta2 %g, epsilon %g\n", config.beta1, config.beta2, config.epsilon);
    std::printf("Max iterations %d, save interval %d, save images %s\n", config.max_iterations, config.save_interval,
                config.save_images ? "yes" : "no");

    std::vector<float> scratch(target.size());
    if (config.save_images) {
        if (mkdir(config.output_dir, 0777) != 0) {
            struct stat info;
            if (stat(config.output_dir, &info) != 0 || !S_ISDIR(info.st_mode))
                std::fprintf(stderr, "[warning]: failed to make directory %s\n", config.output_dir);
        }
        const std::string path = std::string(config.output_dir) + "/target." + config.image_format;  // :124
        if (xad_image_save(path.c_str(), width, height, target.data()) != XAD_OK) return fail("Failed to save the target");
    }

    const double pixels = static_cast<double>(width) * height;
    for (int iteration = xad_trainer_iteration(trainer); iteration < config.max_iterations; ++iteration) {
        const auto start = std::chrono::steady_clock::now();
        const bool report = iteration % 10 == 0;
        double loss = 0.0;
        if (xad_trainer_run(trainer, 1, report ? &loss : nullptr) != XAD_OK) return fail("Training failed");
        if (report) {
            const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - start).count();
            std::printf("Iteration %4d | average Loss: %.6e | Time: %.3fms\n", iteration, loss / pixels, ms);
        }
        if (config.save_images && iteration % config.save_interval == 0)
            if (!save_rendering(trainer, config, width, height, iteration, scratch)) return fail("Failed to save an image");
        if (config.checkpoint_interval > 0 && (iteration + 1) % config.checkpoint_interval == 0)
            if (xad_trainer_save_checkpoint(trainer, config.checkpoint_path) != XAD_OK) return fail("Failed to write a checkpoint");
    }
    if (config.save_images)
        if (!save_rendering(trainer, config, width, height, config.max_iterations, scratch)) return fail("Failed to save an image");
    if (config.checkpoint_path[0]) {
        if (xad_trainer_save_checkpoint(trainer, config.checkpoint_path) != XAD_OK) return fail("Failed to write a checkpoint");
        std::printf("Checkpoint: %s (iteration %d)\n", config.checkpoint_path, xad_trainer_iteration(trainer));
    }
    xad_trainer_destroy(trainer);
    std::printf("Training completed!\nProgram completed successfully!\n");
    return 0;
}
