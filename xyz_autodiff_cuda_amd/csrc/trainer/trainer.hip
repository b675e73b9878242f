// Training run of the splatting example on the current device, and the C ABI
// of the trainer front-end (images, checkpoints).
//
// Host-side counterpart of GaussianSplattingTrainer and GaussianCollection of
// xyz-autodiff-cuda (examples/mini-gaussian-splatting/gaussian_splatting_training.cu:14-181,
// gaussian_parameters.cu:9-116): it owns the device state and drives
// xad_splat_step and xad_adam_step_f32; all arithmetic happens there.
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <new>
#include <string>
#include <vector>

#include "../common.cuh"
#include "../rng.cuh"
#include "checkpoint.h"
#include "image_io.h"

// How far the host may run ahead of the device: every kProbeEvery iterations the count of withheld updates is
// copied to one of kProbeSlots pinned words, and a slot is waited for before it is used again.
constexpr int kProbeEvery = 8;
constexpr int kProbeSlots = 4;

struct xad_trainer {
    xad_training_config config;
    int width = 0, height = 0, gaussians = 0;
    int iteration = 0;
    long long repeated = 0;  // iterations run a second time because their first run did not fit the tile lists
    int device = 0;
    hipStream_t stream = nullptr;
    xad_splat_context* splat = nullptr;
    // one allocation: params | grads | m | v (9G each) | depth (G) | the count of withheld updates (one word)
    float* state = nullptr;
    float* target = nullptr;
    float* image = nullptr;
    const std::uint32_t* overflow_word = nullptr;  // device: not zero while a step's lists have overflowed unseen by the host
    std::uint32_t* probe = nullptr;                // pinned: kProbeSlots copies of the count + one for the final read
    hipEvent_t probe_done[kProbeSlots] = {};
    bool probe_pending[kProbeSlots] = {};

    std::size_t g() const { return static_cast<std::size_t>(gaussians); }
    std::size_t pixels() const { return static_cast<std::size_t>(width) * height; }
    float* params() const { return state; }
    float* grads() const { return state + 9 * g(); }
    float* m() const { return state + 18 * g(); }
    float* v() const { return state + 27 * g(); }
    float* depth() const { return state + 36 * g(); }
    std::uint32_t* withheld() const { return reinterpret_cast<std::uint32_t*>(state + 37 * g()); }
};

namespace {

// Initial values of GaussianCollection::initialize_random
// (gaussian_parameters.cu:27-66), one random stream per row.
void initial_gaussians(const xad_trainer& t, std::vector<float>& params, std::vector<float>& depth) {
    const std::size_t g = t.g();
    params.assign(9 * g, 0.0f);
    depth.assign(g, 0.0f);
    struct Row { int row; float lo, hi; };
    const Row rows[] = {{0, 0.0f, static_cast<float>(t.width)}, {1, 0.0f, static_cast<float>(t.height)},
                        {2, 0.0f, 2.0f}, {3, 0.0f, 2.0f},
                        {5, 0.1f, 0.2f}, {6, 0.1f, 0.2f}, {7, 0.1f, 0.2f}, {8, 0.05f, 0.1f}};
    for (const Row& r : rows) {
        const std::uint64_t key = xad_rng::stream_key(t.config.seed, static_cast<std::uint64_t>(r.row));
        for (std::size_t i = 0; i < g; ++i) {
            float value = xad_rng::uniform(xad_rng::bits(key, i), r.lo, r.hi);
            if (r.row == 2 || r.row == 3) value = std::fmax(1.0f, value);
            params[r.row * g + i] = value;
        }
    }
    const std::uint64_t key = xad_rng::stream_key(t.config.seed, 9);
    for (std::size_t i = 0; i < g; ++i) depth[i] = xad_rng::unit_float(xad_rng::bits(key, i));
}

int bind_device(const xad_trainer* t) {
    XAD_HIP_TRY(hipSetDevice(t->device));
    return XAD_OK;
}

int upload(const xad_trainer* t, float* dst, const float* src, std::size_t count) {
    XAD_HIP_TRY(hipMemcpyAsync(dst, src, count * sizeof(float), hipMemcpyHostToDevice, t->stream));
    XAD_HIP_TRY(hipStreamSynchronize(t->stream));
    return XAD_OK;
}

int download(const xad_trainer* t, float* dst, const float* src, std::size_t count) {
    XAD_HIP_TRY(hipMemcpyAsync(dst, src, count * sizeof(float), hipMemcpyDeviceToHost, t->stream));
    XAD_HIP_TRY(hipStreamSynchronize(t->stream));
    return XAD_OK;
}

int create(const xad_training_config* config, int width, int height, const float* target_rgb, xad_trainer* t) {
    t->config = *config;
    t->width = width;
    t->height = height;
    t->gaussians = config->num_gaussians;
    XAD_HIP_TRY(hipGetDevice(&t->device));
    XAD_HIP_TRY(hipStreamCreate(&t->stream));
    // room for Gaussians that grow during training: four times the default (an overflow costs iterations run twice;
    // the lists take about 16 bytes per pair)
    if (int st = xad_splat_create(width, height, t->gaussians, static_cast<std::size_t>(t->gaussians) * 32 + 4096, &t->splat)) return st;
    // depth is drawn once and never trained: promise that, so that an iteration never waits for the device
    if (int st = xad_splat_set_depth_mode(t->splat, XAD_SPLAT_DEPTH_STATIC)) return st;
    if (int st = xad_splat_overflow_word(t->splat, &t->overflow_word)) return st;
    XAD_HIP_TRY(hipMalloc(&t->state, (37 * t->g() + 1) * sizeof(float)));
    XAD_HIP_TRY(hipMalloc(&t->target, 3 * t->pixels() * sizeof(float)));
    XAD_HIP_TRY(hipMalloc(&t->image, 3 * t->pixels() * sizeof(float)));
    XAD_HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&t->probe), (kProbeSlots + 1) * sizeof(std::uint32_t)));
    for (int k = 0; k <= kProbeSlots; ++k) t->probe[k] = 0;
    for (auto& e : t->probe_done) XAD_HIP_TRY(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    XAD_HIP_TRY(hipMemsetAsync(t->state, 0, (37 * t->g() + 1) * sizeof(float), t->stream));
    XAD_HIP_TRY(hipMemsetAsync(t->image, 0, 3 * t->pixels() * sizeof(float), t->stream));
    std::vector<float> params, depth;
    initial_gaussians(*t, params, depth);
    if (int st = upload(t, t->params(), params.data(), params.size())) return st;
    if (int st = upload(t, t->depth(), depth.data(), depth.size())) return st;
    return upload(t, t->target, target_rgb, 3 * t->pixels());
}

}  // namespace

extern "C" int xad_trainer_create(const xad_training_config* config, int width, int height, const float* target_rgb,
                                  xad_trainer** out) {
    XAD_REQUIRE(config && target_rgb && out, "config, target_rgb and out must not be null");
    XAD_REQUIRE(width > 0 && height > 0, "image size must be positive, got %d x %d", width, height);
    XAD_REQUIRE(config->num_gaussians > 0, "Number of Gaussians must be positive");
    XAD_REQUIRE(config->lr_center > 0 && config->lr_scale > 0 && config->lr_rotation > 0 && config->lr_color > 0 &&
                    config->lr_opacity > 0,
                "All learning rates must be positive");
    XAD_REQUIRE(config->beta1 > 0 && config->beta1 < 1, "Beta1 must be in range (0, 1)");
    XAD_REQUIRE(config->beta2 > 0 && config->beta2 < 1, "Beta2 must be in range (0, 1)");
    XAD_REQUIRE(config->epsilon > 0, "Epsilon must be positive");
    *out = nullptr;
    xad_trainer* t = new (std::nothrow) xad_trainer();
    XAD_REQUIRE(t, "out of host memory");
    const int status = create(config, width, height, target_rgb, t);
    if (status != XAD_OK) {
        // keep the message of the failure, not of the clean-up
        const std::string message = xad_last_error();
        xad_trainer_destroy(t);
        return xad::fail(status, "%s", message.c_str());
    }
    *out = t;
    return XAD_OK;
}

extern "C" void xad_trainer_destroy(xad_trainer* t) {
    if (!t) return;
    (void)hipSetDevice(t->device);
    if (t->stream) (void)hipStreamSynchronize(t->stream);
    if (t->splat) xad_splat_destroy(t->splat);
    if (t->state) (void)hipFree(t->state);
    if (t->target) (void)hipFree(t->target);
    if (t->image) (void)hipFree(t->image);
    if (t->probe) (void)hipHostFree(t->probe);
    for (auto& e : t->probe_done)
        if (e) (void)hipEventDestroy(e);
    if (t->stream) (void)hipStreamDestroy(t->stream);
    delete t;
}

namespace {

// Waits for the stream and takes the count of updates that were withheld since it was last taken.
int take_withheld(xad_trainer* t, std::uint32_t* count) {
    std::uint32_t* slot = t->probe + kProbeSlots;
    XAD_HIP_TRY(hipMemcpyAsync(slot, t->withheld(), sizeof(std::uint32_t), hipMemcpyDeviceToHost, t->stream));
    XAD_HIP_TRY(hipMemsetAsync(t->withheld(), 0, sizeof(std::uint32_t), t->stream));
    XAD_HIP_TRY(hipStreamSynchronize(t->stream));
    for (bool& pending : t->probe_pending) pending = false;  // whatever the probes would say is in this count
    *count = *slot;
    return XAD_OK;
}

}  // namespace

// An iteration that does not report its loss only queues work, so nobody looks at whether its tile lists
// fitted their buffers.  The update is therefore gated on the device: xad_adam_step_gated_f32 leaves
// parameters and moments alone from the first step whose lists overflowed until the host has dealt with it,
// and counts the updates it withheld.  With the parameters frozen every later iteration repeats the one that
// overflowed.  Whenever the host next looks (a reported loss, a probe, the end of the run), it takes that
// count, steps the iteration number back by it, has the lists enlarged by a step that waits, and runs those
// iterations again: every update that is applied used complete gradients and its own step number.
extern "C" int xad_trainer_run(xad_trainer* t, int iterations, double* loss_out) {
    XAD_REQUIRE(t, "trainer must not be null");
    XAD_REQUIRE(iterations >= 0, "iterations must not be negative");
    if (int st = bind_device(t)) return st;
    const xad_training_config& c = t->config;
    const float learning_rates[9] = {c.lr_center, c.lr_center, c.lr_scale, c.lr_scale, c.lr_rotation,
                                     c.lr_color,  c.lr_color,  c.lr_color, c.lr_opacity};
    const int target = t->iteration + iterations;
    bool look = false;  // the next step waits for the device (it follows iterations that have to be run again)
    double unused = 0.0;
    int queued = 0;
    for (;;) {
        while (t->iteration < target) {
            const bool last = t->iteration + 1 == target;
            double* loss = (last && loss_out) ? loss_out : (look ? &unused : nullptr);
            int st = xad_splat_step(t->splat, t->params(), t->depth(), t->target, t->image, t->grads(), loss, t->stream);
            // XAD_ERR_INCOMPLETE: this step is complete, steps before it were not; their updates were withheld,
            // which the count below says more precisely
            if (st != XAD_OK && st != XAD_ERR_INCOMPLETE) return st;
            if (loss) {
                std::uint32_t withheld = 0;
                if (int st = take_withheld(t, &withheld)) return st;
                look = false;
                if (withheld != 0) {
                    // the parameters are those of `withheld` iterations ago: this step belongs to that iteration
                    // number.  The lists fit now; go back and run from there (the step just computed is discarded)
                    t->iteration -= static_cast<int>(withheld);
                    t->repeated += withheld;
                    look = true;
                    continue;
                }
            }
            if (int st = xad_adam_step_gated_f32(t->g(), 9, t->params(), t->grads(), t->m(), t->v(), learning_rates, c.beta1,
                                                 c.beta2, c.epsilon, t->iteration + 1, t->overflow_word, t->withheld(), t->stream))
                return st;
            ++t->iteration;
            if (++queued % kProbeEvery == 0) {
                // a look at the count that costs no wait unless the host is kProbeSlots probes ahead of the device:
                // the probes that have arrived are read, the slot to be used again is waited for
                const int reuse = (queued / kProbeEvery) % kProbeSlots;
                bool withholding = false;
                for (int k = 0; k < kProbeSlots; ++k) {
                    if (!t->probe_pending[k]) continue;
                    if (k == reuse) {
                        XAD_HIP_TRY(hipEventSynchronize(t->probe_done[k]));
                    } else {
                        const hipError_t e = hipEventQuery(t->probe_done[k]);
                        if (e == hipErrorNotReady) continue;
                        XAD_HIP_TRY(e);
                    }
                    t->probe_pending[k] = false;
                    withholding = withholding || t->probe[k] != 0;
                }
                if (withholding) break;  // updates are being withheld: stop queueing, settle below
                XAD_HIP_TRY(hipMemcpyAsync(t->probe + reuse, t->withheld(), sizeof(std::uint32_t), hipMemcpyDeviceToHost, t->stream));
                XAD_HIP_TRY(hipEventRecord(t->probe_done[reuse], t->stream));
                t->probe_pending[reuse] = true;
            }
        }
        std::uint32_t withheld = 0;
        if (int st = take_withheld(t, &withheld)) return st;
        if (withheld == 0 && t->iteration >= target) break;
        t->iteration -= static_cast<int>(withheld);
        t->repeated += withheld;
        look = withheld != 0;
    }
    return XAD_OK;
}

extern "C" long long xad_trainer_repeated_iterations(const xad_trainer* t) { return t ? t->repeated : -1; }

extern "C" int xad_trainer_iteration(const xad_trainer* t) { return t ? t->iteration : -1; }

extern "C" int xad_trainer_download_image(xad_trainer* t, float* rgb) {
    XAD_REQUIRE(t && rgb, "trainer and rgb must not be null");
    if (int st = bind_device(t)) return st;
    return download(t, rgb, t->image, 3 * t->pixels());
}

extern "C" int xad_trainer_get_state(xad_trainer* t, float* params, float* m, float* v, float* depth) {
    XAD_REQUIRE(t, "trainer must not be null");
    if (int st = bind_device(t)) return st;
    if (params)
        if (int st = download(t, params, t->params(), 9 * t->g())) return st;
    if (m)
        if (int st = download(t, m, t->m(), 9 * t->g())) return st;
    if (v)
        if (int st = download(t, v, t->v(), 9 * t->g())) return st;
    if (depth)
        if (int st = download(t, depth, t->depth(), t->g())) return st;
    return XAD_OK;
}

extern "C" int xad_trainer_set_params(xad_trainer* t, const float* params, const float* depth) {
    XAD_REQUIRE(t, "trainer must not be null");
    if (int st = bind_device(t)) return st;
    if (params)
        if (int st = upload(t, t->params(), params, 9 * t->g())) return st;
    if (depth) {
        if (int st = upload(t, t->depth(), depth, t->g())) return st;
        // the renderer keeps the order of the depths it saw first (static mode): it has to order again
        if (int st = xad_splat_set_depth_mode(t->splat, XAD_SPLAT_DEPTH_STATIC)) return st;
    }
    return XAD_OK;
}

extern "C" int xad_trainer_save_checkpoint(xad_trainer* t, const char* path) {
    XAD_REQUIRE(t && path && path[0], "trainer and path must not be null or empty");
    if (int st = bind_device(t)) return st;
    xad_train::CheckpointState state;
    xad_train::CheckpointHeader& h = state.header;
    std::memset(&h, 0, sizeof h);
    h.width = t->width;
    h.height = t->height;
    h.num_gaussians = t->gaussians;
    h.iteration = t->iteration;
    h.lr_center = t->config.lr_center;
    h.lr_scale = t->config.lr_scale;
    h.lr_rotation = t->config.lr_rotation;
    h.lr_color = t->config.lr_color;
    h.lr_opacity = t->config.lr_opacity;
    h.beta1 = t->config.beta1;
    h.beta2 = t->config.beta2;
    h.epsilon = t->config.epsilon;
    h.seed = t->config.seed;
    state.params.resize(9 * t->g());
    state.m.resize(9 * t->g());
    state.v.resize(9 * t->g());
    state.depth.resize(t->g());
    if (int st = xad_trainer_get_state(t, state.params.data(), state.m.data(), state.v.data(), state.depth.data()))
        return st;
    const std::string err = xad_train::write_checkpoint(path, state);
    XAD_REQUIRE(err.empty(), "%s", err.c_str());
    return XAD_OK;
}

extern "C" int xad_trainer_load_checkpoint(xad_trainer* t, const char* path) {
    XAD_REQUIRE(t && path && path[0], "trainer and path must not be null or empty");
    if (int st = bind_device(t)) return st;
    xad_train::CheckpointState state;
    const std::string err = xad_train::read_checkpoint(path, state);
    XAD_REQUIRE(err.empty(), "%s", err.c_str());
    const xad_train::CheckpointHeader& h = state.header;
    XAD_REQUIRE(h.num_gaussians == t->gaussians, "checkpoint holds %d Gaussians, the trainer %d", h.num_gaussians,
                t->gaussians);
    XAD_REQUIRE(h.width == t->width && h.height == t->height, "checkpoint is for a %d x %d image, the trainer for %d x %d",
                h.width, h.height, t->width, t->height);
    if (int st = upload(t, t->params(), state.params.data(), state.params.size())) return st;
    if (int st = upload(t, t->m(), state.m.data(), state.m.size())) return st;
    if (int st = upload(t, t->v(), state.v.data(), state.v.size())) return st;
    if (int st = upload(t, t->depth(), state.depth.data(), state.depth.size())) return st;
    if (int st = xad_splat_set_depth_mode(t->splat, XAD_SPLAT_DEPTH_STATIC)) return st;  // other depths: order again
    t->iteration = h.iteration;
    return XAD_OK;
}

// ---- images ----------------------------------------------------------------------

extern "C" int xad_image_load(const char* path, int* width, int* height, float** rgb) {
    XAD_REQUIRE(path && width && height && rgb, "path, width, height and rgb must not be null");
    xad_train::Image image;
    const std::string err = xad_train::load_image(path, image);
    XAD_REQUIRE(err.empty(), "%s", err.c_str());
    float* copy = static_cast<float*>(std::malloc(image.rgb.size() * sizeof(float)));
    XAD_REQUIRE(copy, "out of host memory");
    std::memcpy(copy, image.rgb.data(), image.rgb.size() * sizeof(float));
    *width = image.width;
    *height = image.height;
    *rgb = copy;
    return XAD_OK;
}

extern "C" void xad_image_free(float* rgb) { std::free(rgb); }

extern "C" int xad_image_save(const char* path, int width, int height, const float* rgb) {
    XAD_REQUIRE(path && rgb, "path and rgb must not be null");
    XAD_REQUIRE(width > 0 && height > 0, "image size must be positive, got %d x %d", width, height);
    const std::string err = xad_train::save_image(path, width, height, rgb);
    XAD_REQUIRE(err.empty(), "%s", err.c_str());
    return XAD_OK;
}

extern "C" int xad_image_save_jpeg(const char* path, int width, int height, const float* rgb, int quality) {
    XAD_REQUIRE(path && rgb, "path and rgb must not be null");
    XAD_REQUIRE(width > 0 && height > 0, "image size must be positive, got %d x %d", width, height);
    XAD_REQUIRE(quality >= 1 && quality <= 100, "JPEG quality must be within 1..100, got %d", quality);
    const std::string err = xad_train::save_image_jpeg(path, width, height, rgb, quality);
    XAD_REQUIRE(err.empty(), "%s", err.c_str());
    return XAD_OK;
}

extern "C" int xad_image_test_pattern(int width, int height, float* rgb) {
    XAD_REQUIRE(rgb, "rgb must not be null");
    XAD_REQUIRE(width > 0 && height > 0, "image size must be positive, got %d x %d", width, height);
    xad_train::test_pattern(width, height, rgb);
    return XAD_OK;
}
