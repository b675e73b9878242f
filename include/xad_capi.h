/* C ABI of libxad_hip.so: the GPU entry points of the per-thread autodiff hot
 * path on AMD MI355X (gfx950), plus the host-core build of the same templates.
 *
 * xyz-autodiff-cuda has no C ABI, plugin or FFI: its boundary is a C++
 * template API used inside user kernels (kept, header for header, under
 * include/xyz_autodiff/).  What a binding would wrap are the kernels and host
 * launchers that its tests and examples build on top of those templates; each
 * entry point below names the one it stands in for.
 *
 * Conventions
 *   - every pointer documented as "device" is HBM memory of the current HIP
 *     device; "host" pointers are ordinary process memory;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     calls are asynchronous with respect to the host unless stated otherwise;
 *   - the return value is XAD_OK or one of the XAD_ERR_* codes; the text of the
 *     last failure on the calling thread is available from xad_last_error().
 *     (The reference's host helpers throw std::runtime_error instead,
 *     include/xyz_autodiff/util/error_checker.cuh:9-20.)
 *   - nothing here falls back to the CPU: an entry point without the xad_host_
 *     prefix either runs on the GPU or fails;
 *   - the library keeps no global state besides the thread-local error text:
 *     calls from several host threads are independent as long as they do not
 *     share a context object (xad_splat_context, xad_trainer), which serves one
 *     call at a time, or write to the same device memory.
 */
#ifndef XAD_CAPI_H
#define XAD_CAPI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define XAD_OK 0
#define XAD_ERR_INVALID_ARGUMENT 1 /* null pointer, bad size, bad enum value    */
#define XAD_ERR_HIP 2              /* a HIP runtime call or kernel launch failed */
#define XAD_ERR_UNSUPPORTED 3      /* valid request this build cannot serve      */
#define XAD_ERR_INCOMPLETE 5       /* an earlier asynchronous call came out incomplete (see xad_splat_step) */

/* Text of the most recent error on this thread ("" if none). */
const char* xad_last_error(void);

/* ABI revision of this library; bumped on incompatible changes. */
int xad_abi_version(void);

/* SHA-256 (hex) of the sources this library was built from, as computed by its
 * build script; "" for a build that did not record it.  Lets a loader refuse a
 * library that is older than the sources next to it. */
const char* xad_source_digest(void);

/* ---------------------------------------------------------------------------
 * Per-thread forward + backward of the benchmark graph, structure of arrays.
 *
 *   es = exp((sx, sy)); Sigma = R(theta) diag(es)^2 R(theta)^T; q = p^T Sigma^-1 p;
 *   w = sigmoid(o) * exp(-q / 2);   outputs: w and d w / d (sx, sy, theta, o, px, py)
 *
 * Six device input arrays and seven device output arrays of n floats each; no
 * two output arrays may overlap each other or an input.  Any 4-byte alignment
 * is accepted.  n may be 0.
 * Stands in for the per-Gaussian graph that gaussian_splatting_kernel builds
 * and runs per (pixel, Gaussian)
 * (examples/mini-gaussian-splatting/gaussian_splatting_kernel.cu:73-111) and for
 * the <<<1,1>>> graph kernels of the reference tests (tests/test_dag_backward.cu:43-67).
 */
int xad_chain_forward_backward_f32(size_t n,
                                   const float* sx, const float* sy, const float* theta,
                                   const float* o, const float* px, const float* py,
                                   float* w, float* d_sx, float* d_sy, float* d_theta,
                                   float* d_o, float* d_px, float* d_py,
                                   void* stream);

/* The same graph from the same templates, compiled for the host and run on
 * `num_threads` host threads (<= 0: all hardware threads).  Host pointers.
 * Synchronous.  This is the "host-core run of the per-thread templates"; GPU
 * entry points never route through it. */
int xad_host_chain_forward_backward_f32(size_t n,
                                        const float* sx, const float* sy, const float* theta,
                                        const float* o, const float* px, const float* py,
                                        float* w, float* d_sx, float* d_sy, float* d_theta,
                                        float* d_o, float* d_px, float* d_py,
                                        int num_threads);
int xad_host_chain_forward_backward_f64(size_t n,
                                        const double* sx, const double* sy, const double* theta,
                                        const double* o, const double* px, const double* py,
                                        double* w, double* d_sx, double* d_sy, double* d_theta,
                                        double* d_o, double* d_px, double* d_py,
                                        int num_threads);

/* ---------------------------------------------------------------------------
 * Parallel gradient accumulation.  Thread i evaluates the graph above on
 * (sx[i], ..., py[i]) and adds its six gradients (d_sx, d_sy, d_theta, d_o, d_px,
 * d_py) into row slot[i] of `grads`, a device array of num_slots x 6 floats,
 * row-major, which the caller has initialised (the kernel only adds).  Entries
 * of slot outside [0, num_slots) contribute nothing.  Floating-point sums are
 * accumulated in an order that varies from run to run.
 * `strategy` selects how the sums reach HBM:
 *   GLOBAL_ATOMICS  one global atomic per thread per element: the pattern of
 *                   VariableRef::add_grad (include/xyz_autodiff/variable.cuh:48-50;
 *                   tests/test_parallel_gradient_accumulation.cu:25-49);
 *   AUTO            the fastest measured at every slot count from 1 to 1 Mi: LDS while
 *                   one fp64 table holds every slot (3072 slots); beyond that the
 *                   whole LDS of a CU as fp64 rows for the first ~3000 slots (the
 *                   hottest 32 in several copies), every other slot's contributions
 *                   gathered per wavefront in LDS and written to HBM sixteen rows
 *                   at a time, coalesced.  Every input is read once.  That layout
 *                   suits a law that falls with the slot index; a block whose first
 *                   1024 slots say otherwise (fewer than half of them own a row)
 *                   claims 2048 rows on first use instead;
 *   LDS             per-block table of partial sums in LDS, written out once per
 *                   block (the reference's shared-memory pattern,
 *                   tests/test_shared_memory_atomic.cu:29-64, made persistent).
 *                   The table is fp64 (ds_add_f64) while num_slots x 6 doubles fit
 *                   in 144 KiB of LDS (3072 slots), kept in up to 16 copies while
 *                   those fit in 48 KiB so that lanes sharing a slot do not share an
 *                   address; up to 6144 slots the slots are
 *                   dealt to two fp64 tables served by two sets of blocks; beyond
 *                   that rows are claimed on first use (2048 fp64 rows up to
 *                   262 144 slots, 4096 fp32 rows above) and the rest falls
 *                   through to HBM.  LDS_F32 forces fp32 tables (one for all slots
 *                   up to 6144, 4096 claimed rows above);
 *   WAVE_LDS        DPP pre-reduction of equal slots inside each wavefront (groups
 *                   of >= 4 lanes, up to eight groups per call), then as LDS;
 *                   WAVE_LDS_SHALLOW: at most two groups;
 *   *_LEAVES        the same kernels with the graph's leaves bound straight to
 *                   the accumulator (drop-in leaf type), element by element.
 */
#define XAD_ACCUMULATE_GLOBAL_ATOMICS 0
#define XAD_ACCUMULATE_LDS 1
#define XAD_ACCUMULATE_WAVE_LDS 2
#define XAD_ACCUMULATE_WAVE_LDS_SHALLOW 3
#define XAD_ACCUMULATE_LDS_LEAVES 4
#define XAD_ACCUMULATE_GLOBAL_LEAVES 5
#define XAD_ACCUMULATE_LDS_F32 6
#define XAD_ACCUMULATE_AUTO 7
int xad_accumulate_chain_gradients_f32(int strategy, size_t n,
                                       const float* sx, const float* sy, const float* theta,
                                       const float* o, const float* px, const float* py,
                                       const int* slot, float* grads, int num_slots,
                                       void* stream);

/* ---------------------------------------------------------------------------
 * Tile-binned 2D Gaussian splatting: render, loss and parameter gradients.
 *
 * Stands in for launch_gaussian_splatting of the reference example
 * (examples/mini-gaussian-splatting/gaussian_splatting_kernel.cu:114-149), which
 * renders, accumulates the loss and accumulates all gradients in one launch, and
 * for zero_gradients_gpu (gaussian_parameters.cu:243-257): gradients are written,
 * not added, so no separate zeroing call exists.  The per-Gaussian opacity graph
 * is the reference's; the renderer around it is the one the benchmark
 * configuration specifies (16x16 tiles, 3-sigma box binning, (depth, index)
 * order, front-to-back compositing with alpha <= 0.99, stop below T = 1e-4, sum
 * of squared errors), not the reference's additive all-pairs renderer.
 *
 *   params  device, 9 rows of G floats: cx, cy, log-scale x, log-scale y, theta,
 *           r, g, b, opacity logit (the fields of GaussianParams,
 *           gaussian_parameters.h:12-18, as a structure of arrays)
 *   depth   device, G floats (ordering only; not differentiated)
 *   target, image   device, height x width x 3 floats, interleaved RGB
 *   grads   device, 9 rows of G floats, overwritten
 *
 * The context owns all intermediate device buffers (records, tile lists, per-pixel
 * state, binning workspace) in two allocations, one sized by (G, image), one by
 * the capacity of the tile lists in (tile, Gaussian) pairs.  One context serves
 * one stream at a time and belongs to the device that was current when it was
 * created.
 *
 * When the host waits.  The tile lists are built on the device without any
 * read-back (no sort; see csrc/splat_binning.hip).  The host looks at what the
 * device found only
 *   - in the first call after the lists were sized (creation, or enlargement):
 *     did the pairs fit?  If not the lists are enlarged and the binning redone;
 *   - in every call of the default depth mode, XAD_SPLAT_DEPTH_CHECKED: did any
 *     depth change since the call that last ordered the Gaussians?  (The order by
 *     (depth, index) is kept between calls; one changed bit reorders.)
 *   - when the caller asks for the loss.
 * A caller whose depths do not change sets XAD_SPLAT_DEPTH_STATIC (a promise:
 * depth is read by the first call and assumed unchanged afterwards); one whose
 * depths change all the time sets XAD_SPLAT_DEPTH_EVERY_STEP (the order is
 * recomputed by every call, on the device).  In both modes a step with
 * loss_out == NULL only queues work.  What such a call cannot report itself is
 * reported by the next call that waits (a step with loss_out, xad_splat_get_stats,
 * xad_splat_get_lists): XAD_ERR_INCOMPLETE if a step produced more pairs than the
 * lists held (its image and gradients lack the pairs that did not fit; the lists
 * are enlarged at that point), XAD_ERR_INVALID_ARGUMENT if a depth changed under
 * the static promise.  The outputs of a step that returns such a status are
 * themselves complete.  A caller that must not act on incomplete gradients without
 * waiting for them gates its update on the device: see xad_splat_overflow_word.
 *
 * Recording.  In XAD_SPLAT_DEPTH_STATIC mode, after a step with loss_out has
 * returned (the lists are sized then), xad_splat_step with loss_out == NULL is a
 * fixed sequence of kernel launches on `stream`, with no allocation, copy or fill
 * and no host-side state that a launch depends on: it may be recorded by HIP
 * stream capture and the graph replayed, for as long as the context is used by
 * nothing else in between that changes its buffers (a call that reports
 * XAD_ERR_INCOMPLETE enlarges them: record again after it).  Profiling must be off.
 */
typedef struct xad_splat_context xad_splat_context;
int xad_splat_create(int width, int height, int num_gaussians, size_t pair_capacity_hint,
                     xad_splat_context** out);
void xad_splat_destroy(xad_splat_context* ctx);
/* Render only.  In XAD_SPLAT_DEPTH_CHECKED mode the call waits for the binning
 * anyway and enlarges the lists itself when the scene has outgrown them, so its
 * image is always complete; in the other two modes what is said above of calls
 * that only queue work applies. */
int xad_splat_forward(xad_splat_context* ctx, const float* params, const float* depth,
                      float* image, void* stream);
/* Render, loss and gradients.  loss_out (host, may be NULL) receives the sum of
 * squared errors; passing it makes the call wait for the stream (and, should this
 * very step not fit the lists, enlarge them and run it again). */
int xad_splat_step(xad_splat_context* ctx, const float* params, const float* depth,
                   const float* target, float* image, float* grads, double* loss_out,
                   void* stream);
#define XAD_SPLAT_DEPTH_CHECKED 0
#define XAD_SPLAT_DEPTH_STATIC 1
#define XAD_SPLAT_DEPTH_EVERY_STEP 2
int xad_splat_set_depth_mode(xad_splat_context* ctx, int mode);
/* Per-stage GPU times (events around depth order, project, binning, render
 * forward, render backward, parameter backward) are recorded by the next calls
 * when enabled; recording makes each call wait for the stream. */
int xad_splat_set_profiling(xad_splat_context* ctx, int enabled);
/* Of the last call: number of (tile, Gaussian) pairs, longest tile list (either
 * makes the call wait for the device, and reports what calls that did not wait
 * have left behind, see above), and the six stage times in milliseconds (zeros
 * unless profiling is enabled; the first is the depth order, close to zero in a
 * call that kept the order it had).  Any output pointer may be NULL. */
int xad_splat_get_stats(xad_splat_context* ctx, uint64_t* pairs, uint32_t* longest_list, float* stage_ms);
/* The tile lists of the last call, to host memory: tile t (row-major) holds
 * gaussians[range_begin[t] .. range_end[t]), in compositing order.  range_begin and
 * range_end: one entry per tile; gaussians (may be NULL): room for `capacity`
 * entries, at least the pair count.  Waits for the device. */
int xad_splat_get_lists(xad_splat_context* ctx, uint32_t* range_begin, uint32_t* range_end,
                        uint32_t* gaussians, size_t capacity);
/* Device address of one 32-bit word that is zero as long as every step since the
 * host last looked fitted the lists, and not zero from the binning of the first
 * step that did not until a call that waits has enlarged them.  Work queued behind
 * a step on the same stream may read it to decide on the device whether to use
 * that step's gradients (xad_adam_step_gated_f32).  Valid for the context's life.
 * No counterpart in the reference, whose one kernel needs no lists. */
int xad_splat_overflow_word(xad_splat_context* ctx, const uint32_t** device_word);
/* The order in which the step composites: order[i] (device, n words) = the i-th
 * Gaussian by (depth, index), rank (device, n words) its inverse.  A stable radix
 * sort on the device (csrc/splat_sort.hip), the one xad_splat_step runs whenever
 * it has to order (every call in XAD_SPLAT_DEPTH_EVERY_STEP mode).  -0.0 and +0.0
 * are one depth; a NaN sorts by its bit pattern (first with the sign bit set, last
 * without).  n < 2^30.  Allocates its workspace and waits for the stream.
 * No counterpart in the reference, which composites in index order
 * (gaussian_splatting_kernel.cu:33-62). */
int xad_depth_order_f32(size_t n, const float* depth, uint32_t* order, uint32_t* rank, void* stream);
/* The same step on the host cores, every pointer host memory: the CPU figure the
 * GPU step is reported beside.  Tiles are dealt to num_threads threads (0: one per
 * hardware thread); every (pixel, Gaussian) pair builds the renderer's per-pair
 * graph from the library's nodes and runs its forward() and backward()
 * (examples/mini-gaussian-splatting/gaussian_splatting_kernel.cu:42-55, :86-97),
 * the parameters pass through the projection graph as on the GPU.  grads may be
 * NULL (render and loss only); loss_out and pairs_out (number of (tile, Gaussian)
 * pairs) may be NULL.  No entry of a list is skipped, so sums differ from the GPU
 * step's by rounding and by terms with alpha below 1e-8. */
int xad_host_splat_step_f32(int width, int height, int num_gaussians, const float* params,
                            const float* depth, const float* target, float* image, float* grads,
                            double* loss_out, uint64_t* pairs_out, int num_threads);

/* Adam over structure-of-arrays parameters: `rows` rows of n floats each in
 * params, grads, m and v (device); row r uses row_learning_rates[r] (host).
 * iteration counts from 1.  Arithmetic of adam_step_individual_kernel
 * (examples/mini-gaussian-splatting/gaussian_parameters.cu:260-320, launcher
 * :353-386); no clamping. */
int xad_adam_step_f32(size_t n, int rows, float* params, const float* grads, float* m, float* v,
                      const float* row_learning_rates, float beta1, float beta2, float eps,
                      int iteration, void* stream);
/* The same update, decided on the device: the kernel first reads *hold_if_nonzero
 * (device) and, if it is not zero, changes nothing and adds one to *held_count
 * (device, may be NULL).  For training loops that do not wait for the device
 * between the gradients and the update (the reference's loop computes all
 * gradients, then steps, gaussian_splatting_training.cu:127-160: an update never
 * sees partial gradients there). */
int xad_adam_step_gated_f32(size_t n, int rows, float* params, const float* grads, float* m, float* v,
                            const float* row_learning_rates, float beta1, float beta2, float eps,
                            int iteration, const uint32_t* hold_if_nonzero, uint32_t* held_count,
                            void* stream);

/* ---------------------------------------------------------------------------
 * Splatting trainer front-end: configuration, image files, training loop,
 * checkpoints.  Host-side counterpart of the reference's training program
 * (examples/mini-gaussian-splatting/gaussian_splatting_training.cu,
 * training_config.{h,cpp}, image_utils.{h,cpp}, GaussianCollection in
 * gaussian_parameters.{h,cu}), around xad_splat_step and xad_adam_step_f32.
 */

/* The fields of TrainingConfig (training_config.h:7-31) with its defaults,
 * followed by the additions of this build (seed, output directory, checkpoints, image format). */
typedef struct xad_training_config {
    float lr_center, lr_scale, lr_rotation, lr_color, lr_opacity;
    int max_iterations;   /* 500 */
    int save_interval;    /* 25: an image every so many iterations */
    int num_gaussians;    /* 1000 */
    int save_images;      /* 1 */
    float beta1, beta2, epsilon; /* 0.9, 0.999, 1e-8 */
    char target_image_path[1024];
    /* additions */
    uint64_t seed;               /* 0: initial Gaussians are a function of the seed */
    int checkpoint_interval;     /* 0 = only at the end (when checkpoint_path is set) */
    char output_dir[1024];       /* "output" */
    char checkpoint_path[1024];  /* "" = write none */
    char resume_path[1024];      /* "" = start from random Gaussians */
    char image_format[8];        /* "jpg" (what the reference writes), "png" or "ppm": the program's snapshots */
} xad_training_config;

#define XAD_HELP_REQUESTED 4 /* returned by xad_training_config_parse for --help */

void xad_training_config_defaults(xad_training_config* config);
/* argv as given to main: <lr_center> <lr_scale> <lr_rotation> <lr_color>
 * <lr_opacity> then --target PATH, --max-iterations N, --save-interval N,
 * --num-gaussians N, --no-save-images, --beta1 V, --beta2 V, --epsilon V, --help
 * (TrainingConfigParser::parse, training_config.cpp:29-88) and, added here,
 * --seed N, --output-dir DIR, --image-format jpg|png|ppm, --checkpoint PATH,
 * --checkpoint-interval N, --resume PATH.  Fails like the reference: fewer than five positional
 * arguments "Insufficient arguments", an unknown option or an option without
 * its value "Invalid argument", then the checks of validate_config
 * (training_config.cpp:114-146) with its messages. */
int xad_training_config_parse(int argc, const char* const* argv, xad_training_config* config);
int xad_training_config_validate(const xad_training_config* config);
/* The usage text (training_config.cpp:90-112). */
const char* xad_training_usage(void);

/* Image files: float RGB in [0, 1], height x width x 3, host memory.
 * xad_image_load (load_image, image_utils.cpp:12-36) reads a PNG, a JPEG
 * (Huffman-coded, sequential or progressive, grey or colour), an uncompressed
 * BMP or a binary PPM/PGM, told apart by their first bytes, and allocates *rgb (release with
 * xad_image_free); xad_image_save writes 8-bit JPEG (quality 90), PNG or PPM by
 * the extension of `path` (.jpg / .jpeg / .png / .ppm); xad_image_save_jpeg is
 * save_image_jpeg (image_utils.cpp:38-56; quality 1..100, 90 being its default):
 * bytes are (unsigned char)(clamped * 255 + 0.5) as there (:42-46);
 * xad_image_test_pattern fills the gradient of create_test_image (:58-77). */
int xad_image_load(const char* path, int* width, int* height, float** rgb);
void xad_image_free(float* rgb);
int xad_image_save(const char* path, int width, int height, const float* rgb);
int xad_image_save_jpeg(const char* path, int width, int height, const float* rgb, int quality);
int xad_image_test_pattern(int width, int height, float* rgb);

/* A training run on the current device: parameters, gradients and Adam moments
 * (9 rows x num_gaussians each, rows as in xad_splat_step), the target and the
 * last rendering stay on the device.
 *
 * Initial Gaussians follow GaussianCollection::initialize_random
 * (gaussian_parameters.cu:27-66): centre uniform over the image, log-scales
 * max(1, U(0, 2)), rotation 0, colour U(0.1, 0.2), opacity logit U(0.05, 0.1),
 * drawn from the counter-based generator with config->seed; depth (which the
 * reference does not have) is U(0, 1) and is not trained.
 * One iteration is the body of GaussianSplattingTrainer::train
 * (gaussian_splatting_training.cu:127-160): gradients of the loss, then Adam
 * with the five learning rates and iteration + 1 as the step count. */
typedef struct xad_trainer xad_trainer;
int xad_trainer_create(const xad_training_config* config, int width, int height,
                       const float* target_rgb, xad_trainer** out);
void xad_trainer_destroy(xad_trainer* trainer);
/* Runs `iterations` iterations.  loss_out (host, may be NULL) receives the sum
 * of squared errors of the last iteration's rendering, taken before its update.
 * Only an iteration that reports its loss waits for the device (and the host
 * stays at most 32 iterations ahead of it).  No update is ever applied to
 * gradients from tile lists that had outgrown their buffers: such an update is
 * withheld on the device, and when the host next looks the buffers are enlarged
 * and the iterations since then are run again with their own step numbers, so
 * the result is that of a run whose buffers were ample from the start. */
int xad_trainer_run(xad_trainer* trainer, int iterations, double* loss_out);
/* Iterations that had to be run a second time for that reason, over the trainer's life. */
long long xad_trainer_repeated_iterations(const xad_trainer* trainer);
/* Iterations completed so far (continues from the checkpoint after a load). */
int xad_trainer_iteration(const xad_trainer* trainer);
/* The last rendering (zeros before the first iteration), to host memory. */
int xad_trainer_download_image(xad_trainer* trainer, float* rgb);
/* Copies of the state to host memory (9 x num_gaussians floats each, depth
 * num_gaussians); any pointer may be NULL. */
int xad_trainer_get_state(xad_trainer* trainer, float* params, float* m, float* v, float* depth);
/* Replaces parameters and depth (host memory; NULL keeps the current ones). */
int xad_trainer_set_params(xad_trainer* trainer, const float* params, const float* depth);
/* Checkpoint = iteration count, image size, Gaussian count, learning rates and
 * Adam constants, parameters, both Adam moments and depth, with a CRC-32 over
 * the file.  Written to a temporary file and renamed.  Loading requires the
 * same image size and Gaussian count and replaces iteration, parameters,
 * moments and depth (the trainer's own configuration is kept).  The reference
 * only mirrors its state to host memory (gaussian_parameters.cu:93-116). */
int xad_trainer_save_checkpoint(xad_trainer* trainer, const char* path);
int xad_trainer_load_checkpoint(xad_trainer* trainer, const char* path);

/* ---------------------------------------------------------------------------
 * Least-squares fit of  y ~ (x1 - a)^2 + b (x2 - c)^2 + d  by mini-batch SGD, fp64:
 * four parameters shared by every sample, the extreme-contention case of
 * gradient accumulation.
 *
 * Stands in for the kernels of examples/optimization/linear_regression_sgd.cu:
 * select_batch_kernel (:68-81), parallel_gradient_computation_kernel (:86-123),
 * update_parameters_kernel (:126-134) and the loop of main (:186-229).  The
 * per-sample graph is the one of
 * examples/optimization/tests/test_linear_regression_gradient.cu:47-78, i.e. the
 * squared residual (the example itself differentiates the un-squared node,
 * :119-122, on a batch of one, :204-208).  Samples are three arrays, not an
 * array of {x1, x2, y} structs.
 *
 *   strategy  how the four gradients of all samples are summed:
 *     GLOBAL_ATOMICS  VariableRef leaves on the global gradient, one fp64 atomic
 *                     per sample and parameter (the reference pattern)
 *     LDS_LEAVES      the same graph with accumulator leaves (per-block LDS
 *                     table, one global atomic per block and element)
 *     WAVE_LDS        register leaves, per-lane running sums, wavefront
 *                     reduction, then the LDS table
 *   x1, x2, y   device, `total` doubles each
 *   rows        device, n sample indices into x1/x2/y, or NULL for samples 0..n-1
 *   params      device, 4 doubles: a, b, c, d
 *   out         device, 5 doubles, overwritten: sum over the n samples of
 *               d loss / d (a, b, c, d) and of loss = (prediction - y)^2
 */
#define XAD_LINREG_GLOBAL_ATOMICS 0
#define XAD_LINREG_LDS_LEAVES 1
#define XAD_LINREG_WAVE_LDS 2
int xad_linreg_gradient_f64(int strategy, size_t n, size_t total,
                            const double* x1, const double* x2, const double* y, const int* rows,
                            const double* params, double* out, void* stream);
/* `epochs` SGD steps, entirely on the device: step e draws `batch` rows with
 * replacement, row of draw i = random bits (seed, stream 0, e * batch + i)
 * modulo total (see xad_host_rng_bits), sums the gradients with WAVE_LDS, and
 * updates  p -= lr(e) * sum / batch  with  lr(e) = lr_first * (lr_last /
 * lr_first)^(e / epochs)  (linear_regression_sgd.cu:137-140).  params (device, 4
 * doubles) is updated in place; loss_history (device, `epochs` doubles, or NULL)
 * receives the mean batch loss before each update.  Synchronous: returns when
 * the last step has finished. */
int xad_linreg_sgd_f64(size_t total, const double* x1, const double* x2, const double* y,
                       double* params, int batch, int epochs, double lr_first, double lr_last,
                       uint64_t seed, double* loss_history, void* stream);
/* xad_linreg_sgd_f64 for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No
 * counterpart in the reference.  Same arguments, same kernels and same results
 * as xad_linreg_sgd_f64, with two differences:
 *   - the gradient sums of a step live in a 256-byte array that is part of the
 *     library's device image (one copy per device, held until the process ends)
 *     instead of a buffer allocated and freed by the call; the call makes no
 *     hipMalloc, hipFree or other allocating call and no host-device copy;
 *   - it is asynchronous: it returns when the steps are queued on `stream`;
 *     params and loss_history are final when the stream has run them.
 * The scratch does not depend on total or batch; the one size a call bounds is
 * the number of steps it queues (two launches each): epochs beyond
 * XAD_LINREG_STATIC_MAX_EPOCHS are refused with XAD_ERR_INVALID_ARGUMENT.
 * Every call on a device shares that device's array: calls whose work overlaps
 * on one device (two streams, two host threads) race and give wrong sums; calls
 * on one stream, or ordered by events, are fine, and each call clears the sums
 * before its first step.  The first call on a device looks up the array's
 * address (hipGetSymbolAddress); make it outside graph capture, e.g. with
 * epochs = 0. */
#define XAD_LINREG_STATIC_MAX_EPOCHS (1 << 20)
int xad_linreg_sgd_f64_static(size_t total, const double* x1, const double* x2, const double* y,
                              double* params, int batch, int epochs, double lr_first, double lr_last,
                              uint64_t seed, double* loss_history, void* stream);
/* Host cores: the same graph templates compiled for the CPU, one thread; all
 * pointers host. */
int xad_host_linreg_gradient_f64(size_t n, size_t total,
                                 const double* x1, const double* x2, const double* y, const int* rows,
                                 const double* params, double* out);

/* ---------------------------------------------------------------------------
 * Synthetic inputs: counter-based generator, element i of a fill is a pure
 * function of (seed, stream_id, i).  The reference seeds std::mt19937 on the
 * host and uploads (examples/mini-gaussian-splatting/gaussian_parameters.cu:27-66);
 * these fill device memory in place.
 */
int xad_rng_uniform_f32(float* dst, size_t n, uint64_t seed, uint64_t stream_id,
                        float lo, float hi, void* stream);
int xad_rng_normal_f32(float* dst, size_t n, uint64_t seed, uint64_t stream_id,
                       float mean, float stddev, void* stream);
/* Zipf(exponent) over {0, .., num_slots-1}: P(k) ~ (k+1)^-exponent, by inverse
 * CDF (table built on the host in fp64, binary search on the device with 53
 * random bits).  Synchronous: allocates and frees a temporary device table. */
int xad_rng_zipf_i32(int* dst, size_t n, uint64_t seed, uint64_t stream_id,
                     int num_slots, double exponent, void* stream);
/* Host: the raw 64 random bits of elements first .. first+n-1. */
int xad_host_rng_bits(uint64_t* dst, size_t n, uint64_t seed, uint64_t stream_id, uint64_t first);
int xad_host_rng_uniform_f32(float* dst, size_t n, uint64_t seed, uint64_t stream_id,
                             float lo, float hi);

#ifdef __cplusplus
}
#endif
#endif /* XAD_CAPI_H */
