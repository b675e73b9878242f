// The splatting step behind the C ABI: workspace ownership and stage order.
#include <chrono>
#include <new>

#include "common.cuh"
#include "splat_launch.cuh"

using namespace xad_splat;

struct xad_splat_context {
    int width = 0, height = 0, G = 0;
    int device = 0;  // the device that was current at creation: owns every buffer below
    int tiles_x = 0, tiles_y = 0, tiles = 0;
    int key_bits = 0;        // bits of a tile index: what the pair sort looks at
    bool wide_keys = false;  // more than 65 536 tiles: 32-bit pair keys instead of 16-bit
    std::uint32_t capacity = 0;  // pairs the workspace can hold
    std::uint32_t pairs = 0;     // pairs of the last step
    bool profile = false;

    Record* records = nullptr;
    TileRect* rects = nullptr;
    std::uint32_t* counts = nullptr;   // G + 1
    std::uint32_t* offsets = nullptr;  // G + 2: exclusive scan of counts, then the depth-changed flag
    std::uint32_t *depth_keys = nullptr, *depth_keys_sorted = nullptr;  // G each
    std::uint32_t *identity = nullptr, *by_depth = nullptr;  // G each; by_depth = Gaussians in (depth, index) order
    float* ordered_depth = nullptr;  // G: the depths by_depth was computed from
    bool order_valid = false;
    std::uint32_t* counts_by_depth = nullptr;  // G + 1, the last one stays zero
    void *keys = nullptr, *keys_sorted = nullptr;  // 2 or 4 bytes per pair
    std::uint32_t *ids = nullptr, *ids_sorted = nullptr;
    std::uint32_t *range_begin = nullptr, *range_end = nullptr;
    float* final_T = nullptr;
    std::uint32_t* n_contrib = nullptr;
    float* record_grads = nullptr;  // G x 9
    double* loss = nullptr;
    std::uint32_t* host_pairs = nullptr;  // pinned, 2 words: number of pairs, depth-changed flag
    double* host_loss = nullptr;          // pinned
    void* scan_temp = nullptr;
    std::size_t scan_bytes = 0;
    void* depth_sort_temp = nullptr;
    std::size_t depth_sort_bytes = 0;
    void* sort_temp = nullptr;
    std::size_t sort_bytes = 0;

    static constexpr int kStages = 7;  // project, scan+emit, sort, ranges, render fwd, render bwd, parameter bwd
    hipEvent_t marks[kStages + 1] = {};
    float stage_ms[kStages] = {};
    hipEvent_t count_ready = nullptr;  // the read-back of the pair count has arrived
};

namespace {

int free_pair_buffers(xad_splat_context* c) {
    (void)hipFree(c->keys);
    (void)hipFree(c->keys_sorted);
    (void)hipFree(c->ids);
    (void)hipFree(c->ids_sorted);
    (void)hipFree(c->sort_temp);
    c->keys = c->keys_sorted = nullptr;
    c->ids = c->ids_sorted = nullptr;
    c->sort_temp = nullptr;
    return XAD_OK;
}

int allocate_pair_buffers(xad_splat_context* c, std::uint32_t capacity) {
    free_pair_buffers(c);
    c->capacity = 0;  // stays zero if an allocation below fails: the next call then tries again
    const std::size_t key_bytes = c->wide_keys ? 4 : 2;
    XAD_HIP_TRY(hipMalloc(&c->keys, key_bytes * capacity));
    XAD_HIP_TRY(hipMalloc(&c->keys_sorted, key_bytes * capacity));
    XAD_HIP_TRY(hipMalloc(&c->ids, sizeof(std::uint32_t) * capacity));
    XAD_HIP_TRY(hipMalloc(&c->ids_sorted, sizeof(std::uint32_t) * capacity));
    c->sort_bytes = sort_temp_bytes(capacity, c->wide_keys);
    XAD_HIP_TRY(hipMalloc(&c->sort_temp, c->sort_bytes ? c->sort_bytes : 16));
    c->capacity = capacity;
    return XAD_OK;
}

void mark(xad_splat_context* c, int index, hipStream_t s) {
    if (c->profile) (void)hipEventRecord(c->marks[index], s);
}

// (depth, index) order of the Gaussians, kept until a depth changes
int order_by_depth(xad_splat_context* c, const float* depth, hipStream_t s) {
    c->order_valid = false;
    if (int st = launch_depth_keys(s, c->G, depth, c->depth_keys, c->identity)) return st;
    if (int st = sort_by_depth(s, c->depth_sort_temp, c->depth_sort_bytes, c->depth_keys, c->depth_keys_sorted, c->identity,
                               c->by_depth, c->G))
        return st;
    XAD_HIP_TRY(hipMemcpyAsync(c->ordered_depth, depth, sizeof(float) * c->G, hipMemcpyDeviceToDevice, s));
    c->order_valid = true;
    return XAD_OK;
}

int emit(xad_splat_context* c, hipStream_t s) {
    std::uint32_t* depth_changed = c->offsets + c->G + 1;
    return launch_emit(s, c->G, c->by_depth, c->rects, c->offsets, c->tiles_x, c->wide_keys, c->keys, c->ids, c->capacity,
                       c->range_begin, c->tiles * 2, depth_changed);
}

// Places the pairs (scan of the tile counts in depth order) and emits them.  The number of pairs,
// which sizes the sort, and the depth-changed flag are read back: the one wait of a step.  The
// emission is queued before that wait, so it runs while the host is woken: it needs the offsets,
// not the count, and never writes past the capacity.  (The copy that reads the flag is ahead of
// the emission, which resets it, in the stream.)
int place_and_emit(xad_splat_context* c, hipStream_t s) {
    if (int st = launch_permute_counts(s, c->G, c->by_depth, c->counts, c->counts_by_depth)) return st;
    if (int st = exclusive_scan_counts(s, c->scan_temp, c->scan_bytes, c->counts_by_depth, c->offsets, c->G)) return st;
    XAD_HIP_TRY(hipMemcpyAsync(c->host_pairs, c->offsets + c->G, 2 * sizeof(std::uint32_t), hipMemcpyDeviceToHost, s));
    XAD_HIP_TRY(hipEventRecord(c->count_ready, s));
    if (int st = emit(c, s)) return st;
    XAD_HIP_TRY(hipEventSynchronize(c->count_ready));
    c->pairs = c->host_pairs[0];
    return XAD_OK;
}

// project .. tile ranges; leaves the sorted lists in the context
int bin(xad_splat_context* c, const float* params, const float* depth, hipStream_t s) {
    int current = -1;
    XAD_HIP_TRY(hipGetDevice(&current));
    XAD_REQUIRE(current == c->device, "splat: the context belongs to device %d, but device %d is current", c->device, current);
    mark(c, 0, s);
    const bool had_order = c->order_valid;
    if (!had_order)
        if (int st = order_by_depth(c, depth, s)) return st;
    std::uint32_t* depth_changed = c->offsets + c->G + 1;  // zero at creation, reset by every emission
    if (int st = launch_project(s, c->G, params, depth, c->ordered_depth, depth_changed, c->width, c->height, c->records,
                                c->rects, c->counts, c->record_grads, c->loss))
        return st;
    mark(c, 1, s);
    // The order of the previous call is used on the assumption that the depths are the same; the
    // flag read back with the pair count says whether they were, and if not the placement is redone.
    if (int st = place_and_emit(c, s)) return st;
    if (had_order && c->host_pairs[1] != 0) {
        if (int st = order_by_depth(c, depth, s)) return st;
        if (int st = place_and_emit(c, s)) return st;
    }
    if (c->pairs > c->capacity) {
        // the emission above stopped at the old capacity; hipFree waits for it before the buffers go
        const std::uint64_t want = static_cast<std::uint64_t>(c->pairs) + c->pairs / 4 + 1024;
        XAD_REQUIRE(want < 0xffffffffull, "splat: %u pairs exceed the 32-bit pair index", c->pairs);
        if (int st = allocate_pair_buffers(c, static_cast<std::uint32_t>(want))) return st;
        if (int st = emit(c, s)) return st;
    }
    mark(c, 2, s);
    if (int st = sort_pairs(s, c->sort_temp, c->sort_bytes, c->wide_keys, c->keys, c->keys_sorted, c->ids, c->ids_sorted,
                            c->pairs, c->key_bits))
        return st;
    mark(c, 3, s);
    if (int st = launch_ranges(s, c->pairs, c->wide_keys, c->keys_sorted, c->range_begin, c->range_end)) return st;
    mark(c, 4, s);
    return XAD_OK;
}

void collect_times(xad_splat_context* c, int stages) {
    if (!c->profile) return;
    (void)hipEventSynchronize(c->marks[stages]);
    for (int i = 0; i < stages; ++i) (void)hipEventElapsedTime(&c->stage_ms[i], c->marks[i], c->marks[i + 1]);
    for (int i = stages; i < xad_splat_context::kStages; ++i) c->stage_ms[i] = 0.f;
}

}  // namespace

extern "C" int xad_splat_create(int width, int height, int num_gaussians, std::size_t pair_capacity_hint,
                                xad_splat_context** out) {
    const char* who = "xad_splat_create";
    XAD_REQUIRE(out, "%s: out is null", who);
    *out = nullptr;
    XAD_REQUIRE(width > 0 && height > 0 && num_gaussians > 0, "%s: width, height and num_gaussians must be positive", who);
    const int tiles_x = (width + kTile - 1) / kTile, tiles_y = (height + kTile - 1) / kTile;
    XAD_REQUIRE(tiles_x <= 32767 && tiles_y <= 32767, "%s: image too large for 16-bit tile coordinates", who);
    XAD_REQUIRE(static_cast<std::size_t>(tiles_x) * tiles_y < (1u << 30), "%s: too many tiles", who);
    auto* c = new (std::nothrow) xad_splat_context();
    XAD_REQUIRE(c, "%s: out of host memory", who);
    c->width = width;
    c->height = height;
    c->G = num_gaussians;
    if (hipGetDevice(&c->device) != hipSuccess) {
        delete c;
        return xad::fail(XAD_ERR_HIP, "%s: no current device", who);
    }
    c->tiles_x = tiles_x;
    c->tiles_y = tiles_y;
    c->tiles = tiles_x * tiles_y;
    int tile_bits = 1;
    while ((1 << tile_bits) < c->tiles) ++tile_bits;
    c->key_bits = tile_bits;
    c->wide_keys = c->tiles > 65536;
    const std::size_t pixels = static_cast<std::size_t>(width) * height;
    const std::size_t G = static_cast<std::size_t>(num_gaussians);
    int st = XAD_OK;
    auto alloc = [&](auto** p, std::size_t bytes) {
        if (st == XAD_OK && hipMalloc(reinterpret_cast<void**>(p), bytes) != hipSuccess)
            st = xad::fail(XAD_ERR_HIP, "%s: hipMalloc of %zu bytes failed", who, bytes);
    };
    alloc(&c->records, sizeof(Record) * G);
    alloc(&c->rects, sizeof(TileRect) * G);
    alloc(&c->depth_keys, sizeof(std::uint32_t) * G);
    alloc(&c->depth_keys_sorted, sizeof(std::uint32_t) * G);
    alloc(&c->identity, sizeof(std::uint32_t) * G);
    alloc(&c->by_depth, sizeof(std::uint32_t) * G);
    alloc(&c->counts_by_depth, sizeof(std::uint32_t) * (G + 1));
    alloc(&c->counts, sizeof(std::uint32_t) * (G + 1));
    alloc(&c->offsets, sizeof(std::uint32_t) * (G + 2));
    alloc(&c->ordered_depth, sizeof(float) * G);
    alloc(&c->range_begin, sizeof(std::uint32_t) * c->tiles * 2);
    alloc(&c->final_T, sizeof(float) * pixels);
    alloc(&c->n_contrib, sizeof(std::uint32_t) * pixels);
    alloc(&c->record_grads, sizeof(float) * G * kRecordGradStride);
    alloc(&c->loss, sizeof(double));
    if (st == XAD_OK) {
        c->range_end = c->range_begin + c->tiles;
        c->scan_bytes = scan_temp_bytes(num_gaussians);
        alloc(&c->scan_temp, c->scan_bytes ? c->scan_bytes : 16);
        c->depth_sort_bytes = depth_sort_temp_bytes(num_gaussians);
        alloc(&c->depth_sort_temp, c->depth_sort_bytes ? c->depth_sort_bytes : 16);
    }
    if (st == XAD_OK && hipHostMalloc(reinterpret_cast<void**>(&c->host_pairs), 2 * sizeof(std::uint32_t)) != hipSuccess)
        st = xad::fail(XAD_ERR_HIP, "%s: pinned allocation failed", who);
    if (st == XAD_OK && hipHostMalloc(reinterpret_cast<void**>(&c->host_loss), sizeof(double)) != hipSuccess)
        st = xad::fail(XAD_ERR_HIP, "%s: pinned allocation failed", who);
    if (st == XAD_OK && hipMemset(c->counts, 0, sizeof(std::uint32_t) * (G + 1)) != hipSuccess)
        st = xad::fail(XAD_ERR_HIP, "%s: hipMemset failed", who);
    if (st == XAD_OK && hipMemset(c->counts_by_depth, 0, sizeof(std::uint32_t) * (G + 1)) != hipSuccess)
        st = xad::fail(XAD_ERR_HIP, "%s: hipMemset failed", who);
    if (st == XAD_OK && hipMemset(c->offsets, 0, sizeof(std::uint32_t) * (G + 2)) != hipSuccess)  // includes the flag
        st = xad::fail(XAD_ERR_HIP, "%s: hipMemset failed", who);
    if (st == XAD_OK) {
        const std::size_t hint = pair_capacity_hint ? pair_capacity_hint : G * 8 + 1024;
        st = allocate_pair_buffers(c, static_cast<std::uint32_t>(hint < 0xfffffff0ull ? hint : 0xfffffff0ull));
    }
    for (auto& e : c->marks)
        if (st == XAD_OK && hipEventCreate(&e) != hipSuccess) st = xad::fail(XAD_ERR_HIP, "%s: hipEventCreate failed", who);
    if (st == XAD_OK && hipEventCreateWithFlags(&c->count_ready, hipEventDisableTiming) != hipSuccess)
        st = xad::fail(XAD_ERR_HIP, "%s: hipEventCreate failed", who);
    if (st != XAD_OK) {
        xad_splat_destroy(c);
        return st;
    }
    *out = c;
    return XAD_OK;
}

extern "C" void xad_splat_destroy(xad_splat_context* c) {
    if (!c) return;
    free_pair_buffers(c);
    (void)hipFree(c->records);
    (void)hipFree(c->rects);
    (void)hipFree(c->depth_keys);
    (void)hipFree(c->depth_keys_sorted);
    (void)hipFree(c->identity);
    (void)hipFree(c->by_depth);
    (void)hipFree(c->counts_by_depth);
    (void)hipFree(c->ordered_depth);
    (void)hipFree(c->depth_sort_temp);
    (void)hipFree(c->counts);
    (void)hipFree(c->offsets);
    (void)hipFree(c->range_begin);
    (void)hipFree(c->final_T);
    (void)hipFree(c->n_contrib);
    (void)hipFree(c->record_grads);
    (void)hipFree(c->loss);
    (void)hipFree(c->scan_temp);
    if (c->host_pairs) (void)hipHostFree(c->host_pairs);
    if (c->host_loss) (void)hipHostFree(c->host_loss);
    for (auto& e : c->marks)
        if (e) (void)hipEventDestroy(e);
    if (c->count_ready) (void)hipEventDestroy(c->count_ready);
    delete c;
}

extern "C" int xad_splat_set_profiling(xad_splat_context* c, int enabled) {
    XAD_REQUIRE(c, "xad_splat_set_profiling: context is null");
    c->profile = enabled != 0;
    return XAD_OK;
}

extern "C" int xad_splat_forward(xad_splat_context* c, const float* params, const float* depth, float* image,
                                 void* stream) {
    const char* who = "xad_splat_forward";
    XAD_REQUIRE(c && params && depth && image, "%s: null argument", who);
    hipStream_t s = xad::as_stream(stream);
    if (int st = bin(c, params, depth, s)) return st;
    if (int st = launch_render_forward(s, c->width, c->height, c->range_begin, c->range_end, c->ids_sorted, c->records,
                                       image, c->final_T, c->n_contrib))
        return st;
    mark(c, 5, s);
    collect_times(c, 5);
    return XAD_OK;
}

extern "C" int xad_splat_step(xad_splat_context* c, const float* params, const float* depth, const float* target,
                              float* image, float* grads, double* loss_out, void* stream) {
    const char* who = "xad_splat_step";
    XAD_REQUIRE(c && params && depth && target && image && grads, "%s: null argument", who);
    hipStream_t s = xad::as_stream(stream);
    if (int st = bin(c, params, depth, s)) return st;
    if (int st = launch_render_forward(s, c->width, c->height, c->range_begin, c->range_end, c->ids_sorted, c->records,
                                       image, c->final_T, c->n_contrib))
        return st;
    mark(c, 5, s);
    if (int st = launch_render_backward(s, c->width, c->height, c->range_begin, c->range_end, c->ids_sorted, c->records,
                                        image, target, c->final_T, c->n_contrib, c->record_grads, c->loss))
        return st;
    mark(c, 6, s);
    if (int st = launch_gaussian_backward(s, c->G, params, c->record_grads, grads)) return st;
    mark(c, 7, s);
    if (loss_out) {
        XAD_HIP_TRY(hipMemcpyAsync(c->host_loss, c->loss, sizeof(double), hipMemcpyDeviceToHost, s));
        XAD_HIP_TRY(hipStreamSynchronize(s));
        *loss_out = *c->host_loss;
    }
    collect_times(c, 7);
    return XAD_OK;
}

extern "C" int xad_splat_get_stats(const xad_splat_context* c, std::uint64_t* pairs, std::uint32_t* longest_list,
                                   float* stage_ms) {
    const char* who = "xad_splat_get_stats";
    XAD_REQUIRE(c, "%s: context is null", who);
    if (pairs) *pairs = c->pairs;
    if (longest_list) {
        // computed on demand from the tile ranges of the last step
        std::uint32_t* host = new (std::nothrow) std::uint32_t[static_cast<std::size_t>(c->tiles) * 2];
        XAD_REQUIRE(host, "%s: out of host memory", who);
        hipError_t e = hipMemcpy(host, c->range_begin, sizeof(std::uint32_t) * c->tiles * 2, hipMemcpyDeviceToHost);
        std::uint32_t best = 0;
        if (e == hipSuccess)
            for (int t = 0; t < c->tiles; ++t) {
                const std::uint32_t len = host[c->tiles + t] - host[t];
                if (len > best) best = len;
            }
        delete[] host;
        if (e != hipSuccess) return xad::fail(XAD_ERR_HIP, "%s: %s", who, hipGetErrorString(e));
        *longest_list = best;
    }
    if (stage_ms)
        for (int i = 0; i < xad_splat_context::kStages; ++i) stage_ms[i] = c->stage_ms[i];
    return XAD_OK;
}
