// The splatting step behind the C ABI: workspace ownership, stage order, and the few places
// where the host has to look at what the device found.
#include <new>

#include "common.cuh"
#include "splat_launch.cuh"

using namespace xad_splat;

namespace {

// What the device reports back, in pinned host memory: the status words of the step and the loss.
struct HostReport {
    std::uint32_t status[kStatusWords];
    std::uint32_t depth_changed;  // the depth flag as it stood before the binning cleared it
    std::uint32_t sort_gave_up;   // blocks of the depth sort whose bounded wait ran out (never, on a device of one's own)
    double loss;
};

__global__ void clear_words_kernel(std::uint32_t* words, int first, int count) {
    if (static_cast<int>(threadIdx.x) < count) words[first + threadIdx.x] = 0;
}

}  // namespace

struct xad_splat_context {
    int width = 0, height = 0, G = 0;
    int device = 0;  // the device that was current at creation: owns every buffer below
    int tiles_x = 0, tiles_y = 0, tiles = 0;
    int depth_mode = XAD_SPLAT_DEPTH_CHECKED;
    bool profile = false;
    bool order_valid = false;   // by_depth is the (depth, index) order of ordered_depth
    bool capacity_seen = false;  // a step has been seen to fit the pair lists since they were last sized
    std::uint32_t pairs = 0;     // pairs of the last step the host has a report of

    // one allocation for everything whose size is fixed by (G, image): `fixed` is its base
    void* fixed = nullptr;
    Record* records = nullptr;
    TileRect* rects = nullptr;
    TileRect* rects_by_depth = nullptr;  // the same rectangles in depth order
    std::uint32_t* rank = nullptr;       // G: position of every Gaussian in the depth order
    std::uint32_t *depth_keys = nullptr, *depth_keys_sorted = nullptr;  // G each
    std::uint32_t *identity = nullptr, *by_depth = nullptr;             // G each; by_depth = Gaussians in (depth, index) order
    float* ordered_depth = nullptr;                                     // G: the depths by_depth was computed from
    std::uint32_t *range_begin = nullptr, *range_end = nullptr;         // tiles each, adjacent
    float* final_T = nullptr;
    std::uint32_t* n_contrib = nullptr;
    std::uint32_t* tile_order = nullptr;  // 8 * ceil(tiles / 8): which tile each block of the compositing kernels takes
    int segments = 1;                 // pieces a tile's list is cut into for the backward walk
    float4* segment_state = nullptr;  // segments x pixels when segments > 1
    float* record_grads = nullptr;  // G x kRecordGradStride
    double* loss = nullptr;
    std::uint32_t* status = nullptr;  // kStatusWords
    void* depth_sort_temp = nullptr;
    std::size_t depth_sort_bytes = 0;

    // one allocation for everything sized by the pair capacity: `paired` is its base
    void* paired = nullptr;
    std::uint32_t* list = nullptr;  // the tiles' lists
    BinPlan plan{};
    BinScratch bin;

    HostReport* report = nullptr;  // pinned

    static constexpr int kStages = 6;  // depth order, project, binning, render forward, render backward, parameter backward
    hipEvent_t marks[kStages + 1] = {};
    float stage_ms[kStages] = {};
    hipEvent_t report_ready = nullptr;
};

namespace {

// Carves consecutive 256-byte aligned pieces out of one allocation; first pass (base == nullptr) only adds up.
struct Carver {
    char* base;
    std::size_t used = 0;
    template <typename T>
    T* take(std::size_t count) {
        const std::size_t at = used;
        used += (count * sizeof(T) + 255) / 256 * 256;
        return base ? reinterpret_cast<T*>(base + at) : nullptr;
    }
};

void carve_fixed(xad_splat_context* c, char* base, std::size_t* bytes) {
    Carver k{base};
    const std::size_t G = static_cast<std::size_t>(c->G), pixels = static_cast<std::size_t>(c->width) * c->height;
    c->records = k.take<Record>(G);
    c->rects = k.take<TileRect>(G);
    c->rects_by_depth = k.take<TileRect>(G);
    c->rank = k.take<std::uint32_t>(G);
    c->depth_keys = k.take<std::uint32_t>(G);
    c->depth_keys_sorted = k.take<std::uint32_t>(G);
    c->identity = k.take<std::uint32_t>(G);
    c->by_depth = k.take<std::uint32_t>(G);
    c->ordered_depth = k.take<float>(G);
    c->range_begin = k.take<std::uint32_t>(static_cast<std::size_t>(c->tiles) * 2);
    c->range_end = c->range_begin ? c->range_begin + c->tiles : nullptr;
    c->final_T = k.take<float>(pixels);
    c->n_contrib = k.take<std::uint32_t>(pixels);
    c->tile_order = k.take<std::uint32_t>(static_cast<std::size_t>((c->tiles + 7) / 8) * 8);
    c->segment_state = c->segments > 1 ? k.take<float4>(pixels * static_cast<std::size_t>(c->segments)) : nullptr;
    c->record_grads = k.take<float>(G * kRecordGradStride);
    c->loss = k.take<double>(kLossWords);
    c->status = k.take<std::uint32_t>(kStatusWords);
    c->bin.scan_control = k.take<std::uint32_t>(kScanControlWords);
    c->depth_sort_temp = k.take<char>(c->depth_sort_bytes ? c->depth_sort_bytes : 16);
    *bytes = k.used;
}

void carve_paired(xad_splat_context* c, char* base, std::size_t* bytes) {
    Carver k{base};
    c->list = k.take<std::uint32_t>(c->plan.capacity);
    c->bin.list_a = k.take<std::uint32_t>(c->plan.capacity);
    c->bin.matrix_a = k.take<std::uint32_t>(bin_matrix_a_words(c->plan));
    c->bin.matrix_b = k.take<std::uint32_t>(bin_matrix_b_words(c->plan));
    c->bin.first_wave = k.take<std::uint32_t>(static_cast<std::size_t>(c->plan.supers) + 1);
    c->bin.scan_state = k.take<std::uint64_t>(bin_scan_state_words(c->plan));
    *bytes = k.used;
}

// (Re)allocates the buffers sized by the pair capacity.  Waits for the device first: a step may still be using them.
int size_pair_buffers(xad_splat_context* c, std::uint32_t capacity) {
    if (c->paired) {
        XAD_HIP_TRY(hipDeviceSynchronize());
        (void)hipFree(c->paired);
        c->paired = nullptr;
    }
    c->capacity_seen = false;
    c->plan = make_bin_plan(c->G, c->tiles_x, c->tiles_y, capacity, capacity);  // the buffers are sized for this one
    std::size_t bytes = 0;
    carve_paired(c, nullptr, &bytes);
    void* base = nullptr;
    if (hipMalloc(&base, bytes) != hipSuccess) {
        c->plan.capacity = 0;  // the next call tries again
        return xad::fail(XAD_ERR_HIP, "splat: hipMalloc of %zu bytes for %u pairs failed", bytes, capacity);
    }
    c->paired = base;
    carve_paired(c, static_cast<char*>(base), &bytes);
    // the scan's state words must not look like words of a coming epoch
    XAD_HIP_TRY(hipMemset(c->bin.scan_state, 0, bin_scan_state_words(c->plan) * sizeof(std::uint64_t)));
    XAD_HIP_TRY(hipDeviceSynchronize());  // the fill is not on the caller's stream
    return XAD_OK;
}

void mark(xad_splat_context* c, int index, hipStream_t s) {
    if (c->profile) (void)hipEventRecord(c->marks[index], s);
}

// Projection, after ordering the Gaussians by (depth, index) when asked to; the order is then kept until a depth changes.
int project_gaussians(xad_splat_context* c, const float* params, const float* depth, hipStream_t s, bool first_of_step,
                      bool ordering) {
    if (ordering) {
        c->order_valid = false;
        if (int st = sort_by_depth(s, c->depth_sort_temp, c->depth_sort_bytes, depth, c->depth_keys, c->depth_keys_sorted, c->identity,
                                   c->by_depth, c->rank, c->ordered_depth, c->G))
            return st;
        c->order_valid = true;
    }
    mark(c, 1, s);
    if (int st = launch_project(s, c->G, params, depth, c->ordered_depth, c->rank, c->status, c->width, c->height, c->records,
                                c->rects, c->rects_by_depth, c->record_grads, c->loss, first_of_step))
        return st;
    mark(c, 2, s);
    return XAD_OK;
}

int bin_lists(xad_splat_context* c, hipStream_t s, bool clear_depth_flag) {
    return launch_binning(s, c->plan, c->by_depth, c->rects_by_depth, c->rects, c->bin, c->list, c->range_begin, c->range_end,
                          c->status, clear_depth_flag);
}

// Queues a copy of the status words (and the loss) to the host and waits for it.
int fetch_report(xad_splat_context* c, hipStream_t s) {
    XAD_HIP_TRY(hipMemcpyAsync(c->report->status, c->status, sizeof(std::uint32_t) * kStatusWords, hipMemcpyDeviceToHost, s));
    XAD_HIP_TRY(hipMemcpyAsync(&c->report->loss, c->loss, sizeof(double), hipMemcpyDeviceToHost, s));
    XAD_HIP_TRY(hipMemcpyAsync(&c->report->sort_gave_up, static_cast<const char*>(c->depth_sort_temp) + depth_sort_gave_up_offset(),
                               sizeof(std::uint32_t), hipMemcpyDeviceToHost, s));
    XAD_HIP_TRY(hipEventRecord(c->report_ready, s));
    XAD_HIP_TRY(hipEventSynchronize(c->report_ready));
    c->pairs = c->report->status[kStatusPairs];
    if (c->report->sort_gave_up != 0) {
        c->order_valid = false;
        return xad::fail(XAD_ERR_HIP,
                         "splat: %u blocks of the depth sort gave up waiting for other blocks (is the device shared with work that "
                         "never ends?); the depth order of the calls since the last report cannot be trusted",
                         c->report->sort_gave_up);
    }
    return XAD_OK;
}

int clear_status(xad_splat_context* c, hipStream_t s, int first, int count) {
    hipLaunchKernelGGL(clear_words_kernel, dim3(1), dim3(64), 0, s, c->status, first, count);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

// Room for a scene of `pairs` pairs that keeps growing: half as much again.
std::uint32_t grown(std::uint32_t pairs) {
    const std::uint64_t want = static_cast<std::uint64_t>(pairs) + pairs / 2 + 1024;
    return static_cast<std::uint32_t>(want < 0xfffffff0ull ? want : 0xfffffff0ull);
}

// Level A's share of the buffers once a scene's supertile pairs are known: twice that many (the wavefronts
// launched at level B follow it, so it is not simply everything).
std::uint32_t level_a_share(std::uint32_t super_pairs) {
    const std::uint64_t want = 2ull * super_pairs + 1024;
    return static_cast<std::uint32_t>(want < 0xfffffff0ull ? want : 0xfffffff0ull);
}

// A step needed room for `seen` pairs (tile or supertile level, whichever is larger) and did not have it.
// If the buffers themselves are large enough, only level A's share of them was too small: it gets the whole
// buffer back, nothing is allocated.  Otherwise the buffers are replaced by larger ones.
int make_room(xad_splat_context* c, std::uint32_t seen) {
    if (seen <= c->plan.capacity && c->plan.capacity_a < c->plan.capacity) {
        c->plan = make_bin_plan(c->G, c->tiles_x, c->tiles_y, c->plan.capacity, c->plan.capacity);
        c->capacity_seen = false;
        return XAD_OK;
    }
    return size_pair_buffers(c, grown(seen > c->plan.capacity ? seen : c->plan.capacity + 1));
}

std::uint32_t pairs_needed(const HostReport* r) {
    return r->status[kStatusPairs] > r->status[kStatusSuperPairs] ? r->status[kStatusPairs] : r->status[kStatusSuperPairs];
}

// Project and bin; leaves the tiles' lists in the context.  Where the host has to look:
//   - XAD_SPLAT_DEPTH_CHECKED: whether a depth changed, every call (the binning is queued before the
//     wait and runs during it; if a depth did change, order and binning are redone);
//   - the first call after the pair lists were sized, and every call that waits for the depth flag
//     anyway: whether the pairs fit (if not, the lists are enlarged and the binning is redone).
// Otherwise nothing is read back: an overflow or a depth that changed against the caller's promise is
// left in the sticky status words for the next call that waits anyway.
int bin(xad_splat_context* c, const float* params, const float* depth, hipStream_t s, bool first_attempt = true) {
    int current = -1;
    XAD_HIP_TRY(hipGetDevice(&current));
    XAD_REQUIRE(current == c->device, "splat: the context belongs to device %d, but device %d is current", c->device, current);
    if (c->plan.capacity == 0)
        if (int st = size_pair_buffers(c, static_cast<std::uint32_t>(static_cast<std::size_t>(c->G) * 8 + 1024))) return st;
    mark(c, 0, s);
    const bool had_order = c->order_valid && c->depth_mode != XAD_SPLAT_DEPTH_EVERY_STEP;
    if (int st = project_gaussians(c, params, depth, s, first_attempt, !had_order)) return st;
    const bool check_depth = c->depth_mode == XAD_SPLAT_DEPTH_CHECKED && had_order;
    if (check_depth) {
        // the order of the previous call is used on the assumption that the depths are the same; the
        // flag says whether they were.  The copy is ahead of the binning, which clears the flag.
        XAD_HIP_TRY(hipMemcpyAsync(&c->report->depth_changed, c->status + kStatusDepthChanged, sizeof(std::uint32_t),
                                   hipMemcpyDeviceToHost, s));
    }
    // in the static mode the flag stays up until the host has seen it; otherwise every binning clears it
    if (int st = bin_lists(c, s, c->depth_mode != XAD_SPLAT_DEPTH_STATIC)) return st;
    if (check_depth || !c->capacity_seen) {
        // the one wait of this call: the status words of the binning, and with them the depth flag copied above
        if (int st = fetch_report(c, s)) return st;
        if (check_depth && c->report->depth_changed != 0) {
            if (int st = project_gaussians(c, params, depth, s, false, true)) return st;  // the new order, the rectangles in it
            if (int st = bin_lists(c, s, true)) return st;
            if (int st = fetch_report(c, s)) return st;
        }
        // The tile-level pair count is exact even when it exceeds the capacity, unless the supertile lists
        // were cut short as well (then it is a lower bound and the next attempt's count is exact).
        bool made_room = false;
        for (int attempt = 0; c->report->status[kStatusOverflow] != 0; ++attempt) {
            const std::uint32_t seen = pairs_needed(c->report);
            XAD_REQUIRE(attempt < 4 && seen < 0xfffffff0u, "splat: the pair lists overflow at %u pairs", seen);
            if (int st = make_room(c, seen)) return st;
            if (int st = bin_lists(c, s, false)) return st;
            if (int st = fetch_report(c, s)) return st;
            made_room = true;
        }
        if (!c->capacity_seen) {
            c->capacity_seen = true;
            // from now on level A is given only the room this scene needs, with a margin: fewer wavefronts at level B
            // (an overflow of that margin is reported like any other and gives level A the whole buffer back)
            c->plan = make_bin_plan(c->G, c->tiles_x, c->tiles_y, c->plan.capacity, level_a_share(c->report->status[kStatusSuperPairs]));
        }
        // what this call's own attempts left in the sticky word is settled; what earlier calls left there stays
        if (made_room && c->report->status[kStatusStickyBefore] == 0) {
            if (int st = clear_status(c, s, kStatusOverflowSticky, 1)) return st;
            c->report->status[kStatusOverflowSticky] = 0;
        }
    }
    mark(c, 3, s);
    return XAD_OK;
}

void collect_times(xad_splat_context* c, int stages) {
    if (!c->profile) return;
    (void)hipEventSynchronize(c->marks[stages]);
    for (int i = 0; i < stages; ++i) (void)hipEventElapsedTime(&c->stage_ms[i], c->marks[i], c->marks[i + 1]);
    for (int i = stages; i < xad_splat_context::kStages; ++i) c->stage_ms[i] = 0.f;
}

// After a wait: what earlier calls that did not wait have left behind.
int settle_report(xad_splat_context* c, hipStream_t s, const char* who) {
    int st = XAD_OK;
    if (c->depth_mode == XAD_SPLAT_DEPTH_STATIC && c->report->status[kStatusDepthChanged] != 0) {
        c->order_valid = false;
        (void)clear_status(c, s, kStatusDepthChanged, 1);
        st = xad::fail(XAD_ERR_INVALID_ARGUMENT,
                       "%s: a depth changed although the context is in XAD_SPLAT_DEPTH_STATIC mode; the lists of the calls since "
                       "then were ordered by the old depths (the order will be recomputed by the next call)",
                       who);
    }
    if (c->report->status[kStatusOverflowSticky] != 0) {
        const std::uint32_t seen = c->report->status[kStatusOverflowSticky];
        (void)clear_status(c, s, kStatusOverflowSticky, 1);
        c->report->status[kStatusOverflowSticky] = 0;
        if (int grow = make_room(c, seen)) return grow;
        st = xad::fail(XAD_ERR_INCOMPLETE,
                       "%s: a call that did not wait for the device produced more pairs (%u) than the lists held; its image and "
                       "gradients were incomplete.  The lists have been enlarged",
                       who, seen);
    }
    return st;
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
    c->segments = render_segments(width, height);
    c->depth_sort_bytes = depth_sort_temp_bytes(num_gaussians);
    int st = XAD_OK;
    std::size_t bytes = 0;
    carve_fixed(c, nullptr, &bytes);
    if (hipMalloc(&c->fixed, bytes) != hipSuccess) st = xad::fail(XAD_ERR_HIP, "%s: hipMalloc of %zu bytes failed", who, bytes);
    if (st == XAD_OK) {
        carve_fixed(c, static_cast<char*>(c->fixed), &bytes);
        // status words, the scan's control words and the tile ranges start from zero; the scan's epoch from one
        if (hipMemset(c->fixed, 0, bytes) != hipSuccess) st = xad::fail(XAD_ERR_HIP, "%s: hipMemset failed", who);
        const std::uint32_t control[kScanControlWords] = {0u, 0u, 1u};
        if (st == XAD_OK && hipMemcpy(c->bin.scan_control, control, sizeof(control), hipMemcpyHostToDevice) != hipSuccess)
            st = xad::fail(XAD_ERR_HIP, "%s: hipMemcpy failed", who);
    }
    if (st == XAD_OK && hipHostMalloc(reinterpret_cast<void**>(&c->report), sizeof(HostReport)) != hipSuccess)
        st = xad::fail(XAD_ERR_HIP, "%s: pinned allocation failed", who);
    if (st == XAD_OK) {
        *c->report = HostReport{};
        const std::size_t hint = pair_capacity_hint ? pair_capacity_hint : static_cast<std::size_t>(num_gaussians) * 8 + 1024;
        st = size_pair_buffers(c, static_cast<std::uint32_t>(hint < 0xfffffff0ull ? hint : 0xfffffff0ull));
    }
    for (auto& e : c->marks)
        if (st == XAD_OK && hipEventCreate(&e) != hipSuccess) st = xad::fail(XAD_ERR_HIP, "%s: hipEventCreate failed", who);
    if (st == XAD_OK && hipEventCreateWithFlags(&c->report_ready, hipEventDisableTiming) != hipSuccess)
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
    if (c->paired) (void)hipFree(c->paired);
    if (c->fixed) (void)hipFree(c->fixed);
    if (c->report) (void)hipHostFree(c->report);
    for (auto& e : c->marks)
        if (e) (void)hipEventDestroy(e);
    if (c->report_ready) (void)hipEventDestroy(c->report_ready);
    delete c;
}

extern "C" int xad_splat_set_profiling(xad_splat_context* c, int enabled) {
    XAD_REQUIRE(c, "xad_splat_set_profiling: context is null");
    c->profile = enabled != 0;
    return XAD_OK;
}

extern "C" int xad_splat_set_depth_mode(xad_splat_context* c, int mode) {
    XAD_REQUIRE(c, "xad_splat_set_depth_mode: context is null");
    XAD_REQUIRE(mode == XAD_SPLAT_DEPTH_CHECKED || mode == XAD_SPLAT_DEPTH_STATIC || mode == XAD_SPLAT_DEPTH_EVERY_STEP,
                "xad_splat_set_depth_mode: unknown mode %d", mode);
    c->depth_mode = mode;
    c->order_valid = false;  // the next call orders by the depths it is given
    return XAD_OK;
}

extern "C" int xad_splat_forward(xad_splat_context* c, const float* params, const float* depth, float* image,
                                 void* stream) {
    const char* who = "xad_splat_forward";
    XAD_REQUIRE(c && params && depth && image, "%s: null argument", who);
    hipStream_t s = xad::as_stream(stream);
    if (int st = bin(c, params, depth, s)) return st;
    if (int st = launch_render_forward(s, c->width, c->height, c->range_begin, c->range_end, c->list, c->records, image,
                                       c->final_T, c->n_contrib, c->segments, c->segment_state, c->tile_order))
        return st;
    mark(c, 4, s);
    collect_times(c, 4);
    return XAD_OK;
}

extern "C" int xad_splat_step(xad_splat_context* c, const float* params, const float* depth, const float* target,
                              float* image, float* grads, double* loss_out, void* stream) {
    const char* who = "xad_splat_step";
    XAD_REQUIRE(c && params && depth && target && image && grads, "%s: null argument", who);
    hipStream_t s = xad::as_stream(stream);
    bool earlier_steps_overflowed = false;
    for (int attempt = 0;; ++attempt) {
        if (int st = bin(c, params, depth, s, attempt == 0)) return st;
        if (int st = launch_render_forward(s, c->width, c->height, c->range_begin, c->range_end, c->list, c->records, image,
                                           c->final_T, c->n_contrib, c->segments, c->segment_state, c->tile_order))
            return st;
        mark(c, 4, s);
        if (int st = launch_render_backward(s, c->width, c->height, c->range_begin, c->range_end, c->list, c->records, image,
                                            target, c->final_T, c->n_contrib, c->record_grads, c->loss, c->segments,
                                            c->segment_state, c->tile_order))
            return st;
        mark(c, 5, s);
        if (int st = launch_gaussian_backward(s, c->G, params, c->record_grads, grads, c->loss)) return st;
        mark(c, 6, s);
        if (!loss_out) break;
        // the loss is read back, and with it what the device has to report
        if (int st = fetch_report(c, s)) return st;
        if (c->report->status[kStatusOverflow] != 0 && attempt == 0) {
            // this very step did not fit (the scene grew): enlarge the lists and do it again.  Whether steps
            // before it overflowed too is in the word the step saved when it began.
            earlier_steps_overflowed = c->report->status[kStatusStickyBefore] != 0;
            if (int st = make_room(c, pairs_needed(c->report))) return st;
            if (int st = clear_status(c, s, kStatusOverflowSticky, 1)) return st;
            c->report->status[kStatusOverflowSticky] = 0;
            continue;
        }
        *loss_out = c->report->loss;
        if (int st = settle_report(c, s, who)) {
            collect_times(c, 6);
            return st;
        }
        break;
    }
    collect_times(c, 6);
    if (earlier_steps_overflowed)
        return xad::fail(XAD_ERR_INCOMPLETE,
                         "%s: a call that did not wait for the device produced more pairs than the lists held; its image and "
                         "gradients were incomplete.  The lists have been enlarged (this step is complete)",
                         who);
    return XAD_OK;
}

extern "C" int xad_splat_get_stats(xad_splat_context* c, std::uint64_t* pairs, std::uint32_t* longest_list, float* stage_ms) {
    const char* who = "xad_splat_get_stats";
    XAD_REQUIRE(c, "%s: context is null", who);
    if (pairs || longest_list) {
        // waits for everything queued on the device, then reads the status words of the last step
        XAD_HIP_TRY(hipDeviceSynchronize());
        XAD_HIP_TRY(hipMemcpy(c->report->status, c->status, sizeof(std::uint32_t) * kStatusWords, hipMemcpyDeviceToHost));
        c->pairs = c->report->status[kStatusPairs];
    }
    if (pairs) *pairs = c->pairs;
    if (longest_list) {
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
    if (pairs || longest_list) {
        // this call has waited: what calls that did not wait have left behind is reported (and dealt with) here
        const int st = settle_report(c, nullptr, who);
        XAD_HIP_TRY(hipDeviceSynchronize());
        return st;
    }
    return XAD_OK;
}

extern "C" int xad_splat_overflow_word(xad_splat_context* c, const std::uint32_t** device_word) {
    XAD_REQUIRE(c && device_word, "xad_splat_overflow_word: null argument");
    *device_word = c->status + kStatusOverflowSticky;
    return XAD_OK;
}

extern "C" int xad_splat_get_lists(xad_splat_context* c, std::uint32_t* range_begin, std::uint32_t* range_end,
                                   std::uint32_t* gaussians, std::size_t capacity) {
    const char* who = "xad_splat_get_lists";
    XAD_REQUIRE(c && range_begin && range_end, "%s: null argument", who);
    XAD_HIP_TRY(hipDeviceSynchronize());
    XAD_HIP_TRY(hipMemcpy(c->report->status, c->status, sizeof(std::uint32_t) * kStatusWords, hipMemcpyDeviceToHost));
    c->pairs = c->report->status[kStatusPairs];
    {
        // the lists of a step that outgrew the buffers are not handed out: the buffers are enlarged instead
        const bool cut_short = c->report->status[kStatusOverflow] != 0;
        const int st = settle_report(c, nullptr, who);
        XAD_HIP_TRY(hipDeviceSynchronize());
        if (st) return st;
        XAD_REQUIRE(!cut_short, "%s: the last step's lists overflowed", who);
    }
    XAD_HIP_TRY(hipMemcpy(range_begin, c->range_begin, sizeof(std::uint32_t) * c->tiles, hipMemcpyDeviceToHost));
    XAD_HIP_TRY(hipMemcpy(range_end, c->range_end, sizeof(std::uint32_t) * c->tiles, hipMemcpyDeviceToHost));
    if (gaussians) {
        XAD_REQUIRE(capacity >= c->pairs, "%s: room for %zu entries, the lists hold %u", who, capacity, c->pairs);
        if (c->pairs) XAD_HIP_TRY(hipMemcpy(gaussians, c->list, sizeof(std::uint32_t) * c->pairs, hipMemcpyDeviceToHost));
    }
    return XAD_OK;
}
