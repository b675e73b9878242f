// Least-squares fit by mini-batch SGD in fp64: four parameters shared by every
// sample.  The gradient kernel is the accumulator's extreme-contention case
// (every lane of the device adds into the same four addresses); the SGD loop
// keeps parameters, gradient sums and the batch draw on the device.
#include <cmath>
#include <climits>
#include <mutex>

#include <xyz_autodiff/accumulate.cuh>

#include "common.cuh"
#include "linreg.cuh"
#include "rng.cuh"

namespace {

using namespace xyz_autodiff;
using accumulate::BlockAccumulator;
using accumulate::Strategy;

constexpr unsigned kBlock = 256;
constexpr int kWidth = 5;  // four gradients and the loss

struct LinregArgs {
    const double* x1;
    const double* x2;
    const double* y;
    const int* rows;       // explicit sample rows, or null
    const double* params;  // a, b, c, d
    double* out;           // kWidth sums
    std::size_t n;
    std::size_t total;
    std::uint64_t key;         // random stream of the batch draw
    std::uint64_t first_draw;  // index of this launch's first draw
    bool draw;                 // rows come from the random stream
};

__device__ __forceinline__ std::size_t row_of(const LinregArgs& a, std::size_t i) {
    if (a.draw) return static_cast<std::size_t>(xad_rng::bits(a.key, a.first_draw + i) % a.total);
    return a.rows ? static_cast<std::size_t>(a.rows[i]) : i;
}

// The reference pattern: leaves view the global gradient, every add_grad is a
// global fp64 atomic on one of four addresses.
__global__ void __launch_bounds__(kBlock) linreg_global_kernel(LinregArgs a) {
    const std::size_t stride = static_cast<std::size_t>(gridDim.x) * kBlock;
    double* values = const_cast<double*>(a.params);
    for (std::size_t i = static_cast<std::size_t>(blockIdx.x) * kBlock + threadIdx.x; i < a.n; i += stride) {
        const std::size_t r = row_of(a, i);
        if (r >= a.total) continue;  // a row outside the arrays is dropped, not read
        VariableRef<1, double> pa(values + 0, a.out + 0), pb(values + 1, a.out + 1), pc(values + 2, a.out + 2),
            pd(values + 3, a.out + 3);
        const double loss = xad_linreg::run_loss_graph(pa, pb, pc, pd, a.x1[r], a.x2[r], a.y[r]);
        detail::atomic_add(a.out + 4, loss);
    }
}

// Accumulator leaves: same graph, every add_grad lands in the block's LDS table.
__global__ void __launch_bounds__(kBlock) linreg_leaf_kernel(LinregArgs a) {
    using Acc = BlockAccumulator<double, kWidth, Strategy::LdsAtomics>;
    __shared__ __attribute__((aligned(16))) double lds[kWidth];
    Acc acc(lds, 1, a.out, 1);
    double values[4] = {a.params[0], a.params[1], a.params[2], a.params[3]};
    const std::size_t stride = static_cast<std::size_t>(gridDim.x) * kBlock;
    for (std::size_t i = static_cast<std::size_t>(blockIdx.x) * kBlock + threadIdx.x; i < a.n; i += stride) {
        const std::size_t r = row_of(a, i);
        if (r >= a.total) continue;  // a row outside the arrays is dropped, not read
        accumulate::SlotRef<1, double, Acc> pa(values + 0, acc, 0, 0, a.out + 0), pb(values + 1, acc, 0, 1, a.out + 1),
            pc(values + 2, acc, 0, 2, a.out + 2), pd(values + 3, acc, 0, 3, a.out + 3);
        const double loss = xad_linreg::run_loss_graph(pa, pb, pc, pd, a.x1[r], a.x2[r], a.y[r]);
        acc.add_one(0, 4, loss);
    }
    acc.flush();
}

// Register leaves: each lane keeps running sums over its samples, one
// wavefront reduction and one LDS deposit per wavefront, one global atomic per
// block and element.
template <int kUnroll>
__global__ void __launch_bounds__(kBlock) linreg_wave_kernel(LinregArgs a) {
    using Acc = BlockAccumulator<double, kWidth, Strategy::WaveThenLds, 1, 1>;
    __shared__ __attribute__((aligned(16))) double lds[kWidth];
    Acc acc(lds, 1, a.out, 1);
    const double va = a.params[0], vb = a.params[1], vc = a.params[2], vd = a.params[3];
    double sums[kWidth] = {0.0, 0.0, 0.0, 0.0, 0.0};
    // kUnroll samples per trip, all loads issued before the first graph runs: over a large batch the
    // kernel is a pure read stream (24 bytes per sample) and wants that many loads in flight per
    // lane; a small batch is latency-bound and is spread over as many lanes as possible instead
    const std::size_t stride = static_cast<std::size_t>(gridDim.x) * kBlock * kUnroll;
    for (std::size_t base = static_cast<std::size_t>(blockIdx.x) * kBlock * kUnroll + threadIdx.x; base < a.n; base += stride) {
        double x1[kUnroll], x2[kUnroll], y[kUnroll];
        bool use[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const std::size_t i = base + static_cast<std::size_t>(u) * kBlock;
            const std::size_t r = i < a.n ? row_of(a, i) : a.total;
            use[u] = r < a.total;  // a row outside the arrays is dropped, not read
            x1[u] = use[u] ? __builtin_nontemporal_load(a.x1 + r) : 0.0;
            x2[u] = use[u] ? __builtin_nontemporal_load(a.x2 + r) : 0.0;
            y[u] = use[u] ? __builtin_nontemporal_load(a.y + r) : 0.0;
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            if (!use[u]) continue;
            Variable<1, double> pa(va), pb(vb), pc(vc), pd(vd);
            sums[4] += xad_linreg::run_loss_graph(pa, pb, pc, pd, x1[u], x2[u], y[u]);
            sums[0] += pa.grad(0);
            sums[1] += pb.grad(0);
            sums[2] += pc.grad(0);
            sums[3] += pd.grad(0);
        }
    }
    acc.add(0, sums);
    acc.flush();
}

__global__ void linreg_zero_kernel(double* out) {
    if (threadIdx.x < kWidth) out[threadIdx.x] = 0.0;
}

// p -= lr * sum / batch (linear_regression_sgd.cu:126-134 of the reference),
// record the mean loss, and clear the sums for the next step.
__global__ void linreg_update_kernel(double* params, double* sums, double learning_rate, int batch, double* history) {
    if (threadIdx.x < 4) params[threadIdx.x] -= learning_rate * (sums[threadIdx.x] / batch);
    if (threadIdx.x == 4 && history) *history = sums[4] / batch;
    if (threadIdx.x < kWidth) sums[threadIdx.x] = 0.0;
}

int grid_for(std::size_t n, unsigned* blocks) {
    int dev = 0;
    XAD_HIP_TRY(hipGetDevice(&dev));
    int cus = 0;
    XAD_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const std::size_t wanted = (n + kBlock - 1) / kBlock;
    const std::size_t cap = static_cast<std::size_t>(cus) * 8;
    *blocks = static_cast<unsigned>(wanted < cap ? (wanted ? wanted : 1) : cap);
    return XAD_OK;
}

int launch_gradient(int strategy, const LinregArgs& a, unsigned blocks, hipStream_t stream) {
    switch (strategy) {
        case XAD_LINREG_GLOBAL_ATOMICS:
            linreg_global_kernel<<<blocks, kBlock, 0, stream>>>(a);
            break;
        case XAD_LINREG_LDS_LEAVES:
            linreg_leaf_kernel<<<blocks, kBlock, 0, stream>>>(a);
            break;
        case XAD_LINREG_WAVE_LDS:
            if (a.n >= (std::size_t(1) << 20))
                linreg_wave_kernel<4><<<blocks, kBlock, 0, stream>>>(a);
            else
                linreg_wave_kernel<1><<<blocks, kBlock, 0, stream>>>(a);
            break;
        default:
            return xad::fail(XAD_ERR_INVALID_ARGUMENT, "unknown accumulation strategy %d", strategy);
    }
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

}  // namespace

extern "C" int xad_linreg_gradient_f64(int strategy, size_t n, size_t total, const double* x1, const double* x2,
                                       const double* y, const int* rows, const double* params, double* out,
                                       void* stream) {
    XAD_REQUIRE(strategy >= XAD_LINREG_GLOBAL_ATOMICS && strategy <= XAD_LINREG_WAVE_LDS,
                "unknown accumulation strategy %d", strategy);
    XAD_REQUIRE(params && out, "params and out must not be null");
    XAD_REQUIRE(n == 0 || (x1 && x2 && y), "sample arrays must not be null");
    XAD_REQUIRE(rows || n <= total, "n = %zu samples requested from %zu rows without an index array", n, total);
    hipStream_t s = xad::as_stream(stream);
    linreg_zero_kernel<<<1, 64, 0, s>>>(out);
    XAD_HIP_TRY(hipGetLastError());
    if (n == 0) return XAD_OK;
    unsigned blocks = 0;
    if (int st = grid_for(n, &blocks)) return st;
    LinregArgs a{x1, x2, y, rows, params, out, n, total, 0, 0, false};
    return launch_gradient(strategy, a, blocks, s);
}

namespace {

// Queues `epochs` SGD steps on `s`; `sums` is kWidth doubles of device memory that
// nothing else uses until the queued work has run.
int queue_sgd(hipStream_t s, double* sums, std::size_t total, const double* x1, const double* x2, const double* y,
              double* params, int batch, int epochs, double lr_first, double lr_last, std::uint64_t seed,
              double* loss_history) {
    unsigned blocks = 0;
    if (int st = grid_for(static_cast<std::size_t>(batch), &blocks)) return st;
    // the sums start from zero whatever an earlier run left in them (the update kernel clears them
    // again after every step)
    linreg_zero_kernel<<<1, 64, 0, s>>>(sums);
    XAD_HIP_TRY(hipGetLastError());
    const std::uint64_t key = xad_rng::stream_key(seed, 0);
    const double decay = epochs > 0 ? std::log(lr_last / lr_first) / epochs : 0.0;
    for (int e = 0; e < epochs; ++e) {
        LinregArgs a{x1, x2, y, nullptr, params, sums, static_cast<std::size_t>(batch), total,
                     key, static_cast<std::uint64_t>(e) * static_cast<std::uint64_t>(batch), true};
        if (int st = launch_gradient(XAD_LINREG_WAVE_LDS, a, blocks, s)) return st;
        linreg_update_kernel<<<1, 64, 0, s>>>(params, sums, lr_first * std::exp(decay * e), batch,
                                              loss_history ? loss_history + e : nullptr);
        XAD_HIP_TRY(hipGetLastError());
    }
    return XAD_OK;
}

// Gradient sums of xad_linreg_sgd_f64_static: one copy of this array per device, for the life of
// the process.  kWidth doubles are used; the size is the alignment unit.
constexpr int kScratchDoubles = 32;
static __device__ __align__(256) double scratch[kScratchDoubles];
static_assert(kWidth <= kScratchDoubles, "the sums must fit the static array");

// Host code never passes `scratch` itself to a kernel: the name is a host-side handle, not a
// device address.  The address is looked up once per device, with that device current.
constexpr int kMaxDevices = 64;
std::mutex scratch_lock;
double* scratch_address[kMaxDevices] = {};

int scratch_of_current_device(double** out) {
    int dev = -1;
    XAD_HIP_TRY(hipGetDevice(&dev));
    XAD_REQUIRE(dev >= 0 && dev < kMaxDevices, "device %d is beyond the %d devices this entry point keeps scratch for", dev,
                kMaxDevices);
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (!scratch_address[dev]) {
        void* p = nullptr;
        XAD_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        XAD_REQUIRE(p, "hipGetSymbolAddress returned a null address for the scratch array");
        scratch_address[dev] = static_cast<double*>(p);
    }
    *out = scratch_address[dev];
    return XAD_OK;
}

}  // namespace

extern "C" int xad_linreg_sgd_f64(size_t total, const double* x1, const double* x2, const double* y, double* params,
                                  int batch, int epochs, double lr_first, double lr_last, uint64_t seed,
                                  double* loss_history, void* stream) {
    XAD_REQUIRE(x1 && x2 && y && params, "sample arrays and params must not be null");
    XAD_REQUIRE(total > 0 && batch > 0 && epochs >= 0, "total, batch must be positive and epochs non-negative");
    XAD_REQUIRE(lr_first > 0.0 && lr_last > 0.0, "learning rates must be positive");
    hipStream_t s = xad::as_stream(stream);
    double* sums = nullptr;
    XAD_HIP_TRY(hipMalloc(&sums, kWidth * sizeof(double)));
    const int status = queue_sgd(s, sums, total, x1, x2, y, params, batch, epochs, lr_first, lr_last, seed, loss_history);
    const hipError_t waited = hipStreamSynchronize(s);
    const hipError_t freed = hipFree(sums);
    if (status != XAD_OK) return status;
    XAD_HIP_TRY(waited);
    XAD_HIP_TRY(freed);
    return XAD_OK;
}

extern "C" int xad_linreg_sgd_f64_static(size_t total, const double* x1, const double* x2, const double* y,
                                         double* params, int batch, int epochs, double lr_first, double lr_last,
                                         uint64_t seed, double* loss_history, void* stream) {
    const char* who = "xad_linreg_sgd_f64_static";
    XAD_REQUIRE(x1 && x2 && y && params, "%s: sample arrays and params must not be null", who);
    XAD_REQUIRE(total > 0 && batch > 0 && epochs >= 0, "%s: total, batch must be positive and epochs non-negative", who);
    XAD_REQUIRE(lr_first > 0.0 && lr_last > 0.0, "%s: learning rates must be positive", who);
    XAD_REQUIRE(epochs <= XAD_LINREG_STATIC_MAX_EPOCHS,
                "%s: %d steps exceed the %d steps one call may queue; split the run into several calls", who, epochs,
                XAD_LINREG_STATIC_MAX_EPOCHS);
    double* sums = nullptr;
    if (int st = scratch_of_current_device(&sums)) return st;
    return queue_sgd(xad::as_stream(stream), sums, total, x1, x2, y, params, batch, epochs, lr_first, lr_last, seed,
                     loss_history);
}

extern "C" int xad_host_linreg_gradient_f64(size_t n, size_t total, const double* x1, const double* x2,
                                            const double* y, const int* rows, const double* params, double* out) {
    XAD_REQUIRE(params && out, "params and out must not be null");
    XAD_REQUIRE(n == 0 || (x1 && x2 && y), "sample arrays must not be null");
    XAD_REQUIRE(rows || n <= total, "n = %zu samples requested from %zu rows without an index array", n, total);
    double sums[kWidth] = {0.0, 0.0, 0.0, 0.0, 0.0};
    for (std::size_t i = 0; i < n; ++i) {
        const std::size_t r = rows ? static_cast<std::size_t>(rows[i]) : i;
        XAD_REQUIRE(r < total, "row %zu of sample %zu is outside the %zu rows", r, i, total);
        Variable<1, double> pa(params[0]), pb(params[1]), pc(params[2]), pd(params[3]);
        sums[4] += xad_linreg::run_loss_graph(pa, pb, pc, pd, x1[r], x2[r], y[r]);
        sums[0] += pa.grad(0);
        sums[1] += pb.grad(0);
        sums[2] += pc.grad(0);
        sums[3] += pd.grad(0);
    }
    for (int k = 0; k < kWidth; ++k) out[k] = sums[k];
    return XAD_OK;
}
