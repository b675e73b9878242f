// Parallel gradient accumulation: every thread evaluates the benchmark graph
// for its own inputs and adds its six gradients into one of P shared slots.
//
// Three interchangeable strategies (see xyz_autodiff/accumulate.cuh): naive
// global atomics, LDS table + one write-out per block, and wavefront
// pre-reduction in front of the LDS table.  Blocks are persistent: the grid is
// sized to the machine and each block walks a contiguous chunk of threads, so
// the write-out of its table (the only global atomics of the staged
// strategies) is amortised over as many threads as possible.
#include <algorithm>
#include <cmath>
#include <vector>

#include <xyz_autodiff/accumulate.cuh>

#include "chain.cuh"
#include "common.cuh"
#include "rng.cuh"

namespace {

using xyz_autodiff::accumulate::BlockAccumulator;
using xyz_autodiff::accumulate::Strategy;

constexpr unsigned kBlock = 1024;
constexpr int kWidth = 6;
constexpr std::size_t kMaxLdsBytes = 160 * 1024;

struct AccumulateArgs {
    const float* in[6];  // sx, sy, theta, o, px, py
    const int* slot;
    float* grads;  // num_slots x 6
    std::size_t n;
    std::size_t per_block;  // multiple of kBlock
    int num_slots;
    int capacity;
    // The slots are dealt round-robin to 2^part_shift parts; a block serves one part (blockIdx % parts)
    // with a table of its own, and the blocks of all parts walk the same threads.  One part = no split.
    int part_shift;
    // byte offset of the spill staging area in the block's LDS, or 0 for none (tagged tables only)
    unsigned spill_offset;
    // copies of a small table, so that lanes sharing a slot do not share an LDS address
    int replicas;
    // a table smaller than the slot count: rows claimed on first use (1) or owned by the first slots (0)
    int claim_rows;
    // slots below this are the ones kept in `replicas` copies (negative: all)
    int hot_rows;
    // With claim_rows == 0 and a table smaller than the slot count: rows a block falls back to, claimed on
    // first use, if fewer than half of the first slots it sees are among the ones that own a row (0: never).
    // The layout by slot index is made for laws whose low slots are the hot ones; under any other law the
    // hot slots would go through the spill path, one same-address atomic after the other.
    int fallback_rows;
};

// Which part a block serves, the rows of its table and where they live in the global array.
struct Part {
    int index, parts, rows;
    __device__ explicit Part(const AccumulateArgs& a)
        : index(static_cast<int>(blockIdx.x) & ((1 << a.part_shift) - 1)),
          parts(1 << a.part_shift),
          rows((a.num_slots - index + parts - 1) >> a.part_shift) {}
    // table row of slot s, or -1 if s is out of range or belongs to another part
    __device__ __forceinline__ int row_of(int s, const AccumulateArgs& a) const {
        const bool mine = static_cast<unsigned>(s) < static_cast<unsigned>(a.num_slots) && (s & (parts - 1)) == index;
        return mine ? s >> a.part_shift : -1;
    }
};

template <Strategy S, int Peel, typename TableT, bool Spill = false>
__global__ void __launch_bounds__(kBlock) accumulate_kernel(AccumulateArgs a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const Part part(a);
    const std::size_t begin = static_cast<std::size_t>(blockIdx.x >> a.part_shift) * a.per_block;
    const std::size_t end = begin + a.per_block < a.n ? begin + a.per_block : a.n;
    using Acc = BlockAccumulator<float, kWidth, S, Peel, 4, TableT, Spill>;
    if (a.fallback_rows > 0) {  // the same for every block
        // the block's first slots as a sample of the law: who would find a row of its own?
        const std::size_t i = begin + threadIdx.x;
        const int sample = i < end ? part.row_of(a.slot[i], a) : -1;
        const int owners = Acc::main_rows_for(a.capacity, part.rows, a.replicas, a.hot_rows);
        // counted in the first two words of the table's memory, which the accumulator clears afterwards
        int* count = reinterpret_cast<int*>(lds);
        if (threadIdx.x < 2) count[threadIdx.x] = 0;
        __syncthreads();
        const int seen_here = __builtin_popcountll(xyz_autodiff::accumulate::wave::ballot(sample >= 0));
        const int served_here = __builtin_popcountll(xyz_autodiff::accumulate::wave::ballot(sample >= 0 && sample < owners));
        if (xyz_autodiff::accumulate::wave::lane_id() == 0) {
            atomicAdd(count + 0, seen_here);
            atomicAdd(count + 1, served_here);
        }
        __syncthreads();
        const int seen = count[0], served = count[1];
        __syncthreads();
        if (2 * served < seen) {
            a.capacity = a.fallback_rows;
            a.replicas = 1;
            a.claim_rows = 1;
            a.hot_rows = -1;
        }
    }
    Acc acc(lds, a.capacity, a.grads + part.index * kWidth, part.rows, part.parts * kWidth, a.replicas, a.claim_rows != 0,
            a.hot_rows);
    if constexpr (Spill) acc.use_spill_staging(reinterpret_cast<char*>(lds) + a.spill_offset);

    // The inputs of the next trip are requested before the arithmetic of this one, so that a lane has
    // two trips' worth of loads in flight instead of waiting for memory twice per trip (slot, then inputs).
    struct Inputs {
        int slot;  // as stored; -1 past the end
        float x[6];
    };
    auto fetch = [&](std::size_t base) {
        Inputs in{-1, {0.f, 0.f, 0.f, 0.f, 0.f, 0.f}};
        const std::size_t i = base + threadIdx.x;
        if (i < end) {
            in.slot = __builtin_nontemporal_load(a.slot + i);
#pragma unroll
            for (int k = 0; k < 6; ++k) in.x[k] = __builtin_nontemporal_load(a.in[k] + i);
        }
        return in;
    };
    Inputs current = fetch(begin);
    for (std::size_t base = begin; base < end; base += kBlock) {
        const Inputs next = fetch(base + kBlock);
        // a slot outside [0, num_slots) is dropped rather than written out of bounds
        const int slot = part.row_of(current.slot, a);
        float g[kWidth] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (slot >= 0) {
            const auto r = xad_chain::forward_backward<float>(current.x[0], current.x[1], current.x[2], current.x[3],
                                                              current.x[4], current.x[5]);
            g[0] = r.d_sx;
            g[1] = r.d_sy;
            g[2] = r.d_theta;
            g[3] = r.d_o;
            g[4] = r.d_px;
            g[5] = r.d_py;
        }
        acc.add(slot, g);
        current = next;
    }
    acc.flush();
}

// Same work with the accumulator used through drop-in leaves: the graph is
// written with SlotRef leaves in place of VariableRef leaves, and every
// add_grad of the backward pass goes through the LDS table one element at a time.
template <Strategy S, typename TableT>
__global__ void __launch_bounds__(kBlock) accumulate_leaf_kernel(AccumulateArgs a) {
    using namespace xyz_autodiff;
    using Acc = BlockAccumulator<float, kWidth, S, 0, 4, TableT>;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const Part part(a);
    Acc acc(lds, a.capacity, a.grads + part.index * kWidth, part.rows, part.parts * kWidth, a.replicas, true, a.hot_rows);

    const std::size_t begin = static_cast<std::size_t>(blockIdx.x >> a.part_shift) * a.per_block;
    const std::size_t end = begin + a.per_block < a.n ? begin + a.per_block : a.n;
    for (std::size_t base = begin; base < end; base += kBlock) {
        const std::size_t i = base + threadIdx.x;
        if (i < end) {
            float x[6];
#pragma unroll
            for (int k = 0; k < 6; ++k) x[k] = __builtin_nontemporal_load(a.in[k] + i);
            const int raw = __builtin_nontemporal_load(a.slot + i);
            const int slot = part.row_of(raw, a);
            const float* row = a.grads + static_cast<std::size_t>(slot < 0 ? 0 : raw) * kWidth;
            accumulate::SlotRef<2, float, Acc> s(x + 0, acc, slot, 0, row + 0);
            accumulate::SlotRef<1, float, Acc> theta(x + 2, acc, slot, 2, row + 2);
            accumulate::SlotRef<1, float, Acc> opacity(x + 3, acc, slot, 3, row + 3);
            accumulate::SlotRef<2, float, Acc> p(x + 4, acc, slot, 4, row + 4);
            auto es = op::exp(s);
            auto cov = op::scale_rotation_to_covariance_3param(es, theta);
            auto inv = op::sym_matrix2_inv(cov);
            auto q = op::mahalanobis_distance(p, inv);
            auto half_q = q * 0.5f;
            auto neg_half_q = op::neg(half_q);
            auto falloff = op::exp(neg_half_q);
            auto alpha = op::sigmoid(opacity);
            auto w = falloff * alpha;
            w.run();
        }
    }
    acc.flush();
}

__global__ void __launch_bounds__(256) zipf_kernel(int* dst, std::size_t n, std::uint64_t key, const double* cdf,
                                                   int num_slots) {
    const std::size_t stride = static_cast<std::size_t>(gridDim.x) * 256;
    for (std::size_t i = static_cast<std::size_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += stride) {
        const double u = static_cast<double>(xad_rng::bits(key, i) >> 11) * 0x1.0p-53;
        // first k with cdf[k] > u
        int lo = 0, hi = num_slots - 1;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (cdf[mid] > u)
                hi = mid;
            else
                lo = mid + 1;
        }
        dst[i] = lo;
    }
}

int device_compute_units(int* out) {
    int dev = 0;
    XAD_HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    XAD_HIP_TRY(hipGetDeviceProperties(&prop, dev));
    *out = prop.multiProcessorCount;
    return XAD_OK;
}

template <typename Kernel>
int launch(Kernel kernel, AccumulateArgs a, std::size_t lds_bytes, int blocks_per_cu, void* stream) {
    int cus = 0;
    if (int st = device_compute_units(&cus)) return st;
    if (lds_bytes > 64 * 1024)
        XAD_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        static_cast<int>(lds_bytes)));
    const std::size_t chunks = (a.n + kBlock - 1) / kBlock;
    const std::size_t resident = std::max<std::size_t>(1, (static_cast<std::size_t>(cus) * blocks_per_cu) >> a.part_shift);
    std::size_t blocks = std::min<std::size_t>(chunks, resident);  // per part
    const std::size_t chunks_per_block = (chunks + blocks - 1) / blocks;
    a.per_block = chunks_per_block * kBlock;
    blocks = (a.n + a.per_block - 1) / a.per_block;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(blocks << a.part_shift)), dim3(kBlock), lds_bytes,
                       xad::as_stream(stream), a);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

}  // namespace

extern "C" int xad_accumulate_chain_gradients_f32(int strategy, std::size_t n, const float* sx, const float* sy,
                                                  const float* theta, const float* o, const float* px,
                                                  const float* py, const int* slot, float* grads, int num_slots,
                                                  void* stream) {
    const char* who = "xad_accumulate_chain_gradients_f32";
    if (n == 0) return XAD_OK;
    AccumulateArgs a{{sx, sy, theta, o, px, py}, slot, grads, n, 0, num_slots, 0, 0, 0, 1, 1, -1, 0};
    for (int k = 0; k < 6; ++k) XAD_REQUIRE(a.in[k], "%s: input array %d is null", who, k);
    XAD_REQUIRE(slot && grads, "%s: slot or grads is null", who);
    XAD_REQUIRE(num_slots > 0, "%s: num_slots must be positive, got %d", who, num_slots);

    // Strategy AUTO: the LDS table.  With small tables replicated (below) it is the fastest at every
    // slot count measured, 1 to 262 144; the wavefront pre-reduction stays selectable.  Beyond what one
    // fp64 table holds, AUTO gives the rows to the first slots and sends the rest through the coalesced
    // spill: one walk over the inputs, no tags, no probing.
    constexpr std::size_t kSpillBytes = BlockAccumulator<float, kWidth>::spill_bytes(kBlock);
    constexpr std::size_t kRowBytes = kWidth * sizeof(double);
    // The first kHotRows slots are kept in several copies (lane l adds into copy l % copies): under a skewed
    // law over the slot index they take most of the adds, and lanes that share an LDS address serialise.
    constexpr int kHotRows = 64;
    if (strategy == XAD_ACCUMULATE_AUTO) {
        if (static_cast<std::size_t>(num_slots) * kRowBytes > 144 * 1024) {
            const int rows = static_cast<int>((kMaxLdsBytes - kSpillBytes) / kRowBytes);
            a.capacity = rows;
            a.claim_rows = 0;
            // Measured at 16 Mi threads, Zipf(1.1): 8 copies of the 32 hottest rows up to 16 384 slots (4096 slots
            // 0.162 ms against 0.181 without copies), 4 copies beyond, where the rows the copies take away
            // from the other slots cost more (262 144 slots: 0.241 ms with 4 copies, 0.257 with 8, 0.265 with none).
            a.replicas = num_slots <= 32768 ? 8 : 4;
            a.hot_rows = 32;
            a.fallback_rows = 2048;  // with their tags the most fp64 rows in a power of two that fit
            a.spill_offset = static_cast<unsigned>(static_cast<std::size_t>(rows) * kRowBytes);
            return launch(accumulate_kernel<Strategy::LdsAtomics, 0, double, true>, a, a.spill_offset + kSpillBytes, 1, stream);
        }
        if (num_slots > kHotRows) {
            // one fp64 table for every slot, the hot rows in as many copies as the LDS of a CU still holds
            a.hot_rows = kHotRows;
            a.replicas = 16;
            while (a.replicas > 1 &&
                   static_cast<std::size_t>(BlockAccumulator<float, kWidth>::rows_for(num_slots, a.replicas, kHotRows)) * kRowBytes > kMaxLdsBytes)
                a.replicas /= 2;
            a.capacity = BlockAccumulator<float, kWidth>::rows_for(num_slots, a.replicas, kHotRows);
            const std::size_t lds = static_cast<std::size_t>(a.capacity) * kRowBytes;
            return launch(accumulate_kernel<Strategy::LdsAtomics, 0, double>, a, lds, lds <= 72 * 1024 ? 2 : 1, stream);
        }
        strategy = XAD_ACCUMULATE_LDS;
    }
    // LDS table (at most 144 KiB): fp64 rows for every slot if they fit; if they fit in two
    // tables, the slots are dealt to two sets of blocks that each walk all threads (the inputs
    // are read twice, but ds_add_f64 is that much faster than ds_add_f32); otherwise fp32 rows
    // for every slot if those fit; otherwise rows claimed on first use (2048 fp64 or 4096 fp32, below).
    constexpr std::size_t kTableBudget = 144 * 1024;
    std::size_t cells = static_cast<std::size_t>(num_slots) * kWidth;
    bool f32_table = strategy == XAD_ACCUMULATE_LDS_F32;
    const bool staged = strategy != XAD_ACCUMULATE_GLOBAL_ATOMICS && strategy != XAD_ACCUMULATE_GLOBAL_LEAVES;
    if (staged && !f32_table && cells * sizeof(double) > kTableBudget &&
        ((static_cast<std::size_t>(num_slots) + 1) / 2) * kWidth * sizeof(double) <= kTableBudget) {
        a.part_shift = 1;
        cells = ((static_cast<std::size_t>(num_slots) + 1) / 2) * kWidth;
    }
    if (!f32_table && cells * sizeof(double) > kTableBudget) f32_table = true;
    std::size_t cell = f32_table ? sizeof(float) : sizeof(double);
    const bool direct = cells * cell <= kTableBudget;
    // rows claimed on first use: up to 262 144 slots 2048 fp64 rows rather than 4096 fp32 ones (ds_add_f32 is
    // 24x slower than ds_add_f64; beyond that the lower hit rate of the smaller table costs more than the
    // slower adds, measured on Zipf(1.1) slots), unless the fp32 table was asked for by name
    const bool tagged_f64 = !direct && staged && num_slots <= (1 << 18) && strategy != XAD_ACCUMULATE_LDS_F32 &&
                            strategy != XAD_ACCUMULATE_LDS_LEAVES;
    if (tagged_f64) cell = sizeof(double);
    a.capacity = direct ? static_cast<int>(cells / kWidth) : (tagged_f64 ? 2048 : 4096);
    if (direct && staged && a.part_shift == 0) {
        // a small table is replicated: up to 16 copies within 48 KiB (two blocks per CU stay resident)
        const std::size_t copy_rows = static_cast<std::size_t>(num_slots | 1);
        while (a.replicas < 16 && copy_rows * (a.replicas * 2) * kWidth * cell <= 48 * 1024) a.replicas *= 2;
        if (a.replicas > 1) a.capacity = BlockAccumulator<float, kWidth>::rows_for(num_slots, a.replicas, num_slots);
    }
    std::size_t lds = static_cast<std::size_t>(a.capacity) * kWidth * cell + (direct ? 0 : a.capacity * 4u);
    if (lds < 16) lds = 16;
    if (!direct && staged && strategy != XAD_ACCUMULATE_LDS_LEAVES) {
        // slots without a row: gathered per wavefront and written out coalesced
        a.spill_offset = static_cast<unsigned>(lds);
        lds += BlockAccumulator<float, kWidth>::spill_bytes(kBlock);
    }
    XAD_REQUIRE(lds <= kMaxLdsBytes, "%s: LDS table of %zu bytes does not fit", who, lds);
    const int per_cu = lds <= 72 * 1024 ? 2 : 1;  // two 1024-lane blocks fill a CU; 160 KiB of LDS hold two tables up to 72 KiB
    if (a.spill_offset && tagged_f64) {
        switch (strategy) {
            case XAD_ACCUMULATE_WAVE_LDS:
                return launch(accumulate_kernel<Strategy::WaveThenLds, 8, double, true>, a, lds, per_cu, stream);
            case XAD_ACCUMULATE_WAVE_LDS_SHALLOW:
                return launch(accumulate_kernel<Strategy::WaveThenLds, 2, double, true>, a, lds, per_cu, stream);
            default:
                return launch(accumulate_kernel<Strategy::LdsAtomics, 0, double, true>, a, lds, per_cu, stream);
        }
    }
    if (a.spill_offset) {
        switch (strategy) {
            case XAD_ACCUMULATE_WAVE_LDS:
                return launch(accumulate_kernel<Strategy::WaveThenLds, 8, float, true>, a, lds, per_cu, stream);
            case XAD_ACCUMULATE_WAVE_LDS_SHALLOW:
                return launch(accumulate_kernel<Strategy::WaveThenLds, 2, float, true>, a, lds, per_cu, stream);
            default:
                return launch(accumulate_kernel<Strategy::LdsAtomics, 0, float, true>, a, lds, per_cu, stream);
        }
    }
    if (f32_table && strategy != XAD_ACCUMULATE_GLOBAL_ATOMICS && strategy != XAD_ACCUMULATE_GLOBAL_LEAVES) {
        switch (strategy) {
            case XAD_ACCUMULATE_WAVE_LDS:
                return launch(accumulate_kernel<Strategy::WaveThenLds, 8, float>, a, lds, per_cu, stream);
            case XAD_ACCUMULATE_WAVE_LDS_SHALLOW:
                return launch(accumulate_kernel<Strategy::WaveThenLds, 2, float>, a, lds, per_cu, stream);
            case XAD_ACCUMULATE_LDS_LEAVES:
                return launch(accumulate_leaf_kernel<Strategy::LdsAtomics, float>, a, lds, per_cu, stream);
            default:
                return launch(accumulate_kernel<Strategy::LdsAtomics, 0, float>, a, lds, per_cu, stream);
        }
    }

    switch (strategy) {
        case XAD_ACCUMULATE_GLOBAL_ATOMICS:
            return launch(accumulate_kernel<Strategy::GlobalAtomics, 0, double>, a, 0, 2, stream);
        case XAD_ACCUMULATE_LDS:
            return launch(accumulate_kernel<Strategy::LdsAtomics, 0, double>, a, lds, per_cu, stream);
        case XAD_ACCUMULATE_WAVE_LDS:
            return launch(accumulate_kernel<Strategy::WaveThenLds, 8, double>, a, lds, per_cu, stream);
        case XAD_ACCUMULATE_WAVE_LDS_SHALLOW:
            return launch(accumulate_kernel<Strategy::WaveThenLds, 2, double>, a, lds, per_cu, stream);
        case XAD_ACCUMULATE_LDS_LEAVES:
            return launch(accumulate_leaf_kernel<Strategy::LdsAtomics, double>, a, lds, per_cu, stream);
        case XAD_ACCUMULATE_GLOBAL_LEAVES:
            return launch(accumulate_leaf_kernel<Strategy::GlobalAtomics, double>, a, 0, 2, stream);
        default:
            return xad::fail(XAD_ERR_INVALID_ARGUMENT, "%s: unknown strategy %d", who, strategy);
    }
}

extern "C" int xad_rng_zipf_i32(int* dst, std::size_t n, std::uint64_t seed, std::uint64_t stream_id, int num_slots,
                                double exponent, void* stream) {
    const char* who = "xad_rng_zipf_i32";
    if (n == 0) return XAD_OK;
    XAD_REQUIRE(dst, "%s: destination is null", who);
    XAD_REQUIRE(num_slots > 0 && exponent > 0.0, "%s: need num_slots > 0 and exponent > 0", who);
    std::vector<double> cdf(static_cast<std::size_t>(num_slots));
    double total = 0.0;
    for (int k = 0; k < num_slots; ++k) total += std::pow(static_cast<double>(k + 1), -exponent);
    double running = 0.0;
    for (int k = 0; k < num_slots; ++k) {
        running += std::pow(static_cast<double>(k + 1), -exponent);
        cdf[k] = running / total;
    }
    cdf[num_slots - 1] = 2.0;  // the search never runs off the end
    double* d_cdf = nullptr;
    XAD_HIP_TRY(hipMalloc(&d_cdf, cdf.size() * sizeof(double)));
    hipError_t st = hipMemcpy(d_cdf, cdf.data(), cdf.size() * sizeof(double), hipMemcpyHostToDevice);
    if (st == hipSuccess) {
        const unsigned grid = static_cast<unsigned>(std::min<std::size_t>((n + 255) / 256, 256u * 32u));
        hipLaunchKernelGGL(zipf_kernel, dim3(grid), dim3(256), 0, xad::as_stream(stream), dst, n,
                           xad_rng::stream_key(seed, stream_id), d_cdf, num_slots);
        st = hipGetLastError();
        if (st == hipSuccess) st = hipStreamSynchronize(xad::as_stream(stream));
    }
    (void)hipFree(d_cdf);
    if (st != hipSuccess) return xad::fail(XAD_ERR_HIP, "%s: %s", who, hipGetErrorString(st));
    return XAD_OK;
}
