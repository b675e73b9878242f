#pragma once
// Gradient accumulation for parameters shared by many threads.
//
// When thousands of lanes add into the same few gradient slots, one global
// atomic per lane per element (what VariableRef::add_grad does, and all that
// xyz-autodiff-cuda offers: include/xyz_autodiff/variable.cuh:48-50, exercised
// by tests/test_parallel_gradient_accumulation.cu:25-49) serialises at the L2
// channel that owns the hot cache line.  BlockAccumulator stages the sums on
// chip instead, in up to three levels:
//
//   1. wavefront   lanes of one wavefront that hit the same slot are summed
//                  with DPP row operations (no memory traffic at all) and only
//                  the group's first lane goes on;
//   2. block       the partial sums are added into a table in LDS with native
//                  LDS floating-point atomics;
//   3. device      once per block the table is written out with one global
//                  atomic per touched element.
//
// The table's element type is a template parameter and defaults to double even
// for float gradients.  Measured on MI355X with 16 wavefronts per CU: a
// ds_add_f32 wavefront instruction occupies the LDS pipeline for 192 cycles
// whatever its addresses (3 cycles per lane), a ds_add_f64 for 8 cycles when
// the 64 addresses are distinct, plus about 3 cycles per lane that shares an
// address with another.  So partial sums are kept in fp64 (which also makes them
// more accurate than the fp32 running sums of plain atomics).  Two ways to take
// the sharing lanes out of the LDS instruction: rows can be replicated, lane l
// adding into copy l % replicas (no extra instructions; the fastest at every
// slot count measured): every row of a small table, or only the first
// `hot_rows` rows of a large one, which under a skewed law over the slot index
// take most of the adds; or level 1 can sum a group of m sharing lanes
// first, which costs about 60 VALU issue cycles per group and saves about
// 3 m Width LDS cycles (MinGroup = 4 is where that starts to pay).
//
// The LDS table holds `capacity` slots of Width values, stored element-major
// (all slots' element 0, then element 1, ...) so that the lanes of one
// instruction, which all address the same element, spread over the banks.  If
// all num_slots fit, slot s uses row s.  Otherwise either the first `capacity`
// slots own the rows (no tags, no probing: right when the hot slots are the
// low-numbered ones, as with a Zipf law over the slot index) or rows are
// claimed on first use through a tag array (hashed, one probe, no eviction:
// under skewed access the hot slots arrive first and most often, so they own
// the rows wherever they are).  A slot without a row falls through to global
// atomics.
//
// Collective-call rules: construct(), add(), add_one() and flush() must be
// reached by every lane of every wavefront of the block, in uniform control
// flow (lanes with nothing to add pass a negative slot); the block size must
// be a multiple of 64.
//
// SlotRef<N, T, Acc> is a drop-in leaf: a VariableRef whose add_grad goes
// through an accumulator, so graphs and op logic stay unchanged.

#include <cstddef>
#include <cstdint>

#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/detail/atomic.cuh>
#include <xyz_autodiff/detail/config.cuh>

#if defined(__HIPCC__)

namespace xyz_autodiff {
namespace accumulate {

enum class Strategy {
    GlobalAtomics,  // level 3 only: one global atomic per lane per element
    LdsAtomics,     // levels 2 + 3
    WaveThenLds,    // levels 1 + 2 + 3
};

namespace wave {

__device__ __forceinline__ unsigned lane_id() { return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }

__device__ __forceinline__ std::uint64_t ballot(bool predicate) { return __builtin_amdgcn_ballot_w64(predicate); }

template <int Ctrl>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), Ctrl, 0xF, 0xF, true);
    return v + __builtin_bit_cast(float, moved);
}

__device__ __forceinline__ float read_lane(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// 64-bit values travel as two 32-bit halves.
template <int Ctrl>
__device__ __forceinline__ double dpp_add(double v) {
    const std::uint64_t u = __builtin_bit_cast(std::uint64_t, v);
    const unsigned lo = __builtin_amdgcn_update_dpp(0, static_cast<int>(u), Ctrl, 0xF, 0xF, true);
    const unsigned hi = __builtin_amdgcn_update_dpp(0, static_cast<int>(u >> 32), Ctrl, 0xF, 0xF, true);
    return v + __builtin_bit_cast(double, (static_cast<std::uint64_t>(hi) << 32) | lo);
}

__device__ __forceinline__ double read_lane(double v, int lane) {
    const std::uint64_t u = __builtin_bit_cast(std::uint64_t, v);
    const unsigned lo = __builtin_amdgcn_readlane(static_cast<int>(u), lane);
    const unsigned hi = __builtin_amdgcn_readlane(static_cast<int>(u >> 32), lane);
    return __builtin_bit_cast(double, (static_cast<std::uint64_t>(hi) << 32) | lo);
}

// Sum of v over all 64 lanes, returned to every lane.  Four DPP steps reduce
// each row of 16 (quad swaps, then the two mirrors), four scalar reads combine
// the rows.
template <typename V>
__device__ __forceinline__ V sum(V v) {
    v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v);  // row_half_mirror
    v = dpp_add<0x140>(v);  // row_mirror
    return (read_lane(v, 0) + read_lane(v, 16)) + (read_lane(v, 32) + read_lane(v, 48));
}

}  // namespace wave

template <typename T, int Width, Strategy S = Strategy::LdsAtomics, int PeelRounds = 8, int MinGroup = 4,
          typename TableT = double, bool Spill = false>
class BlockAccumulator {
    static_assert(!Spill || sizeof(T) == 4, "spill staging is implemented for 4-byte values");


public:
    using table_type = TableT;
    static constexpr int kEmpty = -1;

    // Bytes of LDS the block must provide for `capacity` rows.
    // (tagged: rows claimed on first use, which needs a tag per row)
    __host__ __device__ static constexpr std::size_t lds_bytes(int capacity, bool tagged) {
        if (S == Strategy::GlobalAtomics) return 0;
        return static_cast<std::size_t>(capacity) * Width * sizeof(TableT) + (tagged ? static_cast<std::size_t>(capacity) * 4 : 0);
    }

    // `lds`: at least lds_bytes(capacity, tagged) bytes, 16-byte aligned.  `capacity`: rows of the table.
    // `global`: num_slots rows of Width values, already initialised; row s starts at
    // global + s * row_stride (row_stride = Width for a dense row-major array; a larger
    // stride lets several accumulators share one array, each owning every k-th row).
    // `claim_rows` (only matters when the slots do not all get a row): true = rows are claimed on
    // first use through the tag array (capacity must then be a power of two, replicas 1); false = the
    // first slots own the rows and no tags are kept.
    // `replicas` (a power of two; 1 = none) and `hot_rows` (negative = every slot): slots below
    // hot_rows are kept in that many copies and lane l adds into copy l % replicas, so lanes of one
    // instruction that share such a slot no longer share an address (each sharing lane costs an LDS
    // atomic about 3 cycles); flush() adds the copies up.  The copies take (replicas - 1) *
    // (hot_rows | 1) rows of the capacity, after the rows of the slots themselves (rows_for()).
    // Clears the table; ends with a block barrier.
    __device__ BlockAccumulator(void* lds, int capacity, T* global, int num_slots, int row_stride = Width,
                                int replicas = 1, bool claim_rows = true, int hot_rows = -1)
        : table_(static_cast<TableT*>(lds)),
          tags_(reinterpret_cast<int*>(static_cast<TableT*>(lds) + static_cast<std::size_t>(capacity) * Width)),
          global_(global),
          capacity_(capacity),
          num_slots_(num_slots),
          row_stride_(row_stride),
          tagged_(replicas == 1 && num_slots > capacity && claim_rows),
          shift_(32 - __builtin_ctz(static_cast<unsigned>(capacity))),
          replicas_(replicas) {
        hot_ = replicas > 1 ? (hot_rows < 0 || hot_rows > num_slots ? num_slots : hot_rows) : 0;
        hot_stride_ = hot_ | 1;
        main_rows_ = tagged_ ? capacity : main_rows_for(capacity, num_slots, replicas, hot_rows);
        if (hot_ > main_rows_) hot_ = main_rows_;
        copies_base_ = main_rows_ | 1;
        const int copy = static_cast<int>(wave::lane_id() & static_cast<unsigned>(replicas - 1));
        my_copy_ = copy == 0 ? 0 : copies_base_ + (copy - 1) * hot_stride_;
        clear();
    }

    // Slots that own a row of a table of `capacity` rows that is not tagged: all of them if they fit, else the
    // first ones, as many as the rows left once the copies of the hot ones are set aside (the copies start at
    // an odd row: main rows | 1 must fit in front of them).
    __host__ __device__ static constexpr int main_rows_for(int capacity, int num_slots, int replicas, int hot_rows) {
        const int hot = replicas > 1 ? (hot_rows < 0 || hot_rows > num_slots ? num_slots : hot_rows) : 0;
        const int in_front = capacity - (replicas - 1) * (hot | 1);
        const int left = replicas > 1 ? ((in_front & 1) ? in_front : in_front - 1) : capacity;
        return num_slots < left ? num_slots : left;
    }

    // Rows a table needs for `slots` slots of which the first `hot_rows` are kept in `replicas` copies.
    __host__ __device__ static constexpr int rows_for(int slots, int replicas, int hot_rows) {
        return replicas > 1 ? (slots | 1) + (replicas - 1) * (hot_rows | 1) : slots;
    }

    // Rows a wavefront can stage per round of the spill path below.
    static constexpr int kStageRows = 16;

    // Bytes of LDS for use_spill_staging() in a block of `threads` lanes.
    __host__ __device__ static constexpr std::size_t spill_bytes(int threads) {
        return static_cast<std::size_t>(threads / 64) * kStageRows * (Width + 1) * 4;
    }

    // With Spill (tables of 4-byte values that do not hold every slot): contributions that find no
    // row are not sent to `global` lane by lane (Width instructions, each touching up to 64 rows) but
    // are first gathered per wavefront in `staging` (spill_bytes(blockDim.x) bytes of LDS, 4-byte
    // aligned), kStageRows at a time, and written out with consecutive lanes on consecutive elements
    // of consecutive rows, which cuts the number of memory requests several times.  Rows wait there
    // until kStageRows have come together; flush() writes out what is left.  Must be called
    // before the first add(); add() must then be reached by all lanes of a wavefront together
    // whatever the strategy.
    __device__ void use_spill_staging(void* staging) {
        static_assert(Spill, "declare the accumulator with Spill = true");
        spill_ = static_cast<std::uint32_t*>(staging) + (threadIdx.x / 64) * kStageRows * (Width + 1);
    }

    // Adds g[0..Width) to slot `slot` (no-op for slot < 0).
    __device__ __forceinline__ void add(int slot, const T (&g)[Width]) {
        if constexpr (S == Strategy::GlobalAtomics) {
            if (slot >= 0) {
#pragma unroll
                for (int k = 0; k < Width; ++k) detail::atomic_add(global_ + static_cast<std::size_t>(slot) * row_stride_ + k, g[k]);
            }
        } else {
            if constexpr (S == Strategy::WaveThenLds) slot = peel(slot, g);
            if constexpr (Spill)
                deposit_together(slot, g);
            else if (slot >= 0)
                deposit(slot, g);
        }
    }

    // Adds one value to element `element` of slot `slot`.
    __device__ __forceinline__ void add_one(int slot, int element, T value) {
        if constexpr (S == Strategy::GlobalAtomics) {
            if (slot >= 0) detail::atomic_add(global_ + static_cast<std::size_t>(slot) * row_stride_ + element, value);
        } else {
            if (slot < 0) return;
            const int row = find_row(slot);
            if (row >= 0)
                detail::atomic_add(table_ + element * capacity_ + row, static_cast<TableT>(value));
            else
                detail::atomic_add(global_ + static_cast<std::size_t>(slot) * row_stride_ + element, value);
        }
    }

    // Writes the table out (one global atomic per non-zero element) and clears
    // it, so the object can take another round of add().
    __device__ void flush() {
        if constexpr (S == Strategy::GlobalAtomics) return;
        if constexpr (Spill) {
            if (spill_ != nullptr && staged_ != 0) write_out_staged();
        }
        __syncthreads();
        // e runs over the global layout (slot-major) so the atomics of a
        // wavefront touch consecutive addresses.
        for (int e = threadIdx.x; e < main_rows_ * Width; e += blockDim.x) {
            const int row = e / Width, element = e % Width;
            const int slot = tagged_ ? tags_[row] : row;
            TableT sum = table_[element * capacity_ + row];
            if (row < hot_)
                for (int copy = 1; copy < replicas_; ++copy)
                    sum += table_[element * capacity_ + copies_base_ + (copy - 1) * hot_stride_ + row];
            const T v = static_cast<T>(sum);
            if (slot != kEmpty && v != T(0)) detail::atomic_add(global_ + static_cast<std::size_t>(slot) * row_stride_ + element, v);
        }
        __syncthreads();
        clear();
    }

private:
    __device__ void clear() {
        if constexpr (S == Strategy::GlobalAtomics) return;
        for (int e = threadIdx.x; e < capacity_ * Width; e += blockDim.x) table_[e] = TableT(0);
        if (tagged_)
            for (int e = threadIdx.x; e < capacity_; e += blockDim.x) tags_[e] = kEmpty;
        __syncthreads();
    }

    // Row of the LDS table that holds `slot`, or -1 if the slot has none.
    __device__ __forceinline__ int find_row(int slot) {
        if (!tagged_) return slot < hot_ ? slot + my_copy_ : (slot < main_rows_ ? slot : -1);
        const int row = static_cast<int>((static_cast<unsigned>(slot) * 2654435761u) >> shift_);
        int owner = tags_[row];
        if (owner == kEmpty) {
            const int seen = atomicCAS(tags_ + row, kEmpty, slot);
            owner = seen == kEmpty ? slot : seen;
        }
        return owner == slot ? row : -1;
    }

    __device__ __forceinline__ void deposit(int slot, const T (&g)[Width]) {
        const int row = find_row(slot);
        if (row >= 0) {
#pragma unroll
            for (int k = 0; k < Width; ++k) detail::atomic_add(table_ + k * capacity_ + row, static_cast<TableT>(g[k]));
        } else {
#pragma unroll
            for (int k = 0; k < Width; ++k) detail::atomic_add(global_ + static_cast<std::size_t>(slot) * row_stride_ + k, g[k]);
        }
    }

    // deposit() for a whole wavefront (lanes with slot < 0 have nothing): hits go to the table,
    // misses are compacted into the wavefront's staging rows.
    __device__ __forceinline__ void deposit_together(int slot, const T (&g)[Width]) {
        const int row = slot >= 0 ? find_row(slot) : -1;
        if (row >= 0) {
#pragma unroll
            for (int k = 0; k < Width; ++k) detail::atomic_add(table_ + k * capacity_ + row, static_cast<TableT>(g[k]));
        }
        // Misses wait in the staging rows until these are full (or until flush()): a round of stores for
        // the one or two misses of a typical call would cost more than the misses themselves.
        bool miss = slot >= 0 && row < 0;
        for (std::uint64_t missing = wave::ballot(miss); missing != 0; missing = wave::ballot(miss)) {
            const unsigned before = __builtin_amdgcn_mbcnt_hi(static_cast<unsigned>(missing >> 32),
                                                              __builtin_amdgcn_mbcnt_lo(static_cast<unsigned>(missing), 0u));
            const unsigned room = static_cast<unsigned>(kStageRows) - staged_;
            if (miss && before < room) {
                std::uint32_t* mine = spill_ + (staged_ + before) * (Width + 1);
                mine[0] = static_cast<std::uint32_t>(slot);
#pragma unroll
                for (int k = 0; k < Width; ++k) mine[1 + k] = __builtin_bit_cast(std::uint32_t, g[k]);
                miss = false;
            }
            const unsigned waiting = static_cast<unsigned>(__builtin_popcountll(missing));
            if (waiting <= room) {  // the same for every lane
                staged_ += waiting;
                break;
            }
            staged_ = static_cast<unsigned>(kStageRows);
            write_out_staged();
        }
    }

    // The wavefront's staged rows (slot, g[0..Width)) go out with lane l on element l % Width of staged
    // row l / Width, then the next 64 elements, ...
    __device__ __forceinline__ void write_out_staged() {
        __builtin_amdgcn_wave_barrier();
        const int elements = static_cast<int>(staged_) * Width;
        for (int e = static_cast<int>(wave::lane_id()); e < elements; e += 64) {
            const int entry = e / Width, k = e - entry * Width;
            const std::uint32_t* staged = spill_ + entry * (Width + 1);
            const T value = __builtin_bit_cast(T, staged[1 + k]);
            if (value != T(0))
                detail::atomic_add(global_ + static_cast<std::size_t>(staged[0]) * row_stride_ + k, value);
        }
        __builtin_amdgcn_wave_barrier();
        staged_ = 0;
    }

    // Level 1.  Take the slot of the first lane that is still waiting and find
    // every lane with the same slot.  If they are at least MinGroup, sum their
    // values across the wavefront, let the first of them deposit the sums, and
    // look at the next waiting lane (at most PeelRounds groups per call);
    // otherwise stop: under skewed access a small leading group means the rest
    // of the wavefront is scattered too, and those lanes are cheaper to deposit
    // directly.  Returns the slot this lane still has to deposit itself (-1 if
    // its contribution has been taken care of).
    __device__ __forceinline__ int peel(int slot, const T (&g)[Width]) {
        std::uint64_t waiting = wave::ballot(slot >= 0);
        for (int round = 0; round < PeelRounds && waiting != 0; ++round) {
            const int leader = __builtin_ctzll(waiting);
            const int leader_slot = __builtin_amdgcn_readlane(slot, leader);
            const bool member = slot == leader_slot;
            const std::uint64_t group = wave::ballot(member);
            if (__builtin_popcountll(group) < MinGroup) break;
            waiting &= ~group;
            T total[Width];
#pragma unroll
            for (int k = 0; k < Width; ++k) total[k] = wave::sum(member ? g[k] : T(0));
            if (static_cast<int>(wave::lane_id()) == leader) deposit(leader_slot, total);
            if (member) slot = -1;
        }
        return slot;
    }

    TableT* table_;
    int* tags_;
    T* global_;
    int capacity_;
    int num_slots_;
    int row_stride_;
    bool tagged_;  // rows claimed on first use (tags_ says by which slot)
    int shift_;
    int replicas_;
    int main_rows_;    // slots 0 .. main_rows_-1 own rows 0 .. main_rows_-1 (tagged: all rows, claimed)
    int hot_;          // slots below this are kept in replicas_ copies
    int hot_stride_;   // rows between two copies (odd, so copies of a slot fall into different banks)
    int copies_base_;  // first row of the second copy
    int my_copy_;      // offset of this lane's copy of a hot row (0 for the first copy)
    std::uint32_t* spill_ = nullptr;
    unsigned staged_ = 0;  // rows waiting in spill_; the same in every lane of a wavefront
};

// A leaf that reads its values like a VariableRef and sends its gradients to a
// BlockAccumulator: element i of this leaf is element `offset + i` of slot
// `slot` in the accumulator's table.  zero_grad() is a no-op (the table is
// owned and cleared by the accumulator); grad(i) is not readable before the
// accumulator has been flushed, and returns the global value.
template <std::size_t N, typename T, typename Acc>
class SlotRef {
public:
    using value_type = T;
    static constexpr std::size_t size = N;

    __device__ SlotRef(T* values, Acc& acc, int slot, int offset, const T* global_grads)
        : values_(values), acc_(&acc), grads_(global_grads), slot_(slot), offset_(offset) {}

    __device__ __forceinline__ T& operator[](std::size_t i) const { return values_[i]; }
    __device__ __forceinline__ const T& grad(std::size_t i) const { return grads_[i]; }
    __device__ __forceinline__ void add_grad(std::size_t i, T g) const { acc_->add_one(slot_, offset_ + static_cast<int>(i), g); }
    __device__ __forceinline__ void zero_grad() const {}

private:
    T* values_;
    Acc* acc_;
    const T* grads_;
    int slot_;
    int offset_;
};

}  // namespace accumulate
}  // namespace xyz_autodiff

#endif  // __HIPCC__
