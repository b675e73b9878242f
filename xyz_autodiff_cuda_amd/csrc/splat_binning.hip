// Binning of the splatting step: from the tile rectangle of every Gaussian to one list of Gaussians
// per tile, each in (depth, index) order.  Integer work only; no library primitive, no host read-back.
//
// The lists are a sparse transpose: Gaussian-major (a rectangle of tiles per Gaussian) to tile-major.
// A comparison sort or a radix sort of (tile, Gaussian) pairs moves every pair several times; here a
// pair is written once.  The Gaussians are walked in depth order, and what keeps each list in that
// order is the walk itself, not a sort:
//
//   level A   Gaussians -> supertiles (8 x 8 tiles).  A wavefront takes a range of the depth-ordered
//             Gaussians and 64 supertiles, one per lane.  64 Gaussians are loaded at a time, one per
//             lane; the rectangle of each in turn is broadcast (v_readlane) and every lane tests its
//             own supertile against it.  A first pass counts, the counts of all (supertile, range)
//             cells are scanned in supertile-major order, and a second pass writes each Gaussian at
//             its lane's cursor.  Ranges are visited in order inside every supertile, Gaussians in
//             order inside every range: the list of a supertile comes out in depth order.
//   level B   supertile -> its 64 tiles: a wavefront takes 64 entries of one supertile's list, one per
//             lane.  The lane that loads a Gaussian forms the 64-bit mask of the tiles its rectangle
//             covers inside the supertile (row mask x column multiplier).  Those 64 masks are a 64 x 64
//             bit matrix, entries by tiles; it is transposed across the lanes in six exchange steps,
//             after which lane t holds, for tile t, the mask of the entries that cover it: its
//             population count is the tile's count, and its set bits, walked from the lowest, are the
//             tile's Gaussians in list order.
//
// Work per (Gaussian, supertile) pair is a handful of wavefront instructions; the stores of the final
// lists are 4 bytes per pair, each pair once.  All sizes that depend on the data (pairs per
// supertile, pairs in total) stay on the device: grids are sized by the capacity of the buffers, idle
// wavefronts leave at once, every store is checked against the capacity, and an overflow is
// recorded in the status words for the host to see whenever it next waits for the stream.
//
// Replaces, for the tile-binned renderer, what the reference does not have at all: its renderer
// visits every Gaussian at every pixel (examples/mini-gaussian-splatting/gaussian_splatting_kernel.cu:33-62).
#include <xyz_autodiff/accumulate.cuh>

#include "common.cuh"
#include "splat.cuh"
#include "splat_launch.cuh"

namespace xad_splat {

namespace {

using xyz_autodiff::accumulate::wave::ballot;

__device__ __forceinline__ std::uint32_t read_lane(std::uint32_t v, int lane) {
    return static_cast<std::uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), lane));
}

// ---------------------------------------------------------------------------
// Exclusive scan of n 32-bit counts, in place, in one launch (chained scan with decoupled look-back).
// Blocks take tickets, so a block only ever waits for blocks that are already running.  The state
// words carry the launch's epoch, so nothing has to be cleared between launches: a word of another
// epoch simply is not there yet.  data[n] receives the total.
// Tickets and epoch live in three control words on the device (tickets given out, blocks finished, epoch);
// the block that finishes last puts the first two back to zero and moves the epoch on.  Nothing about
// a launch depends on what the host knows of earlier launches, so a recorded launch can be replayed.
enum : int { kScanTickets = 0, kScanFinished = 1, kScanEpoch = 2 };
constexpr unsigned kScanBlock = 1024;
constexpr unsigned kScanItems = 16;
constexpr unsigned kScanTile = kScanBlock * kScanItems;  // few, large blocks: the chain of look-backs stays short

__device__ __forceinline__ std::uint64_t scan_word(std::uint32_t epoch, std::uint32_t inclusive, std::uint32_t value) {
    return (static_cast<std::uint64_t>((epoch << 1) | inclusive) << 32) | value;
}

__global__ void __launch_bounds__(kScanBlock) scan_kernel(std::uint32_t* __restrict__ data, std::uint32_t n,
                                                          std::uint64_t* __restrict__ state, std::uint32_t* __restrict__ control) {
    __shared__ std::uint32_t wave_total[kScanBlock / 64];
    __shared__ std::uint32_t block_index, block_exclusive, launch_epoch;
    const unsigned t = threadIdx.x;
    if (t == 0) {
        launch_epoch = __hip_atomic_load(control + kScanEpoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // before the ticket: it moves on only after every block has one
        block_index = atomicAdd(control + kScanTickets, 1u);
    }
    __syncthreads();
    const std::uint32_t b = block_index;
    const std::uint32_t epoch = launch_epoch;
    const std::uint32_t first = b * kScanTile + t * kScanItems;

    std::uint32_t v[kScanItems];
    if (first + kScanItems <= n) {
#pragma unroll
        for (unsigned k = 0; k < kScanItems; k += 4) {
            const uint4 q = *reinterpret_cast<const uint4*>(data + first + k);
            v[k] = q.x; v[k + 1] = q.y; v[k + 2] = q.z; v[k + 3] = q.w;
        }
    } else {
#pragma unroll
        for (unsigned k = 0; k < kScanItems; ++k) v[k] = first + k < n ? data[first + k] : 0u;
    }
    std::uint32_t mine = 0;
#pragma unroll
    for (unsigned k = 0; k < kScanItems; ++k) mine += v[k];

    // inclusive scan of the per-thread sums: within each wavefront by shuffles, across the wavefronts through LDS
    const unsigned lane = t & 63u, wave = t >> 6;
    std::uint32_t inclusive_in_wave = mine;
#pragma unroll
    for (unsigned step = 1; step < 64; step *= 2) {
        const std::uint32_t other = __shfl_up(inclusive_in_wave, step, 64);
        if (lane >= step) inclusive_in_wave += other;
    }
    if (lane == 63) wave_total[wave] = inclusive_in_wave;
    __syncthreads();
    std::uint32_t before_wave = 0, aggregate = 0;
#pragma unroll
    for (unsigned w = 0; w < kScanBlock / 64; ++w) {
        const std::uint32_t total = wave_total[w];
        before_wave += w < wave ? total : 0u;
        aggregate += total;
    }
    const std::uint32_t thread_exclusive = before_wave + inclusive_in_wave - mine;

    // Look-back, by the block's first wavefront: 64 predecessors at a time, nearest first.  Each lane waits
    // for its predecessor's word of this epoch (that block holds an earlier ticket, so it is running),
    // the sums up to and including the nearest inclusive prefix are added, and if there was none among
    // the 64 the next 64 are looked at.  Lanes that would reach before block 0 count as an inclusive zero.
    if (t < 64) {
        if (b > 0 && t == 0) __hip_atomic_store(state + b, scan_word(epoch, 0u, aggregate), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        std::uint32_t exclusive = 0;
        for (std::int64_t nearest = static_cast<std::int64_t>(b) - 1; nearest >= 0; nearest -= 64) {
            const std::int64_t mine_at = nearest - static_cast<std::int64_t>(t);
            std::uint64_t word = scan_word(epoch, 1u, 0u);
            if (mine_at >= 0) {
                do {
                    word = __hip_atomic_load(state + mine_at, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
                } while (static_cast<std::uint32_t>(word >> 33) != epoch);
            }
            const std::uint64_t inclusive = ballot(((word >> 32) & 1u) != 0);
            const unsigned stop = static_cast<unsigned>(__builtin_ctzll(inclusive | (std::uint64_t(1) << 63)));
            std::uint32_t part = t <= stop ? static_cast<std::uint32_t>(word) : 0u;
            for (int offset = 32; offset > 0; offset >>= 1) part += __shfl_xor(part, offset, 64);
            exclusive += part;
            if (inclusive != 0) break;
        }
        if (t == 0) {
            __hip_atomic_store(state + b, scan_word(epoch, 1u, exclusive + aggregate), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
            block_exclusive = exclusive;
            if (static_cast<std::uint64_t>(b + 1) * kScanTile >= n) data[n] = exclusive + aggregate;  // the last block: the total
        }
    }
    __syncthreads();

    std::uint32_t running = block_exclusive + thread_exclusive;
    if (first + kScanItems <= n) {
#pragma unroll
        for (unsigned k = 0; k < kScanItems; k += 4) {
            uint4 q;
            q.x = running; running += v[k];
            q.y = running; running += v[k + 1];
            q.z = running; running += v[k + 2];
            q.w = running; running += v[k + 3];
            *reinterpret_cast<uint4*>(data + first + k) = q;
        }
    } else {
#pragma unroll
        for (unsigned k = 0; k < kScanItems; ++k) {
            if (first + k < n) data[first + k] = running;
            running += v[k];
        }
    }
    // the block that finishes last leaves the control words ready for the next launch (epoch 0 is never
    // used: the state words start out as zero)
    if (t == 0 && atomicAdd(control + kScanFinished, 1u) == gridDim.x - 1) {
        const std::uint32_t next = (epoch + 1) & 0x3fffffffu;
        control[kScanTickets] = 0;
        control[kScanFinished] = 0;
        control[kScanEpoch] = next == 0 ? 1u : next;
    }
}

// ---------------------------------------------------------------------------
// Transpose of a 64 x 64 bit matrix held one row per lane (lo = columns 0..31, hi = columns 32..63):
// afterwards lane t holds column t, bit j of it being bit t of lane j's row.  The usual recursive block
// swap: at distance k, the lanes whose bit k is clear keep their columns with bit k clear and receive,
// into their columns with bit k set, the partner's columns with bit k clear; the others the reverse.
__device__ __forceinline__ void transpose_64x64(std::uint32_t& lo, std::uint32_t& hi, int lane) {
    {
        const std::uint32_t other_lo = __shfl_xor(lo, 32, 64), other_hi = __shfl_xor(hi, 32, 64);
        if (lane & 32)
            lo = other_hi;
        else
            hi = other_lo;
    }
    constexpr std::uint32_t kClear[5] = {0x0000ffffu, 0x00ff00ffu, 0x0f0f0f0fu, 0x33333333u, 0x55555555u};
#pragma unroll
    for (int step = 0; step < 5; ++step) {
        const int k = 16 >> step;
        const std::uint32_t m = kClear[step];
        const std::uint32_t other_lo = __shfl_xor(lo, k, 64), other_hi = __shfl_xor(hi, k, 64);
        if (lane & k) {
            lo = ((other_lo >> k) & m) | (lo & ~m);
            hi = ((other_hi >> k) & m) | (hi & ~m);
        } else {
            lo = (lo & m) | ((other_lo & m) << k);
            hi = (hi & m) | ((other_hi & m) << k);
        }
    }
}

// ---------------------------------------------------------------------------
// Both levels turn 64 rectangles into 64 lists the same way.  Lane = rectangle: the 8 x 8 cells it covers,
// as a 64-bit mask (cell = 8 row + column).  After the transpose, lane = cell, and the mask says which of
// the 64 rectangles cover it: its population count is the cell's count, its set bits, from the lowest, are
// the cell's members in order.

// Bits x0..x1 of every row y0..y1 (all within 0..7; empty if a range is).
__device__ __forceinline__ std::uint64_t block_mask(int x0, int x1, int y0, int y1) {
    if (x0 > x1 || y0 > y1) return 0;
    const std::uint64_t row = ((std::uint64_t(1) << (x1 - x0 + 1)) - 1) << x0;
    const std::uint64_t rows = (0x0101010101010101ull >> (8 * (7 - (y1 - y0)))) << (8 * y0);
    return row * rows;  // the multiplier has one bit per row: no carries
}

// Writes the members of every lane's mask (lane j's value `id` for bit j) to out[from ...], lane by lane.
// One entry per lane and turn would scatter every store over 64 cache lines.  The entries go through LDS
// instead: lane t puts its run at [before, before + count) there, and the runs are written out with
// consecutive lanes on consecutive entries of a run (a window of LDS at a time).  Stores at or beyond
// `capacity` are dropped.  Returns the lane's count.  Every lane of the wavefront must call it.
constexpr std::uint32_t kStageEntries = 1024;
struct RunStage {
    std::uint32_t staged[kStageEntries];
    std::uint32_t run_begin[65];
    std::uint32_t run_dest[64];
};

__device__ __forceinline__ std::uint32_t write_runs(RunStage& lds, std::uint64_t mine, std::uint32_t id, std::uint32_t from,
                                                    std::uint32_t* __restrict__ out, std::uint32_t capacity, int lane) {
    const std::uint32_t count = static_cast<std::uint32_t>(__builtin_popcountll(mine));
    std::uint32_t inclusive = count;
#pragma unroll
    for (int step = 1; step < 64; step *= 2) {
        const std::uint32_t other = __shfl_up(inclusive, step, 64);
        if (lane >= step) inclusive += other;
    }
    const std::uint32_t total = read_lane(inclusive, 63);
    std::uint32_t next = inclusive - count;  // where this lane's next entry goes
    __syncthreads();                         // the previous call's readers are done
    lds.run_begin[lane] = next;
    if (lane == 63) lds.run_begin[64] = total;
    lds.run_dest[lane] = from;
    for (std::uint32_t window = 0; window < total; window += kStageEntries) {
        // every lane stays in the loop until the last one is done: the exchange below reads other lanes' registers
        while (ballot(mine != 0 && next < window + kStageEntries) != 0) {
            const bool has = mine != 0 && next < window + kStageEntries;
            const int j = has ? __builtin_ctzll(mine) : 0;
            const std::uint32_t member = __shfl(id, j, 64);
            if (has) {
                lds.staged[next - window] = member;
                ++next;
                mine &= mine - 1;
            }
        }
        __syncthreads();
        const std::uint32_t end = total - window < kStageEntries ? total - window : kStageEntries;
        for (std::uint32_t e = static_cast<std::uint32_t>(lane); e < end; e += 64) {
            const std::uint32_t at = window + e;
            int t = 0;  // the run `at` lies in: the last one that begins at or before it (empty runs begin where the next one does)
#pragma unroll
            for (int step = 32; step > 0; step >>= 1)
                if (lds.run_begin[t + step] <= at) t += step;
            const std::uint32_t dest = lds.run_dest[t] + (at - lds.run_begin[t]);
            if (dest < capacity) out[dest] = lds.staged[e];
        }
        __syncthreads();
    }
    return count;
}

// Supertiles are numbered group by group, a group being 8 x 8 supertiles (row-major within the group,
// groups row-major over the image); numbers whose supertile lies beyond the image stay empty.
struct SuperCoords {
    int x, y;
    bool inside;
};
__device__ __forceinline__ SuperCoords super_coords(const BinPlan& p, int s) {
    const int group = s >> 6, local = s & 63;
    SuperCoords c;
    c.x = (group % p.group_x) * 8 + (local & 7);
    c.y = (group / p.group_x) * 8 + (local >> 3);
    c.inside = c.x < p.super_x && c.y < p.super_y;
    return c;
}

// ---------------------------------------------------------------------------
// Level A.  One wavefront per block; block = (range of Gaussians) x (group of 8 x 8 supertiles), blocks of
// one range adjacent so that they read the same rectangles from the same L2.  64 Gaussians at a time:
// lane = Gaussian, mask = the group's supertiles its rectangle reaches; transposed, lane = supertile.
// kFill = false: matrix_a[supertile * ranges_a + range] = number of Gaussians of the range that
// touch the supertile.  kFill = true: matrix_a holds the scanned counts; the Gaussians are written.
// rects_by_depth[i] is the rectangle of Gaussian by_depth[i]: both loads of a lane are independent and coalesced.
template <bool kFill>
__global__ void __launch_bounds__(64) super_kernel(BinPlan p, const std::uint32_t* __restrict__ by_depth,
                                                   const TileRect* __restrict__ rects_by_depth,
                                                   std::uint32_t* __restrict__ matrix_a, std::uint32_t* __restrict__ list_a) {
    __shared__ RunStage stage;
    const int lane = static_cast<int>(threadIdx.x);
    const int group = static_cast<int>(blockIdx.x % static_cast<unsigned>(p.groups));
    const int range = static_cast<int>(blockIdx.x / static_cast<unsigned>(p.groups));
    const int origin_x = (group % p.group_x) * 8, origin_y = (group / p.group_x) * 8;  // in supertiles
    const std::size_t cell = static_cast<std::size_t>(group * 64 + lane) * p.ranges_a + range;
    std::uint32_t cursor = kFill ? matrix_a[cell] : 0u;
    std::uint32_t count = 0;

    const int first = range * p.range_a;
    const int last = first + p.range_a < p.G ? first + p.range_a : p.G;
    for (int base = first; base < last; base += 64) {
        const int i = base + lane;
        std::uint32_t g = 0;
        std::uint64_t mask = 0;
        if (i < last) {
            g = by_depth[i];
            const TileRect rc = rects_by_depth[i];
            if (rc.x0 <= rc.x1) {
                const int x0 = (rc.x0 >> 3) - origin_x, x1 = (rc.x1 >> 3) - origin_x;
                const int y0 = (rc.y0 >> 3) - origin_y, y1 = (rc.y1 >> 3) - origin_y;
                mask = block_mask(x0 > 0 ? x0 : 0, x1 < 7 ? x1 : 7, y0 > 0 ? y0 : 0, y1 < 7 ? y1 : 7);
            }
        }
        std::uint32_t lo = static_cast<std::uint32_t>(mask), hi = static_cast<std::uint32_t>(mask >> 32);
        transpose_64x64(lo, hi, lane);  // now: which of the 64 Gaussians reach this lane's supertile
        const std::uint64_t mine = (static_cast<std::uint64_t>(hi) << 32) | lo;
        if constexpr (kFill) {
            cursor += write_runs(stage, mine, g, cursor, list_a, p.capacity_a, lane);
        } else {
            count += static_cast<std::uint32_t>(__builtin_popcountll(mine));
        }
    }
    if constexpr (!kFill) matrix_a[cell] = count;
}

// ---------------------------------------------------------------------------
// Between the levels: how many wavefronts every supertile's list needs at level B (at least one, so
// that every tile gets its range written), as a prefix over the supertiles, clamped to the grid that
// will be launched.  One block.  Also records the number of (supertile, Gaussian) pairs and whether
// they fit, and clears the tile ranges (tiles that no wavefront reaches keep an empty range).
__global__ void __launch_bounds__(256) plan_kernel(BinPlan p, const std::uint32_t* __restrict__ offsets_a,
                                                   std::uint32_t* __restrict__ first_wave, std::uint32_t* __restrict__ tile_ranges,
                                                   std::uint32_t* __restrict__ status, bool clear_depth_flag) {
    __shared__ std::uint32_t shared[256];
    __shared__ std::uint32_t carried;
    const unsigned t = threadIdx.x;
    for (std::size_t k = static_cast<std::size_t>(blockIdx.x) * 256 + t; k < static_cast<std::size_t>(p.tiles_x) * p.tiles_y * 2;
         k += static_cast<std::size_t>(gridDim.x) * 256)
        tile_ranges[k] = 0;
    if (blockIdx.x != 0) return;
    if (t == 0) carried = 0;
    __syncthreads();
    for (int base = 0; base < p.supers; base += 256) {
        const int s = base + static_cast<int>(t);
        std::uint32_t waves = 0;
        if (s < p.supers && super_coords(p, s).inside) {
            std::uint32_t begin = offsets_a[static_cast<std::size_t>(s) * p.ranges_a];
            std::uint32_t end = offsets_a[static_cast<std::size_t>(s + 1) * p.ranges_a];
            begin = begin < p.capacity_a ? begin : p.capacity_a;
            end = end < p.capacity_a ? end : p.capacity_a;
            waves = (end - begin + kBinRangeB - 1) / kBinRangeB;
            if (waves == 0) waves = 1;
        }
        shared[t] = waves;
        __syncthreads();
        for (unsigned step = 1; step < 256; step *= 2) {
            const std::uint32_t other = t >= step ? shared[t - step] : 0u;
            __syncthreads();
            shared[t] += other;
            __syncthreads();
        }
        const std::uint32_t exclusive = carried + shared[t] - waves;
        if (s < p.supers) first_wave[s] = exclusive < p.waves_b ? exclusive : p.waves_b;
        __syncthreads();
        if (t == 255) carried += shared[255];
        __syncthreads();
    }
    if (t == 0) {
        first_wave[p.supers] = carried < p.waves_b ? carried : p.waves_b;
        const std::uint32_t super_pairs = offsets_a[static_cast<std::size_t>(p.supers) * p.ranges_a];
        status[kStatusSuperPairs] = super_pairs;
        // this step's verdict starts here; the last kernel of the binning may still raise it
        const bool overflow = super_pairs > p.capacity_a || carried > p.waves_b;
        status[kStatusOverflow] = overflow ? 1u : 0u;
        // the sticky word keeps the largest room any step would have needed (never zero for a step that overflowed)
        if (overflow) atomicMax(status + kStatusOverflowSticky, super_pairs > 0 ? super_pairs : 1u);
        if (clear_depth_flag) status[kStatusDepthChanged] = 0;  // the projection of this step has set it, the host has its copy
    }
}

// ---------------------------------------------------------------------------
// Level B.  One wavefront per block: wavefront w serves entries [64 q, 64 q + 64) of the list of supertile s,
// where first_wave[s] <= w < first_wave[s + 1] and q = w - first_wave[s]; after the transpose, lane = tile of
// the supertile (row-major, 8 per row).  The counts of supertile s live at
// matrix_b[64 first_wave[s] + tile * waves_of_s + q]: scanned as one flat array, that order puts every
// tile's pieces next to each other and the tiles of a supertile one after the other, so the scanned
// value is the position in the final list.  Wavefronts beyond the last supertile clear their 64 cells
// and leave.
template <bool kFill>
__global__ void __launch_bounds__(64) tile_kernel(BinPlan p, const std::uint32_t* __restrict__ offsets_a,
                                                  const std::uint32_t* __restrict__ first_wave,
                                                  const std::uint32_t* __restrict__ list_a, const TileRect* __restrict__ rects,
                                                  std::uint32_t* __restrict__ matrix_b, std::uint32_t* __restrict__ list,
                                                  std::uint32_t* __restrict__ range_begin, std::uint32_t* __restrict__ range_end,
                                                  std::uint32_t* __restrict__ status) {
    __shared__ RunStage stage;
    const int lane = static_cast<int>(threadIdx.x);
    const std::uint32_t w = blockIdx.x;
    const std::uint32_t used = first_wave[p.supers];
    if (w >= used) {
        if constexpr (!kFill) matrix_b[static_cast<std::size_t>(w) * 64 + lane] = 0;
        return;
    }
    // the last supertile whose first wavefront is not after w
    int s = 0;
    for (int hi = p.supers; hi - s > 1;) {
        const int mid = (s + hi) / 2;
        if (first_wave[mid] <= w)
            s = mid;
        else
            hi = mid;
    }
    const std::uint32_t wave0 = first_wave[s], waves = first_wave[s + 1] - wave0, q = w - wave0;
    std::uint32_t begin = offsets_a[static_cast<std::size_t>(s) * p.ranges_a];
    std::uint32_t end = offsets_a[static_cast<std::size_t>(s + 1) * p.ranges_a];
    begin = begin < p.capacity_a ? begin : p.capacity_a;
    end = end < p.capacity_a ? end : p.capacity_a;
    const std::uint32_t i = begin + q * kBinRangeB + static_cast<std::uint32_t>(lane);

    const SuperCoords where = super_coords(p, s);
    const int base_x = where.x * 8, base_y = where.y * 8;
    std::uint32_t g = 0, mask_lo = 0, mask_hi = 0;
    if (i < end) {
        g = list_a[i];
        const TileRect rc = rects[g];
        const std::uint64_t mask = block_mask(rc.x0 - base_x > 0 ? rc.x0 - base_x : 0, rc.x1 - base_x < 7 ? rc.x1 - base_x : 7,
                                              rc.y0 - base_y > 0 ? rc.y0 - base_y : 0, rc.y1 - base_y < 7 ? rc.y1 - base_y : 7);
        mask_lo = static_cast<std::uint32_t>(mask);
        mask_hi = static_cast<std::uint32_t>(mask >> 32);
    }
    transpose_64x64(mask_lo, mask_hi, lane);  // now: which of the 64 entries cover this lane's tile
    const int tx = base_x + (lane & 7), ty = base_y + (lane >> 3);
    const bool owner = tx < p.tiles_x && ty < p.tiles_y;
    std::uint64_t mine = owner ? (static_cast<std::uint64_t>(mask_hi) << 32) | mask_lo : 0;
    const std::size_t cell = static_cast<std::size_t>(wave0) * 64 + static_cast<std::size_t>(lane) * waves + q;

    if constexpr (!kFill) {
        matrix_b[cell] = static_cast<std::uint32_t>(__builtin_popcountll(mine));
    } else {
        const std::uint32_t from = matrix_b[cell];
        write_runs(stage, mine, g, from, list, p.capacity, lane);
        if (q == 0 && owner) {
            // this tile's list: from the first cell of the tile to the first cell of the next one
            const std::size_t next_cell = static_cast<std::size_t>(wave0) * 64 + static_cast<std::size_t>(lane + 1) * waves;
            const std::uint32_t to = matrix_b[next_cell];
            const int tile = ty * p.tiles_x + tx;
            range_begin[tile] = from < p.capacity ? from : p.capacity;
            range_end[tile] = to < p.capacity ? to : p.capacity;
        }
        if (w == 0 && lane == 0) {
            const std::uint32_t pairs = matrix_b[static_cast<std::size_t>(p.waves_b) * 64];  // the scan's total
            status[kStatusPairs] = pairs;
            if (pairs > p.capacity) {
                status[kStatusOverflow] = 1;
                atomicMax(status + kStatusOverflowSticky, pairs);
            }
        }
    }
}

}  // namespace

BinPlan make_bin_plan(int G, int tiles_x, int tiles_y, std::uint32_t capacity, std::uint32_t capacity_a) {
    BinPlan p{};
    p.G = G;
    p.tiles_x = tiles_x;
    p.tiles_y = tiles_y;
    p.super_x = (tiles_x + 7) / 8;
    p.super_y = (tiles_y + 7) / 8;
    p.group_x = (p.super_x + 7) / 8;
    p.groups = p.group_x * ((p.super_y + 7) / 8);
    p.supers = p.groups * 64;  // numbered group by group; those beyond the image stay empty
    // about 8192 wavefronts at level A (short ones: a wavefront's chunks of 64 Gaussians are a chain of memory
    // latencies), and never less than 64 Gaussians per wavefront
    const long long per_wave = (static_cast<long long>(G) * p.groups + 8191) / 8192;
    p.range_a = static_cast<int>(((per_wave > 64 ? per_wave : 64) + 63) / 64 * 64);
    p.ranges_a = (G + p.range_a - 1) / p.range_a;
    p.capacity = capacity;
    p.capacity_a = capacity_a < capacity ? capacity_a : capacity;
    p.waves_b = static_cast<std::uint32_t>((static_cast<std::uint64_t>(p.capacity_a) + kBinRangeB - 1) / kBinRangeB) +
                static_cast<std::uint32_t>(p.supers);
    return p;
}

std::size_t bin_matrix_a_words(const BinPlan& p) { return static_cast<std::size_t>(p.supers) * p.ranges_a + 1; }
std::size_t bin_matrix_b_words(const BinPlan& p) { return static_cast<std::size_t>(p.waves_b) * 64 + 1; }
std::size_t bin_scan_state_words(const BinPlan& p) {
    const std::size_t longest = bin_matrix_a_words(p) > bin_matrix_b_words(p) ? bin_matrix_a_words(p) : bin_matrix_b_words(p);
    return (longest + kScanTile - 1) / kScanTile + 1;
}

namespace {

int launch_scan(hipStream_t s, std::uint32_t* data, std::size_t n, const BinScratch& scratch) {
    XAD_REQUIRE(n > 0 && n < (std::size_t(1) << 32) - 2 * kScanTile, "splat binning: %zu counts do not fit the 32-bit scan", n);
    const unsigned blocks = static_cast<unsigned>((n + kScanTile - 1) / kScanTile);
    hipLaunchKernelGGL(scan_kernel, dim3(blocks), dim3(kScanBlock), 0, s, data, static_cast<std::uint32_t>(n), scratch.scan_state,
                       scratch.scan_control);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

}  // namespace

int launch_binning(hipStream_t s, const BinPlan& p, const std::uint32_t* by_depth, const TileRect* rects_by_depth,
                   const TileRect* rects, BinScratch& scratch,
                   std::uint32_t* list, std::uint32_t* range_begin, std::uint32_t* range_end, std::uint32_t* status,
                   bool clear_depth_flag) {
    XAD_REQUIRE(p.G > 0 && p.supers > 0 && p.ranges_a > 0 && p.capacity > 0, "splat binning: empty plan");
    XAD_REQUIRE(range_end == range_begin + static_cast<std::size_t>(p.tiles_x) * p.tiles_y,
                "splat binning: the two halves of the tile ranges must be adjacent");
    const unsigned waves_a = static_cast<unsigned>(p.ranges_a) * static_cast<unsigned>(p.groups);
    hipLaunchKernelGGL(super_kernel<false>, dim3(waves_a), dim3(64), 0, s, p, by_depth, rects_by_depth, scratch.matrix_a,
                       scratch.list_a);
    XAD_HIP_TRY(hipGetLastError());
    if (int st = launch_scan(s, scratch.matrix_a, bin_matrix_a_words(p) - 1, scratch)) return st;
    const unsigned plan_blocks = static_cast<unsigned>((static_cast<std::size_t>(p.tiles_x) * p.tiles_y * 2 + 4095) / 4096);
    hipLaunchKernelGGL(plan_kernel, dim3(plan_blocks < 1 ? 1 : (plan_blocks > 512 ? 512 : plan_blocks)), dim3(256), 0, s, p,
                       scratch.matrix_a, scratch.first_wave, range_begin, status, clear_depth_flag);
    XAD_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(super_kernel<true>, dim3(waves_a), dim3(64), 0, s, p, by_depth, rects_by_depth, scratch.matrix_a,
                       scratch.list_a);
    XAD_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(tile_kernel<false>, dim3(p.waves_b), dim3(64), 0, s, p, scratch.matrix_a, scratch.first_wave, scratch.list_a,
                       rects, scratch.matrix_b, list, range_begin, range_end, status);
    XAD_HIP_TRY(hipGetLastError());
    if (int st = launch_scan(s, scratch.matrix_b, bin_matrix_b_words(p) - 1, scratch)) return st;
    hipLaunchKernelGGL(tile_kernel<true>, dim3(p.waves_b), dim3(64), 0, s, p, scratch.matrix_a, scratch.first_wave, scratch.list_a,
                       rects, scratch.matrix_b, list, range_begin, range_end, status);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

}  // namespace xad_splat
