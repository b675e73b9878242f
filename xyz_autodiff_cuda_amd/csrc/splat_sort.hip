// The depth order of the Gaussians: a stable least-significant-digit radix sort of (depth bits, index),
// written for this size of problem (10^4 to 10^6 keys of 32 bits), where the time is launches and
// round trips to memory, not bandwidth.  Five launches in all (one, by one block, up to 4096 keys: see
// sort_small_kernel), no library primitive, no host read-back:
//
//   prepare   one lane per Gaussian: the order-preserving bits of its depth, a copy of the depth (what
//             the order was computed from), and the counts of the three lower 8-bit digits (a histogram
//             does not depend on the order of the keys), summed per block in LDS and added to three
//             global histograms.
//   pass 0-3  one launch per digit.  A block takes a ticket, which is its tile of 4096 keys; each of
//             its sixteen wavefronts ranks 4 rounds of 64 keys among the equal digits before them
//             (the lanes with the same digit are found with one ballot per digit bit; a per-wavefront
//             counter table in LDS carries the counts from round to round), the tables are scanned
//             per digit, and lane d of the block finds, for digit d, how many such keys the tiles
//             before this one hold: every tile publishes its own count per digit first and then looks
//             back over its predecessors' words, 64 at a time, until it meets one that already
//             holds a prefix (a chained scan with decoupled look-back, 256 of them side by side).  A
//             tile only waits for tiles with earlier tickets, which are running.  Position = keys of
//             smaller digits (exclusive scan of the global histogram) + equal digits in earlier tiles
//             + in earlier wavefronts of the tile + in earlier rounds and lanes of the wavefront.
//             Every key is written once per pass; the last pass writes the index and the inverse
//             permutation instead of the key.  Pass 2 counts the top digit of its keys into the
//             last pass's histogram.
//
// Nothing is cleared between sorts by a launch of its own: the four histograms and the four ticket
// counters form a ring in which pass p clears what pass p - 1 used (and pass 0 what pass 3 of the
// sort before left behind: that is why the top digit is counted late, into a histogram pass 0 has
// cleared), and the prepare launch clears the tiles' state words.
//
// Sizes: a pass is a chain of round trips to memory (ticket, keys, look-back) whatever the size of a
// tile; the look-back is as long as there are tiles; and the rounds of a wavefront are serial.  So the
// tiles are large (4096 keys: 49 of them at 2 x 10^5 keys, three looks of 16 words) and wide rather than
// deep (sixteen wavefronts of four rounds).  Measured on MI355X, the whole sort at 2 x 10^5 keys, as the
// difference between a splatting step that orders and one that does not: 256 lanes x 8 rounds with a
// look-back of one word at a time 0.32 ms; the same, sixteen words at a time 0.10 ms; 1024 lanes x 16
// rounds 0.20 ms (one compute unit does the work of four); 1024 x 8 0.107; 512 x 8 0.070; 1024 x 4 with
// looks of 8, 16, 24, 32 words 0.071, 0.059-0.064, 0.068, 0.076 ms (more words per look is more code and
// more registers: with 64 and a wait loop per word a pass spent 20 us fetching instructions); tiles
// taken by block index instead of by ticket 0.078 (blocks do not start in index order, so more of
// them wait).  At 10^4 keys (three tiles) 0.05 ms: five launches of about 10 us.  The five steps in one
// launch, with a barrier across the (resident) blocks and agent-scope fences between them: 0.23 ms at
// 2 x 10^5 keys, 0.085 at 10^4 -- the release and acquire of plain data across the XCDs' L2 caches
// (write back, invalidate) cost far more than the launch boundaries they replace.
//
// Equal depths keep index order (every pass is stable and the first one takes the keys in index
// order).  Order of the keys: the total order of the bit patterns in sign-magnitude reading, with
// -0.0 and +0.0 taken as the same depth; a NaN sorts by its bits, before everything when its sign bit
// is set and after everything when it is not.
//
// No counterpart in xyz-autodiff-cuda: its renderer visits every Gaussian at every pixel in index
// order (examples/mini-gaussian-splatting/gaussian_splatting_kernel.cu:33-62).
#include <xyz_autodiff/accumulate.cuh>

#include "common.cuh"
#include "splat_launch.cuh"

namespace xad_splat {

namespace {

using xyz_autodiff::accumulate::wave::ballot;

constexpr unsigned kSortBlock = 1024;                          // sixteen wavefronts
constexpr unsigned kSortWaves = kSortBlock / 64;
constexpr unsigned kSortRounds = 4;                            // keys per lane
constexpr unsigned kSortWaveKeys = 64 * kSortRounds;           // a wavefront's share of a tile, contiguous
constexpr unsigned kSortTile = kSortBlock * kSortRounds;       // 4096 keys per block
constexpr int kLookBack = 16;                                  // predecessors whose words are requested together
constexpr unsigned kDigits = 256;
constexpr int kPasses = 4;

// State word of (pass, tile, digit): two flag bits and a 30-bit count.
constexpr std::uint32_t kFlagAggregate = 1u << 30;  // the tile's own count of the digit
constexpr std::uint32_t kFlagPrefix = 2u << 30;     // the count of the digit in this tile and all tiles before it
constexpr std::uint32_t kCountMask = (1u << 30) - 1;

// Layout of the workspace, in 32-bit words.
//   [0, 1024)                 the four global histograms, one per digit position
//   [1024, 1024 + 4)          the four ticket counters, one per pass
//   1024 + 8                  number of blocks that gave up waiting for a predecessor (never, unless the device is
//                             shared with something that keeps a block with an earlier ticket from running)
//   [1088, ...)               state words, [pass][tile][digit]
constexpr std::size_t kHistWords = kPasses * kDigits;
constexpr std::size_t kTicketAt = kHistWords;
constexpr std::size_t kGaveUpAt = kHistWords + 8;
constexpr std::size_t kStateAt = kHistWords + 64;
// A wait for a predecessor's word ends after this many looks at it (each a round trip to L2, about a
// microsecond): the block then writes nothing and reports itself, so that no launch can wait forever.
constexpr std::uint32_t kSpinLimit = 1u << 21;

// Adds one to table[digit] for every valid lane, with one LDS atomic per distinct digit of the wavefront
// instead of one per lane: lanes that share a digit are found with one ballot per digit bit and the first of
// them adds their number.  (An LDS atomic costs about two cycles per lane that shares its address; the high
// digits of depths share nearly all of theirs.)
__device__ __forceinline__ void count_digit(std::uint32_t* table, std::uint32_t digit, bool valid, std::uint64_t below) {
    std::uint64_t same = ballot(valid);
#pragma unroll
    for (unsigned bit = 0; bit < 8; ++bit) {
        const std::uint64_t set = ballot(((digit >> bit) & 1u) != 0);
        same &= ((digit >> bit) & 1u) ? set : ~set;
    }
    if (valid && (same & below) == 0) atomicAdd(table + digit, static_cast<std::uint32_t>(__builtin_popcountll(same)));
}

// Order-preserving map from float to unsigned; the two zeros map to one key.
__device__ __forceinline__ std::uint32_t depth_key(float f) {
    std::uint32_t u = __builtin_bit_cast(std::uint32_t, f);
    if (u == 0x80000000u) u = 0u;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// The keys, a copy of the depths, and the counts of the keys' three lower digits.  Tiles as large as the
// passes': every block adds its counts to the same 768 words, and atomics on one address are taken one after
// the other (with 256 keys per block this launch took 10 us at 2 x 10^5 keys for that reason alone).
__global__ void __launch_bounds__(kSortBlock) sort_prepare_kernel(int G, const float* __restrict__ depth,
                                                                  std::uint32_t* __restrict__ keys,
                                                                  float* __restrict__ ordered_depth,
                                                                  std::uint32_t* __restrict__ work, std::size_t state_words) {
    __shared__ std::uint32_t hist[kPasses - 1][kDigits];
    const unsigned t = threadIdx.x;
    if (t < (kPasses - 1) * kDigits) (&hist[0][0])[t] = 0;
    // every tile starts every pass with empty state words
    for (std::size_t i = static_cast<std::size_t>(blockIdx.x) * kSortBlock + t; i < state_words;
         i += static_cast<std::size_t>(gridDim.x) * kSortBlock)
        work[kStateAt + i] = 0;
    __syncthreads();
    const std::size_t base = static_cast<std::size_t>(blockIdx.x) * kSortTile;
    const std::uint64_t below = (std::uint64_t(1) << (t & 63u)) - 1;
#pragma unroll
    for (unsigned i = 0; i < kSortRounds; ++i) {
        const std::size_t g = base + i * kSortBlock + t;
        const bool valid = g < static_cast<std::size_t>(G);
        std::uint32_t key = 0;
        if (valid) {
            const float d = depth[g];
            key = depth_key(d);
            keys[g] = key;
            ordered_depth[g] = d;
        }
#pragma unroll
        for (int p = 0; p < kPasses - 1; ++p) count_digit(hist[p], (key >> (8 * p)) & 255u, valid, below);
    }
    __syncthreads();
    if (t < (kPasses - 1) * kDigits && (&hist[0][0])[t] != 0) atomicAdd(work + t, (&hist[0][0])[t]);
}

// One digit.  kFirst: the values are the keys' own indices (nothing to read); kLast: the keys are not
// written any more, the values go to `values_out` (the order) and every value's position to `rank`;
// kCountNext: the next digit of the keys is counted into the next pass's histogram.
template <bool kFirst, bool kLast, bool kCountNext>
__global__ void __launch_bounds__(kSortBlock) sort_pass_kernel(int G, int pass, const std::uint32_t* __restrict__ keys_in,
                                                               const std::uint32_t* __restrict__ values_in,
                                                               std::uint32_t* __restrict__ keys_out,
                                                               std::uint32_t* __restrict__ values_out,
                                                               std::uint32_t* __restrict__ rank,
                                                               std::uint32_t* __restrict__ work) {
    __shared__ std::uint32_t count[kSortWaves][kDigits];  // per wavefront: running counts, then offsets inside the tile
    __shared__ std::uint32_t digit_base[kDigits];         // where the tile's keys of a digit begin in the output
    __shared__ std::uint32_t next_digit[kDigits];         // the tile's counts of the digit the next pass sorts by
    __shared__ std::uint32_t wave_sum[kDigits / 64];
    __shared__ std::uint32_t tile_index, gave_up;
    const unsigned t = threadIdx.x, lane = t & 63u, w = t >> 6;
    if (t == 0) {
        tile_index = atomicAdd(work + kTicketAt + pass, 1u);
        gave_up = 0;
    }
#pragma unroll
    for (unsigned k = 0; k < kSortWaves * kDigits / kSortBlock; ++k) (&count[0][0])[k * kSortBlock + t] = 0;
    if (t < kDigits) next_digit[t] = 0;
    __syncthreads();
    const std::uint32_t b = tile_index;
    const std::size_t tiles = gridDim.x;
    const unsigned shift = 8u * static_cast<unsigned>(pass);
    // the ring: what the pass before this one used is cleared here (by pass 0: what pass 3 of the sort before used)
    if (b == 0 && t < kDigits) {
        const int behind = (pass + kPasses - 1) % kPasses;
        // (stores that go where the other blocks' atomics go, not through a cached line next to words in use)
        __hip_atomic_store(work + behind * kDigits + t, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (t == 0) __hip_atomic_store(work + kTicketAt + behind, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // a wavefront's keys are contiguous; in round i lane l holds key i * 64 + l of them
    const std::size_t chunk = static_cast<std::size_t>(b) * kSortTile + static_cast<std::size_t>(w) * kSortWaveKeys;
    std::uint32_t key[kSortRounds], value[kSortRounds], place[kSortRounds];
#pragma unroll
    for (unsigned i = 0; i < kSortRounds; ++i) {
        const std::size_t at = chunk + i * 64 + lane;
        const bool valid = at < static_cast<std::size_t>(G);
        key[i] = valid ? keys_in[at] : 0u;
        value[i] = kFirst ? static_cast<std::uint32_t>(at) : (valid ? values_in[at] : 0u);
    }
    const std::uint64_t below = (std::uint64_t(1) << lane) - 1;
#pragma unroll
    for (unsigned i = 0; i < kSortRounds; ++i) {
        const bool valid = chunk + i * 64 + lane < static_cast<std::size_t>(G);
        const std::uint32_t digit = (key[i] >> shift) & 255u;
        std::uint64_t same = ballot(valid);
#pragma unroll
        for (unsigned bit = 0; bit < 8; ++bit) {
            const std::uint64_t set = ballot(((digit >> bit) & 1u) != 0);
            same &= ((digit >> bit) & 1u) ? set : ~set;
        }
        // lanes of one instruction that share a digit read the same counter; the first of them moves it on
        // (volatile: another lane's store of the round before must be read, not a value kept in a register)
        volatile std::uint32_t* counter = &count[w][digit];
        const std::uint32_t before = *counter;
        place[i] = before + static_cast<std::uint32_t>(__builtin_popcountll(same & below));
        if (valid && (same & below) == 0) *counter = before + static_cast<std::uint32_t>(__builtin_popcountll(same));
        if constexpr (kCountNext) count_digit(next_digit, (key[i] >> ((shift + 8) & 31u)) & 255u, valid, below);
    }
    __syncthreads();

    // lane d of the block (the first 256): digit d.  Offsets of the wavefronts inside the tile, the tile's count,
    // the look-back, and the digit's place among all keys.
    std::uint32_t earlier_tiles = 0, inclusive = 0, total = 0;
    if (t < kDigits) {
        std::uint32_t in_tile = 0;
#pragma unroll
        for (unsigned k = 0; k < kSortWaves; ++k) {
            const std::uint32_t c = count[k][t];
            count[k][t] = in_tile;
            in_tile += c;
        }
        total = work[pass * kDigits + t];  // asked for here, needed after the look-back
        if constexpr (kCountNext)
            if (next_digit[t] != 0) atomicAdd(work + (pass + 1) * kDigits + t, next_digit[t]);
        std::uint32_t* state = work + kStateAt + static_cast<std::size_t>(pass) * tiles * kDigits;
        std::uint32_t* mine = state + static_cast<std::size_t>(b) * kDigits + t;
        if (b > 0) {
            __hip_atomic_store(mine, kFlagAggregate | in_tile, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // The words of kLookBack predecessors are requested together (one round trip to L2 for all of them,
            // not one each: with all tiles running at once nearly every word is there at the first look) and
            // summed, nearest first, up to and including the first that holds a prefix, without a branch per
            // word.  If one of them was not there yet, a small loop waits for each in turn and they are
            // requested again.  (Kept small on purpose: unrolled with a wait loop per word this part alone
            // was 20 us of instruction fetch per launch.)
            bool open = true;
            for (std::int32_t nearest = static_cast<std::int32_t>(b) - 1; nearest >= 0 && open; nearest -= kLookBack) {
                // word k of this look belongs to tile nearest - k: a constant distance below `first`
                const std::uint32_t* first = state + (static_cast<std::uint32_t>(nearest) * kDigits + t);
                std::uint32_t word[kLookBack];
                bool missing;
                do {
                    missing = false;
#pragma unroll
                    for (int k = 0; k < kLookBack; ++k)
                        word[k] = k <= nearest ? __hip_atomic_load(first - k * static_cast<int>(kDigits), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                               : kFlagPrefix;  // before tile 0: a prefix of nothing
                    std::uint32_t all_flags = ~0u;
#pragma unroll
                    for (int k = 0; k < kLookBack; ++k) all_flags &= (word[k] >> 30) != 0 ? ~0u : 0u;
                    missing = all_flags == 0;
                    if (missing) {
#pragma unroll 1
                        for (int k = 0; k < kLookBack && k <= nearest; ++k) {
                            std::uint32_t looks = 0;  // that tile holds an earlier ticket: it is running or done
                            while ((__hip_atomic_load(first - k * static_cast<int>(kDigits), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 30) == 0 &&
                                   ++looks < kSpinLimit) {
                            }
                            if (looks >= kSpinLimit) {
                                gave_up = 1;
                                missing = false;
                                open = false;
                            }
                        }
                    }
                } while (missing);
#pragma unroll
                for (int k = 0; k < kLookBack; ++k) {
                    earlier_tiles += open ? (word[k] & kCountMask) : 0u;
                    open = open && (word[k] & kFlagPrefix) == 0;
                }
            }
        }
        __hip_atomic_store(mine, kFlagPrefix | (earlier_tiles + in_tile), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

        // keys of smaller digits, anywhere: exclusive scan of the global histogram of this digit position
        inclusive = total;
#pragma unroll
        for (unsigned step = 1; step < 64; step *= 2) {
            const std::uint32_t other = __shfl_up(inclusive, step, 64);
            if (lane >= step) inclusive += other;
        }
        if (lane == 63) wave_sum[w] = inclusive;
    }
    __syncthreads();
    if (t < kDigits) {
        std::uint32_t smaller_digits = inclusive - total;
#pragma unroll
        for (unsigned k = 0; k < kDigits / 64; ++k) smaller_digits += k < w ? wave_sum[k] : 0u;
        digit_base[t] = smaller_digits + earlier_tiles;
    }
    __syncthreads();

    if (gave_up != 0) {
        if (t == 0) atomicAdd(work + kGaveUpAt, 1u);
        return;
    }
#pragma unroll
    for (unsigned i = 0; i < kSortRounds; ++i) {
        if (chunk + i * 64 + lane < static_cast<std::size_t>(G)) {
            const std::uint32_t digit = (key[i] >> shift) & 255u;
            const std::uint32_t at = digit_base[digit] + count[w][digit] + place[i];
            if (at < static_cast<std::uint32_t>(G)) {  // always, unless an earlier tile gave up
                if constexpr (!kLast) keys_out[at] = key[i];
                values_out[at] = value[i];
                if constexpr (kLast) rank[value[i]] = at;
            }
        }
    }
}

// The whole sort in one block, for scenes of up to kSmallSortKeys Gaussians: no tickets, no look-back, no
// histograms in memory, one launch instead of five (which cost about 10 us each whatever the size).  Every
// lane keeps kRounds keys in registers; a pass ranks them as above, scans the 256 digit counts of the block,
// writes every key and value to its place in `keys` / `values` (global scratch: the block's own stores, read
// back by the same block after a barrier) and takes its next keys from there; the last pass writes the order
// and its inverse instead.  Measured (kernel time): 14.6 us with two keys per lane, 26.5 with four, 51 with
// eight, 74 with twelve, against 52 us for the five launches up to 12 288 keys: a round of ranking costs 1.5 us
// per pass wherever it runs, and the tiles of the five launches run theirs side by side on different compute
// units.  So one block sorts alone up to four keys per lane.
constexpr unsigned kSmallSortMaxRounds = 4;
constexpr unsigned kSmallSortKeys = kSortBlock * kSmallSortMaxRounds;  // 4096

template <unsigned kRounds>
__global__ void __launch_bounds__(kSortBlock) sort_small_kernel(int G, const float* __restrict__ depth, std::uint32_t* keys,
                                                                std::uint32_t* values, std::uint32_t* __restrict__ by_depth,
                                                                std::uint32_t* __restrict__ rank,
                                                                float* __restrict__ ordered_depth) {
    __shared__ std::uint32_t count[kSortWaves][kDigits];
    __shared__ std::uint32_t digit_base[kDigits];
    __shared__ std::uint32_t wave_sum[kDigits / 64];
    const unsigned t = threadIdx.x, lane = t & 63u, w = t >> 6;
    const unsigned chunk = w * 64u * kRounds;  // a wavefront's keys are contiguous; in round i lane l holds key i * 64 + l of them
    const unsigned n = static_cast<unsigned>(G);
    const std::uint64_t below = (std::uint64_t(1) << lane) - 1;
    std::uint32_t key[kRounds], value[kRounds], place[kRounds];
#pragma unroll
    for (unsigned i = 0; i < kRounds; ++i) {
        const unsigned at = chunk + i * 64 + lane;
        key[i] = 0u;
        value[i] = at;
        if (at < n) {
            const float d = depth[at];
            key[i] = depth_key(d);
            ordered_depth[at] = d;
        }
    }
#pragma unroll 1
    for (unsigned pass = 0; pass < static_cast<unsigned>(kPasses); ++pass) {
        const unsigned shift = 8u * pass;
#pragma unroll
        for (unsigned k = 0; k < kSortWaves * kDigits / kSortBlock; ++k) (&count[0][0])[k * kSortBlock + t] = 0;
        __syncthreads();
#pragma unroll
        for (unsigned i = 0; i < kRounds; ++i) {
            const bool valid = chunk + i * 64 + lane < n;
            const std::uint32_t digit = (key[i] >> shift) & 255u;
            std::uint64_t same = ballot(valid);
#pragma unroll
            for (unsigned bit = 0; bit < 8; ++bit) {
                const std::uint64_t set = ballot(((digit >> bit) & 1u) != 0);
                same &= ((digit >> bit) & 1u) ? set : ~set;
            }
            volatile std::uint32_t* counter = &count[w][digit];
            const std::uint32_t before = *counter;
            place[i] = before + static_cast<std::uint32_t>(__builtin_popcountll(same & below));
            if (valid && (same & below) == 0) *counter = before + static_cast<std::uint32_t>(__builtin_popcountll(same));
        }
        __syncthreads();
        // lane d of the block (the first 256): digit d.  Offsets of the wavefronts, then of the digits.
        std::uint32_t inclusive = 0, total = 0;
        if (t < kDigits) {
#pragma unroll
            for (unsigned k = 0; k < kSortWaves; ++k) {
                const std::uint32_t c = count[k][t];
                count[k][t] = total;
                total += c;
            }
            inclusive = total;
#pragma unroll
            for (unsigned step = 1; step < 64; step *= 2) {
                const std::uint32_t other = __shfl_up(inclusive, step, 64);
                if (lane >= step) inclusive += other;
            }
            if (lane == 63) wave_sum[w] = inclusive;
        }
        __syncthreads();
        if (t < kDigits) {
            std::uint32_t smaller_digits = inclusive - total;
#pragma unroll
            for (unsigned k = 0; k < kDigits / 64; ++k) smaller_digits += k < w ? wave_sum[k] : 0u;
            digit_base[t] = smaller_digits;
        }
        __syncthreads();
        const bool last = pass + 1 == static_cast<unsigned>(kPasses);
#pragma unroll
        for (unsigned i = 0; i < kRounds; ++i) {
            if (chunk + i * 64 + lane < n) {
                const std::uint32_t digit = (key[i] >> shift) & 255u;
                const std::uint32_t at = digit_base[digit] + count[w][digit] + place[i];
                if (at < n) {  // always: the places of n keys are a permutation of [0, n)
                    if (last) {
                        by_depth[at] = value[i];
                        rank[value[i]] = at;
                    } else {
                        keys[at] = key[i];
                        values[at] = value[i];
                    }
                }
            }
        }
        if (last) break;
        __syncthreads();  // the block's stores are visible to the block
#pragma unroll
        for (unsigned i = 0; i < kRounds; ++i) {
            const unsigned at = chunk + i * 64 + lane;
            if (at < n) {
                key[i] = keys[at];
                value[i] = values[at];
            }
        }
    }
}

template <unsigned kRounds>
void launch_small_sort(hipStream_t s, int G, const float* depth, std::uint32_t* keys, std::uint32_t* values,
                       std::uint32_t* by_depth, std::uint32_t* rank, float* ordered_depth) {
    hipLaunchKernelGGL(sort_small_kernel<kRounds>, dim3(1), dim3(kSortBlock), 0, s, G, depth, keys, values, by_depth, rank,
                       ordered_depth);
}

unsigned sort_tiles(int G) { return static_cast<unsigned>((static_cast<std::size_t>(G) + kSortTile - 1) / kSortTile); }

}  // namespace

std::size_t depth_sort_gave_up_offset() { return kGaveUpAt * sizeof(std::uint32_t); }

std::size_t depth_sort_temp_bytes(int G) {
    return (kStateAt + static_cast<std::size_t>(kPasses) * sort_tiles(G) * kDigits) * sizeof(std::uint32_t);
}

int sort_by_depth(hipStream_t s, void* temp, std::size_t temp_bytes, const float* depth, std::uint32_t* keys_a,
                  std::uint32_t* keys_b, std::uint32_t* values_a, std::uint32_t* by_depth, std::uint32_t* rank,
                  float* ordered_depth, int G) {
    XAD_REQUIRE(G > 0 && static_cast<std::uint32_t>(G) <= kCountMask, "depth sort: %d keys do not fit the 30-bit counts", G);
    XAD_REQUIRE(temp && temp_bytes >= depth_sort_temp_bytes(G), "depth sort: workspace of %zu bytes, %zu needed", temp_bytes,
                depth_sort_temp_bytes(G));
    if (static_cast<unsigned>(G) <= kSmallSortKeys) {
        const unsigned rounds = (static_cast<unsigned>(G) + kSortBlock - 1) / kSortBlock;
        if (rounds <= 2)
            launch_small_sort<2>(s, G, depth, keys_a, values_a, by_depth, rank, ordered_depth);
        else
            launch_small_sort<kSmallSortMaxRounds>(s, G, depth, keys_a, values_a, by_depth, rank, ordered_depth);
        XAD_HIP_TRY(hipGetLastError());
        return XAD_OK;
    }
    std::uint32_t* work = static_cast<std::uint32_t*>(temp);
    const dim3 grid(sort_tiles(G)), block(kSortBlock);
    const std::size_t state_words = static_cast<std::size_t>(kPasses) * sort_tiles(G) * kDigits;
    hipLaunchKernelGGL(sort_prepare_kernel, grid, block, 0, s, G, depth, keys_a, ordered_depth, work, state_words);
    XAD_HIP_TRY(hipGetLastError());
    // keys a -> b -> a -> b; values (index) -> values_a -> by_depth -> values_a -> by_depth
    hipLaunchKernelGGL((sort_pass_kernel<true, false, false>), grid, block, 0, s, G, 0, keys_a, nullptr, keys_b, values_a, nullptr, work);
    XAD_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL((sort_pass_kernel<false, false, false>), grid, block, 0, s, G, 1, keys_b, values_a, keys_a, by_depth, nullptr, work);
    XAD_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL((sort_pass_kernel<false, false, true>), grid, block, 0, s, G, 2, keys_a, by_depth, keys_b, values_a, nullptr, work);
    XAD_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL((sort_pass_kernel<false, true, false>), grid, block, 0, s, G, 3, keys_b, values_a, nullptr, by_depth, rank, work);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

}  // namespace xad_splat

extern "C" int xad_depth_order_f32(std::size_t n, const float* depth, std::uint32_t* order, std::uint32_t* rank, void* stream) {
    const char* who = "xad_depth_order_f32";
    if (n == 0) return XAD_OK;
    XAD_REQUIRE(depth && order && rank, "%s: null array", who);
    XAD_REQUIRE(n < (std::size_t(1) << 30), "%s: at most 2^30 - 1 depths, got %zu", who, n);
    const int G = static_cast<int>(n);
    const std::size_t temp_bytes = xad_splat::depth_sort_temp_bytes(G);
    const std::size_t array_bytes = (n * sizeof(std::uint32_t) + 255) / 256 * 256;
    char* base = nullptr;
    XAD_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&base), 4 * array_bytes + temp_bytes));
    hipStream_t s = xad::as_stream(stream);
    int st = XAD_OK;
    if (hipMemsetAsync(base + 4 * array_bytes, 0, temp_bytes, s) != hipSuccess) st = xad::fail(XAD_ERR_HIP, "%s: hipMemsetAsync failed", who);
    if (st == XAD_OK)
        st = xad_splat::sort_by_depth(s, base + 4 * array_bytes, temp_bytes, depth, reinterpret_cast<std::uint32_t*>(base),
                                      reinterpret_cast<std::uint32_t*>(base + array_bytes),
                                      reinterpret_cast<std::uint32_t*>(base + 2 * array_bytes), order, rank,
                                      reinterpret_cast<float*>(base + 3 * array_bytes), G);
    // the workspace is released here, so the call waits for the stream
    std::uint32_t gave_up = 0;
    hipError_t waited = hipStreamSynchronize(s);
    if (waited == hipSuccess) waited = hipMemcpy(&gave_up, base + 4 * array_bytes + xad_splat::depth_sort_gave_up_offset(), sizeof gave_up, hipMemcpyDeviceToHost);
    (void)hipFree(base);
    if (st == XAD_OK && waited != hipSuccess) st = xad::fail(XAD_ERR_HIP, "%s: %s", who, hipGetErrorString(waited));
    if (st == XAD_OK && gave_up != 0) st = xad::fail(XAD_ERR_HIP, "%s: %u blocks gave up waiting for a block with an earlier ticket", who, gave_up);
    return st;
}
