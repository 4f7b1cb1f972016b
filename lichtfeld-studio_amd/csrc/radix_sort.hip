// radix_sort.hip - stable LSD radix sort of (int64 key, int32 value) pairs on key bits [begin_bit, end_bit)
// (gsplat/IntersectTile.cu:290-328 calls cub::DeviceRadixSort::SortPairs with a DoubleBuffer), and the same sort
// for (uint16 tile index, int32 value) pairs.
//
// 8-bit digits.  A large sort is one launch per pass behind two small ones: a fill of the bookkeeping words, one
// read of the keys that counts the digits of every pass, then the chained passes below (2 + P launches; the 45-bit
// keys of the reference's sort: 8 instead of 18).  Smaller sorts, the entry point that brings no workspace and more
// than 2^30 pairs take three launches per pass: block histograms -> one scan block per digit turns its row of the
// digit-major table into running counts and leaves the digit's total -> stable scatter (every block adds the
// exclusive scan of the 256 totals itself; no atomics between blocks, nothing to zero).  A
// block owns a tile of 256 x ITEMS consecutive pairs; inside the block each 64-lane wave owns a quarter of them
// and ranks them 64 at a time with wave-wide match masks (one 64-bit mask per digit in LDS, set by atomic OR), so
// the order (wave, round, lane) equals the input order and the sort is stable.  The ranked pairs are first placed in LDS in digit order and then
// written out by consecutive lanes, so that every (tile, digit) run leaves the block as whole cache lines.
#include <algorithm>
#include <mutex>
#include <vector>

#include "gsx_common.h"
#include "gsx_lookback.h"

namespace gsx {

static constexpr uint32_t kRadixBits = 8;
static constexpr uint32_t kRadix = 1u << kRadixBits;
static constexpr uint32_t kItemsLarge = 16; // pairs per lane: 4096-pair tiles
static constexpr uint32_t kItemsSmall = 4;  // 1024-pair tiles when there are too few pairs to fill the GPU otherwise
static constexpr int64_t kSmallSortLimit = 1ll << 21;

__device__ __forceinline__ uint32_t digit_of(int64_t key, uint32_t shift, uint32_t mask) {
    return (uint32_t)((uint64_t)key >> shift) & mask;
}
__device__ __forceinline__ uint32_t digit_of(uint16_t key, uint32_t shift, uint32_t mask) {
    return ((uint32_t)key >> shift) & mask;
}

template <typename KeyT>
__global__ void __launch_bounds__(256) radix_hist_kernel(uint32_t n, const KeyT* __restrict__ keys,
                                                          uint32_t items, uint32_t shift, uint32_t mask,
                                                          uint32_t nblocks,
                                                          uint32_t* __restrict__ hist /*[kRadix][nblocks]*/) {
    __shared__ uint32_t lh[kRadix];
    lh[threadIdx.x] = 0;
    __syncthreads();
    const uint32_t base = blockIdx.x * 256u * items;
    if (sizeof(KeyT) == 2 && ((uintptr_t)keys & 15u) == 0) {
        // 16-bit keys, eight to a 16-byte load (a tile starts at a multiple of 1024 keys)
        const uint4* __restrict__ k8 = reinterpret_cast<const uint4*>(keys + base);
        for (uint32_t v = threadIdx.x; v < 32u * items; v += 256u) {
            const uint32_t first = base + v * 8u;
            if (first + 8u <= n) {
                const uint4 q = k8[v];
                const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
                for (uint32_t h = 0; h < 4; ++h) {
                    atomicAdd(&lh[((w[h] & 0xffffu) >> shift) & mask], 1u);
                    atomicAdd(&lh[((w[h] >> 16) >> shift) & mask], 1u);
                }
            } else {
                for (uint32_t idx = first; idx < n && idx < first + 8u; ++idx)
                    atomicAdd(&lh[digit_of(keys[idx], shift, mask)], 1u);
            }
        }
    } else {
#pragma unroll 4
        for (uint32_t i = 0; i < items; ++i) {
            const uint32_t idx = base + i * 256u + threadIdx.x;
            if (idx < n)
                atomicAdd(&lh[digit_of(keys[idx], shift, mask)], 1u);
        }
    }
    __syncthreads();
    hist[threadIdx.x * nblocks + blockIdx.x] = lh[threadIdx.x];
}

// ---- per-digit scan --------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t wave_inclusive_scan_u32(uint32_t v, uint32_t lane) {
#pragma unroll
    for (uint32_t off = 1; off < 64; off <<= 1) {
        const uint32_t up = __shfl_up(v, off, 64);
        if (lane >= off)
            v += up;
    }
    return v;
}

// Block d owns digit d: hist[d][0..nblocks) becomes the number of pairs with digit d in earlier sort blocks, and
// digit_total[d] the number of pairs with digit d.  (The scatter adds the pairs with a smaller digit: an exclusive
// scan of the 256 totals, which every sort block forms for itself - no atomics, nothing to zero beforehand.)
__global__ void __launch_bounds__(256) radix_scan_kernel(uint32_t nblocks, uint32_t* __restrict__ hist,
                                                          uint32_t* __restrict__ digit_total /*[kRadix]*/) {
    __shared__ uint32_t wsum[4];
    const uint32_t d = blockIdx.x, t = threadIdx.x, lane = t & 63u, w = t >> 6;
    uint32_t carry = 0;
    uint32_t* __restrict__ row = hist + (size_t)d * nblocks;
    for (uint32_t start = 0; start < nblocks; start += 256) {
        const uint32_t i = start + t;
        const uint32_t v = i < nblocks ? row[i] : 0u;
        const uint32_t incl = wave_inclusive_scan_u32(v, lane);
        __syncthreads(); // wsum of the previous round has been read
        if (lane == 63)
            wsum[w] = incl;
        __syncthreads();
        uint32_t before = 0;
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k)
            before += k < w ? wsum[k] : 0u;
        if (i < nblocks)
            row[i] = carry + before + incl - v;
        carry += wsum[0] + wsum[1] + wsum[2] + wsum[3];
    }
    if (t == 0)
        digit_total[d] = carry;
}

// ---- digit counts of all passes in one read of the keys ---------------------------------------------
struct RadixDigits {
    uint32_t passes;
    uint32_t shift[8], mask[8];
};
static constexpr uint32_t kTotalReplicas = 4;

// totals[pass][replica][256] += the number of keys whose digit of that pass is d; a workgroup counts in LDS (a wave
// whose keys share a digit - the upper bytes of sorted or narrow keys - adds once) and adds its counts to one of the
// replicas.  Grid-stride over chunks of 256 x 16 keys.
template <typename KeyT>
__global__ void __launch_bounds__(256) radix_totals_kernel(uint32_t n, const KeyT* __restrict__ keys, RadixDigits dg,
                                                            uint32_t* __restrict__ totals) {
    __shared__ uint32_t lh[8][kRadix];
    const uint32_t t = threadIdx.x, lane = t & 63u;
    for (uint32_t p = 0; p < dg.passes; ++p)
        lh[p][t] = 0;
    __syncthreads();
    for (uint64_t chunk = (uint64_t)blockIdx.x * 4096u; chunk < n; chunk += (uint64_t)gridDim.x * 4096u) {
        KeyT key[16];
#pragma unroll
        for (uint32_t r = 0; r < 16; ++r) {
            const uint64_t idx = chunk + r * 256u + t;
            key[r] = idx < n ? keys[idx] : (KeyT)0;
        }
#pragma unroll
        for (uint32_t r = 0; r < 16; ++r) {
            const bool valid = chunk + r * 256u + t < n;
            const uint64_t active = __ballot(valid);
            if (active == 0)
                continue;
            const uint32_t first = (uint32_t)__builtin_ctzll(active);
            for (uint32_t p = 0; p < dg.passes; ++p) {
                const uint32_t d = digit_of(key[r], dg.shift[p], dg.mask[p]);
                const uint32_t d_first = (uint32_t)__builtin_amdgcn_readlane((int)d, first);
                if (__ballot(valid && d != d_first) == 0) {
                    if (lane == first)
                        atomicAdd(&lh[p][d], (uint32_t)__builtin_popcountll(active));
                } else if (valid) {
                    atomicAdd(&lh[p][d], 1u);
                }
            }
        }
    }
    __syncthreads();
    uint32_t* mine = totals + (size_t)(blockIdx.x % kTotalReplicas) * kRadix;
    for (uint32_t p = 0; p < dg.passes; ++p) {
        const uint32_t c = lh[p][t];
        if (c != 0)
            atomicAdd(mine + (size_t)p * kTotalReplicas * kRadix + t, c);
    }
}

// zeroes the bookkeeping words of a chained sort (digit counts, error word, the first pass's status rows) and leaves
// the number of pairs where the passes read it
// (words n_word and n_word + 1: every word has one writer)
__global__ void __launch_bounds__(256) radix_prepare_kernel(size_t n_words, uint32_t* __restrict__ words,
                                                             size_t n_word, int64_t n) {
    const size_t i = (size_t)blockIdx.x * 256u + threadIdx.x;
    if (i < n_words)
        words[i] = i == n_word ? (uint32_t)(uint64_t)n : i == n_word + 1 ? (uint32_t)((uint64_t)n >> 32) : 0u;
}

// ---- stable scatter -------------------------------------------------------------------------------
// CHAINED = false: the positions come from the scanned histogram table of the two launches before (hist_scanned,
// digit_total).  CHAINED = true: one launch per pass - digit_total holds the digit counts of the whole input (left by
// whoever wrote the keys), every workgroup publishes its 256 digit counts and obtains the counts of the workgroups in front of it by a chained look-back (gsx_lookback.h); the number of
// pairs is read from device memory, and the launch also clears the status words the NEXT pass will use.
struct RadixChain {
    const int64_t* n_dev;   // number of pairs (device); the launch covers min(*n_dev, n) pairs
    uint32_t* status;       // [workgroups][256], empty on entry
    uint32_t* clear_status; // status words of the next pass (nullable): clear_rows rows are cleared by this launch
    uint32_t clear_rows;
    uint32_t* error;        // bit 1 is set when a look-back gave up
    uint32_t total_replicas, total_stride; // digit_total = sum of this many tables, total_stride words apart
    uint32_t spin_limit;    // empty reads after which a look-back gives up
};

// NW waves per workgroup (a tile of 64 NW ITEMS pairs): chained passes take eight or sixteen, for tiles of 8192 pairs -
// half as many places for a look-back to walk; threads 0..255 double as the digits.
template <typename KeyT, uint32_t ITEMS, bool CHAINED, bool WRITE_KEYS, uint32_t NW = 4>
__global__ void __launch_bounds__(64 * NW, NW == 8 ? 4 : 1) radix_scatter_kernel(uint32_t n, const KeyT* __restrict__ keys_in,
                                                             const int32_t* __restrict__ vals_in,
                                                             KeyT* __restrict__ keys_out,
                                                             int32_t* __restrict__ vals_out, uint32_t shift,
                                                             uint32_t mask, uint32_t nblocks,
                                                             const uint32_t* __restrict__ hist_scanned,
                                                             const uint32_t* __restrict__ digit_total,
                                                             RadixChain chain) {
    constexpr uint32_t kThreads = 64 * NW, kTileN = kThreads * ITEMS, kWaveN = 64 * ITEMS;
    __shared__ uint32_t wave_count[NW][kRadix];
    __shared__ uint32_t to_global[kRadix]; // global position of a pair = to_global[digit] + its slot in the tile
    __shared__ uint32_t wsum[4], gsum[4];
    // the match masks of the ranking phase and the reordered tile of the output phase share their bytes
    constexpr uint32_t kMatchBytes = NW * kRadix * 8, kTileBytes = kTileN * (sizeof(KeyT) + 4);
    __shared__ __align__(16) unsigned char overlay[kMatchBytes > kTileBytes ? kMatchBytes : kTileBytes];
    unsigned long long(*match)[kRadix] = reinterpret_cast<unsigned long long(*)[kRadix]>(overlay);
    int32_t* s_vals = reinterpret_cast<int32_t*>(overlay);
    KeyT* s_keys = reinterpret_cast<KeyT*>(overlay + kTileN * 4);
    const uint32_t t_in = threadIdx.x;
    // the 64-bit chained passes (one workgroup per CU) loop over places; the 16-bit ones (two per CU, half the LDS)
    // keep one place per workgroup: the loop costs them registers they do not have
    constexpr bool kLoop = CHAINED && sizeof(KeyT) == 8;
    // A chained launch has no more workgroups than the GPU holds at once; workgroup b takes the places b,
    // b + gridDim.x, ... in turn, so a launch sized for a buffer's capacity does not queue hundreds of empty
    // workgroups behind the few that have work, each waiting for a whole CU's LDS.  (All of them resident matters:
    // place gridDim.x waits for place gridDim.x - 1, whose workgroup must have been started.)
#pragma clang loop unroll(disable)
    for (uint32_t place = blockIdx.x;; place += gridDim.x) {
    // (the lane's index is made opaque once per place: otherwise every address of the body is kept in registers
    // across the loop, and the kernel no longer fits the registers its occupancy allows)
    uint32_t t = t_in;
    asm volatile("" : "+v"(t));
    const uint32_t w = t >> 6, lane = t & 63u;
    const uint64_t lt_mask = (1ull << lane) - 1ull;
    const uint32_t tile_base = place * kTileN;
    const uint32_t wave_base = tile_base + w * kWaveN;
    KeyT key[ITEMS];
    int32_t val[ITEMS];
    uint32_t rank[ITEMS]; // rank among the wave's pairs with the same digit
    // requested before the count is known (chained: it comes from memory too); the buffers hold n entries at least
#pragma unroll
    for (uint32_t r = 0; r < ITEMS; ++r) {
        const uint32_t idx = wave_base + r * 64u + lane;
        const bool in_buffer = idx < n;
        key[r] = in_buffer ? keys_in[idx] : 0;
        val[r] = in_buffer ? vals_in[idx] : 0;
    }
    // the digit totals are requested now as well and first used after the ranking
    const bool is_digit = NW == 4 || t < kRadix; // this thread also stands for digit t
    uint32_t gtot = is_digit ? digit_total[t] : 0u; // pairs with digit t in the whole input
    if (CHAINED && chain.total_replicas > 1 && is_digit) { // up to four tables: the loads are issued together
        uint32_t part[3];
#pragma unroll
        for (uint32_t r = 0; r < 3; ++r)
            part[r] = r + 1 < chain.total_replicas ? digit_total[(r + 1) * chain.total_stride + t] : 0u;
        gtot += part[0] + part[1] + part[2];
    }
    if (CHAINED) {
        if (chain.n_dev != nullptr) {
            const int64_t nd = *chain.n_dev;
            n = nd < (int64_t)n ? (uint32_t)(nd < 0 ? 0 : nd) : n;
        }
        // housekeeping for the pass after this one (its launch starts after this one has ended)
        if (chain.clear_status != nullptr && place == blockIdx.x)
            for (size_t wd = (size_t)place * kThreads + t; wd < (size_t)chain.clear_rows * kRadix;
                 wd += (size_t)gridDim.x * kThreads)
                chain.clear_status[wd] = 0u;
        if ((uint64_t)place * kTileN >= n)
            return; // uniform over the workgroup; later places are empty too
    }
    if (is_digit) {
#pragma unroll
        for (uint32_t i = 0; i < NW; ++i) {
            wave_count[i][t] = 0;
            match[i][t] = 0ull;
        }
    }
    __syncthreads();

#pragma unroll
    for (uint32_t r = 0; r < ITEMS; ++r) {
        const uint32_t idx = wave_base + r * 64u + lane;
        const bool valid = idx < n;
        const uint32_t d = digit_of(key[r], shift, mask);
        // peers: the wave's lanes whose pair has this lane's digit.  Every lane sets its bit in the digit's mask in
        // LDS and reads the mask back (LDS serves one wave's instructions in order); the lowest peer clears it for
        // the next round.  A wave whose pairs all share one digit (sorted or constant input) skips the LDS trip.
        const uint64_t valid_lanes = __ballot(valid);
        uint64_t peers = valid_lanes;
        if (valid_lanes) {
            const uint32_t d_first = (uint32_t)__builtin_amdgcn_readlane((int)d, __builtin_ctzll(valid_lanes));
            if (__ballot(valid && d != d_first)) {
                if (valid)
                    atomicOr(&match[w][d], 1ull << lane);
                __builtin_amdgcn_wave_barrier();
                peers = valid ? match[w][d] : 0ull;
                __builtin_amdgcn_wave_barrier();
                if (valid && (peers & lt_mask) == 0)
                    match[w][d] = 0ull;
                __builtin_amdgcn_wave_barrier();
            }
        }
        uint32_t pre = 0;
        if (valid)
            pre = wave_count[w][d];
        __builtin_amdgcn_wave_barrier();
        rank[r] = pre + (uint32_t)__popcll(peers & lt_mask);
        if (valid && (peers & lt_mask) == 0)
            wave_count[w][d] = pre + (uint32_t)__popcll(peers);
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();
    // digit t: slot at which each wave's pairs with this digit start inside the tile (digits in ascending order,
    // waves in ascending order inside a digit), and the offset from tile slots to global positions
    {
        uint32_t c[NW];
        uint32_t tot = 0;
        if (is_digit) {
#pragma unroll
            for (uint32_t k = 0; k < NW; ++k) {
                c[k] = wave_count[k][t];
                tot += c[k];
            }
            if (CHAINED) // the first place has nobody in front of it: its counts are a complete prefix already
                lb_publish(chain.status + (size_t)place * kRadix + t, place == 0 ? kLbPrefix : kLbAggregate, tot);
        }
        const uint32_t incl = wave_inclusive_scan_u32(tot, lane);
        const uint32_t gincl = wave_inclusive_scan_u32(gtot, lane);
        if (is_digit && lane == 63) {
            wsum[w] = incl;
            gsum[w] = gincl;
        }
        __syncthreads();
        if (is_digit) {
            uint32_t before = 0, gbefore = 0;
#pragma unroll
            for (uint32_t k = 0; k < 4; ++k) {
                before += k < w ? wsum[k] : 0u;
                gbefore += k < w ? gsum[k] : 0u;
            }
            const uint32_t start = before + incl - tot;
            const uint32_t smaller = gbefore + gincl - gtot; // pairs with a smaller digit
            uint32_t run = start;
#pragma unroll
            for (uint32_t k = 0; k < NW; ++k) {
                wave_count[k][t] = run;
                run += c[k];
            }
            uint32_t earlier; // pairs with digit t in the workgroups in front of this one
            if (CHAINED) {
                earlier = lb_exclusive(chain.status, place, kRadix, t, chain.error, chain.spin_limit);
                if (place != 0)
                    lb_publish(chain.status + (size_t)place * kRadix + t, kLbPrefix, earlier + tot);
            } else {
                earlier = hist_scanned[t * nblocks + blockIdx.x];
            }
            to_global[t] = smaller + earlier - start;
        }
    }
    __syncthreads();
#pragma unroll
    for (uint32_t r = 0; r < ITEMS; ++r) {
        const uint32_t idx = wave_base + r * 64u + lane;
        if (idx < n) {
            const uint32_t slot = wave_count[w][digit_of(key[r], shift, mask)] + rank[r];
            s_keys[slot] = key[r];
            s_vals[slot] = val[r];
        }
    }
    __syncthreads();
    const uint32_t count = min(kTileN, n - tile_base);
#pragma unroll
    for (uint32_t k = 0; k < ITEMS; ++k) {
        const uint32_t slot = k * kThreads + t;
        if (slot < count) {
            const KeyT kk = s_keys[slot];
            const uint32_t pos = to_global[digit_of(kk, shift, mask)] + slot;
            // chained: digit totals that disagree with the keys (a caller's mistake) must not write out of bounds
            if (!CHAINED || pos < n) {
                if (WRITE_KEYS)
                    keys_out[pos] = kk;
                vals_out[pos] = s_vals[slot];
            }
        }
    }
    if (!kLoop)
        break;
    __syncthreads(); // the tile in LDS has been written out
    }
}

} // namespace gsx

namespace gsx {
namespace {
template <typename KeyT>
int chained_pass(uint32_t n_max, const KeyT* kin, const int32_t* vin, KeyT* kout, int32_t* vout, uint32_t shift,
                 uint32_t bits, const uint32_t* digit_total, const RadixChainArgs& a, bool write_keys, void* stream);
} // namespace
} // namespace gsx

using namespace gsx;

namespace {
static constexpr uint32_t kMaxPasses = 8;
struct SortLayout {
    // the three-launch pass: histogram table [256][nblocks] and the digit totals
    uint32_t nblocks;
    size_t hist_off, totals_off, tabled_total;
    // the chained sort, behind it: digit counts of every pass [8][kTotalReplicas][256], a line with the error word
    // and the number of pairs, two status tables of `rows` x 256 words used in turn
    uint32_t rows;
    size_t digits_off, misc_off, status_off[2], total;
};
static constexpr size_t kDigitsBytes = (size_t)kMaxPasses * kTotalReplicas * kRadix * 4;
// whether sort_pairs takes the chained passes for this size
bool sort_is_chained(int64_t n, uint32_t key_bytes) {
    return n < (1ll << kLbValueBits) && n > (key_bytes == 8 ? kSmallSortLimit : (1ll << 25));
}
uint32_t sort_items(int64_t n) { return n <= kSmallSortLimit ? kItemsSmall : kItemsLarge; }
SortLayout sort_layout(int64_t n) {
    SortLayout L;
    L.nblocks = cdiv((uint64_t)n, 256u * sort_items(n));
    L.hist_off = 0;
    L.totals_off = align_up((size_t)L.nblocks * kRadix * 4, 256);
    L.tabled_total = L.totals_off + (size_t)kRadix * 4;
    L.rows = radix_chained_rows(n);
    L.digits_off = align_up(L.tabled_total, 256);
    L.misc_off = L.digits_off + kDigitsBytes;
    L.status_off[0] = L.misc_off + 256;
    L.status_off[1] = L.status_off[0] + (size_t)L.rows * kRadix * 4;
    L.total = L.status_off[1] + (size_t)L.rows * kRadix * 4;
    return L;
}
} // namespace

// monotone in n (a workspace sized for a capacity serves every smaller sort, whichever tile size that one uses)
extern "C" size_t gsx_radix_sort_pairs_workspace_bytes(int64_t n) {
    if (n <= 0)
        return 256;
    const size_t need = sort_layout(n).total;
    const size_t small_max = sort_layout(kSmallSortLimit).total;
    return n > kSmallSortLimit && small_max > need ? small_max : need;
}

extern "C" int gsx_radix_sort_pairs_selector(int64_t n, uint32_t begin_bit, uint32_t end_bit) {
    if (n <= 0 || end_bit <= begin_bit)
        return 0;
    return (int)(((end_bit - begin_bit + kRadixBits - 1) / kRadixBits) & 1u); // one ping-pong per digit pass
}

namespace {
// first_hist_done: the caller's own kernel has already left the first pass's histogram table in the workspace
// (gsx::radix_first_pass_table)
// chained: the workspace holds gsx_radix_sort_pairs_workspace_bytes(n) (false: only the three-launch pass's part)
template <typename KeyT>
int sort_pairs(const char* what, int64_t n, KeyT* keys0, int32_t* vals0, KeyT* keys1, int32_t* vals1,
               uint32_t begin_bit, uint32_t end_bit, void* workspace, size_t workspace_bytes, int* selector_host,
               void* stream, bool first_hist_done = false, bool chained = true) {
    if (selector_host)
        *selector_host = 0;
    if (n <= 0)
        return GSX_OK; // IntersectTile.cu:298-300
    GSX_REQUIRE(n < (1ll << 31), GSX_ERR_OVERFLOW, "%s: n = %lld does not fit int32", what, (long long)n);
    GSX_REQUIRE(keys0 && vals0 && keys1 && vals1, GSX_ERR_INVALID_ARGUMENT, "%s: null buffer", what);
    GSX_REQUIRE(end_bit >= 1 && end_bit <= 8 * sizeof(KeyT) && begin_bit < end_bit, GSX_ERR_INVALID_ARGUMENT,
                "%s: bits [%u, %u)", what, begin_bit, end_bit);
    const SortLayout L = sort_layout(n);
    // measured: the chained sort is ahead from ~2 M pairs with 64-bit keys (310 against 339 us at 5.67 M pairs and 45
    // bits, 834 against 973 us at 16 M) and from ~30 M pairs with 16-bit keys (706 against 812 us at 64 M); below, its
    // few large workgroups and the extra read of the keys cost more than the launches they save
    chained = chained && sort_is_chained(n, (uint32_t)sizeof(KeyT));
    const size_t need = chained ? L.total : L.tabled_total;
    GSX_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0 && workspace_bytes >= need,
                GSX_ERR_WORKSPACE, "%s: workspace needs %zu bytes, 256-byte aligned", what, need);
    uint32_t* hist = (uint32_t*)((char*)workspace + L.hist_off);
    uint32_t* totals = (uint32_t*)((char*)workspace + L.totals_off);
    hipStream_t s = (hipStream_t)stream;
    // digits as equal as possible: ceil(bits / 8) passes of floor or ceil(bits / passes) bits (13 tile bits sort
    // as 7 + 6, whose longer runs per (block, digit) scatter in fuller cache lines than 8 + 5)
    const uint32_t n_bits = end_bit - begin_bit;
    const uint32_t passes = (n_bits + kRadixBits - 1) / kRadixBits;
    GSX_REQUIRE(passes <= kMaxPasses, GSX_ERR_INVALID_ARGUMENT, "%s: %u passes", what, passes);
    const uint32_t width_lo = n_bits / passes, n_wide = n_bits % passes;
    int sel = 0;
    uint32_t shift = begin_bit;
    if (chained) {
        char* ws = (char*)workspace;
        uint32_t* digits = (uint32_t*)(ws + L.digits_off);
        uint32_t* error = (uint32_t*)(ws + L.misc_off);
        int64_t* n_slot = (int64_t*)(ws + L.misc_off + 8);
        uint32_t* status[2] = {(uint32_t*)(ws + L.status_off[0]), (uint32_t*)(ws + L.status_off[1])};
        // digit counts, the line with the error word and the first status table are one run of words
        const size_t n_words = (L.status_off[1] - L.digits_off) / 4;
        hipLaunchKernelGGL(radix_prepare_kernel, dim3((uint32_t)cdiv((uint64_t)n_words, 256u)), dim3(256), 0, s, n_words,
                           digits, (size_t)((uint32_t*)n_slot - digits), n);
        GSX_LAUNCH_CHECK();
        RadixDigits dg;
        dg.passes = passes;
        for (uint32_t pass = 0, at = begin_bit; pass < kMaxPasses; ++pass) {
            const uint32_t bits = pass < passes ? width_lo + (pass < n_wide ? 1u : 0u) : 0u;
            dg.shift[pass] = at, dg.mask[pass] = (1u << bits) - 1u;
            at += bits;
        }
        const uint32_t blocks = (uint32_t)std::min<uint64_t>(cdiv((uint64_t)n, 4096u), 1024u);
        hipLaunchKernelGGL(radix_totals_kernel<KeyT>, dim3(blocks), dim3(256), 0, s, (uint32_t)n, keys0, dg, digits);
        GSX_LAUNCH_CHECK();
        for (uint32_t pass = 0; pass < passes; ++pass) {
            const uint32_t bits = width_lo + (pass < n_wide ? 1u : 0u);
            RadixChainArgs a;
            a.n_dev = n_slot, a.status = status[pass & 1u], a.error = error;
            a.clear_status = pass + 1 < passes ? status[(pass + 1) & 1u] : nullptr, a.clear_rows = L.rows;
            a.total_replicas = kTotalReplicas, a.total_stride = kRadix;
            const int rc = chained_pass<KeyT>((uint32_t)n, sel ? keys1 : keys0, sel ? vals1 : vals0, sel ? keys0 : keys1,
                                              sel ? vals0 : vals1, shift, bits,
                                              digits + (size_t)pass * kTotalReplicas * kRadix, a, true, stream);
            if (rc != GSX_OK)
                return rc;
            sel ^= 1;
            shift += bits;
        }
        if (selector_host)
            *selector_host = sel;
        return GSX_OK;
    }
    const uint32_t items = sort_items(n);
    for (uint32_t pass = 0; pass < passes; ++pass) {
        const uint32_t bits = width_lo + (pass < n_wide ? 1u : 0u);
        const uint32_t mask = (1u << bits) - 1u;
        const KeyT* kin = sel ? keys1 : keys0;
        const int32_t* vin = sel ? vals1 : vals0;
        KeyT* kout = sel ? keys0 : keys1;
        int32_t* vout = sel ? vals0 : vals1;
        if (!(first_hist_done && pass == 0)) {
            hipLaunchKernelGGL(radix_hist_kernel<KeyT>, dim3(L.nblocks), dim3(256), 0, s, (uint32_t)n, kin, items,
                               shift, mask, L.nblocks, hist);
            GSX_LAUNCH_CHECK();
        }
        hipLaunchKernelGGL(radix_scan_kernel, dim3(kRadix), dim3(256), 0, s, L.nblocks, hist, totals);
        GSX_LAUNCH_CHECK();
        if (items == kItemsSmall)
            hipLaunchKernelGGL((radix_scatter_kernel<KeyT, kItemsSmall, false, true>), dim3(L.nblocks), dim3(256), 0,
                               s, (uint32_t)n, kin, vin, kout, vout, shift, mask, L.nblocks, hist, totals,
                               RadixChain{});
        else
            hipLaunchKernelGGL((radix_scatter_kernel<KeyT, kItemsLarge, false, true>), dim3(L.nblocks), dim3(256), 0,
                               s, (uint32_t)n, kin, vin, kout, vout, shift, mask, L.nblocks, hist, totals,
                               RadixChain{});
        GSX_LAUNCH_CHECK();
        sel ^= 1;
        shift += bits;
    }
    if (selector_host)
        *selector_host = sel;
    return GSX_OK;
}
} // namespace

namespace gsx {
// Where a kernel that writes the keys of a sort on bits [begin_bit, begin_bit + 32) can leave the first pass's
// histogram itself: sort block b covers keys [b * 256 * items, (b + 1) * 256 * items) and table[d * nblocks + b]
// counts its keys whose bits [begin_bit, begin_bit + 8) equal d.
RadixFirstPass radix_first_pass_table(int64_t n, void* workspace) {
    const SortLayout L = sort_layout(n);
    RadixFirstPass f;
    f.items = sort_items(n);
    f.nblocks = L.nblocks;
    f.table = (uint32_t*)((char*)workspace + L.hist_off);
    return f;
}
int radix_sort_pairs_32_bits(int64_t n, int64_t* keys0, int32_t* vals0, int64_t* keys1, int32_t* vals1,
                             uint32_t begin_bit, void* workspace, size_t workspace_bytes, int* selector_host,
                             void* stream, bool first_hist_done) {
    return sort_pairs<int64_t>("radix_sort_pairs", n, keys0, vals0, keys1, vals1, begin_bit, begin_bit + 32, workspace,
                               workspace_bytes, selector_host, stream, first_hist_done);
}
} // namespace gsx

namespace gsx {
// ---- one launch per pass (declared in gsx_common.h) ------------------------------------------------
// chained passes always take tiles of kChainedTile pairs: the look-back walks as many places as there are workgroups
// with work.  (The status table is sized for tiles of 4096 pairs; the passes use its first rows.)  A pass is bound by
// the latency of what one wave does one thing after the other - ranking, reordering and writing its share of the
// tile - so the 64-bit passes (one workgroup per CU either way) split the tile over sixteen waves of 8 pairs per lane;
// the 16-bit passes keep eight waves of 16, of which two workgroups fit a CU.
static constexpr uint32_t kChainedTile = 8192;
template <typename KeyT>
struct ChainedShape {
    static constexpr uint32_t kWaves = sizeof(KeyT) == 8 ? 16 : 8, kItems = kChainedTile / (64 * kWaves);
};
// How many workgroups of `kernel` (no dynamic LDS) one device runs at the same time: what the runtime's occupancy
// calculation gives per CU, times the CUs.  Remembered per (device, kernel).
int resident_workgroups(const void* kernel, int threads, uint32_t* out) {
    struct Entry {
        int device;
        const void* kernel;
        uint32_t value;
    };
    static std::mutex mutex;
    static std::vector<Entry> known;
    int dev = -1;
    GSX_HIP_CHECK(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(mutex);
    for (const Entry& e : known)
        if (e.device == dev && e.kernel == kernel) {
            *out = e.value;
            return GSX_OK;
        }
    int per_cu = 0, cus = 0;
    GSX_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, 0));
    GSX_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    GSX_REQUIRE(per_cu >= 1 && cus >= 1, GSX_ERR_HIP, "chained radix pass: %d workgroups per CU on %d CUs", per_cu, cus);
    known.push_back({dev, kernel, (uint32_t)per_cu * (uint32_t)cus});
    *out = known.back().value;
    return GSX_OK;
}

uint32_t radix_chained_rows(int64_t n_max) { return n_max <= 0 ? 1u : cdiv((uint64_t)n_max, 256u * kItemsLarge); }

namespace {
template <typename KeyT>
int chained_pass(uint32_t n_max, const KeyT* kin, const int32_t* vin, KeyT* kout, int32_t* vout, uint32_t shift,
                 uint32_t bits, const uint32_t* digit_total, const RadixChainArgs& a, bool write_keys, void* stream) {
    GSX_REQUIRE(n_max > 0 && n_max < (1u << kLbValueBits), GSX_ERR_OVERFLOW,
                "chained radix pass: %u pairs (limit 2^30 - 1)", n_max);
    GSX_REQUIRE(bits >= 1 && bits <= kRadixBits && kin && vin && vout && (kout || !write_keys) && digit_total &&
                    a.status && a.error,
                GSX_ERR_INVALID_ARGUMENT, "chained radix pass: bad argument");
    const uint32_t rows = cdiv((uint64_t)n_max, kChainedTile);
    const uint32_t mask = (1u << bits) - 1u;
    RadixChain c;
    c.n_dev = a.n_dev, c.status = a.status, c.clear_status = a.clear_status;
    c.clear_rows = a.clear_rows, c.error = a.error;
    GSX_REQUIRE(a.total_replicas <= 4, GSX_ERR_INVALID_ARGUMENT, "chained radix pass: at most 4 total tables");
    c.total_replicas = a.total_replicas ? a.total_replicas : 1u, c.total_stride = a.total_stride;
    c.spin_limit = lookback_spin_limit();
    hipStream_t s = (hipStream_t)stream;
    using Shape = ChainedShape<KeyT>;
    // as many workgroups as the device holds at once - asked of the runtime for this very kernel, whose registers
    // and LDS decide it; each takes the places blockIdx.x, blockIdx.x + groups, ... in turn
    uint32_t resident = 0;
    if (write_keys) {
        const int rc = resident_workgroups((const void*)radix_scatter_kernel<KeyT, Shape::kItems, true, true, Shape::kWaves>,
                                           64 * Shape::kWaves, &resident);
        if (rc != GSX_OK)
            return rc;
    } else {
        const int rc = resident_workgroups((const void*)radix_scatter_kernel<KeyT, Shape::kItems, true, false, Shape::kWaves>,
                                           64 * Shape::kWaves, &resident);
        if (rc != GSX_OK)
            return rc;
    }
    const uint32_t groups = sizeof(KeyT) == 8 ? std::min(rows, resident) : rows;
#define GSX_CHAINED(WK)                                                                                        \
    hipLaunchKernelGGL((radix_scatter_kernel<KeyT, Shape::kItems, true, WK, Shape::kWaves>), dim3(groups),    \
                       dim3(64 * Shape::kWaves), 0, s, n_max, kin, vin, kout, vout, shift, mask, rows,        \
                       (const uint32_t*)nullptr, digit_total, c)
    if (write_keys)
        GSX_CHAINED(true);
    else
        GSX_CHAINED(false);
#undef GSX_CHAINED
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}
} // namespace

int radix_chained_pass_i64(uint32_t n_max, const int64_t* kin, const int32_t* vin, int64_t* kout, int32_t* vout,
                           uint32_t shift, uint32_t bits, const uint32_t* digit_total, const RadixChainArgs& a,
                           void* stream) {
    return chained_pass<int64_t>(n_max, kin, vin, kout, vout, shift, bits, digit_total, a, true, stream);
}
int radix_chained_pass_u16(uint32_t n_max, const uint16_t* kin, const int32_t* vin, uint16_t* kout, int32_t* vout,
                           uint32_t shift, uint32_t bits, const uint32_t* digit_total, const RadixChainArgs& a,
                           bool write_keys, void* stream) {
    return chained_pass<uint16_t>(n_max, kin, vin, kout, vout, shift, bits, digit_total, a, write_keys, stream);
}
} // namespace gsx

extern "C" uint32_t* gsx_radix_sort_pairs_error(int64_t n, uint32_t key_bytes, void* workspace) {
    if (workspace == nullptr || n <= 0 || (key_bytes != 8 && key_bytes != 2) || !sort_is_chained(n, key_bytes))
        return nullptr;
    return (uint32_t*)((char*)workspace + sort_layout(n).misc_off);
}

extern "C" int gsx_radix_sort_pairs(int64_t n, int64_t* keys0, int32_t* vals0, int64_t* keys1, int32_t* vals1,
                                    uint32_t begin_bit, uint32_t end_bit, void* workspace, size_t workspace_bytes,
                                    int* selector_host, void* stream) {
    return sort_pairs<int64_t>("radix_sort_pairs", n, keys0, vals0, keys1, vals1, begin_bit, end_bit, workspace,
                               workspace_bytes, selector_host, stream);
}

// The same sort for 16-bit keys (tile indices of one camera, bits [0, n_bits)): a third of the bytes per pass.
extern "C" int gsx_radix_sort_tile_pairs(int64_t n, uint16_t* keys0, int32_t* vals0, uint16_t* keys1, int32_t* vals1,
                                         uint32_t n_bits, void* workspace, size_t workspace_bytes,
                                         int* selector_host, void* stream) {
    return sort_pairs<uint16_t>("radix_sort_tile_pairs", n, keys0, vals0, keys1, vals1, 0, n_bits, workspace,
                                workspace_bytes, selector_host, stream);
}

// ---- the pair sort for callers that cannot allocate (and so cannot bring a workspace) ----------------------------
// The histogram table and the digit totals live in a file-scope device array.  Every GPU the library runs on holds
// its own copy of the array at its own address (4 MiB + 1.25 KiB until the process ends); the address is looked up
// once per device and only that pointer is ever handed to kernels.
namespace {
static constexpr size_t kStaticScratchBytes =
    (size_t)(GSX_RADIX_SORT_STATIC_MAX_PAIRS / (256 * kItemsLarge)) * kRadix * 4 + 256 + kRadix * 4;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

static constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {};

// the device address of `scratch` on the current device
int static_scratch(void** out) {
    int dev = -1;
    GSX_HIP_CHECK(hipGetDevice(&dev));
    GSX_REQUIRE(dev >= 0 && dev < kMaxDevices, GSX_ERR_UNSUPPORTED, "radix_sort_pairs_static: device ordinal %d", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        GSX_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        GSX_REQUIRE(p != nullptr && ((uintptr_t)p & 255) == 0, GSX_ERR_HIP,
                    "radix_sort_pairs_static: the scratch array's device address %p is unusable", p);
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return GSX_OK;
}
} // namespace

extern "C" int gsx_radix_sort_pairs_static(int64_t n, int64_t* keys0, int32_t* vals0, int64_t* keys1, int32_t* vals1,
                                           uint32_t begin_bit, uint32_t end_bit, int* selector_host, void* stream) {
    if (selector_host)
        *selector_host = 0;
    if (n <= 0)
        return GSX_OK;
    GSX_REQUIRE(n <= (int64_t)GSX_RADIX_SORT_STATIC_MAX_PAIRS, GSX_ERR_WORKSPACE,
                "radix_sort_pairs_static: n = %lld exceeds the built-in scratch's limit of %lld pairs "
                "(use gsx_radix_sort_pairs with a workspace)",
                (long long)n, (long long)GSX_RADIX_SORT_STATIC_MAX_PAIRS);
    GSX_REQUIRE(sort_layout(n).tabled_total <= kStaticScratchBytes, GSX_ERR_WORKSPACE,
                "radix_sort_pairs_static: %zu bytes of scratch needed, %zu built in", sort_layout(n).tabled_total,
                kStaticScratchBytes);
    void* ws = nullptr;
    const int st = static_scratch(&ws);
    if (st != GSX_OK)
        return st;
    return sort_pairs<int64_t>("radix_sort_pairs_static", n, keys0, vals0, keys1, vals1, begin_bit, end_bit, ws,
                               kStaticScratchBytes, selector_host, stream, false, false);
}
