// tile_lists.hip - the per-tile lists of one camera in nine launches, without the pair count crossing to the host.
//
// What gsplat::intersect_tile + radix_sort_double_buffer + intersect_offset produce for one camera
// (gsplat/Intersect.cpp:41-137, IntersectTile.cu:23-114, 206-252, 290-328) and what the rasterizers read of it:
// flatten_ids (Gaussian ids, grouped by tile, depth order inside a tile, ties by id) and tile_offsets.  The result is
// element for element the one of the separate operators; the organisation is not:
//
//  1. depth_keys_kernel      keys (tile rectangle << 32 | depth bits) of the Gaussians that touch a tile, compacted
//                            in index order (nine in ten Gaussians of a training view touch none), and the four
//                            byte histograms of their depth bits (counted while the look-back waits);
//  2. four chained radix passes (radix_sort.hip) order the keys by depth, one launch each;
//  3. tile_table_kernel      +1 / -1 at every rectangle's corners in a (Th + 1) x (Tw + 1) grid and a 2-D prefix
//                            sum over it give every tile's list length, hence tile_offsets, the pair count, and the
//                            digit histograms of the pair sort - before a single pair exists;
//  4. super_emit_kernel      The tile grid is cut into at most 256 SUPER-TILES of 4 x 4 ... 16 x 16 tiles.  Every
//                            Gaussian, in depth order, leaves one entry (super-tile << 32 | rectangle, id) per
//                            super-tile its rectangle meets - 1.2 - 2 entries a Gaussian, against 7 - 30 (tile,
//                            Gaussian) pairs; a workgroup's position in the output comes from a chained look-back over
//                            the workgroups' entry counts;
//  5. one chained radix pass over the super-tile byte groups the entries by super-tile, depth order kept;
//  6. tile_gather_kernel     a workgroup takes a slice of up to 2 048 entries of one super-tile, turns every
//                            entry's rectangle into a bit mask over the super-tile's tiles, counts and then writes,
//                            per tile, the ids whose bit is set - in order, to the tile's place in flatten_ids;
//                            slices of one super-tile meet through a chained look-back over per-tile counts.  Every
//                            list is written once, front to back, and no (tile, id) pair is ever sorted.
//
// Everything downstream sizes its work by `capacity` and reads the actual count from device memory.  If the count
// exceeds the capacity, every tile's list is left EMPTY (tile_offsets all zero), bit 0 of the error word is set and
// the true count is still reported, so that the caller can grow its buffers and run the step again; nothing is
// written or read out of bounds.
//
// Atomics on addresses that many workgroups share are kept out of these kernels: on this GPU they cost far more
// than the work around them (1.1 M additions onto 5 000 counters took 0.32 ms, one returning addition per workgroup
// on a single word 20 ns each, serialised).  Counts meet through per-workgroup rows and replicas instead.
#include <algorithm>
#include <mutex>
#include <vector>

#include "gsx_common.h"
#include "gsx_lookback.h"
#include "gsx_tiles.h"

namespace gsx {

static constexpr uint32_t kKeysThreads = 1024;  // depth_keys_kernel: few, large workgroups keep the look-back short
static constexpr uint32_t kKeysPerBlock = 4 * kKeysThreads; // 4 consecutive Gaussians per lane
static constexpr uint32_t kEmitThreads = 1024;  // tile_emit_chained_kernel: likewise
static constexpr uint32_t kTableBlocks = 32;    // tile_table_kernel: workgroups that share the corner counting
static constexpr uint32_t kMaxLdsCells = 36 * 1024; // corner grids up to this many cells are counted in LDS
static constexpr uint32_t kSliceEntries = 2048; // tile_gather_kernel: entries of one super-tile a workgroup takes
static constexpr uint32_t kHistReplicas = 4;    // copies of the depth-byte histograms (fewer additions per address)

// adds 1 to hist[digit] for every live lane; one LDS atomic per wave when all its live lanes share the digit
__device__ __forceinline__ void wave_hist_add(uint32_t* hist, uint32_t digit, bool live) {
    const uint64_t lanes = __ballot(live);
    if (lanes == 0)
        return;
    const uint32_t first = (uint32_t)__builtin_amdgcn_readlane((int)digit, __builtin_ctzll(lanes));
    if (__ballot(live && digit != first) == 0) {
        if ((threadIdx.x & 63u) == (uint32_t)__builtin_ctzll(lanes))
            atomicAdd(&hist[first], (uint32_t)__popcll(lanes));
    } else if (live) {
        atomicAdd(&hist[digit], 1u);
    }
}

// Keys of the Gaussians that touch a tile, in index order (a chained look-back over the workgroups' counts places
// them).
__global__ void __launch_bounds__(kKeysThreads) depth_keys_kernel(
    uint32_t n, const float* __restrict__ means2d, const int32_t* __restrict__ radii,
    const float* __restrict__ depths, float tile_size, uint32_t tile_width, uint32_t tile_height,
    int64_t* __restrict__ keys, int32_t* __restrict__ vals, uint32_t* __restrict__ rects,
    uint32_t* __restrict__ status /*[blocks]*/, int64_t* __restrict__ counts, uint32_t* __restrict__ error,
    uint32_t* __restrict__ clear_status, uint32_t clear_rows, uint32_t* __restrict__ clear_emit_status,
    uint32_t clear_emit_words, uint32_t* __restrict__ clear_super_hist, uint32_t* __restrict__ clear_gather_status,
    uint32_t gather_rows_max, uint32_t n_super, uint32_t* __restrict__ depth_hist, uint32_t spin_limit) {
    constexpr uint32_t kWaves = kKeysThreads / 64u;
    __shared__ uint32_t wave_total[kWaves];
    __shared__ uint32_t base_s;
    __shared__ uint32_t lh[4][256]; // the four byte histograms of this workgroup's depth bits
    const uint32_t t = threadIdx.x, lane = t & 63u, wv = t >> 6;
    static_assert(kKeysThreads == 1024, "one histogram word per lane");
    lh[t >> 8][t & 255u] = 0u;
    // housekeeping for the launches behind this one
    for (uint32_t wd = blockIdx.x * kKeysThreads + t; wd < clear_rows * 256u; wd += gridDim.x * kKeysThreads)
        clear_status[wd] = 0u;
    for (uint32_t wd = blockIdx.x * kKeysThreads + t; wd < clear_emit_words; wd += gridDim.x * kKeysThreads)
        clear_emit_status[wd] = 0u;
    if (blockIdx.x == 0) // the entry counts per super-tile of the call before (kHistReplicas x 256 words)
        clear_super_hist[t] = 0u;
    {
        // the status rows the gather of the call before used: its entry count is still in counts[3]
        const uint32_t rows = min(gather_rows_max, (uint32_t)counts[3] / kSliceEntries + n_super);
        for (uint32_t wd = blockIdx.x * kKeysThreads + t; wd < rows * 256u; wd += gridDim.x * kKeysThreads)
            clear_gather_status[wd] = 0u;
    }
    uint32_t lo[4], hi[4];
    uint32_t mine = 0;
    // the lane's four Gaussians: every load leaves before the first result is used (indices clamped, results
    // discarded beyond n) - a load inside a condition would be waited for on the spot, twelve times in a row
    const uint32_t i0 = blockIdx.x * kKeysPerBlock + t * 4u;
    float2 m4[4];
    int2 r4[4];
    float d4[4];
    if (i0 + 3u < n) {
        const float4 ma = reinterpret_cast<const float4*>(means2d)[i0 / 2u], mb = reinterpret_cast<const float4*>(means2d)[i0 / 2u + 1u];
        const int4 ra = reinterpret_cast<const int4*>(radii)[i0 / 2u], rb = reinterpret_cast<const int4*>(radii)[i0 / 2u + 1u];
        const float4 dd = reinterpret_cast<const float4*>(depths)[i0 / 4u];
        m4[0] = make_float2(ma.x, ma.y), m4[1] = make_float2(ma.z, ma.w), m4[2] = make_float2(mb.x, mb.y), m4[3] = make_float2(mb.z, mb.w);
        r4[0] = make_int2(ra.x, ra.y), r4[1] = make_int2(ra.z, ra.w), r4[2] = make_int2(rb.x, rb.y), r4[3] = make_int2(rb.z, rb.w);
        d4[0] = dd.x, d4[1] = dd.y, d4[2] = dd.z, d4[3] = dd.w;
    } else {
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            const uint32_t i = min(i0 + k, n - 1u);
            m4[k] = reinterpret_cast<const float2*>(means2d)[i];
            r4[k] = reinterpret_cast<const int2*>(radii)[i];
            d4[k] = depths[i];
        }
    }
#pragma unroll
    for (uint32_t k = 0; k < 4; ++k) {
        lo[k] = 0, hi[k] = 0;
        TileRect r;
        if (i0 + k < n && tile_rect_of(m4[k], r4[k], tile_size, tile_width, tile_height, &r) && r.y1 > r.y0 &&
            r.x1 > r.x0) {
            lo[k] = f2u(d4[k]);
            hi[k] = r.x0 | (r.y0 << 8) | (r.x1 << 16) | (r.y1 << 24); // non-zero: x1 > x0 >= 0
            ++mine;
        }
    }
    uint32_t incl = mine;
#pragma unroll
    for (uint32_t off = 1; off < 64; off <<= 1) {
        const uint32_t up = (uint32_t)__shfl_up((int)incl, off, 64);
        if (lane >= off)
            incl += up;
    }
    if (lane == 63)
        wave_total[wv] = incl;
    __syncthreads(); // also: the histograms are zeroed
    uint32_t block_total = 0;
#pragma unroll
    for (uint32_t k = 0; k < kWaves; ++k)
        block_total += wave_total[k];
    if (wv == 0 && lane == 0)
        lb_publish(status + blockIdx.x, blockIdx.x == 0 ? kLbPrefix : kLbAggregate, block_total);
    // the byte histograms do not depend on where the keys go: counted while the look-back waits
#pragma unroll
    for (uint32_t k = 0; k < 4; ++k)
#pragma unroll
        for (uint32_t b = 0; b < 4; ++b)
            wave_hist_add(lh[b], (lo[k] >> (8u * b)) & 255u, hi[k] != 0u);
    if (wv == 0) {
        const uint32_t before = lb_exclusive_wave(status, blockIdx.x, error, spin_limit);
        if (lane == 0) {
            if (blockIdx.x != 0)
                lb_publish(status + blockIdx.x, kLbPrefix, before + block_total);
            if (blockIdx.x == gridDim.x - 1)
                counts[2] = (int64_t)(before + block_total); // Gaussians that touch a tile
            base_s = before;
        }
    }
    __syncthreads();
    uint32_t pos = base_s + incl - mine;
#pragma unroll
    for (uint32_t k = 0; k < kWaves; ++k)
        pos += k < wv ? wave_total[k] : 0u;
#pragma unroll
    for (uint32_t k = 0; k < 4; ++k)
        if (hi[k] != 0u) {
            keys[pos] = (int64_t)(((uint64_t)hi[k] << 32) | lo[k]);
            vals[pos] = (int32_t)(blockIdx.x * kKeysPerBlock + t * 4u + k);
            rects[pos] = hi[k]; // a copy the sort does not move: the tile table is formed beside the sort
            ++pos;
        }
    // (the barrier behind the look-back also orders every wave's histogram additions before this read)
    const uint32_t hv = lh[t >> 8][t & 255u];
    if (hv != 0u)
        atomicAdd(&depth_hist[(blockIdx.x % kHistReplicas) * 1024u + t], hv);
}

// Up to kTableBlocks workgroups of 1024 lanes.  Every workgroup counts the rectangle corners (+1 / -1) of its share of the
// keys into a private grid (LDS; a shared grid in global memory when the grid is too large for that) and leaves
// it in `replicas`; the last one to finish adds the replicas up and turns the corner counts into per-tile counts
// (2-D inclusive prefix sum), tile_offsets [n_tiles + 1] (exclusive prefix in row-major tile order, the count in the
// last entry), counts[0] = the count the launches behind this one use (0 when it exceeds the capacity), counts[1] =
// the true count.
template <bool in_lds>
__global__ void __launch_bounds__(1024) tile_table_kernel(
    const uint32_t* __restrict__ rects, uint32_t tile_width, uint32_t tile_height,
    int32_t* __restrict__ replicas /*[kTableBlocks][cells], or [cells] zeroed when !in_lds*/,
    uint32_t* __restrict__ done_counter, int64_t capacity, int32_t* __restrict__ tile_offsets,
    int64_t* __restrict__ counts, int64_t* host_slot, uint32_t* __restrict__ error) {
    extern __shared__ int32_t lds_grid[];
    __shared__ unsigned long long wave_tot[16];
    __shared__ uint32_t last_s;
    const uint32_t t = threadIdx.x, lane = t & 63u, wv = t >> 6;
    const uint32_t gw = tile_width + 1u, gh = tile_height + 1u, n_tiles = tile_width * tile_height;
    const uint32_t cells = gw * gh;
    // the grid is named by its address space so that the LDS instance counts with LDS instructions
#define GSX_GRID(i) (*(in_lds ? &lds_grid[i] : &replicas[i]))
    if (in_lds) {
        for (uint32_t i = t; i < cells; i += 1024u)
            GSX_GRID(i) = 0;
        __syncthreads();
    }
    const uint32_t n = (uint32_t)counts[2];
    for (uint32_t i0 = blockIdx.x * 1024u + t; i0 < n; i0 += gridDim.x * 8192u) {
        uint32_t hi8[8]; // eight keys requested together: every one comes from memory
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
            const uint32_t i = i0 + j * gridDim.x * 1024u;
            hi8[j] = i < n ? rects[i] : 0u;
        }
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
            const uint32_t hi = hi8[j];
            if (hi == 0u)
                continue; // no key: a rectangle has x1 > 0
            const uint32_t x0 = hi & 255u, y0 = (hi >> 8) & 255u, x1 = (hi >> 16) & 255u, y1 = hi >> 24;
            if (in_lds) {
                atomicAdd(&lds_grid[y0 * gw + x0], 1);
                atomicAdd(&lds_grid[y0 * gw + x1], -1);
                atomicAdd(&lds_grid[y1 * gw + x0], -1);
                atomicAdd(&lds_grid[y1 * gw + x1], 1);
            } else {
                atomicAdd(&replicas[y0 * gw + x0], 1);
                atomicAdd(&replicas[y0 * gw + x1], -1);
                atomicAdd(&replicas[y1 * gw + x0], -1);
                atomicAdd(&replicas[y1 * gw + x1], 1);
            }
        }
    }
    __syncthreads();
    // (a shared grid in global memory: its cells are only ever touched by device-scope atomics and, below, read by
    // the last workgroup with device-scope loads)
    // The replicas cross between workgroups (and XCDs) through device-scope stores and loads of the words
    // themselves; a fence here would write back and invalidate this XCD's whole L2, dirty with the sort's keys.
    if (in_lds && gridDim.x > 1)
        for (uint32_t i = t; i < cells; i += 1024u)
            __hip_atomic_store(&replicas[(size_t)blockIdx.x * cells + i], GSX_GRID(i), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    // The election below must not overtake the replicas: every lane waits for its own stores to be acknowledged
    // (vmcnt(0): they are device-scope stores, acknowledged by the level the other XCDs read) before the barrier
    // lets thread 0 add to the counter.  The workgroup that finds the counter complete therefore sees every replica.
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
    __syncthreads();
    if (t == 0)
        last_s = atomicAdd(done_counter, 1u) == gridDim.x - 1u ? 1u : 0u;
    __syncthreads();
    if (!last_s)
        return;
    if (t == 0)
        *done_counter = 0u;
    if (in_lds && gridDim.x > 1) {
        for (uint32_t i = t; i < cells; i += 1024u) {
            int32_t sum = 0;
            for (uint32_t r0 = 0; r0 < gridDim.x; r0 += 8u) { // eight loads in flight, then their sum
                int32_t v[8];
#pragma unroll
                for (uint32_t j = 0; j < 8; ++j)
                    v[j] = r0 + j < gridDim.x ? __hip_atomic_load(&replicas[(size_t)(r0 + j) * cells + i],
                                                                  __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                              : 0;
#pragma unroll
                for (uint32_t j = 0; j < 8; ++j)
                    sum += v[j];
            }
            GSX_GRID(i) = sum;
        }
        __syncthreads();
    }
    // rows (a wave per row, 64 entries at a time), then columns (a lane per column)
    for (uint32_t y = wv; y < gh; y += 16u) {
        int32_t carry = 0;
        for (uint32_t xb = 0; xb < gw; xb += 64u) {
            const uint32_t x = xb + lane;
            int32_t v = 0;
            if (x < gw)
                v = in_lds ? lds_grid[y * gw + x]
                           : __hip_atomic_load(&replicas[y * gw + x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (uint32_t off = 1; off < 64; off <<= 1) {
                const int32_t up = __shfl_up(v, off, 64);
                if (lane >= off)
                    v += up;
            }
            v += carry;
            if (x < gw)
                GSX_GRID(y * gw + x) = v;
            carry = __shfl(v, 63, 64);
        }
    }
    __syncthreads();
    for (uint32_t x = t; x < tile_width; x += 1024u) { // in place: cell (y, x) becomes the length of tile (y, x)'s list
        int32_t run = 0;
#pragma unroll 8
        for (uint32_t y = 0; y < tile_height; ++y) {
            run += GSX_GRID(y * gw + x);
            GSX_GRID(y * gw + x) = run;
        }
    }
    __syncthreads();
    auto tile_count = [&](uint32_t i) { return (uint32_t)GSX_GRID((i / tile_width) * gw + i % tile_width); };
    // exclusive prefix over the tiles: a contiguous chunk per lane
    const uint32_t chunk = (n_tiles + 1023u) / 1024u;
    const uint32_t first = min(t * chunk, n_tiles), last = min(first + chunk, n_tiles);
    unsigned long long mine = 0;
    for (uint32_t i = first; i < last; ++i)
        mine += tile_count(i);
    unsigned long long incl = mine;
#pragma unroll
    for (uint32_t off = 1; off < 64; off <<= 1) {
        const unsigned long long up = __shfl_up(incl, off, 64);
        if (lane >= off)
            incl += up;
    }
    if (lane == 63)
        wave_tot[wv] = incl;
    __syncthreads();
    unsigned long long before = 0, total = 0;
#pragma unroll
    for (uint32_t k = 0; k < 16; ++k) {
        before += k < wv ? wave_tot[k] : 0ull;
        total += wave_tot[k];
    }
    const bool fits = total <= (unsigned long long)capacity && total <= (unsigned long long)kLbValueMask;
    unsigned long long run = before + incl - mine;
    for (uint32_t i = first; i < last; ++i) {
        tile_offsets[i] = fits ? (int32_t)run : 0;
        run += tile_count(i);
    }
    __syncthreads();
    if (!in_lds) // the shared grid in global memory is left zeroed for the next call
        for (uint32_t i = t; i < cells; i += 1024u)
            GSX_GRID(i) = 0;
    if (t == 0) {
        tile_offsets[n_tiles] = fits ? (int32_t)total : 0;
        counts[0] = fits ? (int64_t)total : 0;
        counts[1] = (int64_t)total;
        if (!fits)
            atomicOr(error, 1u);
        if (host_slot != nullptr) // pinned host memory: one 8-byte store at system scope
            __hip_atomic_store(host_slot, (int64_t)total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}
#undef GSX_GRID

// Entries (super-tile << 32 | rectangle, id) in depth order from the sorted keys: one per super-tile a Gaussian's
// rectangle meets.  Workgroup p covers sorted positions [1024 p, 1024 p + 1024); its first output position is the
// entry count of all positions in front of it, obtained by a chained look-back over the workgroups' counts.  Inside
// the workgroup a wave flattens the runs of its 64 positions so that consecutive lanes write consecutive entries.
// The launch also counts the entries per super-tile (the digit totals of the pass behind it).
__global__ void __launch_bounds__(kEmitThreads) super_emit_kernel(
    const int64_t* __restrict__ sorted_keys, const int32_t* __restrict__ order, uint32_t sx_shift, uint32_t sy_shift,
    uint32_t super_width, uint32_t capacity, int64_t* __restrict__ counts, uint32_t* __restrict__ status,
    int64_t* __restrict__ entry_keys, int32_t* __restrict__ entry_ids, uint32_t* __restrict__ super_hist,
    uint32_t* __restrict__ clear_status, uint32_t clear_rows, uint32_t* __restrict__ clear_key_status,
    uint32_t clear_key_words, uint32_t* __restrict__ clear_depth_hist, uint32_t* __restrict__ error,
    uint32_t spin_limit) {
    constexpr uint32_t kWaves = kEmitThreads / 64u;
    __shared__ uint32_t s_incl[kWaves][64], s_hi[kWaves][64], s_idx[kWaves][64];
    __shared__ uint32_t wave_total[kWaves];
    __shared__ uint32_t base_s;
    __shared__ uint32_t sh[256];
    const uint32_t t = threadIdx.x, lane = t & 63u, wv = t >> 6;
    const uint32_t place = blockIdx.x;
    for (uint32_t wd = place * kEmitThreads + t; wd < clear_rows * 256u; wd += gridDim.x * kEmitThreads)
        clear_status[wd] = 0u;
    for (uint32_t wd = place * kEmitThreads + t; wd < clear_key_words; wd += gridDim.x * kEmitThreads)
        clear_key_status[wd] = 0u;
    static_assert(kEmitThreads == 1024, "one histogram word per lane");
    for (uint32_t r = place; r < kHistReplicas; r += gridDim.x)
        clear_depth_hist[r * 1024u + t] = 0u;
    // Nothing here waits for the tile table: entries are written while they fit the buffers (an entry stands for at
    // least one pair, so they all do when the pairs do; when the pairs do not, the gather leaves every list empty).
    const uint32_t limit = capacity;
    const uint32_t n = (uint32_t)counts[2]; // Gaussians that touch a tile
    if (place * kEmitThreads >= n) {
        if (place == 0 && t == 0)
            counts[3] = 0; // no entries (every later workgroup returns as well)
        return; // nobody behind this workgroup needs its (empty) contribution
    }
    if (t < 256)
        sh[t] = 0u;
    const uint32_t i = place * kEmitThreads + t;
    uint32_t hi = 0, cnt = 0, idx = 0;
    if (i < n) {
        hi = (uint32_t)((uint64_t)sorted_keys[i] >> 32);
        const uint32_t X0 = (hi & 255u) >> sx_shift, X1 = ((((hi >> 16) & 255u) - 1u) >> sx_shift) + 1u;
        const uint32_t Y0 = ((hi >> 8) & 255u) >> sy_shift, Y1 = (((hi >> 24) - 1u) >> sy_shift) + 1u;
        cnt = (X1 - X0) * (Y1 - Y0);
        idx = (uint32_t)order[i];
    }
    uint32_t incl = cnt;
#pragma unroll
    for (uint32_t off = 1; off < 64; off <<= 1) {
        const uint32_t up = (uint32_t)__shfl_up((int)incl, off, 64);
        if (lane >= off)
            incl += up;
    }
    s_incl[wv][lane] = incl;
    s_hi[wv][lane] = hi;
    s_idx[wv][lane] = idx;
    if (lane == 63)
        wave_total[wv] = incl;
    __syncthreads();
    uint32_t block_total = 0;
#pragma unroll
    for (uint32_t k = 0; k < kWaves; ++k)
        block_total += wave_total[k];
    if (wv == 0) {
        if (lane == 0)
            lb_publish(status + place, place == 0 ? kLbPrefix : kLbAggregate, block_total);
        const uint32_t before = lb_exclusive_wave(status, place, error, spin_limit);
        if (lane == 0) {
            // (saturating: counts beyond 2^30 - 1 cannot fit any buffer, and must not reach the state bits)
            if (place != 0)
                lb_publish(status + place, kLbPrefix, min(before + block_total, kLbValueMask));
            if ((place + 1u) * kEmitThreads >= n)
                counts[3] = (int64_t)(before + block_total); // entries there are
            base_s = before;
        }
    }
    __syncthreads();
    uint32_t wave_base = base_s;
#pragma unroll
    for (uint32_t k = 0; k < kWaves; ++k)
        wave_base += k < wv ? wave_total[k] : 0u;
    const uint32_t total = wave_total[wv];
    for (uint32_t k = lane; k < total; k += 64u) {
        uint32_t lo = 0, up = 63; // smallest l with incl[l] > k
#pragma unroll
        for (uint32_t step = 0; step < 6; ++step) {
            const uint32_t mid = (lo + up) >> 1;
            if (s_incl[wv][mid] > k)
                up = mid;
            else
                lo = mid + 1;
        }
        const uint32_t l = lo;
        const uint32_t local = k - (l ? s_incl[wv][l - 1] : 0u);
        const uint32_t h = s_hi[wv][l];
        const uint32_t X0 = (h & 255u) >> sx_shift, X1 = ((((h >> 16) & 255u) - 1u) >> sx_shift) + 1u;
        const uint32_t Y0 = ((h >> 8) & 255u) >> sy_shift;
        const uint32_t gw = X1 - X0;
        const uint32_t row = local / gw;
        const uint32_t super_id = (Y0 + row) * super_width + X0 + (local - row * gw);
        const uint32_t pos = wave_base + k;
        if (pos < limit) {
            entry_keys[pos] = (int64_t)(((uint64_t)super_id << 32) | h);
            entry_ids[pos] = (int32_t)s_idx[wv][l];
        }
        atomicAdd(&sh[super_id & 255u], 1u);
    }
    __syncthreads();
    if (t < 256 && sh[t] != 0u)
        atomicAdd(&super_hist[(place % kHistReplicas) * 256u + t], sh[t]);
}

// flatten_ids from the entries grouped by super-tile.  A workgroup takes one SLICE: up to kSliceEntries consecutive
// entries of one super-tile.  Staging a slice in LDS turns every entry's rectangle into a bit mask over the tiles of
// the super-tile (bit l = tile l, row-major inside the super-tile; WORDS x 32 bits); whether an entry belongs to a
// tile is then one bit test, and 64 entries are tested with two vector instructions.  The 16 waves share the
// super-tile's tiles; for a tile a wave walks the slice 64 entries at a time - once to count the entries of the tile,
// once to write them.  Between the two, the slice's per-tile counts are chained to those of the slices in front of
// it within the super-tile by a look-back over one status row per slice (a column per tile; the first slice of a
// super-tile publishes a complete prefix, which ends the walk): the k-th entry of tile T in this slice goes to
// flatten_ids[tile_offsets[T] + entries of T in earlier slices + k].  Every list is written front to back in depth
// order; no (tile, id) pair is formed or sorted.
template <uint32_t WORDS>
__global__ void __launch_bounds__(1024) tile_gather_kernel(
    const int64_t* __restrict__ entry_keys, const int32_t* __restrict__ entry_ids,
    const uint32_t* __restrict__ super_hist, const int64_t* __restrict__ counts,
    const int32_t* __restrict__ tile_offsets, uint32_t tile_width, uint32_t tile_height, uint32_t sx_shift,
    uint32_t sy_shift, uint32_t super_width, uint32_t n_super, uint32_t* __restrict__ status,
    uint32_t* __restrict__ error, uint32_t spin_limit, int32_t* __restrict__ flatten_ids) {
    constexpr uint32_t kTilesPerWave = WORDS * 2u;       // 32 WORDS tiles over 16 waves
    constexpr uint32_t kSlice = kSliceEntries;
    __shared__ uint32_t s_mask[WORDS][kSlice];
    __shared__ int32_t s_id[kSlice];
    __shared__ uint32_t seg_start[256], seg_len[256], slice_start[256];
    __shared__ uint32_t wave_a[4], wave_b[4];
    __shared__ uint32_t cnt[WORDS * 32u], base[WORDS * 32u];
    const uint32_t t = threadIdx.x, lane = t & 63u, wv = t >> 6;
    const uint32_t place = blockIdx.x;
    // counts[0] == 0: the pairs do not fit their buffer and every list stays empty.  Beyond the last slice there can
    // be (entries / slice + one partial slice per super-tile): nothing to do
    if (counts[0] == 0 || place >= (uint32_t)counts[3] / kSlice + n_super)
        return;
    // entries and slices in front of every super-tile (exclusive prefix sums over at most 256 counts)
    uint32_t len = 0, nsl = 0, in_len = 0, in_nsl = 0;
    if (t < 256) {
        if (t < n_super)
#pragma unroll
            for (uint32_t r = 0; r < kHistReplicas; ++r)
                len += super_hist[r * 256u + t];
        nsl = (len + kSlice - 1u) / kSlice;
        in_len = len, in_nsl = nsl;
#pragma unroll
        for (uint32_t off = 1; off < 64; off <<= 1) {
            const uint32_t ua = (uint32_t)__shfl_up((int)in_len, off, 64), ub = (uint32_t)__shfl_up((int)in_nsl, off, 64);
            if (lane >= off) {
                in_len += ua;
                in_nsl += ub;
            }
        }
        if (lane == 63) {
            wave_a[wv] = in_len;
            wave_b[wv] = in_nsl;
        }
    }
    __syncthreads();
    if (t < 256) {
        uint32_t ba = 0, bb = 0;
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            ba += k < wv ? wave_a[k] : 0u;
            bb += k < wv ? wave_b[k] : 0u;
        }
        seg_start[t] = ba + in_len - len;
        seg_len[t] = len;
        slice_start[t] = bb + in_nsl - nsl;
    }
    __syncthreads();
    if (place >= wave_b[0] + wave_b[1] + wave_b[2] + wave_b[3])
        return;
    // the super-tile of this slice: the last one whose first slice is not behind `place`
    uint32_t lo = 0, hi = 255;
#pragma unroll
    for (uint32_t step = 0; step < 8; ++step) {
        const uint32_t mid = (lo + hi + 1u) >> 1;
        if (slice_start[mid] <= place)
            lo = mid;
        else
            hi = mid - 1u;
    }
    const uint32_t sup = lo, k_slice = place - slice_start[sup];
    const uint32_t a = seg_start[sup] + k_slice * kSlice;
    const uint32_t n_here = min(kSlice, seg_start[sup] + seg_len[sup] - a);
    const uint32_t tx0 = (sup % super_width) << sx_shift, ty0 = (sup / super_width) << sy_shift;
    const uint32_t sx = 1u << sx_shift, sy = 1u << sy_shift;
    const uint32_t rows_per_word = 32u >> sx_shift;
#pragma unroll
    for (uint32_t k = 0; k < kSlice / 1024u; ++k) {
        const uint32_t j = k * 1024u + t;
        uint32_t m[WORDS];
#pragma unroll
        for (uint32_t w = 0; w < WORDS; ++w)
            m[w] = 0u;
        int32_t id = 0;
        if (j < n_here) {
            const uint32_t r = (uint32_t)(uint64_t)entry_keys[a + j];
            id = entry_ids[a + j];
            // the rectangle inside this super-tile, in its own tile coordinates
            const uint32_t x0 = max(r & 255u, tx0) - tx0, x1 = min((r >> 16) & 255u, tx0 + sx) - tx0;
            const uint32_t y0 = max((r >> 8) & 255u, ty0) - ty0, y1 = min(r >> 24, ty0 + sy) - ty0;
            const uint32_t row_bits = (1u << x1) - (1u << x0);
#pragma unroll
            for (uint32_t w = 0; w < WORDS; ++w)
                for (uint32_t q = 0; q < rows_per_word; ++q) {
                    const uint32_t row = w * rows_per_word + q;
                    if (row >= y0 && row < y1)
                        m[w] |= row_bits << (q << sx_shift);
                }
        }
#pragma unroll
        for (uint32_t w = 0; w < WORDS; ++w)
            s_mask[w][j] = m[w]; // zero beyond the slice's end: no entry
        s_id[j] = id;
    }
    const uint64_t below = (1ull << lane) - 1ull;
    __syncthreads();
    // tiles wv, wv + 16, ... of the super-tile: tile wv + 16 i is bit (wv + 16 (i & 1)) of word i / 2
    uint32_t c[kTilesPerWave];
#pragma unroll
    for (uint32_t i = 0; i < kTilesPerWave; ++i)
        c[i] = 0u;
    const uint32_t bit0 = 1u << wv, bit1 = 1u << (wv + 16u);
    const uint32_t groups = (n_here + 63u) / 64u;
    for (uint32_t g = 0; g < groups; ++g) {
        uint32_t m[WORDS];
#pragma unroll
        for (uint32_t w = 0; w < WORDS; ++w)
            m[w] = s_mask[w][g * 64u + lane];
#pragma unroll
        for (uint32_t i = 0; i < kTilesPerWave; ++i)
            c[i] += (uint32_t)__popcll(__ballot((m[i >> 1] & ((i & 1u) ? bit1 : bit0)) != 0u));
    }
    if (lane == 0)
#pragma unroll
        for (uint32_t i = 0; i < kTilesPerWave; ++i)
            cnt[wv + 16u * i] = c[i];
    __syncthreads();
    if (t < WORDS * 32u) {
        const uint32_t mine = cnt[t];
        uint32_t before = 0;
        const uint32_t tx = tx0 + (t & (sx - 1u)), ty = ty0 + (t >> sx_shift);
        const bool on_grid = (t >> sx_shift) < sy && tx < tile_width && ty < tile_height;
        const uint32_t offset = on_grid ? (uint32_t)tile_offsets[ty * tile_width + tx] : 0u;
        if (k_slice == 0) {
            lb_publish(status + (size_t)place * 256u + t, kLbPrefix, mine);
        } else {
            lb_publish(status + (size_t)place * 256u + t, kLbAggregate, mine);
            before = lb_exclusive(status, place, 256u, t, error, spin_limit);
            lb_publish(status + (size_t)place * 256u + t, kLbPrefix, before + mine);
        }
        base[t] = before + offset;
    }
    __syncthreads();
    uint32_t at[kTilesPerWave];
#pragma unroll
    for (uint32_t i = 0; i < kTilesPerWave; ++i)
        at[i] = base[wv + 16u * i];
    for (uint32_t g = 0; g < groups; ++g) {
        uint32_t m[WORDS];
#pragma unroll
        for (uint32_t w = 0; w < WORDS; ++w)
            m[w] = s_mask[w][g * 64u + lane];
        const int32_t id = s_id[g * 64u + lane];
#pragma unroll
        for (uint32_t i = 0; i < kTilesPerWave; ++i) {
            const bool in = (m[i >> 1] & ((i & 1u) ? bit1 : bit0)) != 0u;
            const uint64_t mask = __ballot(in);
            // (a position is the tile's offset + entries in front: below the pair count, which fits the buffer)
            if (in)
                flatten_ids[at[i] + (uint32_t)__popcll(mask & below)] = id;
            at[i] += (uint32_t)__popcll(mask);
        }
    }
}

__global__ void __launch_bounds__(256) zero_words_kernel(size_t n, uint32_t* __restrict__ out) {
    const size_t i = (size_t)blockIdx.x * 256u + threadIdx.x;
    if (i < n)
        out[i] = 0u;
}

} // namespace gsx

using namespace gsx;

namespace {
struct ListsLayout {
    // zeroed by gsx_tile_lists_init and left zero by every call: the head of the workspace
    size_t depth_hist, super_hist, counts, error, done_counter, kstatus, shared_grid, head_end;
    size_t keys0, keys1, vals0, vals1, rects; // depth sort: i64 [N] x 2, i32 [N] x 2; u32 [N]
    size_t replicas;
    size_t dstatus0, dstatus1, estatus, pstatus, gstatus;
    uint32_t grows; // status rows of the gather: one per slice there can be
    size_t ekeys0, ekeys1, eids0, eids1; // entries: i64 [capacity] x 2, i32 [capacity] x 2
    size_t total;
    uint32_t kblocks, drows, prows, ewords, cells, table_blocks;
    uint32_t sx_shift, sy_shift, super_width, n_super, parts; // super-tiles of (1 << sx_shift) x (1 << sy_shift) tiles
    bool grid_in_lds;
};
ListsLayout lists_layout(uint32_t N, int64_t capacity, uint32_t tw, uint32_t th) {
    ListsLayout L;
    size_t o = 0;
    auto take = [&](size_t bytes) {
        const size_t at = o;
        o += align_up(bytes, 256);
        return at;
    };
    L.kblocks = cdiv(N, kKeysPerBlock);
    L.drows = radix_chained_rows(N);
    L.prows = radix_chained_rows(capacity);
    L.ewords = cdiv(N, kEmitThreads);
    L.cells = (tw + 1) * (th + 1);
    L.grid_in_lds = L.cells <= kMaxLdsCells;
    L.table_blocks = std::min(kTableBlocks, std::max(1u, N / (128u * 1024u)));
    // the smallest super-tiles of which the grid holds at most 256 (one byte of the entry keys names them)
    static const uint32_t shapes[5][2] = {{2, 2}, {3, 2}, {3, 3}, {4, 3}, {4, 4}};
    for (const auto& sh : shapes) {
        L.sx_shift = sh[0], L.sy_shift = sh[1];
        L.super_width = cdiv(tw, 1u << L.sx_shift);
        L.n_super = L.super_width * cdiv(th, 1u << L.sy_shift);
        if (L.n_super <= 256u)
            break;
    }
    L.parts = (1u << (L.sx_shift + L.sy_shift)) / 16u;
    L.depth_hist = take((size_t)kHistReplicas * 4 * 256 * 4);
    L.super_hist = take((size_t)kHistReplicas * 256 * 4);
    L.counts = take(4 * 8);
    L.error = take(2 * 4);
    L.done_counter = take(4);
    L.kstatus = take((size_t)L.kblocks * 4);
    L.shared_grid = take(L.grid_in_lds ? 0 : (size_t)L.cells * 4);
    L.head_end = o;
    L.replicas = take(L.grid_in_lds ? (size_t)kTableBlocks * L.cells * 4 : 0);
    L.keys0 = take((size_t)N * 8);
    L.keys1 = take((size_t)N * 8);
    L.vals0 = take((size_t)N * 4);
    L.vals1 = take((size_t)N * 4);
    L.rects = take((size_t)N * 4);
    L.dstatus0 = take((size_t)L.drows * 1024);
    L.dstatus1 = take((size_t)L.drows * 1024);
    L.estatus = take((size_t)L.ewords * 4);
    L.pstatus = take((size_t)L.prows * 1024);
    L.grows = (uint32_t)cdiv((uint64_t)capacity, kSliceEntries) + L.n_super;
    L.gstatus = take((size_t)L.grows * 1024);
    // an entry stands for at least one (tile, Gaussian) pair: entries that exceed the pair capacity cannot occur
    // once the pairs fit
    L.ekeys0 = take((size_t)capacity * 8);
    L.ekeys1 = take((size_t)capacity * 8);
    L.eids0 = take((size_t)capacity * 4);
    L.eids1 = take((size_t)capacity * 4);
    L.total = o;
    return L;
}
// two events per (device, stream) for the fork / join with a caller's second stream (created once, never destroyed):
// calls on different streams - other workspaces, other host threads - do not share them
struct SideEvents {
    int device;
    void* stream;
    hipEvent_t keys_done, table_done;
};
int side_events(void* stream, SideEvents** out) {
    static std::mutex mutex;
    static std::vector<SideEvents*> known;
    int dev = -1;
    GSX_HIP_CHECK(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(mutex);
    for (SideEvents* e : known)
        if (e->device == dev && e->stream == stream) {
            *out = e;
            return GSX_OK;
        }
    SideEvents* e = new SideEvents{dev, stream, nullptr, nullptr};
    GSX_HIP_CHECK(hipEventCreateWithFlags(&e->keys_done, hipEventDisableTiming));
    GSX_HIP_CHECK(hipEventCreateWithFlags(&e->table_done, hipEventDisableTiming));
    known.push_back(e);
    *out = e;
    return GSX_OK;
}
int check_lists_args(const char* who, uint32_t N, int64_t capacity, uint32_t tw, uint32_t th) {
    GSX_REQUIRE(tw >= 1 && th >= 1 && tw <= 255 && th <= 255, GSX_ERR_UNSUPPORTED,
                "%s: a %u x %u tile grid (limit 255 x 255: the keys carry the tile rectangle in four bytes)", who, tw,
                th);
    GSX_REQUIRE(N >= 1 && N < (1u << kLbValueBits), GSX_ERR_OVERFLOW, "%s: N = %u (limit 2^30 - 1)", who, N);
    GSX_REQUIRE(capacity >= 1 && capacity < (1ll << kLbValueBits), GSX_ERR_OVERFLOW,
                "%s: capacity = %lld pairs (limit 2^30 - 1)", who, (long long)capacity);
    return GSX_OK;
}
} // namespace

extern "C" size_t gsx_tile_lists_workspace_bytes(uint32_t N, int64_t capacity, uint32_t tile_width,
                                                 uint32_t tile_height) {
    if (N == 0 || capacity <= 0 || tile_width == 0 || tile_height == 0)
        return 256;
    return lists_layout(N, capacity, tile_width, tile_height).total;
}

// the head of the workspace (digit histogram, counts, error words, look-back words of the first launch, ...) must be
// zero before the first call; every call leaves it as the next one needs it
extern "C" int gsx_tile_lists_init(uint32_t N, int64_t capacity, uint32_t tile_width, uint32_t tile_height,
                                   void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_lists_args("tile_lists_init", N, capacity, tile_width, tile_height);
    if (rc != GSX_OK)
        return rc;
    const ListsLayout L = lists_layout(N, capacity, tile_width, tile_height);
    GSX_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0 && workspace_bytes >= L.total,
                GSX_ERR_WORKSPACE, "tile_lists_init: workspace needs %zu bytes, 256-byte aligned", L.total);
    const size_t words = L.head_end / 4;
    hipLaunchKernelGGL(zero_words_kernel, dim3(cdiv(words, 256)), dim3(256), 0, (hipStream_t)stream, words,
                       (uint32_t*)workspace);
    GSX_LAUNCH_CHECK();
    // the gather's status rows: a call clears the rows the call before it used, so all of them start out zero
    const size_t gwords = (size_t)L.grows * 256;
    hipLaunchKernelGGL(zero_words_kernel, dim3(cdiv(gwords, 256)), dim3(256), 0, (hipStream_t)stream, gwords,
                       (uint32_t*)((char*)workspace + L.gstatus));
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_tile_lists(uint32_t N, const float* means2d, const int32_t* radii, const float* depths,
                              uint32_t tile_size, uint32_t tile_width, uint32_t tile_height, int64_t capacity,
                              void* workspace, size_t workspace_bytes, int32_t* flatten_ids, int32_t* tile_offsets,
                              int64_t* n_isects_host_slot, void* stream, void* side_stream) {
    int rc = check_lists_args("tile_lists", N, capacity, tile_width, tile_height);
    if (rc != GSX_OK)
        return rc;
    GSX_REQUIRE(means2d && radii && depths && flatten_ids && tile_offsets, GSX_ERR_INVALID_ARGUMENT,
                "tile_lists: null tensor");
    GSX_REQUIRE(tile_size > 0, GSX_ERR_INVALID_ARGUMENT, "tile_lists: tile_size is 0");
    GSX_REQUIRE(((((uintptr_t)means2d) | ((uintptr_t)radii) | ((uintptr_t)depths)) & 15u) == 0, GSX_ERR_INVALID_ARGUMENT,
                "tile_lists: means2d / radii / depths need 16-byte alignment");
    const ListsLayout L = lists_layout(N, capacity, tile_width, tile_height);
    GSX_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0 && workspace_bytes >= L.total,
                GSX_ERR_WORKSPACE, "tile_lists: workspace needs %zu bytes, 256-byte aligned", L.total);
    int64_t* slot = nullptr;
    if (n_isects_host_slot != nullptr) {
        hipPointerAttribute_t attr;
        const bool known = hipPointerGetAttributes(&attr, n_isects_host_slot) == hipSuccess;
        if (!known)
            (void)hipGetLastError();
        GSX_REQUIRE(known && attr.type == hipMemoryTypeHost && attr.devicePointer != nullptr, GSX_ERR_INVALID_ARGUMENT,
                    "tile_lists: n_isects_host_slot must be pinned host memory (hipHostMalloc)");
        slot = (int64_t*)attr.devicePointer;
    }
    const size_t table_lds = L.grid_in_lds ? (size_t)L.cells * 4 : 0;
    if (table_lds > 48 * 1024) { // beyond the default limit of dynamically sized LDS
        static bool raised = false; // per process; the attribute is idempotent
        if (!raised) {
            GSX_HIP_CHECK(hipFuncSetAttribute((const void*)tile_table_kernel<true>,
                                              hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLdsCells * 4));
            raised = true;
        }
    }
    char* ws = (char*)workspace;
    auto u32p = [&](size_t off) { return (uint32_t*)(ws + off); };
    int64_t* keys[2] = {(int64_t*)(ws + L.keys0), (int64_t*)(ws + L.keys1)};
    int32_t* vals[2] = {(int32_t*)(ws + L.vals0), (int32_t*)(ws + L.vals1)};
    uint32_t* dstatus[2] = {u32p(L.dstatus0), u32p(L.dstatus1)};
    uint32_t* error = u32p(L.error);
    int64_t* counts = (int64_t*)(ws + L.counts);
    hipStream_t s = (hipStream_t)stream;
    const uint32_t spin_limit = lookback_spin_limit();

    hipLaunchKernelGGL(depth_keys_kernel, dim3(L.kblocks), dim3(kKeysThreads), 0, s, N, means2d, radii, depths,
                       (float)tile_size, tile_width, tile_height, keys[0], vals[0], u32p(L.rects), u32p(L.kstatus),
                       counts, error, dstatus[0], L.drows, u32p(L.estatus), L.ewords, u32p(L.super_hist),
                       u32p(L.gstatus), L.grows, L.n_super, u32p(L.depth_hist), spin_limit);
    GSX_LAUNCH_CHECK();
    // The tile table needs the rectangles only, not their depth order: with a second stream it is formed while the
    // sort runs.
    hipStream_t ts = side_stream != nullptr && side_stream != stream ? (hipStream_t)side_stream : s;
    SideEvents* ev = nullptr;
    if (ts != s) {
        if ((rc = side_events(stream, &ev)) != GSX_OK)
            return rc;
        GSX_HIP_CHECK(hipEventRecord(ev->keys_done, s));
        GSX_HIP_CHECK(hipStreamWaitEvent(ts, ev->keys_done, 0));
    }
    if (L.grid_in_lds)
        hipLaunchKernelGGL(tile_table_kernel<true>, dim3(L.table_blocks), dim3(1024), table_lds, ts, u32p(L.rects),
                           tile_width, tile_height, (int32_t*)(ws + L.replicas), u32p(L.done_counter), capacity,
                           tile_offsets, counts, slot, error);
    else
        hipLaunchKernelGGL(tile_table_kernel<false>, dim3(L.table_blocks), dim3(1024), 0, ts, u32p(L.rects),
                           tile_width, tile_height, (int32_t*)(ws + L.shared_grid), u32p(L.done_counter), capacity,
                           tile_offsets, counts, slot, error);
    GSX_LAUNCH_CHECK();
    if (ts != s)
        GSX_HIP_CHECK(hipEventRecord(ev->table_done, ts));
    for (uint32_t pass = 0; pass < 4; ++pass) { // depth bits, a byte per pass; the result ends in keys[0] / vals[0]
        const uint32_t in = pass & 1u, out = in ^ 1u;
        RadixChainArgs a;
        a.n_dev = counts + 2, a.status = dstatus[in], a.error = error;
        a.total_replicas = kHistReplicas, a.total_stride = 1024;
        a.clear_status = pass < 3 ? dstatus[out] : nullptr, a.clear_rows = L.drows;
        if ((rc = radix_chained_pass_i64(N, keys[in], vals[in], keys[out], vals[out], 8u * pass, 8u,
                                         u32p(L.depth_hist) + 256u * pass, a, s)) != GSX_OK)
            return rc;
    }
    int64_t* ekeys[2] = {(int64_t*)(ws + L.ekeys0), (int64_t*)(ws + L.ekeys1)};
    int32_t* eids[2] = {(int32_t*)(ws + L.eids0), (int32_t*)(ws + L.eids1)};
    hipLaunchKernelGGL(super_emit_kernel, dim3(L.ewords), dim3(kEmitThreads), 0, s, keys[0], vals[0], L.sx_shift,
                       L.sy_shift, L.super_width, (uint32_t)capacity, counts, u32p(L.estatus), ekeys[0], eids[0],
                       u32p(L.super_hist),
                       u32p(L.pstatus), L.prows, u32p(L.kstatus), L.kblocks, u32p(L.depth_hist), error, spin_limit);
    GSX_LAUNCH_CHECK();
    {
        RadixChainArgs a;
        a.n_dev = counts + 3, a.status = u32p(L.pstatus), a.error = error;
        a.total_replicas = kHistReplicas, a.total_stride = 256;
        a.clear_status = nullptr, a.clear_rows = 0;
        if ((rc = radix_chained_pass_i64((uint32_t)capacity, ekeys[0], eids[0], ekeys[1], eids[1], 32u, 8u,
                                         u32p(L.super_hist), a, s)) != GSX_OK)
            return rc;
    }
    if (ts != s) // the gather is the first launch that needs the tile table (tile_offsets, the fit decision)
        GSX_HIP_CHECK(hipStreamWaitEvent(s, ev->table_done, 0));
    // the coverage masks have one bit per tile of a super-tile: 1, 2, 4 or 8 words of 32
    const uint32_t mask_words = std::max(1u, (1u << (L.sx_shift + L.sy_shift)) / 32u);
    auto gather = mask_words == 1   ? tile_gather_kernel<1>
                  : mask_words == 2 ? tile_gather_kernel<2>
                  : mask_words == 4 ? tile_gather_kernel<4>
                                    : tile_gather_kernel<8>;
    hipLaunchKernelGGL(gather, dim3(L.grows), dim3(1024), 0, s, ekeys[1], eids[1], u32p(L.super_hist), counts,
                       tile_offsets, tile_width, tile_height, L.sx_shift, L.sy_shift, L.super_width, L.n_super,
                       u32p(L.gstatus), error, spin_limit, flatten_ids);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

// where a caller can read the outcome of the last call on the device: counts[0] = pairs in the lists (0 if they did
// not fit), counts[1] = pairs there are, counts[2] = Gaussians that touch a tile, counts[3] = (super-tile, Gaussian)
// entries; error[0]: bit 0 = capacity
// exceeded, bit 1 = a look-back gave up; error[1]: free for the caller (gsx_update_args.hold counts there)
extern "C" const int64_t* gsx_tile_lists_counts(uint32_t N, int64_t capacity, uint32_t tile_width,
                                                uint32_t tile_height, const void* workspace) {
    if (workspace == nullptr || N == 0 || capacity <= 0)
        return nullptr;
    return (const int64_t*)((const char*)workspace + lists_layout(N, capacity, tile_width, tile_height).counts);
}
extern "C" uint32_t* gsx_tile_lists_error(uint32_t N, int64_t capacity, uint32_t tile_width, uint32_t tile_height,
                                          void* workspace) {
    if (workspace == nullptr || N == 0 || capacity <= 0)
        return nullptr;
    return (uint32_t*)((char*)workspace + lists_layout(N, capacity, tile_width, tile_height).error);
}
