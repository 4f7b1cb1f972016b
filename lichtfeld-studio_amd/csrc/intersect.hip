// intersect.hip - tile intersection: per-Gaussian tile counts, their prefix sum, key/value emission and the
// per-tile ranges of the sorted keys (gsplat/IntersectTile.cu:23-114, 206-252; gsplat/Intersect.cpp:41-137).
// Integer work: every output is bit-exact given the inputs.
#include "gsx_common.h"
#include "gsx_tiles.h"

namespace gsx {

__global__ void __launch_bounds__(256) tile_count_kernel(uint32_t n, const float* __restrict__ means2d,
                                                          const int32_t* __restrict__ radii, float tile_size,
                                                          uint32_t tile_width, uint32_t tile_height,
                                                          int32_t* __restrict__ tiles_per_gauss) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= n)
        return;
    TileRect r;
    int32_t cnt = 0;
    if (tile_rect(means2d, radii, idx, tile_size, tile_width, tile_height, &r))
        cnt = (int32_t)((r.y1 - r.y0) * (r.x1 - r.x0));
    tiles_per_gauss[idx] = cnt;
}

// A workgroup writes the keys of one block of the sort that follows (256 * items consecutive Gaussians) and leaves
// that block's column of the sort's first histogram table (digit = low byte of the depth bits): the sort starts
// with its scan.
template <bool RECT>
__global__ void __launch_bounds__(256) depth_count_keys_kernel(uint32_t n, const float* __restrict__ means2d,
                                                                const int32_t* __restrict__ radii,
                                                                const float* __restrict__ depths, float tile_size,
                                                                uint32_t tile_width, uint32_t tile_height,
                                                                uint32_t items, uint32_t nblocks,
                                                                int32_t* __restrict__ tiles_per_gauss,
                                                                int64_t* __restrict__ keys,
                                                                int32_t* __restrict__ vals,
                                                                uint32_t* __restrict__ hist /*[256][nblocks]*/) {
    __shared__ uint32_t lh[256];
    lh[threadIdx.x] = 0;
    __syncthreads();
    for (uint32_t k = 0; k < items; ++k) {
        const uint32_t i = (blockIdx.x * items + k) * 256u + threadIdx.x;
        if (i >= n)
            break;
        TileRect r;
        uint32_t cnt = 0;
        if (tile_rect(means2d, radii, i, tile_size, tile_width, tile_height, &r))
            cnt = (r.y1 - r.y0) * (r.x1 - r.x0);
        tiles_per_gauss[i] = (int32_t)cnt;
        const uint32_t lo = cnt ? f2u(depths[i]) : 0xFFFFFFFFu;
        const uint32_t hi = !RECT ? cnt : cnt ? (r.x0 | (r.y0 << 8) | (r.x1 << 16) | (r.y1 << 24)) : 0u;
        keys[i] = (int64_t)(((uint64_t)hi << 32) | lo);
        vals[i] = (int32_t)i;
        atomicAdd(&lh[lo & 255u], 1u);
    }
    __syncthreads();
    hist[threadIdx.x * nblocks + blockIdx.x] = lh[threadIdx.x];
}

// ---- inclusive scan int32 -> int64 (at::cumsum of Intersect.cpp:75) -----------------------------
// per-block sums, then per-block scan + the total of the earlier blocks (summed by each block itself, or for very
// long inputs scanned by one block in a launch of its own)
static constexpr uint32_t kScanItems = 8;
static constexpr uint32_t kScanTile = 256 * kScanItems;

__device__ __forceinline__ int64_t block_exclusive_scan_256(int64_t v, int64_t* lds, int64_t* total) {
    const uint32_t t = threadIdx.x;
    lds[t] = v;
    __syncthreads();
#pragma unroll
    for (uint32_t off = 1; off < 256; off <<= 1) {
        int64_t add = (t >= off) ? lds[t - off] : 0;
        __syncthreads();
        lds[t] += add;
        __syncthreads();
    }
    const int64_t incl = lds[t];
    *total = lds[255];
    __syncthreads();
    return incl - v;
}

// the scan's input: int32 counts, or (keys != nullptr) the high words of 64-bit keys - counts themselves, or
// packed tile rectangles (rect_keys)
__device__ __forceinline__ int32_t scan_input(const int32_t* __restrict__ in, const int64_t* __restrict__ keys,
                                              bool rect_keys, uint32_t i) {
    if (keys == nullptr)
        return in[i];
    const uint32_t hi = (uint32_t)((uint64_t)keys[i] >> 32);
    return (int32_t)(rect_keys ? packed_rect_count(hi) : hi);
}

__global__ void __launch_bounds__(256) scan_block_sums_kernel(uint32_t n, const int32_t* __restrict__ in,
                                                               const int64_t* __restrict__ keys, bool rect_keys,
                                                               int64_t* __restrict__ block_sums) {
    __shared__ int64_t lds[256];
    const uint32_t base = blockIdx.x * kScanTile + threadIdx.x * kScanItems;
    int64_t s = 0;
#pragma unroll
    for (uint32_t i = 0; i < kScanItems; ++i)
        if (base + i < n)
            s += scan_input(in, keys, rect_keys, base + i);
    int64_t total;
    block_exclusive_scan_256(s, lds, &total);
    if (threadIdx.x == 0)
        block_sums[blockIdx.x] = total;
}

// in place: block_sums[b] <- exclusive prefix; *total_out <- grand total
__global__ void __launch_bounds__(256) scan_block_offsets_kernel(uint32_t nb, int64_t* __restrict__ block_sums,
                                                                  int64_t* __restrict__ total_out) {
    __shared__ int64_t lds[256];
    int64_t carry = 0;
    for (uint32_t start = 0; start < nb; start += 256) {
        const uint32_t i = start + threadIdx.x;
        const int64_t v = i < nb ? block_sums[i] : 0;
        int64_t total;
        const int64_t ex = block_exclusive_scan_256(v, lds, &total);
        if (i < nb)
            block_sums[i] = carry + ex;
        carry += total;
    }
    if (threadIdx.x == 0) // total_out may be pinned host memory: one 8-byte store at system scope
        __hip_atomic_store(total_out, carry, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Per-block scan plus the total of the earlier blocks.  SUMS: block_sums holds the blocks' own totals and every block
// adds up the ones in front of it for itself (a few hundred to a few thousand values from L2: cheaper than a launch
// of its own; the last block also leaves the grand total); otherwise it holds the exclusive prefixes already.
template <bool SUMS>
__global__ void __launch_bounds__(256) scan_apply_kernel(uint32_t n, const int32_t* __restrict__ in,
                                                          const int64_t* __restrict__ keys, bool rect_keys,
                                                          const int64_t* __restrict__ block_sums,
                                                          int64_t* __restrict__ out, int64_t* __restrict__ total_out) {
    __shared__ int64_t lds[256];
    const uint32_t base = blockIdx.x * kScanTile + threadIdx.x * kScanItems;
    int32_t v[kScanItems];
    int64_t s = 0;
#pragma unroll
    for (uint32_t i = 0; i < kScanItems; ++i) {
        v[i] = (base + i < n) ? scan_input(in, keys, rect_keys, base + i) : 0;
        s += v[i];
    }
    int64_t offset = 0; // total of the blocks in front of this one
    if (SUMS) {
        int64_t before = 0;
        for (uint32_t b = threadIdx.x; b < blockIdx.x; b += 256)
            before += block_sums[b];
        block_exclusive_scan_256(before, lds, &offset);
    } else {
        offset = block_sums[blockIdx.x];
    }
    int64_t total;
    int64_t run = block_exclusive_scan_256(s, lds, &total) + offset;
#pragma unroll
    for (uint32_t i = 0; i < kScanItems; ++i) {
        run += v[i];
        if (base + i < n)
            out[base + i] = run;
    }
    if (SUMS && blockIdx.x == gridDim.x - 1 && threadIdx.x == 0)
        __hip_atomic_store(total_out, offset + total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// IntersectTile.cu:78-113 second pass: keys and values in emission order (ascending position, row-major tiles
// inside a Gaussian).  The reference lets every thread write its own Gaussian's run, 64 scattered 8-byte stores per
// instruction and a serial loop as long as the largest Gaussian.  Here a wave flattens the runs of its 64
// positions: entry k of the wave's output range belongs to the position whose inclusive count prefix first
// exceeds k (binary search over 64 prefixes in LDS), so the lanes write consecutive entries.
// FROM_KEYS: position i's Gaussian is order[i] and its rectangle and depth bits are the words of sorted_keys[i]
// (depth_count_keys_kernel<true>): sequential reads only, nothing is gathered in sorted order.
// COMPACT (one camera, at most 65 536 tiles): the output key is the 16-bit tile index alone - pairs emitted in depth
// order only ever sort on their tile bits, and the per-tile ranges need nothing else.
template <bool FROM_KEYS, bool COMPACT = false>
__global__ void __launch_bounds__(256) tile_emit_kernel(uint32_t n, uint32_t N, const float* __restrict__ means2d,
                                                         const int32_t* __restrict__ radii,
                                                         const float* __restrict__ depths,
                                                         const int64_t* __restrict__ sorted_keys,
                                                         const int64_t* __restrict__ cum_tiles_per_gauss,
                                                         const int32_t* __restrict__ order, float tile_size,
                                                         uint32_t tile_width, uint32_t tile_height,
                                                         uint32_t tile_n_bits, int64_t capacity,
                                                         int64_t* __restrict__ isect_ids,
                                                         uint16_t* __restrict__ tile_keys /*COMPACT*/,
                                                         int32_t* __restrict__ flatten_ids,
                                                         const int64_t* __restrict__ camera_ids = nullptr) {
    __shared__ uint32_t s_incl[4][64], s_xy[4][64], s_w[4][64], s_idx[4][64], s_lo[COMPACT ? 1 : 4][64],
        s_hi[COMPACT ? 1 : 4][64];
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    const uint32_t lane = threadIdx.x & 63u, wv = threadIdx.x >> 6;
    TileRect r = {0, 0, 0, 0};
    uint32_t idx = 0;
    bool live = false;
    uint32_t depth_bits = 0;
    if (i < n) {
        idx = order != nullptr ? (uint32_t)order[i] : i;
        if (FROM_KEYS) {
            const uint64_t key = (uint64_t)sorted_keys[i];
            const uint32_t hi = (uint32_t)(key >> 32);
            r.x0 = hi & 255u, r.y0 = (hi >> 8) & 255u, r.x1 = (hi >> 16) & 255u, r.y1 = hi >> 24;
            live = hi != 0u;
            depth_bits = (uint32_t)key;
        } else {
            live = tile_rect(means2d, radii, idx, tile_size, tile_width, tile_height, &r);
        }
    }
    const uint32_t w = live ? r.x1 - r.x0 : 0u;
    const uint32_t cnt = live ? (r.y1 - r.y0) * w : 0u;
    int64_t key_base = 0;
    if (cnt) {
        // packed rows name their camera themselves (IntersectTile.cu:86-94)
        const int64_t cid = camera_ids != nullptr ? camera_ids[idx] : (int64_t)(idx / N);
        if (!FROM_KEYS)
            depth_bits = f2u(depths[idx]);
        key_base = (cid << (32 + tile_n_bits)) | (int64_t)(uint64_t)depth_bits; // zero-extended bits (:96-98)
    }
    // inclusive prefix of the counts over the wave
    uint32_t incl = cnt;
#pragma unroll
    for (uint32_t off = 1; off < 64; off <<= 1) {
        const uint32_t up = (uint32_t)__shfl_up((int)incl, off, 64);
        if (lane >= off)
            incl += up;
    }
    const uint32_t total = (uint32_t)__shfl((int)incl, 63, 64);
    s_incl[wv][lane] = incl;
    s_xy[wv][lane] = r.x0 | (r.y0 << 16);
    s_w[wv][lane] = w;
    s_idx[wv][lane] = idx;
    if (!COMPACT) {
        s_lo[wv][lane] = (uint32_t)key_base;
        s_hi[wv][lane] = (uint32_t)(key_base >> 32);
    }
    __syncthreads();
    if (total == 0)
        return; // wave-uniform; no barrier follows
    // where the wave's first position starts in the output
    const uint32_t i0 = i - lane;
    const int64_t wave_base = (i0 == 0) ? 0 : cum_tiles_per_gauss[i0 - 1];
    for (uint32_t k = lane; k < total; k += 64u) {
        // smallest l with incl[l] > k
        uint32_t lo = 0, hi = 63;
#pragma unroll
        for (uint32_t step = 0; step < 6; ++step) {
            const uint32_t mid = (lo + hi) >> 1;
            if (s_incl[wv][mid] > k)
                hi = mid;
            else
                lo = mid + 1;
        }
        const uint32_t l = lo;
        const uint32_t before = l ? s_incl[wv][l - 1] : 0u;
        const uint32_t local = k - before;
        const uint32_t gw = s_w[wv][l], xy = s_xy[wv][l];
        const uint32_t row = local / gw;
        const int64_t tile_id = (int64_t)((xy >> 16) + row) * tile_width + ((xy & 0xffffu) + (local - row * gw));
        if (wave_base + k < capacity) { // a caller that emits before it knows the total bounds the writes
            if (COMPACT) {
                tile_keys[wave_base + k] = (uint16_t)tile_id;
            } else {
                const int64_t kb = ((int64_t)s_hi[wv][l] << 32) | (int64_t)s_lo[wv][l];
                isect_ids[wave_base + k] = kb | (tile_id << 32);
            }
            flatten_ids[wave_base + k] = (int32_t)s_idx[wv][l];
        }
    }
}

// ---- visiting order of the tiles for the rasterizers: longest lists first (tile_order_block, gsx_tiles.h) ---------
__global__ void __launch_bounds__(1024) tile_order_kernel(uint32_t n_tiles, uint32_t n_isects,
                                                           const int32_t* __restrict__ tile_offsets,
                                                           const uint32_t* __restrict__ tile_cost /*nullable*/,
                                                           uint32_t* __restrict__ tile_order) {
    __shared__ uint32_t cursor[kLenClasses];
    __shared__ uint32_t wave_total[16];
    tile_order_block<1024>(n_tiles, n_isects, tile_offsets, tile_cost, tile_order, cursor, wave_total);
}

// What a forward pass leaves per pixel (alpha, position of the last contributor) gives the tile cost too: how far
// the tile's pixels went into its list.  One workgroup per tile.
__global__ void __launch_bounds__(256) tile_walk_kernel(uint32_t image_width, uint32_t image_height,
                                                         uint32_t tile_width, const int32_t* __restrict__ tile_offsets,
                                                         const float* __restrict__ render_alphas,
                                                         const int32_t* __restrict__ last_ids,
                                                         uint32_t* __restrict__ tile_walk) {
    __shared__ uint32_t walk_s;
    const uint32_t tile_id = blockIdx.x, tr = threadIdx.x;
    if (tr == 0)
        walk_s = 0;
    __syncthreads();
    const TilePixel px = tile_pixel(tile_id, tile_width, tr);
    uint32_t w = 0;
    if (px.i < image_height && px.j < image_width) {
        const size_t p = (size_t)px.i * image_width + px.j;
        const int32_t start = tile_offsets[tile_id];
        if (render_alphas[p] > 0.0f && last_ids[p] >= start)
            w = (uint32_t)(last_ids[p] - start) + 1u;
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1)
        w = max(w, (uint32_t)__shfl_xor((int)w, m, 64));
    if ((tr & 63u) == 0)
        atomicMax(&walk_s, w);
    __syncthreads();
    if (tr == 0)
        tile_walk[tile_id] = walk_s;
}

// IntersectTile.cu:206-252
__global__ void __launch_bounds__(256) intersect_offset_kernel(uint32_t n_isects,
                                                                const int64_t* __restrict__ isect_ids, uint32_t C,
                                                                uint32_t n_tiles, uint32_t tile_n_bits,
                                                                int32_t* __restrict__ offsets) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= n_isects)
        return;
    const int64_t tile_mask = ((int64_t)1 << tile_n_bits) - 1;
    const int64_t isect_id_curr = isect_ids[idx] >> 32;
    const int64_t id_curr = (isect_id_curr >> tile_n_bits) * n_tiles + (isect_id_curr & tile_mask);
    if (idx == 0)
        for (int64_t i = 0; i < id_curr + 1; ++i)
            offsets[i] = 0;
    if (idx == n_isects - 1)
        for (int64_t i = id_curr + 1; i < (int64_t)C * n_tiles; ++i)
            offsets[i] = (int32_t)n_isects;
    if (idx > 0) {
        const int64_t isect_id_prev = isect_ids[idx - 1] >> 32;
        if (isect_id_prev == isect_id_curr)
            return;
        const int64_t id_prev = (isect_id_prev >> tile_n_bits) * n_tiles + (isect_id_prev & tile_mask);
        for (int64_t i = id_prev + 1; i < id_curr + 1; ++i)
            offsets[i] = (int32_t)idx;
    }
}

// the same ranges from sorted 16-bit tile indices of one camera; a thread takes `per` consecutive pairs (8 with one
// 16-byte load when the array is aligned for it)
__global__ void __launch_bounds__(256) tile_pairs_offset_kernel(uint32_t n_isects,
                                                                 const uint16_t* __restrict__ tile_keys,
                                                                 uint32_t n_tiles, uint32_t per,
                                                                 int32_t* __restrict__ offsets) {
    const uint32_t first = (blockIdx.x * 256u + threadIdx.x) * per;
    if (first >= n_isects)
        return;
    uint32_t k[8];
    const uint32_t cnt = min(per, n_isects - first);
    if (cnt == 8) {
        const uint4 q = *reinterpret_cast<const uint4*>(tile_keys + first);
        k[0] = q.x & 0xffffu, k[1] = q.x >> 16, k[2] = q.y & 0xffffu, k[3] = q.y >> 16;
        k[4] = q.z & 0xffffu, k[5] = q.z >> 16, k[6] = q.w & 0xffffu, k[7] = q.w >> 16;
    } else {
        for (uint32_t e = 0; e < cnt; ++e)
            k[e] = tile_keys[first + e];
    }
    uint32_t prev = first ? (uint32_t)tile_keys[first - 1] : 0u;
    if (first == 0)
        for (uint32_t i = 0; i < k[0] + 1; ++i)
            offsets[i] = 0;
    for (uint32_t e = 0; e < cnt; ++e) {
        const uint32_t idx = first + e, curr = k[e];
        if (idx > 0)
            for (uint32_t i = prev + 1; i < curr + 1; ++i)
                offsets[i] = (int32_t)idx;
        if (idx == n_isects - 1)
            for (uint32_t i = curr + 1; i < n_tiles; ++i)
                offsets[i] = (int32_t)n_isects;
        prev = curr;
    }
}

__global__ void __launch_bounds__(256) fill_i32_kernel(uint32_t n, int32_t v, int32_t* __restrict__ out) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i < n)
        out[i] = v;
}

} // namespace gsx

using namespace gsx;

extern "C" size_t gsx_intersect_tile_count_workspace_bytes(uint32_t C, uint32_t N) {
    const uint64_t n = (uint64_t)C * N;
    const uint64_t nb = (n + kScanTile - 1) / kScanTile;
    return align_up((nb + 1) * sizeof(int64_t), 256) + 256;
}

namespace {
// prefix sum of the counts (int32 array, or high words of `keys`) into cum, grand total to *total_dev
int scan_counts(uint32_t n, const int32_t* counts, const int64_t* keys, bool rect_keys, int64_t* cum,
                int64_t* block_sums, int64_t* total_dev, hipStream_t s) {
    const uint32_t nb = cdiv(n, kScanTile);
    hipLaunchKernelGGL(scan_block_sums_kernel, dim3(nb), dim3(256), 0, s, n, counts, keys, rect_keys, block_sums);
    GSX_LAUNCH_CHECK();
    if (nb <= 4096) { // every block sums the totals in front of it: at most 8 M additions in all
        hipLaunchKernelGGL(scan_apply_kernel<true>, dim3(nb), dim3(256), 0, s, n, counts, keys, rect_keys, block_sums,
                           cum, total_dev);
    } else {
        hipLaunchKernelGGL(scan_block_offsets_kernel, dim3(1), dim3(256), 0, s, nb, block_sums, total_dev);
        GSX_LAUNCH_CHECK();
        hipLaunchKernelGGL(scan_apply_kernel<false>, dim3(nb), dim3(256), 0, s, n, counts, keys, rect_keys, block_sums,
                           cum, total_dev);
    }
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

// The address under which kernels of the current device can write a pinned host slot, or nullptr for pageable memory.
int64_t* device_view_of_host_slot(int64_t* slot) {
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, slot) != hipSuccess) {
        (void)hipGetLastError(); // not known to the runtime: pageable
        return nullptr;
    }
    if (attr.type != hipMemoryTypeHost || attr.devicePointer == nullptr)
        return nullptr;
    return (int64_t*)attr.devicePointer;
}

// tile grids whose rectangle corners fit a byte each: the depth keys then carry the rectangle
bool rect_keys_fit(uint32_t tile_width, uint32_t tile_height) { return tile_width <= 255 && tile_height <= 255; }

int check_tile_grid(const char* who, uint32_t C, uint32_t tile_size, uint32_t tile_width, uint32_t tile_height) {
    GSX_REQUIRE(tile_size > 0 && tile_width > 0 && tile_height > 0, GSX_ERR_INVALID_ARGUMENT, "%s: empty tile grid",
                who);
    GSX_REQUIRE((uint64_t)tile_width * tile_height < (1ull << 32) &&
                    gsx_n_bits(tile_width * tile_height) + gsx_n_bits(C) <= 32,
                GSX_ERR_INVALID_ARGUMENT, "%s: tile and camera ids need more than 32 bits", who); // Intersect.cpp:50
    GSX_REQUIRE(tile_width < 65536 && tile_height < 65536, GSX_ERR_INVALID_ARGUMENT, "%s: tile grid too large", who);
    return GSX_OK;
}
} // namespace

extern "C" int gsx_intersect_tile_count(uint32_t C, uint32_t N, const float* means2d, const int32_t* radii,
                                        uint32_t tile_size, uint32_t tile_width, uint32_t tile_height,
                                        int32_t* tiles_per_gauss, int64_t* cum_tiles_per_gauss, void* workspace,
                                        size_t workspace_bytes, int64_t* n_isects_host, void* stream) {
    GSX_REQUIRE(n_isects_host != nullptr, GSX_ERR_INVALID_ARGUMENT, "intersect_tile_count: n_isects_host is null");
    *n_isects_host = 0;
    const uint64_t n64 = (uint64_t)C * N;
    if (n64 == 0)
        return GSX_OK; // Intersect.cpp:77-79
    GSX_REQUIRE(means2d && radii && tiles_per_gauss && cum_tiles_per_gauss, GSX_ERR_INVALID_ARGUMENT,
                "intersect_tile_count: null tensor");
    GSX_REQUIRE(n64 < (1ull << 31), GSX_ERR_INVALID_ARGUMENT, "intersect_tile_count: C*N >= 2^31");
    int rc = check_tile_grid("intersect_tile_count", C, tile_size, tile_width, tile_height);
    if (rc != GSX_OK)
        return rc;
    GSX_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0 &&
                    workspace_bytes >= gsx_intersect_tile_count_workspace_bytes(C, N),
                GSX_ERR_WORKSPACE, "intersect_tile_count: workspace needs %zu bytes, 256-byte aligned",
                gsx_intersect_tile_count_workspace_bytes(C, N));
    const uint32_t n = (uint32_t)n64;
    const uint32_t nb = cdiv(n, kScanTile);
    int64_t* block_sums = (int64_t*)workspace;
    int64_t* total = block_sums + nb;
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(tile_count_kernel, dim3(cdiv(n, 256)), dim3(256), 0, s, n, means2d, radii, (float)tile_size,
                       tile_width, tile_height, tiles_per_gauss);
    GSX_LAUNCH_CHECK();
    if ((rc = scan_counts(n, tiles_per_gauss, nullptr, false, cum_tiles_per_gauss, block_sums, total, s)) != GSX_OK)
        return rc;
    // the one sanctioned host synchronisation of the path (Intersect.cpp:76 `.item<int64_t>()`)
    int64_t host_total = 0;
    GSX_HIP_CHECK(hipMemcpyAsync(&host_total, total, sizeof(int64_t), hipMemcpyDeviceToHost, s));
    GSX_HIP_CHECK(hipStreamSynchronize(s));
    *n_isects_host = host_total;
    GSX_REQUIRE(host_total < (1ll << 31), GSX_ERR_OVERFLOW,
                "intersect_tile_count: %lld intersections do not fit int32 indices", (long long)host_total);
    return GSX_OK;
}

// workspace: keys0, keys1 (i64 [N]), vals1 (i32 [N]), scan block sums + total, then the sort's own scratch
namespace {
struct OrderedLayout {
    size_t keys1_off, vals1_off, sums_off, sort_off, total;
};
OrderedLayout ordered_layout(uint32_t N) {
    OrderedLayout L;
    const size_t kb = align_up((size_t)N * 8, 256);
    L.keys1_off = kb;
    L.vals1_off = 2 * kb;
    L.sums_off = L.vals1_off + align_up((size_t)N * 4, 256);
    L.sort_off = L.sums_off + gsx_intersect_tile_count_workspace_bytes(1, N);
    L.total = L.sort_off + gsx_radix_sort_pairs_workspace_bytes(N);
    return L;
}
} // namespace

extern "C" size_t gsx_intersect_tile_count_ordered_workspace_bytes(uint32_t N) { return ordered_layout(N).total; }

namespace gsx {
int64_t* ordered_keys(void* workspace) { return (int64_t*)workspace; }

// The part after the keys are written: sort the N (count << 32 | depth bits) keys in workspace on their low word,
// scan the counts in that order, start the copy of the total.  order must hold 0..N-1 on entry.  rect_keys: the
// high words are packed tile rectangles (depth_count_keys_kernel<true>) instead of counts.
int ordered_counts_from_keys(const char* who, uint32_t N, int32_t* order, int64_t* cum_tiles_per_gauss, void* workspace,
                             size_t workspace_bytes, int64_t* n_isects_host, int wait, void* stream, bool rect_keys,
                             bool first_hist_done) {
    const OrderedLayout L = ordered_layout(N);
    GSX_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0 && workspace_bytes >= L.total,
                GSX_ERR_WORKSPACE, "%s: workspace needs %zu bytes, 256-byte aligned", who, L.total);
    char* ws = (char*)workspace;
    int64_t* keys0 = (int64_t*)ws;
    int64_t* keys1 = (int64_t*)(ws + L.keys1_off);
    int32_t* vals1 = (int32_t*)(ws + L.vals1_off);
    int64_t* block_sums = (int64_t*)(ws + L.sums_off);
    int64_t* total = block_sums + cdiv(N, kScanTile);
    hipStream_t s = (hipStream_t)stream;
    int rc, sel = 0;
    if ((rc = radix_sort_pairs_32_bits(N, keys0, order, keys1, vals1, 0, ws + L.sort_off,
                                       gsx_radix_sort_pairs_workspace_bytes(N), &sel, stream, first_hist_done)) !=
        GSX_OK)
        return rc;
    if (sel) { // four 8-bit passes end in buffer 0; kept for a different digit width
        GSX_HIP_CHECK(hipMemcpyAsync(order, vals1, (size_t)N * 4, hipMemcpyDeviceToDevice, s));
        GSX_HIP_CHECK(hipMemcpyAsync(keys0, keys1, (size_t)N * 8, hipMemcpyDeviceToDevice, s));
    }
    // the sorted keys stay in ordered_keys(workspace) for an emission that reads them.  A caller that does not wait
    // passes a pinned slot: the scan's last block writes the total there itself (no copy launch behind the scan).
    int64_t* slot = wait ? nullptr : device_view_of_host_slot(n_isects_host);
    if ((rc = scan_counts(N, nullptr, keys0, rect_keys, cum_tiles_per_gauss, block_sums, slot ? slot : total, s)) !=
        GSX_OK)
        return rc;
    if (slot == nullptr)
        GSX_HIP_CHECK(hipMemcpyAsync(n_isects_host, total, sizeof(int64_t), hipMemcpyDeviceToHost, s));
    if (wait) {
        GSX_HIP_CHECK(hipStreamSynchronize(s));
        GSX_REQUIRE(*n_isects_host < (1ll << 31), GSX_ERR_OVERFLOW, "%s: %lld intersections do not fit int32 indices",
                    who, (long long)*n_isects_host);
    }
    return GSX_OK;
}
} // namespace gsx

extern "C" int gsx_intersect_tile_count_ordered(uint32_t N, const float* means2d, const int32_t* radii,
                                                const float* depths, uint32_t tile_size, uint32_t tile_width,
                                                uint32_t tile_height, int32_t* order, int32_t* tiles_per_gauss,
                                                int64_t* cum_tiles_per_gauss, void* workspace,
                                                size_t workspace_bytes, int64_t* n_isects_host, int wait,
                                                void* stream) {
    GSX_REQUIRE(n_isects_host != nullptr, GSX_ERR_INVALID_ARGUMENT, "intersect_tile_count_ordered: n_isects_host is null");
    *n_isects_host = 0;
    if (N == 0)
        return GSX_OK;
    if (!wait)
        *n_isects_host = -1; // "not there yet": the device-to-host copy queued below overwrites it with the total
    GSX_REQUIRE(means2d && radii && depths && order && tiles_per_gauss && cum_tiles_per_gauss,
                GSX_ERR_INVALID_ARGUMENT, "intersect_tile_count_ordered: null tensor");
    GSX_REQUIRE(N < (1u << 31), GSX_ERR_INVALID_ARGUMENT, "intersect_tile_count_ordered: N >= 2^31");
    int rc = check_tile_grid("intersect_tile_count_ordered", 1, tile_size, tile_width, tile_height);
    if (rc != GSX_OK)
        return rc;
    GSX_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0 &&
                    workspace_bytes >= ordered_layout(N).total,
                GSX_ERR_WORKSPACE, "intersect_tile_count_ordered: workspace needs %zu bytes, 256-byte aligned",
                ordered_layout(N).total);
    const bool rect_keys = rect_keys_fit(tile_width, tile_height);
    // the key kernel's workgroups are the sort's blocks: each leaves its column of the first pass's histogram
    const gsx::RadixFirstPass fp =
        gsx::radix_first_pass_table(N, (char*)workspace + ordered_layout(N).sort_off);
    if (rect_keys)
        hipLaunchKernelGGL(depth_count_keys_kernel<true>, dim3(fp.nblocks), dim3(256), 0, (hipStream_t)stream, N,
                           means2d, radii, depths, (float)tile_size, tile_width, tile_height, fp.items, fp.nblocks,
                           tiles_per_gauss, gsx::ordered_keys(workspace), order, fp.table);
    else
        hipLaunchKernelGGL(depth_count_keys_kernel<false>, dim3(fp.nblocks), dim3(256), 0, (hipStream_t)stream, N,
                           means2d, radii, depths, (float)tile_size, tile_width, tile_height, fp.items, fp.nblocks,
                           tiles_per_gauss, gsx::ordered_keys(workspace), order, fp.table);
    GSX_LAUNCH_CHECK();
    return gsx::ordered_counts_from_keys("intersect_tile_count_ordered", N, order, cum_tiles_per_gauss, workspace,
                                         workspace_bytes, n_isects_host, wait, stream, rect_keys, true);
}

extern "C" int gsx_intersect_tile_emit(uint32_t C, uint32_t N, const float* means2d, const int32_t* radii,
                                       const float* depths, const int64_t* cum_tiles_per_gauss,
                                       const int32_t* order, uint32_t tile_size, uint32_t tile_width,
                                       uint32_t tile_height, int64_t* isect_ids, int32_t* flatten_ids,
                                       void* stream) {
    return gsx_intersect_tile_emit_capped(C, N, means2d, radii, depths, cum_tiles_per_gauss, order, tile_size,
                                          tile_width, tile_height, INT64_MAX, isect_ids, flatten_ids, stream);
}

extern "C" int gsx_intersect_tile_emit_capped(uint32_t C, uint32_t N, const float* means2d, const int32_t* radii,
                                              const float* depths, const int64_t* cum_tiles_per_gauss,
                                              const int32_t* order, uint32_t tile_size, uint32_t tile_width,
                                              uint32_t tile_height, int64_t capacity, int64_t* isect_ids,
                                              int32_t* flatten_ids, void* stream) {
    const uint64_t n64 = (uint64_t)C * N;
    if (n64 == 0)
        return GSX_OK;
    GSX_REQUIRE(means2d && radii && depths && cum_tiles_per_gauss && isect_ids && flatten_ids,
                GSX_ERR_INVALID_ARGUMENT, "intersect_tile_emit: null tensor");
    GSX_REQUIRE(n64 < (1ull << 31), GSX_ERR_INVALID_ARGUMENT, "intersect_tile_emit: C*N >= 2^31");
    const uint32_t n = (uint32_t)n64;
    GSX_REQUIRE(order == nullptr || C == 1, GSX_ERR_UNSUPPORTED, "intersect_tile_emit: an order needs C == 1");
    hipLaunchKernelGGL(tile_emit_kernel<false>, dim3(cdiv(n, 256)), dim3(256), 0, (hipStream_t)stream, n, N, means2d,
                       radii, depths, (const int64_t*)nullptr, cum_tiles_per_gauss, order, (float)tile_size, tile_width,
                       tile_height, gsx_n_bits(tile_width * tile_height), capacity, isect_ids, (uint16_t*)nullptr,
                       flatten_ids);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

// Packed rows ([nnz] instead of [C, N]; Intersect.cpp:32-39, IntersectTile.cu:50, 86-94): the count is that of one
// camera with nnz rows (a row's tile count does not depend on its camera), the emission takes each row's camera
// from camera_ids; flatten_ids index the packed rows.
extern "C" int gsx_intersect_tile_emit_packed(uint32_t C, uint32_t nnz, const float* means2d, const int32_t* radii,
                                              const float* depths, const int64_t* camera_ids,
                                              const int64_t* cum_tiles_per_gauss, uint32_t tile_size,
                                              uint32_t tile_width, uint32_t tile_height, int64_t* isect_ids,
                                              int32_t* flatten_ids, void* stream) {
    if (nnz == 0)
        return GSX_OK;
    GSX_REQUIRE(means2d && radii && depths && camera_ids && cum_tiles_per_gauss && isect_ids && flatten_ids,
                GSX_ERR_INVALID_ARGUMENT, "intersect_tile_emit_packed: null tensor");
    GSX_REQUIRE(nnz < (1u << 31), GSX_ERR_INVALID_ARGUMENT, "intersect_tile_emit_packed: nnz >= 2^31");
    const int rc = check_tile_grid("intersect_tile_emit_packed", C, tile_size, tile_width, tile_height);
    if (rc != GSX_OK)
        return rc;
    hipLaunchKernelGGL(tile_emit_kernel<false>, dim3(cdiv(nnz, 256)), dim3(256), 0, (hipStream_t)stream, nnz, nnz,
                       means2d, radii, depths, (const int64_t*)nullptr, cum_tiles_per_gauss, (const int32_t*)nullptr,
                       (float)tile_size, tile_width, tile_height, gsx_n_bits(tile_width * tile_height), INT64_MAX,
                       isect_ids, (uint16_t*)nullptr, flatten_ids, camera_ids);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_intersect_tile_emit_ordered(uint32_t N, const float* means2d, const int32_t* radii,
                                               const float* depths, const int64_t* cum_tiles_per_gauss,
                                               const int32_t* order, const void* ordered_workspace,
                                               uint32_t tile_size, uint32_t tile_width, uint32_t tile_height,
                                               int64_t capacity, int64_t* isect_ids, int32_t* flatten_ids,
                                               void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(order && ordered_workspace, GSX_ERR_INVALID_ARGUMENT,
                "intersect_tile_emit_ordered: order / workspace of gsx_intersect_tile_count_ordered is null");
    if (!rect_keys_fit(tile_width, tile_height)) // the keys hold counts: rectangles come from the Gaussians
        return gsx_intersect_tile_emit_capped(1, N, means2d, radii, depths, cum_tiles_per_gauss, order, tile_size,
                                              tile_width, tile_height, capacity, isect_ids, flatten_ids, stream);
    GSX_REQUIRE(cum_tiles_per_gauss && isect_ids && flatten_ids, GSX_ERR_INVALID_ARGUMENT,
                "intersect_tile_emit_ordered: null tensor");
    GSX_REQUIRE(N < (1u << 31), GSX_ERR_INVALID_ARGUMENT, "intersect_tile_emit_ordered: N >= 2^31");
    hipLaunchKernelGGL(tile_emit_kernel<true>, dim3(cdiv(N, 256)), dim3(256), 0, (hipStream_t)stream, N, N,
                       (const float*)nullptr, (const int32_t*)nullptr, (const float*)nullptr,
                       (const int64_t*)gsx::ordered_keys(const_cast<void*>(ordered_workspace)), cum_tiles_per_gauss,
                       order, (float)tile_size, tile_width, tile_height, gsx_n_bits(tile_width * tile_height),
                       capacity, isect_ids, (uint16_t*)nullptr, flatten_ids);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_intersect_tile_pairs_fit(uint32_t tile_width, uint32_t tile_height) {
    return rect_keys_fit(tile_width, tile_height) ? 1 : 0;
}

extern "C" int gsx_intersect_tile_emit_pairs(uint32_t N, const int64_t* cum_tiles_per_gauss, const int32_t* order,
                                             const void* ordered_workspace, uint32_t tile_size, uint32_t tile_width,
                                             uint32_t tile_height, int64_t capacity, uint16_t* tile_keys,
                                             int32_t* flatten_ids, void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(order && ordered_workspace, GSX_ERR_INVALID_ARGUMENT,
                "intersect_tile_emit_pairs: order / workspace of gsx_intersect_tile_count_ordered is null");
    GSX_REQUIRE(rect_keys_fit(tile_width, tile_height), GSX_ERR_UNSUPPORTED,
                "intersect_tile_emit_pairs: a %u x %u tile grid needs the 64-bit keys", tile_width, tile_height);
    GSX_REQUIRE(cum_tiles_per_gauss && tile_keys && flatten_ids, GSX_ERR_INVALID_ARGUMENT,
                "intersect_tile_emit_pairs: null tensor");
    GSX_REQUIRE(N < (1u << 31), GSX_ERR_INVALID_ARGUMENT, "intersect_tile_emit_pairs: N >= 2^31");
    hipLaunchKernelGGL((tile_emit_kernel<true, true>), dim3(cdiv(N, 256)), dim3(256), 0, (hipStream_t)stream, N, N,
                       (const float*)nullptr, (const int32_t*)nullptr, (const float*)nullptr,
                       (const int64_t*)gsx::ordered_keys(const_cast<void*>(ordered_workspace)), cum_tiles_per_gauss,
                       order, (float)tile_size, tile_width, tile_height, gsx_n_bits(tile_width * tile_height),
                       capacity, (int64_t*)nullptr, tile_keys, flatten_ids);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" size_t gsx_tile_order_bytes(uint32_t tile_width, uint32_t tile_height) {
    return 2 * align_up((size_t)tile_width * tile_height * 4, 256);
}

namespace gsx {
// the order for a backward pass from what the forward pass left per pixel; scratch: gsx_tile_order_bytes
int tile_order_from_pixels(int64_t n_isects, uint32_t image_width, uint32_t image_height, const int32_t* tile_offsets,
                           const float* render_alphas, const int32_t* last_ids, void* scratch,
                           const uint32_t** tile_order, void* stream) {
    const uint32_t tw = cdiv(image_width, kTile), th = cdiv(image_height, kTile);
    uint32_t* walk = (uint32_t*)scratch;
    uint32_t* order = (uint32_t*)((char*)scratch + align_up((size_t)tw * th * 4, 256));
    hipLaunchKernelGGL(tile_walk_kernel, dim3(tw * th), dim3(256), 0, (hipStream_t)stream, image_width, image_height,
                       tw, tile_offsets, render_alphas, last_ids, walk);
    GSX_LAUNCH_CHECK();
    *tile_order = order;
    return gsx_tile_order(n_isects, nullptr, walk, tw, th, order, stream);
}
} // namespace gsx

extern "C" int gsx_tile_order(int64_t n_isects, const int32_t* tile_offsets, const uint32_t* tile_cost,
                              uint32_t tile_width, uint32_t tile_height, uint32_t* tile_order, void* stream) {
    const uint64_t n_tiles = (uint64_t)tile_width * tile_height;
    if (n_tiles == 0)
        return GSX_OK;
    GSX_REQUIRE((tile_offsets || tile_cost) && tile_order, GSX_ERR_INVALID_ARGUMENT, "tile_order: null tensor");
    GSX_REQUIRE(n_isects >= GSX_COUNT_IN_OFFSETS && n_isects < (1ll << 31) && n_tiles < (1ull << 31),
                GSX_ERR_OVERFLOW, "tile_order: sizes out of range");
    hipLaunchKernelGGL(tile_order_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, (uint32_t)n_tiles,
                       (uint32_t)n_isects, tile_offsets, tile_cost, tile_order);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_intersect_offset(int64_t n_isects, const int64_t* isect_ids, uint32_t C, uint32_t tile_width,
                                    uint32_t tile_height, int32_t* offsets, void* stream) {
    const uint64_t total_tiles = (uint64_t)C * tile_width * tile_height;
    if (total_tiles == 0)
        return GSX_OK;
    GSX_REQUIRE(offsets != nullptr, GSX_ERR_INVALID_ARGUMENT, "intersect_offset: offsets is null");
    GSX_REQUIRE(n_isects >= 0 && n_isects < (1ll << 31), GSX_ERR_OVERFLOW, "intersect_offset: n_isects out of range");
    GSX_REQUIRE(total_tiles < (1ull << 31), GSX_ERR_INVALID_ARGUMENT, "intersect_offset: too many tiles");
    hipStream_t s = (hipStream_t)stream;
    if (n_isects == 0) { // IntersectTile.cu:268-271
        hipLaunchKernelGGL(fill_i32_kernel, dim3(cdiv(total_tiles, 256)), dim3(256), 0, s, (uint32_t)total_tiles, 0,
                           offsets);
        GSX_LAUNCH_CHECK();
        return GSX_OK;
    }
    GSX_REQUIRE(isect_ids != nullptr, GSX_ERR_INVALID_ARGUMENT, "intersect_offset: isect_ids is null");
    hipLaunchKernelGGL(intersect_offset_kernel, dim3(cdiv(n_isects, 256)), dim3(256), 0, s, (uint32_t)n_isects,
                       isect_ids, C, tile_width * tile_height, gsx_n_bits(tile_width * tile_height), offsets);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_intersect_tile_pairs_offset(int64_t n_isects, const uint16_t* tile_keys, uint32_t tile_width,
                                               uint32_t tile_height, int32_t* offsets, void* stream) {
    const uint64_t n_tiles = (uint64_t)tile_width * tile_height;
    if (n_tiles == 0)
        return GSX_OK;
    GSX_REQUIRE(offsets != nullptr, GSX_ERR_INVALID_ARGUMENT, "intersect_tile_pairs_offset: offsets is null");
    GSX_REQUIRE(n_isects >= 0 && n_isects < (1ll << 31), GSX_ERR_OVERFLOW,
                "intersect_tile_pairs_offset: n_isects out of range");
    GSX_REQUIRE(n_tiles <= 65536, GSX_ERR_UNSUPPORTED, "intersect_tile_pairs_offset: more than 65536 tiles");
    hipStream_t s = (hipStream_t)stream;
    if (n_isects == 0) {
        hipLaunchKernelGGL(fill_i32_kernel, dim3(cdiv(n_tiles, 256)), dim3(256), 0, s, (uint32_t)n_tiles, 0, offsets);
        GSX_LAUNCH_CHECK();
        return GSX_OK;
    }
    GSX_REQUIRE(tile_keys != nullptr, GSX_ERR_INVALID_ARGUMENT, "intersect_tile_pairs_offset: tile_keys is null");
    const uint32_t per = ((uintptr_t)tile_keys & 15u) == 0 ? 8u : 1u;
    hipLaunchKernelGGL(tile_pairs_offset_kernel, dim3(cdiv(n_isects, 256 * per)), dim3(256), 0, s,
                       (uint32_t)n_isects, tile_keys, (uint32_t)n_tiles, per, offsets);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}
