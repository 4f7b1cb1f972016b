// intersect.hip - tile intersection: per-Gaussian tile counts, their prefix sum, key/value emission and the
// per-tile ranges of the sorted keys (gsplat/IntersectTile.cu:23-114, 206-252; gsplat/Intersect.cpp:41-137).
// Integer work: every output is bit-exact given the inputs.
#include "gsx_common.h"

namespace gsx {

struct TileRect {
    uint32_t x0, y0, x1, y1;
};

// IntersectTile.cu:56-76.  The float -> uint32 conversions saturate (negative -> 0): that is what the
// reference's hardware conversion does, and plain C++ casts of negative floats are undefined.
__device__ __forceinline__ bool tile_rect(const float* __restrict__ means2d, const int32_t* __restrict__ radii,
                                          uint32_t idx, float tile_size, uint32_t tile_width, uint32_t tile_height,
                                          TileRect* r) {
    const int2 rad = reinterpret_cast<const int2*>(radii)[idx];
    const float radius_x = (float)rad.x, radius_y = (float)rad.y;
    if (radius_x <= 0 || radius_y <= 0)
        return false;
    const float2 m = reinterpret_cast<const float2*>(means2d)[idx];
    const float tile_radius_x = radius_x / tile_size, tile_radius_y = radius_y / tile_size;
    const float tile_x = m.x / tile_size, tile_y = m.y / tile_size;
    r->x0 = min(sat_u32(gsx::floor(tile_x - tile_radius_x)), tile_width);
    r->y0 = min(sat_u32(gsx::floor(tile_y - tile_radius_y)), tile_height);
    r->x1 = min(sat_u32(gsx::ceil(tile_x + tile_radius_x)), tile_width);
    r->y1 = min(sat_u32(gsx::ceil(tile_y + tile_radius_y)), tile_height);
    return true;
}

// order == nullptr: position i is Gaussian i.  Otherwise position i is Gaussian order[i]; the count goes to
// tiles_per_gauss[order[i]] and, for the prefix sum over positions, to counts_by_position[i].
__global__ void __launch_bounds__(256) tile_count_kernel(uint32_t n, const float* __restrict__ means2d,
                                                          const int32_t* __restrict__ radii, float tile_size,
                                                          uint32_t tile_width, uint32_t tile_height,
                                                          const int32_t* __restrict__ order,
                                                          int32_t* __restrict__ tiles_per_gauss,
                                                          int32_t* __restrict__ counts_by_position) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n)
        return;
    const uint32_t idx = order != nullptr ? (uint32_t)order[i] : i;
    TileRect r;
    int32_t cnt = 0;
    if (tile_rect(means2d, radii, idx, tile_size, tile_width, tile_height, &r))
        cnt = (int32_t)((r.y1 - r.y0) * (r.x1 - r.x0));
    tiles_per_gauss[idx] = cnt;
    if (order != nullptr)
        counts_by_position[i] = cnt;
}

// sort keys for the depth order of one camera's Gaussians: the depth's bit pattern (what the low word of an
// intersection key holds), all ones for a Gaussian that touches no tile
__global__ void __launch_bounds__(256) depth_keys_kernel(uint32_t n, const float* __restrict__ depths,
                                                          const int32_t* __restrict__ radii,
                                                          int64_t* __restrict__ keys, int32_t* __restrict__ vals) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n)
        return;
    const int2 rad = reinterpret_cast<const int2*>(radii)[i];
    const bool live = rad.x > 0 && rad.y > 0;
    keys[i] = live ? (int64_t)(uint64_t)f2u(depths[i]) : (int64_t)0xFFFFFFFFll;
    vals[i] = (int32_t)i;
}

// ---- inclusive scan int32 -> int64 (at::cumsum of Intersect.cpp:75) -----------------------------
// three passes: per-block sums, scan of the sums (one block), per-block scan + offset
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

__global__ void __launch_bounds__(256) scan_block_sums_kernel(uint32_t n, const int32_t* __restrict__ in,
                                                               int64_t* __restrict__ block_sums) {
    __shared__ int64_t lds[256];
    const uint32_t base = blockIdx.x * kScanTile + threadIdx.x * kScanItems;
    int64_t s = 0;
#pragma unroll
    for (uint32_t i = 0; i < kScanItems; ++i)
        if (base + i < n)
            s += in[base + i];
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
    if (threadIdx.x == 0)
        *total_out = carry;
}

__global__ void __launch_bounds__(256) scan_apply_kernel(uint32_t n, const int32_t* __restrict__ in,
                                                          const int64_t* __restrict__ block_offsets,
                                                          int64_t* __restrict__ out) {
    __shared__ int64_t lds[256];
    const uint32_t base = blockIdx.x * kScanTile + threadIdx.x * kScanItems;
    int32_t v[kScanItems];
    int64_t s = 0;
#pragma unroll
    for (uint32_t i = 0; i < kScanItems; ++i) {
        v[i] = (base + i < n) ? in[base + i] : 0;
        s += v[i];
    }
    int64_t total;
    int64_t run = block_exclusive_scan_256(s, lds, &total) + block_offsets[blockIdx.x];
#pragma unroll
    for (uint32_t i = 0; i < kScanItems; ++i) {
        run += v[i];
        if (base + i < n)
            out[base + i] = run;
    }
}

// IntersectTile.cu:78-113 second pass: keys and values in emission order (ascending position, row-major tiles
// inside a Gaussian).  A lane writes the tiles of a small Gaussian itself; the tiles of a Gaussian with more than
// 32 of them are written by the whole wave, 64 at a time, so that one screen-filling Gaussian does not leave
// 63 lanes idle.
__global__ void __launch_bounds__(256) tile_emit_kernel(uint32_t n, uint32_t N, const float* __restrict__ means2d,
                                                         const int32_t* __restrict__ radii,
                                                         const float* __restrict__ depths,
                                                         const int64_t* __restrict__ cum_tiles_per_gauss,
                                                         const int32_t* __restrict__ order, float tile_size,
                                                         uint32_t tile_width, uint32_t tile_height,
                                                         uint32_t tile_n_bits, int64_t* __restrict__ isect_ids,
                                                         int32_t* __restrict__ flatten_ids) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    const uint32_t lane = threadIdx.x & 63u;
    TileRect r = {0, 0, 0, 0};
    uint32_t idx = 0;
    bool live = false;
    if (i < n) {
        idx = order != nullptr ? (uint32_t)order[i] : i;
        live = tile_rect(means2d, radii, idx, tile_size, tile_width, tile_height, &r);
    }
    const uint32_t w = live ? r.x1 - r.x0 : 0u;
    const uint32_t cnt = live ? (r.y1 - r.y0) * w : 0u;
    int64_t key_base = 0;
    int64_t cur = 0;
    if (cnt) {
        const int64_t cid = idx / N;
        key_base = (cid << (32 + tile_n_bits)) | (int64_t)(uint64_t)f2u(depths[idx]); // zero-extended bits (:96-98)
        cur = (i == 0) ? 0 : cum_tiles_per_gauss[i - 1];
    }
    const bool big = cnt > 32u;
    if (cnt && !big) {
        for (uint32_t ty = r.y0; ty < r.y1; ++ty)
            for (uint32_t tx = r.x0; tx < r.x1; ++tx) {
                const int64_t tile_id = (int64_t)ty * tile_width + tx;
                isect_ids[cur] = key_base | (tile_id << 32);
                flatten_ids[cur] = (int32_t)idx;
                ++cur;
            }
    }
    uint64_t todo = __builtin_amdgcn_ballot_w64(big);
    while (todo) {
        const int src = __builtin_ctzll(todo);
        todo &= todo - 1;
        const uint32_t bx0 = (uint32_t)__shfl((int)r.x0, src, 64), by0 = (uint32_t)__shfl((int)r.y0, src, 64);
        const uint32_t bw = (uint32_t)__shfl((int)w, src, 64), bcnt = (uint32_t)__shfl((int)cnt, src, 64);
        const int32_t bidx = __shfl((int)idx, src, 64);
        const int64_t bkey = ((int64_t)__shfl((int)(key_base >> 32), src, 64) << 32) |
                             (int64_t)(uint32_t)__shfl((int)(uint32_t)key_base, src, 64);
        const int64_t bcur = ((int64_t)__shfl((int)(cur >> 32), src, 64) << 32) |
                             (int64_t)(uint32_t)__shfl((int)(uint32_t)cur, src, 64);
        for (uint32_t k = lane; k < bcnt; k += 64u) {
            const uint32_t row = k / bw;
            const int64_t tile_id = (int64_t)(by0 + row) * tile_width + (bx0 + (k - row * bw));
            isect_ids[bcur + k] = bkey | (tile_id << 32);
            flatten_ids[bcur + k] = bidx;
        }
    }
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
    return align_up((nb + 1) * sizeof(int64_t), 256) + 256 + align_up(n * sizeof(int32_t), 256);
}

// depth order of one camera's Gaussians: keys0 / keys1 (i64 [N] each), vals1 (i32 [N]), then the sort's own scratch
extern "C" size_t gsx_depth_order_workspace_bytes(uint32_t N) {
    return 2 * align_up((size_t)N * 8, 256) + align_up((size_t)N * 4, 256) + gsx_radix_sort_pairs_workspace_bytes(N);
}

extern "C" int gsx_depth_order(uint32_t N, const float* depths, const int32_t* radii, int32_t* order, void* workspace,
                               size_t workspace_bytes, void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(depths && radii && order, GSX_ERR_INVALID_ARGUMENT, "depth_order: null tensor");
    GSX_REQUIRE(N < (1u << 31), GSX_ERR_INVALID_ARGUMENT, "depth_order: N >= 2^31");
    GSX_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0 &&
                    workspace_bytes >= gsx_depth_order_workspace_bytes(N),
                GSX_ERR_WORKSPACE, "depth_order: workspace needs %zu bytes, 256-byte aligned",
                gsx_depth_order_workspace_bytes(N));
    char* ws = (char*)workspace;
    int64_t* keys0 = (int64_t*)ws;
    int64_t* keys1 = (int64_t*)(ws + align_up((size_t)N * 8, 256));
    int32_t* vals1 = (int32_t*)(ws + 2 * align_up((size_t)N * 8, 256));
    char* sort_ws = ws + 2 * align_up((size_t)N * 8, 256) + align_up((size_t)N * 4, 256);
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(depth_keys_kernel, dim3(cdiv(N, 256)), dim3(256), 0, s, N, depths, radii, keys0, order);
    GSX_LAUNCH_CHECK();
    int sel = 0;
    const int rc = gsx_radix_sort_pairs(N, keys0, order, keys1, vals1, 0, 32, sort_ws,
                                        gsx_radix_sort_pairs_workspace_bytes(N), &sel, stream);
    if (rc != GSX_OK)
        return rc;
    if (sel) // four 8-bit passes end in buffer 0; kept for a different digit width
        GSX_HIP_CHECK(hipMemcpyAsync(order, vals1, (size_t)N * 4, hipMemcpyDeviceToDevice, s));
    return GSX_OK;
}

extern "C" int gsx_intersect_tile_count(uint32_t C, uint32_t N, const float* means2d, const int32_t* radii,
                                        uint32_t tile_size, uint32_t tile_width, uint32_t tile_height,
                                        const int32_t* order, int32_t* tiles_per_gauss,
                                        int64_t* cum_tiles_per_gauss, void* workspace, size_t workspace_bytes,
                                        int64_t* n_isects_host, void* stream) {
    GSX_REQUIRE(n_isects_host != nullptr, GSX_ERR_INVALID_ARGUMENT, "intersect_tile_count: n_isects_host is null");
    *n_isects_host = 0;
    const uint64_t n64 = (uint64_t)C * N;
    if (n64 == 0)
        return GSX_OK; // Intersect.cpp:77-79
    GSX_REQUIRE(means2d && radii && tiles_per_gauss && cum_tiles_per_gauss, GSX_ERR_INVALID_ARGUMENT,
                "intersect_tile_count: null tensor");
    GSX_REQUIRE(n64 < (1ull << 31), GSX_ERR_INVALID_ARGUMENT, "intersect_tile_count: C*N >= 2^31");
    GSX_REQUIRE(tile_size > 0 && tile_width > 0 && tile_height > 0, GSX_ERR_INVALID_ARGUMENT,
                "intersect_tile_count: empty tile grid");
    GSX_REQUIRE((uint64_t)tile_width * tile_height < (1ull << 32) &&
                    gsx_n_bits(tile_width * tile_height) + gsx_n_bits(C) <= 32,
                GSX_ERR_INVALID_ARGUMENT,
                "intersect_tile_count: tile and camera ids need more than 32 bits"); // Intersect.cpp:50
    GSX_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0 &&
                    workspace_bytes >= gsx_intersect_tile_count_workspace_bytes(C, N),
                GSX_ERR_WORKSPACE, "intersect_tile_count: workspace needs %zu bytes, 256-byte aligned",
                gsx_intersect_tile_count_workspace_bytes(C, N));
    const uint32_t n = (uint32_t)n64;
    const uint32_t nb = cdiv(n, kScanTile);
    GSX_REQUIRE(order == nullptr || C == 1, GSX_ERR_UNSUPPORTED, "intersect_tile_count: an order needs C == 1");
    int64_t* block_sums = (int64_t*)workspace;
    int64_t* total = block_sums + nb;
    int32_t* counts_by_position = (int32_t*)((char*)workspace + align_up((nb + 1) * sizeof(int64_t), 256) + 256);
    const int32_t* scan_in = order != nullptr ? counts_by_position : tiles_per_gauss;
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(tile_count_kernel, dim3(cdiv(n, 256)), dim3(256), 0, s, n, means2d, radii, (float)tile_size,
                       tile_width, tile_height, order, tiles_per_gauss, counts_by_position);
    GSX_LAUNCH_CHECK();
    hipLaunchKernelGGL(scan_block_sums_kernel, dim3(nb), dim3(256), 0, s, n, scan_in, block_sums);
    GSX_LAUNCH_CHECK();
    hipLaunchKernelGGL(scan_block_offsets_kernel, dim3(1), dim3(256), 0, s, nb, block_sums, total);
    GSX_LAUNCH_CHECK();
    hipLaunchKernelGGL(scan_apply_kernel, dim3(nb), dim3(256), 0, s, n, scan_in, block_sums, cum_tiles_per_gauss);
    GSX_LAUNCH_CHECK();
    // the one sanctioned host synchronisation of the path (Intersect.cpp:76 `.item<int64_t>()`)
    int64_t host_total = 0;
    GSX_HIP_CHECK(hipMemcpyAsync(&host_total, total, sizeof(int64_t), hipMemcpyDeviceToHost, s));
    GSX_HIP_CHECK(hipStreamSynchronize(s));
    *n_isects_host = host_total;
    GSX_REQUIRE(host_total < (1ll << 31), GSX_ERR_OVERFLOW,
                "intersect_tile_count: %lld intersections do not fit int32 indices", (long long)host_total);
    return GSX_OK;
}

extern "C" int gsx_intersect_tile_emit(uint32_t C, uint32_t N, const float* means2d, const int32_t* radii,
                                       const float* depths, const int64_t* cum_tiles_per_gauss,
                                       const int32_t* order, uint32_t tile_size, uint32_t tile_width,
                                       uint32_t tile_height, int64_t* isect_ids, int32_t* flatten_ids,
                                       void* stream) {
    const uint64_t n64 = (uint64_t)C * N;
    if (n64 == 0)
        return GSX_OK;
    GSX_REQUIRE(means2d && radii && depths && cum_tiles_per_gauss && isect_ids && flatten_ids,
                GSX_ERR_INVALID_ARGUMENT, "intersect_tile_emit: null tensor");
    GSX_REQUIRE(n64 < (1ull << 31), GSX_ERR_INVALID_ARGUMENT, "intersect_tile_emit: C*N >= 2^31");
    const uint32_t n = (uint32_t)n64;
    GSX_REQUIRE(order == nullptr || C == 1, GSX_ERR_UNSUPPORTED, "intersect_tile_emit: an order needs C == 1");
    hipLaunchKernelGGL(tile_emit_kernel, dim3(cdiv(n, 256)), dim3(256), 0, (hipStream_t)stream, n, N, means2d, radii,
                       depths, cum_tiles_per_gauss, order, (float)tile_size, tile_width, tile_height,
                       gsx_n_bits(tile_width * tile_height), isect_ids, flatten_ids);
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
