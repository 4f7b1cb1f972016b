// raster_fwd.hip - per-tile forward rasterizer "from world" (gsplat/RasterizeToPixelsFromWorld3DGSFwd.cu:19-285).
//
// One 256-lane workgroup (four 64-lane waves) per 16x16 tile, one lane per pixel; every wave owns an 8x8 pixel
// block.  What a (pixel, Gaussian) pair needs from the Gaussian - M = diag(1/scale) R(quat)^T, gro = M (ray_o -
// mean), opacity, colour - does not depend on the tile, so it is built once per Gaussian as a 96-byte record
// (gsx_record.h) by pack_records_kernel (or by the fused per-Gaussian pass of a training step) instead of once per
// tile the Gaussian touches.  The tile's depth-sorted records are staged through LDS 192 at a time; every wave
// then keeps the slots whose exact pixel bounds meet its 8x8 block (ballot + prefix count, order preserved) and
// walks only those, reading each record with wave-uniform addresses (LDS broadcast), evaluating the ray / Gaussian
// response with explicit FMAs and compositing front to back.  Pairs outside the bounds have alpha < 1/255 and are
// skipped by the reference's own test, so skipping them early changes no result.  A wave leaves the batch loop as
// soon as its 64 pixels are saturated; the workgroup stops staging when all four waves are.
#include "gsx_common.h"

namespace gsx {

static constexpr uint32_t kFwdBatch = 192; // list entries staged at a time: 20 KB of LDS, seven workgroups per CU (256: 27 KB, six, and a launch 12 % longer)

// One record per Gaussian (all N: rows of Gaussians that no tile lists are never read).
__global__ void __launch_bounds__(256) pack_records_kernel(uint32_t N, uint32_t CDIM,
                                                            const float* __restrict__ means,
                                                            const float* __restrict__ quats,
                                                            const float* __restrict__ scales,
                                                            const float* __restrict__ opacities,
                                                            const float* __restrict__ colors,
                                                            const float* __restrict__ viewmat,
                                                            const float* __restrict__ Kmat, uint32_t W, uint32_t H,
                                                            bool pinhole, bool rolling,
                                                            float4* __restrict__ records) {
    const uint32_t g = blockIdx.x * 256u + threadIdx.x;
    if (g >= N)
        return;
    const vec3 ray_o = camera_ray_origin(load_cam_pose(viewmat));
    const vec3 xyz = ld3(means, g);
    const float opac = opacities[g];
    const mat3 M = record_whitening(ld4q(quats, g), ld3(scales, g));
    const vec3 gro = mul(M, sub(ray_o, xyz));
    const RecordRegion b =
        record_region(gro, M, opac, xyz, viewmat, Kmat[0], Kmat[4], Kmat[2], Kmat[5], W, H, pinhole);
    const float c0 = colors[(size_t)g * CDIM];
    const float c1 = CDIM > 1 ? colors[(size_t)g * CDIM + 1] : 0.f;
    const float c2 = CDIM > 2 ? colors[(size_t)g * CDIM + 2] : 0.f;
    // rolling shutter: every pixel row / column has its own ray origin, so the record carries the mean and the
    // rasterizers form M (ray_o - mean) per pixel
    store_record(records + (size_t)g * kRecordF4, rolling ? xyz : gro, opac, M, c0, c1, c2, b);
}

// STATS: count instead of rendering (for roofline accounting); stats[0] += (pixel, Gaussian) pairs evaluated,
// [1] += pairs composited, [2] += pairs the backward pass walks (entries up to each pixel's last contributor),
// [3] += (wave, Gaussian) iterations executed, [4] += (wave, Gaussian) iterations removed by the pixel bounds,
// [5] += executed iterations in which at least one pixel reaches the alpha threshold, [6] / [7] += the halves
// (8x4 rows / 4x8 columns) of those iterations' blocks that hold such a pixel.
// DIST: any camera but the perfect pinhole with a global shutter - OpenCV distortion, fisheye, equirectangular,
// rolling shutter (each pixel's ray comes from the model's unprojection under the pose of its exposure time; a pixel
// without a valid ray is done from the start, RasterizeToPixelsFromWorld3DGSFwd.cu:145).
// WIDE: more than 32 channels, CDIM (= 32) of them per launch: channels [c0, c0 + nc) of rows `stride` floats long,
// every one of them read from `colors` (the records' three colours are channels 0-2 of the whole row and are not
// used).  Each launch walks the lists again with the same arithmetic, so a pixel's weights, and with them every
// channel's sum, do not depend on the split; the launch with c0 = 0 writes alphas and last ids.
template <uint32_t CDIM, bool STATS, bool DIST, bool WIDE = false>
__global__ void __launch_bounds__(256) rasterize_fwd_kernel(
    uint32_t n_isects, const float4* __restrict__ records, const float* __restrict__ colors,
    const float* __restrict__ backgrounds, const uint8_t* __restrict__ masks, uint32_t image_width,
    uint32_t image_height, uint32_t tile_width, uint32_t tile_height, const float* __restrict__ viewmat,
    const float* __restrict__ Kmat, int camera_model, const float* __restrict__ radial,
    const float* __restrict__ tangential, const float* __restrict__ thin_prism,
    const float* __restrict__ viewmat1, int rs_type, const int32_t* __restrict__ tile_offsets,
    const int32_t* __restrict__ flatten_ids, const uint32_t* __restrict__ tile_order /*nullable*/,
    uint32_t* __restrict__ tile_walk /*nullable*/, float* __restrict__ render_colors,
    float* __restrict__ render_alphas,
    int32_t* __restrict__ last_ids, unsigned long long* __restrict__ stats, uint32_t stride = CDIM, uint32_t c0 = 0,
    uint32_t nc = CDIM) {
    static_assert(!WIDE || (CDIM == 32 && !STATS), "the wide instance takes 32 channels a launch");
    constexpr uint32_t NX = WIDE ? CDIM : (CDIM > 3 ? CDIM - 3 : 0); // channels staged from `colors`
    if (!WIDE)
        stride = CDIM, c0 = 0, nc = CDIM;
    __shared__ float4 stage[kFwdBatch * 4];
    __shared__ float4 region[kFwdBatch * 2];
    __shared__ float cuts[kFwdBatch];
    __shared__ uint8_t lists[4][kFwdBatch];
    __shared__ int32_t ids[NX ? kFwdBatch : 1];
    __shared__ float extra[NX ? kFwdBatch * NX : 1]; // channels beyond the third (WIDE: all of the launch's)

    const uint32_t tile_id = tile_order != nullptr ? tile_order[blockIdx.x] : blockIdx.x;
    const uint32_t tr = threadIdx.x;
    const TilePixel px = tile_pixel(tile_id, tile_width, tr);
    const uint32_t i = px.i, j = px.j;
    const bool inside = (i < image_height && j < image_width);
    const uint32_t pix_id = i * image_width + j;
    uint8_t* wave_list = lists[tr >> 6];

    // :147-155 masked tile: background colour only
    if (masks != nullptr && !masks[tile_id]) {
        if (inside && !STATS) {
#pragma unroll
            for (uint32_t k = 0; k < CDIM; ++k)
                if (k < nc)
                    render_colors[(size_t)pix_id * stride + c0 + k] = backgrounds == nullptr ? 0.0f : backgrounds[c0 + k];
        }
        if (tile_walk != nullptr && tr == 0 && !STATS)
            tile_walk[tile_id] = 0u; // a masked tile costs nothing
        return;
    }

    const CamPose cp = DIST ? load_cam_pose(viewmat, viewmat1, rs_type, image_width, image_height) : load_cam_pose(viewmat);
    // rolling shutter: the records carry the means and every pixel has its own ray origin
    const bool rolling = DIST && rs_type != GSX_GLOBAL;
    vec3 ray_o, ray_d;
    CameraModel cam;
    cam.type = 0, cam.dist.on = false;
    if (DIST)
        cam = load_camera_model(camera_model, radial, tangential, thin_prism, Kmat[0], Kmat[4], Kmat[2], Kmat[5],
                                image_width, image_height);
    const bool ray_ok =
        pixel_world_ray(cp, (float)j + 0.5f, (float)i + 0.5f, Kmat[0], Kmat[4], Kmat[2], Kmat[5], cam, &ray_o, &ray_d);

    const int32_t range_start = tile_offsets[tile_id];
    // n_isects == kCountInOffsets: tile_offsets has one entry more, the count itself (read on the device)
    const int32_t range_end = (tile_id == tile_width * tile_height - 1 && n_isects != kCountInOffsets)
                                  ? (int32_t)n_isects
                                  : tile_offsets[tile_id + 1];
    const uint32_t num_batches = (uint32_t)(range_end - range_start + (int32_t)kFwdBatch - 1) / kFwdBatch;

    bool done = !inside || !ray_ok;
    float T = 1.0f;
    uint32_t cur_idx = 0;
    float pix_out[CDIM];
#pragma unroll
    for (uint32_t k = 0; k < CDIM; ++k)
        pix_out[k] = 0.f;
    uint32_t n_eval = 0, n_comp = 0, n_iter = 0, n_skip = 0, n_hit = 0, n_half_rows = 0, n_half_cols = 0;

    for (uint32_t b = 0; b < num_batches; ++b) {
        // all four waves saturated: nothing left to stage (:190-194)
        if (__syncthreads_and(done))
            break;
        const uint32_t batch_start = (uint32_t)range_start + kFwdBatch * b;
        const uint32_t batch_size = min(kFwdBatch, (uint32_t)range_end - batch_start);
        const bool wave_active = __builtin_amdgcn_ballot_w64(!done) != 0;
        const uint32_t n_sel = stage_and_select<kFwdBatch>(records, flatten_ids, (int32_t)batch_start, 1, batch_size, tr, px, 0u,
                                                wave_active, stage, region, cuts, NX > 0 ? ids : nullptr,
                                                wave_list);
        if (NX > 0) {
            if (tr < batch_size) {
                const float* row = colors + (size_t)ids[tr] * stride + c0;
#pragma unroll
                for (uint32_t k = CDIM - NX; k < CDIM; ++k)
                    extra[tr * (NX ? NX : 1) + (k - (CDIM - NX))] = k < nc ? row[k] : 0.f;
            }
            __syncthreads();
        }
        if (STATS && wave_active)
            n_skip += batch_size - n_sel;

        // A pixel leaves the loop when it is saturated, the wave when its last pixel has (the loop's own divergence:
        // the lane mask shrinks with scalar instructions only; the counting instance keeps the wave-wide form)
        for (uint32_t s = 0; s < n_sel && (STATS || !done); ++s) {
            if (STATS && __builtin_amdgcn_ballot_w64(!done) == 0)
                break; // this wave's 64 pixels are all saturated
            const uint32_t t = wave_list[s];
            if (STATS)
                ++n_iter;
            if (STATS && done)
                continue;
            if (STATS)
                ++n_eval;
            const float4 a = stage[t * 4 + 0];
            const float4 m0 = stage[t * 4 + 1];
            const float4 m1 = stage[t * 4 + 2];
            const float4 m2 = stage[t * 4 + 3];
            vec3 gro = mk3(a.x, a.y, a.z);
            if (rolling) { // M (ray_o - mean), the record's arithmetic
                const vec3 d = sub(ray_o, gro);
                gro = mk3(fma(m0.z, d.z, fma(m0.y, d.y, m0.x * d.x)), fma(m1.y, d.z, fma(m1.x, d.y, m0.w * d.x)),
                          fma(m2.x, d.z, fma(m1.w, d.y, m1.z * d.x)));
            }
            // grd = normalize(M ray_d)
            const vec3 gd = mk3(fma(m0.z, ray_d.z, fma(m0.y, ray_d.y, m0.x * ray_d.x)),
                                fma(m1.y, ray_d.z, fma(m1.x, ray_d.y, m0.w * ray_d.x)),
                                fma(m2.x, ray_d.z, fma(m1.w, ray_d.y, m1.z * ray_d.x)));
            // safe_normalize (Utils.cuh:181-184) without its test: a zero vector times the finite rsqrt(0) of the
            // written-out sequence is the zero vector the test would have left
            const float l2 = dot(gd, gd);
            const vec3 grd = scale(gd, gsx::rsqrt(l2));
            const vec3 gcrod = cross(grd, gro);
            const float grayDist = dot(gcrod, gcrod);
            const float power = -0.5f * grayDist;
            // below the record's cut-off alpha < 1/255 whatever the rounding: decided without the exp
            const bool far_away = power < cuts[t];
            if (STATS) {
                const bool contributes = !far_away && gsx::min_limit(0.999f, a.w * gsx::exp_nonpos(power)) >= 1.f / 255.f;
                const uint64_t act = __builtin_amdgcn_ballot_w64(true);
                const uint64_t cm = __builtin_amdgcn_ballot_w64(contributes);
                if (cm != 0 && (act & ((1ull << (tr & 63u)) - 1ull)) == 0) { // first active lane counts for the wave
                    ++n_hit;
                    // how many 8x4 (rows 0-3 / 4-7) and 4x8 (columns 0-3 / 4-7) halves of the block hold one
                    n_half_rows += ((cm & 0xffffffffull) != 0) + ((cm >> 32) != 0);
                    n_half_cols += ((cm & 0x0f0f0f0f0f0f0f0full) != 0) + ((cm & 0xf0f0f0f0f0f0f0f0ull) != 0);
                }
            }
            if (__builtin_amdgcn_ballot_w64(!far_away) == 0 || far_away)
                continue;
            const float alpha = gsx::min_limit(0.999f, a.w * gsx::exp_nonpos(power)); // cut <= power <= 0
            if (alpha < 1.f / 255.f)
                continue;
            const float next_T = T * (1.0f - alpha);
            if (next_T <= 1e-4f) { // this pixel is done: exclusive
                done = true;
                continue;
            }
            const float vis = alpha * T;
            if (!WIDE) {
                pix_out[0] = fma(m2.y, vis, pix_out[0]);
                if (CDIM > 1)
                    pix_out[1] = fma(m2.z, vis, pix_out[1]);
                if (CDIM > 2)
                    pix_out[2] = fma(m2.w, vis, pix_out[2]);
            }
#pragma unroll
            for (uint32_t k = CDIM - NX; k < CDIM; ++k)
                pix_out[k] = fma(extra[t * (NX ? NX : 1) + (k - (CDIM - NX))], vis, pix_out[k]);
            cur_idx = batch_start + t;
            T = next_T;
            if (STATS)
                ++n_comp;
        }
    }
    if (STATS) {
        if (inside) {
            atomicAdd(&stats[0], (unsigned long long)n_eval);
            atomicAdd(&stats[1], (unsigned long long)n_comp);
            if (n_comp)
                atomicAdd(&stats[2], (unsigned long long)(cur_idx - (uint32_t)range_start + 1u));
        }
        if ((tr & 63u) == 0) {
            atomicAdd(&stats[3], (unsigned long long)n_iter);
            atomicAdd(&stats[4], (unsigned long long)n_skip);
        }
        atomicAdd(&stats[5], (unsigned long long)n_hit);
        atomicAdd(&stats[6], (unsigned long long)n_half_rows);
        atomicAdd(&stats[7], (unsigned long long)n_half_cols);
        return;
    }

    if (inside) {
        if (c0 == 0) {
            render_alphas[pix_id] = 1.0f - T;
            last_ids[pix_id] = (int32_t)cur_idx;
        }
#pragma unroll
        for (uint32_t k = 0; k < CDIM; ++k)
            if (k < nc)
                render_colors[(size_t)pix_id * stride + c0 + k] =
                    backgrounds == nullptr ? pix_out[k] : fma(T, backgrounds[c0 + k], pix_out[k]);
    }
    if (tile_walk != nullptr) {
        // how far into its list this tile's pixels went (entries up to the last contributor): what the tile costs
        // either rasterizer, for the visiting order of later launches
        __shared__ uint32_t walk_s;
        if (tr == 0)
            walk_s = 0;
        __syncthreads();
        uint32_t w = (inside && cur_idx >= (uint32_t)range_start && range_end > range_start && T < 1.0f)
                         ? cur_idx - (uint32_t)range_start + 1u : 0u;
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1)
            w = max(w, (uint32_t)__shfl_xor((int)w, m, 64));
        if ((tr & 63u) == 0)
            atomicMax(&walk_s, w);
        __syncthreads();
        if (tr == 0)
            tile_walk[tile_id] = walk_s;
    }
}

} // namespace gsx

using namespace gsx;

extern "C" size_t gsx_raster_records_bytes(uint32_t N) { return align_up((size_t)N * kRecordFloats * 4, 256); }

namespace gsx {
int pack_raster_records(uint32_t N, const float* means, const float* quats, const float* scales,
                        const float* opacities, const float* colors, uint32_t channels, const float* viewmat,
                        const float* K, uint32_t image_width, uint32_t image_height, bool pinhole, bool rolling,
                        void* records, void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(means && quats && scales && opacities && colors && viewmat && K && records, GSX_ERR_INVALID_ARGUMENT,
                "pack_raster_records: null tensor");
    GSX_REQUIRE(((uintptr_t)records & 15) == 0, GSX_ERR_WORKSPACE, "pack_raster_records: records need 16-byte alignment");
    const dim3 grid(cdiv(N, 256)), block(256);
    hipStream_t s = (hipStream_t)stream;
    GSX_REQUIRE(raster_channels_built(channels), GSX_ERR_UNSUPPORTED,
                "pack_raster_records: %u channels (%s)", channels, kRasterChannelsText);
    hipLaunchKernelGGL(pack_records_kernel, grid, block, 0, s, N, channels, means, quats, scales, opacities, colors,
                       viewmat, K, image_width, image_height, pinhole, rolling, (float4*)records);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

int rasterize_records_fwd(int64_t n_isects, const void* records, const float* colors, uint32_t channels,
                          const float* backgrounds, const uint8_t* masks, uint32_t image_width, uint32_t image_height,
                          const float* viewmat, const float* K, int camera_model, const float* radial,
                          const float* tangential, const float* thin_prism, const float* viewmat1, int rs_type,
                          const int32_t* tile_offsets, const int32_t* flatten_ids, const uint32_t* tile_order,
                          uint32_t* tile_walk, float* render_colors, float* render_alphas, int32_t* last_ids,
                          void* stream) {
    if (image_width == 0 || image_height == 0)
        return GSX_OK;
    GSX_REQUIRE(n_isects >= GSX_COUNT_IN_OFFSETS && n_isects < (1ll << 31), GSX_ERR_OVERFLOW,
                "rasterize fwd: n_isects out of range");
    GSX_REQUIRE(viewmat && K && tile_offsets && render_colors && render_alphas && last_ids, GSX_ERR_INVALID_ARGUMENT,
                "rasterize fwd: null tensor");
    GSX_REQUIRE(n_isects == 0 || (records && flatten_ids && (channels <= 3 || colors)), GSX_ERR_INVALID_ARGUMENT,
                "rasterize fwd: null Gaussian tensor");
    const uint32_t tw = cdiv(image_width, kTile), th = cdiv(image_height, kTile);
    const dim3 grid(tw * th), block(256);
    hipStream_t s = (hipStream_t)stream;
    const bool distorted = camera_model != GSX_PINHOLE || radial != nullptr || tangential != nullptr ||
                           thin_prism != nullptr || rs_type != GSX_GLOBAL || viewmat1 != nullptr;
#define GSX_LAUNCH_FWD(CD, DI)                                                                                      \
    hipLaunchKernelGGL((rasterize_fwd_kernel<CD, false, DI>), grid, block, 0, s, (uint32_t)n_isects,                \
                       (const float4*)records, colors, backgrounds, masks, image_width, image_height, tw, th,       \
                       viewmat, K, camera_model, radial, tangential, thin_prism, viewmat1, rs_type, tile_offsets,   \
                       flatten_ids, tile_order, tile_walk, render_colors, render_alphas, last_ids,                  \
                       (unsigned long long*)nullptr)
#define GSX_LAUNCH_FWD2(CD)     \
    if (distorted)              \
        GSX_LAUNCH_FWD(CD, true); \
    else                        \
        GSX_LAUNCH_FWD(CD, false)
    switch (channels) { // Rasterization.cpp:106-128 up to 32 channels (LichtFeld's render modes use 1, 3, 4)
    case 1: GSX_LAUNCH_FWD2(1); break;
    case 2: GSX_LAUNCH_FWD2(2); break;
    case 3: GSX_LAUNCH_FWD2(3); break;
    case 4: GSX_LAUNCH_FWD2(4); break;
    case 5: GSX_LAUNCH_FWD2(5); break;
    case 8: GSX_LAUNCH_FWD2(8); break;
    case 9: GSX_LAUNCH_FWD2(9); break;
    case 16: GSX_LAUNCH_FWD2(16); break;
    case 17: GSX_LAUNCH_FWD2(17); break;
    case 32: GSX_LAUNCH_FWD2(32); break;
    default:
        if (!raster_channels_built(channels)) {
            set_error("rasterize fwd: %u channels (%s)", channels, kRasterChannelsText);
            return GSX_ERR_UNSUPPORTED;
        }
        // 33 ... 513 channels: 32 of them per launch, counted at run time
        for (uint32_t c0 = 0; c0 < channels; c0 += 32) {
            const uint32_t nc = channels - c0 < 32u ? channels - c0 : 32u;
            uint32_t* const walk = c0 == 0 ? tile_walk : nullptr;
            if (distorted)
                hipLaunchKernelGGL((rasterize_fwd_kernel<32, false, true, true>), grid, block, 0, s, (uint32_t)n_isects,
                                   (const float4*)records, colors, backgrounds, masks, image_width, image_height, tw,
                                   th, viewmat, K, camera_model, radial, tangential, thin_prism, viewmat1, rs_type,
                                   tile_offsets, flatten_ids, tile_order, walk, render_colors, render_alphas, last_ids,
                                   (unsigned long long*)nullptr, channels, c0, nc);
            else
                hipLaunchKernelGGL((rasterize_fwd_kernel<32, false, false, true>), grid, block, 0, s,
                                   (uint32_t)n_isects, (const float4*)records, colors, backgrounds, masks, image_width,
                                   image_height, tw, th, viewmat, K, camera_model, radial, tangential, thin_prism,
                                   viewmat1, rs_type, tile_offsets, flatten_ids, tile_order, walk, render_colors,
                                   render_alphas, last_ids, (unsigned long long*)nullptr, channels, c0, nc);
        }
        break;
    }
#undef GSX_LAUNCH_FWD2
#undef GSX_LAUNCH_FWD
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}
} // namespace gsx

extern "C" int gsx_pack_raster_records(uint32_t N, const float* means, const float* quats, const float* scales,
                                       const float* opacities, const float* colors, uint32_t channels,
                                       const float* viewmat, const float* K, uint32_t image_width,
                                       uint32_t image_height, void* records, void* stream) {
    return pack_raster_records(N, means, quats, scales, opacities, colors, channels, viewmat, K, image_width,
                               image_height, true, false, records, stream);
}

extern "C" int gsx_rasterize_records_fwd(int64_t n_isects, const void* records, const float* colors,
                                         uint32_t channels, const float* backgrounds, const uint8_t* masks,
                                         uint32_t image_width, uint32_t image_height, const float* viewmat,
                                         const float* K, const int32_t* tile_offsets, const int32_t* flatten_ids,
                                         const uint32_t* tile_order, uint32_t* tile_walk, float* render_colors,
                                         float* render_alphas, int32_t* last_ids, void* stream) {
    return rasterize_records_fwd(n_isects, records, colors, channels, backgrounds, masks, image_width, image_height,
                                 viewmat, K, GSX_PINHOLE, nullptr, nullptr, nullptr, nullptr, GSX_GLOBAL, tile_offsets,
                                 flatten_ids, tile_order, tile_walk, render_colors, render_alphas, last_ids, stream);
}

extern "C" int gsx_rasterize_to_pixels_from_world_3dgs_fwd(
    uint32_t C, uint32_t N, int64_t n_isects, const float* means, const float* quats, const float* scales,
    const float* colors, uint32_t channels, const float* opacities, const float* backgrounds, const uint8_t* masks,
    uint32_t image_width, uint32_t image_height, uint32_t tile_size, const float* viewmats0, const float* viewmats1,
    const float* Ks, int camera_model, gsx_ut_params ut, int rs_type, const float* radial_coeffs,
    const float* tangential_coeffs, const float* thin_prism_coeffs, const int32_t* tile_offsets,
    const int32_t* flatten_ids, float* render_colors, float* render_alphas, int32_t* last_ids, void* workspace,
    size_t workspace_bytes, void* stream) {
    (void)ut;
    int rc = check_camera_args(C, viewmats1, camera_model, rs_type, radial_coeffs, tangential_coeffs,
                               thin_prism_coeffs);
    if (rc != GSX_OK)
        return rc;
    if (image_width == 0 || image_height == 0)
        return GSX_OK;
    GSX_REQUIRE(tile_size == kTile, GSX_ERR_UNSUPPORTED, "rasterize fwd: tile_size %u (only 16 is built)", tile_size);
    GSX_REQUIRE(raster_channels_built(channels), GSX_ERR_UNSUPPORTED,
                "rasterize fwd: %u channels (%s)", channels, kRasterChannelsText);
    GSX_REQUIRE(viewmats0 && Ks, GSX_ERR_INVALID_ARGUMENT, "rasterize fwd: null tensor");
    GSX_REQUIRE(n_isects == 0 || (means && quats && scales && colors && opacities && flatten_ids),
                GSX_ERR_INVALID_ARGUMENT, "rasterize fwd: null Gaussian tensor");
    if (n_isects > 0) {
        GSX_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0 &&
                        workspace_bytes >= gsx_raster_records_bytes(N),
                    GSX_ERR_WORKSPACE, "rasterize fwd: workspace needs %zu bytes, 256-byte aligned",
                    gsx_raster_records_bytes(N));
        const bool rolling = rs_type != GSX_GLOBAL;
        const bool pinhole = camera_model == GSX_PINHOLE && !(radial_coeffs || tangential_coeffs || thin_prism_coeffs) &&
                             !rolling;
        if ((rc = pack_raster_records(N, means, quats, scales, opacities, colors, channels, viewmats0, Ks, image_width,
                                      image_height, pinhole, rolling, workspace, stream)) != GSX_OK)
            return rc;
    }
    // room behind the records for a tile order: visit the tiles longest list first
    const uint32_t* tile_order = nullptr;
    const uint32_t tw = cdiv(image_width, kTile), th = cdiv(image_height, kTile);
    const size_t rec_bytes = gsx_raster_records_bytes(N);
    if (n_isects > 0 && tile_offsets != nullptr && workspace_bytes >= rec_bytes + gsx_tile_order_bytes(tw, th)) {
        uint32_t* order = (uint32_t*)((char*)workspace + rec_bytes);
        if ((rc = gsx_tile_order(n_isects, tile_offsets, nullptr, tw, th, order, stream)) != GSX_OK)
            return rc;
        tile_order = order;
    }
    return rasterize_records_fwd(n_isects, workspace, colors, channels, backgrounds, masks, image_width, image_height,
                                 viewmats0, Ks, camera_model, radial_coeffs, tangential_coeffs, thin_prism_coeffs,
                                 viewmats1, rs_type, tile_offsets, flatten_ids, tile_order, nullptr, render_colors,
                                 render_alphas, last_ids, stream);
}

// Pair counts of one forward pass (no counterpart in the reference; used to turn kernel times into flop rates).
extern "C" int gsx_rasterize_pair_stats(int64_t n_isects, const void* records, uint32_t image_width,
                                        uint32_t image_height, const float* viewmat, const float* K,
                                        const int32_t* tile_offsets, const int32_t* flatten_ids,
                                        unsigned long long* stats_out, void* stream) {
    if (image_width == 0 || image_height == 0 || n_isects <= 0)
        return GSX_OK;
    GSX_REQUIRE(records && viewmat && K && tile_offsets && flatten_ids && stats_out, GSX_ERR_INVALID_ARGUMENT,
                "rasterize_pair_stats: null tensor");
    const uint32_t tw = cdiv(image_width, kTile), th = cdiv(image_height, kTile);
    hipLaunchKernelGGL((rasterize_fwd_kernel<3, true, false>), dim3(tw * th), dim3(256), 0, (hipStream_t)stream,
                       (uint32_t)n_isects, (const float4*)records, (const float*)nullptr, (const float*)nullptr,
                       (const uint8_t*)nullptr, image_width, image_height, tw, th, viewmat, K, (int)GSX_PINHOLE,
                       (const float*)nullptr, (const float*)nullptr, (const float*)nullptr, (const float*)nullptr,
                       (int)GSX_GLOBAL, tile_offsets, flatten_ids, (const uint32_t*)nullptr, (uint32_t*)nullptr,
                       (float*)nullptr,
                       (float*)nullptr, (int32_t*)nullptr, stats_out);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}
