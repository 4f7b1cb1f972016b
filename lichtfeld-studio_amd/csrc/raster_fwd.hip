// raster_fwd.hip - per-tile forward rasterizer "from world" (gsplat/RasterizeToPixelsFromWorld3DGSFwd.cu:19-285).
//
// One 256-lane workgroup (four 64-lane waves) per 16x16 tile, one lane per pixel; wave w owns pixel rows
// 4w..4w+3.  The tile's depth-sorted Gaussians are staged through LDS in batches of 256: each lane loads one
// Gaussian, builds M = diag(1/scale) R(quat)^T once, and stores {xyz, opacity, M, rgb} (64 B, four
// ds_write_b128).  The compositing loop then reads each staged Gaussian with wave-uniform addresses (LDS
// broadcast, no bank conflicts), evaluates the ray/Gaussian response with explicit FMAs and composites front
// to back.  Colours ride along in LDS so the inner loop never touches global memory.  A wave leaves the batch
// loop as soon as all of its 64 pixels are saturated; the workgroup stops staging when all four waves are.
#include "gsx_common.h"

namespace gsx {

static constexpr uint32_t kTile = 16;
static constexpr uint32_t kBatch = 256;
static constexpr float kPowerCut = -5.55f; // exp(-5.55) = 3.8875e-3 < 1/255 = 3.9216e-3

// STATS: also count the (pixel, Gaussian) pairs this launch evaluates / composites (for roofline accounting);
// stats[0] += pairs evaluated, stats[1] += pairs composited, stats[2] += pairs the backward pass will evaluate
// (entries up to each pixel's last contributor).
template <uint32_t CDIM, bool STATS>
__global__ void __launch_bounds__(256) rasterize_fwd_kernel(
    uint32_t n_isects, const float* __restrict__ means, const float* __restrict__ quats,
    const float* __restrict__ scales, const float* __restrict__ colors, const float* __restrict__ opacities,
    const float* __restrict__ backgrounds, const uint8_t* __restrict__ masks, uint32_t image_width,
    uint32_t image_height, uint32_t tile_width, uint32_t tile_height, const float* __restrict__ viewmat,
    const float* __restrict__ Kmat, const int32_t* __restrict__ tile_offsets,
    const int32_t* __restrict__ flatten_ids, float* __restrict__ render_colors, float* __restrict__ render_alphas,
    int32_t* __restrict__ last_ids, unsigned long long* __restrict__ stats) {
    __shared__ float4 stage[kBatch * 4];
    __shared__ float extra[CDIM > 3 ? kBatch * (CDIM - 3) : 1]; // channels beyond the third

    const uint32_t tile_id = blockIdx.x;
    const uint32_t ty = tile_id / tile_width, tx = tile_id % tile_width;
    const uint32_t tr = threadIdx.x;
    const uint32_t i = ty * kTile + (tr >> 4);
    const uint32_t j = tx * kTile + (tr & 15u);
    const bool inside = (i < image_height && j < image_width);
    const uint32_t pix_id = i * image_width + j;

    // :147-155 masked tile: background colour only
    if (masks != nullptr && !masks[tile_id]) {
        if (inside) {
#pragma unroll
            for (uint32_t k = 0; k < CDIM; ++k)
                render_colors[(size_t)pix_id * CDIM + k] = backgrounds == nullptr ? 0.0f : backgrounds[k];
        }
        return;
    }

    const CamPose cp = load_cam_pose(viewmat);
    vec3 ray_o, ray_d;
    pixel_world_ray(cp, (float)j + 0.5f, (float)i + 0.5f, Kmat[0], Kmat[4], Kmat[2], Kmat[5], &ray_o, &ray_d);

    const int32_t range_start = tile_offsets[tile_id];
    const int32_t range_end =
        (tile_id == tile_width * tile_height - 1) ? (int32_t)n_isects : tile_offsets[tile_id + 1];
    const uint32_t num_batches = (uint32_t)(range_end - range_start + (int32_t)kBatch - 1) / kBatch;

    bool done = !inside;
    float T = 1.0f;
    uint32_t cur_idx = 0;
    float pix_out[CDIM];
#pragma unroll
    for (uint32_t k = 0; k < CDIM; ++k)
        pix_out[k] = 0.f;
    uint32_t n_eval = 0, n_comp = 0;

    for (uint32_t b = 0; b < num_batches; ++b) {
        // all four waves saturated: nothing left to stage (:190-194)
        if (__syncthreads_and(done))
            break;
        const uint32_t batch_start = (uint32_t)range_start + kBatch * b;
        const uint32_t idx = batch_start + tr;
        if (idx < (uint32_t)range_end) {
            const int32_t g = flatten_ids[idx];
            const vec3 xyz = ld3(means, g);
            const float opac = opacities[g];
            const mat3 R = quat_to_rotmat(ld4q(quats, g));
            const vec3 s = ld3(scales, g);
            const float is0 = 1.0f / s.x, is1 = 1.0f / s.y, is2 = 1.0f / s.z;
            // M = diag(1/s) R^T  (:214-226)
            float c0 = 0.f, c1 = 0.f, c2 = 0.f;
            c0 = colors[(size_t)g * CDIM];
            if (CDIM > 1)
                c1 = colors[(size_t)g * CDIM + 1];
            if (CDIM > 2)
                c2 = colors[(size_t)g * CDIM + 2];
            // gro = M (ray_o - mean) does not depend on the pixel (one ray origin per global-shutter camera): it is
            // formed here, once per staged Gaussian, with the arithmetic of the per-pair formula
            mat3 M;
            M.m[0][0] = is0 * R.m[0][0], M.m[0][1] = is0 * R.m[1][0], M.m[0][2] = is0 * R.m[2][0];
            M.m[1][0] = is1 * R.m[0][1], M.m[1][1] = is1 * R.m[1][1], M.m[1][2] = is1 * R.m[2][1];
            M.m[2][0] = is2 * R.m[0][2], M.m[2][1] = is2 * R.m[1][2], M.m[2][2] = is2 * R.m[2][2];
            const vec3 gro = mul(M, sub(ray_o, xyz));
            stage[tr * 4 + 0] = make_float4(gro.x, gro.y, gro.z, opac);
            stage[tr * 4 + 1] = make_float4(M.m[0][0], M.m[0][1], M.m[0][2], M.m[1][0]);
            stage[tr * 4 + 2] = make_float4(M.m[1][1], M.m[1][2], M.m[2][0], M.m[2][1]);
            stage[tr * 4 + 3] = make_float4(M.m[2][2], c0, c1, c2);
#pragma unroll
            for (uint32_t k = 3; k < CDIM; ++k)
                extra[tr * (CDIM > 3 ? CDIM - 3 : 1) + (k - 3)] = colors[(size_t)g * CDIM + k];
        }
        __syncthreads();

        const uint32_t batch_size = min(kBatch, (uint32_t)range_end - batch_start);
        for (uint32_t t = 0; t < batch_size; ++t) {
            if (__builtin_amdgcn_ballot_w64(!done) == 0)
                break; // this wave's 64 pixels are all saturated
            if (done)
                continue;
            if (STATS)
                ++n_eval;
            const float4 a = stage[t * 4 + 0];
            const float4 m0 = stage[t * 4 + 1];
            const float4 m1 = stage[t * 4 + 2];
            const float4 m2 = stage[t * 4 + 3];
            const vec3 gro = mk3(a.x, a.y, a.z);
            // grd = normalize(M ray_d)
            const vec3 gd = mk3(fma(m0.z, ray_d.z, fma(m0.y, ray_d.y, m0.x * ray_d.x)),
                                fma(m1.y, ray_d.z, fma(m1.x, ray_d.y, m0.w * ray_d.x)),
                                fma(m2.x, ray_d.z, fma(m1.w, ray_d.y, m1.z * ray_d.x)));
            const vec3 grd = safe_normalize(gd);
            const vec3 gcrod = cross(grd, gro);
            const float grayDist = dot(gcrod, gcrod);
            const float power = -0.5f * grayDist;
            // exp(power) < 1/255 below kPowerCut, so alpha < 1/255 for any opacity <= 1: decided without the exp
            const bool far_away = power < kPowerCut && a.w <= 1.0f;
            if (STATS) {
                const uint64_t act = __builtin_amdgcn_ballot_w64(true);
                const uint64_t nearm = __builtin_amdgcn_ballot_w64(!far_away);
                if ((act & ((1ull << (threadIdx.x & 63u)) - 1ull)) == 0) { // first active lane of the wave
                    atomicAdd(&stats[3], 1ull);
                    if (nearm)
                        atomicAdd(&stats[4], 1ull);
                }
            }
            if (__builtin_amdgcn_ballot_w64(!far_away) == 0 || far_away)
                continue;
            const float alpha = gsx::fmin(0.999f, a.w * gsx::exp(power));
            if (alpha < 1.f / 255.f)
                continue;
            const float next_T = T * (1.0f - alpha);
            if (next_T <= 1e-4f) { // this pixel is done: exclusive
                done = true;
                continue;
            }
            const float vis = alpha * T;
            pix_out[0] = fma(m2.y, vis, pix_out[0]);
            if (CDIM > 1)
                pix_out[1] = fma(m2.z, vis, pix_out[1]);
            if (CDIM > 2)
                pix_out[2] = fma(m2.w, vis, pix_out[2]);
#pragma unroll
            for (uint32_t k = 3; k < CDIM; ++k)
                pix_out[k] = fma(extra[t * (CDIM > 3 ? CDIM - 3 : 1) + (k - 3)], vis, pix_out[k]);
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
        return;
    }

    if (inside) {
        render_alphas[pix_id] = 1.0f - T;
#pragma unroll
        for (uint32_t k = 0; k < CDIM; ++k)
            render_colors[(size_t)pix_id * CDIM + k] =
                backgrounds == nullptr ? pix_out[k] : fma(T, backgrounds[k], pix_out[k]);
        last_ids[pix_id] = (int32_t)cur_idx;
    }
}

} // namespace gsx

using namespace gsx;

extern "C" int gsx_rasterize_to_pixels_from_world_3dgs_fwd(
    uint32_t C, uint32_t N, int64_t n_isects, const float* means, const float* quats, const float* scales,
    const float* colors, uint32_t channels, const float* opacities, const float* backgrounds, const uint8_t* masks,
    uint32_t image_width, uint32_t image_height, uint32_t tile_size, const float* viewmats0, const float* viewmats1,
    const float* Ks, int camera_model, gsx_ut_params ut, int rs_type, const float* radial_coeffs,
    const float* tangential_coeffs, const float* thin_prism_coeffs, const int32_t* tile_offsets,
    const int32_t* flatten_ids, float* render_colors, float* render_alphas, int32_t* last_ids, void* stream) {
    (void)ut;
    (void)N;
    const int rc = check_camera_args(C, viewmats1, camera_model, rs_type, radial_coeffs, tangential_coeffs,
                                     thin_prism_coeffs);
    if (rc != GSX_OK)
        return rc;
    if (image_width == 0 || image_height == 0)
        return GSX_OK;
    GSX_REQUIRE(tile_size == kTile, GSX_ERR_UNSUPPORTED, "rasterize fwd: tile_size %u (only 16 is built)", tile_size);
    GSX_REQUIRE(n_isects >= 0 && n_isects < (1ll << 31), GSX_ERR_OVERFLOW, "rasterize fwd: n_isects out of range");
    GSX_REQUIRE(viewmats0 && Ks && tile_offsets && render_colors && render_alphas && last_ids,
                GSX_ERR_INVALID_ARGUMENT, "rasterize fwd: null tensor");
    GSX_REQUIRE(n_isects == 0 || (means && quats && scales && colors && opacities && flatten_ids),
                GSX_ERR_INVALID_ARGUMENT, "rasterize fwd: null Gaussian tensor");
    const uint32_t tw = cdiv(image_width, kTile), th = cdiv(image_height, kTile);
    const dim3 grid(tw * th), block(256);
    hipStream_t s = (hipStream_t)stream;
#define GSX_LAUNCH_FWD(CD)                                                                                         \
    hipLaunchKernelGGL((rasterize_fwd_kernel<CD, false>), grid, block, 0, s, (uint32_t)n_isects, means, quats, scales, \
                       colors, opacities, backgrounds, masks, image_width, image_height, tw, th, viewmats0, Ks,        \
                       tile_offsets, flatten_ids, render_colors, render_alphas, last_ids,                              \
                       (unsigned long long*)nullptr)
    switch (channels) { // the channel counts the render modes of Rasterization.cpp:374-393 produce
    case 1: GSX_LAUNCH_FWD(1); break;
    case 3: GSX_LAUNCH_FWD(3); break;
    case 4: GSX_LAUNCH_FWD(4); break;
    default:
        set_error("rasterize fwd: %u channels (built: 1, 3, 4)", channels);
        return GSX_ERR_UNSUPPORTED;
    }
#undef GSX_LAUNCH_FWD
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

// Pair counts of one forward pass (no counterpart in the reference; used to turn kernel times into flop rates).
// stats_out: three device uint64 {pairs evaluated by the forward, pairs composited, pairs the backward evaluates};
// they are ADDED to, so zero them first.
extern "C" int gsx_rasterize_pair_stats(uint32_t N, int64_t n_isects, const float* means, const float* quats,
                                        const float* scales, const float* opacities, uint32_t image_width,
                                        uint32_t image_height, const float* viewmat, const float* K,
                                        const int32_t* tile_offsets, const int32_t* flatten_ids,
                                        unsigned long long* stats_out, void* stream) {
    (void)N;
    if (image_width == 0 || image_height == 0 || n_isects <= 0)
        return GSX_OK;
    GSX_REQUIRE(means && quats && scales && opacities && viewmat && K && tile_offsets && flatten_ids && stats_out,
                GSX_ERR_INVALID_ARGUMENT, "rasterize_pair_stats: null tensor");
    const uint32_t tw = cdiv(image_width, kTile), th = cdiv(image_height, kTile);
    // colours are not needed for counting: the means array stands in (3 floats per Gaussian, same layout)
    hipLaunchKernelGGL((rasterize_fwd_kernel<3, true>), dim3(tw * th), dim3(256), 0, (hipStream_t)stream,
                       (uint32_t)n_isects, means, quats, scales, means, opacities, (const float*)nullptr,
                       (const uint8_t*)nullptr, image_width, image_height, tw, th, viewmat, K, tile_offsets,
                       flatten_ids, (float*)nullptr, (float*)nullptr, (int32_t*)nullptr, stats_out);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}
