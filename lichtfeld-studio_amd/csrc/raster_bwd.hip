// raster_bwd.hip - per-tile backward rasterizer "from world"
// (gsplat/RasterizeToPixelsFromWorld3DGSBwd.cu:16-379, VJP helpers gsplat/Utils.cuh:104-158,186-194).
//
// Same tiling as the forward pass (one 256-lane workgroup per 16x16 tile, one lane per pixel, Gaussians staged
// through LDS 128 at a time, walked back to front).  Two things are organised differently from the reference:
//
//  1. What is summed per Gaussian.  The reference pushes every (pixel, Gaussian) pair through the whole chain
//     down to (v_mean, v_quat, v_scale) and reduces those 10 numbers.  That chain is linear in v_M = d L / d M
//     (M = diag(1/s) R^T), and v_M = v_grd (x) ray_d + v_gro (x) (ray_o - mean) reduces exactly to k q (x) M^-1 q
//     with q the nearest point of the pixel's ray to the centre in the Gaussian's frame (derivation at the loop).
//     So the per-pair work stops at k q (3) and the symmetric k q (x) q (6); those are summed per Gaussian (with
//     colour 3 and opacity 1: 13 of the 16 floats of a row) and a per-Gaussian epilogue applies the linear map once.
//  2. How it is summed.  A 64-lane wave reduces its 16 partials with a halving butterfly (the array is split in
//     two at each of the first four steps, so 8+4+2+1+1+1 = 17 exchanges instead of 16*6), after which 16 lanes
//     hold one total each and add it to the workgroup's LDS accumulators; the workgroup flushes one 64-byte row
//     per Gaussian to global memory with a single coalesced atomic-add instruction per four Gaussians.
//
// Sums are formed in a different order than the reference's warp reduce + atomics (whose order is itself
// unspecified), so results agree to rounding, not bitwise.
#include "gsx_common.h"
#include "gsx_wave.h"
#include "gsx_step.h"

namespace gsx {

static constexpr uint32_t kBwdBatch = 128; // list entries staged at a time (256: 1.5 % longer at 1 M Gaussians, 4 - 5 % at 3 M and 6 M)

static constexpr uint32_t kAcc = 16; // floats per Gaussian: rgb 3, k q 3, k q (x) q 6 (symmetric), 3 unused, opacity 1

__global__ void __launch_bounds__(256) fill_f32_kernel(size_t n, float v, float* __restrict__ out) {
    const size_t i = (size_t)blockIdx.x * 256u + threadIdx.x;
    if (i < n)
        out[i] = v;
}

// probe of the wave reductions for tests: in [n_waves][64 lanes][V], out [n_waves][V], V = 16, 13 or 9
template <uint32_t V>
__global__ void __launch_bounds__(64) wave_reduce_probe_kernel(const float* __restrict__ in, float* __restrict__ out) {
    float v[V];
    const uint32_t lane = threadIdx.x;
#pragma unroll
    for (uint32_t k = 0; k < V; ++k)
        v[k] = in[((size_t)blockIdx.x * 64 + lane) * V + k];
    float total;
    uint32_t index;
    if constexpr (V == 16) {
        total = wave_reduce16(v, lane);
        index = wave_component(lane);
    } else if constexpr (V == 13) {
        total = wave_reduce13(v, lane);
        index = wave_reduce13_index(lane);
    } else {
        total = wave_reduce9(v, lane);
        index = wave_reduce9_index(lane);
    }
    if ((lane & 3u) == 0 && index < V)
        out[(size_t)blockIdx.x * V + index] = total;
}

// CDIM = 3: the RGB training path.  CDIM = 1 / 4: the depth render modes (Rasterization.cpp:374-393).  Channels
// beyond the third are staged from `colors`, and their per-Gaussian gradients are reduced on their own into gextra
// [N, CDIM - 3].
// STATS: count instead of differentiating (for roofline accounting): stats[0] += pairs whose alpha is evaluated,
// [1] += valid pairs, [2] += (wave, Gaussian) iterations executed.
// WIDE: more than 32 channels, CDIM (= 32) of them per launch: channels [c0, c0 + nc) of rows `stride` floats long,
// every one read from `colors`.  Every sum of a row is linear in the image gradient, so each launch adds the share
// of its own channels (the launch with c0 = 0 also that of the alpha gradient) to the same accumulators.
template <uint32_t CDIM, bool DIST, bool STATS = false, bool WIDE = false>
__global__ void __launch_bounds__(256) rasterize_bwd_kernel(
    uint32_t n_isects, const float4* __restrict__ records, const float* __restrict__ colors,
    const float* __restrict__ backgrounds,
    const uint8_t* __restrict__ masks, uint32_t image_width, uint32_t image_height, uint32_t tile_width,
    uint32_t tile_height, const float* __restrict__ viewmat, const float* __restrict__ Kmat,
    int camera_model, const float* __restrict__ radial, const float* __restrict__ tangential,
    const float* __restrict__ thin_prism, const float* __restrict__ viewmat1, int rs_type,
    const int32_t* __restrict__ tile_offsets, const uint32_t* __restrict__ tile_order /*nullable*/,
    const int32_t* __restrict__ flatten_ids,
    const float* __restrict__ render_alphas, const int32_t* __restrict__ last_ids,
    const float* __restrict__ v_render_colors, const float* __restrict__ v_render_alphas,
    float* __restrict__ gacc /*[N,16]*/, float* __restrict__ gextra /*[N, CDIM - 3]*/,
    unsigned long long* __restrict__ stats = nullptr, uint32_t stride = CDIM, uint32_t c0 = 0, uint32_t nc = CDIM) {
    static_assert(!WIDE || (CDIM == 32 && !STATS), "the wide instance takes 32 channels a launch");
    if (!WIDE)
        stride = CDIM, c0 = 0, nc = CDIM;
    constexpr uint32_t NC = WIDE ? 0 : (CDIM < 3 ? CDIM : 3); // channels carried by the record
    __shared__ float4 stage[kBwdBatch * 4];
    constexpr uint32_t NX = CDIM - NC; // channels read from `colors`: those beyond the record's three (WIDE: all)
    // up to six of them are staged and accumulated in LDS; beyond that (16 channels and more: not a training path)
    // their colours are read from memory in the loop and every wave adds its sums to memory itself
    constexpr bool XLDS = NX > 0 && NX <= 6;
    __shared__ float extra[XLDS ? kBwdBatch * NX : 1];
    __shared__ float acc_extra[XLDS ? kBwdBatch * NX : 1];
    __shared__ float cuts[kBwdBatch];
    __shared__ uint8_t lists[4][kBwdBatch];
    __shared__ int32_t id_batch[kBwdBatch]; // ids of the batch: for the flush and the extra channels' paths
    // LDS sums of a batch: the 13 numbers in use of a row (slot 12 holds the opacity sum, the row's element 15)
    constexpr uint32_t kAccLds = 13;
    __shared__ __align__(16) float acc[kBwdBatch * kAccLds];
    // the region tests of a batch are over before its first sum is formed: their operands lie in the accumulators'
    // bytes (8 KB less per workgroup: four workgroups per CU instead of three)
    float4* const region = reinterpret_cast<float4*>(acc);
    __shared__ int32_t block_max;

    const uint32_t tile_id = tile_order != nullptr ? tile_order[blockIdx.x] : blockIdx.x;
    if (masks != nullptr && !masks[tile_id]) // :83-87
        return;
    const uint32_t tr = threadIdx.x;
    const uint32_t lane = tr & 63u;
    // which of the 13 per-Gaussian sums this lane ends up with after the wave reduction (15: none)
    const uint32_t sum_index = (lane & 3u) == 0 ? wave_reduce13_index(lane) : 15u;
    const TilePixel px = tile_pixel(tile_id, tile_width, tr);
    const uint32_t i = px.i, j = px.j;
    bool inside = (i < image_height && j < image_width);
    const uint32_t pix_id = min(i * image_width + j, image_width * image_height - 1); // :92-93
    uint8_t* wave_list = lists[tr >> 6];

    const CamPose cp = DIST ? load_cam_pose(viewmat, viewmat1, rs_type, image_width, image_height) : load_cam_pose(viewmat);
    // rolling shutter: the records carry the means and every pixel has its own ray origin
    const bool rolling = DIST && rs_type != GSX_GLOBAL;
    vec3 ray_o, ray_d;
    CameraModel cam;
    cam.type = 0, cam.dist.on = false;
    if (DIST)
        cam = load_camera_model(camera_model, radial, tangential, thin_prism, Kmat[0], Kmat[4], Kmat[2], Kmat[5],
                                image_width, image_height);
    // a pixel without a valid ray takes no part (RasterizeToPixelsFromWorld3DGSBwd.cu:157)
    inside &= pixel_world_ray(cp, (float)j + 0.5f, (float)i + 0.5f, Kmat[0], Kmat[4], Kmat[2], Kmat[5], cam, &ray_o,
                              &ray_d);

    const int32_t range_start = tile_offsets[tile_id];
    int32_t range_end = (tile_id == tile_width * tile_height - 1 && n_isects != kCountInOffsets)
                            ? (int32_t)n_isects
                            : tile_offsets[tile_id + 1];

    const float T_final = 1.0f - render_alphas[pix_id];
    float T = T_final;

    const int32_t bin_final = inside ? last_ids[pix_id] : 0;
    float v_render_c[CDIM];
#pragma unroll
    for (uint32_t k = 0; k < CDIM; ++k)
        v_render_c[k] = (STATS || k >= nc) ? 0.f : v_render_colors[(size_t)pix_id * stride + c0 + k];
    const float v_render_a = (STATS || c0 != 0) ? 0.f : v_render_alphas[pix_id];
    float bg_dot = 0.f;
    if (backgrounds != nullptr) {
#pragma unroll
        for (uint32_t k = 0; k < CDIM; ++k)
            if (k < nc)
                bg_dot += backgrounds[c0 + k] * v_render_c[k];
    }
    // what ra multiplies in v_alpha: T_final (v_render_a - bg . v_render) (:313-321) minus sum_k buffer_k v_render_k
    // (:186, :309), which starts at zero and is updated in the loop
    float behind = T_final * (v_render_a - bg_dot);

    // last contributing list entry over the wave (:201-203) and over the workgroup: entries behind the
    // workgroup's maximum are needed by no pixel, so the walk starts there
    int32_t wave_bin_final = bin_final;
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1)
        wave_bin_final = max(wave_bin_final, __shfl_xor(wave_bin_final, m, 64));
    wave_bin_final = __builtin_amdgcn_readfirstlane(wave_bin_final); // the same in every lane: keep it scalar
    if (tr == 0)
        block_max = 0;
    __syncthreads();
    if (lane == 0)
        atomicMax(&block_max, wave_bin_final);
    if (XLDS && tr < kBwdBatch) {
#pragma unroll
        for (uint32_t k = 0; k < NX; ++k)
            acc_extra[tr * (NX ? NX : 1) + k] = 0.f;
    }
    __syncthreads();
    range_end = min(range_end, block_max + 1);
    if (range_end <= range_start)
        return;
    const uint32_t num_batches = (uint32_t)(range_end - range_start + (int32_t)kBwdBatch - 1) / kBwdBatch;
    uint32_t n_eval = 0, n_valid = 0, n_iter = 0;
    const uint64_t inside_mask = __builtin_amdgcn_ballot_w64(inside);

    for (uint32_t b = 0; b < num_batches; ++b) {
        // back to front: slot 0 of the batch is the farthest Gaussian (:211-216)
        const int32_t batch_end = range_end - 1 - (int32_t)(kBwdBatch * b);
        const int32_t batch_size = min((int32_t)kBwdBatch, batch_end + 1 - range_start);
        // slots in front of t_start lie behind every last contributor of this wave
        const uint32_t t_start = (uint32_t)max(0, batch_end - wave_bin_final);
        const uint32_t n_sel = (uint32_t)__builtin_amdgcn_readfirstlane((int)stage_and_select<kBwdBatch>(
            records, flatten_ids, batch_end, -1, (uint32_t)batch_size, tr, px, t_start,
            t_start < (uint32_t)batch_size, stage, region, cuts, id_batch, wave_list));
        for (uint32_t k = tr; k < kBwdBatch * kAccLds / 4; k += 256u)
            reinterpret_cast<float4*>(acc)[k] = make_float4(0.f, 0.f, 0.f, 0.f);
        __syncthreads();
        if (XLDS) {
            if ((int32_t)tr < batch_size) {
#pragma unroll
                for (uint32_t k = 0; k < NX; ++k)
                    extra[tr * (NX ? NX : 1) + k] = colors[(size_t)id_batch[tr] * stride + NC + k];
            }
            __syncthreads();
        }

        for (uint32_t sidx = 0; sidx < n_sel; ++sidx) {
            const int32_t t = (int32_t)wave_list[sidx];
            bool valid = inside && (batch_end - t <= bin_final);
            const uint64_t reach_mask = __builtin_amdgcn_ballot_w64(batch_end - t <= bin_final) & inside_mask;
            if (STATS) {
                n_eval += (uint32_t)__popcll(__builtin_amdgcn_ballot_w64(valid));
                ++n_iter;
            }
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
            const vec3 grd = mk3(fma(m0.z, ray_d.z, fma(m0.y, ray_d.y, m0.x * ray_d.x)),
                                 fma(m1.y, ray_d.z, fma(m1.x, ray_d.y, m0.w * ray_d.x)),
                                 fma(m2.x, ray_d.z, fma(m1.w, ray_d.y, m1.z * ray_d.x)));
            // safe_normalize (Utils.cuh:181-184) without its test: a zero vector times the finite rsqrt(0) of the
            // written-out sequence is the zero vector the test would have left
            const float l2 = dot(grd, grd);
            const vec3 grd_n = scale(grd, gsx::rsqrt(l2));
            const vec3 gcrod = cross(grd_n, gro);
            const float grayDist = dot(gcrod, gcrod);
            const float power = -0.5f * grayDist;
            // below the record's cut-off alpha < 1/255 whatever the rounding: decided without the exp
            // (the wave-wide tests combine the comparisons' own lane masks: a ballot of the combined flag would first
            // turn it into a register and compare that again)
            const bool near = !(power < cuts[t]);
            const uint64_t near_mask = __builtin_amdgcn_ballot_w64(near);
            valid = valid && near;
            if ((reach_mask & near_mask) == 0)
                continue;
            // (a lane below its cut-off may be far outside exp_nonpos's range: what it gets back is meaningless and
            // stays in that lane - it is not valid, and everything it feeds below goes through a select on `valid`)
            const float vis = gsx::exp_nonpos(power);
            const float alpha = gsx::min_limit(0.999f, a.w * vis);
            // (the reference's `power > 0` never fires: the power is -0.5 times a sum of squares)
            const bool opaque_enough = !(alpha < 1.f / 255.f);
            const uint64_t alpha_mask = __builtin_amdgcn_ballot_w64(opaque_enough);
            valid = valid && opaque_enough;
            if ((reach_mask & near_mask & alpha_mask) == 0)
                continue; // no lane of this wave sees the Gaussian (:286-289)
            if (STATS) {
                n_valid += (uint32_t)__popcll(__builtin_amdgcn_ballot_w64(valid));
                continue;
            }

            // From here on without branches: a lane that is not valid carries ra = 1 and fac = v_alpha = 0, which
            // leaves its T and colour buffer unchanged and makes all 13 of its partials zero.  The decisions above
            // use the forward pass's exact arithmetic; the derivative chain may use the (refined) hardware reciprocal.
            float v[13]; // colours 0-2, k q 3-5, k q (x) q 6-11, opacity 12
            const float ra = valid ? gsx::rcp_refined(1.0f - alpha) : 1.0f;
            T *= ra;
            const float fac = valid ? alpha * T : 0.f;
            const float col[3] = {m2.y, m2.z, m2.w};
            v[0] = NC > 0 ? fac * v_render_c[0] : 0.f;
            v[1] = NC > 1 ? fac * v_render_c[NC > 1 ? 1 : 0] : 0.f;
            v[2] = NC > 2 ? fac * v_render_c[NC > 2 ? 2 : 0] : 0.f;
            // The derivative chain is written with fused multiply-adds (the compiler does not contract on its own
            // here) and folded algebraically; same values as the reference's chain up to rounding, fewer instructions
            // in the loop that bounds the step.
            // Colours: sum_k (c_k T - buffer_k ra) v_render_k (:306-311) = T cdot - ra bdot with cdot = sum_k c_k
            // v_render_k and bdot = sum_k buffer_k v_render_k; buffer_k grows by c_k fac per Gaussian (:343), so bdot
            // grows by cdot fac.  `behind` = T_final (v_render_a - bg . v_render) - bdot collects everything ra
            // multiplies (:313-321): one running scalar per pixel instead of one per channel.
            float cdot = NC > 0 ? col[0] * v_render_c[0] : 0.f;
#pragma unroll
            for (uint32_t k = 1; k < NC; ++k)
                cdot = fma(col[k], v_render_c[k], cdot);
            // (a row of `colors` is the same for the whole wave: the compiler reads it through the scalar path)
            const float* const crow = NX > 0 && !XLDS ? colors + (size_t)id_batch[t] * stride + c0 + NC : nullptr;
#pragma unroll
            for (uint32_t k = 0; k < NX; ++k)
                if (NC + k < nc)
                    cdot = fma(XLDS ? extra[(uint32_t)t * (NX ? NX : 1) + k] : crow[k], v_render_c[NX ? NC + k : 0],
                               cdot);
            const float v_alpha = fma(T, cdot, ra * behind);
            // the clamp at 0.999 has zero derivative (:322)
            const float v_opac = (valid && a.w * vis <= 0.999f) ? vis * v_alpha : 0.f;
            // Geometry (:325-345).  With n = grd / |grd|, g = gro and q = g - (g . n) n (the point of the pixel's ray
            // nearest the Gaussian's centre, in the Gaussian's frame) the reference's chain is, exactly,
            //   v_gro = k q,   v_grd = t v_gro,   k = -opacity v_opacity,   t = -(g . n) / |grd|,
            // and t is the ray parameter of that nearest point p: ray_o + t ray_d = p, p - mean = M^-1 q.  Hence
            //   v_M = v_grd (x) ray_d + v_gro (x) (ray_o - mean) = v_gro (x) (p - mean) = k q (x) M^-1 q:
            // the two terms of the reference's sum, each ~ distance / sigma times larger than the result, cancel
            // identically.  Only k q (for v_mean) and the symmetric k q (x) q are summed per Gaussian - small,
            // well-conditioned terms - and the epilogue applies M^-1 once.  (The reference forms both large terms in
            // fp32 per pair; this evaluation is closer to the exact value than the reference's own, and no ray
            // origin appears in it: a rolling shutter needs nothing extra.)
            // q as (n x g) x n, from the cross product the forward arithmetic already formed: it is then orthogonal
            // to n to rounding (g - (g . n) n leaves an error ALONG n, the one direction in which the sum over a
            // footprint should vanish, and showed 7 times the reference order's error on v_means)
            const vec3 q = cross(gcrod, grd_n);
            const vec3 v_gro = scale(q, -(a.w * v_opac));
            v[3] = v_gro.x;
            v[4] = v_gro.y;
            v[5] = v_gro.z;
            v[6] = v_gro.x * q.x;
            v[7] = v_gro.x * q.y;
            v[8] = v_gro.x * q.z;
            v[9] = v_gro.y * q.y;
            v[10] = v_gro.y * q.z;
            v[11] = v_gro.z * q.z;
            v[12] = v_opac;
            behind = fma(-cdot, fac, behind);
#pragma unroll
            for (uint32_t k = 0; k < NX; ++k) { // the gradients of the channels beyond the third: their own wave sums
                if (!(NC + k < nc))
                    continue;
                float e = fac * v_render_c[NX ? NC + k : 0];
#pragma unroll
                for (int m = 32; m >= 1; m >>= 1)
                    e += __shfl_xor(e, m, 64);
                if (lane == 0) {
                    if (XLDS) {
                        atomicAdd(&acc_extra[(uint32_t)t * (NX ? NX : 1) + k], e);
                    } else if (e != 0.f) {
                        // channel c of the whole row: the first three live in the 16-float rows, the others in
                        // gextra [N, stride - 3]
                        const uint32_t c = c0 + NC + k;
                        float* const at = (WIDE && c < 3u) ? &gacc[(size_t)id_batch[t] * kAcc + c]
                                                           : &gextra[(size_t)id_batch[t] * (stride - 3u) + (c - 3u)];
                        unsafeAtomicAdd(at, e);
                    }
                }
            }
            const float total = wave_reduce13(v, lane);
            if (sum_index < 13u)
                atomicAdd(&acc[(uint32_t)t * kAccLds + sum_index], total); // LDS: ds_add_f32
        }
        __syncthreads();
        if (STATS)
            continue;
        // flush: 16 lanes per Gaussian, one 64-byte row each
#pragma unroll 4
        for (uint32_t s = 0; s < kBwdBatch / 16; ++s) {
            const uint32_t gi = s * 16u + (tr >> 4);
            const uint32_t k = tr & 15u;
            if ((int32_t)gi < batch_size) {
                const float val = (k < 12u || k == 15u) ? acc[gi * kAccLds + min(k, 12u)] : 0.f;
                if (val != 0.f)
                    unsafeAtomicAdd(&gacc[(size_t)id_batch[gi] * kAcc + k], val); // (slot gi = entry batch_end - gi)
            }
        }
        if (XLDS && (int32_t)tr < batch_size) {
#pragma unroll
            for (uint32_t k = 0; k < NX; ++k) {
                const float val = acc_extra[tr * (NX ? NX : 1) + k];
                acc_extra[tr * (NX ? NX : 1) + k] = 0.f;
                if (val != 0.f)
                    unsafeAtomicAdd(&gextra[(size_t)id_batch[tr] * (NX ? NX : 1) + k], val);
            }
        }
        __syncthreads();
    }
    if (STATS && lane == 0) { // the counters are the same in every lane of a wave
        atomicAdd(&stats[0], (unsigned long long)n_eval);
        atomicAdd(&stats[1], (unsigned long long)n_valid);
        atomicAdd(&stats[2], (unsigned long long)n_iter);
    }
}

// Per-Gaussian epilogue: the linear map from the accumulated (sum k q, sum k q (x) q) to
// (v_mean, v_quat, v_scale) - quat_scale_to_preci_half_vjp / quat_to_rotmat_vjp of Utils.cuh:104-158.
__global__ void __launch_bounds__(256) rasterize_bwd_epilogue_kernel(
    uint32_t N, const float* __restrict__ means, const float* __restrict__ quats, const float* __restrict__ scales,
    const float* __restrict__ viewmat, float* __restrict__ gacc, float* __restrict__ gextra, uint32_t channels,
    int clear, float* __restrict__ v_means, float* __restrict__ v_quats, float* __restrict__ v_scales,
    float* __restrict__ v_colors, float* __restrict__ v_opacities) {
    const uint32_t g = blockIdx.x * 256u + threadIdx.x;
    if (g >= N)
        return;
    float4* row = reinterpret_cast<float4*>(gacc + (size_t)g * kAcc);
    const float4 r0 = row[0], r1 = row[1], r2 = row[2], r3 = row[3];
    const bool any_geo = (r0.w != 0.f) | (r1.x != 0.f) | (r1.y != 0.f) | (r1.z != 0.f) | (r1.w != 0.f) |
                         (r2.x != 0.f) | (r2.y != 0.f) | (r2.z != 0.f) | (r2.w != 0.f) | (r3.x != 0.f) |
                         (r3.y != 0.f) | (r3.z != 0.f);
    // leave the accumulators ready for the next backward pass; rows no pixel touched are still zero
    if (clear && (any_geo | (r0.x != 0.f) | (r0.y != 0.f) | (r0.z != 0.f) | (r3.w != 0.f))) {
        const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
        row[0] = z, row[1] = z, row[2] = z, row[3] = z;
    }
    // r0 = rgb.xyz, vo.x ; r1 = vo.y, vo.z, Sxx, Sxy ; r2 = Sxz, Syy, Syz, Szz ; r3 = -, -, -, v_opacity
    v_colors[(size_t)g * channels + 0] = r0.x;
    if (channels > 1)
        v_colors[(size_t)g * channels + 1] = r0.y;
    if (channels > 2)
        v_colors[(size_t)g * channels + 2] = r0.z;
    for (uint32_t k = 3; k < channels; ++k) {
        const size_t at = (size_t)g * (channels - 3) + (k - 3);
        const float e = gextra[at];
        v_colors[(size_t)g * channels + k] = e;
        if (clear && e != 0.f)
            gextra[at] = 0.f;
    }
    v_opacities[g] = r3.w;
    float vm[3] = {0.f, 0.f, 0.f}, vq[4] = {0.f, 0.f, 0.f, 0.f}, vs[3] = {0.f, 0.f, 0.f};
    if (any_geo)
        epilogue_geometry_grads(r0, r1, r2, ld4q(quats, g), ld3(scales, g), vm, vq, vs);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        v_means[(size_t)g * 3 + k] = vm[k];
        v_scales[(size_t)g * 3 + k] = vs[k];
    }
    reinterpret_cast<float4*>(v_quats)[g] = make_float4(vq[0], vq[1], vq[2], vq[3]);
}

} // namespace gsx

using namespace gsx;

extern "C" int gsx_debug_wave_reduce(uint32_t values, uint32_t n_waves, const float* in, float* out, void* stream) {
    GSX_REQUIRE(values == 16 || values == 13 || values == 9, GSX_ERR_INVALID_ARGUMENT,
                "debug_wave_reduce: %u values (16, 13 or 9)", values);
    if (n_waves == 0)
        return GSX_OK;
    GSX_REQUIRE(in && out, GSX_ERR_INVALID_ARGUMENT, "debug_wave_reduce: null tensor");
    if (values == 16)
        hipLaunchKernelGGL(wave_reduce_probe_kernel<16>, dim3(n_waves), dim3(64), 0, (hipStream_t)stream, in, out);
    else if (values == 13)
        hipLaunchKernelGGL(wave_reduce_probe_kernel<13>, dim3(n_waves), dim3(64), 0, (hipStream_t)stream, in, out);
    else
        hipLaunchKernelGGL(wave_reduce_probe_kernel<9>, dim3(n_waves), dim3(64), 0, (hipStream_t)stream, in, out);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

// accumulators only: 16 floats per Gaussian, then one float per Gaussian for a fourth colour channel; the
// whole-operator entry point also packs the records behind them
static size_t accum_extra_offset(uint32_t N) { return align_up((size_t)N * kAcc * 4, 256) + 256; }
extern "C" size_t gsx_rasterize_bwd_accum_bytes_for(uint32_t N, uint32_t channels) {
    return accum_extra_offset(N) + align_up((size_t)N * (channels > 4 ? channels - 3 : 1) * 4, 256);
}
extern "C" size_t gsx_rasterize_bwd_workspace_bytes_for(uint32_t N, uint32_t channels) {
    return gsx_rasterize_bwd_accum_bytes_for(N, channels) + gsx_raster_records_bytes(N);
}
// up to four channels
extern "C" size_t gsx_rasterize_bwd_accum_bytes(uint32_t N) { return gsx_rasterize_bwd_accum_bytes_for(N, 4); }
extern "C" size_t gsx_rasterize_bwd_workspace_bytes(uint32_t N) { return gsx_rasterize_bwd_workspace_bytes_for(N, 4); }

// stage 1: zero the per-Gaussian accumulators
extern "C" int gsx_rasterize_bwd_clear(uint32_t N, void* workspace, size_t workspace_bytes, void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0 &&
                    workspace_bytes >= gsx_rasterize_bwd_accum_bytes(N),
                GSX_ERR_WORKSPACE, "rasterize bwd: accumulators need %zu bytes, 256-byte aligned",
                gsx_rasterize_bwd_accum_bytes(N));
    const size_t n_acc = workspace_bytes / 4; // everything that was given: more than four channels need more
    hipLaunchKernelGGL(fill_f32_kernel, dim3(cdiv(n_acc, 256)), dim3(256), 0, (hipStream_t)stream, n_acc, 0.f,
                       (float*)workspace);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

namespace gsx {
int pack_raster_records(uint32_t N, const float* means, const float* quats, const float* scales,
                        const float* opacities, const float* colors, uint32_t channels, const float* viewmat,
                        const float* K, uint32_t image_width, uint32_t image_height, bool pinhole, bool rolling,
                        void* records, void* stream); // raster_fwd.hip

static int rasterize_bwd_accumulate(uint32_t C, uint32_t N, int64_t n_isects, const void* records,
                                    const float* colors, uint32_t channels, const float* backgrounds,
                                    const uint8_t* masks, uint32_t image_width, uint32_t image_height,
                                    uint32_t tile_size, const float* viewmats0, const float* Ks, int camera_model,
                                    const float* radial, const float* tangential, const float* thin_prism,
                                    const float* viewmats1, int rs_type, const int32_t* tile_offsets,
                                    const uint32_t* tile_order, const int32_t* flatten_ids,
                                    const float* render_alphas, const int32_t* last_ids,
                                    const float* v_render_colors, const float* v_render_alphas, void* workspace,
                                    size_t workspace_bytes, void* stream) {
    GSX_REQUIRE(C == 1, GSX_ERR_UNSUPPORTED, "C = %u cameras: only C == 1 is supported", C);
    if (N == 0 || n_isects == 0 || image_width == 0 || image_height == 0) // ...Bwd.cu:440-443
        return GSX_OK;
    GSX_REQUIRE(tile_size == kTile, GSX_ERR_UNSUPPORTED, "rasterize bwd: tile_size %u (only 16 is built)", tile_size);
    GSX_REQUIRE(n_isects >= GSX_COUNT_IN_OFFSETS && n_isects < (1ll << 31), GSX_ERR_OVERFLOW,
                "rasterize bwd: n_isects out of range");
    GSX_REQUIRE(records && viewmats0 && Ks && tile_offsets && flatten_ids && render_alphas && last_ids &&
                    v_render_colors && v_render_alphas,
                GSX_ERR_INVALID_ARGUMENT, "rasterize bwd: null tensor");
    GSX_REQUIRE(((uintptr_t)records & 15) == 0, GSX_ERR_WORKSPACE, "rasterize bwd: records need 16-byte alignment");
    GSX_REQUIRE(raster_channels_built(channels), GSX_ERR_UNSUPPORTED,
                "rasterize bwd: %u channels (%s)", channels, kRasterChannelsText);
    GSX_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0 &&
                    workspace_bytes >= gsx_rasterize_bwd_accum_bytes_for(N, channels),
                GSX_ERR_WORKSPACE, "rasterize bwd: accumulators need %zu bytes, 256-byte aligned",
                gsx_rasterize_bwd_accum_bytes_for(N, channels));
    GSX_REQUIRE(channels <= 3 || colors != nullptr, GSX_ERR_INVALID_ARGUMENT, "rasterize bwd: colors is null");
    const uint32_t tw = cdiv(image_width, kTile), th = cdiv(image_height, kTile);
    float* gextra = (float*)((char*)workspace + accum_extra_offset(N));
    const bool distorted = camera_model != GSX_PINHOLE || radial != nullptr || tangential != nullptr ||
                           thin_prism != nullptr || rs_type != GSX_GLOBAL || viewmats1 != nullptr;
#define GSX_LAUNCH_BWD(CD, DI)                                                                                       \
    hipLaunchKernelGGL((rasterize_bwd_kernel<CD, DI>), dim3(tw * th), dim3(256), 0, (hipStream_t)stream,             \
                       (uint32_t)n_isects, (const float4*)records, colors, backgrounds, masks, image_width,          \
                       image_height, tw, th, viewmats0, Ks, camera_model, radial, tangential, thin_prism,            \
                       viewmats1, rs_type, tile_offsets, tile_order, flatten_ids, render_alphas, last_ids,           \
                       v_render_colors, v_render_alphas, (float*)workspace, gextra)
#define GSX_LAUNCH_BWD2(CD)       \
    if (distorted)                \
        GSX_LAUNCH_BWD(CD, true); \
    else                          \
        GSX_LAUNCH_BWD(CD, false)
    switch (channels) {
    case 1: GSX_LAUNCH_BWD2(1); break;
    case 2: GSX_LAUNCH_BWD2(2); break;
    case 3: GSX_LAUNCH_BWD2(3); break;
    case 4: GSX_LAUNCH_BWD2(4); break;
    case 5: GSX_LAUNCH_BWD2(5); break;
    case 8: GSX_LAUNCH_BWD2(8); break;
    case 9: GSX_LAUNCH_BWD2(9); break;
    case 16: GSX_LAUNCH_BWD2(16); break;
    case 17: GSX_LAUNCH_BWD2(17); break;
    case 32: GSX_LAUNCH_BWD2(32); break;
    default:
        // 33 ... 513 channels: 32 of them per launch, counted at run time
        for (uint32_t c0 = 0; c0 < channels; c0 += 32) {
            const uint32_t nc = channels - c0 < 32u ? channels - c0 : 32u;
            if (distorted)
                hipLaunchKernelGGL((rasterize_bwd_kernel<32, true, false, true>), dim3(tw * th), dim3(256), 0,
                                   (hipStream_t)stream, (uint32_t)n_isects, (const float4*)records, colors, backgrounds,
                                   masks, image_width, image_height, tw, th, viewmats0, Ks, camera_model, radial,
                                   tangential, thin_prism, viewmats1, rs_type, tile_offsets, tile_order, flatten_ids,
                                   render_alphas, last_ids, v_render_colors, v_render_alphas, (float*)workspace, gextra,
                                   (unsigned long long*)nullptr, channels, c0, nc);
            else
                hipLaunchKernelGGL((rasterize_bwd_kernel<32, false, false, true>), dim3(tw * th), dim3(256), 0,
                                   (hipStream_t)stream, (uint32_t)n_isects, (const float4*)records, colors, backgrounds,
                                   masks, image_width, image_height, tw, th, viewmats0, Ks, camera_model, radial,
                                   tangential, thin_prism, viewmats1, rs_type, tile_offsets, tile_order, flatten_ids,
                                   render_alphas, last_ids, v_render_colors, v_render_alphas, (float*)workspace, gextra,
                                   (unsigned long long*)nullptr, channels, c0, nc);
        }
        break;
    }
#undef GSX_LAUNCH_BWD2
#undef GSX_LAUNCH_BWD
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}
} // namespace gsx

// stage 2: the per-tile kernel, accumulating into the workspace; `records` from gsx_pack_raster_records (or the
// fused per-Gaussian pass) for the same camera and parameters
extern "C" int gsx_rasterize_bwd_accumulate(uint32_t C, uint32_t N, int64_t n_isects, const void* records,
                                            const float* colors, uint32_t channels, const float* backgrounds,
                                            const uint8_t* masks, uint32_t image_width,
                                            uint32_t image_height, uint32_t tile_size, const float* viewmats0,
                                            const float* Ks, const int32_t* tile_offsets, const int32_t* flatten_ids,
                                            const uint32_t* tile_order, const float* render_alphas,
                                            const int32_t* last_ids, const float* v_render_colors,
                                            const float* v_render_alphas, void* workspace, size_t workspace_bytes,
                                            void* stream) {
    return rasterize_bwd_accumulate(C, N, n_isects, records, colors, channels, backgrounds, masks, image_width,
                                    image_height, tile_size, viewmats0, Ks, GSX_PINHOLE, nullptr, nullptr, nullptr,
                                    nullptr, GSX_GLOBAL, tile_offsets, tile_order, flatten_ids, render_alphas, last_ids,
                                    v_render_colors,
                                    v_render_alphas, workspace, workspace_bytes, stream);
}

extern "C" int gsx_rasterize_bwd_pair_stats(int64_t n_isects, const void* records, uint32_t image_width,
                                            uint32_t image_height, const float* viewmat, const float* K,
                                            const int32_t* tile_offsets, const int32_t* flatten_ids,
                                            const float* render_alphas, const int32_t* last_ids,
                                            unsigned long long* stats_out, void* stream) {
    if (image_width == 0 || image_height == 0 || n_isects == 0)
        return GSX_OK;
    GSX_REQUIRE(records && viewmat && K && tile_offsets && flatten_ids && render_alphas && last_ids && stats_out,
                GSX_ERR_INVALID_ARGUMENT, "rasterize_bwd_pair_stats: null tensor");
    GSX_REQUIRE(n_isects >= GSX_COUNT_IN_OFFSETS && n_isects < (1ll << 31), GSX_ERR_OVERFLOW,
                "rasterize_bwd_pair_stats: n_isects out of range");
    const uint32_t tw = cdiv(image_width, kTile), th = cdiv(image_height, kTile);
    // the gradient inputs are read but do not matter for the counts: the alphas (one float per pixel; the kernel
    // reads three) cannot stand in for them, so the counts use a kernel instance that never touches them
    hipLaunchKernelGGL((rasterize_bwd_kernel<3, false, true>), dim3(tw * th), dim3(256), 0, (hipStream_t)stream,
                       (uint32_t)n_isects, (const float4*)records, (const float*)nullptr, (const float*)nullptr,
                       (const uint8_t*)nullptr, image_width, image_height, tw, th, viewmat, K, (int)GSX_PINHOLE,
                       (const float*)nullptr, (const float*)nullptr, (const float*)nullptr, (const float*)nullptr,
                       (int)GSX_GLOBAL, tile_offsets, (const uint32_t*)nullptr, flatten_ids, render_alphas, last_ids,
                       (const float*)nullptr, (const float*)nullptr, (float*)nullptr, (float*)nullptr, stats_out);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

// stage 3: per-Gaussian epilogue, accumulators -> the five gradient tensors (all elements written)
extern "C" int gsx_rasterize_bwd_finish(uint32_t N, const float* means, const float* quats, const float* scales,
                                        const float* viewmats0, void* workspace, size_t workspace_bytes,
                                        int clear_accumulators, uint32_t channels, float* v_means, float* v_quats,
                                        float* v_scales, float* v_colors, float* v_opacities, void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(means && quats && scales && viewmats0 && v_means && v_quats && v_scales && v_colors && v_opacities,
                GSX_ERR_INVALID_ARGUMENT, "rasterize bwd: null tensor");
    GSX_REQUIRE(raster_channels_built(channels), GSX_ERR_UNSUPPORTED,
                "rasterize bwd: %u channels (%s)", channels, kRasterChannelsText);
    GSX_REQUIRE(workspace != nullptr && workspace_bytes >= gsx_rasterize_bwd_accum_bytes_for(N, channels),
                GSX_ERR_WORKSPACE, "rasterize bwd: accumulators need %zu bytes",
                gsx_rasterize_bwd_accum_bytes_for(N, channels));
    hipLaunchKernelGGL(rasterize_bwd_epilogue_kernel, dim3(cdiv(N, 256)), dim3(256), 0, (hipStream_t)stream, N, means,
                       quats, scales, viewmats0, (float*)workspace, (float*)((char*)workspace + accum_extra_offset(N)),
                       channels, clear_accumulators, v_means, v_quats, v_scales, v_colors, v_opacities);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_rasterize_to_pixels_from_world_3dgs_bwd(
    uint32_t C, uint32_t N, int64_t n_isects, const float* means, const float* quats, const float* scales,
    const float* colors, uint32_t channels, const float* opacities, const float* backgrounds, const uint8_t* masks,
    uint32_t image_width, uint32_t image_height, uint32_t tile_size, const float* viewmats0, const float* viewmats1,
    const float* Ks, int camera_model, gsx_ut_params ut, int rs_type, const float* radial_coeffs,
    const float* tangential_coeffs, const float* thin_prism_coeffs, const int32_t* tile_offsets,
    const int32_t* flatten_ids, const float* render_alphas, const int32_t* last_ids, const float* v_render_colors,
    const float* v_render_alphas, float* v_means, float* v_quats, float* v_scales, float* v_colors,
    float* v_opacities, void* workspace, size_t workspace_bytes, void* stream) {
    (void)ut;
    int rc = check_camera_args(C, viewmats1, camera_model, rs_type, radial_coeffs, tangential_coeffs,
                               thin_prism_coeffs);
    if (rc != GSX_OK)
        return rc;
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(raster_channels_built(channels), GSX_ERR_UNSUPPORTED,
                "rasterize bwd: %u channels (%s)", channels, kRasterChannelsText);
    GSX_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0 &&
                    workspace_bytes >= gsx_rasterize_bwd_workspace_bytes_for(N, channels),
                GSX_ERR_WORKSPACE, "rasterize bwd: workspace needs %zu bytes, 256-byte aligned",
                gsx_rasterize_bwd_workspace_bytes_for(N, channels));
    GSX_REQUIRE(means && quats && scales && colors && opacities && viewmats0 && Ks, GSX_ERR_INVALID_ARGUMENT,
                "rasterize bwd: null tensor");
    const size_t acc_bytes = gsx_rasterize_bwd_accum_bytes_for(N, channels);
    void* records = (char*)workspace + acc_bytes;
    if ((rc = gsx_rasterize_bwd_clear(N, workspace, acc_bytes, stream)) != GSX_OK)
        return rc;
    const bool rolling = rs_type != GSX_GLOBAL;
    const bool pinhole =
        camera_model == GSX_PINHOLE && !(radial_coeffs || tangential_coeffs || thin_prism_coeffs) && !rolling;
    if ((rc = pack_raster_records(N, means, quats, scales, opacities, colors, channels, viewmats0, Ks, image_width,
                                  image_height, pinhole, rolling, records, stream)) != GSX_OK)
        return rc;
    // room behind the records for a tile order: visit the tiles dearest first (cost from the forward's outputs)
    const uint32_t* tile_order = nullptr;
    const size_t base_bytes = gsx_rasterize_bwd_workspace_bytes_for(N, channels);
    if (n_isects > 0 && tile_size == kTile && tile_offsets && render_alphas && last_ids &&
        workspace_bytes >= base_bytes + gsx_tile_order_bytes(cdiv(image_width, kTile), cdiv(image_height, kTile))) {
        if ((rc = tile_order_from_pixels(n_isects, image_width, image_height, tile_offsets, render_alphas, last_ids,
                                         (char*)workspace + base_bytes, &tile_order, stream)) != GSX_OK)
            return rc;
    }
    if ((rc = rasterize_bwd_accumulate(C, N, n_isects, records, colors, channels, backgrounds, masks, image_width,
                                       image_height, tile_size, viewmats0, Ks, camera_model, radial_coeffs,
                                       tangential_coeffs, thin_prism_coeffs, viewmats1, rs_type, tile_offsets,
                                       tile_order, flatten_ids, render_alphas, last_ids,
                                       v_render_colors, v_render_alphas, workspace, acc_bytes, stream)) != GSX_OK)
        return rc;
    return gsx_rasterize_bwd_finish(N, means, quats, scales, viewmats0, workspace, acc_bytes, 0, channels, v_means,
                                    v_quats, v_scales, v_colors, v_opacities, stream);
}
