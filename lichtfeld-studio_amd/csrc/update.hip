// update.hip - the tail of a training step in one pass over the Gaussians: rasterizer-backward epilogue
// (Utils.cuh:104-158) -> SH backward with the clamp mask (Rasterization.cpp:608-624) -> VJPs of the activations
// (autograd of splat_data.cpp:271-286) -> Adam on all parameter tensors (adam_kernels.cuh:13-36,
// fused_adam.cpp:22-95).
//
// The separate kernels write 236 B of raw-parameter gradients per Gaussian and the optimiser reads them back; here
// they stay in registers.  Arithmetic is that of the separate kernels (same device functions), so parameters and
// moments come out bit-identical to epilogue + sh_colors_from_world_bwd + activate_params_bwd + adam_step_multi.
// The SH parameter and its two moments are updated where they lie with coalesced 16-byte accesses; the per-Gaussian
// gradient rows reach that layout through LDS.
#include <string.h>

#include "gsx_common.h"
#include "gsx_step.h"

namespace gsx {

struct UpdateArgs {
    uint32_t N, K, sh_degree;
    float *means, *opacity_raw, *scaling_raw, *rotation_raw, *shs;
    float *m_means, *m_opacity, *m_scaling, *m_rotation, *m_shs;
    float *v_means, *v_opacity, *v_scaling, *v_rotation, *v_shs;
    const int32_t* radii;
    const float* colors;
    const float* viewmat;
    float* acc;
    float lr_means, lr_sh0, lr_shN, lr_scaling, lr_rotation, lr_opacity;
    float beta1, beta2, eps, bc1_rcp, bc2_sqrt_rcp;
    int32_t skip_shN;
    float reg_scaling, reg_opacity;
    uint32_t* hold;             // nullable: [0] != 0 -> change nothing and count the call in [1]
    const float* step_scalars;  // nullable: device [3] = bc1_rcp, bc2_sqrt_rcp, skip_shN (0 / 1), read at run time
    uint64_t* hold_report;      // nullable, pinned host memory: receives hold[1] << 32 | hold[0]
};

// new first / second moment of one element (the first two lines of adam_one)
__device__ __forceinline__ float adam_m(float m, float g, float beta1) { return beta1 * m + (1.0f - beta1) * g; }
__device__ __forceinline__ float adam_v(float v, float g, float beta2) { return beta2 * v + (1.0f - beta2) * g * g; }
__device__ __forceinline__ float adam_p(float p, float m1, float v1, float lr, float eps, float c1, float c2) {
    const float denom = gsx::sqrt(v1) * c2 + eps;
    const float step_size = lr * c1;
    return p - step_size * m1 / denom;
}

template <int n>
__device__ __forceinline__ void adam_row(float* __restrict__ P, float* __restrict__ M, float* __restrict__ V,
                                         uint32_t e, const float (&g)[n], float lr, const UpdateArgs& a) {
#pragma unroll
    for (int k = 0; k < n; ++k) {
        float p = P[(size_t)e * n + k], m = M[(size_t)e * n + k], v = V[(size_t)e * n + k];
        adam_one(p, m, v, g[k], lr, a.beta1, a.beta2, a.eps, a.bc1_rcp, a.bc2_sqrt_rcp);
        P[(size_t)e * n + k] = p;
        M[(size_t)e * n + k] = m;
        V[(size_t)e * n + k] = v;
    }
}

template <bool LDS16>
__global__ void __launch_bounds__(256) backward_update_kernel(const UpdateArgs a_in) {
    constexpr uint32_t kGradF4 = 5; // what a lane leaves for the coefficient update: 16 basis values, 3 colour gradients, nb
    __shared__ float4 lds[LDS16 ? 4 * 64 * kGradF4 : 1];
    const uint32_t e = blockIdx.x * 256u + threadIdx.x;
    UpdateArgs a = a_in;
    if (a.step_scalars != nullptr) { // a replayed launch takes the step's scalars from memory
        a.bc1_rcp = a.step_scalars[0];
        a.bc2_sqrt_rcp = a.step_scalars[1];
        a.skip_shN = a.step_scalars[2] != 0.f ? 1 : 0;
    }
    if (a.hold != nullptr && a.hold[0] != 0u) {
        // the step's render is not valid (its tile lists did not fit): parameters and moments stay as they are; the
        // accumulator rows are cleared all the same
        if (e == 0) {
            const uint32_t held = atomicAdd(&a.hold[1], 1u) + 1u;
            if (a.hold_report != nullptr)
                __hip_atomic_store(a.hold_report, ((uint64_t)held << 32) | a.hold[0], __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_SYSTEM);
        }
        if (e < a.N) {
            float4* row = reinterpret_cast<float4*>(a.acc + (size_t)e * 16);
            const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
            row[0] = z, row[1] = z, row[2] = z, row[3] = z;
        }
        return;
    }
    if (e == 0 && a.hold != nullptr && a.hold_report != nullptr)
        __hip_atomic_store(a.hold_report, (uint64_t)a.hold[1] << 32, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    float4* wave_lds = lds + (LDS16 ? wave * 64 * kGradF4 : 0);
    const bool in = e < a.N;

    float B[25];
    int nb = 0;
    float vc[3] = {0.f, 0.f, 0.f}; // d loss / d colour behind the clamp
    if (in) {
        // ---- epilogue of the rasterizer backward ----
        float4* row = reinterpret_cast<float4*>(a.acc + (size_t)e * 16);
        const float4 r0 = row[0], r1 = row[1], r2 = row[2], r3 = row[3];
        const bool any_geo = (r0.w != 0.f) | (r1.x != 0.f) | (r1.y != 0.f) | (r1.z != 0.f) | (r1.w != 0.f) |
                             (r2.x != 0.f) | (r2.y != 0.f) | (r2.z != 0.f) | (r2.w != 0.f) | (r3.x != 0.f) |
                             (r3.y != 0.f) | (r3.z != 0.f);
        if (any_geo | (r0.x != 0.f) | (r0.y != 0.f) | (r0.z != 0.f) | (r3.w != 0.f)) {
            const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
            row[0] = z, row[1] = z, row[2] = z, row[3] = z; // ready for the next backward pass
        }
        const vec3 mean = ld3(a.means, e);
        // requested here with everything else (behind `live` and `&&` they were three round trips of their own)
        const int2 rad = reinterpret_cast<const int2*>(a.radii)[e];
        const float col_in[3] = {a.colors[e * 3 + 0], a.colors[e * 3 + 1], a.colors[e * 3 + 2]};
        const float o_raw = a.opacity_raw[e];
        const vec3 s_raw = ld3(a.scaling_raw, e);
        const quat q_raw = ld4q(a.rotation_raw, e);
        float vm[3] = {0.f, 0.f, 0.f}, vq[4] = {0.f, 0.f, 0.f, 0.f}, vs[3] = {0.f, 0.f, 0.f};
        if (any_geo) {
            const Activated act = activate(o_raw, s_raw, q_raw);
            epilogue_geometry_grads(r0, r1, r2, act.quat, act.scales, vm, vq, vs);
        }
        // ---- VJPs of the activations ----
        quat gq;
        gq.w = vq[0], gq.x = vq[1], gq.y = vq[2], gq.z = vq[3];
        const ActivationVjp av = activation_vjp(o_raw, s_raw, q_raw, r3.w, mk3(vs[0], vs[1], vs[2]), gq);
        // ---- SH backward inputs (sh_colors_from_world_bwd) ----
        const bool live = rad.x > 0 && rad.y > 0;
        if (live) {
            nb = sh_basis(a.sh_degree, sub(mean, campos_from_viewmat(a.viewmat)), B);
            const float v_col[3] = {r0.x, r0.y, r0.z};
#pragma unroll
            for (int c = 0; c < 3; ++c)
                vc[c] = col_in[c] <= 0.0f ? 0.f : v_col[c]; // clamp VJP (Rasterization.cpp:609-610)
        }
        // ---- Adam on the small tensors ----
        adam_row<3>(a.means, a.m_means, a.v_means, e, vm, a.lr_means, a);
        float gs[3] = {av.scaling.x, av.scaling.y, av.scaling.z};
        float go[1] = {av.opacity};
        if (a.reg_scaling != 0.f) { // += (w / n) exp(x), as the regularisation kernel adds it to the finished gradient
            gs[0] += a.reg_scaling * gsx::exp(s_raw.x);
            gs[1] += a.reg_scaling * gsx::exp(s_raw.y);
            gs[2] += a.reg_scaling * gsx::exp(s_raw.z);
        }
        if (a.reg_opacity != 0.f) {
            const float sg = gsx::sigmoid(o_raw);
            go[0] += a.reg_opacity * (sg * (1.0f - sg));
        }
        adam_row<3>(a.scaling_raw, a.m_scaling, a.v_scaling, e, gs, a.lr_scaling, a);
        const float gr[4] = {av.rotation.w, av.rotation.x, av.rotation.y, av.rotation.z};
        adam_row<4>(a.rotation_raw, a.m_rotation, a.v_rotation, e, gr, a.lr_rotation, a);
        adam_row<1>(a.opacity_raw, a.m_opacity, a.v_opacity, e, go, a.lr_opacity, a);
    }

    // ---- Adam on the SH tensor; gradient of coefficient (k, c) = B[k] * vc[c] for k < nb, else 0 ----
    // The update is elementwise, so the parameter and both moments are processed where they lie, with coalesced
    // 16-byte accesses: position q of a wave's 64 rows = float4 (q % 12) of row (q / 12).  The gradient is an outer
    // product, so a lane leaves only its 16 basis values, its three colour gradients and nb in LDS (5 float4) and
    // the lane that owns position q rebuilds the four gradient elements there - the same products B[k] * vc[c].
    // The bytes are streamed in four batches of 3 x 3 float4 per lane; the requests of a batch leave before the
    // batch in front of it is worked on, so that every wave keeps 18 KiB of reads in flight.
    if (LDS16) {
        const uint32_t row0 = blockIdx.x * 256u + wave * 64u;
        if (row0 >= a.N)
            return; // whole wave out of range
        const uint32_t rows = min(64u, a.N - row0), n_f4 = rows * kShRowF4;
        float4* __restrict__ P4 = reinterpret_cast<float4*>(a.shs) + (size_t)row0 * kShRowF4;
        float4* __restrict__ M4 = reinterpret_cast<float4*>(a.m_shs) + (size_t)row0 * kShRowF4;
        float4* __restrict__ V4 = reinterpret_cast<float4*>(a.v_shs) + (size_t)row0 * kShRowF4;
        if (a.skip_shN != 0) {
            // the higher bands are frozen: only the DC coefficient (elements 0..2 of a row) moves; lane = row
            if (lane < rows) {
                const uint32_t q = lane * kShRowF4;
                float4 p = load_streaming(P4 + q), m = load_streaming(M4 + q), v = load_streaming(V4 + q);
                float* pv = reinterpret_cast<float*>(&p);
                float* mv = reinterpret_cast<float*>(&m);
                float* vv = reinterpret_cast<float*>(&v);
#pragma unroll
                for (int t = 0; t < 3; ++t) {
                    const float g = nb > 0 ? B[0] * vc[t] : 0.f;
                    const float m1 = adam_m(mv[t], g, a.beta1);
                    const float v1 = adam_v(vv[t], g, a.beta2);
                    pv[t] = adam_p(pv[t], m1, v1, a.lr_sh0, a.eps, a.bc1_rcp, a.bc2_sqrt_rcp);
                    mv[t] = m1;
                    vv[t] = v1;
                }
                store_streaming(P4 + q, p);
                store_streaming(M4 + q, m);
                store_streaming(V4 + q, v);
            }
            return;
        }
        constexpr uint32_t kPer = 3, kBatches = kShRowF4 / kPer; // float4 per lane, array and batch
        float4 p4[2][kPer], m4[2][kPer], v4[2][kPer];
        // requests of a batch: unconditional, from addresses clamped into the wave's rows
        auto request = [&](uint32_t batch, uint32_t buf) {
#pragma unroll
            for (uint32_t i = 0; i < kPer; ++i) {
                const uint32_t q = min((batch * kPer + i) * 64u + lane, n_f4 - 1u);
                p4[buf][i] = load_streaming(P4 + q);
                m4[buf][i] = load_streaming(M4 + q);
                v4[buf][i] = load_streaming(V4 + q);
            }
        };
        request(0, 0);
        {
            float4* mine = wave_lds + lane * kGradF4;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                mine[j] = make_float4(4 * j + 0 < nb ? B[4 * j + 0] : 0.f, 4 * j + 1 < nb ? B[4 * j + 1] : 0.f,
                                      4 * j + 2 < nb ? B[4 * j + 2] : 0.f, 4 * j + 3 < nb ? B[4 * j + 3] : 0.f);
            mine[4] = make_float4(vc[0], vc[1], vc[2], __int_as_float(nb));
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (uint32_t batch = 0; batch < kBatches; ++batch) {
            const uint32_t cur = batch & 1u;
            if (batch + 1 < kBatches)
                request(batch + 1, cur ^ 1u);
#pragma unroll
            for (uint32_t i = 0; i < kPer; ++i) {
                const uint32_t q = (batch * kPer + i) * 64u + lane;
                const uint32_t r = (q * 43691u) >> 19, col = q - r * kShRowF4; // q / 12 for q < 768
                // elements 4 col .. 4 col + 3 of the row: coefficient k0 from colour c0 on, then coefficient k0 + 1
                const uint32_t i0 = 4u * col, k0 = (i0 * 43u) >> 7 /* i0 / 3 for i0 <= 44 */, c0 = i0 - 3u * k0;
                const float* gf = reinterpret_cast<const float*>(wave_lds + r * kGradF4);
                const float b0 = gf[k0], b1 = gf[k0 + 1u];
                const float4 cv = wave_lds[r * kGradF4 + 4u];
                const int row_nb = __float_as_int(cv.w);
                float* pv = reinterpret_cast<float*>(&p4[cur][i]);
                float* mv = reinterpret_cast<float*>(&m4[cur][i]);
                float* vv = reinterpret_cast<float*>(&v4[cur][i]);
#pragma unroll
                for (uint32_t t = 0; t < 4; ++t) {
                    const uint32_t idx = c0 + t; // 0..5
                    const bool next = idx >= 3u;
                    const uint32_t c = next ? idx - 3u : idx;
                    const float colour = c == 0u ? cv.x : (c == 1u ? cv.y : cv.z);
                    const float gv = (int)(k0 + (next ? 1u : 0u)) < row_nb ? (next ? b1 : b0) * colour : 0.f;
                    const bool dc = col == 0u && t < 3u; // elements 0..2 of a row: the DC coefficient
                    const float m1 = adam_m(mv[t], gv, a.beta1);
                    const float v1 = adam_v(vv[t], gv, a.beta2);
                    pv[t] = adam_p(pv[t], m1, v1, dc ? a.lr_sh0 : a.lr_shN, a.eps, a.bc1_rcp, a.bc2_sqrt_rcp);
                    mv[t] = m1;
                    vv[t] = v1;
                }
                if (q < n_f4) {
                    store_streaming(P4 + q, p4[cur][i]);
                    store_streaming(M4 + q, m4[cur][i]);
                    store_streaming(V4 + q, v4[cur][i]);
                }
            }
        }
        return;
    }
    if (!in)
        return;
    for (uint32_t k = 0; k < a.K; ++k) {
        const bool used = (int)k < nb;
        const float b = B[k < 25 ? k : 24];
        if (k >= 1 && a.skip_shN)
            break;
#pragma unroll
        for (uint32_t c = 0; c < 3; ++c) {
            const size_t i = ((size_t)e * a.K + k) * 3 + c;
            float p = a.shs[i], m = a.m_shs[i], v = a.v_shs[i];
            adam_one(p, m, v, used ? b * vc[c] : 0.f, k == 0 ? a.lr_sh0 : a.lr_shN, a.beta1, a.beta2, a.eps,
                     a.bc1_rcp, a.bc2_sqrt_rcp);
            a.shs[i] = p;
            a.m_shs[i] = m;
            a.v_shs[i] = v;
        }
    }
}

} // namespace gsx

using namespace gsx;

extern "C" int gsx_backward_update_fused(const gsx_update_args* args, void* stream) {
    GSX_REQUIRE(args != nullptr, GSX_ERR_INVALID_ARGUMENT, "backward_update_fused: args is null");
    if (args->N == 0)
        return GSX_OK;
    GSX_REQUIRE(args->means && args->opacity_raw && args->scaling_raw && args->rotation_raw && args->shs &&
                    args->m_means && args->m_opacity && args->m_scaling && args->m_rotation && args->m_shs &&
                    args->v_means && args->v_opacity && args->v_scaling && args->v_rotation && args->v_shs &&
                    args->radii && args->colors && args->viewmat && args->accumulators,
                GSX_ERR_INVALID_ARGUMENT, "backward_update_fused: null tensor");
    GSX_REQUIRE(args->K >= 1 && args->K <= 25, GSX_ERR_INVALID_ARGUMENT, "backward_update_fused: K = %u", args->K);
    const uint32_t need = (args->sh_degree + 1) * (args->sh_degree + 1);
    GSX_REQUIRE(args->sh_degree <= 4 && args->K >= need, GSX_ERR_INVALID_ARGUMENT,
                "backward_update_fused: degree %u needs K >= %u (K = %u)", args->sh_degree, need, args->K);
    GSX_REQUIRE((((uintptr_t)args->accumulators) & 15) == 0 && (((uintptr_t)args->rotation_raw) & 15) == 0 &&
                    (((uintptr_t)args->radii) & 7) == 0,
                GSX_ERR_INVALID_ARGUMENT,
                "backward_update_fused: accumulators / rotation need 16-byte alignment, radii 8-byte");
    UpdateArgs a;
    memset(&a, 0, sizeof(a));
    a.N = args->N, a.K = args->K, a.sh_degree = args->sh_degree;
    a.means = args->means, a.opacity_raw = args->opacity_raw, a.scaling_raw = args->scaling_raw;
    a.rotation_raw = args->rotation_raw, a.shs = args->shs;
    a.m_means = args->m_means, a.m_opacity = args->m_opacity, a.m_scaling = args->m_scaling;
    a.m_rotation = args->m_rotation, a.m_shs = args->m_shs;
    a.v_means = args->v_means, a.v_opacity = args->v_opacity, a.v_scaling = args->v_scaling;
    a.v_rotation = args->v_rotation, a.v_shs = args->v_shs;
    a.radii = args->radii, a.colors = args->colors, a.viewmat = args->viewmat, a.acc = (float*)args->accumulators;
    a.lr_means = args->lr_means, a.lr_sh0 = args->lr_sh0, a.lr_shN = args->lr_shN, a.lr_scaling = args->lr_scaling;
    a.lr_rotation = args->lr_rotation, a.lr_opacity = args->lr_opacity;
    a.beta1 = args->beta1, a.beta2 = args->beta2, a.eps = args->eps;
    a.bc1_rcp = args->bias_correction1_rcp, a.bc2_sqrt_rcp = args->bias_correction2_sqrt_rcp;
    a.skip_shN = args->skip_shN;
    a.reg_scaling = args->reg_scaling, a.reg_opacity = args->reg_opacity;
    a.hold = args->hold, a.step_scalars = args->step_scalars, a.hold_report = args->hold_report;
    if (a.hold_report != nullptr) {
        hipPointerAttribute_t attr;
        const bool known = hipPointerGetAttributes(&attr, a.hold_report) == hipSuccess;
        if (!known)
            (void)hipGetLastError();
        GSX_REQUIRE(known && attr.type == hipMemoryTypeHost && attr.devicePointer != nullptr, GSX_ERR_INVALID_ARGUMENT,
                    "backward_update_fused: hold_report must be pinned host memory (hipHostMalloc)");
        GSX_REQUIRE(a.hold != nullptr, GSX_ERR_INVALID_ARGUMENT, "backward_update_fused: hold_report without hold");
        a.hold_report = (uint64_t*)attr.devicePointer;
    }
    const bool lds16 = a.K == 16 && ((((uintptr_t)a.shs) | ((uintptr_t)a.m_shs) | ((uintptr_t)a.v_shs)) & 15u) == 0;
    const dim3 grid(cdiv(a.N, 256)), block(256);
    if (lds16)
        hipLaunchKernelGGL((backward_update_kernel<true>), grid, block, 0, (hipStream_t)stream, a);
    else
        hipLaunchKernelGGL((backward_update_kernel<false>), grid, block, 0, (hipStream_t)stream, a);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}
