// relocation.hip - MCMC relocation (Eq. 9) and noise injection (gsplat/RelocationCUDA.cu:11-43, 88-144).
#include "gsx_common.h"

namespace gsx {

__global__ void __launch_bounds__(256) relocation_kernel(int M, const float* __restrict__ opacities,
                                                          const float* __restrict__ scales,
                                                          const int32_t* __restrict__ ratios,
                                                          const float* __restrict__ binoms, int n_max,
                                                          float* __restrict__ new_opacities,
                                                          float* __restrict__ new_scales) {
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= M)
        return;
    const int n_idx = ratios[idx];
    const float op = opacities[idx];
    float denom_sum = 0.0f;
    const float new_o = 1.0f - gsx::pow(1.0f - op, 1.0f / (float)n_idx);
    new_opacities[idx] = new_o;
    for (int i = 1; i <= n_idx; ++i)
        for (int k = 0; k <= (i - 1); ++k) {
            const float bin_coeff = binoms[(i - 1) * n_max + k];
            const float sgn = (k & 1) ? -1.0f : 1.0f;
            const float term = (sgn / gsx::sqrt((float)(k + 1))) * gsx::pow(new_o, (float)(k + 1));
            denom_sum += (bin_coeff * term);
        }
    const float coeff = (op / denom_sum);
#pragma unroll
    for (int i = 0; i < 3; ++i)
        new_scales[idx * 3 + i] = coeff * scales[idx * 3 + i];
}

__global__ void __launch_bounds__(256) add_noise_kernel(int N, const float* __restrict__ raw_opacities,
                                                         const float* __restrict__ raw_scales,
                                                         const float* __restrict__ raw_quats,
                                                         const float* __restrict__ noise, float* __restrict__ means,
                                                         float current_lr) {
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= N)
        return;
    const vec3 rs = ld3(raw_scales, idx);
    const float s2[3] = {gsx::exp(2.f * rs.x), gsx::exp(2.f * rs.y), gsx::exp(2.f * rs.z)};
    const mat3 R = quat_to_rotmat(ld4q(raw_quats, idx), 1e+12f);
    mat3 cov; // R diag(s2) R^T
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            float a = (R.m[i][0] * s2[0]) * R.m[j][0];
            a = fma(R.m[i][1] * s2[1], R.m[j][1], a);
            a = fma(R.m[i][2] * s2[2], R.m[j][2], a);
            cov.m[i][j] = a;
        }
    const vec3 tn = mul(cov, ld3(noise, idx));
    const float opacity = 1.0f / (1.f + gsx::exp(-raw_opacities[idx]));
    const float op_sigmoid = 1.0f / (1.f + gsx::exp(100.f * opacity - 0.5f));
    const float noise_factor = current_lr * op_sigmoid;
    means[idx * 3] += noise_factor * tn.x;
    means[idx * 3 + 1] += noise_factor * tn.y;
    means[idx * 3 + 2] += noise_factor * tn.z;
}

} // namespace gsx

using namespace gsx;

extern "C" int gsx_relocation(int M, const float* opacities, const float* scales, const int32_t* ratios,
                              const float* binoms, int n_max, float* new_opacities, float* new_scales, void* stream) {
    if (M <= 0)
        return GSX_OK; // RelocationCUDA.cu:63-66
    GSX_REQUIRE(opacities && scales && ratios && binoms && new_opacities && new_scales, GSX_ERR_INVALID_ARGUMENT,
                "relocation: null tensor");
    GSX_REQUIRE(n_max > 0, GSX_ERR_INVALID_ARGUMENT, "relocation: n_max %d", n_max);
    hipLaunchKernelGGL(relocation_kernel, dim3(cdiv(M, 256)), dim3(256), 0, (hipStream_t)stream, M, opacities, scales,
                       ratios, binoms, n_max, new_opacities, new_scales);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_add_noise(int N, const float* raw_opacities, const float* raw_scales, const float* raw_quats,
                             const float* noise, float* means, float current_lr, void* stream) {
    if (N <= 0)
        return GSX_OK;
    GSX_REQUIRE(raw_opacities && raw_scales && raw_quats && noise && means, GSX_ERR_INVALID_ARGUMENT,
                "add_noise: null tensor");
    hipLaunchKernelGGL(add_noise_kernel, dim3(cdiv(N, 256)), dim3(256), 0, (hipStream_t)stream, N, raw_opacities,
                       raw_scales, raw_quats, noise, means, current_lr);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}
