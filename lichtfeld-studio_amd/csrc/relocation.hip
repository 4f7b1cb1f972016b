// relocation.hip - MCMC relocation (Eq. 9) and noise injection (gsplat/RelocationCUDA.cu:11-43, 88-144).
#include "gsx_common.h"

#include <string.h>

namespace gsx {

// Eq. 9 for one Gaussian: opacity and scale factor after splitting it into n copies (RelocationCUDA.cu:25-42)
__device__ __forceinline__ void relocate_one(float op, int n_idx, const float* __restrict__ binoms, int n_max,
                                             float& new_o, float& coeff) {
    float denom_sum = 0.0f;
    new_o = 1.0f - gsx::pow(1.0f - op, 1.0f / (float)n_idx);
    for (int i = 1; i <= n_idx; ++i)
        for (int k = 0; k <= (i - 1); ++k) {
            const float bin_coeff = binoms[(i - 1) * n_max + k];
            const float sgn = (k & 1) ? -1.0f : 1.0f;
            const float term = (sgn / gsx::sqrt((float)(k + 1))) * gsx::pow(new_o, (float)(k + 1));
            denom_sum += (bin_coeff * term);
        }
    coeff = (op / denom_sum);
}

__global__ void __launch_bounds__(256) relocation_kernel(int M, const float* __restrict__ opacities,
                                                          const float* __restrict__ scales,
                                                          const int32_t* __restrict__ ratios,
                                                          const float* __restrict__ binoms, int n_max,
                                                          float* __restrict__ new_opacities,
                                                          float* __restrict__ new_scales) {
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= M)
        return;
    float new_o, coeff;
    relocate_one(opacities[idx], ratios[idx], binoms, n_max, new_o, coeff);
    new_opacities[idx] = new_o;
#pragma unroll
    for (int i = 0; i < 3; ++i)
        new_scales[idx * 3 + i] = coeff * scales[idx * 3 + i];
}

// ---- MCMC::relocate_gs after the index sets are chosen (mcmc.cpp:141-187) ----
// pass 0 / 1: occurrences of each sampled index (ratios = 1 + count, mcmc.cpp:141-144)
__global__ void __launch_bounds__(256) mcmc_count_kernel(uint32_t n, const int64_t* __restrict__ sampled,
                                                          int32_t* __restrict__ counts, int add) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n)
        return;
    if (add)
        atomicAdd(&counts[sampled[i]], 1);
    else
        counts[sampled[i]] = 0;
}

// pass 2: new opacity / scales of every sampled Gaussian from its CURRENT raw parameters (:136-160); results go to
// scratch so that no thread reads a row that another one has already rewritten
__global__ void __launch_bounds__(256) mcmc_relocate_compute_kernel(
    uint32_t n, const int64_t* __restrict__ sampled, const int32_t* __restrict__ counts,
    const float* __restrict__ opacity_raw, const float* __restrict__ scaling_raw, const float* __restrict__ binoms,
    int n_max, float min_opacity, float* __restrict__ new_opacity_raw, float* __restrict__ new_scaling_raw) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n)
        return;
    const int64_t s = sampled[i];
    const int ratio = min(1 + counts[s], n_max); // :147-148
    const float op = gsx::sigmoid(opacity_raw[s]);
    float new_o, coeff;
    relocate_one(op, ratio, binoms, n_max, new_o, coeff);
    new_o = gsx::fmin(gsx::fmax(new_o, min_opacity), 1.0f - 1e-7f); // :160
    new_opacity_raw[i] = gsx::log(new_o / (1.0f - new_o));           // torch::logit, :165-169
#pragma unroll
    for (int a = 0; a < 3; ++a)
        new_scaling_raw[i * 3 + a] = gsx::log(coeff * gsx::exp(scaling_raw[s * 3 + a])); // :171
}

__global__ void __launch_bounds__(256) mcmc_relocate_store_kernel(uint32_t n, const int64_t* __restrict__ sampled,
                                                                   const float* __restrict__ new_opacity_raw,
                                                                   const float* __restrict__ new_scaling_raw,
                                                                   float* __restrict__ opacity_raw,
                                                                   float* __restrict__ scaling_raw) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n)
        return;
    const int64_t s = sampled[i]; // duplicates of one index carry identical values
    opacity_raw[s] = new_opacity_raw[i];
#pragma unroll
    for (int a = 0; a < 3; ++a)
        scaling_raw[s * 3 + a] = new_scaling_raw[i * 3 + a];
}

struct RowTable {
    float* data[GSX_MCMC_MAX_TENSORS];
    uint32_t row_floats[GSX_MCMC_MAX_TENSORS];
    uint32_t is_state[GSX_MCMC_MAX_TENSORS];
};

// pass 4: parameter rows dead[i] <- sampled[i] (:175-180); optimiser-state rows of sampled[i] <- 0 (:100-104).
// blockIdx.y = tensor; one thread per (i, float of the row)
__global__ void __launch_bounds__(256) mcmc_rows_kernel(uint32_t n, const int64_t* __restrict__ sampled,
                                                         const int64_t* __restrict__ dead, RowTable tab) {
    const uint32_t e = blockIdx.y;
    const uint32_t r = tab.row_floats[e];
    const uint64_t t = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= (uint64_t)n * r)
        return;
    const uint32_t i = (uint32_t)(t / r), f = (uint32_t)(t % r);
    float* __restrict__ p = tab.data[e];
    const int64_t s = sampled[i];
    if (tab.is_state[e] == 1u)
        p[s * r + f] = 0.f; // relocate_gs: moments of the sampled Gaussian restart
    else if (tab.is_state[e] == 2u)
        p[dead[i] * r + f] = 0.f; // add_new_gs: moments of the new row start at zero
    else
        p[dead[i] * r + f] = p[s * r + f];
}

// ---- counter-based normal draws (torch::randn_like of mcmc.cpp:358 generated where it is consumed) ----
// Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11), counter
// (row, offset lo, offset hi, 0), key = seed; two Box-Muller pairs give the row's three N(0,1) values.
__device__ __forceinline__ void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                              uint32_t k1, uint32_t* out) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
        c0 = n0, c1 = n1, c2 = n2, c3 = n3;
        k0 += 0x9E3779B9u, k1 += 0xBB67AE85u;
    }
    out[0] = c0, out[1] = c1, out[2] = c2, out[3] = c3;
}

__device__ __forceinline__ vec3 philox_normal3(uint32_t row, uint64_t seed, uint64_t offset) {
    uint32_t u[4];
    philox4x32_10(row, (uint32_t)offset, (uint32_t)(offset >> 32), 0u, (uint32_t)seed, (uint32_t)(seed >> 32), u);
    const float scale = 5.9604644775390625e-8f; // 2^-24
    // radius from a uniform in (0, 1], angle pi (2 v - 1) with v uniform in [0, 1)
    const float ra = gsx::sqrt(-2.0f * gsx::log((float)((u[0] >> 8) + 1u) * scale));
    const float rb = gsx::sqrt(-2.0f * gsx::log((float)((u[2] >> 8) + 1u) * scale));
    const float pa = 3.14159265358979323846f * (2.0f * ((float)(u[1] >> 8) * scale) - 1.0f);
    const float pb = 3.14159265358979323846f * (2.0f * ((float)(u[3] >> 8) * scale) - 1.0f);
    return mk3(ra * gsx::cos(pa), ra * gsx::sin(pa), rb * gsx::cos(pb));
}

__global__ void __launch_bounds__(256) philox_randn3_kernel(uint32_t N, uint64_t seed, uint64_t offset,
                                                             float* __restrict__ out) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= N)
        return;
    const vec3 z = philox_normal3(idx, seed, offset);
    out[3 * (size_t)idx] = z.x, out[3 * (size_t)idx + 1] = z.y, out[3 * (size_t)idx + 2] = z.z;
}

// NOISE_FROM_RNG: the N(0,1) row is drawn in the kernel (noise == nullptr) instead of read
template <bool NOISE_FROM_RNG>
__global__ void __launch_bounds__(256) add_noise_kernel(int N, const float* __restrict__ raw_opacities,
                                                         const float* __restrict__ raw_scales,
                                                         const float* __restrict__ raw_quats,
                                                         const float* __restrict__ noise, float* __restrict__ means,
                                                         float current_lr, uint64_t seed, uint64_t offset) {
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
    const vec3 tn = mul(cov, NOISE_FROM_RNG ? philox_normal3((uint32_t)idx, seed, offset) : ld3(noise, idx));
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
    hipLaunchKernelGGL(add_noise_kernel<false>, dim3(cdiv(N, 256)), dim3(256), 0, (hipStream_t)stream, N,
                       raw_opacities, raw_scales, raw_quats, noise, means, current_lr, (uint64_t)0, (uint64_t)0);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_philox_randn3(uint32_t N, uint64_t seed, uint64_t offset, float* out, void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(out != nullptr, GSX_ERR_INVALID_ARGUMENT, "philox_randn3: null tensor");
    hipLaunchKernelGGL(philox_randn3_kernel, dim3(cdiv(N, 256)), dim3(256), 0, (hipStream_t)stream, N, seed, offset, out);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_add_noise_philox(int N, const float* raw_opacities, const float* raw_scales,
                                    const float* raw_quats, float* means, float current_lr, uint64_t seed,
                                    uint64_t offset, void* stream) {
    if (N <= 0)
        return GSX_OK;
    GSX_REQUIRE(raw_opacities && raw_scales && raw_quats && means, GSX_ERR_INVALID_ARGUMENT,
                "add_noise_philox: null tensor");
    hipLaunchKernelGGL(add_noise_kernel<true>, dim3(cdiv(N, 256)), dim3(256), 0, (hipStream_t)stream, N,
                       raw_opacities, raw_scales, raw_quats, (const float*)nullptr, means, current_lr, seed, offset);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" size_t gsx_mcmc_relocate_workspace_bytes(uint32_t N, uint32_t n_idx) {
    return align_up((size_t)N * 4, 256) + align_up((size_t)n_idx * 4, 256) + align_up((size_t)n_idx * 12, 256);
}

extern "C" int gsx_mcmc_relocate(uint32_t N, uint32_t n_idx, const int64_t* sampled_idxs, const int64_t* dead_idxs,
                                 const float* binoms, int n_max, float min_opacity, float* opacity_raw,
                                 float* scaling_raw, const gsx_row_tensor* tensors_host, int n_tensors,
                                 void* workspace, size_t workspace_bytes, void* stream) {
    if (n_idx == 0)
        return GSX_OK; // mcmc.cpp:126-127
    GSX_REQUIRE(sampled_idxs && dead_idxs && binoms && opacity_raw && scaling_raw, GSX_ERR_INVALID_ARGUMENT,
                "mcmc_relocate: null tensor");
    GSX_REQUIRE(n_max > 0 && n_tensors >= 0 && n_tensors <= GSX_MCMC_MAX_TENSORS && (n_tensors == 0 || tensors_host),
                GSX_ERR_INVALID_ARGUMENT, "mcmc_relocate: n_max %d, n_tensors %d (max %d)", n_max, n_tensors,
                GSX_MCMC_MAX_TENSORS);
    GSX_REQUIRE(workspace && ((uintptr_t)workspace & 255) == 0 &&
                    workspace_bytes >= gsx_mcmc_relocate_workspace_bytes(N, n_idx),
                GSX_ERR_WORKSPACE, "mcmc_relocate: workspace of %zu bytes, need %zu (256-byte aligned)",
                workspace_bytes, gsx_mcmc_relocate_workspace_bytes(N, n_idx));
    RowTable tab;
    memset(&tab, 0, sizeof(tab));
    uint32_t max_row = 0;
    for (int e = 0; e < n_tensors; ++e) {
        GSX_REQUIRE(tensors_host[e].data && tensors_host[e].row_floats > 0 &&
                        tensors_host[e].is_optimizer_state >= 0 && tensors_host[e].is_optimizer_state <= 2,
                    GSX_ERR_INVALID_ARGUMENT, "mcmc_relocate: tensor %d is null, has empty rows or a bad role", e);
        tab.data[e] = tensors_host[e].data;
        tab.row_floats[e] = tensors_host[e].row_floats;
        tab.is_state[e] = (uint32_t)tensors_host[e].is_optimizer_state;
        max_row = tensors_host[e].row_floats > max_row ? tensors_host[e].row_floats : max_row;
    }
    char* ws = (char*)workspace;
    int32_t* counts = (int32_t*)ws;
    float* new_op = (float*)(ws + align_up((size_t)N * 4, 256));
    float* new_sc = (float*)((char*)new_op + align_up((size_t)n_idx * 4, 256));
    hipStream_t st = (hipStream_t)stream;
    const dim3 g(cdiv(n_idx, 256)), b(256);
    hipLaunchKernelGGL(mcmc_count_kernel, g, b, 0, st, n_idx, sampled_idxs, counts, 0);
    hipLaunchKernelGGL(mcmc_count_kernel, g, b, 0, st, n_idx, sampled_idxs, counts, 1);
    hipLaunchKernelGGL(mcmc_relocate_compute_kernel, g, b, 0, st, n_idx, sampled_idxs, counts, opacity_raw,
                       scaling_raw, binoms, n_max, min_opacity, new_op, new_sc);
    hipLaunchKernelGGL(mcmc_relocate_store_kernel, g, b, 0, st, n_idx, sampled_idxs, new_op, new_sc, opacity_raw,
                       scaling_raw);
    if (n_tensors) {
        const uint64_t per = (uint64_t)n_idx * max_row;
        GSX_REQUIRE((per + 255) / 256 < (1ull << 31), GSX_ERR_OVERFLOW, "mcmc_relocate: %u rows x %u floats", n_idx,
                    max_row);
        hipLaunchKernelGGL(mcmc_rows_kernel, dim3((uint32_t)cdiv(per, (uint64_t)256), n_tensors), b, 0, st, n_idx,
                           sampled_idxs, dead_idxs, tab);
    }
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}
