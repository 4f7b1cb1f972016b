// adam.hip - fused Adam step (src/training/fastgs/optimizer/include/adam_kernels.cuh:13-36; host side
// src/training/optimizers/fused_adam.cpp:22-95).  Pure HBM streaming: 16 B read + 12 B written per element.
// All parameter groups of a step run in ONE launch (the reference launches once per group): a workgroup
// looks up which group its 1024-element chunk belongs to in a small table passed by value.
#include <string.h>

#include "gsx_common.h"
#include "gsx_step.h"

namespace gsx {

static constexpr uint32_t kAdamVec = 4;                 // elements per lane (one 16-byte access per array)
static constexpr uint32_t kAdamChunk = 256 * kAdamVec;  // elements per workgroup

struct AdamTable {
    float* param[GSX_ADAM_MAX_TENSORS];
    float* exp_avg[GSX_ADAM_MAX_TENSORS];
    float* exp_avg_sq[GSX_ADAM_MAX_TENSORS];
    const float* grad[GSX_ADAM_MAX_TENSORS];
    uint32_t n[GSX_ADAM_MAX_TENSORS];
    uint32_t first_block[GSX_ADAM_MAX_TENSORS + 1];
    float lr[GSX_ADAM_MAX_TENSORS], beta1[GSX_ADAM_MAX_TENSORS], beta2[GSX_ADAM_MAX_TENSORS];
    float eps[GSX_ADAM_MAX_TENSORS], bc1_rcp[GSX_ADAM_MAX_TENSORS], bc2_sqrt_rcp[GSX_ADAM_MAX_TENSORS];
    uint32_t period[GSX_ADAM_MAX_TENSORS], split[GSX_ADAM_MAX_TENSORS];
    float lr2[GSX_ADAM_MAX_TENSORS];
    int32_t skip2[GSX_ADAM_MAX_TENSORS];
    int n_groups;
};

__global__ void __launch_bounds__(256) adam_multi_kernel(const AdamTable tab) {
    int gi = 0;
#pragma unroll
    for (int k = 1; k < GSX_ADAM_MAX_TENSORS; ++k)
        if (k < tab.n_groups && blockIdx.x >= tab.first_block[k])
            gi = k;
    const uint32_t n = tab.n[gi];
    const uint32_t base = (blockIdx.x - tab.first_block[gi]) * kAdamChunk + threadIdx.x * kAdamVec;
    if (base >= n)
        return;
    float* __restrict__ P = tab.param[gi];
    float* __restrict__ M = tab.exp_avg[gi];
    float* __restrict__ V = tab.exp_avg_sq[gi];
    const float* __restrict__ G = tab.grad[gi];
    const float lr = tab.lr[gi], b1 = tab.beta1[gi], b2 = tab.beta2[gi], eps = tab.eps[gi];
    const float c1 = tab.bc1_rcp[gi], c2 = tab.bc2_sqrt_rcp[gi];
    const uint32_t period = tab.period[gi], split = tab.split[gi];
    const float lr2 = tab.lr2[gi];
    const bool skip2 = tab.skip2[gi] != 0;
    const bool aligned = ((((uintptr_t)P) | ((uintptr_t)M) | ((uintptr_t)V) | ((uintptr_t)G)) & 15u) == 0;
    if (aligned && base + kAdamVec <= n) {
        // every array is read once and written once per step: streamed past the caches
        float4 p = load_streaming(reinterpret_cast<const float4*>(P + base));
        float4 m = load_streaming(reinterpret_cast<const float4*>(M + base));
        float4 v = load_streaming(reinterpret_cast<const float4*>(V + base));
        const float4 g = load_streaming(reinterpret_cast<const float4*>(G + base));
        float lrs[4] = {lr, lr, lr, lr};
        bool upd[4] = {true, true, true, true};
        if (period) {
#pragma unroll
            for (uint32_t k = 0; k < 4; ++k) {
                const bool second = ((base + k) % period) >= split;
                lrs[k] = second ? lr2 : lr;
                upd[k] = !(second && skip2);
            }
        }
        if (upd[0])
            adam_one(p.x, m.x, v.x, g.x, lrs[0], b1, b2, eps, c1, c2);
        if (upd[1])
            adam_one(p.y, m.y, v.y, g.y, lrs[1], b1, b2, eps, c1, c2);
        if (upd[2])
            adam_one(p.z, m.z, v.z, g.z, lrs[2], b1, b2, eps, c1, c2);
        if (upd[3])
            adam_one(p.w, m.w, v.w, g.w, lrs[3], b1, b2, eps, c1, c2);
        store_streaming(reinterpret_cast<float4*>(P + base), p);
        store_streaming(reinterpret_cast<float4*>(M + base), m);
        store_streaming(reinterpret_cast<float4*>(V + base), v);
    } else {
        for (uint32_t i = base; i < n && i < base + kAdamVec; ++i) {
            const bool second = period && (i % period) >= split;
            if (second && skip2)
                continue;
            float p = P[i], m = M[i], v = V[i];
            adam_one(p, m, v, G[i], second ? lr2 : lr, b1, b2, eps, c1, c2);
            P[i] = p;
            M[i] = m;
            V[i] = v;
        }
    }
}

} // namespace gsx

using namespace gsx;

extern "C" int gsx_adam_step_multi(const gsx_adam_group* groups, int n_groups, void* stream) {
    GSX_REQUIRE(n_groups >= 0 && n_groups <= GSX_ADAM_MAX_TENSORS, GSX_ERR_INVALID_ARGUMENT,
                "adam_step_multi: %d groups (max %d)", n_groups, GSX_ADAM_MAX_TENSORS);
    GSX_REQUIRE(n_groups == 0 || groups != nullptr, GSX_ERR_INVALID_ARGUMENT, "adam_step_multi: groups is null");
    AdamTable tab;
    memset(&tab, 0, sizeof(tab));
    uint64_t blocks = 0;
    int k = 0;
    for (int i = 0; i < n_groups; ++i) {
        const gsx_adam_group& g = groups[i];
        if (g.n == 0 || g.grad == nullptr) // params without a gradient are skipped (fused_adam.cpp:47-50)
            continue;
        GSX_REQUIRE(g.param && g.exp_avg && g.exp_avg_sq, GSX_ERR_INVALID_ARGUMENT, "adam_step_multi: null tensor");
        GSX_REQUIRE(g.n > 0 && g.n < (1ll << 32), GSX_ERR_INVALID_ARGUMENT, "adam_step_multi: group size %lld",
                    (long long)g.n);
        tab.param[k] = g.param;
        tab.exp_avg[k] = g.exp_avg;
        tab.exp_avg_sq[k] = g.exp_avg_sq;
        tab.grad[k] = g.grad;
        tab.n[k] = (uint32_t)g.n;
        tab.first_block[k] = (uint32_t)blocks;
        tab.lr[k] = g.lr;
        tab.beta1[k] = g.beta1;
        tab.beta2[k] = g.beta2;
        tab.eps[k] = g.eps;
        tab.bc1_rcp[k] = g.bias_correction1_rcp;
        tab.bc2_sqrt_rcp[k] = g.bias_correction2_sqrt_rcp;
        tab.period[k] = g.period;
        tab.split[k] = g.split;
        tab.lr2[k] = g.lr2;
        tab.skip2[k] = g.skip2;
        blocks += cdiv((uint64_t)g.n, kAdamChunk);
        ++k;
    }
    tab.n_groups = k;
    tab.first_block[k] = (uint32_t)blocks;
    if (blocks == 0)
        return GSX_OK;
    GSX_REQUIRE(blocks < (1ull << 31), GSX_ERR_INVALID_ARGUMENT, "adam_step_multi: too many elements");
    hipLaunchKernelGGL(adam_multi_kernel, dim3((uint32_t)blocks), dim3(256), 0, (hipStream_t)stream, tab);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_adam_step(float* param, float* exp_avg, float* exp_avg_sq, const float* grad, int64_t n, float lr,
                             float beta1, float beta2, float eps, float bias_correction1_rcp,
                             float bias_correction2_sqrt_rcp, void* stream) {
    if (n == 0)
        return GSX_OK;
    GSX_REQUIRE(grad != nullptr, GSX_ERR_INVALID_ARGUMENT, "adam_step: grad is null");
    gsx_adam_group g;
    g.param = param;
    g.exp_avg = exp_avg;
    g.exp_avg_sq = exp_avg_sq;
    g.grad = grad;
    g.n = n;
    g.lr = lr;
    g.beta1 = beta1;
    g.beta2 = beta2;
    g.eps = eps;
    g.bias_correction1_rcp = bias_correction1_rcp;
    g.bias_correction2_sqrt_rcp = bias_correction2_sqrt_rcp;
    g.period = 0;
    g.split = 0;
    g.lr2 = 0.f;
    g.skip2 = 0;
    return gsx_adam_step_multi(&g, 1, stream);
}
