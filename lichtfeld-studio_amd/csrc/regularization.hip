// regularization.hip - scale / opacity L1 regularisation of the MCMC strategy
// (src/training/kernels/regularization.cu:20-57, 60-90, 96-163, 171-289; called from trainer.cpp:136-174):
//   scale:   loss = w mean(exp(scaling_raw)),       d loss / d scaling_raw += (w / n) exp(x)
//   opacity: loss = w mean(sigmoid(opacity_raw)),   d loss / d opacity_raw += (w / n) s (1 - s)
// The reference copies each loss value to the host right away (a blocking cudaMemcpy per call); here the value
// stays in device memory.  A training loop that uses gsx_backward_update_fused does not need the gradient half at
// all (the fused pass adds the two terms itself) and calls these only when it wants the loss values.
#include "gsx_common.h"

namespace gsx {

static constexpr uint32_t kRegMaxBlocks = 1024;

template <int MODE> // 0: exp, 1: sigmoid
__global__ void __launch_bounds__(256) l1_regularization_kernel(const float* __restrict__ params,
                                                                 float* __restrict__ param_grads, uint32_t n,
                                                                 float grad_scale, float* __restrict__ block_sums) {
    __shared__ float lds[4];
    float local_sum = 0.f;
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += gridDim.x * 256u) {
        const float x = params[i];
        float value, deriv;
        if (MODE == 0) {
            value = gsx::exp(x);
            deriv = value;
        } else {
            value = gsx::sigmoid(x);
            deriv = value * (1.0f - value);
        }
        local_sum += value;
        if (param_grads != nullptr)
            param_grads[i] += grad_scale * deriv; // every element is visited exactly once: no atomic needed
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1)
        local_sum += __shfl_xor(local_sum, m, 64);
    if ((threadIdx.x & 63u) == 0)
        lds[threadIdx.x >> 6] = local_sum;
    __syncthreads();
    if (threadIdx.x == 0)
        block_sums[blockIdx.x] = (lds[0] + lds[1]) + (lds[2] + lds[3]);
}

__global__ void __launch_bounds__(256) l1_regularization_finish_kernel(const float* __restrict__ block_sums,
                                                                        uint32_t num_blocks, float weight, uint32_t n,
                                                                        float* __restrict__ out) {
    __shared__ float lds[4];
    float s = 0.f;
    for (uint32_t i = threadIdx.x; i < num_blocks; i += 256)
        s += block_sums[i];
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1)
        s += __shfl_xor(s, m, 64);
    if ((threadIdx.x & 63u) == 0)
        lds[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0)
        out[0] = weight * (((lds[0] + lds[1]) + (lds[2] + lds[3])) / (float)n); // loss = weight * mean
}

template <int MODE>
static int run(const char* who, const float* params, float* param_grads, int64_t n, float weight, float* partials,
               float* loss_out, void* stream) {
    if (weight == 0.0f || n <= 0) // regularization.cu:96-99, 110-113: nothing to add, loss 0
        return GSX_OK;
    GSX_REQUIRE(params && partials && loss_out, GSX_ERR_INVALID_ARGUMENT, "%s: null tensor", who);
    GSX_REQUIRE(n < (1ll << 31), GSX_ERR_INVALID_ARGUMENT, "%s: n too large", who);
    const uint32_t blocks = min(cdiv((uint64_t)n, 256), kRegMaxBlocks);
    hipLaunchKernelGGL((l1_regularization_kernel<MODE>), dim3(blocks), dim3(256), 0, (hipStream_t)stream, params,
                       param_grads, (uint32_t)n, weight / (float)n, partials);
    GSX_LAUNCH_CHECK();
    hipLaunchKernelGGL(l1_regularization_finish_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, partials, blocks,
                       weight, (uint32_t)n, loss_out);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

} // namespace gsx

extern "C" uint32_t gsx_l1_regularization_partials(void) { return gsx::kRegMaxBlocks; }

extern "C" int gsx_exp_l1_regularization(const float* params, float* param_grads, int64_t n, float weight,
                                         float* partials, float* loss_out, void* stream) {
    return gsx::run<0>("exp_l1_regularization", params, param_grads, n, weight, partials, loss_out, stream);
}

extern "C" int gsx_sigmoid_l1_regularization(const float* params, float* param_grads, int64_t n, float weight,
                                             float* partials, float* loss_out, void* stream) {
    return gsx::run<1>("sigmoid_l1_regularization", params, param_grads, n, weight, partials, loss_out, stream);
}
