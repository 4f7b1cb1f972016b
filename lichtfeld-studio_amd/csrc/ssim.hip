// ssim.hip - fused separable 11x11 SSIM forward / backward (src/training/kernels/ssim.cu:16-27, 64-276, 284-424)
// and the per-pixel parts of the photometric loss around it (src/training/trainer.cpp:126-129,
// include/kernels/fused_ssim.cuh:59-67,84-96,117-122, src/training/rasterization/rasterizer.cpp:205).
//
// One 256-lane workgroup per 16x16 pixel tile and image plane; the 26x26 halo tile is staged in LDS, convolved
// horizontally into a 26x16 intermediate (five moments forward, three chains backward), then vertically.
// Planes are independent workgroups (the reference loops the channels inside one block and re-synchronises).
// Both kernels write every output element, so no zero-fill of the outputs is needed.
#include "gsx_common.h"

namespace gsx {

static constexpr int BX = 16, BY = 16, HALO = 5;
static constexpr int SX = BX + 2 * HALO, SY = BY + 2 * HALO; // 26 x 26
static constexpr int CY = SY;                                // rows of the horizontal-pass result

__constant__ float cGauss[11] = {0.001028380123898387f, 0.0075987582094967365f, 0.036000773310661316f,
                                 0.10936068743467331f,  0.21300552785396576f,   0.26601171493530273f,
                                 0.21300552785396576f,  0.10936068743467331f,   0.036000773310661316f,
                                 0.0075987582094967365f, 0.001028380123898387f};

__device__ __forceinline__ float pix(const float* __restrict__ img, size_t plane, int y, int x, int H, int W) {
    if (x < 0 || x >= W || y < 0 || y >= H)
        return 0.0f;
    return img[plane + (size_t)y * W + x];
}

__global__ void __launch_bounds__(256) fusedssim_kernel(int H, int W, float C1, float C2,
                                                         const float* __restrict__ img1,
                                                         const float* __restrict__ img2, float* __restrict__ ssim_map,
                                                         float* __restrict__ dm_dmu1,
                                                         float* __restrict__ dm_dsigma1_sq,
                                                         float* __restrict__ dm_dsigma12) {
    __shared__ float sTile[SY][SX][2];
    __shared__ float xconv[CY][BX][5];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int pix_x = blockIdx.x * BX + tx, pix_y = blockIdx.y * BY + ty;
    const size_t plane = (size_t)blockIdx.z * H * W;

    // 1) tile + halo, zero padded (:94-119)
    for (int tid = threadIdx.x; tid < SY * SX; tid += 256) {
        const int ly = tid / SX, lx = tid % SX;
        const int gy = blockIdx.y * BY + ly - HALO, gx = blockIdx.x * BX + lx - HALO;
        sTile[ly][lx][0] = pix(img1, plane, gy, gx, H, W);
        sTile[ly][lx][1] = pix(img2, plane, gy, gx, H, W);
    }
    __syncthreads();

    // 2) horizontal 11-tap on the 26 rows (:121-213): symmetric pairs d = 1..5, then the centre
    for (int ly = ty; ly < CY; ly += BY) {
        const int lx = tx + HALO;
        float sumX = 0.f, sumX2 = 0.f, sumY = 0.f, sumY2 = 0.f, sumXY = 0.f;
#pragma unroll
        for (int d = 1; d <= HALO; ++d) {
            const float w = cGauss[HALO - d];
            const float Xl = sTile[ly][lx - d][0], Yl = sTile[ly][lx - d][1];
            const float Xr = sTile[ly][lx + d][0], Yr = sTile[ly][lx + d][1];
            sumX += (Xl + Xr) * w;
            sumX2 += ((Xl * Xl) + (Xr * Xr)) * w;
            sumY += (Yl + Yr) * w;
            sumY2 += ((Yl * Yl) + (Yr * Yr)) * w;
            sumXY += ((Xl * Yl) + (Xr * Yr)) * w;
        }
        const float cX = sTile[ly][lx][0], cY = sTile[ly][lx][1];
        const float wc = cGauss[HALO];
        sumX += cX * wc;
        sumX2 += (cX * cX) * wc;
        sumY += cY * wc;
        sumY2 += (cY * cY) * wc;
        sumXY += (cX * cY) * wc;
        xconv[ly][tx][0] = sumX;
        xconv[ly][tx][1] = sumX2;
        xconv[ly][tx][2] = sumY;
        xconv[ly][tx][3] = sumY2;
        xconv[ly][tx][4] = sumXY;
    }
    __syncthreads();

    // 3) vertical 11-tap + SSIM and its partial derivatives (:215-274)
    {
        const int ly = ty + HALO, lx = tx;
        float out[5] = {0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d = 1; d <= HALO; ++d) {
            const float w = cGauss[HALO - d];
#pragma unroll
            for (int k = 0; k < 5; ++k)
                out[k] += (xconv[ly - d][lx][k] + xconv[ly + d][lx][k]) * w;
        }
#pragma unroll
        for (int k = 0; k < 5; ++k)
            out[k] += xconv[ly][lx][k] * cGauss[HALO];

        if (pix_x < W && pix_y < H) {
            const float mu1 = out[0], mu2 = out[2];
            const float mu1_sq = mu1 * mu1, mu2_sq = mu2 * mu2;
            const float sigma1_sq = out[1] - mu1_sq, sigma2_sq = out[3] - mu2_sq;
            const float sigma12 = out[4] - mu1 * mu2;
            const float A = mu1_sq + mu2_sq + C1;
            const float B = sigma1_sq + sigma2_sq + C2;
            const float C_ = 2.f * mu1 * mu2 + C1;
            const float D_ = 2.f * sigma12 + C2;
            const size_t gi = plane + (size_t)pix_y * W + pix_x;
            ssim_map[gi] = (C_ * D_) / (A * B);
            if (dm_dmu1) {
                dm_dmu1[gi] = ((mu2 * 2.f * D_) / (A * B) - (mu2 * 2.f * C_) / (A * B) -
                               (mu1 * 2.f * C_ * D_) / (A * A * B) + (mu1 * 2.f * C_ * D_) / (A * B * B));
                dm_dsigma1_sq[gi] = (-C_ * D_) / (A * B * B);
                dm_dsigma12[gi] = (2.f * C_) / (A * B);
            }
        }
    }
}

__global__ void __launch_bounds__(256) fusedssim_backward_kernel(
    int H, int W, const float* __restrict__ img1, const float* __restrict__ img2, const float* __restrict__ dL_dmap,
    const float* __restrict__ dm_dmu1, const float* __restrict__ dm_dsigma1_sq, const float* __restrict__ dm_dsigma12,
    float* __restrict__ dL_dimg1) {
    __shared__ float sData[3][SY][SX];
    __shared__ float sScratch[CY][BX][3];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int pix_x = blockIdx.x * BX + tx, pix_y = blockIdx.y * BY + ty;
    const size_t plane = (size_t)blockIdx.z * H * W;

    // (1) load + fuse the chain multiplication (:305-337)
    for (int tid = threadIdx.x; tid < SY * SX; tid += 256) {
        const int row = tid / SX, col = tid % SX;
        const int gy = blockIdx.y * BY + row - HALO, gx = blockIdx.x * BX + col - HALO;
        const float chain = pix(dL_dmap, plane, gy, gx, H, W);
        sData[0][row][col] = pix(dm_dmu1, plane, gy, gx, H, W) * chain;
        sData[1][row][col] = pix(dm_dsigma1_sq, plane, gy, gx, H, W) * chain;
        sData[2][row][col] = pix(dm_dsigma12, plane, gy, gx, H, W) * chain;
    }
    __syncthreads();

    // (2) horizontal pass (:339-383)
    for (int yy = ty; yy < CY; yy += BY) {
        const int lx = tx + HALO;
        float a0 = 0.f, a1 = 0.f, a2 = 0.f;
#pragma unroll
        for (int d = 1; d <= HALO; ++d) {
            const float w = cGauss[HALO - d];
            a0 += (sData[0][yy][lx - d] + sData[0][yy][lx + d]) * w;
            a1 += (sData[1][yy][lx - d] + sData[1][yy][lx + d]) * w;
            a2 += (sData[2][yy][lx - d] + sData[2][yy][lx + d]) * w;
        }
        const float wc = cGauss[HALO];
        a0 += sData[0][yy][lx] * wc;
        a1 += sData[1][yy][lx] * wc;
        a2 += sData[2][yy][lx] * wc;
        sScratch[yy][tx][0] = a0;
        sScratch[yy][tx][1] = a1;
        sScratch[yy][tx][2] = a2;
    }
    __syncthreads();

    // (3) vertical pass -> dL/d(img1) (:385-421)
    if (pix_x < W && pix_y < H) {
        const int ly = ty + HALO, lx = tx;
        float s0 = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int d = 1; d <= HALO; ++d) {
            const float w = cGauss[HALO - d];
            s0 += (sScratch[ly - d][lx][0] + sScratch[ly + d][lx][0]) * w;
            s1 += (sScratch[ly - d][lx][1] + sScratch[ly + d][lx][1]) * w;
            s2 += (sScratch[ly - d][lx][2] + sScratch[ly + d][lx][2]) * w;
        }
        const float wc = cGauss[HALO];
        s0 += sScratch[ly][lx][0] * wc;
        s1 += sScratch[ly][lx][1] * wc;
        s2 += sScratch[ly][lx][2] * wc;
        const size_t gi = plane + (size_t)pix_y * W + pix_x;
        const float p1 = img1[gi], p2 = img2[gi];
        dL_dimg1[gi] = s0 + (2.f * p1) * s1 + (p2)*s2;
    }
}

// ---- loss-side passes ---------------------------------------------------------------------------
static constexpr uint32_t kLossBlock = 256;
static constexpr uint32_t kLossItems = 8;

__device__ __forceinline__ float block_sum_256(float v, float* lds) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1)
        v += __shfl_xor(v, m, 64);
    if ((threadIdx.x & 63u) == 0)
        lds[threadIdx.x >> 6] = v;
    __syncthreads();
    const float r = (lds[0] + lds[1]) + (lds[2] + lds[3]);
    __syncthreads();
    return r;
}

// image[c][y][x] = clamp(render[y][x][c], 0, 1); partial sums of |image - gt| per block
__global__ void __launch_bounds__(256) image_from_render_kernel(uint32_t HW, const float* __restrict__ render_hwc,
                                                                 const float* __restrict__ gt_chw,
                                                                 float* __restrict__ image_chw,
                                                                 float* __restrict__ l1_partials) {
    __shared__ float lds[4];
    float acc = 0.f;
    const uint32_t base = blockIdx.x * kLossBlock * kLossItems;
#pragma unroll
    for (uint32_t it = 0; it < kLossItems; ++it) {
        const uint32_t p = base + it * kLossBlock + threadIdx.x;
        if (p < HW) {
#pragma unroll
            for (uint32_t c = 0; c < 3; ++c) {
                const float r = render_hwc[(size_t)p * 3 + c];
                const float v = gsx::fmin(gsx::fmax(r, 0.0f), 1.0f);
                image_chw[(size_t)c * HW + p] = v;
                if (gt_chw != nullptr)
                    acc += gsx::fabs(v - gt_chw[(size_t)c * HW + p]);
            }
        }
    }
    const float s = block_sum_256(acc, lds);
    if (threadIdx.x == 0 && l1_partials != nullptr)
        l1_partials[blockIdx.x] = s;
}

// partial sums of the SSIM map over the valid crop (whole map when H or W <= 10)
__global__ void __launch_bounds__(256) ssim_valid_partials_kernel(uint32_t CH, uint32_t H, uint32_t W,
                                                                   const float* __restrict__ ssim_map,
                                                                   float* __restrict__ partials) {
    __shared__ float lds[4];
    const bool crop = H > 10 && W > 10;
    const uint32_t HW = H * W;
    float acc = 0.f;
    const uint32_t base = blockIdx.x * kLossBlock * kLossItems;
#pragma unroll
    for (uint32_t it = 0; it < kLossItems; ++it) {
        const uint32_t p = base + it * kLossBlock + threadIdx.x;
        if (p < HW) {
            const uint32_t y = p / W, x = p % W;
            const bool in = !crop || (y >= 5 && y < H - 5 && x >= 5 && x < W - 5);
            if (in)
                for (uint32_t c = 0; c < CH; ++c)
                    acc += ssim_map[(size_t)c * HW + p];
        }
    }
    const float s = block_sum_256(acc, lds);
    if (threadIdx.x == 0)
        partials[blockIdx.x] = s;
}

__global__ void __launch_bounds__(256) photometric_loss_finish_kernel(uint32_t CH, uint32_t H, uint32_t W,
                                                                       float lambda_dssim,
                                                                       const float* __restrict__ l1_partials,
                                                                       const float* __restrict__ ssim_partials,
                                                                       uint32_t n_partials,
                                                                       float* __restrict__ loss_out) {
    __shared__ float lds[4];
    float a = 0.f, b = 0.f;
    // four independent loads in flight per lane: the kernel is one block and pure latency
    float a4[4] = {0.f, 0.f, 0.f, 0.f}, b4[4] = {0.f, 0.f, 0.f, 0.f};
    for (uint32_t i = threadIdx.x; i < n_partials; i += 1024) {
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            const uint32_t j = i + k * 256u;
            if (j < n_partials) {
                a4[k] += l1_partials[j];
                b4[k] += ssim_partials[j];
            }
        }
    }
    a = (a4[0] + a4[1]) + (a4[2] + a4[3]);
    b = (b4[0] + b4[1]) + (b4[2] + b4[3]);
    const float l1_sum = block_sum_256(a, lds);
    const float ss_sum = block_sum_256(b, lds);
    if (threadIdx.x == 0) {
        const bool crop = H > 10 && W > 10;
        const float n_l1 = (float)CH * (float)H * (float)W;
        const float n_ss = crop ? (float)CH * (float)(H - 10) * (float)(W - 10) : n_l1;
        const float l1 = l1_sum / n_l1;
        const float ss = ss_sum / n_ss;
        loss_out[0] = (1.f - lambda_dssim) * l1 + lambda_dssim * (1.f - ss);
        loss_out[1] = l1;
        loss_out[2] = ss;
    }
}

// dL/dmap of mean(map[valid crop]) scaled: `scale` inside the crop, 0 outside (fused_ssim.cuh:84-96)
__global__ void __launch_bounds__(256) ssim_valid_grad_map_kernel(uint32_t CH, uint32_t H, uint32_t W, float scale,
                                                                   float* __restrict__ dL_dmap) {
    const uint32_t HW = H * W;
    const uint32_t p = blockIdx.x * 256u + threadIdx.x;
    if (p >= HW)
        return;
    const bool crop = H > 10 && W > 10;
    const uint32_t y = p / W, x = p % W;
    const bool in = !crop || (y >= 5 && y < H - 5 && x >= 5 && x < W - 5);
    for (uint32_t c = 0; c < CH; ++c)
        dL_dmap[(size_t)c * HW + p] = in ? scale : 0.f;
}

// v_render[y][x][c] = clampVJP( (1-lambda) sign(img - gt) / (3HW) + dL_dimg_ssim[c][y][x] )
__global__ void __launch_bounds__(256) render_grad_from_loss_kernel(uint32_t HW, float l1_scale,
                                                                     const float* __restrict__ render_hwc,
                                                                     const float* __restrict__ image_chw,
                                                                     const float* __restrict__ gt_chw,
                                                                     const float* __restrict__ dL_dimg_ssim,
                                                                     float* __restrict__ v_render_hwc) {
    const uint32_t p = blockIdx.x * 256u + threadIdx.x;
    if (p >= HW)
        return;
#pragma unroll
    for (uint32_t c = 0; c < 3; ++c) {
        const float r = render_hwc[(size_t)p * 3 + c];
        const float d = image_chw[(size_t)c * HW + p] - gt_chw[(size_t)c * HW + p];
        const float sgn = d > 0.f ? 1.f : (d < 0.f ? -1.f : 0.f);
        float g = l1_scale * sgn;
        if (dL_dimg_ssim != nullptr)
            g += dL_dimg_ssim[(size_t)c * HW + p];
        // clamp VJP: gradient passes where 0 <= render <= 1
        v_render_hwc[(size_t)p * 3 + c] = (r >= 0.f && r <= 1.f) ? g : 0.f;
    }
}

// ---- the photometric loss of a training step in two kernels ---------------------------------------
// forward: clamp + HWC -> CHW on load, SSIM moments and derivative maps, per-block partial sums of |image - gt| and
// of the SSIM map over the valid crop (what image_from_render + fusedssim + ssim_valid_partials do in three passes;
// the clamped image and the SSIM map themselves are never written).
__global__ void __launch_bounds__(256) photometric_fwd_kernel(int H, int W, float C1, float C2,
                                                               const float* __restrict__ render_hwc,
                                                               const float* __restrict__ gt_chw,
                                                               float* __restrict__ dm_dmu1,
                                                               float* __restrict__ dm_dsigma1_sq,
                                                               float* __restrict__ dm_dsigma12,
                                                               float* __restrict__ l1_partials,
                                                               float* __restrict__ ssim_partials) {
    __shared__ float sTile[SY][SX][2];
    __shared__ float xconv[CY][BX][5];
    __shared__ float red[4];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int pix_x = blockIdx.x * BX + tx, pix_y = blockIdx.y * BY + ty;
    const int c = blockIdx.z;
    const size_t plane = (size_t)c * H * W;

    for (int tid = threadIdx.x; tid < SY * SX; tid += 256) {
        const int ly = tid / SX, lx = tid % SX;
        const int gy = blockIdx.y * BY + ly - HALO, gx = blockIdx.x * BX + lx - HALO;
        float a = 0.f, b = 0.f;
        if (gx >= 0 && gx < W && gy >= 0 && gy < H) {
            a = gsx::fmin(gsx::fmax(render_hwc[((size_t)gy * W + gx) * 3 + c], 0.0f), 1.0f); // rasterizer.cpp:205
            b = gt_chw[plane + (size_t)gy * W + gx];
        }
        sTile[ly][lx][0] = a;
        sTile[ly][lx][1] = b;
    }
    __syncthreads();
    for (int ly = ty; ly < CY; ly += BY) {
        const int lx = tx + HALO;
        float sumX = 0.f, sumX2 = 0.f, sumY = 0.f, sumY2 = 0.f, sumXY = 0.f;
#pragma unroll
        for (int d = 1; d <= HALO; ++d) {
            const float w = cGauss[HALO - d];
            const float Xl = sTile[ly][lx - d][0], Yl = sTile[ly][lx - d][1];
            const float Xr = sTile[ly][lx + d][0], Yr = sTile[ly][lx + d][1];
            sumX += (Xl + Xr) * w;
            sumX2 += ((Xl * Xl) + (Xr * Xr)) * w;
            sumY += (Yl + Yr) * w;
            sumY2 += ((Yl * Yl) + (Yr * Yr)) * w;
            sumXY += ((Xl * Yl) + (Xr * Yr)) * w;
        }
        const float cX = sTile[ly][lx][0], cY = sTile[ly][lx][1];
        const float wc = cGauss[HALO];
        sumX += cX * wc;
        sumX2 += (cX * cX) * wc;
        sumY += cY * wc;
        sumY2 += (cY * cY) * wc;
        sumXY += (cX * cY) * wc;
        xconv[ly][tx][0] = sumX;
        xconv[ly][tx][1] = sumX2;
        xconv[ly][tx][2] = sumY;
        xconv[ly][tx][3] = sumY2;
        xconv[ly][tx][4] = sumXY;
    }
    __syncthreads();
    float l1 = 0.f, ss = 0.f;
    {
        const int ly = ty + HALO, lx = tx;
        float out[5] = {0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d = 1; d <= HALO; ++d) {
            const float w = cGauss[HALO - d];
#pragma unroll
            for (int k = 0; k < 5; ++k)
                out[k] += (xconv[ly - d][lx][k] + xconv[ly + d][lx][k]) * w;
        }
#pragma unroll
        for (int k = 0; k < 5; ++k)
            out[k] += xconv[ly][lx][k] * cGauss[HALO];
        if (pix_x < W && pix_y < H) {
            const float mu1 = out[0], mu2 = out[2];
            const float mu1_sq = mu1 * mu1, mu2_sq = mu2 * mu2;
            const float sigma1_sq = out[1] - mu1_sq, sigma2_sq = out[3] - mu2_sq;
            const float sigma12 = out[4] - mu1 * mu2;
            const float A = mu1_sq + mu2_sq + C1;
            const float B = sigma1_sq + sigma2_sq + C2;
            const float C_ = 2.f * mu1 * mu2 + C1;
            const float D_ = 2.f * sigma12 + C2;
            const size_t gi = plane + (size_t)pix_y * W + pix_x;
            const bool crop = H > 10 && W > 10;
            if (!crop || (pix_y >= 5 && pix_y < H - 5 && pix_x >= 5 && pix_x < W - 5))
                ss = (C_ * D_) / (A * B);
            dm_dmu1[gi] = ((mu2 * 2.f * D_) / (A * B) - (mu2 * 2.f * C_) / (A * B) -
                           (mu1 * 2.f * C_ * D_) / (A * A * B) + (mu1 * 2.f * C_ * D_) / (A * B * B));
            dm_dsigma1_sq[gi] = (-C_ * D_) / (A * B * B);
            dm_dsigma12[gi] = (2.f * C_) / (A * B);
            l1 = gsx::fabs(sTile[ty + HALO][tx + HALO][0] - sTile[ty + HALO][tx + HALO][1]);
        }
    }
    const uint32_t bid = (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
    const float l1s = block_sum_256(l1, red);
    const float sss = block_sum_256(ss, red);
    if (threadIdx.x == 0) {
        l1_partials[bid] = l1s;
        ssim_partials[bid] = sss;
    }
}

// backward: d loss / d render in one pass - the SSIM chain with d loss / d map = -lambda / count inside the valid crop
// formed on the fly (fused_ssim.cuh:84-96), the L1 sign term, the clamp VJP and the CHW -> HWC permute (what
// fusedssim_backward + render_grad_from_loss do in two passes with two intermediate images).  A block walks the
// three colour planes of its tile and writes the pixel's three gradients together.
__global__ void __launch_bounds__(256) photometric_bwd_kernel(int H, int W, float ssim_scale, float l1_scale,
                                                               const float* __restrict__ render_hwc,
                                                               const float* __restrict__ gt_chw,
                                                               const float* __restrict__ dm_dmu1,
                                                               const float* __restrict__ dm_dsigma1_sq,
                                                               const float* __restrict__ dm_dsigma12,
                                                               float* __restrict__ v_render_hwc) {
    __shared__ float sData[3][SY][SX];
    __shared__ float sScratch[CY][BX][3];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int pix_x = blockIdx.x * BX + tx, pix_y = blockIdx.y * BY + ty;
    const bool inside = pix_x < W && pix_y < H;
    const bool crop = H > 10 && W > 10;
    float g[3] = {0.f, 0.f, 0.f};
    for (int c = 0; c < 3; ++c) {
        const size_t plane = (size_t)c * H * W;
        for (int tid = threadIdx.x; tid < SY * SX; tid += 256) {
            const int row = tid / SX, col = tid % SX;
            const int gy = blockIdx.y * BY + row - HALO, gx = blockIdx.x * BX + col - HALO;
            float d0 = 0.f, d1 = 0.f, d2 = 0.f;
            if (gx >= 0 && gx < W && gy >= 0 && gy < H) {
                const bool valid = !crop || (gy >= 5 && gy < H - 5 && gx >= 5 && gx < W - 5);
                const float chain = valid ? ssim_scale : 0.f;
                const size_t gi = plane + (size_t)gy * W + gx;
                d0 = dm_dmu1[gi] * chain;
                d1 = dm_dsigma1_sq[gi] * chain;
                d2 = dm_dsigma12[gi] * chain;
            }
            sData[0][row][col] = d0;
            sData[1][row][col] = d1;
            sData[2][row][col] = d2;
        }
        __syncthreads();
        for (int yy = ty; yy < CY; yy += BY) {
            const int lx = tx + HALO;
            float a0 = 0.f, a1 = 0.f, a2 = 0.f;
#pragma unroll
            for (int d = 1; d <= HALO; ++d) {
                const float w = cGauss[HALO - d];
                a0 += (sData[0][yy][lx - d] + sData[0][yy][lx + d]) * w;
                a1 += (sData[1][yy][lx - d] + sData[1][yy][lx + d]) * w;
                a2 += (sData[2][yy][lx - d] + sData[2][yy][lx + d]) * w;
            }
            const float wc = cGauss[HALO];
            a0 += sData[0][yy][lx] * wc;
            a1 += sData[1][yy][lx] * wc;
            a2 += sData[2][yy][lx] * wc;
            sScratch[yy][tx][0] = a0;
            sScratch[yy][tx][1] = a1;
            sScratch[yy][tx][2] = a2;
        }
        __syncthreads();
        if (inside) {
            const int ly = ty + HALO, lx = tx;
            float s0 = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll
            for (int d = 1; d <= HALO; ++d) {
                const float w = cGauss[HALO - d];
                s0 += (sScratch[ly - d][lx][0] + sScratch[ly + d][lx][0]) * w;
                s1 += (sScratch[ly - d][lx][1] + sScratch[ly + d][lx][1]) * w;
                s2 += (sScratch[ly - d][lx][2] + sScratch[ly + d][lx][2]) * w;
            }
            const float wc = cGauss[HALO];
            s0 += sScratch[ly][lx][0] * wc;
            s1 += sScratch[ly][lx][1] * wc;
            s2 += sScratch[ly][lx][2] * wc;
            const size_t p = (size_t)pix_y * W + pix_x;
            const float r = render_hwc[p * 3 + c];
            const float p1 = gsx::fmin(gsx::fmax(r, 0.0f), 1.0f), p2 = gt_chw[plane + p];
            const float dssim = s0 + (2.f * p1) * s1 + (p2)*s2;
            const float d = p1 - p2;
            const float sgn = d > 0.f ? 1.f : (d < 0.f ? -1.f : 0.f);
            const float gg = l1_scale * sgn + dssim;
            g[c] = (r >= 0.f && r <= 1.f) ? gg : 0.f; // clamp VJP
        }
        __syncthreads(); // sData / sScratch are rewritten for the next plane
    }
    if (inside) {
        const size_t p = (size_t)pix_y * W + pix_x;
        v_render_hwc[p * 3 + 0] = g[0];
        v_render_hwc[p * 3 + 1] = g[1];
        v_render_hwc[p * 3 + 2] = g[2];
    }
}

} // namespace gsx

using namespace gsx;

extern "C" int gsx_fusedssim(int B, int CH, int H, int W, float C1, float C2, const float* img1, const float* img2,
                             float* ssim_map, float* dm_dmu1, float* dm_dsigma1_sq, float* dm_dsigma12,
                             void* stream) {
    if (B <= 0 || CH <= 0 || H <= 0 || W <= 0)
        return GSX_OK;
    GSX_REQUIRE(img1 && img2 && ssim_map, GSX_ERR_INVALID_ARGUMENT, "fusedssim: null tensor");
    const bool train = dm_dmu1 != nullptr;
    GSX_REQUIRE(train == (dm_dsigma1_sq != nullptr) && train == (dm_dsigma12 != nullptr), GSX_ERR_INVALID_ARGUMENT,
                "fusedssim: the three derivative maps must be given together");
    GSX_REQUIRE((int64_t)B * CH <= 65535, GSX_ERR_INVALID_ARGUMENT, "fusedssim: B*CH too large");
    const dim3 grid((W + BX - 1) / BX, (H + BY - 1) / BY, B * CH);
    hipLaunchKernelGGL(fusedssim_kernel, grid, dim3(256), 0, (hipStream_t)stream, H, W, C1, C2, img1, img2, ssim_map,
                       dm_dmu1, dm_dsigma1_sq, dm_dsigma12);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_fusedssim_backward(int B, int CH, int H, int W, float C1, float C2, const float* img1,
                                      const float* img2, const float* dL_dmap, const float* dm_dmu1,
                                      const float* dm_dsigma1_sq, const float* dm_dsigma12, float* dL_dimg1,
                                      void* stream) {
    (void)C1;
    (void)C2;
    if (B <= 0 || CH <= 0 || H <= 0 || W <= 0)
        return GSX_OK;
    GSX_REQUIRE(img1 && img2 && dL_dmap && dm_dmu1 && dm_dsigma1_sq && dm_dsigma12 && dL_dimg1,
                GSX_ERR_INVALID_ARGUMENT, "fusedssim_backward: null tensor");
    GSX_REQUIRE((int64_t)B * CH <= 65535, GSX_ERR_INVALID_ARGUMENT, "fusedssim_backward: B*CH too large");
    const dim3 grid((W + BX - 1) / BX, (H + BY - 1) / BY, B * CH);
    hipLaunchKernelGGL(fusedssim_backward_kernel, grid, dim3(256), 0, (hipStream_t)stream, H, W, img1, img2, dL_dmap,
                       dm_dmu1, dm_dsigma1_sq, dm_dsigma12, dL_dimg1);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" uint32_t gsx_image_loss_blocks(uint32_t H, uint32_t W) {
    return cdiv((uint64_t)H * W, kLossBlock * kLossItems);
}

extern "C" int gsx_image_from_render(uint32_t H, uint32_t W, const float* render_hwc, const float* gt_chw,
                                     float* image_chw, float* l1_partials, void* stream) {
    if ((uint64_t)H * W == 0)
        return GSX_OK;
    GSX_REQUIRE(render_hwc && image_chw, GSX_ERR_INVALID_ARGUMENT, "image_from_render: null tensor");
    GSX_REQUIRE((uint64_t)H * W < (1ull << 30), GSX_ERR_INVALID_ARGUMENT, "image_from_render: image too large");
    hipLaunchKernelGGL(image_from_render_kernel, dim3(gsx_image_loss_blocks(H, W)), dim3(256), 0,
                       (hipStream_t)stream, H * W, render_hwc, gt_chw, image_chw, l1_partials);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_ssim_valid_partials(uint32_t CH, uint32_t H, uint32_t W, const float* ssim_map, float* partials,
                                       void* stream) {
    if ((uint64_t)H * W == 0)
        return GSX_OK;
    GSX_REQUIRE(ssim_map && partials, GSX_ERR_INVALID_ARGUMENT, "ssim_valid_partials: null tensor");
    hipLaunchKernelGGL(ssim_valid_partials_kernel, dim3(gsx_image_loss_blocks(H, W)), dim3(256), 0,
                       (hipStream_t)stream, CH, H, W, ssim_map, partials);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_photometric_loss_finish(uint32_t CH, uint32_t H, uint32_t W, float lambda_dssim,
                                           const float* l1_partials, const float* ssim_partials, uint32_t n_partials,
                                           float* loss_out, void* stream) {
    GSX_REQUIRE(l1_partials && ssim_partials && loss_out, GSX_ERR_INVALID_ARGUMENT,
                "photometric_loss_finish: null tensor");
    hipLaunchKernelGGL(photometric_loss_finish_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, CH, H, W,
                       lambda_dssim, l1_partials, ssim_partials, n_partials, loss_out);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_ssim_valid_grad_map(uint32_t CH, uint32_t H, uint32_t W, float scale, float* dL_dmap,
                                       void* stream) {
    if ((uint64_t)H * W == 0)
        return GSX_OK;
    GSX_REQUIRE(dL_dmap, GSX_ERR_INVALID_ARGUMENT, "ssim_valid_grad_map: null tensor");
    hipLaunchKernelGGL(ssim_valid_grad_map_kernel, dim3(cdiv((uint64_t)H * W, 256)), dim3(256), 0,
                       (hipStream_t)stream, CH, H, W, scale, dL_dmap);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_render_grad_from_loss(uint32_t H, uint32_t W, float lambda_dssim, const float* render_hwc,
                                         const float* image_chw, const float* gt_chw, const float* dL_dimg_ssim,
                                         float* v_render_hwc, void* stream) {
    if ((uint64_t)H * W == 0)
        return GSX_OK;
    GSX_REQUIRE(render_hwc && image_chw && gt_chw && v_render_hwc, GSX_ERR_INVALID_ARGUMENT,
                "render_grad_from_loss: null tensor");
    const float l1_scale = (1.f - lambda_dssim) / (3.f * (float)H * (float)W);
    hipLaunchKernelGGL(render_grad_from_loss_kernel, dim3(cdiv((uint64_t)H * W, 256)), dim3(256), 0,
                       (hipStream_t)stream, H * W, l1_scale, render_hwc, image_chw, gt_chw, dL_dimg_ssim,
                       v_render_hwc);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" uint32_t gsx_photometric_partials(uint32_t H, uint32_t W) {
    return 3u * cdiv(W, (uint32_t)BX) * cdiv(H, (uint32_t)BY);
}

extern "C" int gsx_photometric_loss_forward(uint32_t H, uint32_t W, float C1, float C2, const float* render_hwc,
                                            const float* gt_chw, float* dm_dmu1, float* dm_dsigma1_sq,
                                            float* dm_dsigma12, float* l1_partials, float* ssim_partials,
                                            void* stream) {
    if ((uint64_t)H * W == 0)
        return GSX_OK;
    GSX_REQUIRE(render_hwc && gt_chw && dm_dmu1 && dm_dsigma1_sq && dm_dsigma12 && l1_partials && ssim_partials,
                GSX_ERR_INVALID_ARGUMENT, "photometric_loss_forward: null tensor");
    GSX_REQUIRE((uint64_t)H * W < (1ull << 30), GSX_ERR_INVALID_ARGUMENT, "photometric_loss_forward: image too large");
    const dim3 grid(cdiv(W, (uint32_t)BX), cdiv(H, (uint32_t)BY), 3);
    hipLaunchKernelGGL(photometric_fwd_kernel, grid, dim3(256), 0, (hipStream_t)stream, (int)H, (int)W, C1, C2,
                       render_hwc, gt_chw, dm_dmu1, dm_dsigma1_sq, dm_dsigma12, l1_partials, ssim_partials);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_photometric_loss_backward(uint32_t H, uint32_t W, float lambda_dssim, const float* render_hwc,
                                             const float* gt_chw, const float* dm_dmu1, const float* dm_dsigma1_sq,
                                             const float* dm_dsigma12, float* v_render_hwc, void* stream) {
    if ((uint64_t)H * W == 0)
        return GSX_OK;
    GSX_REQUIRE(render_hwc && gt_chw && dm_dmu1 && dm_dsigma1_sq && dm_dsigma12 && v_render_hwc,
                GSX_ERR_INVALID_ARGUMENT, "photometric_loss_backward: null tensor");
    const bool crop = H > 10 && W > 10;
    const float count = crop ? 3.f * (float)(H - 10) * (float)(W - 10) : 3.f * (float)H * (float)W;
    const float ssim_scale = -lambda_dssim / count;
    const float l1_scale = (1.f - lambda_dssim) / (3.f * (float)H * (float)W);
    const dim3 grid(cdiv(W, (uint32_t)BX), cdiv(H, (uint32_t)BY));
    hipLaunchKernelGGL(photometric_bwd_kernel, grid, dim3(256), 0, (hipStream_t)stream, (int)H, (int)W, ssim_scale,
                       l1_scale, render_hwc, gt_chw, dm_dmu1, dm_dsigma1_sq, dm_dsigma12, v_render_hwc);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}
