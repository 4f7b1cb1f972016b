// ssim.hip - separable 11x11 SSIM forward / backward as column strips streamed through registers, and the per-pixel
// parts of the photometric loss around it.  What is computed: src/training/kernels/ssim.cu:16-27 (window), :64-276
// (forward), :284-424 (backward); src/training/trainer.cpp:126-129, include/kernels/fused_ssim.cuh:59-67,84-96,117-122
// (valid crop, mean), src/training/rasterization/rasterizer.cpp:205 (clamp).
//
// Organisation (gfx950).  A wave owns a strip of one image plane: 64 adjacent columns (one per lane) by kFwdRows /
// output rows, and walks it top to bottom, one INPUT row per step:
//   * the row's 64 + 10 values per image go through two wave-private LDS rows, from which every lane reads its
//     eleven horizontal taps with unit stride across the lanes (no bank conflicts, no workgroup barrier: the four
//     waves of a workgroup never talk to each other);
//   * the horizontally filtered moments of the last eleven input rows stay in REGISTERS (a sliding window per lane);
//     once the window is full every further input row completes one output row - the vertical filter reads no
//     memory at all;
//   * input rows are requested from memory two steps before they are processed.
// A strip re-reads 10 halo rows per strip and 10 halo columns per 64; neighbouring strips run at the same time
// and meet in L2, and the three colour planes of the interleaved render are three waves of one workgroup, so the
// render's cache lines are fetched once.
// Each output applies the taps in the reference's order (symmetric pairs from the centre outwards, then the centre;
// rows after columns) and the reference's quotients, so results do not depend on the strip geometry and equal the CPU
// checker's to the last bit.  (Sharing two reciprocals between the seven divisions of a pixel saves a seventh of the
// instructions and moves d loss / d render by a few units in the last place - which the gradients of Gaussians that
// vanish by cancellation then show at 13 times their rounding scale: not taken.)
#include "gsx_common.h"

namespace gsx {

static constexpr int HALO = 5;
static constexpr int kStripCols = 64;  // one per lane
static constexpr int kFwdRows = 12;    // output rows per forward strip: (12 + 10) / 12 input rows per output row
static constexpr int kBwdRows = 8;     // backward strips: little arithmetic, more waves to hide the loads behind
static constexpr int kRowFloats = kStripCols + 2 * HALO + 6; // an LDS row, padded to 80 floats

__constant__ float cGauss[11] = {0.001028380123898387f, 0.0075987582094967365f, 0.036000773310661316f,
                                 0.10936068743467331f,  0.21300552785396576f,   0.26601171493530273f,
                                 0.21300552785396576f,  0.10936068743467331f,   0.036000773310661316f,
                                 0.0075987582094967365f, 0.001028380123898387f};

// where a strip lies
struct Strip {
    int col0, row0; // first output column / row
    int H, W;
};

// One value per lane for the columns col0 - 5 + lane (lane 0..63) and, in the lanes below 10, a second one for the
// columns col0 + 59 + lane: the 74 columns an input row contributes to a strip.  Outside the image: 0.
template <class Load>
__device__ __forceinline__ void request_row(const Strip& st, int row, int lane, const Load& load, float* main_v,
                                            float* halo_v) {
    const bool row_in = row >= 0 && row < st.H;
    const int cm = st.col0 - HALO + lane, ch = st.col0 + kStripCols - HALO + lane;
    *main_v = (row_in && cm >= 0 && cm < st.W) ? load(row, cm) : 0.0f;
    *halo_v = (lane < 2 * HALO && row_in && ch < st.W) ? load(row, ch) : 0.0f;
}

// the wave's LDS row receives the 74 values; afterwards lane l finds column col0 + l + d at index l + 5 + d
__device__ __forceinline__ void publish_row(float* lds_row, int lane, float main_v, float halo_v) {
    __builtin_amdgcn_wave_barrier(); // the previous row's taps have been read
    lds_row[lane] = main_v;
    if (lane < 2 * HALO)
        lds_row[kStripCols + lane] = halo_v;
    __builtin_amdgcn_wave_barrier();
}

// eleven-tap filter of one window (index 0 = oldest = top row): pairs from the centre outwards, then the centre
template <int N>
__device__ __forceinline__ void filter_window(const float (&win)[N][11], float (&out)[N]) {
#pragma unroll
    for (int k = 0; k < N; ++k)
        out[k] = 0.f;
#pragma unroll
    for (int d = 1; d <= HALO; ++d) {
        const float w = cGauss[HALO - d];
#pragma unroll
        for (int k = 0; k < N; ++k)
            out[k] += (win[k][HALO - d] + win[k][HALO + d]) * w;
    }
#pragma unroll
    for (int k = 0; k < N; ++k)
        out[k] += win[k][HALO] * cGauss[HALO];
}

// The window slides by register moves (ten per moment and row).  Unrolling the row loop eleven times makes every
// slot a fixed register and removes the moves, but the eleven copies of the loop body no longer fit the instruction
// cache two CUs share: measured 60 / 67 us against 56 / 46 us for the two loss kernels at 1237 x 822.
template <int N>
__device__ __forceinline__ void push_window(float (&win)[N][11], const float (&row)[N]) {
#pragma unroll
    for (int k = 0; k < N; ++k) {
#pragma unroll
        for (int j = 0; j < 10; ++j)
            win[k][j] = win[k][j + 1];
        win[k][10] = row[k];
    }
}

// ---- forward -----------------------------------------------------------------------------------------------------
// X / Y: loaders of the two images for this plane (row, column) -> value.  Per output pixel `emit(row, col, ssim,
// dmu1, dsigma1_sq, dsigma12)` is called (image pixels only); returns the lane's sum of |X - Y| over its output pixels.
// lds: two rows of kRowFloats (X and Y of the current input row).  Input rows are requested two steps ahead of their use.
template <int ROWS, class LoadX, class LoadY, class Emit>
__device__ __forceinline__ float ssim_forward_strip(const Strip& st, float C1, float C2, float* lds,
                                                    const LoadX& loadx, const LoadY& loady, const Emit& emit) {
    const int lane = threadIdx.x & 63;
    const int col = st.col0 + lane;
    const int row_end = min(st.row0 + ROWS, st.H); // one past the last output row
    const int last_in = row_end + HALO;             // one past the last input row
    float* lds_x = lds;
    float* lds_y = lds + kRowFloats;
    float win[5][11];
#pragma unroll
    for (int k = 0; k < 5; ++k)
#pragma unroll
        for (int j = 0; j < 11; ++j)
            win[k][j] = 0.f;
    float l1 = 0.f;
    float xm[2], xh[2], ym[2], yh[2]; // [0]: the next row to publish, [1]: the one after it
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        request_row(st, st.row0 - HALO + k, lane, loadx, &xm[k], &xh[k]);
        request_row(st, st.row0 - HALO + k, lane, loady, &ym[k], &yh[k]);
    }
    for (int row = st.row0 - HALO; row < last_in; ++row) {
        publish_row(lds_x, lane, xm[0], xh[0]);
        publish_row(lds_y, lane, ym[0], yh[0]);
        xm[0] = xm[1], xh[0] = xh[1], ym[0] = ym[1], yh[0] = yh[1];
        if (row + 2 < last_in) { // on its way while this row and the next are filtered
            request_row(st, row + 2, lane, loadx, &xm[1], &xh[1]);
            request_row(st, row + 2, lane, loady, &ym[1], &yh[1]);
        }
        // horizontal taps of this row (ssim.cu:121-213)
        const int c = lane + HALO;
        float sumX = 0.f, sumX2 = 0.f, sumY = 0.f, sumY2 = 0.f, sumXY = 0.f;
#pragma unroll
        for (int d = 1; d <= HALO; ++d) {
            const float w = cGauss[HALO - d];
            const float Xl = lds_x[c - d], Yl = lds_y[c - d];
            const float Xr = lds_x[c + d], Yr = lds_y[c + d];
            sumX += (Xl + Xr) * w;
            sumX2 += ((Xl * Xl) + (Xr * Xr)) * w;
            sumY += (Yl + Yr) * w;
            sumY2 += ((Yl * Yl) + (Yr * Yr)) * w;
            sumXY += ((Xl * Yl) + (Xr * Yr)) * w;
        }
        const float cX = lds_x[c], cY = lds_y[c];
        const float wc = cGauss[HALO];
        sumX += cX * wc;
        sumX2 += (cX * cX) * wc;
        sumY += cY * wc;
        sumY2 += (cY * cY) * wc;
        sumXY += (cX * cY) * wc;
        if (row >= st.row0 && row < row_end && col < st.W)
            l1 += gsx::fabs(cX - cY);
        const float moments[5] = {sumX, sumX2, sumY, sumY2, sumXY};
        push_window(win, moments);
        const int out_row = row - HALO; // the window now spans out_row - 5 .. out_row + 5
        if (out_row >= st.row0 && col < st.W) {
            float m[5];
            filter_window(win, m);
            // ssim.cu:215-274
            const float mu1 = m[0], mu2 = m[2];
            const float mu1_sq = mu1 * mu1, mu2_sq = mu2 * mu2;
            const float sigma1_sq = m[1] - mu1_sq, sigma2_sq = m[3] - mu2_sq;
            const float sigma12 = m[4] - mu1 * mu2;
            const float A = mu1_sq + mu2_sq + C1;
            const float B = sigma1_sq + sigma2_sq + C2;
            const float C_ = 2.f * mu1 * mu2 + C1;
            const float D_ = 2.f * sigma12 + C2;
            emit(out_row, col, (C_ * D_) / (A * B),
                 ((mu2 * 2.f * D_) / (A * B) - (mu2 * 2.f * C_) / (A * B) - (mu1 * 2.f * C_ * D_) / (A * A * B) +
                  (mu1 * 2.f * C_ * D_) / (A * B * B)),
                 (-C_ * D_) / (A * B * B), (2.f * C_) / (A * B));
        }
    }
    return l1;
}

// ---- backward ----------------------------------------------------------------------------------------------------
// chain(row, col, &d0, &d1, &d2): the three derivative maps times d loss / d map at an image pixel (ssim.cu:305-337);
// emit(row, col, s0, s1, s2): the three filtered sums of an output pixel (:385-421).
template <int ROWS, class Chain, class Emit>
__device__ __forceinline__ void ssim_backward_strip(const Strip& st, float* lds0, float* lds1, float* lds2,
                                                    const Chain& chain, const Emit& emit) {
    const int lane = threadIdx.x & 63;
    const int col = st.col0 + lane;
    const int row_end = min(st.row0 + ROWS, st.H);
    const int last_in = row_end + HALO;
    float win[3][11];
#pragma unroll
    for (int k = 0; k < 3; ++k)
#pragma unroll
        for (int j = 0; j < 11; ++j)
            win[k][j] = 0.f;
    auto request = [&](int row, float (&mv)[3], float (&hv)[3]) {
        const bool row_in = row >= 0 && row < st.H;
        const int cm = st.col0 - HALO + lane, ch = st.col0 + kStripCols - HALO + lane;
        mv[0] = mv[1] = mv[2] = hv[0] = hv[1] = hv[2] = 0.f;
        if (row_in && cm >= 0 && cm < st.W)
            chain(row, cm, &mv[0], &mv[1], &mv[2]);
        if (lane < 2 * HALO && row_in && ch < st.W)
            chain(row, ch, &hv[0], &hv[1], &hv[2]);
    };
    float mv[3], hv[3], mv2[3], hv2[3]; // the next row to publish and the one after it
    request(st.row0 - HALO, mv, hv);
    request(st.row0 - HALO + 1, mv2, hv2);
    for (int row = st.row0 - HALO; row < last_in; ++row) {
        publish_row(lds0, lane, mv[0], hv[0]);
        publish_row(lds1, lane, mv[1], hv[1]);
        publish_row(lds2, lane, mv[2], hv[2]);
#pragma unroll
        for (int k = 0; k < 3; ++k)
            mv[k] = mv2[k], hv[k] = hv2[k];
        if (row + 2 < last_in)
            request(row + 2, mv2, hv2);
        const int c = lane + HALO;
        float a0 = 0.f, a1 = 0.f, a2 = 0.f; // ssim.cu:339-383
#pragma unroll
        for (int d = 1; d <= HALO; ++d) {
            const float w = cGauss[HALO - d];
            a0 += (lds0[c - d] + lds0[c + d]) * w;
            a1 += (lds1[c - d] + lds1[c + d]) * w;
            a2 += (lds2[c - d] + lds2[c + d]) * w;
        }
        const float wc = cGauss[HALO];
        a0 += lds0[c] * wc;
        a1 += lds1[c] * wc;
        a2 += lds2[c] * wc;
        const float sums[3] = {a0, a1, a2};
        push_window(win, sums);
        const int out_row = row - HALO;
        if (out_row >= st.row0 && col < st.W) {
            float f[3];
            filter_window(win, f);
            emit(out_row, col, f[0], f[1], f[2]);
        }
    }
}

// the strip of wave `w` (over all waves of the launch): plane-major so that the planes of one strip are neighbours
__device__ __forceinline__ Strip strip_of(uint32_t w, int planes, int H, int W, int rows, int* plane) {
    const int strips_x = (W + kStripCols - 1) / kStripCols;
    *plane = (int)(w % (uint32_t)planes);
    const uint32_t s = w / (uint32_t)planes;
    Strip st;
    st.col0 = (int)(s % (uint32_t)strips_x) * kStripCols;
    st.row0 = (int)(s / (uint32_t)strips_x) * rows;
    st.H = H, st.W = W;
    return st;
}
__host__ __device__ static inline uint32_t strip_count(uint32_t H, uint32_t W, uint32_t rows) {
    return ((W + kStripCols - 1) / kStripCols) * ((H + rows - 1) / rows);
}

// gsplat-style operator (include/kernels/ssim.cuh:11-19): img1 / img2 [planes,H,W] -> map and the derivative maps
__global__ void __launch_bounds__(256) fusedssim_kernel(int planes, int H, int W, float C1, float C2,
                                                         const float* __restrict__ img1,
                                                         const float* __restrict__ img2, float* __restrict__ ssim_map,
                                                         float* __restrict__ dm_dmu1,
                                                         float* __restrict__ dm_dsigma1_sq,
                                                         float* __restrict__ dm_dsigma12) {
    __shared__ float rows[4][2 * kRowFloats];
    const uint32_t wave = threadIdx.x >> 6, w = blockIdx.x * 4u + wave;
    if (w >= strip_count(H, W, kFwdRows) * (uint32_t)planes)
        return;
    int plane;
    const Strip st = strip_of(w, planes, H, W, kFwdRows, &plane);
    const size_t base = (size_t)plane * H * W;
    ssim_forward_strip<kFwdRows>(
        st, C1, C2, rows[wave], [&](int y, int x) { return img1[base + (size_t)y * W + x]; },
        [&](int y, int x) { return img2[base + (size_t)y * W + x]; },
        [&](int y, int x, float ssim, float dmu1, float ds1, float ds12) {
            const size_t gi = base + (size_t)y * W + x;
            ssim_map[gi] = ssim;
            if (dm_dmu1) {
                dm_dmu1[gi] = dmu1;
                dm_dsigma1_sq[gi] = ds1;
                dm_dsigma12[gi] = ds12;
            }
        });
}

// include/kernels/ssim.cuh:21-28 -> d loss / d img1
__global__ void __launch_bounds__(256) fusedssim_backward_kernel(
    int planes, int H, int W, const float* __restrict__ img1, const float* __restrict__ img2,
    const float* __restrict__ dL_dmap, const float* __restrict__ dm_dmu1, const float* __restrict__ dm_dsigma1_sq,
    const float* __restrict__ dm_dsigma12, float* __restrict__ dL_dimg1) {
    __shared__ float rows[4][3][kRowFloats];
    const uint32_t wave = threadIdx.x >> 6, w = blockIdx.x * 4u + wave;
    if (w >= strip_count(H, W, kBwdRows) * (uint32_t)planes)
        return;
    int plane;
    const Strip st = strip_of(w, planes, H, W, kBwdRows, &plane);
    const size_t base = (size_t)plane * H * W;
    ssim_backward_strip<kBwdRows>(
        st, rows[wave][0], rows[wave][1], rows[wave][2],
        [&](int y, int x, float* d0, float* d1, float* d2) {
            const size_t gi = base + (size_t)y * W + x;
            const float ch = dL_dmap[gi];
            *d0 = dm_dmu1[gi] * ch;
            *d1 = dm_dsigma1_sq[gi] * ch;
            *d2 = dm_dsigma12[gi] * ch;
        },
        [&](int y, int x, float s0, float s1, float s2) {
            const size_t gi = base + (size_t)y * W + x;
            const float p1 = img1[gi], p2 = img2[gi];
            dL_dimg1[gi] = s0 + (2.f * p1) * s1 + (p2)*s2;
        });
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
// forward: clamp + HWC -> CHW on load, SSIM moments and derivative maps, and per wave the sums of |image - gt| and of
// the SSIM map over the valid crop (what image_from_render + fusedssim + ssim_valid_partials do in three passes; the
// clamped image and the SSIM map themselves are never written).
__global__ void __launch_bounds__(256) photometric_fwd_kernel(int H, int W, float C1, float C2,
                                                               const float* __restrict__ render_hwc,
                                                               const float* __restrict__ gt_chw,
                                                               float* __restrict__ dm_dmu1,
                                                               float* __restrict__ dm_dsigma1_sq,
                                                               float* __restrict__ dm_dsigma12,
                                                               float* __restrict__ l1_partials,
                                                               float* __restrict__ ssim_partials) {
    __shared__ float rows[4][2 * kRowFloats];
    const uint32_t wave = threadIdx.x >> 6, w = blockIdx.x * 4u + wave;
    if (w >= strip_count(H, W, kFwdRows) * 3u)
        return;
    int c;
    const Strip st = strip_of(w, 3, H, W, kFwdRows, &c);
    const size_t base = (size_t)c * H * W;
    const bool crop = H > 10 && W > 10;
    float ss = 0.f;
    float l1 = ssim_forward_strip<kFwdRows>(
        st, C1, C2, rows[wave],
        [&](int y, int x) { // rasterizer.cpp:205
            return gsx::fmin(gsx::fmax(render_hwc[((size_t)y * W + x) * 3 + c], 0.0f), 1.0f);
        },
        [&](int y, int x) { return gt_chw[base + (size_t)y * W + x]; },
        [&](int y, int x, float ssim, float dmu1, float ds1, float ds12) {
            const size_t gi = base + (size_t)y * W + x;
            if (!crop || (y >= 5 && y < H - 5 && x >= 5 && x < W - 5))
                ss += ssim;
            dm_dmu1[gi] = dmu1;
            dm_dsigma1_sq[gi] = ds1;
            dm_dsigma12[gi] = ds12;
        });
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        l1 += __shfl_xor(l1, m, 64);
        ss += __shfl_xor(ss, m, 64);
    }
    if ((threadIdx.x & 63u) == 0) {
        l1_partials[w] = l1;
        ssim_partials[w] = ss;
    }
}

// backward: d loss / d render in one pass - the SSIM chain with d loss / d map = -lambda / count inside the valid crop
// formed on the fly (fused_ssim.cuh:84-96), the L1 sign term, the clamp VJP and the CHW -> HWC permute (what
// fusedssim_backward + render_grad_from_loss do in two passes with two intermediate images).
__global__ void __launch_bounds__(256) photometric_bwd_kernel(int H, int W, float ssim_scale, float l1_scale,
                                                               const float* __restrict__ render_hwc,
                                                               const float* __restrict__ gt_chw,
                                                               const float* __restrict__ dm_dmu1,
                                                               const float* __restrict__ dm_dsigma1_sq,
                                                               const float* __restrict__ dm_dsigma12,
                                                               float* __restrict__ v_render_hwc) {
    __shared__ float rows[4][3][kRowFloats];
    const uint32_t wave = threadIdx.x >> 6, w = blockIdx.x * 4u + wave;
    if (w >= strip_count(H, W, kBwdRows) * 3u)
        return;
    int c;
    const Strip st = strip_of(w, 3, H, W, kBwdRows, &c);
    const size_t base = (size_t)c * H * W;
    const bool crop = H > 10 && W > 10;
    ssim_backward_strip<kBwdRows>(
        st, rows[wave][0], rows[wave][1], rows[wave][2],
        [&](int y, int x, float* d0, float* d1, float* d2) {
            const bool valid = !crop || (y >= 5 && y < H - 5 && x >= 5 && x < W - 5);
            const float ch = valid ? ssim_scale : 0.f;
            const size_t gi = base + (size_t)y * W + x;
            *d0 = dm_dmu1[gi] * ch;
            *d1 = dm_dsigma1_sq[gi] * ch;
            *d2 = dm_dsigma12[gi] * ch;
        },
        [&](int y, int x, float s0, float s1, float s2) {
            const size_t p = (size_t)y * W + x;
            const float r = render_hwc[p * 3 + c];
            const float p1 = gsx::fmin(gsx::fmax(r, 0.0f), 1.0f), p2 = gt_chw[base + p];
            const float dssim = s0 + (2.f * p1) * s1 + (p2)*s2;
            const float d = p1 - p2;
            const float sgn = d > 0.f ? 1.f : (d < 0.f ? -1.f : 0.f);
            const float gg = l1_scale * sgn + dssim;
            v_render_hwc[p * 3 + c] = (r >= 0.f && r <= 1.f) ? gg : 0.f; // clamp VJP
        });
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
    GSX_REQUIRE((int64_t)B * CH * strip_count((uint32_t)H, (uint32_t)W, kBwdRows) < (1ll << 31),
                GSX_ERR_INVALID_ARGUMENT, "fusedssim: B*CH*H*W too large");
    const uint32_t waves = strip_count((uint32_t)H, (uint32_t)W, kFwdRows) * (uint32_t)(B * CH);
    hipLaunchKernelGGL(fusedssim_kernel, dim3(cdiv(waves, 4)), dim3(256), 0, (hipStream_t)stream, B * CH, H, W, C1, C2,
                       img1, img2, ssim_map, dm_dmu1, dm_dsigma1_sq, dm_dsigma12);
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
    GSX_REQUIRE((int64_t)B * CH * strip_count((uint32_t)H, (uint32_t)W, kBwdRows) < (1ll << 31),
                GSX_ERR_INVALID_ARGUMENT, "fusedssim_backward: B*CH*H*W too large");
    const uint32_t waves = strip_count((uint32_t)H, (uint32_t)W, kBwdRows) * (uint32_t)(B * CH);
    hipLaunchKernelGGL(fusedssim_backward_kernel, dim3(cdiv(waves, 4)), dim3(256), 0, (hipStream_t)stream, B * CH, H,
                       W, img1, img2, dL_dmap, dm_dmu1, dm_dsigma1_sq, dm_dsigma12, dL_dimg1);
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
    return 3u * strip_count(H, W, kFwdRows); // one pair of sums per wave
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
    hipLaunchKernelGGL(photometric_fwd_kernel, dim3(cdiv(3u * strip_count(H, W, kFwdRows), 4)), dim3(256),
                       0, (hipStream_t)stream, (int)H, (int)W, C1, C2,
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
    hipLaunchKernelGGL(photometric_bwd_kernel, dim3(cdiv(3u * strip_count(H, W, kBwdRows), 4)), dim3(256),
                       0, (hipStream_t)stream, (int)H, (int)W, ssim_scale,
                       l1_scale, render_hwc, gt_chw, dm_dmu1, dm_dsigma1_sq, dm_dsigma12, v_render_hwc);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}
