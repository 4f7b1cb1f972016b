// ssim.hip - separable 11x11 SSIM forward / backward as column strips streamed through registers, and the per-pixel
// parts of the photometric loss around it.  What is computed: src/training/kernels/ssim.cu:16-27 (window), :64-276
// (forward), :284-424 (backward); src/training/trainer.cpp:126-129, include/kernels/fused_ssim.cuh:59-67,84-96,117-122
// (valid crop, mean), src/training/rasterization/rasterizer.cpp:205 (clamp).
//
// Organisation (gfx950).  A wave owns a strip of one image plane: 64 adjacent columns (one per lane) by r output
// rows, and walks it top to bottom, one INPUT row per step (r + 10 steps; r is chosen per image so that the launch
// fills the CUs evenly, see strip_rows - 17 at 1237 x 822, three workgroups on every CU):
//   * the row's 64 + 10 values per image go through two wave-private LDS rows, from which every lane reads its
//     eleven horizontal taps with unit stride across the lanes (no bank conflicts, no workgroup barrier: the four
//     waves of a workgroup never talk to each other);
//   * the horizontally filtered moments of the last eleven input rows stay in REGISTERS (a sliding window per lane);
//     once the window is full every further input row completes one output row - the vertical filter reads no
//     memory at all.  The row loop is unrolled eleven times, after which every window slot is back in the register
//     it started in: the window slides without a single move (the steps left over after the last full block of
//     eleven run as a nest of conditions that the walk leaves where it ends);
//   * input rows are requested from memory two steps before they are used, by unconditional loads whose results
//     nothing touches until then.
// A strip re-reads 10 halo rows per r and 10 halo columns per 64; the three colour planes of the interleaved render
// are three waves of one workgroup, and the workgroups of one XCD cover one contiguous eighth of the image, so these
// re-reads are served by that XCD's L2.
// Each output applies the taps in the reference's order (symmetric pairs from the centre outwards, then the centre;
// rows after columns), every accumulation one fused multiply-add, and forms the seven quotients of a pixel as
// products with the two IEEE reciprocals 1/A and 1/B (the reference is built with fast-math: its own quotients are
// reciprocal products and its sums contracted).  Results do not depend on the strip geometry and equal the CPU
// checker's, which fixes the same evaluation, to the last bit.
#include "gsx_common.h"
#include "gsx_tiles.h"

namespace gsx {

static constexpr int HALO = 5;
static constexpr int kStripCols = 64;  // one per lane
// Output rows per strip are chosen per launch (strip_rows): a strip of r rows costs r + 10 steps, so taller strips
// waste less on the halo, while the launch should fill every CU evenly and still leave each SIMD a few waves to hide
// latencies behind.
static constexpr int kMinRows = 12, kMaxRows = 56;
static constexpr int kRowFloats = kStripCols + 2 * HALO + 6; // an LDS row, padded to 80 floats

__constant__ float cGauss[11] = {0.001028380123898387f, 0.0075987582094967365f, 0.036000773310661316f,
                                 0.10936068743467331f,  0.21300552785396576f,   0.26601171493530273f,
                                 0.21300552785396576f,  0.10936068743467331f,   0.036000773310661316f,
                                 0.0075987582094967365f, 0.001028380123898387f};

// where a strip lies
struct Strip {
    int col0, row0; // first output column / row
    int H, W;
    int rows;       // output rows of the strip
};

// The 74 columns an input row contributes to a strip: one value per lane for the columns col0 - 5 + lane and, in the
// lanes below 10, a second one for the columns col0 + 59 + lane.  A request is a pair of UNCONDITIONAL loads from
// addresses clamped into the image, and what it returns is not touched until the row is published two steps later:
// no branch and no arithmetic stands between a load and its wait, so the wait lands where the value is needed
// (a conditional load, or one whose result is clamped or scaled at once, waits for the memory on the spot).
struct RowSlot {
    int row_c, col_m, col_h; // clamped row, clamped columns of the two values
};
__device__ __forceinline__ RowSlot row_slot(const Strip& st, int row, int lane) {
    RowSlot r;
    r.row_c = min(max(row, 0), st.H - 1);
    r.col_m = min(max(st.col0 - HALO + lane, 0), st.W - 1);
    r.col_h = min(st.col0 + kStripCols - HALO + min(lane, 2 * HALO - 1), st.W - 1);
    return r;
}
// whether the two values of a row lie inside the image (else they count as 0)
__device__ __forceinline__ void row_valid(const Strip& st, int row, int lane, bool* main_ok, bool* halo_ok) {
    const bool row_in = row >= 0 && row < st.H;
    const int cm = st.col0 - HALO + lane, ch = st.col0 + kStripCols - HALO + lane;
    *main_ok = row_in && cm >= 0 && cm < st.W;
    *halo_ok = row_in && ch < st.W;
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
            out[k] = fma(win[k][HALO - d] + win[k][HALO + d], w, out[k]);
    }
#pragma unroll
    for (int k = 0; k < N; ++k)
        out[k] = fma(win[k][HALO], cGauss[HALO], out[k]);
}

// One step of the sliding window.  Written as moves; inside the eleven-fold unrolled row loop they are renamings.
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

// The row walk of a strip: `steps` calls of step(0), step(1), ...  Eleven at a time as straight-line code, after which
// the window is back in the registers it started in (a step's shift of the window is a renaming there).  What is left
// over (fewer than eleven steps) runs as a nest of conditions, each step inside the one before: the walk leaves from
// wherever it ends and never rejoins, so no path has to move the window into place for another.
template <int J, class Step>
__device__ __forceinline__ void walk_tail(int it0, int left, const Step& step) {
    if constexpr (J < 10) {
        if (J < left) {
            step(it0 + J);
            walk_tail<J + 1>(it0, left, step);
        }
    }
}
template <class Step>
__device__ __forceinline__ void walk_rows(int steps, const Step& step) {
    int it0 = 0;
    for (; it0 + 11 <= steps; it0 += 11) {
#pragma unroll
        for (int j = 0; j < 11; ++j)
            step(it0 + j);
    }
    walk_tail<0>(it0, steps - it0, step);
}

// ---- forward -----------------------------------------------------------------------------------------------------
// loadx / loady: loaders of the two images for this plane, (row, column) -> the value in memory; prepx: what turns a
// loaded X value into the image value (the clamp of the training path).  Per output pixel `emit(row, col, ssim,
// dmu1, dsigma1_sq, dsigma12)` is called (image pixels only); returns the lane's sum of |X - Y| over its output pixels.
// lds: two rows of kRowFloats (X and Y of the current input row).
template <class LoadX, class PrepX, class LoadY, class Emit>
__device__ __forceinline__ float ssim_forward_strip(const Strip& st, float C1, float C2, float* lds,
                                                    const LoadX& loadx, const PrepX& prepx, const LoadY& loady,
                                                    const Emit& emit) {
    const int lane = threadIdx.x & 63;
    const int col = st.col0 + lane;
    const int row_end = min(st.row0 + st.rows, st.H); // one past the last output row
    float* lds_x = lds;
    float* lds_y = lds + kRowFloats;
    float win[5][11];
#pragma unroll
    for (int k = 0; k < 5; ++k)
#pragma unroll
        for (int j = 0; j < 11; ++j)
            win[k][j] = 0.f;
    float l1 = 0.f;
    float xm[2], xh[2], ym[2], yh[2]; // raw values; [0]: the next row to publish, [1]: the one after it
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const RowSlot q = row_slot(st, st.row0 - HALO + k, lane);
        xm[k] = loadx(q.row_c, q.col_m), xh[k] = loadx(q.row_c, q.col_h);
        ym[k] = loady(q.row_c, q.col_m), yh[k] = loady(q.row_c, q.col_h);
    }
    const int steps = st.rows + 2 * HALO;
    auto step = [&](int it) __attribute__((always_inline)) {
        const int row = st.row0 - HALO + it;
        bool main_ok, halo_ok;
        row_valid(st, row, lane, &main_ok, &halo_ok);
        publish_row(lds_x, lane, main_ok ? prepx(xm[0]) : 0.0f, halo_ok ? prepx(xh[0]) : 0.0f);
        publish_row(lds_y, lane, main_ok ? ym[0] : 0.0f, halo_ok ? yh[0] : 0.0f);
        xm[0] = xm[1], xh[0] = xh[1], ym[0] = ym[1], yh[0] = yh[1];
        { // the row after the next: on its way while this row and the next are filtered
            const RowSlot q = row_slot(st, row + 2, lane);
            xm[1] = loadx(q.row_c, q.col_m), xh[1] = loadx(q.row_c, q.col_h);
            ym[1] = loady(q.row_c, q.col_m), yh[1] = loady(q.row_c, q.col_h);
        }
        // horizontal taps of this row (ssim.cu:121-213)
        const int c = lane + HALO;
        float sumX = 0.f, sumX2 = 0.f, sumY = 0.f, sumY2 = 0.f, sumXY = 0.f;
#pragma unroll
        for (int d = 1; d <= HALO; ++d) {
            const float w = cGauss[HALO - d];
            const float Xl = lds_x[c - d], Yl = lds_y[c - d];
            const float Xr = lds_x[c + d], Yr = lds_y[c + d];
            sumX = fma(Xl + Xr, w, sumX);
            sumX2 = fma(fma(Xl, Xl, Xr * Xr), w, sumX2);
            sumY = fma(Yl + Yr, w, sumY);
            sumY2 = fma(fma(Yl, Yl, Yr * Yr), w, sumY2);
            sumXY = fma(fma(Xl, Yl, Xr * Yr), w, sumXY);
        }
        const float cX = lds_x[c], cY = lds_y[c];
        const float wc = cGauss[HALO];
        sumX = fma(cX, wc, sumX);
        sumX2 = fma(cX * cX, wc, sumX2);
        sumY = fma(cY, wc, sumY);
        sumY2 = fma(cY * cY, wc, sumY2);
        sumXY = fma(cX * cY, wc, sumXY);
        if (row >= st.row0 && row < row_end && col < st.W)
            l1 += gsx::fabs(cX - cY);
        const float moments[5] = {sumX, sumX2, sumY, sumY2, sumXY};
        push_window(win, moments);
        const int out_row = row - HALO; // the window now spans out_row - 5 .. out_row + 5
        if (out_row >= st.row0 && out_row < row_end && col < st.W) {
            float m[5];
            filter_window(win, m);
            // ssim.cu:215-274; the seven quotients of a pixel as products with 1/A and 1/B
            const float mu1 = m[0], mu2 = m[2];
            const float sigma1_sq = fma(-mu1, mu1, m[1]), sigma2_sq = fma(-mu2, mu2, m[3]);
            const float sigma12 = fma(-mu1, mu2, m[4]);
            const float A = fma(mu1, mu1, fma(mu2, mu2, C1));
            const float B = (sigma1_sq + sigma2_sq) + C2;
            const float two_mu1 = mu1 + mu1;
            const float C_ = fma(two_mu1, mu2, C1);
            const float D_ = fma(2.f, sigma12, C2);
            const float rA = 1.0f / A, rB = 1.0f / B;
            const float r = rA * rB, rrB = r * rB;
            const float CD = C_ * D_;
            // d map / d mu1 = 2 mu2 (D - C) / (A B) + 2 mu1 C D (1 / (A B B) - 1 / (A A B))
            emit(out_row, col, CD * r, fma(two_mu1 * CD, rrB - r * rA, ((mu2 + mu2) * (D_ - C_)) * r), -(CD * rrB),
                 (C_ + C_) * r);
        }
    };
    walk_rows(steps, step);
    return l1;
}

// ---- backward ----------------------------------------------------------------------------------------------------
// load4(row, col, v[4]): the three derivative maps at an image pixel as they lie in memory, and a fourth word for
// the factor; factor(row, col, v[3]): d loss / d map there (ssim.cu:305-337 multiplies the two); emit(row, col, s0,
// s1, s2): the three filtered sums of an output pixel (:385-421).
template <class Load4, class Factor, class Emit>
__device__ __forceinline__ void ssim_backward_strip(const Strip& st, float* lds0, float* lds1, float* lds2,
                                                    const Load4& load4, const Factor& factor, const Emit& emit) {
    const int lane = threadIdx.x & 63;
    const int col = st.col0 + lane;
    const int row_end = min(st.row0 + st.rows, st.H);
    float win[3][11];
#pragma unroll
    for (int k = 0; k < 3; ++k)
#pragma unroll
        for (int j = 0; j < 11; ++j)
            win[k][j] = 0.f;
    // raw values of the three derivative maps (+ one more word the factor may need); the factor d loss / d map is
    // applied when a row is published
    auto request = [&](int row, float (&mv)[4], float (&hv)[4]) {
        const RowSlot q = row_slot(st, row, lane);
        load4(q.row_c, q.col_m, mv);
        load4(q.row_c, q.col_h, hv);
    };
    float mv[4], hv[4], mv2[4], hv2[4]; // the next row to publish and the one after it
    request(st.row0 - HALO, mv, hv);
    request(st.row0 - HALO + 1, mv2, hv2);
    const int steps = st.rows + 2 * HALO;
    auto step = [&](int it) __attribute__((always_inline)) {
        const int row = st.row0 - HALO + it;
        bool main_ok, halo_ok;
        row_valid(st, row, lane, &main_ok, &halo_ok);
        const float fm = main_ok ? factor(row, st.col0 - HALO + lane, mv[3]) : 0.0f;
        const float fh = halo_ok ? factor(row, st.col0 + kStripCols - HALO + lane, hv[3]) : 0.0f;
        publish_row(lds0, lane, main_ok ? mv[0] * fm : 0.0f, halo_ok ? hv[0] * fh : 0.0f);
        publish_row(lds1, lane, main_ok ? mv[1] * fm : 0.0f, halo_ok ? hv[1] * fh : 0.0f);
        publish_row(lds2, lane, main_ok ? mv[2] * fm : 0.0f, halo_ok ? hv[2] * fh : 0.0f);
#pragma unroll
        for (int k = 0; k < 4; ++k)
            mv[k] = mv2[k], hv[k] = hv2[k];
        request(row + 2, mv2, hv2);
        const int c = lane + HALO;
        float a0 = 0.f, a1 = 0.f, a2 = 0.f; // ssim.cu:339-383
#pragma unroll
        for (int d = 1; d <= HALO; ++d) {
            const float w = cGauss[HALO - d];
            a0 = fma(lds0[c - d] + lds0[c + d], w, a0);
            a1 = fma(lds1[c - d] + lds1[c + d], w, a1);
            a2 = fma(lds2[c - d] + lds2[c + d], w, a2);
        }
        const float wc = cGauss[HALO];
        a0 = fma(lds0[c], wc, a0);
        a1 = fma(lds1[c], wc, a1);
        a2 = fma(lds2[c], wc, a2);
        const float sums[3] = {a0, a1, a2};
        push_window(win, sums);
        const int out_row = row - HALO;
        if (out_row >= st.row0 && out_row < row_end && col < st.W) {
            float f[3];
            filter_window(win, f);
            emit(out_row, col, f[0], f[1], f[2]);
        }
    };
    walk_rows(steps, step);
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
    st.rows = rows;
    return st;
}
__host__ __device__ static inline uint32_t strip_count(uint32_t H, uint32_t W, uint32_t rows) {
    return ((W + kStripCols - 1) / kStripCols) * ((H + rows - 1) / rows);
}

// Workgroups are handed to the eight XCDs in turn (workgroup b runs on XCD b % 8, each with an L2 of its own).  A
// launch of xcd_grid(n) workgroups gives workgroup b the strips of logical index xcd_block(b, n), so that every XCD
// works through one contiguous eighth of the image: strips that share halo rows and cache lines meet in one L2
// instead of fetching them from memory once per XCD.
__host__ __device__ static inline uint32_t xcd_grid(uint32_t n) { return 8u * ((n + 7u) / 8u); }
__device__ __forceinline__ uint32_t xcd_block(uint32_t b, uint32_t n) { return (b & 7u) * ((n + 7u) / 8u) + (b >> 3); }

// gsplat-style operator (include/kernels/ssim.cuh:11-19): img1 / img2 [planes,H,W] -> map and the derivative maps
__global__ void __launch_bounds__(256) fusedssim_kernel(int rows_per_strip, int planes, int H, int W, float C1, float C2,
                                                         const float* __restrict__ img1,
                                                         const float* __restrict__ img2, float* __restrict__ ssim_map,
                                                         float* __restrict__ dm_dmu1,
                                                         float* __restrict__ dm_dsigma1_sq,
                                                         float* __restrict__ dm_dsigma12) {
    __shared__ float rows[4][2 * kRowFloats];
    const uint32_t n_waves = strip_count(H, W, rows_per_strip) * (uint32_t)planes;
    const uint32_t wave = threadIdx.x >> 6, w = xcd_block(blockIdx.x, (n_waves + 3u) / 4u) * 4u + wave;
    if (w >= n_waves)
        return;
    int plane;
    const Strip st = strip_of(w, planes, H, W, rows_per_strip, &plane);
    const size_t base = (size_t)plane * H * W;
    ssim_forward_strip(
        st, C1, C2, rows[wave], [&](int y, int x) { return img1[base + (size_t)y * W + x]; },
        [](float v) { return v; }, [&](int y, int x) { return img2[base + (size_t)y * W + x]; },
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
    int rows_per_strip, int planes, int H, int W, const float* __restrict__ img1, const float* __restrict__ img2,
    const float* __restrict__ dL_dmap, const float* __restrict__ dm_dmu1, const float* __restrict__ dm_dsigma1_sq,
    const float* __restrict__ dm_dsigma12, float* __restrict__ dL_dimg1) {
    __shared__ float rows[4][3][kRowFloats];
    const uint32_t n_waves = strip_count(H, W, rows_per_strip) * (uint32_t)planes;
    const uint32_t wave = threadIdx.x >> 6, w = xcd_block(blockIdx.x, (n_waves + 3u) / 4u) * 4u + wave;
    if (w >= n_waves)
        return;
    int plane;
    const Strip st = strip_of(w, planes, H, W, rows_per_strip, &plane);
    const size_t base = (size_t)plane * H * W;
    ssim_backward_strip(
        st, rows[wave][0], rows[wave][1], rows[wave][2],
        [&](int y, int x, float (&v)[4]) {
            const size_t gi = base + (size_t)y * W + x;
            v[0] = dm_dmu1[gi], v[1] = dm_dsigma1_sq[gi], v[2] = dm_dsigma12[gi], v[3] = dL_dmap[gi];
        },
        [](int, int, float chain) { return chain; },
        [&](int y, int x, float s0, float s1, float s2) {
            const size_t gi = base + (size_t)y * W + x;
            const float p1 = img1[gi], p2 = img2[gi];
            dL_dimg1[gi] = fma(p2, s2, fma(p1 + p1, s1, s0));
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

// the whole loss from the partial sums, by one workgroup of 256 lanes (contains barriers)
__device__ __forceinline__ void loss_from_partials(uint32_t CH, uint32_t H, uint32_t W, float lambda_dssim,
                                                   const float* __restrict__ l1_partials,
                                                   const float* __restrict__ ssim_partials, uint32_t n_partials,
                                                   float* __restrict__ loss_out, float* lds) {
    float a = 0.f, b = 0.f;
    // four independent loads in flight per lane: one workgroup, pure latency
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

__global__ void __launch_bounds__(256) photometric_loss_finish_kernel(uint32_t CH, uint32_t H, uint32_t W,
                                                                       float lambda_dssim,
                                                                       const float* __restrict__ l1_partials,
                                                                       const float* __restrict__ ssim_partials,
                                                                       uint32_t n_partials,
                                                                       float* __restrict__ loss_out) {
    __shared__ float lds[4];
    loss_from_partials(CH, H, W, lambda_dssim, l1_partials, ssim_partials, n_partials, loss_out, lds);
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
__global__ void __launch_bounds__(256) photometric_fwd_kernel(int rows_per_strip, int H, int W, float C1, float C2,
                                                               const float* __restrict__ render_hwc,
                                                               const float* __restrict__ gt_chw,
                                                               float* __restrict__ dm_dmu1,
                                                               float* __restrict__ dm_dsigma1_sq,
                                                               float* __restrict__ dm_dsigma12,
                                                               float* __restrict__ l1_partials,
                                                               float* __restrict__ ssim_partials) {
    __shared__ float rows[4][2 * kRowFloats];
    const uint32_t n_waves = strip_count(H, W, rows_per_strip) * 3u;
    const uint32_t wave = threadIdx.x >> 6, w = xcd_block(blockIdx.x, (n_waves + 3u) / 4u) * 4u + wave;
    if (w >= n_waves)
        return;
    int c;
    const Strip st = strip_of(w, 3, H, W, rows_per_strip, &c);
    const size_t base = (size_t)c * H * W;
    const bool crop = H > 10 && W > 10;
    float ss = 0.f;
    float l1 = ssim_forward_strip(
        st, C1, C2, rows[wave],
        [&](int y, int x) { return render_hwc[((size_t)y * W + x) * 3 + c]; },
        [](float v) { return gsx::fmin(gsx::fmax(v, 0.0f), 1.0f); }, // rasterizer.cpp:205
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
__global__ void __launch_bounds__(256) photometric_bwd_kernel(int rows_per_strip, int H, int W, float ssim_scale,
                                                               float l1_scale,
                                                               const float* __restrict__ render_hwc,
                                                               const float* __restrict__ gt_chw,
                                                               const float* __restrict__ dm_dmu1,
                                                               const float* __restrict__ dm_dsigma1_sq,
                                                               const float* __restrict__ dm_dsigma12,
                                                               float* __restrict__ v_render_hwc,
                                                               float lambda_dssim,
                                                               const float* __restrict__ l1_partials,
                                                               const float* __restrict__ ssim_partials,
                                                               uint32_t n_partials, float* __restrict__ loss_out,
                                                               uint32_t n_tiles,
                                                               const uint32_t* __restrict__ tile_cost,
                                                               uint32_t* __restrict__ tile_order) {
    if (tile_order != nullptr && blockIdx.x == gridDim.x - 1u) {
        // one workgroup more than the image needs: it sorts the tiles by what they cost the forward rasterizer, for
        // the backward rasterizer that follows this launch (no launch, stream or event of its own)
        __shared__ uint32_t cursor[kLenClasses];
        __shared__ uint32_t wave_total[16];
        tile_order_block<256>(n_tiles, kCountInOffsets, nullptr, tile_cost, tile_order, cursor, wave_total);
        return;
    }
    __shared__ float rows[4][3][kRowFloats];
    if (loss_out != nullptr && blockIdx.x == 0) {
        // the loss value itself, which only gets reported: the forward kernel's partial sums are complete when this
        // launch starts, so its first workgroup adds them up on the way (no launch and no stream of its own)
        __shared__ float lds[4];
        loss_from_partials(3u, (uint32_t)H, (uint32_t)W, lambda_dssim, l1_partials, ssim_partials, n_partials,
                           loss_out, lds);
    }
    const uint32_t n_waves = strip_count(H, W, rows_per_strip) * 3u;
    const uint32_t wave = threadIdx.x >> 6, w = xcd_block(blockIdx.x, (n_waves + 3u) / 4u) * 4u + wave;
    if (w >= n_waves)
        return;
    int c;
    const Strip st = strip_of(w, 3, H, W, rows_per_strip, &c);
    const size_t base = (size_t)c * H * W;
    const bool crop = H > 10 && W > 10;
    ssim_backward_strip(
        st, rows[wave][0], rows[wave][1], rows[wave][2],
        [&](int y, int x, float (&v)[4]) {
            const size_t gi = base + (size_t)y * W + x;
            v[0] = dm_dmu1[gi], v[1] = dm_dsigma1_sq[gi], v[2] = dm_dsigma12[gi], v[3] = 0.f;
        },
        [&](int y, int x, float) {
            const bool valid = !crop || (y >= 5 && y < H - 5 && x >= 5 && x < W - 5);
            return valid ? ssim_scale : 0.f;
        },
        [&](int y, int x, float s0, float s1, float s2) {
            const size_t p = (size_t)y * W + x;
            const float r = render_hwc[p * 3 + c];
            const float p1 = gsx::fmin(gsx::fmax(r, 0.0f), 1.0f), p2 = gt_chw[base + p];
            const float dssim = fma(p2, s2, fma(p1 + p1, s1, s0));
            const float d = p1 - p2;
            const float sgn = d > 0.f ? 1.f : (d < 0.f ? -1.f : 0.f);
            const float gg = l1_scale * sgn + dssim;
            v_render_hwc[p * 3 + c] = (r >= 0.f && r <= 1.f) ? gg : 0.f; // clamp VJP
        });
}

} // namespace gsx

using namespace gsx;

// Output rows per strip for an image of `planes` planes: the launch takes ceil(workgroups / CUs) rounds of r + 10
// steps each on its fullest CU; among the heights that leave every CU at least three workgroups (three waves per
// SIMD to hide latencies behind - below that the walk runs at the speed of its LDS and memory round trips) the
// cheapest wins, the lowest on a tie.  Small images take the lowest strips.
static int g_strip_rows = 0;
extern "C" void gsx_debug_set_ssim_strip_rows(int rows) { g_strip_rows = rows; }
static int strip_rows(uint32_t H, uint32_t W, uint32_t planes) {
    if (g_strip_rows >= 1)
        return g_strip_rows;
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        cus = n;
    }
    int best = kMinRows;
    uint64_t best_cost = ~0ull;
    for (int r = kMinRows; r <= kMaxRows; ++r) {
        const uint64_t wgs = ((uint64_t)strip_count(H, W, (uint32_t)r) * planes + 3) / 4;
        const uint64_t per_cu = (wgs + (uint64_t)cus - 1) / (uint64_t)cus;
        if (per_cu < 3 && r > kMinRows)
            break; // taller strips only thin the launch further
        const uint64_t cost = per_cu * (uint64_t)(r + 2 * HALO);
        if (cost < best_cost)
            best_cost = cost, best = r;
    }
    return best;
}

extern "C" int gsx_fusedssim(int B, int CH, int H, int W, float C1, float C2, const float* img1, const float* img2,
                             float* ssim_map, float* dm_dmu1, float* dm_dsigma1_sq, float* dm_dsigma12,
                             void* stream) {
    if (B <= 0 || CH <= 0 || H <= 0 || W <= 0)
        return GSX_OK;
    GSX_REQUIRE(img1 && img2 && ssim_map, GSX_ERR_INVALID_ARGUMENT, "fusedssim: null tensor");
    const bool train = dm_dmu1 != nullptr;
    GSX_REQUIRE(train == (dm_dsigma1_sq != nullptr) && train == (dm_dsigma12 != nullptr), GSX_ERR_INVALID_ARGUMENT,
                "fusedssim: the three derivative maps must be given together");
    GSX_REQUIRE((int64_t)B * CH * strip_count((uint32_t)H, (uint32_t)W, kMinRows) < (1ll << 31),
                GSX_ERR_INVALID_ARGUMENT, "fusedssim: B*CH*H*W too large");
    const int rows = strip_rows((uint32_t)H, (uint32_t)W, (uint32_t)(B * CH));
    const uint32_t waves = strip_count((uint32_t)H, (uint32_t)W, (uint32_t)rows) * (uint32_t)(B * CH);
    hipLaunchKernelGGL(fusedssim_kernel, dim3(xcd_grid(cdiv(waves, 4))), dim3(256), 0, (hipStream_t)stream, rows, B * CH, H, W, C1, C2,
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
    GSX_REQUIRE((int64_t)B * CH * strip_count((uint32_t)H, (uint32_t)W, kMinRows) < (1ll << 31),
                GSX_ERR_INVALID_ARGUMENT, "fusedssim_backward: B*CH*H*W too large");
    const int rows = strip_rows((uint32_t)H, (uint32_t)W, (uint32_t)(B * CH));
    const uint32_t waves = strip_count((uint32_t)H, (uint32_t)W, (uint32_t)rows) * (uint32_t)(B * CH);
    hipLaunchKernelGGL(fusedssim_backward_kernel, dim3(xcd_grid(cdiv(waves, 4))), dim3(256), 0, (hipStream_t)stream, rows, B * CH, H,
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
    return 3u * strip_count(H, W, (uint32_t)strip_rows(H, W, 3)); // one pair of sums per wave
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
    const int rows = strip_rows(H, W, 3);
    hipLaunchKernelGGL(photometric_fwd_kernel, dim3(xcd_grid(cdiv(3u * strip_count(H, W, (uint32_t)rows), 4))),
                       dim3(256), 0, (hipStream_t)stream, rows, (int)H, (int)W, C1, C2,
                       render_hwc, gt_chw, dm_dmu1, dm_dsigma1_sq, dm_dsigma12, l1_partials, ssim_partials);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

static int photometric_backward(uint32_t H, uint32_t W, float lambda_dssim, const float* render_hwc,
                                const float* gt_chw, const float* dm_dmu1, const float* dm_dsigma1_sq,
                                const float* dm_dsigma12, float* v_render_hwc, const float* l1_partials,
                                const float* ssim_partials, float* loss_out, uint32_t n_tiles,
                                const uint32_t* tile_cost, uint32_t* tile_order, void* stream) {
    if ((uint64_t)H * W == 0)
        return GSX_OK;
    GSX_REQUIRE(render_hwc && gt_chw && dm_dmu1 && dm_dsigma1_sq && dm_dsigma12 && v_render_hwc,
                GSX_ERR_INVALID_ARGUMENT, "photometric_loss_backward: null tensor");
    GSX_REQUIRE(loss_out == nullptr || (l1_partials && ssim_partials), GSX_ERR_INVALID_ARGUMENT,
                "photometric_loss_backward: the loss needs the forward pass's partial sums");
    const bool crop = H > 10 && W > 10;
    const float count = crop ? 3.f * (float)(H - 10) * (float)(W - 10) : 3.f * (float)H * (float)W;
    const float ssim_scale = -lambda_dssim / count;
    const float l1_scale = (1.f - lambda_dssim) / (3.f * (float)H * (float)W);
    const int rows = strip_rows(H, W, 3);
    // (the strips' workgroups find their place from their own index and the strip count, not from the grid size)
    const uint32_t blocks = xcd_grid(cdiv(3u * strip_count(H, W, (uint32_t)rows), 4)) + (tile_order ? 1u : 0u);
    hipLaunchKernelGGL(photometric_bwd_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, rows, (int)H, (int)W,
                       ssim_scale, l1_scale, render_hwc, gt_chw, dm_dmu1, dm_dsigma1_sq, dm_dsigma12, v_render_hwc,
                       lambda_dssim, l1_partials, ssim_partials, gsx_photometric_partials(H, W), loss_out, n_tiles,
                       tile_cost, tile_order);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_photometric_loss_backward(uint32_t H, uint32_t W, float lambda_dssim, const float* render_hwc,
                                             const float* gt_chw, const float* dm_dmu1, const float* dm_dsigma1_sq,
                                             const float* dm_dsigma12, float* v_render_hwc, void* stream) {
    return photometric_backward(H, W, lambda_dssim, render_hwc, gt_chw, dm_dmu1, dm_dsigma1_sq, dm_dsigma12,
                                v_render_hwc, nullptr, nullptr, nullptr, 0, nullptr, nullptr, stream);
}

extern "C" int gsx_photometric_loss_backward_finish(uint32_t H, uint32_t W, float lambda_dssim,
                                                    const float* render_hwc, const float* gt_chw,
                                                    const float* dm_dmu1, const float* dm_dsigma1_sq,
                                                    const float* dm_dsigma12, const float* l1_partials,
                                                    const float* ssim_partials, float* loss_out,
                                                    float* v_render_hwc, void* stream) {
    GSX_REQUIRE(loss_out != nullptr, GSX_ERR_INVALID_ARGUMENT, "photometric_loss_backward_finish: loss_out is null");
    return photometric_backward(H, W, lambda_dssim, render_hwc, gt_chw, dm_dmu1, dm_dsigma1_sq, dm_dsigma12,
                                v_render_hwc, l1_partials, ssim_partials, loss_out, 0, nullptr, nullptr, stream);
}

extern "C" int gsx_photometric_loss_backward_order(uint32_t H, uint32_t W, float lambda_dssim,
                                                   const float* render_hwc, const float* gt_chw,
                                                   const float* dm_dmu1, const float* dm_dsigma1_sq,
                                                   const float* dm_dsigma12, const float* l1_partials,
                                                   const float* ssim_partials, float* loss_out,
                                                   float* v_render_hwc, uint32_t tile_width, uint32_t tile_height,
                                                   const uint32_t* tile_cost, uint32_t* tile_order, void* stream) {
    const uint64_t n_tiles = (uint64_t)tile_width * tile_height;
    GSX_REQUIRE(n_tiles > 0 && n_tiles < (1ull << 31), GSX_ERR_INVALID_ARGUMENT,
                "photometric_loss_backward_order: %u x %u tiles", tile_width, tile_height);
    GSX_REQUIRE(tile_cost && tile_order, GSX_ERR_INVALID_ARGUMENT, "photometric_loss_backward_order: null tile tensor");
    if ((uint64_t)H * W == 0) // no image, no launch to ride on
        return gsx_tile_order(GSX_COUNT_IN_OFFSETS, nullptr, tile_cost, tile_width, tile_height, tile_order, stream);
    return photometric_backward(H, W, lambda_dssim, render_hwc, gt_chw, dm_dmu1, dm_dsigma1_sq, dm_dsigma12,
                                v_render_hwc, l1_partials, ssim_partials, loss_out, (uint32_t)n_tiles, tile_cost,
                                tile_order, stream);
}
