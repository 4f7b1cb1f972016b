/* gsx_debug.h - test and measurement hooks of libgsx.so (C ABI).  NOT part of what a LichtFeld build binds: nothing
 * here has a counterpart in the reference; the tests and bench.py use these entry points to compare device
 * arithmetic with a host build, to calibrate byte counters and to count the pairs a rasterizer launch works on. */
#ifndef GSX_DEBUG_H
#define GSX_DEBUG_H

#include "gsx.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Test hook (no counterpart in the reference): evaluates one of the shared fp32 math primitives element-wise on the
 * device so that a test can compare it bit for bit with a host build.  which: 0 exp, 1 log, 2 rsqrt, 3 sin, 4 acos,
 * 5 sigmoid, 6 saturating float->u32, 7 pow(x, x2), 8 x / x2, 9 sqrt, 10 fma(x, x2, x), 11 exp restricted to
 * -87 <= x <= 0 (the rasterizers' variant; must equal 0 on that range), 12 the hardware reciprocal with one Newton
 * step (the gradient chains' 1 / (1 - alpha)), 13 the bare hardware reciprocal, 15 min_limit(x2, x) (the
 * rasterizers' clamp of alpha: x2 a number, x anything including NaN). */
GSX_API int gsx_debug_math(int which, uint32_t n, const float* x, const float* x2, float* y, void* stream);
/* Measurement hook (no counterpart in the reference): a plain device-to-device copy kernel of `bytes` bytes (a
 * multiple of 16), the known-size yardstick for HBM byte counters and achieved-bandwidth figures. */
GSX_API int gsx_debug_copy(const void* src, void* dst, size_t bytes, void* stream);
/* Test hook: the 64-lane wave reductions of the backward rasterizers, for `values` = 16, 13 (the 3DGUT backward) or 9
 * (the fastgs backward) sums at a time.  in [n_waves,64,values] -> out [n_waves,values]. */
GSX_API int gsx_debug_wave_reduce(uint32_t values, uint32_t n_waves, const float* in, float* out, void* stream);

/* Test hook: how many empty reads a chained look-back (the one-launch radix passes, gsx_tile_lists) waits for a
 * predecessor before it gives up; limit < 0 restores the default (65 536, about a tenth of a second).  With 0 every
 * look-back that meets an empty word gives up at once: the give-up path (bit 1 of the error word, positions that stay
 * inside the buffers, every kernel ending normally) can be exercised without making anything wait.  Process-wide. */
GSX_API int gsx_debug_set_lookback_spin_limit(int64_t limit);

/* Tuning hook: output rows per strip of the SSIM / photometric-loss kernels (0 = chosen per image size).  The buffer
 * sizes gsx_photometric_partials reports follow it: set it before anything is sized.  Process-wide. */
GSX_API void gsx_debug_set_ssim_strip_rows(int rows);

/* Pair counts of one forward pass, for turning kernel times into rates (no counterpart in the reference).
 * stats_out: device uint64[8] = {(pixel, Gaussian) pairs the forward evaluates, pairs composited, pairs the backward
 * walks, (wave, Gaussian) iterations executed, (wave, Gaussian) iterations removed by the pixel bounds, executed
 * iterations with a contributing pixel, 2 reserved};
 * the counts are ADDED to it, so zero it first. */
GSX_API int gsx_rasterize_pair_stats(int64_t n_isects, const void* records, uint32_t image_width,
                                     uint32_t image_height, const float* viewmat, const float* K,
                                     const int32_t* tile_offsets, const int32_t* flatten_ids,
                                     unsigned long long* stats_out, void* stream);

/* Pair counts of one backward pass (the kernel of gsx_rasterize_bwd_accumulate with counters in place of the
 * derivative chain; n_isects may be GSX_COUNT_IN_OFFSETS).  stats_out: device uint64[4] = {(pixel, Gaussian) pairs
 * whose alpha the kernel evaluates (pixels of executed (wave, Gaussian) iterations that lie at or in front of their
 * last contributor), valid pairs (alpha >= 1/255: the pairs that receive a gradient), (wave, Gaussian) iterations
 * executed, reserved}; the counts are ADDED to it, so zero it first. */
GSX_API int gsx_rasterize_bwd_pair_stats(int64_t n_isects, const void* records, uint32_t image_width,
                                         uint32_t image_height, const float* viewmat, const float* K,
                                         const int32_t* tile_offsets, const int32_t* flatten_ids,
                                         const float* render_alphas, const int32_t* last_ids,
                                         unsigned long long* stats_out, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* GSX_DEBUG_H */
