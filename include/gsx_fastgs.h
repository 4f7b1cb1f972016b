/* gsx_fastgs.h - C ABI of the "fastgs" (Jacobian-EWA) rasterization backend, the reference's default training
 * rasterizer: what fast_gs::rasterization::forward_wrapper / backward_wrapper bind
 * (src/training/fastgs/rasterization/include/rasterization_api.h:25-75; src/rasterization_api.cu:16-181), called from
 * FastGSRasterize::{forward,backward} (src/training/rasterization/fast_rasterizer_autograd.cpp:9-163) and
 * fast_rasterize (src/training/rasterization/fast_rasterizer.cpp:12-66).
 *
 * Conventions as in gsx.h (raw device pointers, caller-provided state / workspaces with *_bytes queries, a stream,
 * 0 or a negative gsx_status).  w2c [4,4] row-major and cam_position [3] are HOST pointers (the reference keeps them
 * in device tensors and reads 15 floats per lane).  Inputs are the raw parameters: means [N,3], log-scales [N,3],
 * un-normalised quaternions wxyz [N,4], logit opacities [N], sh0 [N,1,3], shN [N,B,3].
 *
 * The forward is split where the reference synchronises to read its counters (src/forward.cu:99-101):
 *   gsx_fastgs_preprocess  -> per-primitive state + the number of instances (through pinned host memory; wait = 0
 *                             returns at once and the caller synchronises on its own event)
 *   gsx_fastgs_render      -> instance list, tile ranges, image [3,H,W], alpha [1,H,W], per-pixel state
 *   gsx_fastgs_backward    -> blend backward + preprocess backward
 * The state buffers replace the reference's four opaque byte blobs (per primitive / tile / instance / bucket); no
 * per-bucket checkpoints exist here.  Gaussians of equal depth bits are ordered by index (the reference's order among
 * them depends on its atomic compaction). */
#ifndef GSX_FASTGS_H
#define GSX_FASTGS_H
#include "gsx.h"

#ifdef __cplusplus
extern "C" {
#endif

/* FastGSSettings (rasterization_api.h:12-23) without the tensors, plus shN's coefficient count B */
typedef struct gsx_fastgs_settings {
    uint32_t active_sh_bases;      /* (degree + 1)^2: 1, 4, 9 or 16 */
    uint32_t total_bases_sh_rest;  /* B = sh_coefficients_rest.size(1) */
    uint32_t width, height;
    float fx, fy, cx, cy, near_plane, far_plane;
} gsx_fastgs_settings;

GSX_API size_t gsx_fastgs_primitive_state_bytes(uint32_t N);
GSX_API size_t gsx_fastgs_instance_state_bytes(int64_t n_instances, uint32_t width, uint32_t height);
GSX_API size_t gsx_fastgs_pixel_state_bytes(uint32_t width, uint32_t height);
GSX_API size_t gsx_fastgs_accum_bytes(uint32_t N); /* backward accumulator: zeroed once by the caller, left zeroed */

/* preprocess_cu + depth ordering + offsets (kernels_forward.cuh:17-218; src/forward.cu:60-123).  At most 65536
 * tiles, as the reference's u16 tile keys (GSX_ERR_UNSUPPORTED beyond). */
GSX_API int gsx_fastgs_preprocess(uint32_t N, const float* means, const float* scales_raw, const float* rotations_raw,
                                  const float* opacities_raw, const float* sh_coefficients_0,
                                  const float* sh_coefficients_rest, const float* w2c_host,
                                  const float* cam_position_host, const gsx_fastgs_settings* settings,
                                  void* primitive_state, size_t primitive_state_bytes, int64_t* n_instances_host,
                                  int wait, void* stream);
/* create_instances_cu, tile sort, instance ranges, blend_cu (kernels_forward.cuh:220-459; src/forward.cu:125-196).
 * background (nullable, 3 floats on the device): image += (1 - alpha) * background as fast_rasterizer.cpp:63 does
 * after the kernel.  pixel_state receives per pixel the final transmittance and the number of list entries the
 * backward replays, and per tile how far its pixels went into the list plus the tile order the backward visits
 * (dearest tiles first, so that its launch ends with cheap tiles). */
GSX_API int gsx_fastgs_render(uint32_t N, const gsx_fastgs_settings* settings, const void* primitive_state,
                              size_t primitive_state_bytes, int64_t n_instances, void* instance_state,
                              size_t instance_state_bytes, const float* background, float* image, float* alpha,
                              void* pixel_state, size_t pixel_state_bytes, void* stream);
/* where gsx_fastgs_preprocess left the per-primitive records ([N,12] floats: mean2d 2, conic 3, opacity, colour 3
 * (not clamped), footprint box half-widths 2, depth; unspecified for culled primitives) and the number of tiles each
 * primitive contributes to (0 = culled) inside primitive_state (device pointers; for inspection and tests) */
GSX_API int gsx_fastgs_primitive_records(uint32_t N, const void* primitive_state, const float** records,
                                         const uint32_t** n_touched_tiles);
/* where gsx_fastgs_render left the sorted instance list (primitive index per instance) and the first instance of
 * every tile inside instance_state (device pointers; for inspection and tests) */
GSX_API int gsx_fastgs_instance_list(const gsx_fastgs_settings* settings, int64_t n_instances,
                                     const void* instance_state, const int32_t** instance_primitive,
                                     const int32_t** tile_offsets);
/* blend_backward_cu + preprocess_backward_cu (kernels_backward.cuh:17-449; src/backward.cu:14-116).  Every output
 * is fully written (zeros for culled primitives; the reference zero-fills them first).  background: the one given
 * to gsx_fastgs_render (its gradient path through alpha is included).  The three state buffers are checked against
 * the sizes N, n_instances and the image size require (GSX_ERR_WORKSPACE).  grad_w2c (nullable, 16 floats on the device):
 * rows 0-2 as kernels_backward.cuh:177-190.  densification_info (nullable, [2,N]): += as :233-236. */
GSX_API int gsx_fastgs_backward(uint32_t N, const float* means, const float* scales_raw, const float* rotations_raw,
                                const float* sh_coefficients_rest, const float* w2c_host,
                                const float* cam_position_host, const gsx_fastgs_settings* settings,
                                const void* primitive_state, size_t primitive_state_bytes, int64_t n_instances,
                                const void* instance_state, size_t instance_state_bytes, const void* pixel_state,
                                size_t pixel_state_bytes, const float* background, const float* grad_image,
                                const float* grad_alpha, void* accum, size_t accum_bytes, float* grad_means,
                                float* grad_scales_raw, float* grad_rotations_raw, float* grad_opacities_raw,
                                float* grad_sh_coefficients_0, float* grad_sh_coefficients_rest, float* grad_w2c,
                                float* densification_info, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* GSX_FASTGS_H */
