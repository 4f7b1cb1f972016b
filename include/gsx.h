/* gsx.h - C ABI of libgsx.so: hand-written gfx950 (MI355X) kernels for the 3D-Gaussian-splatting
 * training step that sits behind LichtFeld-Studio's gsplat/Ops.h.
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer unless its name ends in _host.  Tensors are contiguous, fp32
 *    unless stated, laid out exactly as the reference's at::Tensor arguments (row-major).
 *  - `stream` is a hipStream_t passed as void* (NULL = the null stream).  No entry point allocates,
 *    frees or synchronises, except gsx_intersect_tile_count (returns a value to the host) and the
 *    functions documented as "convenience" which say so.
 *  - Scratch memory comes from the caller: <op>_workspace_bytes() says how much, and the same
 *    (workspace, workspace_bytes) pair is handed to the op.  Workspaces need 256-byte alignment.
 *  - Return value: GSX_OK or a negative gsx_status.  gsx_last_error() gives a thread-local message.
 *  - Optional pointers may be NULL where the comment says "nullable".
 *  - C = 1 camera; global or rolling shutter (gsx_shutter_type; viewmats1 = the end-of-frame pose, nullable = the
 *    start pose); camera models GSX_PINHOLE (radial [6], tangential [2], thin prism [4]
 *    coefficients, each nullable; LichtFeld's trainer uses the perfect pinhole: rasterizer.cpp:33-35,
 *    rasterizer_autograd.cpp:59-60), GSX_FISHEYE (radial [4], nullable) and GSX_EQUIRECTANGULAR.  Other values
 *    return GSX_ERR_UNSUPPORTED.  backgrounds, where given, is [C, channels] of the colours being blended.
 *
 * All file:line citations are relative to the LichtFeld-Studio tree.
 */
#ifndef GSX_H
#define GSX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(GSX_BUILD)
#define GSX_API __attribute__((visibility("default")))
#else
#define GSX_API
#endif

typedef enum gsx_status {
    GSX_OK = 0,
    GSX_ERR_INVALID_ARGUMENT = -1, /* null pointer, bad size, bad enum */
    GSX_ERR_UNSUPPORTED = -2,      /* C > 1, orthographic camera, CDIM not built */
    GSX_ERR_WORKSPACE = -3,        /* workspace too small or misaligned */
    GSX_ERR_HIP = -4,              /* a HIP runtime call failed (message has the HIP error) */
    GSX_ERR_OVERFLOW = -5          /* n_isects does not fit the int32 index space */
} gsx_status;

/* gsplat/Common.h:46-51 */
typedef enum gsx_camera_model { GSX_PINHOLE = 0, GSX_ORTHO = 1, GSX_FISHEYE = 2, GSX_EQUIRECTANGULAR = 3 } gsx_camera_model;
/* gsplat/Cameras.h:16-22 */
typedef enum gsx_shutter_type {
    GSX_ROLLING_TOP_TO_BOTTOM = 0,
    GSX_ROLLING_LEFT_TO_RIGHT = 1,
    GSX_ROLLING_BOTTOM_TO_TOP = 2,
    GSX_ROLLING_RIGHT_TO_LEFT = 3,
    GSX_GLOBAL = 4
} gsx_shutter_type;
/* gsplat/Cameras.h:27-44 UnscentedTransformParameters (same defaults when zero-initialised via gsx_ut_defaults) */
typedef struct gsx_ut_params {
    float alpha, beta, kappa, in_image_margin_factor;
    int32_t require_all_sigma_points_valid;
} gsx_ut_params;

GSX_API int gsx_version(void);
GSX_API const char* gsx_last_error(void);
GSX_API const char* gsx_status_string(int status);
GSX_API gsx_ut_params gsx_ut_defaults(void);
/* ---- a1: gsplat::projection_ut_3dgs_fused (Ops.h:69-98; kernel ProjectionUT3DGSFused.cu:17-210) ----
 * means [N,3] quats [N,4] (wxyz) scales [N,3] opacities [N] nullable, viewmats0 [C,4,4], Ks [C,3,3]
 * -> radii i32 [C,N,2], means2d [C,N,2], depths [C,N], conics [C,N,3], compensations [C,N] nullable.
 * radial_coeffs [C,6] (GSX_PINHOLE) or [C,4] (GSX_FISHEYE), tangential_coeffs [C,2], thin_prism_coeffs [C,4], each
 * nullable; rs_type: gsx_shutter_type (a rolling shutter iterates every sigma point's projection, Cameras.cuh:346-414).
 * Rows of culled Gaussians (radii 0) are left untouched in means2d/depths/conics/compensations. */
GSX_API int gsx_projection_ut_3dgs_fused(
    uint32_t C, uint32_t N, const float* means, const float* quats, const float* scales, const float* opacities,
    const float* viewmats0, const float* viewmats1 /*[C,4,4] end-of-frame pose, nullable*/, const float* Ks,
    uint32_t image_width, uint32_t image_height, float eps2d, float near_plane, float far_plane, float radius_clip, int camera_model,
    gsx_ut_params ut, int rs_type, const float* radial_coeffs, const float* tangential_coeffs,
    const float* thin_prism_coeffs, int32_t* radii, float* means2d, float* depths, float* conics,
    float* compensations, void* stream);

/* ---- a3: gsplat::spherical_harmonics_fwd / _bwd (Ops.h:12-25; SphericalHarmonicsCUDA.cu:373-529) ----
 * dirs [N,3], coeffs [N,K,3], masks u8/bool [N] nullable -> colors [N,3] (masked rows untouched).
 * bwd: v_coeffs [N,K,3] is fully written (zero for masked rows and unused bands); v_dirs [N,3] nullable
 * (degree <= 3 when requested). */
GSX_API int gsx_spherical_harmonics_fwd(uint32_t N, uint32_t K, uint32_t degrees_to_use, const float* dirs,
                                        const float* coeffs, const uint8_t* masks, float* colors, void* stream);
GSX_API int gsx_spherical_harmonics_bwd(uint32_t N, uint32_t K, uint32_t degrees_to_use, const float* dirs,
                                        const float* coeffs, const uint8_t* masks, const float* v_colors,
                                        float* v_coeffs, float* v_dirs, void* stream);

/* ---- a4: gsplat::intersect_tile (Ops.h:28-38; Intersect.cpp:15-122; IntersectTile.cu:23-114) ----
 * Two calls, as the reference's two passes: count (+ inclusive scan; blocks until the total is on the
 * host, like Intersect.cpp:76) then emit.  cum_tiles_per_gauss is i64 [C*N]. */
GSX_API size_t gsx_intersect_tile_count_workspace_bytes(uint32_t C, uint32_t N);
GSX_API int gsx_intersect_tile_count(uint32_t C, uint32_t N, const float* means2d, const int32_t* radii,
                                     uint32_t tile_size, uint32_t tile_width, uint32_t tile_height,
                                     int32_t* tiles_per_gauss, int64_t* cum_tiles_per_gauss, void* workspace,
                                     size_t workspace_bytes, int64_t* n_isects_host, void* stream);
/* The depth-ordered count (one camera): order[i] = index of the Gaussian with the i-th smallest depth bit pattern
 * (ties by index; Gaussians that touch no tile last), cum_tiles_per_gauss = prefix sum of the tile counts over
 * POSITIONS in that order (tiles_per_gauss stays indexed by Gaussian).  Emitting with this order leaves the pairs
 * sorted by (depth bits, Gaussian index), so the sorted list the reference obtains from one radix sort on all
 * 32 + tile + camera bits (Intersect.cpp:104-113) is reached by sorting on the tile / camera bits alone
 * (gsx_radix_sort_pairs with begin_bit = 32): the sort is stable, the result is the same array bit for bit, and
 * four of its six passes run over N Gaussians instead of n_isects pairs.
 * wait != 0: returns with *n_isects_host valid (and checked against the int32 index space), like the call above.
 * wait == 0: nothing blocks; n_isects_host must be PINNED host memory (the scan's last workgroup stores the total
 * into it directly; memory the runtime does not know as pinned gets an asynchronous copy instead).  It reads -1
 * from the return of this call until the total has arrived (0 at once when N == 0): the caller synchronises with
 * the stream or simply watches the slot, checks the value is below 2^31, and may queue work that does not need the
 * count in between. */
GSX_API size_t gsx_intersect_tile_count_ordered_workspace_bytes(uint32_t N);
GSX_API int gsx_intersect_tile_count_ordered(uint32_t N, const float* means2d, const int32_t* radii,
                                             const float* depths, uint32_t tile_size, uint32_t tile_width,
                                             uint32_t tile_height, int32_t* order, int32_t* tiles_per_gauss,
                                             int64_t* cum_tiles_per_gauss, void* workspace, size_t workspace_bytes,
                                             int64_t* n_isects_host, int wait, void* stream);
/* order: nullable (i32 [N], C == 1): emit position by position in that order, cum_tiles_per_gauss by position */
GSX_API int gsx_intersect_tile_emit(uint32_t C, uint32_t N, const float* means2d, const int32_t* radii,
                                    const float* depths, const int64_t* cum_tiles_per_gauss, const int32_t* order,
                                    uint32_t tile_size, uint32_t tile_width, uint32_t tile_height, int64_t* isect_ids,
                                    int32_t* flatten_ids, void* stream);
/* Packed rows (means2d [nnz,2], radii [nnz,2], depths [nnz], camera_ids i64 [nnz] with values in [0, C);
 * Intersect.cpp:32-39, IntersectTile.cu:50, 86-94): count with gsx_intersect_tile_count(1, nnz, ...) - a row's tile
 * count does not depend on its camera -, then emit with this call; flatten_ids index the packed rows.  gaussian_ids
 * are not needed here (the reference's kernel does not read them either). */
GSX_API int gsx_intersect_tile_emit_packed(uint32_t C, uint32_t nnz, const float* means2d, const int32_t* radii,
                                           const float* depths, const int64_t* camera_ids,
                                           const int64_t* cum_tiles_per_gauss, uint32_t tile_size,
                                           uint32_t tile_width, uint32_t tile_height, int64_t* isect_ids,
                                           int32_t* flatten_ids, void* stream);
/* The same with the writes bounded to the first `capacity` entries: lets a caller that reuses its buffers emit
 * while the total is still on its way to the host, and repeat the call only if the total exceeded the buffers. */
GSX_API int gsx_intersect_tile_emit_capped(uint32_t C, uint32_t N, const float* means2d, const int32_t* radii,
                                           const float* depths, const int64_t* cum_tiles_per_gauss,
                                           const int32_t* order, uint32_t tile_size, uint32_t tile_width,
                                           uint32_t tile_height, int64_t capacity, int64_t* isect_ids,
                                           int32_t* flatten_ids, void* stream);
/* The emission after gsx_intersect_tile_count_ordered, given that call's workspace (unchanged since): for tile grids
 * up to 255 x 255 the sorted depth keys in it carry every Gaussian's tile rectangle, so positions are emitted from
 * sequential reads of (key, order, cum) alone - nothing is gathered in sorted order; larger grids take the path of
 * gsx_intersect_tile_emit_capped.  Same outputs either way; capacity as above (INT64_MAX = unbounded). */
GSX_API int gsx_intersect_tile_emit_ordered(uint32_t N, const float* means2d, const int32_t* radii,
                                            const float* depths, const int64_t* cum_tiles_per_gauss,
                                            const int32_t* order, const void* ordered_workspace, uint32_t tile_size,
                                            uint32_t tile_width, uint32_t tile_height, int64_t capacity,
                                            int64_t* isect_ids, int32_t* flatten_ids, void* stream);
/* Intersect.cpp:46-47: floor(log2(n)) + 1 */
GSX_API uint32_t gsx_n_bits(uint32_t n);

/* ---- a5: gsplat::radix_sort_double_buffer (Intersect.h:39-46; IntersectTile.cu:290-328) ----
 * Stable ascending LSD radix sort of (i64 key, i32 value) pairs on key bits [begin_bit, end_bit) (the reference
 * passes begin_bit = 0).  Buffers 0 (keys0/vals0, the input) and 1 (keys1/vals1) are ping-ponged; *selector_host
 * (host int) says which pair holds the result (like cub::DoubleBuffer::selector).  The workspace needs no particular
 * contents on entry; from 2 M pairs on, the sort is a fill of its bookkeeping words, one count of the digits of
 * every pass and one launch per 8-bit pass, below that three launches per pass (same result either way).
 * The one-launch passes chain their workgroups by a look-back whose every wait is bounded (about a tenth of a second):
 * should a wait run out - a GPU so over-subscribed that a workgroup's predecessor does not get to run - the pass ends
 * normally, every position it writes stays inside the buffers, bit 1 of an error word inside the workspace is set and
 * the result is NOT sorted.  gsx_radix_sort_pairs_error gives that word's device address (NULL for sizes that take the
 * three-launch passes, which cannot fail this way); each call clears it first.  A caller that cannot rule the
 * condition out reads the word (4 bytes) after the sort and sorts again if it is not zero. */
GSX_API size_t gsx_radix_sort_pairs_workspace_bytes(int64_t n);
/* key_bytes: 8 (gsx_radix_sort_pairs) or 2 (gsx_radix_sort_tile_pairs) */
GSX_API uint32_t* gsx_radix_sort_pairs_error(int64_t n, uint32_t key_bytes, void* workspace);
/* the selector gsx_radix_sort_pairs will report for this size and bit range (known before the sort runs) */
GSX_API int gsx_radix_sort_pairs_selector(int64_t n, uint32_t begin_bit, uint32_t end_bit);
GSX_API int gsx_radix_sort_pairs(int64_t n, int64_t* keys0, int32_t* vals0, int64_t* keys1, int32_t* vals1,
                                 uint32_t begin_bit, uint32_t end_bit, void* workspace, size_t workspace_bytes,
                                 int* selector_host, void* stream);
/* The same sort for callers that cannot allocate device memory and so cannot bring a workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference (its sort takes
 * its temporary storage from the caching allocator, IntersectTile.cu:305-327).  The histogram table lives in an
 * array built into the library: 4 MiB + 1.25 KiB of device memory on every GPU the library runs on, held until the
 * process ends.  n > GSX_RADIX_SORT_STATIC_MAX_PAIRS returns GSX_ERR_WORKSPACE.  The call allocates and frees
 * nothing and does not synchronise; its first use on a device looks the array's address up once (make that call
 * outside a capture).  All calls on one GPU share the one array: calls that overlap on a GPU (two streams, two
 * threads) race - serialise them.  Nothing in the array has to start at zero, so no clearing is queued. */
#define GSX_RADIX_SORT_STATIC_MAX_PAIRS (1ll << 24)
GSX_API int gsx_radix_sort_pairs_static(int64_t n, int64_t* keys0, int32_t* vals0, int64_t* keys1, int32_t* vals1,
                                        uint32_t begin_bit, uint32_t end_bit, int* selector_host, void* stream);

/* ---- a6: gsplat::intersect_offset (Ops.h:39-43; IntersectTile.cu:206-286) -> offsets i32 [C,Th,Tw] ---- */
GSX_API int gsx_intersect_offset(int64_t n_isects, const int64_t* isect_ids, uint32_t C, uint32_t tile_width,
                                 uint32_t tile_height, int32_t* offsets, void* stream);

/* ---- a4-a6 for a caller that only wants the per-tile lists (one camera, grids up to 255 x 255) ----
 * After gsx_intersect_tile_count_ordered the pairs leave in depth order, so the sort only ever looks at their tile
 * bits and the ranges only at the tile index: the key of a pair can be its 16-bit tile index alone (the reference's
 * other backend sorts u16 tile keys the same way, src/training/fastgs/rasterization/src/forward.cu:141-147).
 * tile_keys u16 [n_isects] + flatten_ids i32 [n_isects] -> sorted on bits [0, n_bits) -> offsets i32 [Th,Tw].
 * flatten_ids and offsets equal, element for element, what gsx_intersect_tile_emit_ordered +
 * gsx_radix_sort_pairs(32, 32 + n_bits) + gsx_intersect_offset produce; a pass moves 6 instead of 12 bytes a pair.
 * gsx_intersect_tile_pairs_fit: 1 when the grid is within the limit (else GSX_ERR_UNSUPPORTED from the emission);
 * the sort's workspace is gsx_radix_sort_pairs_workspace_bytes(n). */
GSX_API int gsx_intersect_tile_pairs_fit(uint32_t tile_width, uint32_t tile_height);
GSX_API int gsx_intersect_tile_emit_pairs(uint32_t N, const int64_t* cum_tiles_per_gauss, const int32_t* order,
                                          const void* ordered_workspace, uint32_t tile_size, uint32_t tile_width,
                                          uint32_t tile_height, int64_t capacity, uint16_t* tile_keys,
                                          int32_t* flatten_ids, void* stream);
GSX_API int gsx_radix_sort_tile_pairs(int64_t n, uint16_t* keys0, int32_t* vals0, uint16_t* keys1, int32_t* vals1,
                                      uint32_t n_bits, void* workspace, size_t workspace_bytes, int* selector_host,
                                      void* stream);
GSX_API int gsx_intersect_tile_pairs_offset(int64_t n_isects, const uint16_t* tile_keys, uint32_t tile_width,
                                            uint32_t tile_height, int32_t* offsets, void* stream);

/* ---- a4-a6 as one call whose pair count never crosses to the host (one camera, grids up to 255 x 255) ----
 * No single counterpart in the reference: this is intersect_tile + radix_sort_double_buffer + intersect_offset
 * (Intersect.cpp:41-137, IntersectTile.cu:23-114, 206-252, 290-328) for the caller that only feeds the rasterizers,
 * without the `.item()` of Intersect.cpp:76.  Nine launches: depth keys (+ byte histograms), four one-launch radix
 * passes over the depth keys of the Gaussians that touch a tile, the tile table (+1 / -1 at every rectangle's corners
 * and a 2-D prefix sum give every list's length, hence tile_offsets and the count, before a pair exists), the
 * emission of one (super-tile, rectangle, id) entry per super-tile a Gaussian meets (the grid is cut into at most 256
 * super-tiles), one one-launch radix pass that groups the entries by super-tile, and a gather that writes every
 * tile's list front to back from its super-tile's entries - no (tile, id) pair is sorted.  The one-launch passes and
 * the gather chain their workgroups by a bounded look-back over per-workgroup counts.
 *   means2d [N,2], radii [N,2], depths [N] as the projection leaves them; 16-byte aligned
 *   flatten_ids  i32 [capacity]            out: element for element the flatten_ids of the separate operators
 *   tile_offsets i32 [Th * Tw + 1]         out: the operators' tile_offsets, and the pair count in the last entry
 *   n_isects_host_slot                     nullable; pinned host memory (hipHostMalloc): receives the pair count
 *                                          with one 8-byte store from the device (write -1 there first to see it land)
 * Consumers take the count from the device: pass n_isects = GSX_COUNT_IN_OFFSETS to gsx_tile_order,
 * gsx_rasterize_records_fwd and gsx_rasterize_bwd_accumulate together with this tile_offsets.
 * If the pairs exceed `capacity` (or 2^30 - 1) every list is left empty (tile_offsets all zero), bit 0 of the error
 * word is set and the true count is still reported: grow the buffers and run the step again.  Nothing is read or
 * written out of bounds in that case.  Bit 1 of the error word: a look-back's bounded wait ran out (results invalid).
 * side_stream: nullable; a second stream of the same device (default priority) on which the tile table is formed
 * while the depth sort runs on `stream` (forked and joined with events inside the call; all results are ordered on
 * `stream` when the call returns).
 * The workspace's head must be zeroed once by gsx_tile_lists_init; every call leaves it ready for the next one.  Calls
 * that share a workspace must not overlap, and host threads that call with the same `stream` must take turns: the
 * events that fork and join the two streams are kept per device and `stream`. */
#define GSX_COUNT_IN_OFFSETS (-1ll)
GSX_API size_t gsx_tile_lists_workspace_bytes(uint32_t N, int64_t capacity, uint32_t tile_width,
                                              uint32_t tile_height);
GSX_API int gsx_tile_lists_init(uint32_t N, int64_t capacity, uint32_t tile_width, uint32_t tile_height,
                                void* workspace, size_t workspace_bytes, void* stream);
GSX_API int gsx_tile_lists(uint32_t N, const float* means2d, const int32_t* radii, const float* depths,
                           uint32_t tile_size, uint32_t tile_width, uint32_t tile_height, int64_t capacity,
                           void* workspace, size_t workspace_bytes, int32_t* flatten_ids, int32_t* tile_offsets,
                           int64_t* n_isects_host_slot, void* stream, void* side_stream);
/* device addresses inside the workspace: counts i64 [2] = {pairs in the lists (0 if they did not fit), pairs there
 * are}; error u32 (bits above; sticky until the caller clears it or calls gsx_tile_lists_init) */
GSX_API const int64_t* gsx_tile_lists_counts(uint32_t N, int64_t capacity, uint32_t tile_width,
                                             uint32_t tile_height, const void* workspace);
GSX_API uint32_t* gsx_tile_lists_error(uint32_t N, int64_t capacity, uint32_t tile_width, uint32_t tile_height,
                                       void* workspace);

/* ---- a7: gsplat::rasterize_to_pixels_from_world_3dgs_fwd (Ops.h:100-129; ...3DGSFwd.cu:19-285) ----
 * colors [C,N,channels] (channels in {1,2,3,4,5,8,9,16,17,32,33,64,65,128,129,256,257,512,513}, the counts of
 * Rasterization.cpp:106-128; any other GSX_ERR_UNSUPPORTED; beyond 32 the rasterizers run once per 32 channels),
 * opacities [C,N], backgrounds [C,channels] nullable,
 * masks u8 [C,Th,Tw] nullable, tile_offsets i32 [C,Th,Tw], flatten_ids i32 [n_isects]
 * -> render_colors [C,H,W,channels], render_alphas [C,H,W,1], last_ids i32 [C,H,W]. tile_size must be 16.
 *
 * The rasterizers read one 96-byte RECORD per Gaussian (whitening matrix diag(1/s) R^T, camera centre in whitened
 * coordinates, opacity, first three colour channels, exact pixel bounds of alpha >= 1/255) instead of the five
 * parameter tensors: gsx_pack_raster_records builds them for one camera, gsx_rasterize_records_fwd renders from
 * them.  The whole-operator entry point does both and needs gsx_raster_records_bytes(N) of workspace. */
GSX_API size_t gsx_raster_records_bytes(uint32_t N);
GSX_API int gsx_pack_raster_records(uint32_t N, const float* means, const float* quats, const float* scales,
                                    const float* opacities, const float* colors, uint32_t channels,
                                    const float* viewmat, const float* K, uint32_t image_width,
                                    uint32_t image_height, void* records, void* stream);
/* The order in which the rasterizers visit the tiles (no counterpart in the reference): tile ids, dearest first, so
 * that the cheap tiles fill the end of a launch instead of a few dear ones running on alone.  A tile's cost is
 * tile_cost[tile] (u32, e.g. the tile_walk a forward pass left), or with tile_cost == NULL the length of its list in
 * tile_offsets.  tile_order: u32 [tile_width * tile_height]; no result depends on it (the order inside one of the
 * logarithmic cost classes is unspecified). */
GSX_API int gsx_tile_order(int64_t n_isects, const int32_t* tile_offsets, const uint32_t* tile_cost,
                           uint32_t tile_width, uint32_t tile_height, uint32_t* tile_order, void* stream);
/* The whole-operator rasterizer entry points (gsx_rasterize_to_pixels_from_world_3dgs_fwd / _bwd) order their tiles
 * themselves when the workspace they are given is this much larger than their own requirement: the forward by list
 * length, the backward by the cost read from render_alphas / last_ids. */
GSX_API size_t gsx_tile_order_bytes(uint32_t tile_width, uint32_t tile_height);
/* colors is only read for channels beyond the third (channels > 3); nullable otherwise.  tile_order: nullable (tiles
 * in index order), else any permutation of the tile ids (gsx_tile_order).  tile_walk: nullable, u32 [tiles]: receives
 * per tile how far its pixels went into the list (entries up to the last contributor, 0 = none) - what the tile cost
 * this pass and will cost the backward pass. */
GSX_API int gsx_rasterize_records_fwd(int64_t n_isects, const void* records, const float* colors, uint32_t channels,
                                      const float* backgrounds, const uint8_t* masks, uint32_t image_width,
                                      uint32_t image_height, const float* viewmat, const float* K,
                                      const int32_t* tile_offsets, const int32_t* flatten_ids,
                                      const uint32_t* tile_order, uint32_t* tile_walk, float* render_colors,
                                      float* render_alphas, int32_t* last_ids, void* stream);
GSX_API int gsx_rasterize_to_pixels_from_world_3dgs_fwd(
    uint32_t C, uint32_t N, int64_t n_isects, const float* means, const float* quats, const float* scales,
    const float* colors, uint32_t channels, const float* opacities, const float* backgrounds, const uint8_t* masks,
    uint32_t image_width, uint32_t image_height, uint32_t tile_size, const float* viewmats0,
    const float* viewmats1 /*[C,4,4] end-of-frame pose, nullable*/, const float* Ks, int camera_model, gsx_ut_params ut, int rs_type,
    const float* radial_coeffs, const float* tangential_coeffs, const float* thin_prism_coeffs,
    const int32_t* tile_offsets, const int32_t* flatten_ids, float* render_colors, float* render_alphas,
    int32_t* last_ids, void* workspace, size_t workspace_bytes, void* stream);

/* ---- a8: gsplat::rasterize_to_pixels_from_world_3dgs_bwd (Ops.h:131-166; ...3DGSBwd.cu:16-379) ----
 * channels as in the forward pass (LichtFeld itself uses 1, 3, 4: RGB and the depth render modes of
 * Rasterization.cpp:374-393).  The five gradient outputs are fully WRITTEN (no zero-fill needed; the reference
 * zero-fills and accumulates, Rasterization.cpp:190-194): v_means [N,3], v_quats [N,4], v_scales [N,3],
 * v_colors [C,N,channels], v_opacities [C,N].  Workspace of the whole operator: 16 + max(1, channels - 3) accumulator
 * floats per Gaussian followed by the records (the ..._for functions; the two without a channel count serve up to
 * four channels). */
GSX_API size_t gsx_rasterize_bwd_workspace_bytes(uint32_t N);           /* up to four channels */
GSX_API size_t gsx_rasterize_bwd_accum_bytes(uint32_t N);               /* up to four channels */
GSX_API size_t gsx_rasterize_bwd_workspace_bytes_for(uint32_t N, uint32_t channels);
GSX_API size_t gsx_rasterize_bwd_accum_bytes_for(uint32_t N, uint32_t channels);
/* The backward pass is three launches - clear the accumulators, the per-tile kernel, the per-Gaussian epilogue -
 * that can also be called one by one (a training loop shares the forward's records and can fold the epilogue into
 * its own per-Gaussian pass); these three take the accumulator part (gsx_rasterize_bwd_accum_bytes[_for]) only;
 * gsx_rasterize_bwd_clear zeroes all workspace_bytes it is given. */
GSX_API int gsx_rasterize_bwd_clear(uint32_t N, void* workspace, size_t workspace_bytes, void* stream);
/* colors [N,channels] is read for channels beyond the third only (nullable otherwise); tile_order: nullable, see
 * gsx_tile_order */
GSX_API int gsx_rasterize_bwd_accumulate(uint32_t C, uint32_t N, int64_t n_isects, const void* records,
                                         const float* colors, uint32_t channels, const float* backgrounds,
                                         const uint8_t* masks, uint32_t image_width,
                                         uint32_t image_height, uint32_t tile_size, const float* viewmats0,
                                         const float* Ks, const int32_t* tile_offsets, const int32_t* flatten_ids,
                                         const uint32_t* tile_order, const float* render_alphas,
                                         const int32_t* last_ids,
                                         const float* v_render_colors, const float* v_render_alphas, void* workspace,
                                         size_t workspace_bytes, void* stream);
/* clear_accumulators != 0: the epilogue zeroes each accumulator row after reading it, so the next backward pass
 * needs no gsx_rasterize_bwd_clear */
GSX_API int gsx_rasterize_bwd_finish(uint32_t N, const float* means, const float* quats, const float* scales,
                                     const float* viewmats0, void* workspace, size_t workspace_bytes,
                                     int clear_accumulators, uint32_t channels, float* v_means, float* v_quats,
                                     float* v_scales, float* v_colors, float* v_opacities, void* stream);
GSX_API int gsx_rasterize_to_pixels_from_world_3dgs_bwd(
    uint32_t C, uint32_t N, int64_t n_isects, const float* means, const float* quats, const float* scales,
    const float* colors, uint32_t channels, const float* opacities, const float* backgrounds, const uint8_t* masks,
    uint32_t image_width, uint32_t image_height, uint32_t tile_size, const float* viewmats0,
    const float* viewmats1 /*[C,4,4] end-of-frame pose, nullable*/, const float* Ks, int camera_model, gsx_ut_params ut, int rs_type,
    const float* radial_coeffs, const float* tangential_coeffs, const float* thin_prism_coeffs,
    const int32_t* tile_offsets, const int32_t* flatten_ids, const float* render_alphas, const int32_t* last_ids,
    const float* v_render_colors, const float* v_render_alphas, float* v_means, float* v_quats, float* v_scales,
    float* v_colors, float* v_opacities, void* workspace, size_t workspace_bytes, void* stream);

/* ---- g1 glue of a9 (Rasterization.cpp:356-378 and :608-624), fused into one pass each ----
 * fwd: colors [N,3] = max(SH(means - campos(viewmat)) + 0.5, 0) where radii > 0, else 0.
 * bwd: v_sh_coeffs [N,K,3] fully written from v_colors with the clamp mask applied.
 * radii [N,2] on an 8-byte boundary (a Gaussian's two radii are read with one load), here and in the fused passes
 * below that take them. */
GSX_API int gsx_sh_colors_from_world(uint32_t N, uint32_t K, uint32_t sh_degree, const float* means,
                                     const float* sh_coeffs, const int32_t* radii, const float* viewmat,
                                     float* colors, void* stream);
/* gsx_sh_colors_from_world + gsx_pack_raster_records (channels = 3) in one pass, same results; records of
 * Gaussians with radii == 0 are left untouched (no tile lists them) and their SH rows are not read. */
GSX_API int gsx_sh_colors_records_from_world(uint32_t N, uint32_t K, uint32_t sh_degree, const float* means,
                                             const float* quats, const float* scales, const float* opacities,
                                             const float* sh_coeffs, const int32_t* radii, const float* viewmat,
                                             const float* Kmat, uint32_t image_width, uint32_t image_height,
                                             float* colors, void* records, void* stream);
GSX_API int gsx_sh_colors_from_world_bwd(uint32_t N, uint32_t K, uint32_t sh_degree, const float* means,
                                         const int32_t* radii, const float* viewmat, const float* colors,
                                         const float* v_colors, float* v_sh_coeffs, void* stream);

/* ---- a10: fusedssim / fusedssim_backward (include/kernels/ssim.cuh:11-28; src/training/kernels/ssim.cu) ----
 * img1, img2 [B,CH,H,W].  dm_* nullable together (train == false). */
GSX_API int gsx_fusedssim(int B, int CH, int H, int W, float C1, float C2, const float* img1, const float* img2,
                          float* ssim_map, float* dm_dmu1, float* dm_dsigma1_sq, float* dm_dsigma12, void* stream);
GSX_API int gsx_fusedssim_backward(int B, int CH, int H, int W, float C1, float C2, const float* img1,
                                   const float* img2, const float* dL_dmap, const float* dm_dmu1,
                                   const float* dm_dsigma1_sq, const float* dm_dsigma12, float* dL_dimg1,
                                   void* stream);

/* ---- a11: adam_step (fastgs/optimizer/include/adam_kernels.cuh:13-36; src/adam_api.cu:8-33) ----
 * gsx_adam_step_multi runs up to GSX_ADAM_MAX_TENSORS parameter groups in ONE launch (the reference
 * launches once per group, fused_adam.cpp:29-94); entries with n == 0 or grad == NULL are skipped. */
GSX_API int gsx_adam_step(float* param, float* exp_avg, float* exp_avg_sq, const float* grad, int64_t n, float lr,
                          float beta1, float beta2, float eps, float bias_correction1_rcp,
                          float bias_correction2_sqrt_rcp, void* stream);
#define GSX_ADAM_MAX_TENSORS 8
typedef struct gsx_adam_group {
    float* param;
    float* exp_avg;
    float* exp_avg_sq;
    const float* grad;
    int64_t n;
    float lr, beta1, beta2, eps, bias_correction1_rcp, bias_correction2_sqrt_rcp;
    /* Two parameter groups stored interleaved in one tensor (sh0 | shN as one [N,K,3] array): when period > 0,
     * elements with (index % period) >= split use lr2, and are left untouched (moments too) when skip2 != 0
     * (fused_adam.cpp:69-70 skips the shN group early in training).  period == 0: plain group. */
    uint32_t period, split;
    float lr2;
    int32_t skip2;
} gsx_adam_group;
GSX_API int gsx_adam_step_multi(const gsx_adam_group* groups_host, int n_groups, void* stream);

/* ---- a12: gsplat::relocation (Ops.h:52-57; RelocationCUDA.cu:11-43) ---- */
GSX_API int gsx_relocation(int M, const float* opacities, const float* scales, const int32_t* ratios,
                           const float* binoms, int n_max, float* new_opacities, float* new_scales, void* stream);
/* ---- a12 caller glue: MCMC::relocate_gs once the dead and the sampled index sets are chosen (mcmc.cpp:141-187;
 * the multinomial draw of :132 stays with the caller, random streams cannot be reproduced across libraries) ----
 *   ratios[i]      = min(1 + #{j : sampled[j] == sampled[i]}, n_max)                               (:141-148)
 *   new_o, new_s   = relocation(sigmoid(opacity_raw[s]), exp(scaling_raw[s]), ratios)               (:151-156)
 *   opacity_raw[s] = logit(clamp(new_o, min_opacity, 1 - 1e-7)),  scaling_raw[s] = log(new_s)       (:160-171)
 *   parameter rows:        row[dead[i]] = row[sampled[i]]  for every tensor with is_optimizer_state == 0  (:175-180)
 *   optimiser-state rows:  row[sampled[i]] = 0             for every tensor with is_optimizer_state == 1  (:100-104)
 * MCMC::add_new_gs (mcmc.cpp:192-347) is the same computation with the "dead" indices being the rows appended to
 * the (re-allocated, N = old N + n_idx) tensors, except that the moments of the sampled Gaussians are kept and the
 * new rows' moments are zero: state tensors take is_optimizer_state == 2 (row[dead[i]] = 0) there.
 * sampled_idxs / dead_idxs: i64 [n_idx], disjoint sets, values < N.  opacity_raw [N] and scaling_raw [N,3] must ALSO
 * be listed in tensors_host to have their rows copied to the dead indices. */
#define GSX_MCMC_MAX_TENSORS 24
typedef struct gsx_row_tensor {
    float* data;         /* [N, row_floats] */
    uint32_t row_floats; /* floats per Gaussian */
    int32_t is_optimizer_state; /* 0 parameter, 1 state cleared at sampled[i], 2 state cleared at dead[i] */
} gsx_row_tensor;
GSX_API size_t gsx_mcmc_relocate_workspace_bytes(uint32_t N, uint32_t n_idx);
GSX_API int gsx_mcmc_relocate(uint32_t N, uint32_t n_idx, const int64_t* sampled_idxs, const int64_t* dead_idxs,
                              const float* binoms, int n_max, float min_opacity, float* opacity_raw,
                              float* scaling_raw, const gsx_row_tensor* tensors_host, int n_tensors, void* workspace,
                              size_t workspace_bytes, void* stream);
/* ---- a13: gsplat::add_noise (Ops.h:59-65; RelocationCUDA.cu:112-144); means updated in place ---- */
GSX_API int gsx_add_noise(int N, const float* raw_opacities, const float* raw_scales, const float* raw_quats,
                          const float* noise, float* means, float current_lr, void* stream);
/* The same with the N(0,1) draws of mcmc.cpp:358 (torch::randn_like) generated where they are consumed: row i of the
 * noise is a function of (seed, offset, i) only - Philox4x32-10 with counter (i, offset) and key seed, two Box-Muller
 * pairs - so no [N,3] tensor is written and read back.  A caller advances `offset` per call.  The stream of values
 * is not torch's (no implementation outside torch reproduces that); gsx_philox_randn3 writes the same rows out for
 * callers that want them (out [N,3]): gsx_add_noise with that tensor equals gsx_add_noise_philox bit for bit. */
GSX_API int gsx_philox_randn3(uint32_t N, uint64_t seed, uint64_t offset, float* out, void* stream);
GSX_API int gsx_add_noise_philox(int N, const float* raw_opacities, const float* raw_scales, const float* raw_quats,
                                 float* means, float current_lr, uint64_t seed, uint64_t offset, void* stream);
/* ---- a14: gsplat::quats_to_rotmats (Ops.h:46-48; QuatToRotmatCUDA.cu:14-39) -> [N,3,3] row-major ---- */
GSX_API int gsx_quats_to_rotmats(int N, const float* quats, float* rotmats, void* stream);

/* ---- a15: step-driver passes that LichtFeld runs as ATen ops around the boundary, one kernel each ----
 * activations (src/core/splat_data.cpp:271-286): opacity = sigmoid(raw) [N], scales = exp(raw) [N,3],
 * quats = raw / max(|raw|, 1e-12) [N,4].  Their VJPs (what autograd applies after Ops.h's backward):
 * v_opacity_raw = v_o * o (1 - o), v_scaling_raw = v_s * s, v_rotation_raw = normalize VJP. */
GSX_API int gsx_activate_params(uint32_t N, const float* opacity_raw, const float* scaling_raw,
                                const float* rotation_raw, float* opacities, float* scales, float* quats,
                                void* stream);
/* gsx_activate_params + gsx_projection_ut_3dgs_fused (one pinhole camera, global shutter, opacities given, no
 * compensations) in one pass with the same results; conics nullable. */
GSX_API int gsx_activate_project_ut(uint32_t N, const float* means, const float* opacity_raw,
                                    const float* scaling_raw, const float* rotation_raw, const float* viewmat,
                                    const float* K, uint32_t image_width, uint32_t image_height, float eps2d,
                                    float near_plane, float far_plane, float radius_clip, gsx_ut_params ut,
                                    float* opacities, float* scales, float* quats, int32_t* radii, float* means2d,
                                    float* depths, float* conics, void* stream);
/* gsx_activate_project_ut + gsx_sh_colors_records_from_world: the whole per-Gaussian front of a forward pass
 * (splat_data.cpp:271-286 activations, ProjectionUT3DGSFused.cu:17-210, Rasterization.cpp:356-378 colours, the raster
 * records) with the same results.  For K = 16 coefficient rows on a 16-byte boundary it is one pass over the Gaussians
 * - the activated parameters and the visibility stay in registers, the parameters are read once - otherwise the two
 * launches. */
GSX_API int gsx_activate_project_sh_records(uint32_t N, uint32_t K, uint32_t sh_degree, const float* means,
                                            const float* opacity_raw, const float* scaling_raw,
                                            const float* rotation_raw, const float* sh_coeffs, const float* viewmat,
                                            const float* Kmat, uint32_t image_width, uint32_t image_height,
                                            float eps2d, float near_plane, float far_plane, float radius_clip,
                                            gsx_ut_params ut, float* opacities, float* scales, float* quats,
                                            int32_t* radii, float* means2d, float* depths, float* conics,
                                            float* colors, void* records, void* stream);
GSX_API int gsx_activate_params_bwd(uint32_t N, const float* opacity_raw, const float* scaling_raw,
                                    const float* rotation_raw, const float* v_opacities, const float* v_scales,
                                    const float* v_quats, float* v_opacity_raw, float* v_scaling_raw,
                                    float* v_rotation_raw, void* stream);
/* ---- scale / opacity L1 regularisation (include/kernels/regularization.cuh:12-48; regularization.cu:20-289;
 * trainer.cpp:136-174) ----  loss = weight * mean(f(params)), f = exp (scaling_raw) / sigmoid (opacity_raw);
 * param_grads (nullable) += (weight / n) f'(params).  partials: gsx_l1_regularization_partials() floats of scratch;
 * loss_out: one float in DEVICE memory (the reference blocks on a cudaMemcpy of it per call).  weight == 0: no-op. */
GSX_API uint32_t gsx_l1_regularization_partials(void);
GSX_API int gsx_exp_l1_regularization(const float* params, float* param_grads, int64_t n, float weight,
                                      float* partials, float* loss_out, void* stream);
GSX_API int gsx_sigmoid_l1_regularization(const float* params, float* param_grads, int64_t n, float weight,
                                          float* partials, float* loss_out, void* stream);

/* The tail of a training step in ONE pass over the Gaussians (no counterpart in the reference, which runs them as
 * separate kernels and ATen ops): rasterizer-backward epilogue (as gsx_rasterize_bwd_finish with
 * clear_accumulators = 1, on the ACTIVATIONS of the raw parameters) -> SH backward with the clamp mask (as
 * gsx_sh_colors_from_world_bwd) -> activation VJPs (as gsx_activate_params_bwd) -> Adam on the five raw parameter
 * tensors (as gsx_adam_step_multi with sh0 | shN interleaved in `shs` [N,K,3]).  The 236 B / Gaussian of gradients
 * never reach memory; parameters and moments come out bit-identical to the separate calls.  Must run before the
 * parameters change in any other way: it re-derives the activations from the raw parameters. */
typedef struct gsx_update_args {
    uint32_t N, K, sh_degree;
    float *means, *opacity_raw, *scaling_raw, *rotation_raw, *shs;                        /* parameters (in / out) */
    float *m_means, *m_opacity, *m_scaling, *m_rotation, *m_shs;                          /* exp_avg (in / out) */
    float *v_means, *v_opacity, *v_scaling, *v_rotation, *v_shs;                          /* exp_avg_sq (in / out) */
    const int32_t* radii;  /* [N,2] of the forward pass; 8-byte aligned */
    const float* colors;   /* [N,3] of the forward pass (clamp mask) */
    const float* viewmat;  /* [4,4] */
    void* accumulators;    /* gsx_rasterize_bwd_accumulate's workspace; consumed rows are zeroed */
    float lr_means, lr_sh0, lr_shN, lr_scaling, lr_rotation, lr_opacity;
    float beta1, beta2, eps, bias_correction1_rcp, bias_correction2_sqrt_rcp;
    int32_t skip_shN;      /* fused_adam.cpp:69-70 */
    /* regularisation gradients folded in: scaling grad += reg_scaling * exp(scaling_raw), opacity grad +=
     * reg_opacity * s (1 - s); reg_* = weight / element count as in gsx_*_l1_regularization (0 = off) */
    float reg_scaling, reg_opacity;
    /* nullable, device u32 [2] (e.g. gsx_tile_lists_error): while hold[0] != 0 the call changes no parameter or
     * moment (it still clears the accumulator rows) and adds 1 to hold[1] - a step whose tile lists did not fit its
     * buffers must not reach the optimiser */
    uint32_t* hold;
    /* nullable, device f32 [3] = {bias_correction1_rcp, bias_correction2_sqrt_rcp, skip_shN as 0 / 1}: read when the
     * kernel runs, in place of the three fields above (a launch replayed from a HIP graph keeps its by-value
     * arguments; the step's scalars change every iteration) */
    const float* step_scalars;
    /* nullable, PINNED HOST memory (hipHostMalloc), one u64: with `hold` given, every launch stores
     * hold[1] << 32 | hold[0] there as they stand after the launch (one 8-byte store at system scope) - the host sees
     * the sticky error bits and the number of calls held back so far without a synchronisation */
    uint64_t* hold_report;
} gsx_update_args;
GSX_API int gsx_backward_update_fused(const gsx_update_args* args_host, void* stream);

/* image = clamp(render HWC -> CHW, 0, 1) (rasterizer.cpp:205) and the per-pixel part of the photometric
 * loss of trainer.cpp:126-129: partial sums of |image - gt| into l1_partials [gsx_image_loss_blocks()]. */
GSX_API uint32_t gsx_image_loss_blocks(uint32_t H, uint32_t W);
GSX_API int gsx_image_from_render(uint32_t H, uint32_t W, const float* render_hwc, const float* gt_chw,
                                  float* image_chw, float* l1_partials, void* stream);
/* mean of the SSIM map over the "valid" crop [5:H-5, 5:W-5] (fused_ssim.cuh:59-67,117-122) as partial sums */
GSX_API int gsx_ssim_valid_partials(uint32_t CH, uint32_t H, uint32_t W, const float* ssim_map, float* partials,
                                    void* stream);
/* loss = (1-lambda) * mean|img-gt| + lambda * (1 - mean_valid(ssim)); one block; writes loss_out[0..2] =
 * (loss, l1, ssim) on the device */
GSX_API int gsx_photometric_loss_finish(uint32_t CH, uint32_t H, uint32_t W, float lambda_dssim,
                                        const float* l1_partials, const float* ssim_partials, uint32_t n_partials,
                                        float* loss_out, void* stream);
/* The same loss in two kernels for a training loop: forward = clamp + permute on load, SSIM derivative maps and
 * the per-block partial sums (l1_partials / ssim_partials hold gsx_photometric_partials(H, W) floats each; the
 * clamped image and the SSIM map are not written), then gsx_photometric_loss_finish; backward = v_render [H,W,3]
 * from the derivative maps, with d loss / d map of the valid crop formed on the fly.  Per-pixel arithmetic is that
 * of the separate kernels; the loss value differs from theirs by summation order only. */
GSX_API uint32_t gsx_photometric_partials(uint32_t H, uint32_t W);
GSX_API int gsx_photometric_loss_forward(uint32_t H, uint32_t W, float C1, float C2, const float* render_hwc,
                                         const float* gt_chw, float* dm_dmu1, float* dm_dsigma1_sq,
                                         float* dm_dsigma12, float* l1_partials, float* ssim_partials, void* stream);
GSX_API int gsx_photometric_loss_backward(uint32_t H, uint32_t W, float lambda_dssim, const float* render_hwc,
                                          const float* gt_chw, const float* dm_dmu1, const float* dm_dsigma1_sq,
                                          const float* dm_dsigma12, float* v_render_hwc, void* stream);
/* the same launch, which also does gsx_photometric_loss_finish's work on the way (its first workgroup adds up the
 * forward pass's partial sums; loss_out[0..2] as there, same bits): a step that differentiates needs no launch for
 * the loss value */
GSX_API int gsx_photometric_loss_backward_finish(uint32_t H, uint32_t W, float lambda_dssim, const float* render_hwc,
                                                 const float* gt_chw, const float* dm_dmu1,
                                                 const float* dm_dsigma1_sq, const float* dm_dsigma12,
                                                 const float* l1_partials, const float* ssim_partials,
                                                 float* loss_out, float* v_render_hwc, void* stream);
/* gsx_photometric_loss_backward(_finish, with loss_out != NULL) and gsx_tile_order by tile_cost in one launch (no
 * counterpart in the reference): one workgroup more than the image needs sorts the tiles for the backward rasterizer
 * that follows, so that the order costs neither a launch nor a second stream with its events.  tile_cost: u32
 * [tile_width * tile_height] (the tile_walk of gsx_rasterize_records_fwd), tile_order: as gsx_tile_order writes it.
 * loss_out, l1_partials, ssim_partials: nullable together (no loss value then). */
GSX_API int gsx_photometric_loss_backward_order(uint32_t H, uint32_t W, float lambda_dssim, const float* render_hwc,
                                                const float* gt_chw, const float* dm_dmu1,
                                                const float* dm_dsigma1_sq, const float* dm_dsigma12,
                                                const float* l1_partials, const float* ssim_partials,
                                                float* loss_out, float* v_render_hwc, uint32_t tile_width,
                                                uint32_t tile_height, const uint32_t* tile_cost,
                                                uint32_t* tile_order, void* stream);
/* v_render [H,W,3] = d loss / d render: L1 sign term + lambda * SSIM term (dL_dimg_ssim is
 * gsx_fusedssim_backward's output for dL_dmap = -lambda / count on the valid crop, 0 elsewhere), passed through
 * the clamp VJP (zero where render < 0 or > 1) and the CHW -> HWC permute. */
GSX_API int gsx_ssim_valid_grad_map(uint32_t CH, uint32_t H, uint32_t W, float scale, float* dL_dmap, void* stream);
GSX_API int gsx_render_grad_from_loss(uint32_t H, uint32_t W, float lambda_dssim, const float* render_hwc,
                                      const float* image_chw, const float* gt_chw, const float* dL_dimg_ssim,
                                      float* v_render_hwc, void* stream);

/* ---- trained model on disk: binary little-endian PLY, one float32 row per Gaussian ----
 * writer: SplatData::save_ply / to_point_cloud / get_attribute_names / write_ply_impl (src/core/splat_data.cpp:
 * 113-169, 402-418, 484-506); reader: load_ply / parse_header / extract_* (src/loader/formats/ply.cpp:185-323,
 * 446-496, 500-637).  Row of the writer (gsx_ply_row_floats(K) = 14 + 3K floats): x y z nx ny nz f_dc_0..2
 * f_rest_0..3(K-1)-1 opacity scale_0..2 rot_0..3 with normals 0, f_rest channel-major (all R, then G, then B),
 * opacity / scales raw (logit / log), rotation normalised.  shs here is [N,K,3] (sh0 and shN concatenated).
 * The row image is assembled / taken apart on the GPU; the *_file functions only move whole buffers. */
typedef struct gsx_ply_layout {
    uint64_t vertex_count;
    uint64_t data_offset;   /* byte offset of the first vertex row */
    uint32_t stride_floats; /* floats per vertex row */
    int32_t pos[3];         /* float index inside a row; -1 = property absent */
    int32_t opacity;
    int32_t scale[3];
    int32_t rot[4];
    int32_t dc_start, dc_count, rest_start, rest_count;
} gsx_ply_layout;
GSX_API uint32_t gsx_ply_row_floats(uint32_t K);
/* header text of the writer; returns its length (buf may be null to query), negative status on error */
GSX_API int64_t gsx_ply_format_header(uint64_t N, uint32_t K, char* buf, size_t capacity);
/* parse_header (ply.cpp:185-323): LF or CRLF lines, '#' / empty lines skipped, properties found by name in any
 * order, unknown float properties skipped over.  Errors as the reference's (missing magic, not binary little
 * endian, no vertex element, no end_header, > 10000 lines); a non-float vertex property is GSX_ERR_UNSUPPORTED
 * (the reference would misread the rows). */
GSX_API int gsx_ply_parse_header(const char* data, size_t size, gsx_ply_layout* layout);
/* K of the tensors a file unpacks to: dc_count/3 (1 if absent) + rest_count/3 (15 if absent, ply.cpp:554) */
GSX_API uint32_t gsx_ply_layout_sh_coeffs(const gsx_ply_layout* layout);
GSX_API int gsx_ply_pack_rows(uint64_t N, uint32_t K, const float* means, const float* shs, const float* opacity_raw,
                              const float* scaling_raw, const float* rotation_raw, float* rows, void* stream);
/* rows: device copy of the vertex rows (vertex_count * stride_floats floats).  Absent properties get the
 * reference's defaults: 0, log-scale -5 (ply.cpp:583), rotation (1,0,0,0) (ply.cpp:608). */
GSX_API int gsx_ply_unpack_rows(const gsx_ply_layout* layout, const float* rows, float* means, float* shs,
                                float* opacity_raw, float* scaling_raw, float* rotation_raw, void* stream);
GSX_API int gsx_ply_write_file(const char* path, uint64_t N, uint32_t K, const float* rows_host);
GSX_API int gsx_ply_read_file_header(const char* path, gsx_ply_layout* layout);
GSX_API int gsx_ply_read_file_rows(const char* path, const gsx_ply_layout* layout, float* rows_host);

#ifdef __cplusplus
}
#endif
#endif /* GSX_H */
