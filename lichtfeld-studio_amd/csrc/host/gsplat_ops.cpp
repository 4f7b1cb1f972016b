// gsplat_ops.cpp - the C++ host layer of the path: at::Tensor in / out with the validation, allocation and error
// behaviour of LichtFeld-Studio's gsplat/*.cpp host functions (Projection.cpp:16-110, SphericalHarmonics.cpp:15-75,
// Intersect.cpp:15-137, QuatToRotmat.cpp:14-26, Relocation.cpp:15-50, Rasterization.cpp:20-261,267-642,
// src/training/kernels/ssim.cu:431-510, fastgs/optimizer/src/adam_api.cu:8-33), calling the gfx950 kernels through
// the C ABI of gsx.h on torch's current stream.  Torch is used for tensors, the caching allocator and the stream.
#include "gsplat_api.h"

#include <ATen/Functions.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <c10/util/Exception.h>
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <deque>
#include <memory>
#include <mutex>
#include <optional>
#include <vector>

#include "gsx.h"

namespace {

// gsplat/Common.h:12-19
#define GSX_CHECK_CUDA(x) TORCH_CHECK((x).is_cuda(), #x " must be a CUDA tensor")
#define GSX_CHECK_CONTIGUOUS(x) TORCH_CHECK((x).is_contiguous(), #x " must be contiguous")
#define CHECK_INPUT(x)  \
    GSX_CHECK_CUDA(x);  \
    GSX_CHECK_CONTIGUOUS(x)
#define DEVICE_GUARD(t) const c10::DeviceGuard device_guard((t).device())

using gsplat::OptT;

inline void* cur_stream(const at::Tensor& t) { return (void*)c10::hip::getCurrentHIPStream(t.device().index()).stream(); }

// the channel counts the rasterizers take (Rasterization.cpp:106-128)
inline bool channels_built(uint32_t c) {
    return c == 1 || c == 2 || c == 3 || c == 4 || c == 5 || c == 8 || c == 9 || c == 16 || c == 17 || c == 32 ||
           c == 33 || c == 64 || c == 65 || c == 128 || c == 129 || c == 256 || c == 257 || c == 512 || c == 513;
}
inline void gsx_check(int status) { TORCH_CHECK(status == GSX_OK, "gsx (", gsx_status_string(status), "): ", gsx_last_error()); }

inline bool has(const OptT& t) { return t.has_value() && t->defined() && t->numel() > 0; }
inline const float* fptr(const OptT& t) { return has(t) ? t->data_ptr<float>() : nullptr; }
inline const uint8_t* bptr(const OptT& t) { return has(t) ? static_cast<const uint8_t*>(t->data_ptr()) : nullptr; }

inline gsx_ut_params to_gsx(const UnscentedTransformParameters& p) {
    gsx_ut_params u;
    u.alpha = p.alpha;
    u.beta = p.beta;
    u.kappa = p.kappa;
    u.in_image_margin_factor = p.in_image_margin_factor;
    u.require_all_sigma_points_valid = p.require_all_sigma_points_valid ? 1 : 0;
    return u;
}

// The kernels index by these extents: a tensor of another shape would be read or written out of bounds.
// -1 leaves an extent free.
inline void sized(const at::Tensor& t, const char* name, std::initializer_list<int64_t> shape) {
    bool ok = t.dim() == (int64_t)shape.size();
    int64_t i = 0;
    for (const int64_t want : shape) {
        ok = ok && (want < 0 || t.size(i) == want);
        ++i;
    }
    TORCH_CHECK(ok, name, " must be ", c10::IntArrayRef(shape.begin(), shape.size()), " (-1 = any), got ", t.sizes());
}
inline void sized(const OptT& t, const char* name, std::initializer_list<int64_t> shape) {
    if (has(t))
        sized(t.value(), name, shape);
}

// [C,4,4] poses, [C,3,3] intrinsics; coefficient rows as the kernels read them (ProjectionUT3DGSFused.cu:101-126):
// radial [C,6] (pinhole) or [C,4] (fisheye), tangential [C,2], thin prism [C,4]
inline void check_camera_tensors(int64_t C, gsplat::CameraModelType camera_model, const at::Tensor& viewmats0,
                                 const OptT& viewmats1, const at::Tensor& Ks, const OptT& radial_coeffs,
                                 const OptT& tangential_coeffs, const OptT& thin_prism_coeffs) {
    sized(viewmats0, "viewmats0", {C, 4, 4});
    sized(viewmats1, "viewmats1", {C, 4, 4});
    sized(Ks, "Ks", {C, 3, 3});
    sized(radial_coeffs, "radial_coeffs", {C, camera_model == gsplat::FISHEYE ? 4 : 6});
    sized(tangential_coeffs, "tangential_coeffs", {C, 2});
    sized(thin_prism_coeffs, "thin_prism_coeffs", {C, 4});
}

inline at::Tensor workspace(size_t bytes, const at::Tensor& like) {
    return at::empty({(int64_t)(bytes < 256 ? 256 : bytes)}, like.options().dtype(at::kByte));
}

} // namespace

namespace gsplat {

at::Tensor spherical_harmonics_fwd(const uint32_t degrees_to_use, const at::Tensor dirs, const at::Tensor coeffs,
                                   const OptT masks) {
    DEVICE_GUARD(dirs);
    CHECK_INPUT(dirs);
    CHECK_INPUT(coeffs);
    if (masks.has_value()) {
        CHECK_INPUT(masks.value());
    }
    TORCH_CHECK(coeffs.size(-1) == 3, "coeffs must have last dimension 3");
    TORCH_CHECK(dirs.size(-1) == 3, "dirs must have last dimension 3");
    at::Tensor colors = at::empty_like(dirs);
    gsx_check(gsx_spherical_harmonics_fwd((uint32_t)(dirs.numel() / 3), (uint32_t)coeffs.size(-2), degrees_to_use,
                                          dirs.data_ptr<float>(), coeffs.data_ptr<float>(), bptr(masks),
                                          colors.data_ptr<float>(), cur_stream(dirs)));
    return colors;
}

std::tuple<at::Tensor, at::Tensor> spherical_harmonics_bwd(const uint32_t K, const uint32_t degrees_to_use,
                                                           const at::Tensor dirs, const at::Tensor coeffs,
                                                           const OptT masks, const at::Tensor v_colors,
                                                           bool compute_v_dirs) {
    DEVICE_GUARD(dirs);
    CHECK_INPUT(dirs);
    CHECK_INPUT(coeffs);
    CHECK_INPUT(v_colors);
    if (masks.has_value()) {
        CHECK_INPUT(masks.value());
    }
    TORCH_CHECK(v_colors.size(-1) == 3, "v_colors must have last dimension 3");
    TORCH_CHECK(coeffs.size(-1) == 3, "coeffs must have last dimension 3");
    TORCH_CHECK(dirs.size(-1) == 3, "dirs must have last dimension 3");
    at::Tensor v_coeffs = at::empty_like(coeffs); // the kernel writes every element
    at::Tensor v_dirs;
    if (compute_v_dirs)
        v_dirs = at::zeros_like(dirs);
    gsx_check(gsx_spherical_harmonics_bwd((uint32_t)(dirs.numel() / 3), K, degrees_to_use, dirs.data_ptr<float>(),
                                          coeffs.data_ptr<float>(), bptr(masks), v_colors.data_ptr<float>(),
                                          v_coeffs.data_ptr<float>(),
                                          compute_v_dirs ? v_dirs.data_ptr<float>() : nullptr, cur_stream(dirs)));
    return std::make_tuple(v_coeffs, v_dirs);
}

namespace {
void sort_pairs(const int64_t n_isects, const uint32_t begin_bit, const uint32_t end_bit, at::Tensor& isect_ids,
                at::Tensor& flatten_ids, at::Tensor& isect_ids_sorted, at::Tensor& flatten_ids_sorted);
}

void radix_sort_double_buffer(const int64_t n_isects, const uint32_t tile_n_bits, const uint32_t cam_n_bits,
                              at::Tensor isect_ids, at::Tensor flatten_ids, at::Tensor isect_ids_sorted,
                              at::Tensor flatten_ids_sorted) {
    sort_pairs(n_isects, 0, 32 + tile_n_bits + cam_n_bits, isect_ids, flatten_ids, isect_ids_sorted,
               flatten_ids_sorted);
}

namespace {
void sort_pairs(const int64_t n_isects, const uint32_t begin_bit, const uint32_t end_bit, at::Tensor& isect_ids,
                at::Tensor& flatten_ids, at::Tensor& isect_ids_sorted, at::Tensor& flatten_ids_sorted) {
    if (n_isects <= 0)
        return;
    at::Tensor ws = workspace(gsx_radix_sort_pairs_workspace_bytes(n_isects), isect_ids);
    int selector = 0;
    gsx_check(gsx_radix_sort_pairs(n_isects, isect_ids.data_ptr<int64_t>(), flatten_ids.data_ptr<int32_t>(),
                                   isect_ids_sorted.data_ptr<int64_t>(), flatten_ids_sorted.data_ptr<int32_t>(),
                                   begin_bit, end_bit, ws.data_ptr(), (size_t)ws.numel(), &selector,
                                   cur_stream(isect_ids)));
    if (selector == 0) { // sorted items ended up in the input buffers (IntersectTile.cu:315-328)
        isect_ids_sorted.set_(isect_ids);
        flatten_ids_sorted.set_(flatten_ids);
    }
}
} // namespace

std::tuple<at::Tensor, at::Tensor, at::Tensor> intersect_tile(const at::Tensor means2d, const at::Tensor radii,
                                                              const at::Tensor depths, const OptT camera_ids,
                                                              const OptT gaussian_ids, const uint32_t C,
                                                              const uint32_t tile_size, const uint32_t tile_width,
                                                              const uint32_t tile_height, const bool sort) {
    DEVICE_GUARD(means2d);
    CHECK_INPUT(means2d);
    CHECK_INPUT(radii);
    CHECK_INPUT(depths);
    const bool packed = means2d.dim() == 2;
    const uint32_t tile_n_bits = gsx_n_bits(tile_width * tile_height);
    const uint32_t cam_n_bits = gsx_n_bits(C);
    at::Tensor tiles_per_gauss = at::empty_like(depths, depths.options().dtype(at::kInt));
    if (packed) { // rows [nnz], each naming its camera (Intersect.cpp:32-39, IntersectTile.cu:50, 86-94)
        TORCH_CHECK(camera_ids.has_value() && gaussian_ids.has_value(),
                    "When packed is set, camera_ids and gaussian_ids must be provided.");
        CHECK_INPUT(camera_ids.value());
        CHECK_INPUT(gaussian_ids.value());
        const int64_t nnz = means2d.size(0);
        TORCH_CHECK(camera_ids->scalar_type() == at::kLong && gaussian_ids->scalar_type() == at::kLong,
                    "camera_ids and gaussian_ids must be int64");
        TORCH_CHECK(means2d.size(1) == 2 && radii.dim() == 2 && radii.size(0) == nnz && radii.size(1) == 2 &&
                        depths.numel() == nnz && camera_ids->numel() == nnz && gaussian_ids->numel() == nnz,
                    "packed intersect_tile: means2d [nnz,2], radii [nnz,2], depths / camera_ids / gaussian_ids [nnz]");
        void* stream = cur_stream(means2d);
        at::Tensor cum = at::empty({nnz}, depths.options().dtype(at::kLong));
        int64_t n_isects = 0;
        at::Tensor ws = workspace(gsx_intersect_tile_count_workspace_bytes(1, (uint32_t)nnz), depths);
        gsx_check(gsx_intersect_tile_count(1, (uint32_t)nnz, means2d.data_ptr<float>(), radii.data_ptr<int32_t>(),
                                           tile_size, tile_width, tile_height, tiles_per_gauss.data_ptr<int32_t>(),
                                           cum.data_ptr<int64_t>(), ws.data_ptr(), (size_t)ws.numel(), &n_isects,
                                           stream));
        at::Tensor isect_ids = at::empty({n_isects}, depths.options().dtype(at::kLong));
        at::Tensor flatten_ids = at::empty({n_isects}, depths.options().dtype(at::kInt));
        if (n_isects)
            gsx_check(gsx_intersect_tile_emit_packed(C, (uint32_t)nnz, means2d.data_ptr<float>(),
                                                     radii.data_ptr<int32_t>(), depths.data_ptr<float>(),
                                                     camera_ids->data_ptr<int64_t>(), cum.data_ptr<int64_t>(),
                                                     tile_size, tile_width, tile_height,
                                                     isect_ids.data_ptr<int64_t>(), flatten_ids.data_ptr<int32_t>(),
                                                     stream));
        if (n_isects && sort) {
            at::Tensor isect_ids_sorted = at::empty_like(isect_ids);
            at::Tensor flatten_ids_sorted = at::empty_like(flatten_ids);
            sort_pairs(n_isects, 0u, 32 + tile_n_bits + cam_n_bits, isect_ids, flatten_ids, isect_ids_sorted,
                       flatten_ids_sorted);
            return std::make_tuple(tiles_per_gauss, isect_ids_sorted, flatten_ids_sorted);
        }
        return std::make_tuple(tiles_per_gauss, isect_ids, flatten_ids);
    }
    const uint32_t N = (uint32_t)means2d.size(1);
    // one camera, sorted output: visit the Gaussians in depth order and sort on the tile bits only (same array as
    // one sort on every bit, Intersect.cpp:104-113, because the sort is stable)
    const bool two_level = sort && C == 1;
    at::Tensor order;
    const int32_t* order_ptr = nullptr;
    at::Tensor cum = at::empty({(int64_t)C * N}, depths.options().dtype(at::kLong));
    int64_t n_isects = 0;
    void* stream = cur_stream(means2d);
    at::Tensor ordered_ws; // holds the sorted depth keys the emission reads: alive until that launch is queued
    if (two_level && N > 0) {
        order = at::empty({(int64_t)N}, depths.options().dtype(at::kInt));
        order_ptr = order.data_ptr<int32_t>();
        ordered_ws = workspace(gsx_intersect_tile_count_ordered_workspace_bytes(N), depths);
        at::Tensor& ws = ordered_ws;
        gsx_check(gsx_intersect_tile_count_ordered(N, means2d.data_ptr<float>(), radii.data_ptr<int32_t>(),
                                                   depths.data_ptr<float>(), tile_size, tile_width, tile_height,
                                                   order.data_ptr<int32_t>(), tiles_per_gauss.data_ptr<int32_t>(),
                                                   cum.data_ptr<int64_t>(), ws.data_ptr(), (size_t)ws.numel(),
                                                   &n_isects, 1, stream));
    } else {
        at::Tensor ws = workspace(gsx_intersect_tile_count_workspace_bytes(C, N), depths);
        gsx_check(gsx_intersect_tile_count(C, N, means2d.data_ptr<float>(), radii.data_ptr<int32_t>(), tile_size,
                                           tile_width, tile_height, tiles_per_gauss.data_ptr<int32_t>(),
                                           cum.data_ptr<int64_t>(), ws.data_ptr(), (size_t)ws.numel(), &n_isects,
                                           stream));
    }
    at::Tensor isect_ids = at::empty({n_isects}, depths.options().dtype(at::kLong));
    at::Tensor flatten_ids = at::empty({n_isects}, depths.options().dtype(at::kInt));
    if (n_isects && ordered_ws.defined()) {
        gsx_check(gsx_intersect_tile_emit_ordered(N, means2d.data_ptr<float>(), radii.data_ptr<int32_t>(),
                                                  depths.data_ptr<float>(), cum.data_ptr<int64_t>(), order_ptr,
                                                  ordered_ws.data_ptr(), tile_size, tile_width, tile_height, INT64_MAX,
                                                  isect_ids.data_ptr<int64_t>(), flatten_ids.data_ptr<int32_t>(),
                                                  stream));
    } else if (n_isects) {
        gsx_check(gsx_intersect_tile_emit(C, N, means2d.data_ptr<float>(), radii.data_ptr<int32_t>(),
                                          depths.data_ptr<float>(), cum.data_ptr<int64_t>(), order_ptr, tile_size,
                                          tile_width, tile_height, isect_ids.data_ptr<int64_t>(),
                                          flatten_ids.data_ptr<int32_t>(), stream));
    }
    if (n_isects && sort) {
        at::Tensor isect_ids_sorted = at::empty_like(isect_ids);
        at::Tensor flatten_ids_sorted = at::empty_like(flatten_ids);
        sort_pairs(n_isects, two_level ? 32u : 0u, 32 + tile_n_bits + cam_n_bits, isect_ids, flatten_ids,
                   isect_ids_sorted, flatten_ids_sorted);
        return std::make_tuple(tiles_per_gauss, isect_ids_sorted, flatten_ids_sorted);
    }
    return std::make_tuple(tiles_per_gauss, isect_ids, flatten_ids);
}

namespace {
// flatten_ids and offsets of one camera as intersect_tile(sort = true) + intersect_offset return them, without
// forming the 64-bit keys: pairs in depth order with their 16-bit tile index as the sort key (the fused forward
// keeps no isect_ids, Rasterization.cpp:413-424).  false where the grid needs the 64-bit keys.
bool tile_lists(const at::Tensor& means2d, const at::Tensor& radii, const at::Tensor& depths, uint32_t tile_size,
                uint32_t tile_width, uint32_t tile_height, at::Tensor* flatten_ids, at::Tensor* offsets) {
    if (means2d.size(0) != 1 || !gsx_intersect_tile_pairs_fit(tile_width, tile_height))
        return false;
    const uint32_t N = (uint32_t)means2d.size(1);
    void* stream = cur_stream(means2d);
    const auto i32 = depths.options().dtype(at::kInt);
    *offsets = at::empty({1, (int64_t)tile_height, (int64_t)tile_width}, i32);
    int64_t n = 0;
    at::Tensor order = at::empty({(int64_t)N}, i32), tiles_per_gauss = at::empty({(int64_t)N}, i32);
    at::Tensor cum = at::empty({(int64_t)N}, depths.options().dtype(at::kLong));
    at::Tensor ws = workspace(gsx_intersect_tile_count_ordered_workspace_bytes(N), depths);
    if (N > 0)
        gsx_check(gsx_intersect_tile_count_ordered(N, means2d.data_ptr<float>(), radii.data_ptr<int32_t>(),
                                                   depths.data_ptr<float>(), tile_size, tile_width, tile_height,
                                                   order.data_ptr<int32_t>(), tiles_per_gauss.data_ptr<int32_t>(),
                                                   cum.data_ptr<int64_t>(), ws.data_ptr(), (size_t)ws.numel(), &n, 1,
                                                   stream));
    at::Tensor keys[2] = {at::empty({n}, depths.options().dtype(at::kShort)),
                          at::empty({n}, depths.options().dtype(at::kShort))};
    at::Tensor vals[2] = {at::empty({n}, i32), at::empty({n}, i32)};
    int sel = 0;
    if (n > 0) {
        gsx_check(gsx_intersect_tile_emit_pairs(N, cum.data_ptr<int64_t>(), order.data_ptr<int32_t>(), ws.data_ptr(),
                                                tile_size, tile_width, tile_height, n,
                                                (uint16_t*)keys[0].data_ptr<int16_t>(), vals[0].data_ptr<int32_t>(),
                                                stream));
        at::Tensor ws2 = workspace(gsx_radix_sort_pairs_workspace_bytes(n), depths);
        gsx_check(gsx_radix_sort_tile_pairs(n, (uint16_t*)keys[0].data_ptr<int16_t>(), vals[0].data_ptr<int32_t>(),
                                            (uint16_t*)keys[1].data_ptr<int16_t>(), vals[1].data_ptr<int32_t>(),
                                            gsx_n_bits(tile_width * tile_height), ws2.data_ptr(),
                                            (size_t)ws2.numel(), &sel, stream));
    }
    gsx_check(gsx_intersect_tile_pairs_offset(n, (const uint16_t*)keys[sel].data_ptr<int16_t>(), tile_width,
                                              tile_height, offsets->data_ptr<int32_t>(), stream));
    *flatten_ids = vals[sel];
    return true;
}
} // namespace

at::Tensor intersect_offset(const at::Tensor isect_ids, const uint32_t C, const uint32_t tile_width,
                            const uint32_t tile_height) {
    DEVICE_GUARD(isect_ids);
    CHECK_INPUT(isect_ids);
    at::Tensor offsets = at::empty({C, tile_height, tile_width}, isect_ids.options().dtype(at::kInt));
    gsx_check(gsx_intersect_offset(isect_ids.size(0), isect_ids.data_ptr<int64_t>(), C, tile_width, tile_height,
                                   offsets.data_ptr<int32_t>(), cur_stream(isect_ids)));
    return offsets;
}

at::Tensor quats_to_rotmats(const at::Tensor quats) {
    DEVICE_GUARD(quats);
    CHECK_INPUT(quats);
    const int64_t N = quats.size(0);
    sized(quats, "quats", {N, 4});
    at::Tensor rotmats = at::empty({N, 3, 3}, quats.options());
    gsx_check(gsx_quats_to_rotmats((int)N, quats.data_ptr<float>(), rotmats.data_ptr<float>(), cur_stream(quats)));
    return rotmats;
}

std::tuple<at::Tensor, at::Tensor> relocation(at::Tensor opacities, at::Tensor scales, at::Tensor ratios,
                                              at::Tensor binoms, const int n_max) {
    DEVICE_GUARD(opacities);
    CHECK_INPUT(opacities);
    CHECK_INPUT(scales);
    CHECK_INPUT(ratios);
    CHECK_INPUT(binoms);
    const int64_t n = opacities.size(0);
    sized(opacities, "opacities", {n});
    sized(scales, "scales", {n, 3});
    sized(ratios, "ratios", {n});
    sized(binoms, "binoms", {n_max, n_max});
    at::Tensor new_opacities = at::empty_like(opacities);
    at::Tensor new_scales = at::empty_like(scales);
    gsx_check(gsx_relocation((int)opacities.size(0), opacities.data_ptr<float>(), scales.data_ptr<float>(),
                             ratios.data_ptr<int32_t>(), binoms.data_ptr<float>(), n_max,
                             new_opacities.data_ptr<float>(), new_scales.data_ptr<float>(), cur_stream(opacities)));
    return std::make_tuple(new_opacities, new_scales);
}

void add_noise(at::Tensor raw_opacities, at::Tensor raw_scales, at::Tensor raw_quats, at::Tensor noise,
               at::Tensor means, const float current_lr) {
    DEVICE_GUARD(raw_opacities);
    CHECK_INPUT(raw_opacities);
    CHECK_INPUT(raw_scales);
    CHECK_INPUT(raw_quats);
    CHECK_INPUT(noise);
    CHECK_INPUT(means);
    const int64_t n = means.size(0);
    sized(means, "means", {n, 3});
    sized(noise, "noise", {n, 3});
    sized(raw_quats, "raw_quats", {n, 4});
    sized(raw_scales, "raw_scales", {n, 3});
    TORCH_CHECK(raw_opacities.numel() == n, "raw_opacities must hold ", n, " values, got ", raw_opacities.sizes());
    gsx_check(gsx_add_noise((int)raw_opacities.size(0), raw_opacities.data_ptr<float>(), raw_scales.data_ptr<float>(),
                            raw_quats.data_ptr<float>(), noise.data_ptr<float>(), means.data_ptr<float>(), current_lr,
                            cur_stream(means)));
}

std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor> projection_ut_3dgs_fused(
    const at::Tensor means, const at::Tensor quats, const at::Tensor scales, const OptT opacities,
    const at::Tensor viewmats0, const OptT viewmats1, const at::Tensor Ks, const uint32_t image_width,
    const uint32_t image_height, const float eps2d, const float near_plane, const float far_plane,
    const float radius_clip, const bool calc_compensations, const CameraModelType camera_model,
    const UnscentedTransformParameters ut_params, ShutterType rs_type, const OptT radial_coeffs,
    const OptT tangential_coeffs, const OptT thin_prism_coeffs) {
    DEVICE_GUARD(means);
    CHECK_INPUT(means);
    CHECK_INPUT(quats);
    CHECK_INPUT(scales);
    if (opacities.has_value()) {
        CHECK_INPUT(opacities.value());
    }
    CHECK_INPUT(viewmats0);
    if (viewmats1.has_value()) {
        CHECK_INPUT(viewmats1.value());
    }
    CHECK_INPUT(Ks);
    if (radial_coeffs.has_value()) {
        CHECK_INPUT(radial_coeffs.value());
    }
    if (tangential_coeffs.has_value()) {
        CHECK_INPUT(tangential_coeffs.value());
    }
    if (thin_prism_coeffs.has_value()) {
        CHECK_INPUT(thin_prism_coeffs.value());
    }
    const uint32_t N = (uint32_t)means.size(0), C = (uint32_t)viewmats0.size(0);
    sized(means, "means", {N, 3});
    sized(quats, "quats", {N, 4});
    sized(scales, "scales", {N, 3});
    sized(opacities, "opacities", {N});
    check_camera_tensors(C, camera_model, viewmats0, viewmats1, Ks, radial_coeffs, tangential_coeffs,
                         thin_prism_coeffs);
    auto opt = means.options();
    at::Tensor radii = at::empty({C, N, 2}, opt.dtype(at::kInt));
    at::Tensor means2d = at::empty({C, N, 2}, opt);
    at::Tensor depths = at::empty({C, N}, opt);
    at::Tensor conics = at::empty({C, N, 3}, opt);
    at::Tensor compensations;
    if (calc_compensations)
        compensations = at::zeros({C, N}, opt); // Projection.cpp:77
    gsx_check(gsx_projection_ut_3dgs_fused(
        C, N, means.data_ptr<float>(), quats.data_ptr<float>(), scales.data_ptr<float>(), fptr(opacities),
        viewmats0.data_ptr<float>(), fptr(viewmats1), Ks.data_ptr<float>(), image_width, image_height, eps2d,
        near_plane, far_plane, radius_clip, (int)camera_model, to_gsx(ut_params), (int)rs_type, fptr(radial_coeffs),
        fptr(tangential_coeffs), fptr(thin_prism_coeffs), radii.data_ptr<int32_t>(), means2d.data_ptr<float>(),
        depths.data_ptr<float>(), conics.data_ptr<float>(),
        calc_compensations ? compensations.data_ptr<float>() : nullptr, cur_stream(means)));
    return std::make_tuple(radii, means2d, depths, conics, compensations);
}

std::tuple<at::Tensor, at::Tensor, at::Tensor> rasterize_to_pixels_from_world_3dgs_fwd(
    const at::Tensor means, const at::Tensor quats, const at::Tensor scales, const at::Tensor colors,
    const at::Tensor opacities, const OptT backgrounds, const OptT masks, const uint32_t image_width,
    const uint32_t image_height, const uint32_t tile_size, const at::Tensor viewmats0, const OptT viewmats1,
    const at::Tensor Ks, const CameraModelType camera_model, const UnscentedTransformParameters ut_params,
    ShutterType rs_type, const OptT radial_coeffs, const OptT tangential_coeffs, const OptT thin_prism_coeffs,
    const at::Tensor tile_offsets, const at::Tensor flatten_ids) {
    DEVICE_GUARD(means);
    CHECK_INPUT(means);
    CHECK_INPUT(quats);
    CHECK_INPUT(scales);
    CHECK_INPUT(colors);
    CHECK_INPUT(opacities);
    CHECK_INPUT(tile_offsets);
    CHECK_INPUT(flatten_ids);
    if (has(backgrounds)) {
        CHECK_INPUT(backgrounds.value());
    }
    if (masks.has_value()) {
        CHECK_INPUT(masks.value());
    }
    const uint32_t C = (uint32_t)tile_offsets.size(0), N = (uint32_t)means.size(0);
    const uint32_t channels = (uint32_t)colors.size(-1);
    TORCH_CHECK(!has(backgrounds) || (backgrounds->dim() == 2 && backgrounds->size(0) == C &&
                                      backgrounds->size(1) == channels),
                "backgrounds must be [C, channels] = [", C, ", ", channels, "], got ", backgrounds->sizes());
    const int64_t th = tile_size ? (image_height + tile_size - 1) / tile_size : 0;
    const int64_t tw = tile_size ? (image_width + tile_size - 1) / tile_size : 0;
    sized(means, "means", {N, 3});
    sized(quats, "quats", {N, 4});
    sized(scales, "scales", {N, 3});
    sized(colors, "colors", {C, N, channels});
    sized(opacities, "opacities", {C, N});
    sized(tile_offsets, "tile_offsets", {C, th, tw});
    sized(masks, "masks", {C, th, tw});
    check_camera_tensors(C, camera_model, viewmats0, viewmats1, Ks, radial_coeffs, tangential_coeffs,
                         thin_prism_coeffs);
    auto opt = means.options();
    at::Tensor renders = at::empty({C, image_height, image_width, channels}, opt);
    at::Tensor alphas = at::empty({C, image_height, image_width, 1}, opt);
    at::Tensor last_ids = at::empty({C, image_height, image_width}, opt.dtype(at::kInt));
    // records + room for the tile visiting order
    at::Tensor ws = workspace(gsx_raster_records_bytes(N) + gsx_tile_order_bytes((uint32_t)tw, (uint32_t)th), means);
    const int st = gsx_rasterize_to_pixels_from_world_3dgs_fwd(
        C, N, flatten_ids.size(0), means.data_ptr<float>(), quats.data_ptr<float>(), scales.data_ptr<float>(),
        colors.data_ptr<float>(), channels, opacities.data_ptr<float>(), fptr(backgrounds), bptr(masks), image_width,
        image_height, tile_size, viewmats0.data_ptr<float>(), fptr(viewmats1), Ks.data_ptr<float>(), (int)camera_model,
        to_gsx(ut_params), (int)rs_type, fptr(radial_coeffs), fptr(tangential_coeffs), fptr(thin_prism_coeffs),
        tile_offsets.data_ptr<int32_t>(), flatten_ids.data_ptr<int32_t>(), renders.data_ptr<float>(),
        alphas.data_ptr<float>(), last_ids.data_ptr<int32_t>(), ws.data_ptr(), (size_t)ws.numel(), cur_stream(means));
    TORCH_CHECK(st != GSX_ERR_UNSUPPORTED || channels_built(channels), "Unsupported number of channels: ",
                channels); // Rasterization.cpp:126-127
    gsx_check(st);
    return std::make_tuple(renders, alphas, last_ids);
}

std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor> rasterize_to_pixels_from_world_3dgs_bwd(
    const at::Tensor means, const at::Tensor quats, const at::Tensor scales, const at::Tensor colors,
    const at::Tensor opacities, const OptT backgrounds, const OptT masks, const uint32_t image_width,
    const uint32_t image_height, const uint32_t tile_size, const at::Tensor viewmats0, const OptT viewmats1,
    const at::Tensor Ks, const CameraModelType camera_model, const UnscentedTransformParameters ut_params,
    ShutterType rs_type, const OptT radial_coeffs, const OptT tangential_coeffs, const OptT thin_prism_coeffs,
    const at::Tensor tile_offsets, const at::Tensor flatten_ids, const at::Tensor render_alphas,
    const at::Tensor last_ids, const at::Tensor v_render_colors, const at::Tensor v_render_alphas) {
    DEVICE_GUARD(means);
    CHECK_INPUT(means);
    CHECK_INPUT(quats);
    CHECK_INPUT(scales);
    CHECK_INPUT(colors);
    CHECK_INPUT(opacities);
    CHECK_INPUT(tile_offsets);
    CHECK_INPUT(flatten_ids);
    CHECK_INPUT(render_alphas);
    CHECK_INPUT(last_ids);
    CHECK_INPUT(v_render_colors);
    CHECK_INPUT(v_render_alphas);
    if (has(backgrounds)) {
        CHECK_INPUT(backgrounds.value());
    }
    if (masks.has_value()) {
        CHECK_INPUT(masks.value());
    }
    const uint32_t channels = (uint32_t)colors.size(-1);
    TORCH_CHECK(channels_built(channels), "Unsupported number of channels: ", channels);
    TORCH_CHECK(!has(backgrounds) || (backgrounds->dim() == 2 && backgrounds->size(0) == tile_offsets.size(0) &&
                                      backgrounds->size(1) == channels),
                "backgrounds must be [C, channels] = [", tile_offsets.size(0), ", ", channels, "], got ",
                backgrounds->sizes());
    const uint32_t C = (uint32_t)tile_offsets.size(0), N = (uint32_t)means.size(0);
    const int64_t th = tile_size ? (image_height + tile_size - 1) / tile_size : 0;
    const int64_t tw = tile_size ? (image_width + tile_size - 1) / tile_size : 0;
    sized(means, "means", {N, 3});
    sized(quats, "quats", {N, 4});
    sized(scales, "scales", {N, 3});
    sized(colors, "colors", {C, N, channels});
    sized(opacities, "opacities", {C, N});
    sized(tile_offsets, "tile_offsets", {C, th, tw});
    sized(masks, "masks", {C, th, tw});
    sized(render_alphas, "render_alphas", {C, image_height, image_width, 1});
    sized(last_ids, "last_ids", {C, image_height, image_width});
    sized(v_render_colors, "v_render_colors", {C, image_height, image_width, channels});
    sized(v_render_alphas, "v_render_alphas", {C, image_height, image_width, 1});
    check_camera_tensors(C, camera_model, viewmats0, viewmats1, Ks, radial_coeffs, tangential_coeffs,
                         thin_prism_coeffs);
    // the kernels write every element of the five outputs (the reference zero-fills, Rasterization.cpp:190-194)
    at::Tensor v_means = at::empty_like(means), v_quats = at::empty_like(quats), v_scales = at::empty_like(scales);
    at::Tensor v_colors = at::empty_like(colors), v_opacities = at::empty_like(opacities);
    at::Tensor ws = workspace(gsx_rasterize_bwd_workspace_bytes_for(N, channels) +
                                  gsx_tile_order_bytes((uint32_t)tw, (uint32_t)th),
                              means); // + room for the tile visiting order
    gsx_check(gsx_rasterize_to_pixels_from_world_3dgs_bwd(
        C, N, flatten_ids.size(0), means.data_ptr<float>(), quats.data_ptr<float>(), scales.data_ptr<float>(),
        colors.data_ptr<float>(), channels, opacities.data_ptr<float>(), fptr(backgrounds), bptr(masks), image_width,
        image_height, tile_size, viewmats0.data_ptr<float>(), fptr(viewmats1), Ks.data_ptr<float>(), (int)camera_model,
        to_gsx(ut_params), (int)rs_type, fptr(radial_coeffs), fptr(tangential_coeffs), fptr(thin_prism_coeffs),
        tile_offsets.data_ptr<int32_t>(), flatten_ids.data_ptr<int32_t>(), render_alphas.data_ptr<float>(),
        last_ids.data_ptr<int32_t>(), v_render_colors.data_ptr<float>(), v_render_alphas.data_ptr<float>(),
        v_means.data_ptr<float>(), v_quats.data_ptr<float>(), v_scales.data_ptr<float>(), v_colors.data_ptr<float>(),
        v_opacities.data_ptr<float>(), ws.data_ptr(), (size_t)ws.numel(), cur_stream(means)));
    return std::make_tuple(v_means, v_quats, v_scales, v_colors, v_opacities);
}


namespace {

// ---------------------------------------------------------------------------------------------------------------
// The training camera's path through the two fused operators (one perfect pinhole, global shutter, RGB, no
// compensations): the sequence gs::training::rasterize reaches every iteration (rasterizer.cpp:138-166).  Same
// results as the general composition below, with what the reference allocates, recomputes and waits for per call
// kept between calls instead:
//  - scratch (tile-list workspace, backward accumulators, the pinned count slot, a second stream) lives in a
//    StepScratch per (device, stream);
//  - the pair count stays on the device until everything up to the rasterizer is queued (Intersect.cpp:76 blocks on
//    it before the emission can even be sized);
//  - the raster records and the per-tile costs of the forward pass ride in the storage of the `colors` output, so the
//    backward pass that gets `colors` back finds them there (weak reference to the storage: no stale hits).
// ---------------------------------------------------------------------------------------------------------------
struct StepScratch {
    int device = -1;
    void* stream = nullptr;
    std::mutex busy;  // one call at a time per (device, stream); other streams have their own scratch
    uint32_t N = 0, tw = 0, th = 0;
    int64_t cap = 0;
    at::Tensor lists_ws, pinned, accum, order;
    uint32_t accum_N = 0;
    hipStream_t side = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
};

std::mutex g_scratch_mutex;
std::vector<std::unique_ptr<StepScratch>> g_scratch;

StepScratch& scratch_for(const at::Tensor& like, void* stream) {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    const int dev = like.device().index();
    for (auto& s : g_scratch)
        if (s->device == dev && s->stream == stream)
            return *s;
    auto s = std::make_unique<StepScratch>();
    s->device = dev;
    s->stream = stream;
    s->side = c10::hip::getStreamFromPool(/*isHighPriority=*/false, (c10::DeviceIndex)dev).stream();
    TORCH_CHECK(hipEventCreateWithFlags(&s->fork, hipEventDisableTiming) == hipSuccess &&
                    hipEventCreateWithFlags(&s->join, hipEventDisableTiming) == hipSuccess,
                "gsx: hipEventCreate failed");
    s->pinned = at::empty({1}, at::TensorOptions().dtype(at::kLong).pinned_memory(true));
    g_scratch.push_back(std::move(s));
    return *g_scratch.back();
}

// what a forward pass left in the storage behind its `colors` output
struct ForwardExtras {
    c10::weak_intrusive_ptr<c10::StorageImpl> storage;
    uint32_t N, W, H, tw, th;
    int64_t records_at, walk_at;  // float offsets into the storage
    const void *means, *viewmat, *K;
};
std::mutex g_extras_mutex;
std::deque<ForwardExtras> g_extras;

void remember_extras(ForwardExtras e) {
    std::lock_guard<std::mutex> lock(g_extras_mutex);
    g_extras.erase(std::remove_if(g_extras.begin(), g_extras.end(), [](const ForwardExtras& x) { return x.storage.expired(); }),
                   g_extras.end());
    if (g_extras.size() >= 16)
        g_extras.pop_front();
    g_extras.push_back(std::move(e));
}

std::optional<ForwardExtras> find_extras(const at::Tensor& colors) {
    if (!colors.defined() || !colors.has_storage())
        return std::nullopt;
    const c10::StorageImpl* impl = colors.storage().unsafeGetStorageImpl();
    std::lock_guard<std::mutex> lock(g_extras_mutex);
    for (auto it = g_extras.rbegin(); it != g_extras.rend(); ++it)
        if (it->storage._unsafe_get_target() == impl && !it->storage.expired())
            return *it;
    return std::nullopt;
}

inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

// the pair count of gsx_tile_lists, once it has landed in the pinned slot
int64_t await_count(const at::Tensor& pinned, void* stream) {
    volatile int64_t* slot = pinned.data_ptr<int64_t>();
    for (int i = 0; i < 4000000; ++i) {
        const int64_t n = *slot;
        if (n >= 0)
            return n;
    }
    TORCH_CHECK(hipStreamSynchronize((hipStream_t)stream) == hipSuccess, "gsx: hipStreamSynchronize failed");
    return *slot;
}

bool training_camera(const at::Tensor& viewmats0, const gsplat::OptT& viewmats1, const gsplat::OptT& masks,
                     gsplat::CameraModelType camera_model, ShutterType rs_type, const gsplat::OptT& radial,
                     const gsplat::OptT& tangential, const gsplat::OptT& thin_prism, bool calc_compensations,
                     int render_mode, uint32_t tile_size, uint32_t tile_width, uint32_t tile_height) {
    (void)masks;
    return viewmats0.size(0) == 1 && !has(viewmats1) && camera_model == gsplat::PINHOLE && rs_type == ShutterType::GLOBAL &&
           !has(radial) && !has(tangential) && !has(thin_prism) && !calc_compensations && render_mode == 0 &&
           tile_size == 16 && gsx_intersect_tile_pairs_fit(tile_width, tile_height);
}

} // namespace

// The fused operators hand the caller's background ([C,3] from gs::training::rasterize, rasterizer.cpp:84-87, 147)
// to a kernel that blends `channels` values per pixel (Rasterization.cpp:401-407): with RGB + depth it would read one
// float past each row.  Here the missing channels' background is 0 and surplus ones are dropped (for one camera the
// values the reference's kernel reads).
static OptT fit_backgrounds(const OptT& backgrounds, int64_t channels) {
    if (!backgrounds.has_value() || !backgrounds->defined() || backgrounds->numel() == 0)
        return at::nullopt;
    const at::Tensor& b = backgrounds.value();
    const int64_t have = b.size(-1);
    if (have > channels)
        return b.slice(-1, 0, channels).contiguous();
    if (have < channels) {
        auto shape = b.sizes().vec();
        shape.back() = channels - have;
        return at::cat({b, at::zeros(shape, b.options())}, -1).contiguous();
    }
    return b;
}

std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor,
           at::Tensor>
rasterize_from_world_with_sh_fwd(const at::Tensor means, const at::Tensor quats, const at::Tensor scales,
                                 const at::Tensor opacities, const at::Tensor sh_coeffs, const uint32_t sh_degree,
                                 const OptT backgrounds, const OptT masks, const uint32_t image_width,
                                 const uint32_t image_height, const uint32_t tile_size, const at::Tensor viewmats0,
                                 const OptT viewmats1, const at::Tensor Ks, const CameraModelType camera_model,
                                 const float eps2d, const float near_plane, const float far_plane,
                                 const float radius_clip, const float scaling_modifier, const bool calc_compensations,
                                 const int render_mode, const UnscentedTransformParameters ut_params,
                                 ShutterType rs_type, const OptT radial_coeffs, const OptT tangential_coeffs,
                                 const OptT thin_prism_coeffs) {
    DEVICE_GUARD(means);
    CHECK_INPUT(means);
    CHECK_INPUT(quats);
    CHECK_INPUT(scales);
    CHECK_INPUT(opacities);
    CHECK_INPUT(sh_coeffs);
    CHECK_INPUT(viewmats0);
    CHECK_INPUT(Ks);
    TORCH_CHECK(render_mode >= 0 && render_mode <= 4, "render_mode ", render_mode, ": must be 0 .. 4");
    const uint32_t N = (uint32_t)means.size(0), C = (uint32_t)viewmats0.size(0);
    at::Tensor op_flat = opacities.reshape({-1});
    at::Tensor scaled_scales = scaling_modifier == 1.0f ? scales : at::mul(scales, scaling_modifier); // Rasterization.cpp:327
    auto proj = projection_ut_3dgs_fused(means, quats, scaled_scales, op_flat, viewmats0, viewmats1, Ks, image_width,
                                         image_height, eps2d, near_plane, far_plane, radius_clip, calc_compensations,
                                         camera_model, ut_params, rs_type, radial_coeffs, tangential_coeffs,
                                         thin_prism_coeffs);
    at::Tensor radii = std::get<0>(proj), means2d = std::get<1>(proj), depths = std::get<2>(proj);
    at::Tensor compensations = std::get<4>(proj);
    const uint32_t tile_width = (image_width + tile_size - 1) / tile_size;
    const uint32_t tile_height = (image_height + tile_size - 1) / tile_size;
    if (N > 0 && image_width > 0 && image_height > 0 &&
        training_camera(viewmats0, viewmats1, masks, camera_model, rs_type, radial_coeffs, tangential_coeffs,
                        thin_prism_coeffs, calc_compensations, render_mode, tile_size, tile_width, tile_height)) {
        sized(sh_coeffs, "sh_coeffs", {N, -1, 3});
        const OptT bg = fit_backgrounds(backgrounds, 3);
        TORCH_CHECK(!has(bg) || (bg->dim() == 2 && bg->size(0) == 1), "backgrounds must be [C, channels], got ",
                    bg->sizes());
        sized(masks, "masks", {1, tile_height, tile_width});
        void* stream = cur_stream(means);
        StepScratch& sc = scratch_for(means, stream);
        std::lock_guard<std::mutex> busy(sc.busy);
        const uint32_t tiles = tile_width * tile_height;
        // colours | raster records | per-tile walk lengths in one storage: the backward pass finds the last two
        // behind the colours it is handed back
        const int64_t records_at = round_up(3 * (int64_t)N, 64);
        const int64_t walk_at = records_at + (int64_t)(gsx_raster_records_bytes(N) / 4);
        at::Tensor pack = at::empty({walk_at + tiles}, means.options());
        at::Tensor colors = pack.narrow(0, 0, 3 * (int64_t)N).view({1, (int64_t)N, 3});
        float* records = pack.data_ptr<float>() + records_at;
        uint32_t* walk = reinterpret_cast<uint32_t*>(pack.data_ptr<float>() + walk_at);
        auto hip_ok = [](hipError_t e) { TORCH_CHECK(e == hipSuccess, "gsx: ", hipGetErrorString(e)); };
        hip_ok(hipEventRecord(sc.fork, (hipStream_t)stream));
        hip_ok(hipStreamWaitEvent(sc.side, sc.fork, 0));
        // SH colours + records beside the (latency-bound) tile lists
        gsx_check(gsx_sh_colors_records_from_world(N, (uint32_t)sh_coeffs.size(1), sh_degree, means.data_ptr<float>(),
                                                   quats.data_ptr<float>(), scaled_scales.data_ptr<float>(),
                                                   op_flat.data_ptr<float>(), sh_coeffs.data_ptr<float>(),
                                                   radii.data_ptr<int32_t>(), viewmats0.data_ptr<float>(),
                                                   Ks.data_ptr<float>(), image_width, image_height,
                                                   colors.data_ptr<float>(), records, sc.side));
        hip_ok(hipEventRecord(sc.join, sc.side));
        auto opt = means.options();
        at::Tensor renders = at::empty({1, image_height, image_width, 3}, opt);
        at::Tensor alphas = at::empty({1, image_height, image_width, 1}, opt);
        at::Tensor last_ids = at::empty({1, image_height, image_width}, opt.dtype(at::kInt));
        at::Tensor flat, offsets_full;
        int64_t n = 0;
        for (int attempt = 0;; ++attempt) {
            if (sc.cap == 0)
                sc.cap = 1 << 20;
            if (sc.N != N || sc.tw != tile_width || sc.th != tile_height || !sc.lists_ws.defined()) {
                const size_t bytes = gsx_tile_lists_workspace_bytes(N, sc.cap, tile_width, tile_height);
                sc.lists_ws = workspace(bytes, means);
                gsx_check(gsx_tile_lists_init(N, sc.cap, tile_width, tile_height, sc.lists_ws.data_ptr(),
                                              (size_t)sc.lists_ws.numel(), stream));
                sc.order = at::empty({(int64_t)tiles}, opt.dtype(at::kInt));
                sc.N = N, sc.tw = tile_width, sc.th = tile_height;
            }
            flat = at::empty({sc.cap}, opt.dtype(at::kInt));
            offsets_full = at::empty({(int64_t)tiles + 1}, opt.dtype(at::kInt));
            *sc.pinned.data_ptr<int64_t>() = -1;
            gsx_check(gsx_tile_lists(N, means2d.data_ptr<float>(), radii.data_ptr<int32_t>(), depths.data_ptr<float>(),
                                     tile_size, tile_width, tile_height, sc.cap, sc.lists_ws.data_ptr(),
                                     (size_t)sc.lists_ws.numel(), flat.data_ptr<int32_t>(),
                                     offsets_full.data_ptr<int32_t>(), sc.pinned.data_ptr<int64_t>(), stream, sc.side));
            gsx_check(gsx_tile_order(GSX_COUNT_IN_OFFSETS, offsets_full.data_ptr<int32_t>(), nullptr, tile_width,
                                     tile_height, (uint32_t*)sc.order.data_ptr<int32_t>(), stream));
            if (attempt == 0)
                hip_ok(hipStreamWaitEvent((hipStream_t)stream, sc.join, 0));
            gsx_check(gsx_rasterize_records_fwd(GSX_COUNT_IN_OFFSETS, records, nullptr, 3, fptr(bg), bptr(masks),
                                                image_width, image_height, viewmats0.data_ptr<float>(),
                                                Ks.data_ptr<float>(), offsets_full.data_ptr<int32_t>(),
                                                flat.data_ptr<int32_t>(), (const uint32_t*)sc.order.data_ptr<int32_t>(),
                                                walk, renders.data_ptr<float>(), alphas.data_ptr<float>(),
                                                last_ids.data_ptr<int32_t>(), stream));
            // everything up to the rasterizer is queued: only now does the host look at the count
            n = await_count(sc.pinned, stream);
            TORCH_CHECK(n < (1ll << 31), "gsx: ", n, " intersections do not fit int32 indices (Intersect.cpp:84-85)");
            if (n <= sc.cap) {
                if (n > sc.cap - sc.cap / 10) {  // room for the next call
                    sc.cap = n + n / 4 + 1024;
                    sc.lists_ws = at::Tensor();
                }
                break;
            }
            TORCH_CHECK(attempt == 0, "gsx: tile lists did not fit their buffers twice");
            // the lists did not fit and were left empty: larger buffers (a fresh workspace, whose error word is
            // clear), and the lists and the render once more
            sc.cap = n + n / 4 + 1024;
            sc.lists_ws = at::Tensor();
        }
        ForwardExtras ex{pack.storage().getWeakStorageImpl(), N, image_width, image_height, tile_width, tile_height, records_at, walk_at, means.data_ptr(),
                         viewmats0.data_ptr(), Ks.data_ptr()};
        remember_extras(std::move(ex));
        at::Tensor offsets = offsets_full.narrow(0, 0, tiles).view({1, (int64_t)tile_height, (int64_t)tile_width});
        return std::make_tuple(renders, alphas, radii, means2d, depths, colors, offsets, flat.narrow(0, 0, n), last_ids,
                               compensations);
    }
    at::Tensor colors;
    if (render_mode == 0 || render_mode == 3 || render_mode == 4) {
        // Rasterization.cpp:356-378 in one pass: dirs, radii mask, SH, + 0.5, clamp
        colors = at::empty({C, N, 3}, means.options());
        gsx_check(gsx_sh_colors_from_world(N, (uint32_t)sh_coeffs.size(1), sh_degree, means.data_ptr<float>(),
                                           sh_coeffs.data_ptr<float>(), radii.data_ptr<int32_t>(),
                                           viewmats0.data_ptr<float>(), colors.data_ptr<float>(), cur_stream(means)));
        if (render_mode != 0) // RGB + depth (:385-387)
            colors = at::cat({colors, depths.unsqueeze(-1)}, -1).contiguous();
    } else { // depth only (:389-392)
        colors = depths.unsqueeze(-1).contiguous();
    }
    at::Tensor final_opacities = op_flat.unsqueeze(0);
    if (calc_compensations && compensations.defined() && compensations.numel() > 0)
        final_opacities = at::mul(final_opacities, compensations).contiguous();
    at::Tensor flatten_ids, offsets;
    if (!tile_lists(means2d, radii, depths, tile_size, tile_width, tile_height, &flatten_ids, &offsets)) {
        auto isect = intersect_tile(means2d, radii, depths, at::nullopt, at::nullopt, C, tile_size, tile_width,
                                    tile_height, true);
        flatten_ids = std::get<2>(isect);
        offsets = intersect_offset(std::get<1>(isect), C, tile_width, tile_height);
    }
    auto r = rasterize_to_pixels_from_world_3dgs_fwd(means, quats, scaled_scales, colors, final_opacities.contiguous(),
                                                     fit_backgrounds(backgrounds, colors.size(-1)), masks, image_width, image_height, tile_size,
                                                     viewmats0, viewmats1, Ks, camera_model, ut_params, rs_type,
                                                     radial_coeffs, tangential_coeffs, thin_prism_coeffs, offsets,
                                                     flatten_ids);
    return std::make_tuple(std::get<0>(r), std::get<1>(r), radii, means2d, depths, colors, offsets, flatten_ids,
                           std::get<2>(r), compensations);
}

std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor> rasterize_from_world_with_sh_bwd(
    const at::Tensor means, const at::Tensor quats, const at::Tensor scales, const at::Tensor opacities,
    const at::Tensor sh_coeffs, const uint32_t sh_degree, const OptT backgrounds, const OptT masks,
    const uint32_t image_width, const uint32_t image_height, const uint32_t tile_size, const at::Tensor viewmats0,
    const OptT viewmats1, const at::Tensor Ks, const CameraModelType camera_model, const float eps2d,
    const float near_plane, const float far_plane, const float radius_clip, const float scaling_modifier,
    const bool calc_compensations, const int render_mode, const UnscentedTransformParameters ut_params,
    ShutterType rs_type, const OptT radial_coeffs, const OptT tangential_coeffs, const OptT thin_prism_coeffs,
    const at::Tensor render_alphas, const at::Tensor last_ids, const at::Tensor tile_offsets,
    const at::Tensor flatten_ids, const at::Tensor colors, const at::Tensor radii, const at::Tensor means2d,
    const at::Tensor depths, const at::Tensor compensations, const at::Tensor v_render_colors,
    const at::Tensor v_render_alphas) {
    (void)eps2d, (void)near_plane, (void)far_plane, (void)radius_clip, (void)means2d, (void)depths;
    DEVICE_GUARD(means);
    CHECK_INPUT(means);
    CHECK_INPUT(quats);
    CHECK_INPUT(scales);
    CHECK_INPUT(opacities);
    CHECK_INPUT(sh_coeffs);
    CHECK_INPUT(v_render_colors);
    CHECK_INPUT(v_render_alphas);
    TORCH_CHECK(render_mode >= 0 && render_mode <= 4, "render_mode ", render_mode, ": must be 0 .. 4");
    at::Tensor final_opacities = opacities.reshape({1, -1});
    if (calc_compensations && compensations.defined() && compensations.numel() > 0)
        final_opacities = at::mul(final_opacities, compensations).contiguous();
    at::Tensor scaled_scales = scaling_modifier == 1.0f ? scales : at::mul(scales, scaling_modifier);
    const uint32_t N = (uint32_t)means.size(0);
    const uint32_t tile_width = tile_size ? (image_width + tile_size - 1) / tile_size : 0;
    const uint32_t tile_height = tile_size ? (image_height + tile_size - 1) / tile_size : 0;
    const std::optional<ForwardExtras> found = find_extras(colors);
    if (N > 0 && tile_size == 16 && found && found->N == N && found->W == image_width &&
        found->H == image_height && found->means == means.data_ptr() && found->viewmat == viewmats0.data_ptr() &&
        found->K == Ks.data_ptr() &&
        training_camera(viewmats0, viewmats1, masks, camera_model, rs_type, radial_coeffs, tangential_coeffs,
                        thin_prism_coeffs, calc_compensations, render_mode, tile_size, tile_width, tile_height)) {
        // the forward pass of the same inputs left its records and per-tile costs behind `colors`
        const ForwardExtras& ex = *found;
        CHECK_INPUT(colors);
        CHECK_INPUT(tile_offsets);
        CHECK_INPUT(flatten_ids);
        CHECK_INPUT(render_alphas);
        CHECK_INPUT(last_ids);
        CHECK_INPUT(radii);
        CHECK_INPUT(viewmats0);
        sized(means, "means", {N, 3});
        sized(quats, "quats", {N, 4});
        sized(scales, "scales", {N, 3});
        TORCH_CHECK(opacities.numel() == N, "opacities must hold ", N, " values, got ", opacities.sizes());
        sized(sh_coeffs, "sh_coeffs", {N, -1, 3});
        sized(colors, "colors", {1, N, 3});
        sized(radii, "radii", {1, N, 2});
        sized(tile_offsets, "tile_offsets", {1, tile_height, tile_width});
        sized(masks, "masks", {1, tile_height, tile_width});
        sized(render_alphas, "render_alphas", {1, image_height, image_width, 1});
        sized(last_ids, "last_ids", {1, image_height, image_width});
        sized(v_render_colors, "v_render_colors", {1, image_height, image_width, 3});
        sized(v_render_alphas, "v_render_alphas", {1, image_height, image_width, 1});
        const OptT bg = fit_backgrounds(backgrounds, 3);
        void* stream = cur_stream(means);
        StepScratch& sc = scratch_for(means, stream);
        std::lock_guard<std::mutex> busy(sc.busy);
        const size_t accum_bytes = gsx_rasterize_bwd_accum_bytes(N);
        if (sc.accum_N != N || !sc.accum.defined()) {  // zeroed once: the epilogue leaves the rows it read zeroed
            sc.accum = at::zeros({(int64_t)accum_bytes}, means.options().dtype(at::kByte));
            sc.accum_N = N;
        }
        const uint32_t tiles = tile_width * tile_height;
        if (!sc.order.defined() || sc.order.numel() != tiles)
            sc.order = at::empty({(int64_t)tiles}, means.options().dtype(at::kInt));
        const float* base = static_cast<const float*>(colors.storage().data());
        const float* records = base + ex.records_at;
        const uint32_t* walk = reinterpret_cast<const uint32_t*>(base + ex.walk_at);
        const int64_t n = flatten_ids.size(0);
        gsx_check(gsx_tile_order(n, nullptr, walk, tile_width, tile_height, (uint32_t*)sc.order.data_ptr<int32_t>(),
                                 stream));
        gsx_check(gsx_rasterize_bwd_accumulate(
            1, N, n, records, nullptr, 3, fptr(bg), bptr(masks), image_width, image_height, tile_size,
            viewmats0.data_ptr<float>(), Ks.data_ptr<float>(), tile_offsets.data_ptr<int32_t>(),
            flatten_ids.data_ptr<int32_t>(), (const uint32_t*)sc.order.data_ptr<int32_t>(),
            render_alphas.data_ptr<float>(), last_ids.data_ptr<int32_t>(), v_render_colors.data_ptr<float>(),
            v_render_alphas.data_ptr<float>(), sc.accum.data_ptr(), accum_bytes, stream));
        at::Tensor v_means = at::empty_like(means), v_quats = at::empty_like(quats), v_scales = at::empty_like(scales);
        at::Tensor v_colors = at::empty_like(colors), v_opacities = at::empty_like(opacities);
        gsx_check(gsx_rasterize_bwd_finish(N, means.data_ptr<float>(), quats.data_ptr<float>(),
                                           scaled_scales.data_ptr<float>(), viewmats0.data_ptr<float>(),
                                           sc.accum.data_ptr(), accum_bytes, 1, 3, v_means.data_ptr<float>(),
                                           v_quats.data_ptr<float>(), v_scales.data_ptr<float>(),
                                           v_colors.data_ptr<float>(), v_opacities.data_ptr<float>(), stream));
        at::Tensor v_sh = at::empty_like(sh_coeffs);
        gsx_check(gsx_sh_colors_from_world_bwd(N, (uint32_t)sh_coeffs.size(1), sh_degree, means.data_ptr<float>(),
                                               radii.data_ptr<int32_t>(), viewmats0.data_ptr<float>(),
                                               colors.data_ptr<float>(), v_colors.data_ptr<float>(),
                                               v_sh.data_ptr<float>(), stream));
        if (scaling_modifier != 1.0f)
            v_scales = at::mul(v_scales, scaling_modifier);  // Rasterization.cpp:633
        return std::make_tuple(v_means, v_quats, v_scales, v_opacities, v_sh);
    }
    auto g = rasterize_to_pixels_from_world_3dgs_bwd(means, quats, scaled_scales, colors, final_opacities.contiguous(),
                                                     fit_backgrounds(backgrounds, colors.size(-1)), masks, image_width, image_height, tile_size,
                                                     viewmats0, viewmats1, Ks, camera_model, ut_params, rs_type,
                                                     radial_coeffs, tangential_coeffs, thin_prism_coeffs, tile_offsets,
                                                     flatten_ids, render_alphas, last_ids, v_render_colors,
                                                     v_render_alphas);
    at::Tensor v_sh;
    if (render_mode == 0 || render_mode == 3 || render_mode == 4) {
        at::Tensor rgb = colors, v_rgb = std::get<3>(g);
        if (render_mode != 0) { // the depth channel's gradient is dropped (:587-606)
            rgb = colors.slice(-1, 0, 3).contiguous();
            v_rgb = v_rgb.slice(-1, 0, 3).contiguous();
        }
        v_sh = at::empty_like(sh_coeffs);
        gsx_check(gsx_sh_colors_from_world_bwd((uint32_t)means.size(0), (uint32_t)sh_coeffs.size(1), sh_degree,
                                               means.data_ptr<float>(), radii.data_ptr<int32_t>(),
                                               viewmats0.data_ptr<float>(), rgb.data_ptr<float>(),
                                               v_rgb.data_ptr<float>(), v_sh.data_ptr<float>(), cur_stream(means)));
    } else {
        v_sh = at::zeros_like(sh_coeffs); // :625-629
    }
    at::Tensor v_scales = std::get<2>(g);
    if (scaling_modifier != 1.0f)
        v_scales = at::mul(v_scales, scaling_modifier); // Rasterization.cpp:633
    return std::make_tuple(std::get<0>(g), std::get<1>(g), v_scales, std::get<4>(g), v_sh);
}

} // namespace gsplat

// src/training/kernels/ssim.cu:431-468
std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor> fusedssim(float C1, float C2, at::Tensor& img1,
                                                                     at::Tensor& img2, bool train) {
    const c10::DeviceGuard device_guard(img1.device());
    const int B = (int)img1.size(0), CH = (int)img1.size(1), H = (int)img1.size(2), W = (int)img1.size(3);
    at::Tensor a = img1.contiguous(), b = img2.contiguous();
    at::Tensor ssim_map = at::empty_like(a);
    at::Tensor d1 = train ? at::empty_like(a) : at::empty({0}, a.options());
    at::Tensor d2 = train ? at::empty_like(a) : at::empty({0}, a.options());
    at::Tensor d3 = train ? at::empty_like(a) : at::empty({0}, a.options());
    gsx_check(gsx_fusedssim(B, CH, H, W, C1, C2, a.data_ptr<float>(), b.data_ptr<float>(), ssim_map.data_ptr<float>(),
                            train ? d1.data_ptr<float>() : nullptr, train ? d2.data_ptr<float>() : nullptr,
                            train ? d3.data_ptr<float>() : nullptr, cur_stream(a)));
    return std::make_tuple(ssim_map, d1, d2, d3);
}

// src/training/kernels/ssim.cu:476-510
at::Tensor fusedssim_backward(float C1, float C2, at::Tensor& img1, at::Tensor& img2, at::Tensor& dL_dmap,
                              at::Tensor& dm_dmu1, at::Tensor& dm_dsigma1_sq, at::Tensor& dm_dsigma12) {
    const c10::DeviceGuard device_guard(img1.device());
    const int B = (int)img1.size(0), CH = (int)img1.size(1), H = (int)img1.size(2), W = (int)img1.size(3);
    at::Tensor a = img1.contiguous(), b = img2.contiguous(), g = dL_dmap.contiguous();
    at::Tensor d1 = dm_dmu1.contiguous(), d2 = dm_dsigma1_sq.contiguous(), d3 = dm_dsigma12.contiguous();
    at::Tensor out = at::empty_like(a);
    gsx_check(gsx_fusedssim_backward(B, CH, H, W, C1, C2, a.data_ptr<float>(), b.data_ptr<float>(), g.data_ptr<float>(),
                                     d1.data_ptr<float>(), d2.data_ptr<float>(), d3.data_ptr<float>(),
                                     out.data_ptr<float>(), cur_stream(a)));
    return out;
}

// value of fused_ssim(img1, img2, padding) (include/kernels/fused_ssim.cuh:117-122), no autograd node
at::Tensor fused_ssim_value(at::Tensor img1, at::Tensor img2, const std::string& padding) {
    TORCH_CHECK(padding == "same" || padding == "valid", "fused_ssim: padding must be \"same\" or \"valid\" (got \"",
                padding, "\")");
    if (img1.dim() == 3)
        img1 = img1.unsqueeze(0);
    if (img2.dim() == 3)
        img2 = img2.unsqueeze(0);
    TORCH_CHECK(img1.dim() == 4 && img2.dim() == 4, "fused_ssim expects 4D tensors [N,C,H,W]");
    TORCH_CHECK(img1.sizes() == img2.sizes(), "img1 and img2 must have the same shape");
    img1 = img1.contiguous();
    img2 = img2.contiguous();
    at::Tensor map = std::get<0>(fusedssim(0.01f * 0.01f, 0.03f * 0.03f, img1, img2, false));
    const int64_t h = map.size(2), w = map.size(3);
    if (padding == "valid" && h > 10 && w > 10)
        map = map.slice(2, 5, h - 5).slice(3, 5, w - 5);
    return map.mean();
}

void fast_gs::optimizer::adam_step_wrapper(at::Tensor& param, at::Tensor& exp_avg, at::Tensor& exp_avg_sq,
                                           const at::Tensor& param_grad, const float lr, const float beta1,
                                           const float beta2, const float eps, const float bias_correction1_rcp,
                                           const float bias_correction2_sqrt_rcp) {
    const c10::DeviceGuard device_guard(param.device());
    gsx_check(gsx_adam_step(param.data_ptr<float>(), exp_avg.data_ptr<float>(), exp_avg_sq.data_ptr<float>(),
                            param_grad.data_ptr<float>(), param.numel(), lr, beta1, beta2, eps, bias_correction1_rcp,
                            bias_correction2_sqrt_rcp, cur_stream(param)));
}
