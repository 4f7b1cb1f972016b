// sanitize_driver.cpp - one small training iteration through the CPU checker's C entry points with every buffer
// allocated on the heap at exactly its documented size, for a build under -fsanitize=address,undefined
// (oracle/build.py --sanitize builds and runs it).  Test infrastructure: an overrun, a misaligned access or
// undefined arithmetic inside the checker aborts the run; the driver itself only checks a few invariants.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

extern "C" {
int orc_projection_ut_3dgs_fused(uint32_t C, uint32_t N, const float* means, const float* quats, const float* scales,
                                 const float* opacities, const float* viewmats0, const float* Ks, uint32_t image_width,
                                 uint32_t image_height, float eps2d, float near_plane, float far_plane,
                                 float radius_clip, float ut_alpha, float ut_beta, float ut_kappa, float ut_margin,
                                 int ut_require_all, int32_t* radii, float* means2d, float* depths, float* conics,
                                 float* compensations);
int orc_intersect_tile_count(uint32_t C, uint32_t N, const float* means2d, const int32_t* radii, uint32_t tile_size,
                             uint32_t tile_width, uint32_t tile_height, int32_t* tiles_per_gauss,
                             int64_t* cum_tiles_per_gauss, int64_t* n_isects);
int orc_intersect_tile_emit(uint32_t C, uint32_t N, const float* means2d, const int32_t* radii, const float* depths,
                            const int64_t* cum_tiles_per_gauss, uint32_t tile_size, uint32_t tile_width,
                            uint32_t tile_height, int64_t* isect_ids, int32_t* flatten_ids);
int orc_intersect_tile_emit_packed(uint32_t nnz, const float* means2d, const int32_t* radii, const float* depths,
                                   const int64_t* camera_ids, const int64_t* cum_tiles_per_gauss, uint32_t tile_size,
                                   uint32_t tile_width, uint32_t tile_height, int64_t* isect_ids, int32_t* flatten_ids);
uint32_t orc_tile_n_bits(uint32_t n_tiles);
int orc_radix_sort_pairs(int64_t n, const int64_t* keys_in, const int32_t* vals_in, uint32_t end_bit,
                         int64_t* keys_out, int32_t* vals_out);
int orc_intersect_offset(int64_t n_isects, const int64_t* isect_ids, uint32_t C, uint32_t tile_width,
                         uint32_t tile_height, int32_t* offsets);
int orc_rasterize_to_pixels_from_world_3dgs_fwd(uint32_t C, uint32_t N, int64_t n_isects, const float* means,
                                                const float* quats, const float* scales, const float* colors,
                                                uint32_t CDIM, const float* opacities, const float* backgrounds,
                                                const uint8_t* masks, uint32_t image_width, uint32_t image_height,
                                                uint32_t tile_size, const float* viewmats0, const float* Ks,
                                                const int32_t* tile_offsets, const int32_t* flatten_ids,
                                                float* render_colors, float* render_alphas, int32_t* last_ids,
                                                int64_t* pairs_evaluated);
int orc_rasterize_to_pixels_from_world_3dgs_bwd(uint32_t C, uint32_t N, int64_t n_isects, const float* means,
                                                const float* quats, const float* scales, const float* colors,
                                                uint32_t CDIM, const float* opacities, const float* backgrounds,
                                                const uint8_t* masks, uint32_t image_width, uint32_t image_height,
                                                uint32_t tile_size, const float* viewmats0, const float* Ks,
                                                const int32_t* tile_offsets, const int32_t* flatten_ids,
                                                const float* render_alphas, const int32_t* last_ids,
                                                const float* v_render_colors, const float* v_render_alphas,
                                                float* v_means, float* v_quats, float* v_scales, float* v_colors,
                                                float* v_opacities);
int orc_rasterize_bwd_f64(uint32_t N, int64_t n_isects, const float* means, const float* quats, const float* scales,
                          const float* colors, const float* opacities, const float* backgrounds, uint32_t image_width,
                          uint32_t image_height, uint32_t tile_size, const float* viewmats0, const float* Ks,
                          const int32_t* tile_offsets, const int32_t* flatten_ids, const float* render_alphas,
                          const int32_t* last_ids, const float* v_render_colors, const float* v_render_alphas,
                          double* grads, double* bound);
int orc_sh_colors_from_world(uint32_t N, uint32_t K, uint32_t degree, const float* means, const float* sh_coeffs,
                             const int32_t* radii, const float* viewmat, float* colors);
int orc_sh_colors_from_world_bwd(uint32_t N, uint32_t K, uint32_t degree, const float* means, const int32_t* radii,
                                 const float* viewmat, const float* colors, const float* v_colors, float* v_coeffs);
int orc_activate_params(uint32_t N, const float* opacity_raw, const float* scaling_raw, const float* rotation_raw,
                        float* opacities, float* scales, float* quats);
int orc_activate_params_bwd(uint32_t N, const float* opacity_raw, const float* scaling_raw, const float* rotation_raw,
                            const float* v_opacities, const float* v_scales, const float* v_quats,
                            float* v_opacity_raw, float* v_scaling_raw, float* v_rotation_raw);
int orc_photometric_loss(uint32_t H, uint32_t W, float lambda_dssim, const float* render_hwc, const float* gt_chw,
                         float* image_chw, double* out, float* v_render_hwc);
int orc_adam_step(float* param, float* exp_avg, float* exp_avg_sq, const float* grad, int64_t n, float lr, float beta1,
                  float beta2, float eps, float bias_correction1_rcp, float bias_correction2_sqrt_rcp);
int orc_relocation(int M, const float* opacities, const float* scales, const int32_t* ratios, const float* binoms,
                   int n_max, float* new_opacities, float* new_scales);
int orc_add_noise(int N, const float* raw_opacities, const float* raw_scales, const float* raw_quats,
                  const float* noise, float* means, float current_lr);
int orc_quats_to_rotmats(int N, const float* quats, float* rotmats);
}

#define CHECK(x)                                                                    \
    do {                                                                            \
        if (!(x)) {                                                                 \
            std::fprintf(stderr, "sanitize_driver: %s failed (line %d)\n", #x, __LINE__); \
            return 1;                                                               \
        }                                                                           \
    } while (0)

int main() {
    const uint32_t N = 3000, K = 16, W = 150, H = 101, tile = 16;  // odd sizes: partial tiles at both edges
    const uint32_t tw = (W + tile - 1) / tile, th = (H + tile - 1) / tile;
    std::mt19937 rng(7);
    std::normal_distribution<float> nrm(0.f, 1.f);
    std::uniform_real_distribution<float> uni(0.f, 1.f);
    std::vector<float> means(3 * N), scaling_raw(3 * N), rotation_raw(4 * N), opacity_raw(N), shs((size_t)N * K * 3);
    for (auto& v : means) v = 0.6f * nrm(rng);
    for (auto& v : scaling_raw) v = -3.0f + 0.6f * nrm(rng);
    for (auto& v : rotation_raw) v = nrm(rng);
    for (auto& v : opacity_raw) v = nrm(rng);
    for (size_t i = 0; i < shs.size(); ++i) shs[i] = (i % (3 * K)) < 3 ? uni(rng) : 0.05f * nrm(rng);
    const float viewmat[16] = {1, 0, 0, 0, 0, 1, 0, 0, 0, 0, 1, 4, 0, 0, 0, 1};
    const float Kmat[9] = {140.f, 0, W * 0.5f, 0, 140.f, H * 0.5f, 0, 0, 1};
    std::vector<float> op(N), scales(3 * N), quats(4 * N);
    CHECK(orc_activate_params(N, opacity_raw.data(), scaling_raw.data(), rotation_raw.data(), op.data(), scales.data(),
                              quats.data()) == 0);
    std::vector<int32_t> radii(2 * N);
    std::vector<float> means2d(2 * N), depths(N), conics(3 * N), comp(N);
    CHECK(orc_projection_ut_3dgs_fused(1, N, means.data(), quats.data(), scales.data(), op.data(), viewmat, Kmat, W, H,
                                       0.3f, 0.01f, 1e4f, 0.f, 0.1f, 2.f, 0.f, 0.1f, 1, radii.data(), means2d.data(),
                                       depths.data(), conics.data(), comp.data()) == 0);
    std::vector<float> colors(3 * N);
    CHECK(orc_sh_colors_from_world(N, K, 3, means.data(), shs.data(), radii.data(), viewmat, colors.data()) == 0);
    std::vector<int32_t> tiles_per(N);
    std::vector<int64_t> cum(N);
    int64_t n_isects = 0;
    CHECK(orc_intersect_tile_count(1, N, means2d.data(), radii.data(), tile, tw, th, tiles_per.data(), cum.data(),
                                   &n_isects) == 0);
    CHECK(n_isects > 1000);
    std::vector<int64_t> ids(n_isects), ids_sorted(n_isects);
    std::vector<int32_t> flat(n_isects), flat_sorted(n_isects), offsets(tw * th);
    CHECK(orc_intersect_tile_emit(1, N, means2d.data(), radii.data(), depths.data(), cum.data(), tile, tw, th,
                                  ids.data(), flat.data()) == 0);
    {
        // the same rows as packed rows of two cameras: the same keys up to the camera bits
        std::vector<int64_t> cams(N), pids(n_isects);
        std::vector<int32_t> pflat(n_isects);
        for (uint32_t i = 0; i < N; ++i)
            cams[i] = i & 1;
        CHECK(orc_intersect_tile_emit_packed(N, means2d.data(), radii.data(), depths.data(), cams.data(), cum.data(),
                                             tile, tw, th, pids.data(), pflat.data()) == 0);
        const int64_t low = (1ll << (32 + orc_tile_n_bits(tw * th))) - 1;
        for (int64_t i = 0; i < n_isects; ++i)
            CHECK((pids[i] & low) == ids[i] && pflat[i] == flat[i] && (pids[i] >> (32 + orc_tile_n_bits(tw * th))) == (flat[i] & 1));
    }
    CHECK(orc_radix_sort_pairs(n_isects, ids.data(), flat.data(), 32 + orc_tile_n_bits(tw * th) + 1, ids_sorted.data(),
                               flat_sorted.data()) == 0);
    CHECK(orc_intersect_offset(n_isects, ids_sorted.data(), 1, tw, th, offsets.data()) == 0);
    const float bg[3] = {0.1f, 0.2f, 0.3f};
    std::vector<float> render((size_t)H * W * 3), alpha((size_t)H * W);
    std::vector<int32_t> last_ids((size_t)H * W);
    int64_t pairs = 0;
    CHECK(orc_rasterize_to_pixels_from_world_3dgs_fwd(1, N, n_isects, means.data(), quats.data(), scales.data(),
                                                      colors.data(), 3, op.data(), bg, nullptr, W, H, tile, viewmat,
                                                      Kmat, offsets.data(), flat_sorted.data(), render.data(),
                                                      alpha.data(), last_ids.data(), &pairs) == 0);
    double a_sum = 0;
    for (float a : alpha) a_sum += a;
    CHECK(a_sum > 0.05 * H * W);
    std::vector<float> gt((size_t)3 * H * W), image((size_t)3 * H * W), v_render((size_t)H * W * 3);
    for (auto& v : gt) v = uni(rng);
    double loss[3];
    CHECK(orc_photometric_loss(H, W, 0.2f, render.data(), gt.data(), image.data(), loss, v_render.data()) == 0);
    CHECK(std::isfinite(loss[0]) && loss[0] > 0);
    std::vector<float> v_alpha((size_t)H * W, 0.f), v_means(3 * N), v_quats(4 * N), v_scales(3 * N), v_colors(3 * N),
        v_op(N);
    CHECK(orc_rasterize_to_pixels_from_world_3dgs_bwd(1, N, n_isects, means.data(), quats.data(), scales.data(),
                                                      colors.data(), 3, op.data(), bg, nullptr, W, H, tile, viewmat,
                                                      Kmat, offsets.data(), flat_sorted.data(), alpha.data(),
                                                      last_ids.data(), v_render.data(), v_alpha.data(), v_means.data(),
                                                      v_quats.data(), v_scales.data(), v_colors.data(),
                                                      v_op.data()) == 0);
    std::vector<double> g64((size_t)N * 14), b64((size_t)N * 14);
    CHECK(orc_rasterize_bwd_f64(N, n_isects, means.data(), quats.data(), scales.data(), colors.data(), op.data(), bg, W,
                                H, tile, viewmat, Kmat, offsets.data(), flat_sorted.data(), alpha.data(),
                                last_ids.data(), v_render.data(), v_alpha.data(), g64.data(), b64.data()) == 0);
    std::vector<float> v_shs(shs.size()), g_op(N), g_sc(3 * N), g_rot(4 * N);
    CHECK(orc_sh_colors_from_world_bwd(N, K, 3, means.data(), radii.data(), viewmat, colors.data(), v_colors.data(),
                                       v_shs.data()) == 0);
    CHECK(orc_activate_params_bwd(N, opacity_raw.data(), scaling_raw.data(), rotation_raw.data(), v_op.data(),
                                  v_scales.data(), v_quats.data(), g_op.data(), g_sc.data(), g_rot.data()) == 0);
    std::vector<float> m1(3 * N, 0.f), m2(3 * N, 0.f);
    CHECK(orc_adam_step(means.data(), m1.data(), m2.data(), v_means.data(), 3 * N, 1.6e-4f, 0.9f, 0.999f, 1e-15f, 10.f,
                        31.6f) == 0);
    const int n_max = 51, M = 200;
    std::vector<float> binoms((size_t)n_max * n_max, 0.f), new_o(M), new_s(3 * M);
    for (int n = 0; n < n_max; ++n)
        for (int k = 0; k <= n; ++k)
            binoms[(size_t)n * n_max + k] = k == 0 ? 1.f : binoms[(size_t)n * n_max + k - 1] * (float)(n - k + 1) / (float)k;
    std::vector<int32_t> ratios(M);
    for (int i = 0; i < M; ++i) ratios[i] = 1 + i % n_max;
    CHECK(orc_relocation(M, op.data(), scales.data(), ratios.data(), binoms.data(), n_max, new_o.data(), new_s.data()) == 0);
    std::vector<float> noise(3 * N);
    for (auto& v : noise) v = nrm(rng);
    CHECK(orc_add_noise((int)N, opacity_raw.data(), scaling_raw.data(), rotation_raw.data(), noise.data(), means.data(),
                        80.f) == 0);
    std::vector<float> rot(9 * N);
    CHECK(orc_quats_to_rotmats((int)N, quats.data(), rot.data()) == 0);
    std::printf("sanitize_driver ok: %lld intersections, %lld pairs evaluated, loss %.6f\n", (long long)n_isects,
                (long long)pairs, loss[0]);
    return 0;
}
