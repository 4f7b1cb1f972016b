"""The gradient / Adam-state parity bars, shared by the GPU tests and the smoke check.

TEST INFRASTRUCTURE ONLY (tests/, __graft_entry__.smoke(), bench.py's parity leg): nothing shipped imports this.

The stated bar is "gradients and Adam state within 1e-3 relative".  Every per-Gaussian gradient is a sum of signed
per-pixel terms, and the reference forms d/d(quat, scale) through v_M = v_grd (x) ray_d + v_gro (x) (ray_o - mean), two
terms ~ (distance / sigma) times larger than their sum (RasterizeToPixelsFromWorld3DGSBwd.cu:300-345), so an fp32
evaluation - the reference's own order first of all - misses 1e-3 relative on the elements that are small by
cancellation.  The float64 evaluation (orc_rasterize_bwd_f64) therefore also returns, per element, BOUND = the same
chain evaluated with every term replaced by its absolute value: u * BOUND (u = 2^-24) is the first-order forward error
of one rounding applied to every term, the textbook scale of what an fp32 evaluation in any order can lose.  Each check

  1. MEASURES the literal bar and prints it: the fraction of elements outside |a - b| <= 1e-3 |b| for
     (GPU | fp32 reference-order checker), (GPU | float64 evaluation) and (fp32 checker | float64 evaluation);
  2. asserts that the GPU misses the float64 value no more often than MISS_RATIO x the fp32 checker does (+ MISS_SLACK
     of the elements, three elements at least: below that the two fractions are a handful of elements each and
     their ratio is noise).  The fp32
     checker rounds every pair as the reference does but adds the pairs up in double, so its fraction is a lower
     bound for any implementation that sums in fp32 (the reference's warp reduction + atomics, or this one);
  3. asserts every element: |gpu - f64| <= 1e-3 |f64| + c * u * BOUND with c = max(COND_MULT, COND_RATIO x the
     smallest c the fp32 checker itself needs on that tensor), and prints both (`need`).  BOUND counts one rounding
     per term; the running transmittance takes one more per list entry walked, which is why the fp32 checker needs
     c of several hundred on the opacity gradients of long lists - and the GPU the same;
  4. asserts the whole tensor: ||gpu - f64|| / ||f64|| <= L2_MULT x the same figure of the fp32 checker (+ L2_EPS,
     four fp32 roundings: a tensor that is exact to rounding as a whole needs no yardstick).

Where no BOUND exists for a tensor, step 3 uses the fp32 checker's own error as the yardstick:
max(FLOOR_MULT * E999, MAX_MULT * EMAX), its 99.9th percentile and maximum |error| against float64 on that tensor.

Measured over every test of the suite (operator tests of all camera models, list lengths around the staging batches,
2 000-entry lists, configurations 1, 3, 4 and 5 at full size, two iterations of the benchmarked path), largest figure of
each kind:
  miss fraction   GPU 1.05 x the fp32 checker's on the step's tensors, 1.21 x on one operator test where both are below
                  1e-3 (quaternions and scales 0.2 - 0.5: the kernel sums k q (x) q per Gaussian and never forms the
                  two large terms, the checker follows the reference and cancels them in fp32 for every pair)
  L2              GPU at most 1.35 x the fp32 checker's on means, quaternions, scales and opacities; colour gradients of
                  stacked faint Gaussians 2.1 x and SH coefficients up to 12 x on tensors whose whole error is 5e-8 and
                  2.6e-7, i.e. two roundings: what L2_EPS is for
  per element     c needed by the GPU within 1.05 x of what the fp32 checker needs (opacity gradients of long lists:
                  710 against 709), and below 1.8 where the checker needs less than 2
The multipliers leave head-room for the order of the atomic additions, which changes from run to run:
MISS_RATIO 1.5, L2_MULT 2, COND_RATIO 1.5 with COND_MULT 4 as the least bar.
"""
import numpy as np

from . import oracle as orc

REL = 1e-3
U32 = 2.0 ** -24
COND_MULT = 4.0
COND_RATIO = 1.5
FLOOR_MULT = 8.0
MAX_MULT = 4.0
L2_MULT = 2.0
L2_EPS = 4 * 1.1920929e-07
MISS_RATIO = 1.5
MISS_SLACK = 2e-4
# The same comparison in its plain form, against the fp32 reference-order checker itself:
#   |gpu - fp32| <= PLAIN_RTOL |fp32| + PLAIN_ATOL_RMS * rms(fp32 tensor over the Gaussians that carry a gradient).
# The absolute term is what the cancellation in the reference's own order costs the CHECKER on the elements that are
# small sums of large terms (the float64 columns of the report show on which side the error lies).
PLAIN_RTOL = 1e-3
PLAIN_ATOL_RMS = 1e-3
PLAIN = []  # (tag + name, needed atol / rms) of every call, for the summary

REPORT = []  # lines for the end-of-session summary (tests/conftest.py prints them)


def report(line):
    REPORT.append(line)
    print(line, flush=True)


def miss_fractions(gpu, o32, f64, rel=REL):
    """fractions of the elements with a non-zero float64 value that lie outside |a - b| <= rel |b|"""
    g, o, t = (np.asarray(x, np.float64).reshape(-1) for x in (gpu, o32, f64))
    live = t != 0
    n = max(int(live.sum()), 1)
    g, o, t = g[live], o[live], t[live]
    return dict(n=n,
                gpu_vs_fp32=float((np.abs(g - o) > rel * np.abs(o)).sum()) / n,
                gpu_vs_f64=float((np.abs(g - t) > rel * np.abs(t)).sum()) / n,
                fp32_vs_f64=float((np.abs(o - t) > rel * np.abs(t)).sum()) / n)


def gradient_bar(tag, name, gpu, o32, f64, bound=None, rel=REL):
    """One gradient tensor (any shape; rows = Gaussians) against its float64 evaluation; bound = the float64
    evaluation's absolute-value chain for the same elements (None: the fp32 checker's own error is the yardstick).
    Returns the absolute floor used (array with a bound, scalar without)."""
    g, o, t = (np.asarray(x, np.float64) for x in (gpu, o32, f64))
    assert g.shape == o.shape == t.shape, (name, g.shape, o.shape, t.shape)
    assert np.isfinite(g).all(), f"{tag}{name}: non-finite gradient"
    rows = t.reshape(t.shape[0], -1)
    seen = np.abs(rows).sum(1) > 0
    assert seen.sum() > 100, f"{tag}{name}: only {int(seen.sum())} Gaussians carry a gradient"
    assert np.all(g.reshape(rows.shape)[~seen] == 0), f"{tag}{name}: gradient on a Gaussian no pixel saw"
    m = miss_fractions(g, o, t, rel)
    ex_g = np.abs(g - t) - rel * np.abs(t)
    ex_o = np.abs(o - t) - rel * np.abs(t)
    nt = np.linalg.norm(t)
    l2g, l2o = float(np.linalg.norm(g - t) / nt), float(np.linalg.norm(o - t) / nt)
    # plain rtol + atol form against the fp32 checker
    live_rows = np.abs(o.reshape(rows.shape)).sum(1) > 0
    rms = float(np.sqrt(np.mean(np.square(o.reshape(rows.shape)[live_rows])))) if live_rows.any() else 0.0
    plain_need = float((np.abs(g - o) - PLAIN_RTOL * np.abs(o)).max()) / max(rms, 1e-300)
    PLAIN.append((f"{tag}{name}", plain_need))
    report(f"{tag}{name:12s} plain form: |gpu - fp32| <= {PLAIN_RTOL:g} |fp32| + atol needs atol = "
           f"{max(plain_need, 0.0):.2e} x rms(fp32) (bar {PLAIN_ATOL_RMS:g}; rms {rms:.3e})")
    assert plain_need <= PLAIN_ATOL_RMS, (f"{tag}{name}: |gpu - fp32 checker| exceeds {PLAIN_RTOL:g} |fp32| + "
                                          f"{PLAIN_ATOL_RMS:g} rms by needing {plain_need:.3e} rms")
    head = (f"{tag}{name:12s} n={m['n']:9d} miss>1e-3: gpu|fp32 {m['gpu_vs_fp32']:.2e} gpu|f64 {m['gpu_vs_f64']:.2e} "
            f"fp32|f64 {m['fp32_vs_f64']:.2e}  need: ")
    tail = f", L2 {l2g / max(l2o, 1e-300):.2f} x fp32's ({l2g:.1e} vs {l2o:.1e})"
    if bound is not None:
        b = np.asarray(bound, np.float64).reshape(t.shape)
        assert (b >= np.abs(t) * (1 - 1e-6)).all(), f"{tag}{name}: the absolute-value chain is below the value"
        ub = np.maximum(U32 * b, 1e-300)
        need_g, need_o = float((ex_g / ub).max()), float((ex_o / ub).max())
        report(head + f"floor {max(need_g, 0.0):.2f} x u BOUND (fp32 checker {max(need_o, 0.0):.2f})" + tail)
        c = max(COND_MULT, COND_RATIO * need_o)
        floor = c * U32 * b
        assert need_g <= c, f"{tag}{name}: an element needs {need_g:.1f} x u BOUND (bar {c:.1f}, fp32 checker {need_o:.1f})"
    else:
        e999 = float(np.quantile(np.abs(o - t).reshape(rows.shape)[seen], 0.999))
        emax = float(np.abs(o - t).max())
        floor = max(FLOOR_MULT * e999, MAX_MULT * emax)
        excess = float(ex_g.max())
        report(head + f"floor {max(excess, 0.0) / max(e999, 1e-300):.2f} x E999 or "
               f"{max(excess, 0.0) / max(emax, 1e-300):.2f} x EMAX" + tail)
        assert excess <= floor, (f"{tag}{name}: excess {excess:.3e} vs max({FLOOR_MULT} x E999 = {FLOOR_MULT * e999:.3e}, "
                                 f"{MAX_MULT} x EMAX = {MAX_MULT * emax:.3e})")
    assert m["gpu_vs_f64"] <= MISS_RATIO * m["fp32_vs_f64"] + max(MISS_SLACK, 3.0 / m["n"]), \
        f"{tag}{name}: {m['gpu_vs_f64']:.3e} of the elements miss 1e-3 against float64, the fp32 checker {m['fp32_vs_f64']:.3e}"
    assert l2g <= L2_MULT * l2o + L2_EPS, f"{tag}{name}: L2 rel {l2g:.3e} (fp32 checker {l2o:.3e})"
    return floor


RASTER_COLUMNS = (("v_means", slice(0, 3)), ("v_quats", slice(3, 7)), ("v_scales", slice(7, 10)),
                  ("v_colors", slice(10, 13)), ("v_opacities", slice(13, 14)))


def f64_raw_gradients(ref):
    """float64 evaluation of the raw-parameter gradients of an OracleTrainStep's last iteration: the float64
    rasterizer backward of the same pairs, then the activation VJPs (splat_data.cpp:271-286) in float64; the SH
    backward is linear in v_colors and runs in the checker on the rounded float64 colours."""
    P = ref.params
    viewmat, K, W, H = ref.cam
    op, scales, quats = ref.act
    renders, alphas, radii, means2d, depths, colors, offsets, flat, last_ids, comp, ids = ref.fwd
    g64, b64 = orc.rasterize_bwd_f64(P["means"], quats, scales, colors, op[None], ref.bg, W, H, 16, viewmat[None],
                                     K[None], offsets, flat, alphas, last_ids, ref.v_render[None],
                                     np.zeros_like(alphas))
    raw_q = P["rotation"].astype(np.float64)
    nq = np.maximum(np.linalg.norm(raw_q, axis=1, keepdims=True), 1e-12)
    qh = raw_q / nq
    vq = g64[:, 3:7]
    o = 1.0 / (1.0 + np.exp(-P["opacity"].astype(np.float64)))
    s = np.exp(P["scaling"].astype(np.float64))
    out = dict(means=g64[:, 0:3].copy(), rotation=(vq - qh * (qh * vq).sum(1, keepdims=True)) / nq,
               scaling=g64[:, 7:10] * s, opacity=g64[:, 13] * o * (1.0 - o))
    # the absolute-value chain through the same VJPs
    bq = b64[:, 3:7]
    bound = dict(means=b64[:, 0:3].copy(), rotation=(bq + np.abs(qh) * (np.abs(qh) * bq).sum(1, keepdims=True)) / nq,
                 scaling=b64[:, 7:10] * s, opacity=b64[:, 13] * o * (1.0 - o))
    if ref.scale_reg > 0:
        out["scaling"] += (np.float64(ref.scale_reg) / s.size) * s
        bound["scaling"] += (np.float64(ref.scale_reg) / s.size) * s
    if ref.opacity_reg > 0:
        out["opacity"] += (np.float64(ref.opacity_reg) / o.size) * o * (1.0 - o)
        bound["opacity"] += (np.float64(ref.opacity_reg) / o.size) * o * (1.0 - o)
    sh_bwd = lambda v: orc.sh_colors_from_world_bwd(
        ref.sh_degree, P["means"], ref.K, radii[0], viewmat, np.ascontiguousarray(colors[0][:, :3]),
        np.ascontiguousarray(v.astype(np.float32))).astype(np.float64)
    out["shs"] = sh_bwd(g64[:, 10:13])
    # every SH gradient element is one product basis x v_colour: its absolute-value chain is |basis| x BOUND
    bound["shs"] = np.abs(sh_bwd(b64[:, 10:13]))
    out["_bound"] = bound
    return out


def step_with_truth(ref, viewmat, K, W, H, gt_chw):
    """one iteration of an OracleTrainStep; returns the float64 raw-parameter gradients of that iteration (taken
    before Adam changes the parameters they are evaluated at)"""
    ref.forward(viewmat, K, W, H)
    ref.loss_and_backward(gt_chw)
    truth = f64_raw_gradients(ref)
    ref.adam()
    return truth


def _groups(ts_lrs, K):
    """(name, tensor key, column slice of the [N, -1] view, learning rate): sh0 and shN are separate parameter groups
    of one [N,K,3] tensor (mcmc.cpp:487-492)"""
    g = [("means", "means", slice(None), ts_lrs["means"]), ("sh0", "shs", slice(0, 3), ts_lrs["sh0"])]
    if K > 1:
        g.append(("shN", "shs", slice(3, 3 * K), ts_lrs["shN"]))
    g += [("scaling", "scaling", slice(None), ts_lrs["scaling"]), ("rotation", "rotation", slice(None), ts_lrs["rotation"]),
          ("opacity", "opacity", slice(None), ts_lrs["opacity"])]
    return g


def check_update_from_identical_state(tag, gpu, ref, truth, prev=None, betas=(0.9, 0.999)):
    """Adam moments and parameters after an iteration that GPU and checker started from IDENTICAL parameters and
    moments.  gpu: dict(params, exp_avg, exp_avg_sq, lrs, grads or None) of numpy arrays; ref: the OracleTrainStep
    after the same iteration; truth: f64_raw_gradients(ref); prev: (exp_avg, exp_avg_sq) dicts BEFORE the iteration
    (None = zeros).

      gradients (when the GPU path materialises them) and exp_avg, read back as the gradient that produced it
      ((m - beta1 m_prev) / (1 - beta1)): gradient_bar, i.e. |. - f64| <= 1e-3 |f64| + F, F = FLOOR_MULT * E999;
      exp_avg_sq: v = beta2 v_prev + (1 - beta2) g^2, so with b = 1e-3 |g| + F the same bar on g reads
      |v - v_f64| <= (1 - beta2) (2 |g| b + b^2) element by element (+ 1e-6 v for the rounding of v itself and the
      smallest normal fp32 number where g^2 underflows);
      parameters: each group against its OWN learning rate: the normalised step m / sqrt(v) changes by at most
      ~ (1e-3 + F / |g|) when g changes within its bar (an element whose gradient is below the noise floor may step
      the other way: 2 lr), plus one rounding of the parameter itself."""
    b1, b2 = betas
    K = ref.K
    floors = {}
    for k in ("means", "shs", "scaling", "rotation", "opacity"):
        t = np.asarray(truth[k], np.float64)
        rows = lambda a: np.asarray(a, np.float64).reshape(t.shape)
        bnd = None if truth.get("_bound") is None else rows(truth["_bound"][k])
        if gpu.get("grads") is not None:
            gradient_bar(tag, "grad " + k, rows(gpu["grads"][k]), rows(ref.grads[k]), t, bnd)
        mp = 0.0 if prev is None else rows(prev[0][k])
        vp = 0.0 if prev is None else rows(prev[1][k])
        # the kernels' own fp32 product beta1 * m_prev, so that a Gaussian without gradient reads back as exactly 0
        bm = 0.0 if prev is None else (np.float32(b1) * np.asarray(prev[0][k], np.float32)).astype(np.float64).reshape(t.shape)
        m_g = (rows(gpu["exp_avg"][k]) - bm) / (1.0 - b1)
        m_o = (rows(ref.exp_avg[k]) - bm) / (1.0 - b1)
        F = gradient_bar(tag, "exp_avg " + k, m_g, m_o, t, bnd)
        floors[k] = F
        v_t = b2 * vp + (1.0 - b2) * t * t
        bar = REL * np.abs(t) + F
        # + the smallest normal fp32 number: g^2 of a gradient below 1e-19 is subnormal or zero in fp32
        allowed = (1.0 - b2) * (2.0 * np.abs(t) * bar + bar * bar) + 1e-6 * v_t + 1.1754944e-38
        err = np.abs(rows(gpu["exp_avg_sq"][k]) - v_t)
        live = v_t != 0
        miss_g = float((err[live] > 2 * REL * v_t[live]).mean())
        miss_o = float((np.abs(rows(ref.exp_avg_sq[k]) - v_t)[live] > 2 * REL * v_t[live]).mean())
        report(f"{tag}{'exp_avg_sq ' + k:20s} miss>2e-3: gpu|f64 {miss_g:.2e} fp32|f64 {miss_o:.2e}  "
               f"worst err / element bar {float((err / np.maximum(allowed, 1e-300)).max()):.2f}")
        assert (err <= allowed).all(), f"{tag}exp_avg_sq {k}: {int((err > allowed).sum())} elements outside the bar"
        assert miss_g <= MISS_RATIO * miss_o + MISS_SLACK, f"{tag}exp_avg_sq {k}"
    for name, k, cols, lr in _groups(gpu["lrs"], K):
        N = ref.params[k].shape[0]
        p_g = np.asarray(gpu["params"][k], np.float64).reshape(N, -1)[:, cols]
        p_o = np.asarray(ref.params[k], np.float64).reshape(N, -1)[:, cols]
        t = np.abs(np.asarray(truth[k], np.float64).reshape(N, -1)[:, cols])
        moved = np.abs(p_g - p_o)
        F = floors[k] if np.isscalar(floors[k]) else np.asarray(floors[k]).reshape(N, -1)[:, cols]
        rel_change = np.minimum(1.0, REL + F / np.maximum(t, 1e-300))
        allowed = 2.1 * lr * rel_change + np.spacing(np.abs(p_o).astype(np.float32)).astype(np.float64)
        seen = t > 0
        q999 = float(np.quantile(moved[seen], 0.999)) if seen.any() else 0.0
        report(f"{tag}{'param ' + name:20s} lr {lr:.2e}: moved vs checker max {moved.max() / lr:.2e} lr, 99.9 % {q999 / lr:.2e} lr, "
               f"worst moved / element bar {float((moved / allowed).max()):.2f}")
        assert (moved <= allowed).all(), f"{tag}param {name}: {int((moved > allowed).sum())} elements outside the bar"
        assert (moved[~seen] == 0).all(), f"{tag}param {name}: a Gaussian without gradient moved"
