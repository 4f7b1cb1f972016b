"""Comparison of one GPU training iteration (TrainStep) with the CPU restatement (OracleTrainStep) that ran the same
iteration from the same state; shared by the reduced-size and the full-size step tests.  The gradient / Adam bars
themselves are in oracle/checks.py."""
import numpy as np

from oracle import checks


def N(t):
    return t.detach().cpu().numpy()


def check_forward_bit_exact(ts, ref, min_isects=10_000):
    """identical inputs on both sides -> bit-exact keys, order, ranges, image"""
    rf = ref.fwd
    assert ts.n_isects == rf[7].shape[0] > min_isects
    assert np.array_equal(N(ts.isect_ids[:ts.n_isects]), rf[10]), "tile keys"
    assert np.array_equal(N(ts.flatten_ids[:ts.n_isects]), rf[7]), "sort order"
    assert np.array_equal(N(ts.offsets), rf[6]), "per-tile ranges"
    assert np.abs(N(ts.render) - rf[0]).max() <= 1e-5
    assert np.array_equal(N(ts.render).view(np.uint32), rf[0].view(np.uint32)), "image bit-exact"
    assert np.array_equal(N(ts.alpha).view(np.uint32), rf[1].view(np.uint32)), "alpha bit-exact"
    assert np.array_equal(N(ts.last_ids), rf[8]), "last ids"


def check_loss(ts, ref):
    loss = [float(x) for x in ts.loss_out.cpu()]
    assert abs(loss[0] - ref.loss[0]) <= 1e-5, (loss, ref.loss)
    assert abs(loss[1] - ref.loss[1]) <= 1e-5, "L1"
    assert abs(loss[2] - ref.loss[2]) <= 1e-5, "SSIM"
    if not ts.fused_loss:  # the two-kernel loss never writes the clamped image
        assert np.array_equal(N(ts.image)[0].view(np.uint32), ref.image.view(np.uint32)), "clamped image"


def gpu_state(ts):
    """what check_update_from_identical_state reads of a TrainStep"""
    d = lambda x: {k: N(v) for k, v in x.items()}
    return dict(params=d(ts.params), exp_avg=d(ts.exp_avg), exp_avg_sq=d(ts.exp_avg_sq), lrs=ts.lrs,
                grads=None if ts.fused_update else d(ts.grads))


def check_first_step(ts, ref, truth, tag="", prev=None):
    """gradients, Adam moments and parameters after an iteration that both sides started from identical state;
    truth = oracle.checks.step_with_truth's float64 gradients of that iteration"""
    v = N(ts.v_render)[0]
    assert np.abs(v - ref.v_render).max() <= 1e-5 * np.abs(ref.v_render).max() + 1e-12
    checks.check_update_from_identical_state(tag, gpu_state(ts), ref, truth, prev)


def check_params_close(ts, ref, steps_done, frac):
    """Iterations that did NOT start from bit-identical state (a second iteration after a toleranced first one): a
    parameter moves by at most ~lr per step; elements whose gradient is rounding noise may step in either direction,
    the 99.9th percentile must agree to `frac` of the group's own step"""
    for name, k, cols, lr in checks._groups(ts.lrs, ref.K):
        n = ref.params[k].shape[0]
        p_a = N(ts.params[k]).reshape(n, -1)[:, cols].astype(np.float64)
        p_b = ref.params[k].reshape(n, -1)[:, cols].astype(np.float64)
        moved = np.abs(p_a - p_b)
        ulp = float(np.spacing(np.float32(np.abs(p_b).max())))
        assert np.quantile(moved, 0.999) <= frac * lr * steps_done + ulp, \
            f"param {name}: 99.9 % {np.quantile(moved, 0.999):.3e} vs lr {lr:.1e}"
        assert moved.max() <= 2.1 * lr * steps_done + ulp, f"param {name}"
