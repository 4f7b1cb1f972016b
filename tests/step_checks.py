"""Comparison of one GPU training iteration (TrainStep) with the CPU restatement (OracleTrainStep) that ran the same
iteration from the same state; shared by the reduced-size and the full-size step tests."""
import numpy as np


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
    assert abs(loss[2] - ref.loss[2]) <= 1e-5, "SSIM"
    assert np.array_equal(N(ts.image)[0].view(np.uint32), ref.image.view(np.uint32)), "clamped image"


def check_first_step(ts, ref, steps_done=1):
    """gradients, Adam moments and parameters after an iteration that started from identical state"""
    v = N(ts.v_render)[0]
    assert np.abs(v - ref.v_render).max() <= 1e-5 * np.abs(ref.v_render).max() + 1e-12
    # raw-parameter gradients: 1e-3 relative with a floor of 1e-3 of the tensor's 99.9th percentile magnitude for
    # the well-conditioned ones; quaternion / scale rows that vanish by cancellation are covered in
    # test_gpu_parity.py against a float64 evaluation
    for k in ("means", "shs", "opacity"):
        a, b = N(ts.grads[k]).reshape(-1), ref.grads[k].reshape(-1)
        floor = 1e-3 * np.quantile(np.abs(b[b != 0]), 0.999)
        err = np.abs(a - b) / (np.abs(b) + floor)
        assert err.max() < 1e-3, f"grad {k}: {err.max():.2e}"
    for k in ("scaling", "rotation"):
        a, b = N(ts.grads[k]), ref.grads[k]
        rel = np.linalg.norm(a - b) / np.linalg.norm(b)
        assert rel < 1e-4, f"grad {k}: L2 rel {rel:.2e}"
    # Adam state and parameters (Adam normalises the step: compare relative to the step size lr)
    for k in ("means", "shs", "scaling", "rotation", "opacity"):
        m_a, m_b = N(ts.exp_avg[k]).reshape(-1), ref.exp_avg[k].reshape(-1)
        floor = 1e-3 * np.quantile(np.abs(m_b[m_b != 0]), 0.999)
        if k in ("means", "shs", "opacity"):
            assert (np.abs(m_a - m_b) / (np.abs(m_b) + floor)).max() < 1e-3, f"exp_avg {k}"
        else:
            assert np.linalg.norm(m_a - m_b) / np.linalg.norm(m_b) < 1e-4, f"exp_avg {k}"
        v_a, v_b = N(ts.exp_avg_sq[k]).reshape(-1), ref.exp_avg_sq[k].reshape(-1)
        assert np.linalg.norm(v_a - v_b) / np.linalg.norm(v_b) < 1e-4, f"exp_avg_sq {k}"
    check_params_close(ts, ref, steps_done, 1e-3)


def check_params_close(ts, ref, steps_done, frac):
    """a parameter moves by at most ~lr per step; elements whose gradient is rounding noise may step in either
    direction, everything else must agree to `frac` of the step"""
    lr = max(ts.lrs.values())
    for k in ("means", "shs", "scaling", "rotation", "opacity"):
        p_a, p_b = N(ts.params[k]).reshape(-1), ref.params[k].reshape(-1)
        moved = np.abs(p_a - p_b)
        assert np.quantile(moved, 0.999) <= frac * lr * steps_done + 1e-7 * np.abs(p_b).max(), f"param {k}"
        assert moved.max() <= 2.1 * lr * steps_done, f"param {k}"
