"""gsx_tile_lists (one call, pair count on the device, one launch per radix pass) against the separate operators
intersect_tile + radix sort + intersect_offset, element for element, and against the CPU checker's stable sort."""
import ctypes

import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def N(t):
    return t.detach().cpu().numpy()


def T(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def inputs(tw, th, n, seed, big=0.0):
    W, H = tw * 16 - 3, th * 16 - 5
    rng = np.random.default_rng(seed)
    means2d = np.stack([rng.uniform(-20, W + 20, n), rng.uniform(-20, H + 20, n)], 1).astype(np.float32)[None]
    radii = rng.integers(0, 40, (1, n, 2)).astype(np.int32)
    radii[0, ::7] = 0
    if big:  # a share of screen-filling footprints: long runs per Gaussian
        k = int(n * big)
        radii[0, 3:3 + k] = rng.integers(200, 900, (k, 2))
    depths = rng.uniform(0.1, 50.0, (1, n)).astype(np.float32)
    if n > 300:
        depths[0, 100:200] = depths[0, 100:101]  # ties: broken by index
    return means2d, radii, depths


class Lists:
    def __init__(self, gsx, cuda, n, tw, th, cap, side=False):
        self.side = torch.cuda.Stream(cuda) if side else None
        from lichtfeld_studio_amd._lib import c_i64, c_p, c_sz, c_u32, check, lib
        self.L, self.check = lib(), check
        self.n, self.tw, self.th, self.cap, self.dev = n, tw, th, cap, cuda
        self.dims = (c_u32(n), c_i64(cap), c_u32(tw), c_u32(th))
        nbytes = self.L.gsx_tile_lists_workspace_bytes(*self.dims)
        self.ws = torch.full((nbytes,), 0x5A, dtype=torch.uint8, device=cuda)  # dirty on purpose
        self.stream = c_p(torch.cuda.current_stream(cuda).cuda_stream)
        check(self.L.gsx_tile_lists_init(*self.dims, c_p(self.ws.data_ptr()), c_sz(nbytes), self.stream))
        self.flat = torch.full((cap,), -1, dtype=torch.int32, device=cuda)
        self.off = torch.full((th * tw + 1,), -1, dtype=torch.int32, device=cuda)
        self.slot = torch.full((1,), -1, dtype=torch.int64).pin_memory()

    def run(self, m, r, d):
        from lichtfeld_studio_amd._lib import c_i64, c_p, c_sz, c_u32
        p = lambda t: c_p(t.data_ptr())
        self.slot[0] = -1
        self.check(self.L.gsx_tile_lists(c_u32(self.n), p(m), p(r), p(d), c_u32(16), c_u32(self.tw), c_u32(self.th),
                                         c_i64(self.cap), p(self.ws), c_sz(self.ws.numel()), p(self.flat), p(self.off),
                                         c_p(self.slot.data_ptr()), self.stream,
                                         c_p(self.side.cuda_stream if self.side is not None else None)))
        torch.cuda.synchronize()
        base = self.ws.data_ptr()
        c_at = self.L.gsx_tile_lists_counts(*self.dims, c_p(base)) - base
        e_at = self.L.gsx_tile_lists_error(*self.dims, c_p(base)) - base
        counts = N(self.ws[c_at:c_at + 16]).view(np.int64)
        err = int(N(self.ws[e_at:e_at + 4]).view(np.uint32)[0])
        return counts, err


@pytest.mark.parametrize("grid,n,big", [((78, 52), 60_000, 0.0), ((255, 255), 20_000, 0.0), ((3, 2), 500, 0.0),
                                        ((16, 16), 1, 0.0), ((16, 16), 9, 0.0), ((78, 52), 300_000, 0.002), ((240, 135), 150_000, 0.001),
                                        ((7, 5), 5000, 0.5)])
def test_tile_lists_match_the_separate_operators(gsx, orc, cuda, grid, n, big):
    ops = gsx.ops
    tw, th = grid
    means2d, radii, depths = inputs(tw, th, n, tw * 1000 + th + n, big)
    m, r, d = T(means2d, cuda), T(radii, cuda), T(depths, cuda)
    _, ids, want_flat = ops.intersect_tile(m, r, d, None, None, 1, 16, tw, th, True)
    want_off = ops.intersect_offset(ids, 1, tw, th)
    ni = want_flat.numel()
    assert ni > 0 or n == 1  # n = 1: a Gaussian without footprint, every list empty
    # the checker's own lists: std::stable_sort on the full (tile << 32 | depth) key
    _, o_ids, o_flat = orc.intersect_tile(means2d, radii, depths, 1, 16, tw, th, sort=True)
    assert np.array_equal(N(want_flat), o_flat)

    lists = Lists(gsx, cuda, n, tw, th, cap=ni + 1000, side=(n % 2 == 0))  # half the cases with a second stream
    for rep in range(3):  # the workspace is left ready for the next call
        counts, err = lists.run(m, r, d)
        assert err == 0 and counts[0] == ni and counts[1] == ni and int(lists.slot[0]) == ni, (rep, counts, err)
        assert np.array_equal(N(lists.flat[:ni]), N(want_flat)), f"flatten_ids, call {rep}"
        assert np.array_equal(N(lists.off[:-1]), N(want_off).reshape(-1)), f"tile_offsets, call {rep}"
        assert int(lists.off[-1]) == ni
        assert (N(lists.flat[ni:]) == -1).all(), "nothing is written beyond the count"
    # a different input through the same workspace (fewer pairs)
    means2d2, radii2, depths2 = inputs(tw, th, n, 7 + n)
    radii2[0, ::2] = 0
    m2, r2, d2 = T(means2d2, cuda), T(radii2, cuda), T(depths2, cuda)
    _, ids2, want_flat2 = ops.intersect_tile(m2, r2, d2, None, None, 1, 16, tw, th, True)
    n2 = want_flat2.numel()
    if n2 and n2 <= lists.cap:
        counts, err = lists.run(m2, r2, d2)
        assert err == 0 and counts[0] == n2
        assert np.array_equal(N(lists.flat[:n2]), N(want_flat2))
        assert np.array_equal(N(lists.off[:-1]), N(ops.intersect_offset(ids2, 1, tw, th)).reshape(-1))


def test_tile_lists_capacity_exceeded_leaves_empty_lists(gsx, cuda):
    """more pairs than the buffers hold: every list empty, the true count reported, bit 0 of the error word set,
    nothing written; the same workspace then serves an input that fits"""
    ops = gsx.ops
    tw, th, n = 40, 30, 30_000
    means2d, radii, depths = inputs(tw, th, n, 11)
    m, r, d = T(means2d, cuda), T(radii, cuda), T(depths, cuda)
    _, ids, want_flat = ops.intersect_tile(m, r, d, None, None, 1, 16, tw, th, True)
    ni = want_flat.numel()
    lists = Lists(gsx, cuda, n, tw, th, cap=ni // 2)
    counts, err = lists.run(m, r, d)
    assert err == 1 and counts[0] == 0 and counts[1] == ni and int(lists.slot[0]) == ni
    assert (N(lists.off) == 0).all() and (N(lists.flat) == -1).all()
    radii2 = radii.copy()
    radii2[0, ::3] = 0
    radii2[0, 1::3] = 0
    r2 = T(radii2, cuda)
    _, ids2, want_flat2 = ops.intersect_tile(m, r2, d, None, None, 1, 16, tw, th, True)
    n2 = want_flat2.numel()
    assert 0 < n2 <= lists.cap
    counts, err = lists.run(m, r2, d)
    assert err == 1, "the error word is sticky"
    assert counts[0] == n2 and np.array_equal(N(lists.flat[:n2]), N(want_flat2))


def test_tile_lists_rejects_what_it_cannot_hold(gsx, cuda):
    from lichtfeld_studio_amd._lib import GsxError, c_i64, c_p, c_sz, c_u32, check, lib
    L = lib()
    with pytest.raises(GsxError, match="255"):
        check(L.gsx_tile_lists_init(c_u32(10), c_i64(10), c_u32(256), c_u32(4), c_p(256), c_sz(1 << 30), c_p(0)))
    with pytest.raises(GsxError, match="capacity"):
        check(L.gsx_tile_lists_init(c_u32(10), c_i64(1 << 30), c_u32(4), c_u32(4), c_p(256), c_sz(1 << 40), c_p(0)))
    with pytest.raises(GsxError, match="workspace"):
        check(L.gsx_tile_lists_init(c_u32(10), c_i64(10), c_u32(4), c_u32(4), c_p(256), c_sz(16), c_p(0)))
