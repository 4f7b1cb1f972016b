"""gsx_radix_sort_pairs_static - the pair sort whose histogram table is an array built into the library, for callers
that cannot allocate - against gsx_radix_sort_pairs (caller's workspace) on the same inputs: keys and values bit for
bit, on two calls in a row of which the second is smaller (the array keeps the first call's contents), and once more
on a size of the other tile class.  Collected last on purpose: the file name sorts after every other test file.
"""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _pairs(n, seed):
    rng = np.random.default_rng(seed)
    depth = rng.integers(0, 1 << 32, max(2, n // 40), dtype=np.uint64)[rng.integers(0, max(2, n // 40), n)]
    tile = rng.integers(0, 4056, n).astype(np.uint64)
    keys = ((tile << np.uint64(32)) | depth).astype(np.int64)  # many exact ties: stability is exercised
    vals = rng.permutation(n).astype(np.int32)
    return keys, vals


def _sort(gsx, cuda, keys, vals, begin_bit, end_bit, static):
    L = gsx._lib
    lib = L.lib()
    n = keys.shape[0]
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    k = [torch.from_numpy(keys).to(cuda), torch.empty(n, dtype=torch.int64, device=cuda)]
    v = [torch.from_numpy(vals).to(cuda), torch.empty(n, dtype=torch.int32, device=cuda)]
    sel = ctypes.c_int(-1)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    if static:
        L.check(lib.gsx_radix_sort_pairs_static(ctypes.c_int64(n), p(k[0]), p(v[0]), p(k[1]), p(v[1]),
                                                ctypes.c_uint32(begin_bit), ctypes.c_uint32(end_bit),
                                                ctypes.byref(sel), stream))
    else:
        ws = torch.empty(lib.gsx_radix_sort_pairs_workspace_bytes(ctypes.c_int64(n)), dtype=torch.uint8, device=cuda)
        L.check(lib.gsx_radix_sort_pairs(ctypes.c_int64(n), p(k[0]), p(v[0]), p(k[1]), p(v[1]),
                                         ctypes.c_uint32(begin_bit), ctypes.c_uint32(end_bit), p(ws),
                                         ctypes.c_size_t(ws.numel()), ctypes.byref(sel), stream))
    torch.cuda.synchronize()
    assert sel.value in (0, 1)
    return k[sel.value].cpu().numpy(), v[sel.value].cpu().numpy(), sel.value


def test_static_sort_equals_workspace_sort(gsx, cuda):
    # 5 M pairs (4096-pair blocks), then 300 k (1024-pair blocks, a different table shape in the same array), then a
    # bit range with an odd number of passes, then a handful of pairs
    for n, seed, bits in ((5_000_000, 1, (0, 45)), (300_000, 2, (0, 45)), (2_500_000, 3, (32, 45)), (77, 4, (0, 64))):
        print(f"static sort: n = {n}, bits {bits}", flush=True)
        keys, vals = _pairs(n, seed)
        ref_k, ref_v, ref_sel = _sort(gsx, cuda, keys, vals, *bits, static=False)
        got_k, got_v, got_sel = _sort(gsx, cuda, keys, vals, *bits, static=True)
        assert got_sel == ref_sel
        assert np.array_equal(got_k, ref_k) and np.array_equal(got_v, ref_v), (n, bits)
        # and the result is a sort at all: keys ascending on the selected bits, ties in input order
        d = (got_k.view(np.uint64) >> np.uint64(bits[0])) & np.uint64((1 << (bits[1] - bits[0])) - 1)
        assert (d[1:] >= d[:-1]).all()


def test_static_sort_rejects_what_does_not_fit(gsx, cuda):
    L = gsx._lib
    lib = L.lib()
    one = ctypes.c_void_p(256)
    sel = ctypes.c_int(5)
    st = lib.gsx_radix_sort_pairs_static(ctypes.c_int64((1 << 24) + 1), one, one, one, one, ctypes.c_uint32(0),
                                         ctypes.c_uint32(45), ctypes.byref(sel), ctypes.c_void_p(None))
    assert st == L.GSX_ERR_WORKSPACE and b"limit" in lib.gsx_last_error() and sel.value == 0
    assert lib.gsx_radix_sort_pairs_static(ctypes.c_int64(0), None, None, None, None, ctypes.c_uint32(0),
                                           ctypes.c_uint32(45), ctypes.byref(sel), ctypes.c_void_p(None)) == L.GSX_OK
