"""qmll_sort_by_type_noalloc (counters in a device array built into the library) against
qmll_sort_by_type (counters in a caller workspace), both through the C ABI: bit-exact, on
two calls in a row of which the second is smaller, so stale counters of the first call
would show.  Also: the size limit is refused on the host."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(L, types, slots, ne):
    dev = torch.device("cuda:0")
    ty = torch.tensor(types, dtype=torch.int32, device=dev)
    sl = torch.tensor(slots, dtype=torch.int32, device=dev)
    A = len(slots)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = []
    # outputs pre-filled with a pattern: every entry must be written by the call
    for which in ("workspace", "noalloc"):
        so = torch.full((max(A, 1),), -7, dtype=torch.int32, device=dev)
        off = torch.full((ne + 1,), -7, dtype=torch.int32, device=dev)
        if which == "workspace":
            nbytes = int(L.qmll_sort_by_type_workspace(A, ne))
            work = torch.empty(max(nbytes // 4, 1), dtype=torch.int32, device=dev)
            rc = L.qmll_sort_by_type(_ptr(ty), _ptr(sl), A, ne, _ptr(work), nbytes, _ptr(so), _ptr(off), stream)
        else:
            rc = L.qmll_sort_by_type_noalloc(_ptr(ty), _ptr(sl), A, ne, _ptr(so), _ptr(off), stream)
        assert rc == 0, L.qmll_last_error()
        torch.cuda.synchronize()
        out.append((so.cpu().numpy()[:A], off.cpu().numpy()))
    return out


def test_noalloc_sort_equals_workspace_sort_on_two_calls_in_a_row():
    from qml_lightning_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(7)
    # first call large (many workgroups' counters), second small and with fewer types
    for A, N, ne in ((70001, 90000, 5), (1000, 1400, 3), (300, 300, 4), (0, 4, 2)):
        print("sort_by_type_noalloc A=%d N=%d ne=%d" % (A, N, ne), flush=True)
        types = rng.integers(-1, ne + 1, N).astype(np.int32)
        slots = np.sort(rng.choice(N, size=A, replace=False)).astype(np.int32)
        (s_ws, o_ws), (s_na, o_na) = _both(L, types, slots, ne)
        assert np.array_equal(o_ws, o_na)
        assert np.array_equal(s_ws, s_na)
        # and both equal the stable counting sort itself
        t_atoms = types[slots]
        known = (t_atoms >= 0) & (t_atoms < ne)
        ref = slots[known][np.argsort(t_atoms[known], kind="stable")]
        assert np.array_equal(s_na[:len(ref)], ref) and (s_na[len(ref):] == 0).all()
        assert np.array_equal(o_na, np.concatenate([[0], np.cumsum(np.bincount(t_atoms[known], minlength=ne))]))


def test_noalloc_sort_refuses_sizes_beyond_its_scratch():
    from qml_lightning_amd import _lib
    L = _lib.lib()
    p = ctypes.c_void_p(256)
    # ceil(A/256)*ne = 4097*32 > 131072 counters
    rc = L.qmll_sort_by_type_noalloc(p, p, 4097 * 256, 32, p, p, None)
    assert rc == _lib.QMLL_ERR_INVALID
    assert b"scratch" in L.qmll_last_error()
    assert L.qmll_sort_by_type_noalloc(p, p, 10, 33, p, p, None) == _lib.QMLL_ERR_INVALID
