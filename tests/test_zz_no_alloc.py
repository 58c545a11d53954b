"""The entry point that allocates nothing (ugk_dedup_static) against the entry point it is a variant of
(ugk_dedup_u32 / ugk_dedup_i64 with a caller-side workspace), through the C-ABI, bit for bit where the interface
defines the bits: the number of distinct keys, the set of distinct keys, and — once both results are put into the one
order that does not depend on which workgroup claimed a key first (ascending key) — the inverse and the first
occurrences.  Two calls in a row, the second with a smaller input; then more, to show that nothing of a call leaks into
the next."""
import ctypes as C
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from ugache_amd import hip  # noqa: E402

if torch.cuda.is_available():
    from gpu_util import dev_bytes, dev_zeros_u32, ptr, sync, to_dev, to_np


def _canonical(keys, uniq, inv, rep, k):
    """(distinct keys ascending, inverse into that order, first occurrence per distinct key in that order)"""
    u = uniq[:k]
    order = np.argsort(u, kind="stable")
    pos = np.empty(k, np.int64)
    pos[order] = np.arange(k)
    assert np.array_equal(u[inv], keys)                      # inverse names each key's distinct key
    assert np.array_equal(keys[rep[:k]], u)                  # a representative holds its key
    assert np.array_equal(inv[rep[:k]], np.arange(k))        # ... and is numbered as itself
    return u[order], pos[inv], rep[:k][order]


def _run_existing(keys, kdtype, ws, ws_bytes, epoch):
    n = len(keys)
    uniq = dev_bytes(max(n, 1) * np.dtype(kdtype).itemsize)
    inv, nu, rep = dev_zeros_u32(n), dev_zeros_u32(1), dev_zeros_u32(n)
    fn = "ugk_dedup_i64" if kdtype == np.int64 else "ugk_dedup_u32"
    d_keys = to_dev(keys)
    hip.call(fn, ptr(d_keys), n, ptr(ws), ws_bytes, epoch, ptr(uniq), ptr(inv), ptr(rep), ptr(nu), None, None)
    sync()
    k = int(to_np(nu, np.uint32)[0])
    return k, to_np(uniq, kdtype), to_np(inv, np.uint32)[:n], to_np(rep, np.uint32)[:n]


def _run_static(keys, kdtype):
    n = len(keys)
    uniq = dev_bytes(max(n, 1) * np.dtype(kdtype).itemsize)
    inv, rep = dev_zeros_u32(n), dev_zeros_u32(n)
    nu = torch.full((1,), 12345, dtype=torch.int32, device="cuda")  # the call clears it itself
    d_keys = to_dev(keys)
    hip.call("ugk_dedup_static", ptr(d_keys), np.dtype(kdtype).itemsize, n, ptr(uniq), ptr(inv), ptr(rep), ptr(nu),
             None, None)
    sync()
    k = int(to_np(nu, np.uint32)[0])
    return k, to_np(uniq, kdtype), to_np(inv, np.uint32)[:n], to_np(rep, np.uint32)[:n]


@pytest.mark.parametrize("kdtype", [np.int64, np.uint32])
def test_static_scratch_dedup_matches_the_workspace_one(kdtype):
    rng = np.random.default_rng(2024)
    space = (1 << 31) if kdtype == np.uint32 else (1 << 40)
    max_keys = 1 << 20
    ws_bytes = hip.lib().ugk_dedup_workspace_bytes(max_keys)
    ws = dev_bytes(ws_bytes, fill=0)
    pool = rng.integers(0, space, size=300_000)
    epoch = 0
    # the first two calls are the contract: a large batch, then a smaller one; the rest alternate sizes and skew
    for n in (700_000, 90_000, max_keys, 1, 257, 500_000, 3):
        keys = pool[rng.integers(0, len(pool), size=n)].astype(kdtype)
        if n == 257:
            keys[:] = keys[0]
        epoch += 1
        k0, u0, i0, r0 = _run_existing(keys, kdtype, ws, ws_bytes, epoch)
        k1, u1, i1, r1 = _run_static(keys, kdtype)
        assert k0 == k1 == len(np.unique(keys)), n
        cu0, ci0, cr0 = _canonical(keys, u0, i0, r0, k0)
        cu1, ci1, cr1 = _canonical(keys, u1, i1, r1, k1)
        assert cu0.tobytes() == cu1.tobytes() == np.unique(keys).tobytes(), n
        assert np.array_equal(ci0, ci1), n
        # which occurrence represents a key is whichever claimed it first: both must name an occurrence of the key
        assert np.array_equal(keys[cr0], keys[cr1]), n
    # an empty batch clears the count and launches nothing else
    nu = torch.full((1,), 7, dtype=torch.int32, device="cuda")
    hip.call("ugk_dedup_static", None, 8, 0, None, None, None, ptr(nu), None, None)
    sync()
    assert int(nu.cpu()[0]) == 0
    # ... also in the pinned word that mirrors it, which still holds the count of the batch before
    from gpu_util import PinnedArray
    host_word = PinnedArray((4,), np.uint32)
    try:
        keys = to_dev(np.array([5, 5, 9], kdtype))
        uniq, inv = dev_bytes(3 * 8), dev_zeros_u32(3)
        hip.call("ugk_dedup_static", ptr(keys), keys.element_size(), 3, ptr(uniq), ptr(inv), None, ptr(nu),
                 host_word.ptr, None)
        sync()
        assert int(host_word.array[0]) == 2
        hip.call("ugk_dedup_static", None, 8, 0, None, None, None, ptr(nu), host_word.ptr, None)
        sync()
        assert int(host_word.array[0]) == 0 and int(nu.cpu()[0]) == 0
    finally:
        sync()
        host_word.free()


def test_static_scratch_dedup_refuses_what_does_not_fit():
    n = (1 << 20) + 1
    keys = torch.zeros(n, dtype=torch.int64, device="cuda")
    out = torch.empty(n, dtype=torch.int64, device="cuda")
    inv, nu = dev_zeros_u32(n), dev_zeros_u32(1)
    with pytest.raises(hip.UgkError, match="exceeds"):
        hip.call("ugk_dedup_static", ptr(keys), 8, n, ptr(out), ptr(inv), None, ptr(nu), None, None)
    with pytest.raises(hip.UgkError, match="4 or 8"):
        hip.call("ugk_dedup_static", ptr(keys), 2, 10, ptr(out), ptr(inv), None, ptr(nu), None, None)
    sync()


def test_static_scratch_dedup_allocates_nothing():
    """device memory in use does not move over a hundred calls (the driver's own count, which sees every hipMalloc)"""
    rng = np.random.default_rng(1)
    n = 200_000
    keys = to_dev(rng.integers(0, 50_000, size=n).astype(np.int64))
    uniq = dev_bytes(n * 8)
    inv, rep, nu = dev_zeros_u32(n), dev_zeros_u32(n), dev_zeros_u32(1)
    hip.call("ugk_dedup_static", ptr(keys), 8, n, ptr(uniq), ptr(inv), ptr(rep), ptr(nu), None, None)
    sync()
    free0, total = C.c_size_t(), C.c_size_t()
    hip.call("ugk_mem_info", C.byref(free0), C.byref(total))
    for _ in range(100):
        hip.call("ugk_dedup_static", ptr(keys), 8, n, ptr(uniq), ptr(inv), ptr(rep), ptr(nu), None, None)
    sync()
    free1 = C.c_size_t()
    hip.call("ugk_mem_info", C.byref(free1), C.byref(total))
    assert free1.value == free0.value
    assert int(to_np(nu, np.uint32)[0]) == len(np.unique(to_np(keys, np.int64)))
