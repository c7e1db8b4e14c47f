"""The SGEMM entry point that allocates nothing (aspen_hip_sgemm_static) against the allocating one
(aspen_hip_sgemm) and the oracle, through the C ABI: two calls in a row, the second on a smaller problem, so that
whatever the first call left in the shared static staging buffer must not leak into the second."""
import numpy as np
import pytest

from aspen_amd import api
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _run(L, fn, M, N, K, act, seed):
    from oracle import cpu
    rng = np.random.default_rng(seed)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((N, K)).astype(np.float32)
    bias = rng.standard_normal(M).astype(np.float32)
    ldc = (M + 3) // 4 * 4
    dA, dB, dC, db = (L.aspen_hip_alloc(x) for x in (A.nbytes, B.nbytes, N * ldc * 4, bias.nbytes))
    assert dA and dB and dC and db
    for d, h in ((dA, A), (dB, B), (db, bias)):
        assert L.aspen_hip_h2d(d, h.ctypes.data, h.nbytes) == 0
    assert fn(M, N, K, dA, K, dB, K, dC, ldc, db, act) == 0, L.aspen_hip_last_error()
    assert L.aspen_hip_sync() == 0
    got = np.zeros((N, ldc), np.float32)
    assert L.aspen_hip_d2h(got.ctypes.data, dC, got.nbytes) == 0
    for d in (dA, dB, dC, db):
        L.aspen_hip_free(d)
    want = cpu.activate(cpu.sgemm_packed(cpu.pack_weight(A), B, M, np.tile(bias, (N, 1))), act)
    return got, want


def test_sgemm_static_matches_the_allocating_entry_point_twice_in_a_row(gpu):
    L = api.lib()
    limit = L.aspen_hip_sgemm_static_max_bytes()
    assert limit == 8 << 20
    # first a problem that fills a good part of the staging buffer, then a smaller one with fewer rows AND a
    # shorter K (its padded rows and the tail of the buffer still hold the first call's data)
    for M, N, K, act, seed in ((300, 200, 1024, 4, 1), (70, 45, 96, 0, 2)):
        print(f"sgemm_static M={M} N={N} K={K}", flush=True)
        assert (M + 127) // 128 * 128 * K * 4 <= limit
        got_static, want = _run(L, L.aspen_hip_sgemm_static, M, N, K, act, seed)
        got_alloc, _ = _run(L, L.aspen_hip_sgemm, M, N, K, act, seed)
        assert np.array_equal(got_static, got_alloc)                     # same kernel, same inputs: bit-identical
        assert H.rel_l2(got_static[:, :M], want) <= H.REL_L2_TOL
        assert (got_static[:, M:] == 0).all()                            # padding rows of C are never written


def test_sgemm_static_refuses_what_does_not_fit(gpu):
    L = api.lib()
    d = L.aspen_hip_alloc(1 << 20)
    # roundup (M, 128) * K * 4 beyond the static buffer: refused before anything is launched
    assert L.aspen_hip_sgemm_static(4096, 64, 4096, d, 4096, d, 4096, d, 4096, None, 0) != 0
    assert b"exceeds the static staging buffer" in L.aspen_hip_last_error()
    assert L.aspen_hip_sgemm_static(64, 64, 33, d, 36, d, 36, d, 64, None, 0) != 0
    assert b"multiple" in L.aspen_hip_last_error()
    assert L.aspen_hip_sync() == 0
    L.aspen_hip_free(d)
