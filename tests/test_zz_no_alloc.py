"""The entry point that allocates nothing (cavs_sgemm_splitk_static) against the entry
point it is a variant of (cavs_sgemm_splitk): bit for bit, on two calls in a row, the
second with a smaller input, so that what the first call left in the built-in scratch
is there when the second runs; and the device's free memory is the same before and after
the calls.  Collected last, so that a failure here hides no other test."""
import numpy as np
import pytest

from cavs_amd import hip, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def g():
    import torch

    assert torch.cuda.is_available(), "these tests need the MI355X"
    import gpuutil

    hip.call("cavs_init", 0)
    return gpuutil


def _product(g, oracle, tA, tB, M, N, K, seed):
    import torch

    r = synth.SplitMix64(seed)
    A = r.bulk_uniform(M * K, -1, 1).reshape((K, M) if tA else (M, K))
    B = r.bulk_uniform(K * N, -1, 1).reshape((N, K) if tB else (K, N))
    C0 = r.bulk_uniform(M * N, -1, 1).reshape(M, N)
    nbytes = hip.lib().cavs_sgemm_splitk_workspace(M, N, K)
    assert 0 < nbytes <= hip.lib().cavs_sgemm_splitk_static_max_bytes(), "the case must split K and fit"
    ws = torch.empty(nbytes // 4, dtype=torch.float32, device="cuda")
    Ad, Bd = g.devf(A), g.devf(B)
    want_d, got_d = g.devf(C0), g.devf(C0)
    print(f"[case] splitk tA={tA} tB={tB} M={M} N={N} K={K} seed={seed}", flush=True)
    g.call("cavs_sgemm_splitk", tA, tB, M, N, K, 1.0, g.P(Ad), A.shape[1], g.P(Bd), B.shape[1], 0.5,
           g.P(want_d), N, g.P(ws), nbytes, g.stream())
    # nothing is allocated by the call: the device reports the same free memory before and after
    # (torch's caching allocator is not involved: the call sees raw pointers only)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    g.call("cavs_sgemm_splitk_static", tA, tB, M, N, K, 1.0, g.P(Ad), A.shape[1], g.P(Bd), B.shape[1], 0.5,
           g.P(got_d), N, g.stream())
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, f"device memory changed across the call: {free_before} -> {free_after} bytes free"
    want, got = g.host(want_d), g.host(got_d)
    np.testing.assert_array_equal(got, want)
    # and the product itself is right (not two equal wrong answers)
    ref = oracle.sgemm(tA, tB, A, B, beta=0.5, Cin=C0)
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-5 * max(1.0, float(np.abs(ref).max())))
    g.release()


def test_static_scratch_entry_point_matches_the_workspace_one_on_two_calls_in_a_row(g, oracle):
    # the deferred weight gradient of the headline batch (X^T * dY, K = all vertices), then a
    # smaller product that reuses the front of the same scratch
    _product(g, oracle, 1, 0, 300, 2048, 2482, seed=11)
    _product(g, oracle, 1, 0, 64, 96, 3000, seed=12)
    # a third, in the NT form
    _product(g, oracle, 0, 1, 192, 256, 1024, seed=13)


def test_static_scratch_entry_point_refuses_what_does_not_fit(g):
    import torch

    M, N, K = 1024, 1024, 16384  # twelve splits of 4 MiB each
    need = hip.lib().cavs_sgemm_splitk_workspace(M, N, K)
    if need <= hip.lib().cavs_sgemm_splitk_static_max_bytes():
        pytest.skip("this shape does not split far enough on this device")
    A = torch.zeros(K, M, device="cuda")
    B = torch.zeros(K, N, device="cuda")
    Cd = torch.zeros(M, N, device="cuda")
    with pytest.raises(hip.CavsError, match="built-in"):
        hip.call("cavs_sgemm_splitk_static", 1, 0, M, N, K, 1.0, A.data_ptr(), M, B.data_ptr(), N, 0.0,
                 Cd.data_ptr(), N, g.stream())
