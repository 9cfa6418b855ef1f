"""GPU parity of every op-level entry point of the C ABI against the oracle.
Bit-exact for row movement and index work, fp32 tolerance (1e-4 rel / 1e-5 abs,
the bar of the path) for arithmetic."""
import ctypes as C

import numpy as np
import pytest

from cavs_amd import hip, synth

from tolerance import close

pytestmark = pytest.mark.gpu

_ARITHMETIC = ("sgemm", "colsum", "softmax_xent", "treelstm_gates_fwd", "treelstm_gates_bwd", "lstm_gates_fwd",
               "lstm_gates_bwd", "treefc_fwd", "treefc_bwd", "model_step")


class _InDouble:
    """The oracle with its arithmetic evaluated in double (the ord_* build of the same sources):
    what the fp32 kernels are held to 1e-4 relative / 1e-5 absolute against.  Row movement and
    index work pass through unchanged (they are compared bit for bit)."""

    def __init__(self, oracle):
        self._o = oracle

    def __getattr__(self, name):
        fn = getattr(self._o, name)
        if name in _ARITHMETIC:
            return lambda *a, **k: fn(*a, **{"precise": True, **k})
        return fn


@pytest.fixture
def oracle(oracle):
    return _InDouble(oracle)


@pytest.fixture(scope="module")
def g():
    import torch

    assert torch.cuda.is_available(), "these tests need the MI355X"
    import gpuutil

    hip.call("cavs_init", 0)
    return gpuutil


@pytest.fixture(autouse=True)
def _release_device_temporaries(g):
    yield
    g.release()


def rng(seed):
    return synth.SplitMix64(seed)


# ---------------------------------------------------------------- row movement
@pytest.mark.parametrize("n,w,ld_extra", [(1, 4, 0), (7, 1024, 0), (33, 256, 0), (130, 36, 4),
                                           (50, 37, 3), (5, 2048, 0), (1000, 512, 0),
                                           # few, very wide rows (a flat parameter viewed as one row): split along the columns
                                           (1, 786432, 0), (3, 100003, 1), (2, 65536, 4)])
def test_gather_scatter_zero_copy_rows_bit_exact(g, oracle, n, w, ld_extra):
    r = rng(n * 131 + w)
    rows = 2 * n + 3
    ld = w + ld_extra
    src = r.bulk_normal(rows * ld).reshape(rows, ld)
    ids = (np.floor(r.bulk_uniform(n) * rows)).astype(np.int32)
    ids[::5] = -1  # "no row"
    want = np.zeros((n, w), np.float32)
    ok = ids >= 0
    want[ok] = oracle.gather_rows(src, ids[ok], w=w)
    out = g.zeros(n, w, fill=7.0)
    g.call("cavs_gather_rows", g.P(out), w, g.P(g.devf(src)), ld, g.P(g.devi(ids)), n, w, g.stream())
    np.testing.assert_array_equal(g.host(out), want)

    # scatter: unique destinations so the result is order independent
    perm = np.argsort(r.bulk_uniform(rows))[:n].astype(np.int32)
    perm[1::4] = -1
    inp = r.bulk_normal(n * ld).reshape(n, ld)
    dst0 = r.bulk_normal(rows * w).reshape(rows, w)
    want = dst0.copy()
    ok = perm >= 0
    tmp = np.ascontiguousarray(inp[ok][:, :w])
    oracle.scatter_rows(want, perm[ok], tmp)
    dst = g.devf(dst0)
    g.call("cavs_scatter_rows", g.P(dst), w, g.P(g.devi(perm)), g.P(g.devf(inp)), ld, n, w, g.stream())
    np.testing.assert_array_equal(g.host(dst), want)

    # zero / copy through a leading dimension touch only the [n, w] block
    buf0 = r.bulk_normal(n * ld).reshape(n, ld)
    buf = g.devf(buf0)
    g.call("cavs_zero_rows", g.P(buf), ld, n, w, g.stream())
    want = buf0.copy()
    want[:, :w] = 0
    np.testing.assert_array_equal(g.host(buf), want)
    buf = g.devf(buf0)
    g.call("cavs_copy_rows", g.P(buf), ld, g.P(g.devf(src)), ld, n, w, g.stream())
    want = buf0.copy()
    want[:, :w] = src[:n, :w]
    np.testing.assert_array_equal(g.host(buf), want)
    g.call("cavs_add_rows", g.P(buf), ld, g.P(g.devf(src)), ld, n, w, g.stream())
    want[:, :w] += src[:n, :w]
    np.testing.assert_array_equal(g.host(buf), want)


def test_row_ops_accept_empty_and_reject_bad_shapes(g):
    out = g.zeros(4, 8)
    hip.call("cavs_gather_rows", g.P(out), 8, None, 8, None, 0, 8, g.stream())  # n == 0 is a no-op
    hip.call("cavs_scatter_rows", g.P(out), 8, None, None, 8, 0, 8, g.stream())
    with pytest.raises(hip.CavsError, match="bad shape"):
        hip.call("cavs_gather_rows", g.P(out), 4, g.P(out), 8, g.P(out), 2, 8, g.stream())
    with pytest.raises(hip.CavsError, match="null pointer"):
        hip.call("cavs_gather_rows", g.P(out), 8, None, 8, g.P(out), 2, 8, g.stream())


@pytest.mark.parametrize("n,w,hw", [(1, 8, 4), (9, 1024, 512), (64, 20, 8), (31, 6, 3)])
def test_gather_children(g, oracle, n, w, hw):
    r = rng(n + w)
    rows = 3 * n + 2
    pool = r.bulk_normal(rows * w).reshape(rows, w)
    ids = np.floor(r.bulk_uniform(2 * n) * rows).astype(np.int32)
    if n > 2:
        ids[2:4] = -1
    G = g.zeros(2 * n, w, fill=3.0)
    hs = g.zeros(n, hw, fill=3.0)
    g.call("cavs_gather_children", g.P(G), g.P(hs), g.P(g.devf(pool)), g.P(g.devi(ids)), n, w, hw, g.stream())
    want = np.zeros((2 * n, w), np.float32)
    ok = ids >= 0
    want[ok] = oracle.gather_rows(pool, ids[ok])
    np.testing.assert_array_equal(g.host(G), want)
    np.testing.assert_array_equal(g.host(hs), want[0::2, :hw] + want[1::2, :hw])


# ---------------------------------------------------------------- GEMM
SHAPES = [(13, 17, 29), (1, 64, 64), (200, 256, 64), (128, 128, 16), (129, 131, 300), (77, 2048, 300),
          (300, 1536, 512), (5, 512, 40), (640, 5, 512), (512, 384, 2052),
          # between one and two rounds of resident 64x64 workgroups: the narrow-K-panel variant
          (2482, 2048, 300), (2100, 2050, 70)]


@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_sgemm_matches_oracle(g, oracle, tA, tB, M, N, K):
    r = rng(M * 7 + N * 3 + K + 2 * tA + tB)
    A = r.bulk_uniform(M * K, -1, 1).reshape((K, M) if tA else (M, K))
    B = r.bulk_uniform(N * K, -1, 1).reshape((N, K) if tB else (K, N))
    C0 = r.bulk_uniform(M * N, -1, 1).reshape(M, N)
    want = oracle.sgemm(tA, tB, A, B, alpha=0.5, beta=2.0, Cin=C0)
    Cd = g.devf(C0)
    g.call("cavs_sgemm", tA, tB, M, N, K, 0.5, g.P(g.devf(A)), A.shape[1], g.P(g.devf(B)), B.shape[1],
           2.0, g.P(Cd), N, g.stream())
    close(g.host(Cd), want, "sgemm alpha/beta")
    # beta = 0 must not read C (NaNs in C stay out of the result)
    Cd = g.zeros(M, N, fill=float("nan"))
    g.call("cavs_sgemm", tA, tB, M, N, K, 1.0, g.P(g.devf(A)), A.shape[1], g.P(g.devf(B)), B.shape[1],
           0.0, g.P(Cd), N, g.stream())
    exact = (A.T if tA else A).astype(np.float64) @ (B.T if tB else B).astype(np.float64)
    close(g.host(Cd), exact, "sgemm vs fp64")


@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("M,N,K", [(2900, 2950, 116), (1000, 1100, 4100), (2944, 2944, 128)])
def test_sgemm_on_the_large_tile_with_ragged_edges(g, tA, tB, M, N, K):
    """Shapes that take the 128 x 128 tile (alone, and with K split over workgroups): tiles at the
    ragged edges and the k tail go through the general loads, everything else through the fast part of
    the k loop; each form against the fp64 product."""
    import torch

    r = rng(M + 3 * N + 5 * K + 2 * tA + tB)
    A = r.bulk_uniform(M * K, -1, 1).reshape((K, M) if tA else (M, K))
    B = r.bulk_uniform(N * K, -1, 1).reshape((N, K) if tB else (K, N))
    nbytes = hip.lib().cavs_sgemm_splitk_workspace(M, N, K)
    ws = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device="cuda")
    Cd = g.zeros(M, N + 4, fill=float("nan"))
    Cd[:, N:] = 5.0
    g.call("cavs_sgemm_splitk", tA, tB, M, N, K, 1.0, g.P(g.devf(A)), A.shape[1], g.P(g.devf(B)), B.shape[1], 0.0, g.P(Cd), N + 4,
           g.P(ws), nbytes, g.stream())
    got = g.host(Cd)
    np.testing.assert_array_equal(got[:, N:], 5.0)
    exact = (A.T if tA else A).astype(np.float64) @ (B.T if tB else B).astype(np.float64)
    close(got[:, :N], exact, "large-tile product vs fp64")


def test_sgemm_strided_operands_and_addrows(g, oracle):
    """The shapes the Tree-LSTM backward uses: A is a column block of a wider slab,
    C a column block of the child-gradient slab, plus the per-vertex addend."""
    r = rng(5)
    n, H = 37, 64
    dF = r.bulk_normal(2 * n * H).reshape(2 * n, H)
    Uf = r.bulk_uniform(H * H, -0.3, 0.3).reshape(H, H)
    dhlr = r.bulk_normal(n * H).reshape(n, H)
    dG0 = r.bulk_normal(2 * n * 2 * H).reshape(2 * n, 2 * H)
    dG = g.devf(dG0)
    g.call("cavs_sgemm_addrows", 0, 1, 2 * n, H, H, g.P(g.devf(dF)), H, g.P(g.devf(Uf)), H,
           g.P(g.devf(dhlr)), H, 1, g.P(dG), 2 * H, None, 0, g.stream())
    want = dG0.copy()
    want[:, :H] = oracle.sgemm(0, 1, dF, Uf) + np.repeat(dhlr, 2, axis=0)
    close(g.host(dG), want)
    np.testing.assert_array_equal(g.host(dG)[:, H:], dG0[:, H:])  # c half untouched
    # A = first 3H columns of a [n,4H] slab (lda = 4H)
    dxW = r.bulk_normal(n * 4 * H).reshape(n, 4 * H)
    U = r.bulk_uniform(H * 3 * H, -0.3, 0.3).reshape(H, 3 * H)
    out = g.zeros(n, H)
    g.call("cavs_sgemm", 0, 1, n, H, 3 * H, 1.0, g.P(g.devf(dxW)), 4 * H, g.P(g.devf(U)), 3 * H, 0.0,
           g.P(out), H, g.stream())
    close(g.host(out), oracle.sgemm(0, 1, np.ascontiguousarray(dxW[:, :3 * H]), U))


@pytest.mark.parametrize("M,N,K", [(64, 96, 3000), (300, 2048, 2482), (12, 20, 777), (512, 1536, 64)])
def test_sgemm_splitk_is_deterministic_and_correct(g, oracle, M, N, K):
    import torch

    r = rng(M + N + K)
    A = r.bulk_uniform(K * M, -1, 1).reshape(K, M)  # TN: the weight-gradient form
    B = r.bulk_uniform(K * N, -1, 1).reshape(K, N)
    C0 = r.bulk_uniform(M * N, -1, 1).reshape(M, N)
    nbytes = hip.lib().cavs_sgemm_splitk_workspace(M, N, K)
    ws = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device="cuda")
    outs = []
    for _ in range(2):
        Cd = g.devf(C0)
        g.call("cavs_sgemm_splitk", 1, 0, M, N, K, 1.0, g.P(g.devf(A)), M, g.P(g.devf(B)), N, 1.0,
               g.P(Cd), N, g.P(ws), nbytes, g.stream())
        outs.append(g.host(Cd))
    np.testing.assert_array_equal(outs[0], outs[1])
    exact = A.T.astype(np.float64) @ B.astype(np.float64) + C0
    close(outs[0], exact)
    close(outs[0], oracle.sgemm(1, 0, A, B, beta=1.0, Cin=C0))


GROUPS = {
    # the once-per-step block of the Tree-LSTM backward at the headline shape: de, dW, dU_iou, dU_f
    "treelstm_step": [(0, 1, 2482, 300, 2048), (1, 0, 300, 2048, 2482), (1, 0, 512, 1536, 1241), (1, 0, 512, 512, 2482)],
    # all four forms, ragged edges, one empty product, K below one tile, K not a multiple of 4
    "ragged": [(0, 0, 70, 33, 300), (1, 1, 40, 72, 641), (0, 1, 0, 16, 64), (1, 0, 5, 130, 31)],
    "single": [(1, 0, 64, 96, 3000)],
    # one product large enough for the big tile (it runs by itself) next to two that share a launch
    "mixed": [(1, 0, 1024, 1024, 4096), (0, 1, 700, 512, 2048), (1, 0, 512, 512, 700)],
}


@pytest.mark.parametrize("name", sorted(GROUPS))
def test_sgemm_group_matches_separate_products(g, oracle, name):
    """Several products in one launch: each equals its own fp64 product and the oracle's
    sgemm (alpha, beta honoured), bit-identical when repeated, neighbours untouched."""
    import ctypes as C

    import torch

    shapes = GROUPS[name]
    r = rng(len(name) + 11)
    descs = (hip.GemmDesc * len(shapes))()
    keep, host = [], []
    for p, (tA, tB, M, N, K) in enumerate(shapes):
        A = r.bulk_uniform(max(M * K, 1), -1, 1)[:M * K].reshape((K, M) if tA else (M, K))
        B = r.bulk_uniform(max(N * K, 1), -1, 1)[:N * K].reshape((N, K) if tB else (K, N))
        beta = 0.0 if p % 2 == 0 else 0.5
        C0 = r.bulk_uniform(max(M * (N + 3), 1), -1, 1)[:M * (N + 3)].reshape(M, N + 3)  # ldc = N + 3: a column block of a wider slab
        Ad, Bd = g.devf(A.reshape(-1) if A.size else np.zeros(1)), g.devf(B.reshape(-1) if B.size else np.zeros(1))
        keep += [Ad, Bd]
        host.append((A, B, C0, beta))
        descs[p] = hip.GemmDesc(tA, tB, M, N, K, 1.5, beta, g.P(Ad), max(A.shape[1], 1), g.P(Bd), max(B.shape[1], 1), None, N + 3)
    nbytes = hip.lib().cavs_sgemm_group_workspace(len(shapes), descs)
    ws = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device="cuda")
    runs = []
    for _ in range(2):
        outs = []
        for p, (A, B, C0, beta) in enumerate(host):
            Cd = g.devf(C0 if C0.size else np.zeros(1))
            if beta == 0.0 and C0.size:  # beta = 0 must not read C
                Cd[:, :C0.shape[1] - 3] = float("nan")
            outs.append(Cd)
            descs[p].C = g.P(Cd)
        g.call("cavs_sgemm_group", len(shapes), descs, g.P(ws), nbytes, g.stream())
        runs.append([g.host(o) for o in outs])
    for p, ((tA, tB, M, N, K), (A, B, C0, beta)) in enumerate(zip(shapes, host)):
        if M == 0:
            continue
        got = runs[0][p]
        np.testing.assert_array_equal(got, runs[1][p])
        np.testing.assert_array_equal(got[:, N:], C0[:, N:])  # columns beyond N untouched
        exact = 1.5 * (A.T if tA else A).astype(np.float64) @ (B.T if tB else B).astype(np.float64) + beta * C0[:, :N]
        close(got[:, :N], exact, f"product {p} vs fp64")
        if 2.0 * M * N * K < 2e9:  # the oracle's plain loops take seconds beyond this
            close(got[:, :N], oracle.sgemm(tA, tB, A, B, alpha=1.5, beta=beta, Cin=np.ascontiguousarray(C0[:, :N])), f"product {p} vs oracle")
    with pytest.raises(hip.CavsError, match="at most 8"):
        g.call("cavs_sgemm_group", 9, descs, g.P(ws), nbytes, g.stream())
    if nbytes:
        with pytest.raises(hip.CavsError, match="workspace"):
            g.call("cavs_sgemm_group", len(shapes), descs, g.P(ws), nbytes - 256, g.stream())


# (the 7331-row case runs as lookup + product on the 128 x 128 tile, the others in one launch)
@pytest.mark.parametrize("n,E,N,ld_e,urows,ucol", [(2482, 300, 2048, 304, 1260, 1536), (7331, 512, 2048, 512, 3700, 1536),
                                                   (320, 128, 512, 128, 130, 384), (70, 33, 50, 40, 64, 3), (200, 64, 256, 64, 200, 1)])
def test_pull_lookup_and_product_with_an_unused_block(g, n, E, N, ld_e, urows, ucol):
    """cavs_embed_pull_sgemm with rows below `urows` not wanted from column `ucol` on (the forget-gate
    columns of the leaves): everything else, the looked-up rows and the ids are those of the call
    without the block, bit for bit; inside the block an element is the product or zero, and the
    tiles that lie wholly inside it are zero."""
    V, nx = 211, n + 9
    r = rng(n + E + 1)
    x = np.floor(r.bulk_uniform(nx) * V).astype(np.float32)
    x[::7] = -1.0
    rows = np.argsort(r.bulk_uniform(nx))[:n].astype(np.int32)
    table, B = r.bulk_uniform(V * E, -1, 1).reshape(V, E), r.bulk_uniform(E * N, -1, 1).reshape(E, N)
    d_x, d_rows, d_table, d_B = g.devf(x), g.devi(rows), g.devf(table), g.devf(B)
    res = []
    for ur, uc in ((0, 0), (urows, ucol)):
        e_out, ids_out, Cd = g.devf(np.full((n, ld_e), 9, np.float32)), g.devf(np.full(n, 9, np.float32)), g.devf(np.full((n, N + 4), 9, np.float32))
        g.call("cavs_embed_pull_sgemm", g.P(Cd), N + 4, g.P(e_out), ld_e, g.P(ids_out), g.P(d_x), g.P(d_rows), g.P(d_table), n, E,
               g.P(d_B), N, N, ur, uc, g.stream())
        res.append((g.host(Cd), g.host(e_out), g.host(ids_out)))
    (want, e_want, ids_want), (got, e_got, ids_got) = res
    np.testing.assert_array_equal(e_got, e_want)
    np.testing.assert_array_equal(ids_got, ids_want)
    inside = np.zeros_like(want, dtype=bool)
    inside[:urows, ucol:N] = True
    np.testing.assert_array_equal(got[~inside], want[~inside])
    assert np.all((got[inside] == want[inside]) | (got[inside] == 0))
    # tiles of 128 rows and columns that lie wholly inside the block (whatever tile the plan took)
    r1, c0 = urows // 128 * 128, -(-ucol // 128) * 128
    if r1 > 0 and c0 < N:
        assert not got[:r1, c0:N].any()
    with pytest.raises(hip.CavsError, match="unused block"):
        g.call("cavs_embed_pull_sgemm", g.P(Cd), N + 4, g.P(e_out), ld_e, g.P(ids_out), g.P(d_x), g.P(d_rows), g.P(d_table), n, E,
               g.P(d_B), N, N, -1, 0, g.stream())


HINTED = {
    # the deferred products of a batch of trees whose first 1260 slab rows are leaves: de = dxW * W^T
    # and dW = e^T * dxW, the forget-gate columns of dxW zero in the leaves' rows
    "c3": [(0, 1, 2482, 300, 2048, hip.GEMM_A_ZERO, 1260, 1536), (1, 0, 304, 2048, 2482, hip.GEMM_B_ZERO, 1260, 1536),
           (1, 0, 512, 1536, 1222, 0, 0, 0)],
    # large enough for the 128 x 128 tile, each by itself
    "alone": [(0, 1, 9000, 1024, 2048, hip.GEMM_A_ZERO, 4500, 1536), (1, 0, 1024, 2048, 9000, hip.GEMM_B_ZERO, 4500, 1536)],
    # hints that do not apply (transposed operand, a first zero k that is no multiple of 4) are ignored
    "ignored": [(1, 1, 300, 200, 512, hip.GEMM_A_ZERO, 100, 256), (0, 1, 300, 200, 512, hip.GEMM_A_ZERO, 100, 255),
                (0, 1, 300, 200, 512, hip.GEMM_B_ZERO, 100, 64)],
}


@pytest.mark.parametrize("name", sorted(HINTED))
def test_sgemm_group_with_known_zero_blocks(g, name):
    """Products whose descriptor names a zero block of an operand: bit for bit the results of the
    same products without the hint.  Where the hint applies and the tiles are wholly inside it the
    block is not read at all -- shown by a second run with NaN there (rows below a multiple of 128,
    columns from a multiple of 128 on: inside for every tile shape)."""
    import torch

    shapes = HINTED[name]
    r = rng(len(name) + 23)
    n = len(shapes)
    plain, hinted = (hip.GemmDesc * n)(), (hip.GemmDesc * n)()
    keep, outs, poison = [], [], []
    for p, (tA, tB, M, N, K, kind, zr, zc) in enumerate(shapes):
        A = r.bulk_uniform(M * K, -1, 1).reshape((K, M) if tA else (M, K))
        B = r.bulk_uniform(N * K, -1, 1).reshape((N, K) if tB else (K, N))
        applies = (kind == hip.GEMM_A_ZERO and not tA and zc % 4 == 0) or (kind == hip.GEMM_B_ZERO and not tB)
        Z = A if kind == hip.GEMM_A_ZERO else B
        if applies:
            Z[:zr, zc:] = 0.0
        Ad, Bd = g.devf(A), g.devf(B)
        keep += [Ad, Bd]
        plain[p] = hip.GemmDesc(tA, tB, M, N, K, 1.0, 0.0, g.P(Ad), A.shape[1], g.P(Bd), B.shape[1], None, N)
        hinted[p] = hip.GemmDesc(tA, tB, M, N, K, 1.0, 0.0, g.P(Ad), A.shape[1], g.P(Bd), B.shape[1], None, N, kind, zr, zc)
        # rows of the block every tile shape skips: A rows in whole 128-row tiles; B rows k below a multiple of 32
        skip_rows = zr // 128 * 128 if kind == hip.GEMM_A_ZERO else zr // 32 * 32
        poison.append((Ad if kind == hip.GEMM_A_ZERO else Bd, skip_rows, zc) if applies and zc % 128 == 0 else None)
    nbytes = hip.lib().cavs_sgemm_group_workspace(n, hinted)
    assert nbytes == hip.lib().cavs_sgemm_group_workspace(n, plain)
    ws = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device="cuda")
    results = []
    for descs, nan in ((plain, False), (hinted, False), (hinted, True)):
        if nan:
            for q in poison:
                if q:
                    q[0][:q[1], q[2]:] = float("nan")
        outs = []
        for p, (tA, tB, M, N, K, *_h) in enumerate(shapes):
            Cd = g.devf(np.full((M, N), 7, np.float32))
            outs.append(Cd)
            descs[p].C = g.P(Cd)
        g.call("cavs_sgemm_group", n, descs, g.P(ws), nbytes, g.stream())
        results.append([g.host(o) for o in outs])
    for p in range(n):
        np.testing.assert_array_equal(results[1][p], results[0][p], err_msg=f"product {p}: hinted vs plain")
        np.testing.assert_array_equal(results[2][p], results[0][p], err_msg=f"product {p}: the block was read")
    bad = (hip.GemmDesc * 1)()
    bad[0] = hinted[0]
    bad[0].zero_kind = 4
    with pytest.raises(hip.CavsError, match="block hint"):
        g.call("cavs_sgemm_group", 1, bad, g.P(ws), nbytes, g.stream())


@pytest.mark.parametrize("n,E,N,ld_e", [(2482, 300, 2048, 304), (7331, 512, 2048, 512), (320, 128, 512, 128), (70, 33, 50, 40), (5, 8, 64, 8)])
def test_pull_lookup_and_product_in_one_launch(g, n, E, N, ld_e):
    """cavs_embed_pull_sgemm against cavs_embed_pull_fwd + cavs_sgemm: the product, the looked-up rows
    it leaves behind (padding columns untouched) and the ids, bit for bit; an id below zero reads as a
    zero row."""
    V, nx = 211, n + 9
    r = rng(n + E)
    x = np.floor(r.bulk_uniform(nx) * V).astype(np.float32)
    x[::7] = -1.0
    rows = np.argsort(r.bulk_uniform(nx)).astype(np.int32)[:n]
    table, B = r.bulk_normal(V * E).reshape(V, E), r.bulk_uniform(E * N, -0.1, 0.1).reshape(E, N)
    d_x, d_rows, d_table, d_B = g.devf(x), g.devi(rows), g.devf(table), g.devf(B)
    res = []
    for fused in (False, True):
        e_out, ids_out, Cd = g.devf(np.full((n, ld_e), 9, np.float32)), g.devf(np.full(n, 9, np.float32)), g.devf(np.full((n, N + 4), 9, np.float32))
        if fused:
            g.call("cavs_embed_pull_sgemm", g.P(Cd), N + 4, g.P(e_out), ld_e, g.P(ids_out), g.P(d_x), g.P(d_rows), g.P(d_table), n, E,
                   g.P(d_B), N, N, 0, 0, g.stream())
        else:
            g.call("cavs_embed_pull_fwd", g.P(e_out), ld_e, g.P(ids_out), g.P(d_x), g.P(d_rows), g.P(d_table), n, E, g.stream())
            g.call("cavs_sgemm", 0, 0, n, N, E, 1.0, g.P(e_out), ld_e, g.P(d_B), N, 0.0, g.P(Cd), N + 4, g.stream())
        res.append((g.host(Cd), g.host(e_out), g.host(ids_out)))
    ids = x[rows]
    want_e = np.where(ids[:, None] >= 0, table[np.maximum(ids, 0).astype(np.int64)], 0).astype(np.float32)
    np.testing.assert_array_equal(res[1][1][:, :E], want_e)
    np.testing.assert_array_equal(res[1][1][:, E:], 9)
    np.testing.assert_array_equal(res[1][2], ids)
    np.testing.assert_array_equal(res[1][0][:, N:], 9)
    close(res[1][0][:, :N], want_e.astype(np.float64) @ B.astype(np.float64), "product vs fp64")
    if E >= 64 and n > 1024:  # same tile kernel on both sides (smaller shapes take the skinny kernel when called alone)
        np.testing.assert_array_equal(res[1][0], res[0][0])
    else:
        close(res[1][0][:, :N], res[0][0][:, :N], "fused vs separate")


@pytest.mark.parametrize("name,k", [("treelstm_step", 0), ("ragged", 0), ("single", 0), ("mixed", 1), ("mixed", 0)])
def test_sgemm_group_with_the_embedding_gradient_behind_one_product(g, name, k):
    """cavs_sgemm_group_embed_bwd: the products come out bit for bit as from cavs_sgemm_group (the one
    that feeds the table too, whether its K was split, not split, or it ran alone on the large tile) and
    the table as from cavs_embed_bwd on that product (atomic adds: to the tolerance, in fp64 terms)."""
    import torch

    shapes = GROUPS[name]
    n, E = shapes[k][2], shapes[k][3]
    V = 97
    r = rng(len(name) * 7 + k)
    descs = (hip.GemmDesc * len(shapes))()
    keep = []
    for p, (tA, tB, M, N, K) in enumerate(shapes):
        A = r.bulk_uniform(max(M * K, 1), -1, 1)[:M * K].reshape((K, M) if tA else (M, K))
        B = r.bulk_uniform(max(N * K, 1), -1, 1)[:N * K].reshape((N, K) if tB else (K, N))
        Ad, Bd = g.devf(A.reshape(-1) if A.size else np.zeros(1)), g.devf(B.reshape(-1) if B.size else np.zeros(1))
        keep += [Ad, Bd]
        descs[p] = hip.GemmDesc(tA, tB, M, N, K, 1.0, 0.0, g.P(Ad), max(A.shape[1], 1), g.P(Bd), max(B.shape[1], 1), None, N + 4)
    ids = np.floor(r.bulk_uniform(max(n, 1)) * V).astype(np.float32)[:n]
    ids[:n // 2] = 3.0  # one row looked up by half of the vertices, as in a batch of parse trees
    d_ids = g.devf(ids if n else np.zeros(1))
    table0 = r.bulk_normal(V * E).reshape(V, E)
    nbytes = hip.lib().cavs_sgemm_group_workspace(len(shapes), descs)
    ws = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device="cuda")
    res = []
    for combined in (False, True):
        outs = [torch.full((max(M, 1), N + 4), float("nan"), dtype=torch.float32, device="cuda") for (_, _, M, N, _) in shapes]
        for p, o in enumerate(outs):
            descs[p].C = g.P(o)
        table = g.devf(table0)
        if combined:
            g.call("cavs_sgemm_group_embed_bwd", len(shapes), descs, k, g.P(table), g.P(d_ids), g.P(ws), nbytes, g.stream())
        else:
            g.call("cavs_sgemm_group", len(shapes), descs, g.P(ws), nbytes, g.stream())
            g.call("cavs_embed_bwd", g.P(table), g.P(d_ids), g.P(outs[k]), E + 4, n, E, g.stream())
        res.append(([g.host(o) for o in outs], g.host(table)))
    for p, (_, _, M, N, _) in enumerate(shapes):
        if M:
            np.testing.assert_array_equal(res[0][0][p][:, :N], res[1][0][p][:, :N])
    if n:
        want = table0.astype(np.float64)
        np.add.at(want, ids.astype(np.int64), res[0][0][k][:n, :E].astype(np.float64))
        close(res[0][1], want, "table, separate calls")
        close(res[1][1], want, "table, combined call")
    with pytest.raises(hip.CavsError, match="alpha = 1"):
        descs[k].beta = 0.5
        g.call("cavs_sgemm_group_embed_bwd", len(shapes), descs, k, g.P(table), g.P(d_ids), g.P(ws), nbytes, g.stream())


@pytest.mark.parametrize("tA,tB,M,N,K", [(0, 0, 30, 1536, 512), (0, 1, 8, 512, 1536), (0, 1, 130, 512, 512),
                                          (0, 0, 1, 64, 4096), (1, 1, 40, 72, 640), (0, 0, 33, 40, 300),
                                          (0, 1, 65, 33, 68), (0, 0, 600, 1536, 512), (0, 1, 1200, 512, 1536),
                                          (0, 1, 2482, 5, 512), (1, 0, 5, 512, 2482)])
def test_small_products(g, oracle, tA, tB, M, N, K):
    """Tail-round shapes (skinny kernel or split K through the workspace): correct and
    bit-identical when repeated."""
    import torch

    r = rng(M * 3 + N + K)
    A = r.bulk_uniform(M * K, -1, 1).reshape((K, M) if tA else (M, K))
    B = r.bulk_uniform(N * K, -1, 1).reshape((N, K) if tB else (K, N))
    nbytes = hip.lib().cavs_sgemm_splitk_workspace(M, N, K)
    ws = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device="cuda")
    exact = (A.T if tA else A).astype(np.float64) @ (B.T if tB else B).astype(np.float64)
    outs = []
    for _ in range(3):
        Cd = g.zeros(M, N, fill=float("nan"))
        g.call("cavs_sgemm_splitk", tA, tB, M, N, K, 1.0, g.P(g.devf(A)), A.shape[1], g.P(g.devf(B)), B.shape[1],
               0.0, g.P(Cd), N, g.P(ws), nbytes, g.stream())
        outs.append(g.host(Cd))
    close(outs[0], exact)
    np.testing.assert_array_equal(outs[0], outs[1])
    np.testing.assert_array_equal(outs[0], outs[2])
    if not tA and tB:  # with the per-vertex addend of the Tree-LSTM backward
        D = r.bulk_normal(((M + 1) // 2) * N).reshape((M + 1) // 2, N)
        Cd = g.zeros(M, N)
        g.call("cavs_sgemm_addrows", tA, tB, M, N, K, g.P(g.devf(A)), K, g.P(g.devf(B)), K, g.P(g.devf(D)), N, 1,
               g.P(Cd), N, g.P(ws), nbytes, g.stream())
        close(g.host(Cd), exact + np.repeat(D, 2, axis=0)[:M])


# ---------------------------------------------------------------- gates
@pytest.mark.parametrize("n,H", [(1, 4), (9, 8), (33, 512), (7, 6)])
def test_treelstm_gates(g, oracle, n, H):
    r = rng(n * H)
    xW = r.bulk_normal(n * 4 * H).reshape(n, 4 * H)
    hU = r.bulk_normal(n * 3 * H).reshape(n, 3 * H)
    hUf = r.bulk_normal(2 * n * H).reshape(2 * n, H)
    G = r.bulk_normal(2 * n * 2 * H).reshape(2 * n, 2 * H)
    bias = r.bulk_normal(4 * H)
    gates_w, msg_w = oracle.treelstm_gates_fwd(xW, hU, hUf, G, bias)
    gates, msg = g.zeros(n, 6 * H), g.zeros(n, 2 * H)
    dG_ = g.devf(G)
    g.call("cavs_treelstm_gates_fwd", g.P(g.devf(xW)), 4 * H, g.P(g.devf(hU)), g.P(g.devf(hUf)), g.P(dG_),
           g.P(g.devf(bias)), g.P(gates), g.P(msg), n, H, g.stream())
    close(g.host(gates), gates_w, "gates")
    close(g.host(msg), msg_w, "msg")
    # a round of leaves: children are zero
    gates_l, msg_l = oracle.treelstm_gates_fwd(xW, 0 * hU, 0 * hUf, 0 * G, bias)
    g.call("cavs_treelstm_gates_fwd", g.P(g.devf(xW)), 4 * H, None, None, None, g.P(g.devf(bias)),
           g.P(gates), g.P(msg), n, H, g.stream())
    close(g.host(gates), gates_l, "leaf gates")
    close(g.host(msg), msg_l, "leaf msg")
    # the same launch with Scatter and Push / PopRet folded in: bit for bit the gates and the message,
    # the message also in the pool rows the list names (-1: nowhere), its h in the listed output rows
    pair = np.arange(n, dtype=np.int32)[::-1] * 2
    pair[::3] = -1
    out_rows = (np.arange(n, dtype=np.int32) * 5 + 1) % n if n > 1 else np.zeros(1, np.int32)
    out_rows = np.argsort(np.argsort(out_rows, kind="stable"), kind="stable").astype(np.int32)  # a permutation
    for with_msg in (True, False):
        gates2, msg2, pool, go = g.zeros(n, 6 * H), g.zeros(n, 2 * H), g.zeros(2 * n, 2 * H, fill=7.0), g.zeros(n, H)
        g.call("cavs_treelstm_gates_fwd", g.P(g.devf(xW)), 4 * H, g.P(g.devf(hU)), g.P(g.devf(hUf)), g.P(dG_), g.P(g.devf(bias)), g.P(gates),
               g.P(msg), n, H, g.stream())
        g.call("cavs_treelstm_gates_fwd_scatter", g.P(g.devf(xW)), 4 * H, g.P(g.devf(hU)), g.P(g.devf(hUf)), g.P(dG_), g.P(g.devf(bias)),
               g.P(gates2), g.P(msg2) if with_msg else None, g.P(pool), g.P(g.devi(pair)), g.P(go), g.P(g.devi(out_rows)), n, H, g.stream())
        m = g.host(msg)
        np.testing.assert_array_equal(g.host(gates2), g.host(gates))
        np.testing.assert_array_equal(g.host(msg2), m if with_msg else 0 * m)
        want_pool = np.full((2 * n, 2 * H), 7.0, np.float32)
        want_pool[pair[pair >= 0]] = m[pair >= 0]
        np.testing.assert_array_equal(g.host(pool), want_pool)
        want_go = np.zeros((n, H), np.float32)
        want_go[out_rows] = m[:, :H]
        np.testing.assert_array_equal(g.host(go), want_go)

    dmsg = r.bulk_normal(n * 2 * H).reshape(n, 2 * H)
    dret = r.bulk_normal(n * H).reshape(n, H)
    dxW_w, dF_w, dG_w = oracle.treelstm_gates_bwd(dmsg, dret, gates_w, G)
    dxW, dF, dG = g.zeros(n, 4 * H), g.zeros(2 * n, H), g.zeros(2 * n, 2 * H)
    g.call("cavs_treelstm_gates_bwd", g.P(g.devf(dmsg)), g.P(g.devf(dret)), g.P(g.devf(gates_w)), g.P(dG_),
           g.P(dxW), 4 * H, g.P(dF), g.P(dG), n, H, g.stream())
    close(g.host(dxW), dxW_w, "dxW")
    close(g.host(dF), dF_w, "dF")
    close(g.host(dG), dG_w, "dG")
    dxW_l, _, _ = oracle.treelstm_gates_bwd(dmsg, dret, gates_l, 0 * G)
    g.call("cavs_treelstm_gates_bwd", g.P(g.devf(dmsg)), g.P(g.devf(dret)), g.P(g.devf(gates_l)), None,
           g.P(dxW), 4 * H, None, None, n, H, g.stream())
    close(g.host(dxW), dxW_l, "leaf dxW")


@pytest.mark.parametrize("n,H", [(1, 4), (19, 128), (5, 6)])
def test_lstm_and_treefc_gates(g, oracle, n, H):
    r = rng(3 * n + H)
    a = r.bulk_normal(n * 4 * H).reshape(n, 4 * H)
    a2 = r.bulk_normal(n * 4 * H).reshape(n, 4 * H)
    G = r.bulk_normal(n * 2 * H).reshape(n, 2 * H)
    bias = r.bulk_normal(4 * H)
    gates_w, msg_w = oracle.lstm_gates_fwd(a + a2, G, bias)
    gates, msg = g.zeros(n, 5 * H), g.zeros(n, 2 * H)
    g.call("cavs_lstm_gates_fwd", g.P(g.devf(a)), 4 * H, g.P(g.devf(a2)), g.P(g.devf(G)), g.P(g.devf(bias)),
           g.P(gates), g.P(msg), n, H, g.stream())
    close(g.host(gates), gates_w)
    close(g.host(msg), msg_w)
    gates_0, msg_0 = oracle.lstm_gates_fwd(a, 0 * G, bias)
    g.call("cavs_lstm_gates_fwd", g.P(g.devf(a)), 4 * H, None, None, g.P(g.devf(bias)), g.P(gates), g.P(msg),
           n, H, g.stream())
    close(g.host(msg), msg_0)
    dmsg, dret = r.bulk_normal(n * 2 * H).reshape(n, 2 * H), r.bulk_normal(n * H).reshape(n, H)
    da_w, dG_w = oracle.lstm_gates_bwd(dmsg, dret, gates_w, G)
    da, dG = g.zeros(n, 4 * H), g.zeros(n, 2 * H)
    g.call("cavs_lstm_gates_bwd", g.P(g.devf(dmsg)), g.P(g.devf(dret)), g.P(g.devf(gates_w)), g.P(g.devf(G)),
           g.P(da), 4 * H, g.P(dG), n, H, g.stream())
    close(g.host(da), da_w)
    close(g.host(dG), dG_w)

    for act in (0, 1):
        z, b, x = r.bulk_normal(n * H).reshape(n, H), r.bulk_normal(H), r.bulk_normal(n * H).reshape(n, H)
        h = g.zeros(n, H)
        g.call("cavs_treefc_fwd", g.P(g.devf(z)), g.P(g.devf(b)), g.P(g.devf(x)), g.P(h), n, H, act, g.stream())
        hw = oracle.treefc_fwd(z, b, x, act)
        close(g.host(h), hw)
        g.call("cavs_treefc_fwd", None, g.P(g.devf(b)), g.P(g.devf(x)), g.P(h), n, H, act, g.stream())
        close(g.host(h), oracle.treefc_fwd(0 * z, b, x, act))
        d1, d2 = r.bulk_normal(n * H).reshape(n, H), r.bulk_normal(n * H).reshape(n, H)
        dz = g.zeros(n, H)
        g.call("cavs_treefc_bwd", g.P(g.devf(d1)), g.P(g.devf(d2)), g.P(g.devf(hw)), g.P(dz), n, H, act, g.stream())
        close(g.host(dz), oracle.treefc_bwd(d1, d2, hw, act))


# ---------------------------------------------------------------- the rest
@pytest.mark.parametrize("n,w", [(1, 1), (50, 7), (2482, 2048), (5000, 100), (3, 4096)])
def test_colsum(g, oracle, n, w):
    r = rng(n + w)
    X = r.bulk_normal(n * w).reshape(n, w)
    exact = X.astype(np.float64).sum(0)
    out = g.zeros(w, fill=float("nan"))
    g.call("cavs_colsum", g.P(out), g.P(g.devf(X)), w, n, w, 0, g.stream())
    close(g.host(out), exact)
    acc0 = r.bulk_normal(w)
    out = g.devf(acc0)
    g.call("cavs_colsum", g.P(out), g.P(g.devf(X)), w, n, w, 1, g.stream())
    close(g.host(out), exact + acc0)


@pytest.mark.parametrize("V,E,n", [(23, 6, 31), (21701, 300, 500), (1000, 128, 64), (21701, 300, 2482), (50, 512, 1100)])
def test_embedding(g, oracle, V, E, n):
    r = rng(V + E)
    table = r.bulk_normal(V * E).reshape(V, E)
    ids = np.floor(r.bulk_uniform(n) * V).astype(np.float32)
    ids[: n // 3] = ids[0]  # duplicates exercise the atomic accumulation
    out = g.zeros(n, E)
    g.call("cavs_embed_fwd", g.P(out), E, g.P(g.devf(ids)), g.P(g.devf(table)), n, E, g.stream())
    np.testing.assert_array_equal(g.host(out), oracle.embed_fwd(ids, table))
    # Pull of the id and the lookup in one pass: vertex b of the slab is vertex rows[b] of the feed
    rows = np.argsort(r.bulk_uniform(n)).astype(np.int32)
    out2, ids2 = g.zeros(n, E + 4, fill=7.0), g.zeros(n)
    g.call("cavs_embed_pull_fwd", g.P(out2), E + 4, g.P(ids2), g.P(g.devf(ids)), g.P(g.devi(rows)), g.P(g.devf(table)),
           n, E, g.stream())
    np.testing.assert_array_equal(g.host(ids2), ids[rows])
    np.testing.assert_array_equal(g.host(out2)[:, :E], oracle.embed_fwd(ids[rows], table))
    np.testing.assert_array_equal(g.host(out2)[:, E:], np.full((n, 4), 7.0, np.float32))  # beyond E untouched
    dy = r.bulk_normal(n * E).reshape(n, E)
    d0 = r.bulk_normal(V * E).reshape(V, E)
    want = oracle.embed_bwd(d0.copy(), ids, dy)
    dt = g.devf(d0)
    g.call("cavs_embed_bwd", g.P(dt), g.P(g.devf(ids)), g.P(g.devf(dy)), E, n, E, g.stream())
    close(g.host(dt), want)


# (rows of 512 to 16384 classes in whole float4s go a workgroup per row, in four register sizes;
# the others a wavefront per row)
@pytest.mark.parametrize("n,C_", [(19, 5), (300, 1000), (1, 2), (64, 10000), (7, 512), (5, 2052), (3, 4100), (4, 12000),
                                  (3, 16384), (6, 1001), (2, 16388)])
def test_softmax_xent_bias_sgd(g, oracle, n, C_):
    r = rng(n + C_)
    logits = 3 * r.bulk_normal(n * C_).reshape(n, C_)
    labels = np.floor(r.bulk_uniform(n) * C_).astype(np.float32)
    loss_w, d_w = oracle.softmax_xent(logits, labels)
    loss, d = g.zeros(n), g.zeros(n, C_)
    g.call("cavs_softmax_xent", g.P(loss), g.P(d), g.P(g.devf(logits)), g.P(g.devf(labels)), n, C_, g.stream())
    close(g.host(loss), loss_w)
    close(g.host(d), d_w, atol=1e-7)
    bias = r.bulk_normal(C_)
    out = g.zeros(n, C_)
    g.call("cavs_bias_add_rows", g.P(out), g.P(g.devf(logits)), g.P(g.devf(bias)), n, C_, g.stream())
    np.testing.assert_array_equal(g.host(out), logits + bias[None, :])
    w, grad = g.devf(logits), d_w.astype(np.float32)
    g.call("cavs_sgd", g.P(w), g.P(g.devf(grad)), 0.5, n * C_, g.stream())
    np.testing.assert_array_equal(g.host(w), logits - np.float32(0.5) * grad)


@pytest.mark.parametrize("n,C_", [(40, 10000), (23, 600), (9, 7)])
def test_softmax_xent_of_a_batch_in_parts_is_the_whole_row_for_row(g, n, C_):
    """The loss head of a wide classifier runs chunk by chunk: a part's rows come out bit for bit as
    in the call over the whole batch (the gradient's 1/n is the batch's)."""
    r = rng(n * 3 + C_)
    logits = g.devf(3 * r.bulk_normal(n * C_).reshape(n, C_))
    labels = g.devf(np.floor(r.bulk_uniform(n) * C_).astype(np.float32))
    loss, d = g.zeros(n), g.zeros(n, C_)
    g.call("cavs_softmax_xent", g.P(loss), g.P(d), g.P(logits), g.P(labels), n, C_, g.stream())
    loss2, d2 = g.zeros(n), g.zeros(n, C_)
    cut = [0, n // 3, n // 3, n - 2, n]  # (one part is empty)
    for a, b in zip(cut[:-1], cut[1:]):
        g.call("cavs_softmax_xent_part", g.P(loss2) + 4 * a, g.P(d2) + 4 * a * C_, g.P(logits) + 4 * a * C_, g.P(labels) + 4 * a, b - a, C_, n,
               g.stream())
    np.testing.assert_array_equal(g.host(loss2), g.host(loss))
    np.testing.assert_array_equal(g.host(d2), g.host(d))


def test_elementwise_family(g):
    r = rng(3)
    n, w = 37, 20
    a, b = r.bulk_normal(n * w), r.bulk_normal(n * w)
    row = r.bulk_normal(w)
    sig = lambda x: 1.0 / (1.0 + np.exp(-x.astype(np.float64)))
    cases = {"add": a + b, "sub": a - b, "mul": a * b, "div": a / b,
             "sigmoid_grad": a * (b * (1 - b)), "tanh_grad": a * (1 - b * b),
             "relu_grad": np.where(b > 0, a, 0), "equal": (a == b).astype(np.float32)}
    for name, want in cases.items():
        out = g.zeros(n * w)
        g.call("cavs_ew_binary", hip.EW_BINARY[name], g.P(out), g.P(g.devf(a)), n * w, g.P(g.devf(b)), n * w,
               n * w, 0, g.stream())
        close(g.host(out), want, name)
    out = g.zeros(n * w)  # row broadcast (bias add) and scalar
    g.call("cavs_ew_binary", 0, g.P(out), g.P(g.devf(a)), n * w, g.P(g.devf(row)), w, n * w, 0, g.stream())
    np.testing.assert_array_equal(g.host(out), (a.reshape(n, w) + row).ravel())
    out = g.devf(a)  # accumulate form
    g.call("cavs_ew_binary", 2, g.P(out), g.P(g.devf(a)), n * w, g.P(g.devf(row[:1])), 1, n * w, 1, g.stream())
    close(g.host(out), a + a * row[0])
    un = {"assign": a, "neg": -a, "abs": np.abs(a), "square": a * a, "sigmoid": sig(a), "tanh": np.tanh(a.astype(np.float64)),
          "relu": np.maximum(a, 0)}
    for name, want in un.items():
        out = g.zeros(n * w)
        g.call("cavs_ew_unary", hip.EW_UNARY[name], g.P(out), g.P(g.devf(a)), n * w, 0, g.stream())
        close(g.host(out), want, name)
    out = g.zeros(n * w)
    g.call("cavs_scale", g.P(out), g.P(g.devf(a)), 0.25, n * w, g.stream())
    np.testing.assert_array_equal(g.host(out), np.float32(0.25) * a)
    with pytest.raises(hip.CavsError, match="unknown op"):
        hip.call("cavs_ew_unary", 99, g.P(out), g.P(out), 4, 0, g.stream())


def test_fill_zero_and_copies(g):
    import torch

    t = torch.full((1003,), 5.0, device="cuda")
    g.call("cavs_zero", g.P(t) + 4, 4 * 1001, g.stream())  # unaligned start
    want = np.zeros(1003, np.float32)
    want[0] = want[-1] = 5
    np.testing.assert_array_equal(g.host(t), want)
    g.call("cavs_fill", g.P(t), 2.5, 1003, g.stream())
    assert (g.host(t) == 2.5).all()
    src = np.arange(100, dtype=np.float32)
    d = g.zeros(100)
    g.call("cavs_memcpy_h2d", g.P(d), src.ctypes.data, 400, g.stream())
    back = np.zeros(100, np.float32)
    g.call("cavs_memcpy_d2h", back.ctypes.data, g.P(d), 400, g.stream())
    g.call("cavs_stream_sync", g.stream())
    np.testing.assert_array_equal(back, src)


def test_fused_kernel_interface(g):
    """The two fused groups of the reference's fusion smoke test
    (cavs/frontend/cxx/fusion_session_test.cc): E = C + (A + B) and YY = (X + Y) + Z,
    in the generator's dialect (idx % count reads, atomicAdd for narrower outputs)."""
    src = r'''
extern "C" __global__ void FusedKernel_0(float *E, const float *A, const float *B, const float *C,
    const int E_count, const int A_count, const int B_count, const int C_count, const int n_elements)
{
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < n_elements) {
    float tmp_A = A[idx%A_count];
    float tmp_B = B[idx%B_count];
    float tmp_C = C[idx%C_count];
    float tmp_D = tmp_A + tmp_B;
    float tmp_E = tmp_C + tmp_D;
    if (E_count < n_elements) {
      float ori_E = E[idx%E_count];
      atomicAdd(&E[idx%E_count], (tmp_E - ori_E));
    } else {
      E[idx%E_count] = tmp_E;
    }
  }
}'''
    h = C.c_void_p()
    hip.call("cavs_fused_compile", b"FusedKernel_0", src.encode(), C.byref(h))
    A = np.array([1, 2, 3, 4, 5, 6], np.float32)
    B = np.array([6, 5, 4, 3, 2, 1], np.float32)
    Cc = np.array([0.1, 0.2, 0.3, 0.4, 0.5, 0.6], np.float32)
    out = g.zeros(6)
    dA, dB, dC = g.devf(A), g.devf(B), g.devf(Cc)
    outs = (C.c_void_p * 1)(g.P(out))
    ins = (C.c_void_p * 3)(g.P(dA), g.P(dB), g.P(dC))
    oc = (C.c_int * 1)(6)
    ic = (C.c_int * 3)(6, 6, 6)
    hip.call("cavs_fused_launch", h, outs, 1, ins, 3, oc, ic, 6, g.stream())
    np.testing.assert_allclose(g.host(out), [7.1, 7.2, 7.3, 7.4, 7.5, 7.6], rtol=1e-6)
    # an output narrower than the element range: the generator's atomicAdd branch.  Six elements onto
    # a row of three (elements k and k + 3 land on E[k]); E starts at zero, as ZeroEnforced makes it
    row = g.zeros(3)
    outs = (C.c_void_p * 1)(g.P(row))
    oc = (C.c_int * 1)(3)
    hip.call("cavs_fused_launch", h, outs, 1, ins, 3, oc, ic, 6, g.stream())
    np.testing.assert_allclose(g.host(row), [7.1 + 7.4, 7.2 + 7.5, 7.3 + 7.6], rtol=1e-6)
    hip.call("cavs_fused_release", h)
    # the form this build's fusion pass emits for a reducing output: the element's contribution is
    # added, nothing is read back; a broadcast operand wraps
    src2 = r'''
extern "C" __global__ void FusedKernel_1(float *S, float *Y, const float *X, const float *b,
    const int S_count, const int Y_count, const int X_count, const int b_count, const int n_elements)
{
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < n_elements) {
    float tmp_X = X[idx];
    float tmp_b = b[idx % b_count];
    float tmp_Y = tmp_X * tmp_b;
    float tmp_S = tmp_Y;
    atomicAdd(&S[idx % S_count], tmp_S);
    Y[idx] = tmp_Y;
  }
}'''
    hip.call("cavs_fused_compile", b"FusedKernel_1", src2.encode(), C.byref(h))
    n, w = 700, 40
    r = rng(5)
    X, bvec = r.bulk_normal(n * w).reshape(n, w), r.bulk_normal(w)
    S, Y = g.zeros(w), g.zeros(n, w)
    outs = (C.c_void_p * 2)(g.P(S), g.P(Y))
    ins = (C.c_void_p * 2)(g.P(g.devf(X)), g.P(g.devf(bvec)))
    oc = (C.c_int * 2)(w, n * w)
    ic = (C.c_int * 2)(n * w, w)
    hip.call("cavs_fused_launch", h, outs, 2, ins, 2, oc, ic, n * w, g.stream())
    want = X.astype(np.float64) * bvec.astype(np.float64)
    close(g.host(Y), want, "Y")
    close(g.host(S), want.sum(0), "column sums through atomicAdd")
    hip.call("cavs_fused_release", h)
    bad = C.c_void_p()
    with pytest.raises(hip.CavsError, match="compile"):
        hip.call("cavs_fused_compile", b"k", b"this is not a kernel", C.byref(bad))


def test_generated_cell_module_interface(g):
    """cavs_cell_compile / cavs_cell_launch: a module that defines the eight kernels by name, each
    taking one struct of 8-byte slots by value; the bytes passed are the struct.  A stand-in source
    whose kernels write what they were given."""
    names = ["cell_fwd", "cell_leaves", "cell_bwd", "cell_bwd_rows", "cell_pack", "cell_bias", "cell_bwd_gates", "cell_bwd_pool"]
    src = "struct Args { float *out; long a, b; };\n" + "".join(
        f'extern "C" __global__ void {n}(Args s) {{ if (threadIdx.x == 0) s.out[{k} * 8 + blockIdx.x + 2 * blockIdx.y] = '
        f'{k} * 1000.f + s.a * 10.f + s.b + blockDim.x / 64; }}\n' for k, n in enumerate(names))
    h = C.c_void_p()
    hip.call("cavs_cell_compile", src.encode(), C.byref(h))
    h2 = C.c_void_p()
    hip.call("cavs_cell_compile", src.encode(), C.byref(h2))  # the same source: the same module
    assert h2.value == h.value
    out = g.zeros(64)

    class Args(C.Structure):
        _fields_ = [("out", C.c_void_p), ("a", C.c_long), ("b", C.c_long)]

    for k in range(len(names)):
        a = Args(g.P(out), 3 + k, 5)
        hip.call("cavs_cell_launch", h, k, 2, 2, 1, 64 * (1 + k % 4), C.byref(a), C.sizeof(a), g.stream())
    got = g.host(out).reshape(8, 8)
    for k in range(len(names)):
        np.testing.assert_array_equal(got[k, :4], k * 1000 + (3 + k) * 10 + 5 + (1 + k % 4))
    a = Args(g.P(out), 0, 0)
    with pytest.raises(hip.CavsError, match="no kernel"):
        hip.call("cavs_cell_launch", h, 8, 1, 1, 1, 64, C.byref(a), C.sizeof(a), g.stream())
    with pytest.raises(hip.CavsError, match="launch shape"):
        hip.call("cavs_cell_launch", h, 0, 1, 1, 1, 96, C.byref(a), C.sizeof(a), g.stream())
    hip.call("cavs_cell_launch", h, 0, 0, 1, 1, 64, C.byref(a), C.sizeof(a), g.stream())  # an empty grid is no launch
    hip.call("cavs_cell_release", h)
    hip.call("cavs_cell_release", h2)
    bad = C.c_void_p()
    with pytest.raises(hip.CavsError, match="compile"):
        hip.call("cavs_cell_compile", b"this is not a kernel", C.byref(bad))
    with pytest.raises(hip.CavsError, match="loading"):  # compiles, but a kernel is missing
        hip.call("cavs_cell_compile", b'extern "C" __global__ void cell_fwd(int) {}', C.byref(bad))


@pytest.mark.parametrize("kind,seed,B,lo,hi", [("tree", 1, 1, 2, 2), ("tree", 2, 7, 2, 30), ("tree", 3, 64, 2, 56),
                                               ("chain", 4, 9, 2, 40), ("tree", 5, 40, 32, 256)])
def test_device_frontier_matches_host_schedule_bit_exact(g, oracle, kind, seed, B, lo, hi):
    import torch

    graph = (synth.tree_batch if kind == "tree" else synth.chain_batch)(seed, B, lo, hi)[0]
    tr = oracle.sched_trace(graph)
    N = tr["N"]
    parent, off = [], 0
    for row in graph:
        n = int(np.argmax(row == -1)) + 1
        parent += [off + int(p) if p >= 0 else -1 for p in row[:n]]
        off += n
    I = lambda k: torch.full((k,), -7, dtype=torch.int32, device="cuda")
    t2j, j2t, rot, r2o, nr, scratch = I(N), I(N), I(N), I(N + 2), I(1), I(4 * N)
    g.call("cavs_schedule_frontier", g.P(g.devi(parent)), N, g.P(t2j), g.P(j2t), g.P(rot), g.P(r2o), g.P(nr),
           g.P(scratch), g.stream())
    R = int(g.host(nr)[0])
    assert R == len(tr["fwd"])
    assert g.host(r2o)[: R + 1].tolist() == tr["round2offset"]
    assert g.host(t2j).tolist() == tr["tids_to_jobids"]
    inv = np.empty(N, np.int64)
    inv[np.array(tr["tids_to_jobids"])] = np.arange(N)
    assert g.host(j2t).tolist() == inv.tolist()
    want_round = np.concatenate([[r] * len(rd["exec"]) for r, rd in enumerate(tr["fwd"])])
    assert g.host(rot).tolist() == want_round.tolist()


def _device_arena(g, graph, nch, pairing):
    """Runs cavs_schedule_arena on a graph feed; returns (meta, lists) as numpy arrays."""
    import torch

    graph = np.ascontiguousarray(graph, np.int32)
    B, maxlen = graph.shape
    cap = B * maxlen + 7  # any capacity of at least B * maxlen rows
    I = lambda k: torch.full((k,), -77, dtype=torch.int32, device="cuda")
    t2j, pair, child, kid, roots, orph, meta = I(cap), I(cap), I(nch * cap), I(nch * cap), I(B), I(B), I(maxlen + 9)
    nbytes = hip.lib().cavs_schedule_arena_scratch(B, maxlen)
    scratch = I(nbytes // 4)
    g.call("cavs_schedule_arena", g.P(g.devi(graph)), B, maxlen, nch, 0 if pairing == "reference" else 1, g.P(t2j), g.P(pair),
           g.P(child), g.P(kid), g.P(roots), g.P(orph), cap, g.P(meta), g.P(scratch), nbytes, g.stream())
    return g.host(meta), dict(t2j=g.host(t2j), pair=g.host(pair), child=g.host(child), kid=g.host(kid), roots=g.host(roots),
                              orphans=g.host(orph))


def _check_device_arena(g, oracle, graph, nch, pairing):
    import arena

    want = arena.expected_arena(oracle.sched_trace(graph), graph, nch, pairing)
    meta, got = _device_arena(g, graph, nch, pairing)
    N, R = want["N"], want["R"]
    assert meta[2] == 0, f"error bits {meta[2]}"
    assert (meta[0], meta[1]) == (N, R)
    assert meta[8: 8 + R + 1].tolist() == want["round2offset"].tolist()
    assert meta[3] == int(np.diff(want["round2offset"]).max())
    assert got["t2j"][:N].tolist() == want["t2j"].tolist()
    assert got["pair"][:N].tolist() == want["pair"].tolist()
    assert got["child"][: nch * N].tolist() == want["child"].tolist()
    assert got["kid"][: nch * N].tolist() == want["kid"].tolist()
    assert got["roots"].tolist() == want["roots"].tolist()
    assert got["orphans"].tolist() == want["orphans"].tolist()


@pytest.mark.parametrize("pairing", ["reference", "rowid"])
def test_device_scheduler_writes_the_whole_index_arena_bit_exact(g, oracle, pairing):
    """cavs_schedule_arena against the lists of the oracle's scheduler: the hand-derived known
    answers, skewed and same-shape batches of trees and chains, and the graphs of the benchmark
    configurations C1-C5 at their own batch sizes."""
    import json
    import os

    kats = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "sched_kat.json")))["cases"]
    for case in kats:
        graph = np.array(case["graph"], np.int32)
        tr = oracle.sched_trace(graph)
        # the arena is defined for what the kernels run: every internal vertex with all its children
        arity = {len([1 for c in range(2) if rd["gather"][c]]) for rd in tr["fwd"][1:]}
        if len(arity) != 1 or any(len(rd["gather"][c]) not in (0, len(rd["exec"])) for rd in tr["fwd"] for c in range(2)):
            continue
        print(f"[case] arena KAT {case['name']} pairing={pairing}", flush=True)
        _check_device_arena(g, oracle, graph, arity.pop(), pairing)
    for kind, seed, B, lo, hi in [("tree", 1, 1, 2, 2), ("tree", 2, 7, 2, 30), ("chain", 4, 9, 2, 40), ("tree", 5, 40, 32, 256),
                                  ("chain", 6, 300, 1 + 1, 70)]:
        print(f"[case] arena {kind} seed={seed} B={B} pairing={pairing}", flush=True)
        graph = (synth.tree_batch if kind == "tree" else synth.chain_batch)(seed, B, lo, hi)[0]
        _check_device_arena(g, oracle, graph, 2 if kind == "tree" else 1, pairing)
    for name in ("C1", "C2", "C3", "C4", "C5"):
        w = synth.make_workload(name, scale=0.03125)  # the graphs do not depend on the widths
        print(f"[case] arena {name} B={w['graph'].shape[0]} N={w['N']} pairing={pairing}", flush=True)
        _check_device_arena(g, oracle, w["graph"], 1 if w["model"] == "lstm" else 2, pairing)


def test_device_scheduler_flags_what_the_host_scheduler_rejects(g):
    bad = {
        1: [[1, 2, 0, 0]],                      # no -1 within maxlen
        2: [[5, 2, -1, -1]],                    # parent out of range
        4: [[3, 3, 3, -1]],                     # three children
        8: [[-1, -1, -1, -1], [1, -1, -1, -1]],  # single-vertex sample
        16: [[1, 0, 3, -1]],                    # vertices 0 and 1 are each other's parent
    }
    for bit, graph in bad.items():
        print(f"[case] arena error bit {bit}", flush=True)
        meta, _ = _device_arena(g, np.array(graph, np.int32), 2, "reference")
        assert meta[2] & bit, (bit, meta[:4])
    # a chain fed to a binary vertex function: internal vertices with one child
    meta, _ = _device_arena(g, np.array([[1, 2, -1]], np.int32), 2, "reference")
    assert meta[2] & 4
    meta, _ = _device_arena(g, np.array([[1, 2, -1]], np.int32), 1, "reference")
    assert meta[2] == 0 and meta[0] == 3 and meta[1] == 3


def test_reference_elementwise_smoke_values(g):
    """The Add the reference's op_impl_elementwise_test.cc prints: {1..6} + {0..5}."""
    import json
    import os

    kat = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "smoke_kats.json")))["elementwise_add"]
    a, b = np.array(kat["a"], np.float32), np.array(kat["b"], np.float32)
    out = g.zeros(6)
    g.call("cavs_ew_binary", hip.EW_BINARY["add"], g.P(out), g.P(g.devf(a)), 6, g.P(g.devf(b)), 6, 6, 0, g.stream())
    np.testing.assert_array_equal(g.host(out), np.array(kat["expect"], np.float32))


@pytest.mark.parametrize("n,H", [(1, 32), (16, 64), (17, 32), (33, 96), (64, 64), (65, 32), (130, 64), (600, 64), (300, 512),
                                 (40, 512), (3, 1024), (100, 128), (90, 256)])
def test_fused_tree_lstm_rounds(g, oracle, n, H):
    """A whole round in one launch (forward) / two (backward) against the same round
    composed from the oracle's gather, GEMM and gate functions."""
    r = rng(7 * n + H)
    P_rows = 2 * n + 5                      # pool: children rows, then this round's rows
    pool = (r.bulk_normal((P_rows + n) * 2 * H).reshape(P_rows + n, 2 * H) * 0.5).astype(np.float32)
    perm = np.argsort(r.bulk_normal(P_rows))[: 2 * n].astype(np.int32)
    child = perm.copy()
    pair = (P_rows + np.arange(n)).astype(np.int32)
    if n > 2:
        child[3] = -1                       # a missing child reads as zero
        pair[n - 1] = -1                    # a root: its message goes nowhere
    xW = r.bulk_normal(n * 4 * H).reshape(n, 4 * H)
    U = (r.bulk_normal(4 * H * H) / np.sqrt(H)).astype(np.float32)
    Uiou, Uf = U[: 3 * H * H].reshape(H, 3 * H), U[3 * H * H:].reshape(H, H)
    bias = r.bulk_normal(4 * H)
    # expected, from the oracle's pieces
    def gather0(src, ids):  # the oracle's gather with "-1 reads as zero" of the C ABI on top
        out = oracle.gather_rows(src, np.maximum(ids, 0))
        out[ids < 0] = 0
        return out

    G_w = gather0(pool, child)                                              # [2n, 2H]
    hlr_w = (G_w[0::2, :H] + G_w[1::2, :H]).astype(np.float32)
    hU_w = oracle.sgemm(0, 0, hlr_w, Uiou)
    hUf_w = oracle.sgemm(0, 0, np.ascontiguousarray(G_w[:, :H]), Uf)
    gates_w, msg_w = oracle.treelstm_gates_fwd(xW, hU_w, hUf_w, G_w, bias)
    pool_w = pool.copy()
    pool_w[pair[pair >= 0]] = msg_w[pair >= 0]

    d_pool, d_child, d_pair = g.devf(pool), g.devi(child), g.devi(pair)
    G, hlr, gates, msg = g.zeros(2 * n, 2 * H), g.zeros(n, H), g.zeros(n, 6 * H), g.zeros(n, 2 * H)
    out_rows = np.argsort(r.bulk_normal(n + 3))[:n].astype(np.int32)     # Push + PopRet folded in
    go = g.zeros(n + 3, H, fill=-7.0)
    g.call("cavs_treelstm_round_fwd", g.P(d_pool), g.P(d_child), g.P(d_pair), g.P(g.devf(xW)), 4 * H, g.P(g.devf(U)),
           g.P(g.devf(bias)), g.P(G), g.P(hlr), g.P(gates), g.P(msg), g.P(go), g.P(g.devi(out_rows)), n, H, g.stream())
    go_w = np.full((n + 3, H), -7.0, np.float32)
    go_w[out_rows] = msg_w[:, :H]
    close(g.host(go), go_w, "graph_out")
    np.testing.assert_array_equal(g.host(G), G_w)
    np.testing.assert_array_equal(g.host(hlr), hlr_w)
    close(g.host(gates), gates_w, "gates")
    close(g.host(msg), msg_w, "msg")
    close(g.host(d_pool), pool_w, "pool")

    # backward: message gradients of this round sit in dpool rows pair[b]
    dpool = r.bulk_normal((P_rows + n) * 2 * H).reshape(P_rows + n, 2 * H)
    dret = r.bulk_normal(n * H).reshape(n, H)
    dmsg_w = gather0(dpool, pair)
    dxW_w, dF_w, dG_w = oracle.treelstm_gates_bwd(dmsg_w, dret, gates_w, G_w)
    dhlr_w = oracle.sgemm(0, 1, np.ascontiguousarray(dxW_w[:, : 3 * H]), np.ascontiguousarray(Uiou))
    dGh_w = oracle.sgemm(0, 1, dF_w, np.ascontiguousarray(Uf)) + np.repeat(dhlr_w, 2, axis=0)
    dG_w[:, :H] = dGh_w
    dpool_w = dpool.copy()
    dpool_w[child[child >= 0]] = dG_w[child >= 0]

    UT = g.zeros(4 * H * H)
    d_U = g.devf(U)
    g.call("cavs_transpose", g.P(UT), g.P(d_U), H, 3 * H, g.stream())
    g.call("cavs_transpose", g.P(UT) + 4 * 3 * H * H, g.P(d_U) + 4 * 3 * H * H, H, H, g.stream())
    np.testing.assert_array_equal(g.host(UT)[: 3 * H * H].reshape(3 * H, H), Uiou.T)
    np.testing.assert_array_equal(g.host(UT)[3 * H * H:].reshape(H, H), Uf.T)
    # both in one launch
    UT2 = g.zeros(4 * H * H)
    tasks = (hip.Task * 2)(hip.Task(hip.TASK_TRANSPOSE, 0.0, H, 3 * H, 0, g.P(UT2), g.P(d_U), None, None),
                           hip.Task(hip.TASK_TRANSPOSE, 0.0, H, H, 0, g.P(UT2) + 4 * 3 * H * H, g.P(d_U) + 4 * 3 * H * H, None, None))
    g.call("cavs_run_tasks", 2, tasks, g.stream())
    np.testing.assert_array_equal(g.host(UT2), g.host(UT))
    d_dpool, dxW, dF = g.devf(dpool), g.zeros(n, 4 * H), g.zeros(2 * n, H)
    g.call("cavs_treelstm_round_bwd_gates", g.P(d_dpool), g.P(d_pair), g.P(d_child), g.P(g.devf(dret)), None, g.P(g.devf(gates_w)),
           g.P(g.devf(G_w)), g.P(dxW), 4 * H, g.P(dF), n, H, g.stream())
    g.call("cavs_treelstm_round_bwd_children", g.P(dxW), 4 * H, g.P(dF), g.P(UT), g.P(d_child), g.P(d_dpool), n, H, g.stream())
    close(g.host(dxW), dxW_w, "dxW")
    close(g.host(dF), dF_w, "dF")
    close(g.host(d_dpool), dpool_w, "dpool")

    # a round of leaves: no children, nothing scattered downwards
    gates_l, _ = oracle.treelstm_gates_fwd(xW, 0 * hU_w, 0 * hUf_w, 0 * G_w, bias)
    dxW_l, _, _ = oracle.treelstm_gates_bwd(dmsg_w, dret, gates_l, 0 * G_w)
    d_dpool2 = g.devf(dpool)
    g.call("cavs_treelstm_round_bwd_gates", g.P(d_dpool2), g.P(d_pair), None, g.P(g.devf(dret)), None, g.P(g.devf(gates_l)),
           None, g.P(dxW), 4 * H, None, n, H, g.stream())
    close(g.host(dxW), dxW_l, "leaf dxW")
    np.testing.assert_array_equal(g.host(d_dpool2), dpool)
    # the same with the return-value gradient read through a row list (grad of PopRet folded in)
    dgo = np.zeros((n + 3, H), np.float32)
    dgo[out_rows] = dret
    dxW2 = g.zeros(n, 4 * H)
    g.call("cavs_treelstm_round_bwd_gates", g.P(d_dpool2), g.P(d_pair), None, g.P(g.devf(dgo)), g.P(g.devi(out_rows)),
           g.P(g.devf(gates_l)), None, g.P(dxW2), 4 * H, None, n, H, g.stream())
    np.testing.assert_array_equal(g.host(dxW2), g.host(dxW))
    # a round of leaves forward: gates, message, Scatter and PopRet in one launch
    _, msg_l = oracle.treelstm_gates_fwd(xW, 0 * hU_w, 0 * hUf_w, 0 * G_w, bias)
    pool2, gates2, msg2, go2 = g.devf(pool), g.zeros(n, 6 * H), g.zeros(n, 2 * H), g.zeros(n + 3, H, fill=-7.0)
    g.call("cavs_treelstm_round_leaves_fwd", g.P(pool2), g.P(d_pair), g.P(g.devf(xW)), 4 * H, g.P(g.devf(bias)), g.P(gates2),
           g.P(msg2), g.P(go2), g.P(g.devi(out_rows)), n, H, g.stream())
    close(g.host(gates2), gates_l, "leaf gates")
    close(g.host(msg2), msg_l, "leaf msg")
    pool_l = pool.copy()
    pool_l[pair[pair >= 0]] = msg_l[pair >= 0]
    close(g.host(pool2), pool_l, "leaf pool")
    go_l = np.full((n + 3, H), -7.0, np.float32)
    go_l[out_rows] = msg_l[:, :H]
    close(g.host(go2), go_l, "leaf graph_out")


@pytest.mark.parametrize("L,m,n,H", [(20, 5, 3, 32), (300, 70, 40, 64), (900, 200, 130, 64), (2600, 100, 1100, 32), (1300, 500, 300, 512),
                                     (300, 70, 40, 512), (300, 100, 90, 128)])
def test_backward_rounds_with_the_childrens_gate_gradients_folded_in(g, oracle, L, m, n, H):
    """Three levels over whole-batch slabs (leaves, a middle round, a top round of roots): the
    roots' gate gradients from the row-list launch, then one launch per round that hands d h,
    d c on to the children and does their gate gradients, against the same chain composed
    round by round from the oracle's gate-gradient and GEMM functions."""
    r = rng(11 * L + 3 * n + H)
    N = L + m + n
    mid0, top0 = L, L + m
    order = np.argsort(r.bulk_normal(L)).astype(np.int32)
    kids = np.full(2 * N, -1, np.int32)
    kids[2 * mid0: 2 * top0] = order[: 2 * m]                      # the middle round's children are leaves
    assert m <= 2 * n - 1 and 2 * m + 2 * n - m <= L
    top_kids = np.concatenate([np.arange(mid0, top0, dtype=np.int32), order[2 * m: 2 * m + 2 * n - m]])
    top_kids = top_kids[np.argsort(r.bulk_normal(2 * n))]          # the top round's: every middle row, and leaves
    top_kids[np.flatnonzero(top_kids < L)[0]] = -1                 # a missing child
    kids[2 * top0:] = top_kids
    sig = lambda a: (1.0 / (1.0 + np.exp(-a))).astype(np.float32)
    gates = r.bulk_normal(N * 6 * H).reshape(N, 6 * H)
    gates[:, : 2 * H] = sig(gates[:, : 2 * H])
    gates[:, 2 * H: 3 * H] = np.tanh(gates[:, 2 * H: 3 * H])
    gates[:, 3 * H: 5 * H] = sig(gates[:, 3 * H: 5 * H])
    gates[:, 5 * H:] = np.tanh(gates[:, 5 * H:])
    G = (r.bulk_normal(2 * N * 2 * H).reshape(2 * N, 2 * H) * 0.5).astype(np.float32)
    G[: 2 * L] = 0                                                 # leaves gathered nothing
    U = (r.bulk_normal(4 * H * H) / np.sqrt(H)).astype(np.float32)
    Uiou, Uf = U[: 3 * H * H].reshape(H, 3 * H), U[3 * H * H:].reshape(H, H)
    dret_rows = np.argsort(r.bulk_normal(N + 3))[:N].astype(np.int32)
    dgo = r.bulk_normal((N + 3) * H).reshape(N + 3, H)

    # expected, top-down
    dmsg = np.zeros((N, 2 * H), np.float32)
    reached = np.zeros(N, bool)
    reached[top0:] = True
    dxW_w, dF_w = np.zeros((N, 4 * H), np.float32), np.zeros((2 * N, H), np.float32)
    for lo, hi in ((top0, N), (mid0, top0), (0, L)):
        a, b, c = oracle.treelstm_gates_bwd(dmsg[lo:hi], dgo[dret_rows[lo:hi]], gates[lo:hi], G[2 * lo: 2 * hi])
        dxW_w[lo:hi], dF_w[2 * lo: 2 * hi] = a, b
        if lo == 0:
            break
        dhlr = oracle.sgemm(0, 1, np.ascontiguousarray(a[:, : 3 * H]), np.ascontiguousarray(Uiou))
        c[:, :H] = oracle.sgemm(0, 1, b, np.ascontiguousarray(Uf)) + np.repeat(dhlr, 2, axis=0)
        k = kids[2 * lo: 2 * hi]
        dmsg[k[k >= 0]] = c[k >= 0]
        reached[k[k >= 0]] = True

    UT = g.zeros(4 * H * H)
    d_U = g.devf(U)
    g.call("cavs_transpose", g.P(UT), g.P(d_U), H, 3 * H, g.stream())
    g.call("cavs_transpose", g.P(UT) + 4 * 3 * H * H, g.P(d_U) + 4 * 3 * H * H, H, H, g.stream())
    dxW, dF, dc = g.zeros(N, 4 * H, fill=-3.0), g.zeros(2 * N, H, fill=-3.0), g.zeros(N, H, fill=-3.0)
    d_gates, d_G, d_dgo, d_rows, d_kids = g.devf(gates), g.devf(G), g.devf(dgo), g.devi(dret_rows), g.devi(kids)
    roots = np.arange(top0, N, dtype=np.int32)
    g.call("cavs_treelstm_bwd_gates_rows", g.P(g.devi(roots)), n, g.P(d_dgo), g.P(d_rows), g.P(d_gates), g.P(d_G), g.P(dxW), 4 * H,
           g.P(dF), g.P(dc), L, H, g.stream())
    close(g.host(dxW)[top0:], dxW_w[top0:], "roots dxW")
    close(g.host(dF)[2 * top0:], dF_w[2 * top0:], "roots dF")
    assert (g.host(dxW)[:top0] == -3.0).all() and (g.host(dc)[:top0] == -3.0).all()
    for lo, cnt in ((top0, n), (mid0, m)):
        g.call("cavs_treelstm_round_bwd_children_gates", g.P(dxW), 4 * H, g.P(dF), g.P(dc), g.P(UT), g.P(d_kids) + 4 * 2 * lo,
               g.P(d_gates), g.P(d_G), g.P(d_dgo), g.P(d_rows), lo, cnt, L, H, g.stream())
    got_x, got_F = g.host(dxW), g.host(dF)
    close(got_x[reached], dxW_w[reached], "dxW")
    internal = reached.copy()
    internal[:L] = False
    close(got_F[np.repeat(internal, 2)], dF_w[np.repeat(internal, 2)], "dF")
    # rows no message reaches are left alone, and so are the leaves' rows of dF and dc
    assert (got_x[~reached] == -3.0).all()
    assert (got_F[: 2 * L] == -3.0).all() and (g.host(dc)[:L] == -3.0).all()


def pack_tiles(B):
    """The tile-major layout of CAVS_TASK_PACK_T, spelled out: B [K, N] -> [K/16][N/16][slot][x][c]."""
    K, N = B.shape
    out = np.zeros(K * N, np.float32)
    g, t, sl, x, c = np.meshgrid(np.arange(K // 16), np.arange(N // 16), np.arange(4), np.arange(16), np.arange(4), indexing="ij")
    out[((((g * (N // 16) + t) * 4 + sl) * 16 + x) * 4 + c).ravel()] = B[(16 * g + 4 * sl + c).ravel(), (16 * t + x).ravel()]
    return out


@pytest.mark.parametrize("L,m,n,H", [(300, 70, 40, 512), (1300, 500, 300, 512), (300, 100, 90, 128), (40, 9, 5, 1024), (60, 16, 13, 512),
                                     (12, 4, 1, 512), (400, 120, 70, 512)])
def test_packed_transposed_weights_give_the_same_backward_round_bit_for_bit(g, L, m, n, H):
    """The pack job against the layout written out in numpy, then the backward launch reading
    the packed weights against the one reading the plain transposes: same products in the same
    order, so every output agrees bit for bit."""
    r = rng(17 * L + n + H)
    N = L + m + n
    U = (r.bulk_normal(4 * H * H) / np.sqrt(H)).astype(np.float32)
    Uiou, Uf = U[: 3 * H * H].reshape(H, 3 * H), U[3 * H * H:].reshape(H, H)
    d_U, UT, UTp = g.devf(U), g.zeros(4 * H * H), g.zeros(4 * H * H, fill=-9.0)
    T = hip.Task
    jobs = [T(hip.TASK_TRANSPOSE, 0.0, H, 3 * H, 0, g.P(UT), g.P(d_U), None, None),
            T(hip.TASK_TRANSPOSE, 0.0, H, H, 0, g.P(UT) + 4 * 3 * H * H, g.P(d_U) + 4 * 3 * H * H, None, None),
            T(hip.TASK_PACK_T, 0.0, H, 3 * H, 0, g.P(UTp), g.P(d_U), None, None),
            T(hip.TASK_PACK_T, 0.0, H, H, 0, g.P(UTp) + 4 * 3 * H * H, g.P(d_U) + 4 * 3 * H * H, None, None)]
    g.call("cavs_run_tasks", len(jobs), (T * len(jobs))(*jobs), g.stream())
    got = g.host(UTp)
    np.testing.assert_array_equal(got[: 3 * H * H], pack_tiles(np.ascontiguousarray(Uiou.T)))
    np.testing.assert_array_equal(got[3 * H * H:], pack_tiles(np.ascontiguousarray(Uf.T)))

    mid0, top0 = L, L + m
    order = np.argsort(r.bulk_normal(L)).astype(np.int32)
    kids = np.full(2 * N, -1, np.int32)
    kids[2 * mid0: 2 * top0] = order[: 2 * m]
    top_kids = np.concatenate([np.arange(mid0, top0, dtype=np.int32), order[2 * m: 2 * m + 2 * n - m]])
    kids[2 * top0:] = top_kids[np.argsort(r.bulk_normal(2 * n))]
    gates = np.tanh(r.bulk_normal(N * 6 * H).reshape(N, 6 * H)).astype(np.float32)
    G = (r.bulk_normal(2 * N * 2 * H).reshape(2 * N, 2 * H) * 0.5).astype(np.float32)
    dret_rows = np.argsort(r.bulk_normal(N))[:N].astype(np.int32)
    dgo = r.bulk_normal(N * H).reshape(N, H)
    d_gates, d_G, d_dgo, d_rows, d_kids = g.devf(gates), g.devf(G), g.devf(dgo), g.devi(dret_rows), g.devi(kids)
    roots = g.devi(np.arange(top0, N, dtype=np.int32))
    outs = []
    for entry, W in (("cavs_treelstm_round_bwd_children_gates", UT), ("cavs_treelstm_round_bwd_children_gates_packed", UTp)):
        dxW, dF, dc = g.zeros(N, 4 * H, fill=-3.0), g.zeros(2 * N, H, fill=-3.0), g.zeros(N, H, fill=-3.0)
        g.call("cavs_treelstm_bwd_gates_rows", g.P(roots), n, g.P(d_dgo), g.P(d_rows), g.P(d_gates), g.P(d_G), g.P(dxW), 4 * H,
               g.P(dF), g.P(dc), L, H, g.stream())
        for lo, cnt in ((top0, n), (mid0, m)):
            assert hip.lib().cavs_round_packed_ok(cnt, H) == 1
            g.call(entry, g.P(dxW), 4 * H, g.P(dF), g.P(dc), g.P(W), g.P(d_kids) + 4 * 2 * lo, g.P(d_gates), g.P(d_G), g.P(d_dgo),
                   g.P(d_rows), lo, cnt, L, H, g.stream())
        outs.append((g.host(dxW), g.host(dF), g.host(dc)))
    for a, b, what in zip(outs[0], outs[1], ("dxW", "dF", "dc")):
        if min(n, m) <= 32:
            # rounds of at most 32 rows run on tiles of four rows, whose k slots are added up
            # after the loop instead of inside the MFMA: the same terms in another order
            close(b, a.astype(np.float64), what)
        else:
            np.testing.assert_array_equal(a, b, err_msg=what)
    assert (outs[0][0][:L] != -3.0).any()
    assert hip.lib().cavs_round_packed_ok(40, 96) == 0 and hip.lib().cavs_round_packed_ok(2000, 512) == 0
    with pytest.raises(hip.CavsError, match="cavs_round_packed_ok"):
        hip.call("cavs_treelstm_round_bwd_children_gates_packed", 16, 4 * 96, 16, 16, 16, 16, 16, 16, 16, 16, 0, 5, 0, 96, 0)


@pytest.mark.parametrize("n,H", [(40, 512), (300, 512), (1000, 512), (90, 128), (5, 1024), (1, 512), (4, 512), (13, 512), (16, 1024), (31, 512), (100, 512), (128, 1024)])
def test_packed_weights_give_the_same_forward_round_bit_for_bit(g, n, H):
    """The update-and-pack job against w - lr * g and the layout written out in numpy, then the
    forward launch reading the packed weights against the one reading the plain ones."""
    r = rng(29 * n + H)
    U = (r.bulk_normal(4 * H * H) / np.sqrt(H)).astype(np.float32)
    dU = r.bulk_normal(4 * H * H)
    lr = np.float32(0.125)
    d_U, d_plain, d_dU, Upk = g.devf(U), g.devf(U), g.devf(dU), g.zeros(4 * H * H, fill=-9.0)
    T = hip.Task
    at = 4 * 3 * H * H
    jobs = [T(hip.TASK_SGD_PACK, lr, H, 3 * H, 0, g.P(Upk), g.P(d_U), g.P(d_dU), None),
            T(hip.TASK_SGD_PACK, lr, H, H, 0, g.P(Upk) + at, g.P(d_U) + at, g.P(d_dU) + at, None),
            T(hip.TASK_SGD, lr, 4 * H * H, 0, 0, g.P(d_plain), g.P(d_dU), None, None)]
    g.call("cavs_run_tasks", len(jobs), (T * len(jobs))(*jobs), g.stream())
    U1 = g.host(d_U)
    np.testing.assert_array_equal(U1, g.host(d_plain))           # the same update as the plain job's
    close(U1, U - lr * dU, "updated weights")
    got = g.host(Upk)
    np.testing.assert_array_equal(got[: 3 * H * H], pack_tiles(U1[: 3 * H * H].reshape(H, 3 * H)))
    np.testing.assert_array_equal(got[3 * H * H:], pack_tiles(U1[3 * H * H:].reshape(H, H)))
    # without a gradient: the pack alone, the weights untouched
    again = g.zeros(4 * H * H, fill=-9.0)
    jobs = [T(hip.TASK_SGD_PACK, lr, H, 3 * H, 0, g.P(again), g.P(d_U), None, None),
            T(hip.TASK_SGD_PACK, lr, H, H, 0, g.P(again) + at, g.P(d_U) + at, None, None)]
    g.call("cavs_run_tasks", len(jobs), (T * len(jobs))(*jobs), g.stream())
    np.testing.assert_array_equal(g.host(again), got)
    np.testing.assert_array_equal(g.host(d_U), U1)

    P_rows = 2 * n + 5
    pool = (r.bulk_normal((P_rows + n) * 2 * H).reshape(P_rows + n, 2 * H) * 0.5).astype(np.float32)
    child = np.argsort(r.bulk_normal(P_rows))[: 2 * n].astype(np.int32)
    pair = (P_rows + np.arange(n)).astype(np.int32)
    child[min(3, 2 * n - 1)] = -1
    pair[n - 1] = -1
    d_child, d_pair = g.devi(child), g.devi(pair)
    d_xW, d_bias = g.devf(r.bulk_normal(n * 4 * H)), g.devf(r.bulk_normal(4 * H))
    d_rows = g.devi(np.argsort(r.bulk_normal(n + 3))[:n].astype(np.int32))
    assert hip.lib().cavs_round_packed_ok(n, H) == 1
    outs = []
    for packed in (False, True):
        d_pool = g.devf(pool)
        G, hlr, gates, msg, go = g.zeros(2 * n, 2 * H), g.zeros(n, H), g.zeros(n, 6 * H), g.zeros(n, 2 * H), g.zeros(n + 3, H, fill=-7.0)
        weights = (g.P(d_U), g.P(Upk)) if packed else (g.P(d_U),)
        g.call("cavs_treelstm_round_fwd_packed" if packed else "cavs_treelstm_round_fwd", g.P(d_pool), g.P(d_child), g.P(d_pair),
               g.P(d_xW), 4 * H, *weights, g.P(d_bias), g.P(G), g.P(hlr), g.P(gates), g.P(msg), g.P(go), g.P(d_rows), n, H, g.stream())
        outs.append([g.host(t) for t in (d_pool, G, hlr, gates, msg, go)])
    for a, b, what in zip(outs[0], outs[1], ("pool", "G", "hlr", "gates", "msg", "graph_out")):
        if n <= 32 and what not in ("G", "hlr"):
            # rounds of at most 32 rows run on tiles of four rows, whose k slots are added up
            # after the loop instead of inside the MFMA: the same terms in another order
            close(b, a.astype(np.float64), what)
        else:
            np.testing.assert_array_equal(a, b, err_msg=what)
    assert (outs[0][3] != 0).all()
    with pytest.raises(hip.CavsError, match="cavs_round_packed_ok"):
        hip.call("cavs_treelstm_round_fwd_packed", 16, 16, 16, 16, 4 * 96, 16, 16, 16, 16, 16, 16, 0, 0, 0, 5, 96, 0)
    with pytest.raises(hip.CavsError, match="bad shape to pack"):
        bad = T(hip.TASK_SGD_PACK, lr, 24, 64, 0, g.P(Upk), g.P(d_U), None, None)
        g.call("cavs_run_tasks", 1, (T * 1)(bad), g.stream())


@pytest.mark.parametrize("rows,cols", [(10000, 512), (1000, 32), (37, 70), (1, 5), (64, 64)])
def test_update_and_transposed_copy_in_one_job(g, rows, cols):
    """CAVS_TASK_SGD_TRANSPOSE: the weights after the job are those of the plain update job bit for
    bit and the copy is their transpose; without a gradient the job only copies."""
    r = rng(rows + 3 * cols)
    W, dW = r.bulk_normal(rows * cols).reshape(rows, cols), r.bulk_normal(rows * cols).reshape(rows, cols)
    lr = np.float32(0.375)
    d_W, d_plain, d_dW, WT = g.devf(W), g.devf(W), g.devf(dW), g.zeros(cols, rows, fill=-9.0)
    T = hip.Task
    jobs = [T(hip.TASK_SGD_TRANSPOSE, lr, rows, cols, 0, g.P(WT), g.P(d_W), g.P(d_dW), None),
            T(hip.TASK_SGD, lr, rows * cols, 0, 0, g.P(d_plain), g.P(d_dW), None, None)]
    g.call("cavs_run_tasks", len(jobs), (T * len(jobs))(*jobs), g.stream())
    W1 = g.host(d_W)
    np.testing.assert_array_equal(W1, g.host(d_plain))
    close(W1, W.astype(np.float64) - float(lr) * dW.astype(np.float64), "updated weights")
    np.testing.assert_array_equal(g.host(WT), W1.T)
    again = g.zeros(cols, rows, fill=-9.0)
    g.call("cavs_run_tasks", 1, (T * 1)(T(hip.TASK_SGD_TRANSPOSE, lr, rows, cols, 0, g.P(again), g.P(d_W), None, None)), g.stream())
    np.testing.assert_array_equal(g.host(again), W1.T)
    np.testing.assert_array_equal(g.host(d_W), W1)
    with pytest.raises(hip.CavsError, match="aliased"):
        g.call("cavs_run_tasks", 1, (T * 1)(T(hip.TASK_SGD_TRANSPOSE, lr, rows, cols, 0, g.P(d_W), g.P(d_W), None, None)), g.stream())


@pytest.mark.parametrize("L,m,n,H", [(300, 90, 100, 256), (200, 30, 40, 512), (500, 128, 128, 512), (1500, 500, 600, 256)])
def test_packed_weights_give_the_same_chain_lstm_rounds_bit_for_bit(g, L, m, n, H):
    """Chain LSTM: the forward launch and the folded backward launch reading W' / W'^T tile-major
    against the ones reading them row-major (themselves checked against the oracle above)."""
    r = rng(31 * L + n + H)
    N = L + m + n
    Wh = (r.bulk_normal(4 * H * H) / np.sqrt(H)).astype(np.float32)          # W' [H, 4H]
    d_Wh, WhT, Whp, WhTp = g.devf(Wh), g.zeros(4 * H * H), g.zeros(4 * H * H), g.zeros(4 * H * H)
    T = hip.Task
    jobs = [T(hip.TASK_TRANSPOSE, 0.0, H, 4 * H, 0, g.P(WhT), g.P(d_Wh), None, None),
            T(hip.TASK_PACK_T, 0.0, H, 4 * H, 0, g.P(WhTp), g.P(d_Wh), None, None),
            T(hip.TASK_SGD_PACK, 0.0, H, 4 * H, 0, g.P(Whp), g.P(d_Wh), None, None)]
    g.call("cavs_run_tasks", len(jobs), (T * len(jobs))(*jobs), g.stream())
    np.testing.assert_array_equal(g.host(Whp), pack_tiles(Wh.reshape(H, 4 * H)))
    np.testing.assert_array_equal(g.host(WhTp), pack_tiles(np.ascontiguousarray(Wh.reshape(H, 4 * H).T)))
    assert hip.lib().cavs_lstm_round_packed_ok(n, H) == 1 and hip.lib().cavs_lstm_round_packed_ok(m, H) == 1

    # forward: one round of n vertices over a pool of L + m earlier rows
    pool = (r.bulk_normal((N + 2) * 2 * H).reshape(N + 2, 2 * H) * 0.5).astype(np.float32)
    child = np.argsort(r.bulk_normal(L + m))[:n].astype(np.int32)
    child[1] = -1
    pair = (L + m + np.arange(n)).astype(np.int32)
    pair[n - 1] = -1
    d_child, d_pair = g.devi(child), g.devi(pair)
    d_xW, d_bias = g.devf(r.bulk_normal(n * 4 * H)), g.devf(r.bulk_normal(4 * H))
    d_out = g.devi(np.argsort(r.bulk_normal(n + 3))[:n].astype(np.int32))
    outs = []
    for entry, W in (("cavs_lstm_round_fwd", d_Wh), ("cavs_lstm_round_fwd_packed", Whp)):
        d_pool = g.devf(pool)
        G, gates, msg, go = g.zeros(n, 2 * H), g.zeros(n, 5 * H), g.zeros(n, 2 * H), g.zeros(n + 3, H, fill=-7.0)
        g.call(entry, g.P(d_pool), g.P(d_child), g.P(d_pair), g.P(d_xW), 4 * H, g.P(W), g.P(d_bias), g.P(G), g.P(gates), g.P(msg),
               g.P(go), g.P(d_out), n, H, g.stream())
        outs.append([g.host(t) for t in (d_pool, G, gates, msg, go)])
    for a, b, what in zip(outs[0], outs[1], ("pool", "G", "gates", "msg", "graph_out")):
        np.testing.assert_array_equal(a, b, err_msg=what)
    assert (outs[0][2] != 0).all()

    # backward: the top n rows from the row-list launch, then two folded launches (top, middle)
    order = np.argsort(r.bulk_normal(L)).astype(np.int32)
    kids = np.full(N, -1, np.int32)
    kids[L: L + m] = order[:m]
    top_kids = np.concatenate([np.arange(L, L + m, dtype=np.int32), order[m: n]]) if n > m else np.arange(L, L + n, dtype=np.int32)
    kids[L + m:] = top_kids[np.argsort(r.bulk_normal(n))]
    gates = np.tanh(r.bulk_normal(N * 5 * H).reshape(N, 5 * H)).astype(np.float32)
    G = (r.bulk_normal(N * 2 * H).reshape(N, 2 * H) * 0.5).astype(np.float32)
    d_gates, d_G, d_kids = g.devf(gates), g.devf(G), g.devi(kids)
    d_dgo, d_rows = g.devf(r.bulk_normal(N * H)), g.devi(np.argsort(r.bulk_normal(N)).astype(np.int32))
    roots = g.devi(np.arange(L + m, N, dtype=np.int32))
    outs = []
    for entry, W in (("cavs_lstm_round_bwd_children_gates", WhT), ("cavs_lstm_round_bwd_children_gates_packed", WhTp)):
        dA, dc = g.zeros(N, 4 * H, fill=-3.0), g.zeros(N, H, fill=-3.0)
        g.call("cavs_lstm_bwd_gates_rows", g.P(roots), n, g.P(d_dgo), g.P(d_rows), g.P(d_gates), g.P(d_G), g.P(dA), 4 * H, g.P(dc), L, H,
               g.stream())
        for lo, cnt in ((L + m, n), (L, m)):
            g.call(entry, g.P(dA), 4 * H, g.P(dc), g.P(W), g.P(d_kids) + 4 * lo, g.P(d_gates), g.P(d_G), g.P(d_dgo), g.P(d_rows), lo, cnt,
                   L, H, g.stream())
        outs.append((g.host(dA), g.host(dc)))
    np.testing.assert_array_equal(outs[0][0], outs[1][0], err_msg="dA")
    np.testing.assert_array_equal(outs[0][1], outs[1][1], err_msg="dc")
    assert (outs[0][0][order[:m]] != -3.0).all()
    assert hip.lib().cavs_lstm_round_packed_ok(16, 128) == 0 and hip.lib().cavs_lstm_round_packed_ok(100, 128) == 0
    with pytest.raises(hip.CavsError, match="cavs_lstm_round_packed_ok"):
        hip.call("cavs_lstm_round_fwd_packed", 16, 16, 16, 16, 4 * 128, 16, 16, 16, 16, 16, 0, 0, 16, 128, 0)
    with pytest.raises(hip.CavsError, match="cavs_lstm_round_packed_ok"):
        hip.call("cavs_lstm_round_bwd_children_gates_packed", 16, 4 * 128, 16, 16, 16, 16, 16, 16, 16, 0, 16, 0, 128, 0)


def test_fused_round_entry_points_reject_bad_shapes():
    with pytest.raises(hip.CavsError, match="multiple of 32"):
        hip.call("cavs_treelstm_round_fwd", 0, 0, 0, 0, 4 * 24, 0, 0, 0, 0, 0, 0, 0, 0, 5, 24, 0)
    with pytest.raises(hip.CavsError, match="multiple of 32"):
        hip.call("cavs_treelstm_round_bwd_children", 0, 4 * 24, 0, 0, 0, 0, 5, 24, 0)
    with pytest.raises(hip.CavsError, match="all set"):
        hip.call("cavs_treelstm_round_bwd_gates", 16, 16, 16, 16, 0, 16, 0, 16, 4 * 32, 0, 5, 32, 0)
    with pytest.raises(hip.CavsError, match="multiple of 32"):
        hip.call("cavs_treelstm_round_bwd_children_gates", 16, 4 * 24, 16, 16, 16, 16, 16, 16, 16, 16, 0, 5, 0, 24, 0)
    with pytest.raises(hip.CavsError, match="null pointer"):
        hip.call("cavs_treelstm_bwd_gates_rows", 0, 5, 16, 16, 16, 16, 16, 4 * 32, 16, 16, 0, 32, 0)


@pytest.mark.parametrize("n,H,C_", [(1, 64, 2), (19, 96, 5), (2482, 512, 5), (300, 100, 8), (77, 1024, 3)])
def test_fused_classifier_head(g, oracle, n, H, C_):
    """FullyConnected + softmax cross-entropy and their gradients in two launches, against
    the oracle's GEMM, softmax and column-sum pieces."""
    import ctypes as C

    r = rng(n + H + C_)
    X = r.bulk_normal(n * H).reshape(n, H)
    W = (r.bulk_normal(C_ * H).reshape(C_, H) / np.sqrt(H)).astype(np.float32)
    b = r.bulk_normal(C_)
    labels = np.floor(r.bulk_uniform(n) * C_).astype(np.float32)
    logits_w = oracle.sgemm(0, 1, X, W) + b[None, :]
    loss_w, d_w = oracle.softmax_xent(logits_w, labels)
    dX_w = oracle.sgemm(0, 0, d_w, W)
    dW_w = oracle.sgemm(1, 0, d_w, X)
    db_w = d_w.astype(np.float64).sum(0)
    nb = hip.lib().cavs_fc_softmax_xent_workspace(n, H, C_)
    assert nb > 0
    ws = g.zeros(nb // 4)
    loss, logits, dX, dW, db = g.zeros(n), g.zeros(n, C_), g.zeros(n, H), g.zeros(C_, H), g.zeros(C_)
    args = (g.P(g.devf(X)), g.P(g.devf(W)), g.P(g.devf(b)), g.P(g.devf(labels)), g.P(loss), g.P(logits))
    g.call("cavs_fc_softmax_xent", *args, g.P(dX), g.P(dW), g.P(db), g.P(ws), nb, n, H, C_, g.stream())
    close(g.host(logits), logits_w, "logits")
    close(g.host(loss), loss_w, "loss")
    close(g.host(dX), dX_w, "dX", atol=1e-7)
    close(g.host(dW), dW_w, "dW", atol=1e-6)
    close(g.host(db), db_w, "db", atol=1e-6)
    # dX alone: the weight-gradient partials stay in the workspace and a job of the multi-job
    # launch adds them up -- the same sums, bit for bit
    dX2, dW2, db2 = g.zeros(n, H), g.zeros(C_, H), g.zeros(C_)
    ws2 = g.zeros(nb // 4)
    g.call("cavs_fc_softmax_xent", *args, g.P(dX2), None, None, g.P(ws2), nb, n, H, C_, g.stream())
    parts = hip.lib().cavs_fc_softmax_xent_parts(n)
    assert parts * (C_ * H + C_) * 4 == nb
    job = hip.Task(hip.TASK_SUM_PARTS, 0.0, parts, C_ * H + C_, C_ * H, g.P(ws2), g.P(dW2), g.P(db2), None)
    g.call("cavs_run_tasks", 1, (hip.Task * 1)(job), g.stream())
    for a, b2, what in ((dX2, dX, "dX"), (dW2, dW, "dW"), (db2, db, "db")):
        np.testing.assert_array_equal(g.host(a), g.host(b2), what)
    # forward only: no gradient buffers, no workspace
    loss2 = g.zeros(n)
    g.call("cavs_fc_softmax_xent", *args[:4], g.P(loss2), None, None, None, None, None, 0, n, H, C_, g.stream())
    np.testing.assert_array_equal(g.host(loss2), g.host(loss))
    assert hip.lib().cavs_fc_softmax_xent_workspace(10, 512, 9) == 0      # too many classes
    assert hip.lib().cavs_fc_softmax_xent_workspace(10, 4096, 5) == 0     # accumulators exceed LDS
    with pytest.raises(hip.CavsError, match="unsupported shape"):
        hip.call("cavs_fc_softmax_xent", 16, 16, 16, 16, 16, 0, 0, 0, 0, 0, 0, 4, 512, 9, 0)


def test_sgd_over_several_tensors_and_sparse_embedding_update(g):
    import ctypes as C

    r = rng(11)
    sizes = [5, 1000, 0, 77777, 3, 64, 512, 129, 1, 4096]      # more than one batch of eight, one empty
    ws = [r.bulk_normal(max(k, 1))[:k] for k in sizes]
    gs = [r.bulk_normal(max(k, 1))[:k] for k in sizes]
    dw, dg = [g.devf(a) if len(a) else None for a in ws], [g.devf(a) if len(a) else None for a in gs]
    pw = (C.c_void_p * len(sizes))(*[g.P(t) for t in dw])
    pg = (C.c_void_p * len(sizes))(*[g.P(t) for t in dg])
    pn = (C.c_size_t * len(sizes))(*sizes)
    g.call("cavs_sgd_multi", len(sizes), pw, pg, pn, 0.25, g.stream())
    for a, b, t in zip(ws, gs, dw):
        if len(a):
            np.testing.assert_array_equal(g.host(t), a - np.float32(0.25) * b)

    # the row-sparse update equals the dense one when the gradient is zero off the listed rows
    V, E, n = 500, 37, 120
    table = r.bulk_normal(V * E).reshape(V, E)
    ids = np.floor(r.bulk_uniform(n) * V).astype(np.float32)
    ids[:40] = ids[0]                                           # one row looked up many times
    grad = np.zeros((V, E), np.float32)
    rows = np.unique(ids.astype(np.int64))
    grad[rows] = r.bulk_normal(len(rows) * E).reshape(len(rows), E)
    stamp = g.devi(np.zeros(V, np.int32))
    t, dgrad, dids = g.devf(table), g.devf(grad), g.devf(ids)
    want = table.copy()
    for epoch in (1, 2):                                        # a second step must update again
        g.call("cavs_embed_sgd", g.P(t), g.P(dgrad), g.P(dids), n, E, 0.5, g.P(stamp), epoch, g.stream())
        want = want - np.float32(0.5) * grad
        np.testing.assert_array_equal(g.host(t), want)
    g.call("cavs_embed_zero_rows", g.P(dgrad), g.P(dids), n, E, g.stream())
    assert not g.host(dgrad).any()


def test_several_small_jobs_in_one_launch(g):
    """cavs_run_tasks: transposes, clearing of looked-up rows, dense SGD updates and the row-sparse
    embedding update as one launch give what the separate entry points give (bit-exact)."""
    r = rng(23)
    A, B = r.bulk_normal(70 * 33).reshape(70, 33), r.bulk_normal(64 * 192).reshape(64, 192)
    V, E, n = 300, 41, 90
    ids = np.floor(r.bulk_uniform(n) * V).astype(np.float32)
    ids[:30] = ids[0]
    rows = np.unique(ids.astype(np.int64))
    dirty = r.bulk_normal(V * E).reshape(V, E)                  # to be cleared in the listed rows only
    table = r.bulk_normal(V * E).reshape(V, E)
    grad = np.zeros((V, E), np.float32)
    grad[rows] = r.bulk_normal(len(rows) * E).reshape(len(rows), E)
    w1, g1 = r.bulk_normal(100003), r.bulk_normal(100003)
    w2, g2 = r.bulk_normal(7), r.bulk_normal(7)
    dA, dB, dAT, dBT = g.devf(A), g.devf(B), g.zeros(33, 70), g.zeros(192, 64)
    d_dirty, d_ids, d_table, d_grad = g.devf(dirty), g.devf(ids), g.devf(table), g.devf(grad)
    d_w1, d_g1, d_w2, d_g2 = g.devf(w1), g.devf(g1), g.devf(w2), g.devf(g2)
    stamp = g.devi(np.zeros(V, np.int32))
    T = hip.Task
    jobs = [T(hip.TASK_TRANSPOSE, 0.0, 70, 33, 0, g.P(dAT), g.P(dA), None, None),
            T(hip.TASK_SGD, 0.25, 100003, 0, 0, g.P(d_w1), g.P(d_g1), None, None),
            T(hip.TASK_ZERO_ROWS, 0.0, n, E, 0, g.P(d_dirty), g.P(d_ids), None, None),
            T(hip.TASK_TRANSPOSE, 0.0, 64, 192, 0, g.P(dBT), g.P(dB), None, None),
            T(hip.TASK_SGD, 0.5, 0, 0, 0, None, None, None, None),                     # an empty job is skipped
            T(hip.TASK_EMBED_SGD, 0.5, n, E, 1, g.P(d_table), g.P(d_grad), g.P(d_ids), g.P(stamp)),
            T(hip.TASK_SGD, 2.0, 7, 0, 0, g.P(d_w2), g.P(d_g2), None, None)]
    g.call("cavs_run_tasks", len(jobs), (T * len(jobs))(*jobs), g.stream())
    np.testing.assert_array_equal(g.host(dAT), A.T)
    np.testing.assert_array_equal(g.host(dBT), B.T)
    np.testing.assert_array_equal(g.host(d_w1), w1 - np.float32(0.25) * g1)
    np.testing.assert_array_equal(g.host(d_w2), w2 - np.float32(2.0) * g2)
    want = dirty.copy()
    want[rows] = 0
    np.testing.assert_array_equal(g.host(d_dirty), want)
    np.testing.assert_array_equal(g.host(d_table), table - np.float32(0.5) * grad)
    # a gradient that arrives in another block order than its parameter's
    bw, perm = 37, [0, 3, 2, 1]
    src, wb = r.bulk_normal(4 * bw), r.bulk_normal(4 * bw)
    d_src, d_wb, d_gb = g.devf(src), g.devf(wb), g.zeros(4 * bw)
    code = sum(d << (4 * k) for k, d in enumerate(perm))
    g.call("cavs_run_tasks", 1, (T * 1)(T(hip.TASK_BLOCKS_SGD, 0.5, bw, 4, code, g.P(d_wb), g.P(d_src), g.P(d_gb), None)), g.stream())
    want_g = np.empty(4 * bw, np.float32)
    for k, d in enumerate(perm):
        want_g[d * bw:(d + 1) * bw] = src[k * bw:(k + 1) * bw]
    np.testing.assert_array_equal(g.host(d_gb), want_g)
    np.testing.assert_array_equal(g.host(d_wb), wb - np.float32(0.5) * want_g)
    # the gate gradients of listed slab rows (the roots) as a job, beside a transpose: what the
    # entry point of their own gives, bit for bit
    R, H, leaf_rows = 20, 32, 5
    rows_l = np.array([19, 2, 7, 11, 0, 5, 16], np.int32)
    dret_rows = np.argsort(r.bulk_uniform(R)).astype(np.int32)
    gates, Gm, dgo = r.bulk_uniform(R * 6 * H), r.bulk_normal(2 * R * 2 * H), r.bulk_normal(R * H)
    d_rows_l, d_dret_rows, d_gates, d_Gm, d_dgo = g.devi(rows_l), g.devi(dret_rows), g.devf(gates), g.devf(Gm), g.devf(dgo)
    outs = []
    for as_job in (False, True):
        dxW, dF, dc = g.devf(np.full(R * 4 * H, 7, np.float32)), g.devf(np.full(2 * R * H, 7, np.float32)), g.devf(np.full(R * H, 7, np.float32))
        if as_job:
            jobs = [T(hip.TASK_TRANSPOSE, 0.0, 70, 33, 0, g.P(dAT), g.P(dA), None, None),
                    T(hip.TASK_TREELSTM_GATES_ROWS, 0.0, len(rows_l), H, leaf_rows | ((4 * H) << 32), g.P(d_rows_l), g.P(d_dgo),
                      g.P(d_dret_rows), g.P(d_gates), g.P(d_Gm), g.P(dxW), g.P(dF), g.P(dc))]
            g.call("cavs_run_tasks", len(jobs), (T * len(jobs))(*jobs), g.stream())
        else:
            g.call("cavs_treelstm_bwd_gates_rows", g.P(d_rows_l), len(rows_l), g.P(d_dgo), g.P(d_dret_rows), g.P(d_gates), g.P(d_Gm),
                   g.P(dxW), 4 * H, g.P(dF), g.P(dc), leaf_rows, H, g.stream())
        outs.append((g.host(dxW), g.host(dF), g.host(dc)))
    for a_, b_ in zip(*outs):
        assert (a_ != 7).any()
        np.testing.assert_array_equal(a_, b_)
    with pytest.raises(hip.CavsError, match="null pointer"):
        g.call("cavs_run_tasks", 1, (T * 1)(T(hip.TASK_TREELSTM_GATES_ROWS, 0.0, 3, H, leaf_rows | ((4 * H) << 32), g.P(d_rows_l), g.P(d_dgo),
                                              g.P(d_dret_rows), g.P(d_gates))), g.stream())
    with pytest.raises(hip.CavsError, match="not a permutation"):
        g.call("cavs_run_tasks", 1, (T * 1)(T(hip.TASK_BLOCKS_SGD, 0.5, bw, 4, 0, g.P(d_wb), g.P(d_src), g.P(d_gb), None)), g.stream())
    with pytest.raises(hip.CavsError, match="unknown kind"):
        g.call("cavs_run_tasks", 1, (T * 1)(T(99, 0.0, 1, 1, 0, g.P(dA), g.P(dB), None, None)), g.stream())
    with pytest.raises(hip.CavsError, match="at most 12"):
        g.call("cavs_run_tasks", 14, (T * 14)(), g.stream())
    with pytest.raises(hip.CavsError, match="more than 12 jobs"):
        g.call("cavs_run_tasks", 13, (T * 13)(*[T(hip.TASK_SGD, 0.5, 4, 0, 0, g.P(dA), g.P(dB), None, None)] * 13), g.stream())


@pytest.mark.parametrize("n,bw,perm", [(1, 4, [0]), (2482, 512, [0, 3, 2, 1]), (63, 6, [2, 0, 1]), (5000, 64, [1, 0])])
def test_column_sums_of_permuted_blocks(g, n, bw, perm):
    import ctypes as C

    r = rng(n + bw)
    nb = len(perm)
    ld = bw * nb + 8
    X = r.bulk_normal(n * ld).reshape(n, ld)
    exact = X[:, : bw * nb].astype(np.float64).sum(0).reshape(nb, bw)
    want = np.zeros((nb, bw))
    for k, d in enumerate(perm):
        want[d] = exact[k]
    nbytes = hip.lib().cavs_colsum_blocks_workspace(n, bw, nb)
    ws, out = g.zeros(nbytes // 4), g.zeros(nb * bw, fill=float("nan"))
    dst = (C.c_int * nb)(*perm)
    dX = g.devf(X)
    g.call("cavs_colsum_blocks", g.P(out), g.P(dX), ld, n, bw, nb, dst, g.P(ws), nbytes, g.stream())
    first = g.host(out).copy()
    close(first, want.ravel())
    g.call("cavs_colsum_blocks", g.P(out), g.P(dX), ld, n, bw, nb, dst, g.P(ws), nbytes, g.stream())
    np.testing.assert_array_equal(g.host(out), first)           # fixed summation order
    # the same in two halves: the chunk sums left in the workspace, added up (permuted, and
    # applied to a parameter) by a job of the launch that ends a step
    parts = hip.lib().cavs_colsum_parts(n)
    assert 1 <= parts and parts * bw * nb * 4 == nbytes
    g.call("cavs_colsum_blocks", None, g.P(dX), ld, n, bw, nb, None, g.P(ws), nbytes, g.stream())
    w0 = r.bulk_normal(nb * bw)
    d_w, out2 = g.devf(w0), g.zeros(nb * bw, fill=float("nan"))
    bmap = sum(d << (4 * k) for k, d in enumerate(perm)) | (parts << 32)
    job = (hip.Task * 1)(hip.Task(hip.TASK_BLOCKS_SGD, 0.5, bw, nb, bmap, g.P(d_w), g.P(ws), g.P(out2), None))
    g.call("cavs_run_tasks", 1, job, g.stream())
    second = g.host(out2).copy()
    close(second, want.ravel())
    np.testing.assert_array_equal(g.host(d_w), w0 - np.float32(0.5) * second)
    job[0].p0 = None                                            # gradient only, again: same bits
    g.call("cavs_run_tasks", 1, job, g.stream())
    np.testing.assert_array_equal(g.host(out2), second)
    with pytest.raises(hip.CavsError, match="permutation"):
        hip.call("cavs_colsum_blocks", 16, 16, ld, n, bw, nb, (C.c_int * nb)(*([0] * nb)), 16, nbytes, 0) if nb > 1 else \
            hip.call("cavs_colsum_blocks", 16, 16, ld, n, bw, nb, (C.c_int * 1)(3), 16, nbytes, 0)


@pytest.mark.parametrize("n,H,K,nchild", [(1, 32, 128, 1), (40, 64, 256, 1), (130, 32, 32, 2), (300, 64, 64, 2), (17, 96, 96, 2),
                                          # k ranges of whole pipeline stages: the loops that fetch B through buffer loads
                                          (130, 64, 256, 1), (40, 64, 512, 2), (64, 32, 1024, 1), (700, 32, 512, 2)])
def test_children_gradient_product_with_scatter(g, n, H, K, nchild):
    """dpool[child[b*nchild+p]][0:H) = dA[b] * BT[:, p*H:(p+1)*H): product and Scatter in one launch."""
    r = rng(n + H + K)
    dA = r.bulk_normal(n * (K + 4)).reshape(n, K + 4)           # leading dimension wider than K
    BT = (r.bulk_normal(K * nchild * H).reshape(K, nchild * H) / np.sqrt(K)).astype(np.float32)
    rows = nchild * n + 7
    mw = 2 * H if nchild == 1 else H
    child = np.argsort(r.bulk_normal(rows))[: nchild * n].astype(np.int32)
    if n > 2:
        child[1] = -1
    dpool = r.bulk_normal(rows * mw).reshape(rows, mw)
    want = dpool.astype(np.float64).copy()
    full = dA[:, :K].astype(np.float64) @ BT.astype(np.float64)  # [n, nchild*H]
    for b in range(n):
        for p in range(nchild):
            c = child[b * nchild + p]
            if c >= 0:
                want[c, :H] = full[b, p * H:(p + 1) * H]
    d = g.devf(dpool)
    g.call("cavs_round_bwd_children", g.P(g.devf(dA)), K + 4, K, g.P(g.devf(BT)), nchild * H, nchild, g.P(g.devi(child)),
           g.P(d), mw, n, H, g.stream())
    close(g.host(d), want, "dpool")


@pytest.mark.parametrize("model,L,m,n,H", [("lstm", 20, 2, 3, 32), ("lstm", 300, 60, 70, 64), ("lstm", 2600, 600, 1100, 32),
                                           ("treefc", 20, 5, 3, 32), ("treefc", 400, 100, 70, 64), ("treefc", 2600, 100, 1100, 32),
                                           ("treefc", 900, 200, 130, 96),
                                           # hidden sizes whose k ranges are whole pipeline stages (buffer-load loops)
                                           ("lstm", 300, 60, 70, 256), ("treefc", 400, 100, 70, 256), ("treefc", 300, 60, 40, 512)])
def test_chain_and_tree_fc_backward_rounds_with_the_childrens_pointwise_part_folded_in(g, oracle, model, L, m, n, H):
    """The construction of the Tree-LSTM test above for the other two vertex functions: three
    levels over whole-batch slabs, the top rows from the row-list launch, then one launch per
    round, against the chain composed round by round from the oracle's functions."""
    r = rng(13 * L + 5 * n + H + len(model))
    nch = 1 if model == "lstm" else 2
    N = L + m + n
    mid0, top0 = L, L + m
    order = np.argsort(r.bulk_normal(L)).astype(np.int32)
    kids = np.full(nch * N, -1, np.int32)
    kids[nch * mid0: nch * top0] = order[: nch * m]
    assert m <= nch * n - 1 and nch * m + nch * n - m <= L
    top_kids = np.concatenate([np.arange(mid0, top0, dtype=np.int32), order[nch * m: nch * m + nch * n - m]])
    top_kids = top_kids[np.argsort(r.bulk_normal(nch * n))]
    top_kids[np.flatnonzero(top_kids < L)[0]] = -1
    kids[nch * top0:] = top_kids
    dret_rows = np.argsort(r.bulk_normal(N + 3))[:N].astype(np.int32)
    dgo = r.bulk_normal((N + 3) * H).reshape(N + 3, H)
    act = 1 if L in (400, 900) else 0
    if model == "lstm":
        sig = lambda a: (1.0 / (1.0 + np.exp(-a))).astype(np.float32)
        gates = r.bulk_normal(N * 5 * H).reshape(N, 5 * H)
        gates[:, : 2 * H] = sig(gates[:, : 2 * H])
        gates[:, 2 * H: 3 * H] = np.tanh(gates[:, 2 * H: 3 * H])
        gates[:, 3 * H: 4 * H] = sig(gates[:, 3 * H: 4 * H])
        gates[:, 4 * H:] = np.tanh(gates[:, 4 * H:])
        G = (r.bulk_normal(N * 2 * H).reshape(N, 2 * H) * 0.5).astype(np.float32)
        G[:L] = 0
        W = (r.bulk_normal(H * 4 * H).reshape(H, 4 * H) / np.sqrt(H)).astype(np.float32)   # W' [H,4H]
        K, wd = 4 * H, 2 * H
    else:
        h = np.tanh(r.bulk_normal(N * H).reshape(N, H)).astype(np.float32)                 # relu: sign of h decides
        W = (r.bulk_normal(2 * H * H).reshape(2 * H, H) / np.sqrt(H)).astype(np.float32)   # W [2H,H]
        K, wd = H, H
    WT = np.ascontiguousarray(W.T)                                                         # [K, nch*H]

    dmsg = np.zeros((N, wd), np.float32)
    reached = np.zeros(N, bool)
    reached[top0:] = True
    dA_w = np.zeros((N, K), np.float32)
    for lo, hi in ((top0, N), (mid0, top0), (0, L)):
        if model == "lstm":
            a, c = oracle.lstm_gates_bwd(dmsg[lo:hi], dgo[dret_rows[lo:hi]], gates[lo:hi], G[lo:hi])
        else:
            a = oracle.treefc_bwd(dmsg[lo:hi], dgo[dret_rows[lo:hi]], h[lo:hi], act)
        dA_w[lo:hi] = a
        if lo == 0:
            break
        dh = oracle.sgemm(0, 0, a, WT)                       # [rows, nch*H]
        k = kids[nch * lo: nch * hi]
        if model == "lstm":
            c[:, :H] = dh
            dmsg[k[k >= 0]] = c[k >= 0]
        else:
            dmsg[k[k >= 0]] = dh.reshape(-1, H)[k >= 0]
        reached[k[k >= 0]] = True

    dA, dc = g.zeros(N, K, fill=-3.0), g.zeros(N, H, fill=-3.0)
    d_dgo, d_rows, d_kids, d_WT = g.devf(dgo), g.devi(dret_rows), g.devi(kids), g.devf(WT)
    roots = g.devi(np.arange(top0, N, dtype=np.int32))
    if model == "lstm":
        d_gates, d_G = g.devf(gates), g.devf(G)
        g.call("cavs_lstm_bwd_gates_rows", g.P(roots), n, g.P(d_dgo), g.P(d_rows), g.P(d_gates), g.P(d_G), g.P(dA), K, g.P(dc), L, H,
               g.stream())
    else:
        d_h = g.devf(h)
        g.call("cavs_treefc_bwd_rows", g.P(roots), n, g.P(d_dgo), g.P(d_rows), g.P(d_h), g.P(dA), H, act, g.stream())
    close(g.host(dA)[top0:], dA_w[top0:], "top rows")
    assert (g.host(dA)[:top0] == -3.0).all()
    for lo, cnt in ((top0, n), (mid0, m)):
        if model == "lstm":
            g.call("cavs_lstm_round_bwd_children_gates", g.P(dA), K, g.P(dc), g.P(d_WT), g.P(d_kids) + 4 * lo, g.P(d_gates), g.P(d_G),
                   g.P(d_dgo), g.P(d_rows), lo, cnt, L, H, g.stream())
        else:
            g.call("cavs_treefc_round_bwd_children_act", g.P(dA), g.P(d_WT), g.P(d_kids) + 4 * 2 * lo, g.P(d_h), g.P(d_dgo), g.P(d_rows),
                   lo, cnt, H, act, g.stream())
    got = g.host(dA)
    close(got[reached], dA_w[reached], "dA")
    assert (got[~reached] == -3.0).all()
    assert (g.host(dc)[:L] == -3.0).all()


def test_gradient_clipping_by_the_sum_of_norms(g):
    """Clip of the reference: every tensor times clip / max(sum of the tensors' 2-norms, clip)."""
    import ctypes as C

    r = rng(17)
    sizes = [5, 70000, 0, 333, 1]
    gs = [r.bulk_normal(max(k, 1))[:k] for k in sizes]
    total = sum(float(np.sqrt((a.astype(np.float64) ** 2).sum())) for a in gs)
    nb = hip.lib().cavs_clip_grads_workspace(len(sizes))
    for clip in (0.5 * total, 10 * total):            # active, then inactive (factor exactly 1)
        ws = g.zeros(nb // 4)
        dg = [g.devf(a) if len(a) else None for a in gs]
        pg = (C.c_void_p * len(sizes))(*[g.P(t) for t in dg])
        pn = (C.c_size_t * len(sizes))(*sizes)
        g.call("cavs_clip_grads", len(sizes), pg, pn, clip, g.P(ws), nb, g.stream())
        factor, norm_sum = g.host(ws)[512], g.host(ws)[513]
        assert abs(norm_sum - total) <= 1e-5 * total
        want = clip / max(total, clip)
        assert abs(factor - want) <= 1e-6
        for a, t in zip(gs, dg):
            if len(a):
                close(g.host(t), a * np.float32(factor), "scaled gradient", rtol=1e-6, atol=1e-7)
    with pytest.raises(hip.CavsError, match="bad arguments"):
        hip.call("cavs_clip_grads", 1, 16, 16, 0.0, 16, nb, 0)


def test_kernel_stamped_timing_probe(g):
    """cavs_profile_arm: the kernels of the next entry points stamp start / stop themselves;
    disarm reports whether anything was launched."""
    import ctypes as C

    e0, e1 = C.c_void_p(), C.c_void_p()
    hip.call("cavs_event_create", C.byref(e0))
    hip.call("cavs_event_create", C.byref(e1))
    n = 1 << 22
    a, out = g.zeros(n, fill=1.0), g.zeros(n)
    launched = C.c_int(-1)
    hip.call("cavs_profile_arm", e0, e1)
    hip.call("cavs_profile_disarm", C.byref(launched))
    assert launched.value == 0                       # armed, nothing launched
    hip.call("cavs_profile_arm", e0, e1)
    g.call("cavs_scale", g.P(out), g.P(a), 2.0, n, g.stream())
    g.call("cavs_scale", g.P(out), g.P(out), 2.0, n, g.stream())   # stop moves to the last kernel
    hip.call("cavs_profile_disarm", C.byref(launched))
    assert launched.value == 1
    ms = C.c_float(-1)
    hip.call("cavs_event_elapsed_ms", C.byref(ms), e0, e1)
    # two passes over 16 MiB in and out: at least 8 us at 8 TB/s, and far below a millisecond
    assert 0.008 <= ms.value < 1.0, ms.value
    np.testing.assert_array_equal(g.host(out)[:4], np.full(4, 4.0, np.float32))
    g.call("cavs_scale", g.P(out), g.P(a), 3.0, n, g.stream())     # disarmed: plain launch
    assert g.host(out)[0] == 3.0
    hip.call("cavs_event_destroy", e0)
    hip.call("cavs_event_destroy", e1)
    with pytest.raises(hip.CavsError, match="null event"):
        hip.call("cavs_profile_arm", None, None)
