"""Pins the op restatements in oracle/ops.c against numpy / torch closed forms."""
import numpy as np
import pytest
import torch

from cavs_amd import synth


def _rng(seed):
    return synth.SplitMix64(seed)


def test_row_copies_are_permutation_closed_forms(oracle):
    r = _rng(1)
    src = r.bulk_normal(40 * 24).reshape(40, 24)
    perm = np.argsort(r.bulk_uniform(40)).astype(np.int32)
    g = oracle.gather_rows(src, perm)
    np.testing.assert_array_equal(g, src[perm])
    out = np.zeros_like(src)
    oracle.scatter_rows(out, perm, g)  # scatter o gather on a permutation = identity
    np.testing.assert_array_equal(out, src)
    # column sub-block through the leading dimension
    np.testing.assert_array_equal(oracle.gather_rows(src, perm[:7], w=5), src[perm[:7], :5])


@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_sgemm_against_numpy(oracle, tA, tB):
    r = _rng(2 + 2 * tA + tB)
    M, N, K = 13, 17, 29
    A = r.bulk_normal(M * K).reshape((K, M) if tA else (M, K))
    B = r.bulk_normal(N * K).reshape((N, K) if tB else (K, N))
    C0 = r.bulk_normal(M * N).reshape(M, N)
    want = 0.5 * ((A.T if tA else A).astype(np.float64) @ (B.T if tB else B).astype(np.float64)) + 2.0 * C0
    got = oracle.sgemm(tA, tB, A, B, alpha=0.5, beta=2.0, Cin=C0)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(oracle.sgemm(tA, tB, A, B), (A.T if tA else A) @ (B.T if tB else B),
                               rtol=1e-5, atol=1e-5)


def test_colsum_embed_softmax(oracle):
    r = _rng(9)
    X = r.bulk_normal(50 * 7).reshape(50, 7)
    np.testing.assert_allclose(oracle.colsum(X), X.sum(0), rtol=1e-5, atol=1e-5)
    acc = np.ones(7, np.float32)
    np.testing.assert_allclose(oracle.colsum(X, accumulate_into=acc), 1 + X.sum(0), rtol=1e-5, atol=1e-5)

    V, E = 23, 6
    table = r.bulk_normal(V * E).reshape(V, E)
    ids = np.floor(r.bulk_uniform(31) * V).astype(np.float32)
    np.testing.assert_array_equal(oracle.embed_fwd(ids, table), table[ids.astype(int)])
    dy = r.bulk_normal(31 * E).reshape(31, E)
    want = torch.zeros(V, E, dtype=torch.float64).index_add_(
        0, torch.tensor(ids.astype(np.int64)), torch.tensor(dy, dtype=torch.float64)).numpy()
    got = oracle.embed_bwd(np.zeros((V, E), np.float32), ids, dy)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)

    logits = 3 * r.bulk_normal(19 * 5).reshape(19, 5)
    labels = np.floor(r.bulk_uniform(19) * 5).astype(np.float32)
    t = torch.tensor(logits, dtype=torch.float64, requires_grad=True)
    rows = torch.nn.functional.cross_entropy(t, torch.tensor(labels.astype(np.int64)), reduction="none")
    rows.mean().backward()
    loss, d = oracle.softmax_xent(logits, labels)
    np.testing.assert_allclose(loss, rows.detach().numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(d, t.grad.numpy(), rtol=1e-5, atol=1e-7)


def test_embedding_offset_is_float_product_truncated(oracle):
    """op_impl_embedding_lookup.cu:27: offset = int(float(id) * E).  Exact for every
    configured (vocab, E); a fractional id truncates toward the row it starts in."""
    for V, E in [(21701, 300), (10000, 512), (1000, 128), (21701, 1024)]:
        ids = np.array([0, 1, V // 2, V - 1], np.float32)
        assert ((ids * np.float32(E)).astype(np.int64) == ids.astype(np.int64) * E).all()
    table = np.arange(12, dtype=np.float32).reshape(4, 3)
    np.testing.assert_array_equal(oracle.embed_fwd(np.array([2.0], np.float32), table), table[2:3])


def test_treelstm_gates_against_autograd(oracle):
    r = _rng(77)
    n, H = 9, 8
    xW, hU = r.bulk_normal(n * 4 * H).reshape(n, 4 * H), r.bulk_normal(n * 3 * H).reshape(n, 3 * H)
    hUf, G = r.bulk_normal(2 * n * H).reshape(2 * n, H), r.bulk_normal(2 * n * 2 * H).reshape(2 * n, 2 * H)
    bias = r.bulk_normal(4 * H)
    dmsg, dret = r.bulk_normal(n * 2 * H).reshape(n, 2 * H), r.bulk_normal(n * H).reshape(n, H)
    T = lambda a: torch.tensor(a, dtype=torch.float64, requires_grad=True)
    txW, thU, thUf, tG, tb = T(xW), T(hU), T(hUf), T(G), T(bias)
    cl, cr = tG[0::2, H:], tG[1::2, H:]
    i = torch.sigmoid(txW[:, :H] + thU[:, :H] + tb[:H])
    o = torch.sigmoid(txW[:, H:2 * H] + thU[:, H:2 * H] + tb[3 * H:])
    u = torch.tanh(txW[:, 2 * H:3 * H] + thU[:, 2 * H:] + tb[2 * H:3 * H])
    fl = torch.sigmoid(txW[:, 3 * H:] + thUf[0::2] + tb[H:2 * H])
    fr = torch.sigmoid(txW[:, 3 * H:] + thUf[1::2] + tb[H:2 * H])
    c = i * u + fl * cl + fr * cr
    h = o * torch.tanh(c)
    gates, msg = oracle.treelstm_gates_fwd(xW, hU, hUf, G, bias)
    np.testing.assert_allclose(msg, torch.cat([h, c], 1).detach().numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(gates[:, :H], i.detach().numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(gates[:, 4 * H:5 * H], fr.detach().numpy(), rtol=1e-5, atol=1e-6)
    # the message [h|c] receives dmsg, the pushed h receives dret
    (torch.cat([h, c], 1) * torch.tensor(dmsg, dtype=torch.float64)).sum().add(
        (h * torch.tensor(dret, dtype=torch.float64)).sum()).backward()
    dxW, dF, dG = oracle.treelstm_gates_bwd(dmsg, dret, gates, G)
    np.testing.assert_allclose(dxW, txW.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(dxW[:, :3 * H], thU.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(dF, thUf.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(dG[:, H:], tG.grad.numpy()[:, H:], rtol=1e-4, atol=1e-5)


def test_lstm_and_treefc_gates_against_autograd(oracle):
    r = _rng(78)
    n, H = 7, 8
    a, G, bias = r.bulk_normal(n * 4 * H).reshape(n, 4 * H), r.bulk_normal(n * 2 * H).reshape(n, 2 * H), r.bulk_normal(4 * H)
    dmsg, dret = r.bulk_normal(n * 2 * H).reshape(n, 2 * H), r.bulk_normal(n * H).reshape(n, H)
    T = lambda v: torch.tensor(v, dtype=torch.float64, requires_grad=True)
    ta, tG = T(a), T(G)
    z = ta + torch.tensor(bias, dtype=torch.float64)
    i, f, u, o = torch.sigmoid(z[:, :H]), torch.sigmoid(z[:, H:2 * H]), torch.tanh(z[:, 2 * H:3 * H]), torch.sigmoid(z[:, 3 * H:])
    c = i * u + f * tG[:, H:]
    h = o * torch.tanh(c)
    gates, msg = oracle.lstm_gates_fwd(a, G, bias)
    np.testing.assert_allclose(msg, torch.cat([h, c], 1).detach().numpy(), rtol=1e-5, atol=1e-6)
    ((torch.cat([h, c], 1) * torch.tensor(dmsg, dtype=torch.float64)).sum()
     + (h * torch.tensor(dret, dtype=torch.float64)).sum()).backward()
    da, dG = oracle.lstm_gates_bwd(dmsg, dret, gates, G)
    np.testing.assert_allclose(da, ta.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(dG[:, H:], tG.grad.numpy()[:, H:], rtol=1e-4, atol=1e-5)

    for act in (0, 1):
        zz, b, x = r.bulk_normal(n * H).reshape(n, H), r.bulk_normal(H), r.bulk_normal(n * H).reshape(n, H)
        tz = T(zz)
        pre = tz + torch.tensor(b, dtype=torch.float64) + torch.tensor(x, dtype=torch.float64)
        hh = torch.tanh(pre) if act else torch.relu(pre)
        got = oracle.treefc_fwd(zz, b, x, act)
        np.testing.assert_allclose(got, hh.detach().numpy(), rtol=1e-5, atol=1e-6)
        d1, d2 = r.bulk_normal(n * H).reshape(n, H), r.bulk_normal(n * H).reshape(n, H)
        (hh * torch.tensor(d1 + d2, dtype=torch.float64)).sum().backward()
        np.testing.assert_allclose(oracle.treefc_bwd(d1, d2, got, act), tz.grad.numpy(), rtol=1e-4, atol=1e-5)
