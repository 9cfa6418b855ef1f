"""Independent fp64 PyTorch-CPU formulations used to pin the oracle.

`per_sample_*`  : textbook recursive evaluation of each sample on its own -- no
                  scheduler, no batching, no message pool.  This is what a
                  correct batched execution must equal (row-id pairing, serial
                  scheduling, or any batch whose roots come last in their round).
`round_based`   : executes the rounds of a scheduler trace with torch index ops
                  using the reference's pairing (b-th list entry <-> b-th slab
                  row) and lets autograd derive the backward, which pins the
                  oracle's hand-written backward as the transpose of its forward.
"""
import numpy as np
import torch

D = torch.float64


def _adj(graph):
    parents, off = [], 0
    for row in graph:
        n = int(np.argmax(row == -1)) + 1
        parents += [off + int(p) if p >= 0 else -1 for p in row[:n]]
        off += n
    children = [[] for _ in parents]
    for v, p in enumerate(parents):
        if p >= 0:
            children[p].append(v)
    return parents, children


def tparams(params):
    return {k: torch.tensor(np.asarray(v), dtype=D, requires_grad=True) for k, v in params.items()}


def _head(GO, P, labels, loss, parents):
    if loss == "softmax":
        logits = GO @ P["Wfc"].T + P["bfc"]
        rows = torch.nn.functional.cross_entropy(
            logits, torch.tensor(np.asarray(labels), dtype=torch.long), reduction="none")
        return rows, rows.mean()
    if loss == "root_sq":
        roots = [v for v, p in enumerate(parents) if p < 0]
        t = (GO[roots] ** 2).sum()
        return t.reshape(1), t
    t = GO.abs().sum()
    return t.reshape(1), t


def _treelstm_cell(P, H, xid, hl, cl, hr, cr):
    W, U, Bv = P["W"], P["U"], P["Bv"]
    U_iou = U[: 3 * H * H].reshape(H, 3 * H)
    U_f = U[3 * H * H :].reshape(H, H)
    e = P["Emb"][xid]
    xW = e @ W
    hU = (hl + hr) @ U_iou
    i = torch.sigmoid(xW[..., 0:H] + hU[..., 0:H] + Bv[0:H])
    o = torch.sigmoid(xW[..., H : 2 * H] + hU[..., H : 2 * H] + Bv[3 * H :])
    u = torch.tanh(xW[..., 2 * H : 3 * H] + hU[..., 2 * H :] + Bv[2 * H : 3 * H])
    fl = torch.sigmoid(xW[..., 3 * H :] + hl @ U_f + Bv[H : 2 * H])
    fr = torch.sigmoid(xW[..., 3 * H :] + hr @ U_f + Bv[H : 2 * H])
    c = i * u + fl * cl + fr * cr
    return o * torch.tanh(c), c


def _treelstm2_cell(P, H, xid, hl, cl, hr, cr):
    """Forget gates with a recurrent matrix per child; bias blocks in the order of the gate columns."""
    W, U, Bv = P["W"], P["U"], P["Bv"]
    U_iou = U[: 3 * H * H].reshape(H, 3 * H)
    U_fl = U[3 * H * H : 4 * H * H].reshape(H, H)
    U_fr = U[4 * H * H :].reshape(H, H)
    xW = P["Emb"][xid] @ W
    iou = xW[..., : 3 * H] + (hl + hr) @ U_iou + Bv[: 3 * H]
    i, o, u = torch.sigmoid(iou[..., :H]), torch.sigmoid(iou[..., H : 2 * H]), torch.tanh(iou[..., 2 * H :])
    fl = torch.sigmoid(xW[..., 3 * H :] + hl @ U_fl + Bv[3 * H :])
    fr = torch.sigmoid(xW[..., 3 * H :] + hr @ U_fr + Bv[3 * H :])
    c = i * u + fl * cl + fr * cr
    return o * torch.tanh(c), c


def _treegate_cell(P, H, xid, hl, hr):
    """One state block: z = sigmoid(x W_z + (h_l + h_r) U_z + b_z), u = tanh(x W_u + [h_l, h_r] U_lr + b_u),
    h = u z + g - z g with g = (h_l + h_r) sigmoid(h_l + h_r)."""
    W, U, Bv = P["W"], P["U"], P["Bv"]
    E = P["Emb"].shape[1]
    U_z = U[: H * H].reshape(H, H)
    U_lr = U[H * H :].reshape(2 * H, H)
    xW = P["Emb"][xid] @ W.reshape(E, 2 * H)
    hs = hl + hr
    z = torch.sigmoid(xW[..., :H] + hs @ U_z + Bv[:H])
    u = torch.tanh(xW[..., H:] + torch.cat([hl, hr], -1) @ U_lr + Bv[H:])
    g = hs * torch.sigmoid(hs)
    return u * z + g - z * g


def _treegru_cell(P, H, xid, hl, hr):
    """Child-sum tree GRU: r, z = sigmoid(x W_{r,z} + (h_l + h_r) U_{r,z} + b_{r,z}),
    c = tanh(x W_c + (r (h_l + h_r)) U_c + b_c), h = z (h_l + h_r) + (1 - z) c.  The candidate's product
    takes a left operand that depends on another product of the same vertex."""
    W, U, Bv = P["W"], P["U"], P["Bv"]
    E = P["Emb"].shape[1]
    U_r, U_z, U_c = (U[i * H * H : (i + 1) * H * H].reshape(H, H) for i in range(3))
    xW = P["Emb"][xid] @ W.reshape(E, 3 * H)
    hs = hl + hr
    r = torch.sigmoid(xW[..., :H] + hs @ U_r + Bv[:H])
    z = torch.sigmoid(xW[..., H : 2 * H] + hs @ U_z + Bv[H : 2 * H])
    c = torch.tanh(xW[..., 2 * H :] + (r * hs) @ U_c + Bv[2 * H :])
    return z * hs + (1 - z) * c


def _treedeep_cell(P, H, xid, hl, hr):
    """Three stages of products sharing a weight block, a block of x W and a bias across stages:
    a = sigmoid(xW_0 + hs U_1 + b_1), m = tanh(xW_1 + (a hs) U_2 + b_1), q = tanh(xW_0 + m U_1 + b_2),
    h = a q + (1 - a) hs."""
    W, U, Bv = P["W"], P["U"], P["Bv"]
    E = P["Emb"].shape[1]
    U_1, U_2 = (U[i * H * H : (i + 1) * H * H].reshape(H, H) for i in range(2))
    xW = P["Emb"][xid] @ W.reshape(E, 2 * H)
    hs = hl + hr
    a = torch.sigmoid(xW[..., :H] + hs @ U_1 + Bv[:H])
    m = torch.tanh(xW[..., H:] + (a * hs) @ U_2 + Bv[:H])
    q = torch.tanh(xW[..., :H] + m @ U_1 + Bv[H:])
    return a * q + (1 - a) * hs


def _lstm_cell(P, H, xid, hp, cp):
    Wf = P["W"]
    Ux = Wf[: 4 * H * H].reshape(H, 4 * H)
    Wh = Wf[4 * H * H :].reshape(H, 4 * H)
    a = P["Emb"][xid] @ Ux + hp @ Wh + P["Bv"]
    i, f = torch.sigmoid(a[..., 0:H]), torch.sigmoid(a[..., H : 2 * H])
    u, o = torch.tanh(a[..., 2 * H : 3 * H]), torch.sigmoid(a[..., 3 * H :])
    c = i * u + f * cp
    return o * torch.tanh(c), c


def _fc_cell(P, hl, hr, xin, act, use_bias):
    z = torch.cat([hl, hr], -1) @ P["W"]
    if use_bias:
        z = z + P["Bv"]
    if xin is not None:
        z = z + xin
    return torch.tanh(z) if act else torch.relu(z)


def per_sample(model, graph, x, labels, params, H, loss="softmax", act=0, use_bias=False,
               use_x=False):
    P = tparams(params)
    parents, children = _adj(graph)
    n = len(parents)
    xs = torch.tensor(np.asarray(x), dtype=D)
    zero = torch.zeros(H, dtype=D)
    h, c = [None] * n, [None] * n
    order, indeg = [], [len(ch) for ch in children]
    stack = [v for v in range(n) if indeg[v] == 0]
    while stack:  # any topological order
        v = stack.pop()
        order.append(v)
        p = parents[v]
        if p >= 0:
            indeg[p] -= 1
            if indeg[p] == 0:
                stack.append(p)
    for v in order:
        ch = sorted(children[v])
        if model in ("treelstm", "treelstm2"):
            hl, cl = (h[ch[0]], c[ch[0]]) if ch else (zero, zero)
            hr, cr = (h[ch[1]], c[ch[1]]) if len(ch) > 1 else (zero, zero)
            cell = _treelstm_cell if model == "treelstm" else _treelstm2_cell
            h[v], c[v] = cell(P, H, int(xs[v]), hl, cl, hr, cr)
        elif model == "treegate":
            hl = h[ch[0]] if ch else zero
            hr = h[ch[1]] if len(ch) > 1 else zero
            h[v] = _treegate_cell(P, H, int(xs[v]), hl, hr)
        elif model in ("treegru", "treedeep"):
            hl = h[ch[0]] if ch else zero
            hr = h[ch[1]] if len(ch) > 1 else zero
            h[v] = (_treegru_cell if model == "treegru" else _treedeep_cell)(P, H, int(xs[v]), hl, hr)
        elif model == "lstm":
            hp, cp = (h[ch[0]], c[ch[0]]) if ch else (zero, zero)
            h[v], c[v] = _lstm_cell(P, H, int(xs[v]), hp, cp)
        else:
            hl = h[ch[0]] if ch else zero
            hr = h[ch[1]] if ch else zero
            h[v] = _fc_cell(P, hl, hr, xs[v] if use_x else None, act, use_bias)
    GO = torch.stack(h)
    GO.retain_grad()
    rows, total = _head(GO, P, labels, loss, parents)
    total.backward()
    grads = {"d" + k: (v.grad.numpy() if v.grad is not None else np.zeros(v.shape)) for k, v in P.items()}
    return dict(loss=rows.detach().numpy(), graph_out=GO.detach().numpy(),
                dgraph_out=GO.grad.numpy(), grads=grads)


def round_based(model, graph, trace, x, labels, params, H, loss="softmax", act=0,
                use_bias=False, use_x=False, pairing="reference"):
    P = tparams(params)
    parents, _ = _adj(graph)
    N = trace["N"]
    mw = H if model == "treefc" else 2 * H
    xs = torch.tensor(np.asarray(x), dtype=D)
    pool = torch.zeros(N + 1, mw, dtype=D)
    ret = [None] * N
    for rd in trace["fwd"]:
        jobs, off, n = rd["exec"], rd["offset"], len(rd["exec"])
        G = []
        for cidx in range(2):
            lst = rd["gather"][cidx]
            g = torch.zeros(n, mw, dtype=D)
            if lst:
                g = torch.cat([pool[lst], g[len(lst):]], 0)
            G.append(g)
        if model in ("treelstm", "treelstm2"):
            cell = _treelstm_cell if model == "treelstm" else _treelstm2_cell
            hh, cc = cell(P, H, xs[jobs].long(), G[0][:, :H], G[0][:, H:], G[1][:, :H], G[1][:, H:])
            msg = torch.cat([hh, cc], 1)
        elif model == "lstm":
            hh, cc = _lstm_cell(P, H, xs[jobs].long(), G[0][:, :H], G[0][:, H:])
            msg = torch.cat([hh, cc], 1)
        else:
            hh = _fc_cell(P, G[0], G[1], xs[jobs] if use_x else None, act, use_bias)
            msg = hh
        lst = rd["scatter"][0]
        if lst:
            src = msg[: len(lst)] if pairing == "reference" else msg[[t - off for t in lst]]
            pool = pool.index_copy(0, torch.tensor(lst), src)
        for b, v in enumerate(jobs):
            ret[v] = hh[b]
    GO = torch.stack(ret)
    GO.retain_grad()
    rows, total = _head(GO, P, labels, loss, parents)
    total.backward()
    grads = {"d" + k: (v.grad.numpy() if v.grad is not None else np.zeros(v.shape)) for k, v in P.items()}
    return dict(loss=rows.detach().numpy(), graph_out=GO.detach().numpy(),
                dgraph_out=GO.grad.numpy(), grads=grads)
