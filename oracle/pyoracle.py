"""ctypes binding of the CPU checker (oracle/libcavs_oracle.so).

Test infrastructure: imported only by tests/, the smoke check and the
cpu_baseline leg of bench.py.  The product package never imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libcavs_oracle.so")

MODEL = {"treelstm": 0, "lstm": 1, "treefc": 2, "treelstm2": 3}
LOSS = {"softmax": 0, "root_sq": 1, "sum_abs": 2}
PAIR = {"reference": 0, "rowid": 1}


def build(force=False):
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libcavs_oracle.so"])
    return _SO


class _Config(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("model", "loss", "pairing", "batching", "V", "E", "H",
                                      "C", "act", "use_bias", "use_x", "threads")]


class _Params(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("Emb", "W", "U", "Bv", "Wfc", "bfc")]


class _Grads(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("dEmb", "dW", "dU", "dBv", "dWfc", "dbfc")]


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
        _lib.or_sched_trace.restype = C.c_int
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def _fx(a, precise):
    """The array as the checker's `real`: fp32, or (precise) the same fp32 values widened to
    double for the ord_* build, which evaluates the same dataflow in double."""
    if a is None:
        return None
    if precise and np.asarray(a).dtype == np.float64:
        return np.ascontiguousarray(a)  # a double result of an earlier stage: chained as it is
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a.astype(np.float64) if precise else a


def _fn(name, precise):
    return getattr(lib(), ("ord_" if precise else "or_") + name)


def _dt(precise):
    return np.float64 if precise else np.float32


def _real(v, precise):
    return C.c_double(v) if precise else C.c_float(v)


def sched_trace(graph, batching=True, with_backward=True):
    """Returns dict(N, fwd=[round...], bwd=[round...], tids_to_jobids, round2offset);
    each round is dict(offset, exec, gather=[l0,l1], scatter=[l0,l1], gather_init)."""
    g = np.ascontiguousarray(graph, dtype=np.int32)
    B, maxlen = g.shape
    cap = 64 + 40 * g.size
    out = np.zeros(cap, np.int32)
    n = lib().or_sched_trace(_p(g), B, maxlen, int(batching), int(with_backward), _p(out), cap)
    if n < 0:
        out = np.zeros(-n, np.int32)
        n = lib().or_sched_trace(_p(g), B, maxlen, int(batching), int(with_backward), _p(out), -n)
    assert n > 0, "scheduler rejected the graph"
    pos = [3]

    def take_list():
        k = int(out[pos[0]])
        v = out[pos[0] + 1 : pos[0] + 1 + k].tolist()
        pos[0] += 1 + k
        return v

    def take_round():
        off = int(out[pos[0]])
        pos[0] += 1
        ex = take_list()
        g0, g1, s0, s1 = take_list(), take_list(), take_list(), take_list()
        init = take_list()
        return dict(offset=off, exec=ex, gather=[g0, g1], scatter=[s0, s1], gather_init=init)

    N, rf, rb = int(out[0]), int(out[1]), int(out[2])
    fwd = [take_round() for _ in range(rf)]
    bwd = [take_round() for _ in range(rb)]
    t2j = out[pos[0] : pos[0] + N].tolist()
    pos[0] += N
    r2o = take_list()
    return dict(N=N, fwd=fwd, bwd=bwd, tids_to_jobids=t2j, round2offset=r2o)


def gather_rows(inp, ids, w=None):
    inp = _f32(inp)
    ids = np.ascontiguousarray(ids, np.int32)
    w = inp.shape[1] if w is None else w
    out = np.zeros((len(ids), w), np.float32)
    lib().or_gather_rows(_p(out), w, _p(inp), inp.shape[1], _p(ids), len(ids), w)
    return out


def scatter_rows(out, ids, inp):
    ids = np.ascontiguousarray(ids, np.int32)
    inp = _f32(inp)
    lib().or_scatter_rows(_p(out), out.shape[1], _p(ids), _p(inp), inp.shape[1], len(ids),
                          inp.shape[1])
    return out


def sgemm(tA, tB, A, B, alpha=1.0, beta=0.0, Cin=None, precise=False):
    A, B = _fx(A, precise), _fx(B, precise)
    M, K = (A.shape[1], A.shape[0]) if tA else A.shape
    N = B.shape[0] if tB else B.shape[1]
    Cm = np.zeros((M, N), _dt(precise)) if Cin is None else _fx(Cin, precise).copy()
    _fn("sgemm", precise)(int(tA), int(tB), M, N, K, _real(alpha, precise), _p(A), A.shape[1], _p(B),
                          B.shape[1], _real(beta, precise), _p(Cm), N)
    return Cm


def colsum(inp, accumulate_into=None, precise=False):
    inp = _fx(inp, precise)
    n, w = inp.shape
    out = np.zeros(w, _dt(precise)) if accumulate_into is None else _fx(accumulate_into, precise).copy()
    _fn("colsum", precise)(_p(out), _p(inp), w, n, w, int(accumulate_into is not None))
    return out


def embed_fwd(ids, table):
    ids, table = _f32(ids), _f32(table)
    E = table.shape[1]
    out = np.zeros((len(ids), E), np.float32)
    lib().or_embed_fwd(_p(out), E, _p(ids), _p(table), len(ids), E)
    return out


def embed_bwd(dtable, ids, dy):
    ids, dy = _f32(ids), _f32(dy)
    lib().or_embed_bwd(_p(dtable), _p(ids), _p(dy), dy.shape[1], len(ids), dy.shape[1])
    return dtable


def softmax_xent(logits, labels, precise=False):
    logits, labels = _fx(logits, precise), _fx(labels, precise)
    n, Cc = logits.shape
    loss = np.zeros(n, _dt(precise))
    d = np.zeros((n, Cc), _dt(precise))
    _fn("softmax_xent", precise)(_p(loss), _p(d), _p(logits), _p(labels), n, Cc)
    return loss, d


def treelstm_gates_fwd(xW, hU, hUf, G, bias, precise=False):
    xW, hU, hUf, G, bias = (_fx(a, precise) for a in (xW, hU, hUf, G, bias))
    n, H = xW.shape[0], xW.shape[1] // 4
    gates = np.zeros((n, 6 * H), _dt(precise))
    msg = np.zeros((n, 2 * H), _dt(precise))
    _fn("treelstm_gates_fwd", precise)(_p(xW), 4 * H, _p(hU), _p(hUf), _p(G), _p(bias), _p(gates),
                                       _p(msg), n, H)
    return gates, msg


def treelstm_gates_bwd(dmsg, dret, gates, G, precise=False):
    dmsg, dret, gates, G = (_fx(a, precise) for a in (dmsg, dret, gates, G))
    n, H = dret.shape
    dxW = np.zeros((n, 4 * H), _dt(precise))
    dF = np.zeros((2 * n, H), _dt(precise))
    dG = np.zeros((2 * n, 2 * H), _dt(precise))
    _fn("treelstm_gates_bwd", precise)(_p(dmsg), _p(dret), _p(gates), _p(G), _p(dxW), 4 * H, _p(dF),
                                       _p(dG), n, H)
    return dxW, dF, dG


def lstm_gates_fwd(a, G, bias, precise=False):
    a, G, bias = (_fx(t, precise) for t in (a, G, bias))
    n, H = a.shape[0], a.shape[1] // 4
    gates = np.zeros((n, 5 * H), _dt(precise))
    msg = np.zeros((n, 2 * H), _dt(precise))
    _fn("lstm_gates_fwd", precise)(_p(a), 4 * H, _p(G), _p(bias), _p(gates), _p(msg), n, H)
    return gates, msg


def lstm_gates_bwd(dmsg, dret, gates, G, precise=False):
    dmsg, dret, gates, G = (_fx(a, precise) for a in (dmsg, dret, gates, G))
    n, H = dret.shape
    da = np.zeros((n, 4 * H), _dt(precise))
    dG = np.zeros((n, 2 * H), _dt(precise))
    _fn("lstm_gates_bwd", precise)(_p(dmsg), _p(dret), _p(gates), _p(G), _p(da), 4 * H, _p(dG), n, H)
    return da, dG


def treefc_fwd(z, bias, x, act, precise=False):
    z = _fx(z, precise)
    n, H = z.shape
    h = np.zeros((n, H), _dt(precise))
    bias, x = _fx(bias, precise), _fx(x, precise)
    _fn("treefc_fwd", precise)(_p(z), _p(bias), _p(x), _p(h), n, H, int(act))
    return h


def treefc_bwd(dh_m, dret, h, act, precise=False):
    dh_m, dret, h = (_fx(a, precise) for a in (dh_m, dret, h))
    n, H = h.shape
    dz = np.zeros((n, H), _dt(precise))
    _fn("treefc_bwd", precise)(_p(dh_m), _p(dret), _p(h), _p(dz), n, H, int(act))
    return dz


def model_step(model, graph, x, labels, params, *, H, E=0, V=0, Cc=0, loss="softmax",
               pairing="reference", batching=True, act=0, use_bias=False, use_x=False,
               threads=1, want_grads=True, precise=False):
    """One fwd+bwd pass.  Returns dict(N, loss, graph_out, dgraph_out, msg_pool, grads).
    precise: the same dataflow with every value and sum in double (ord_model_step); the
    results come back as float64."""
    g = np.ascontiguousarray(graph, np.int32)
    B, maxlen = g.shape
    x, labels = _fx(x, precise), _fx(labels, precise)
    dt = _dt(precise)
    cfg = _Config(MODEL[model], LOSS[loss], PAIR[pairing], int(batching), V, E, H, Cc, int(act),
                  int(use_bias), int(use_x), threads)
    keep = {k: _fx(v, precise) for k, v in params.items()}
    prm = _Params(*[_p(keep.get(k)) for k in ("Emb", "W", "U", "Bv", "Wfc", "bfc")])
    N = int(sum(int(np.argmax(r == -1)) + 1 for r in g))
    mw = H if model == "treefc" else 2 * H
    Ee = H if model == "lstm" else E
    loss_rows = np.zeros(N if loss == "softmax" else 1, dt)
    GO = np.zeros((N, H), dt)
    dGO = np.zeros((N, H), dt)
    pool = np.zeros((N, mw), dt)
    grads = {}
    if want_grads:
        if model in ("treelstm", "treelstm2"):
            grads = dict(dEmb=np.zeros((V, Ee), dt), dW=np.zeros((Ee, 4 * H), dt),
                         dU=np.zeros((5 if model == "treelstm2" else 4) * H * H, dt), dBv=np.zeros(4 * H, dt))
        elif model == "lstm":
            grads = dict(dEmb=np.zeros((V, Ee), dt), dW=np.zeros(8 * H * H, dt),
                         dBv=np.zeros(4 * H, dt))
        else:
            grads = dict(dW=np.zeros((2 * H, H), dt), dBv=np.zeros(H, dt))
        if loss == "softmax":
            grads["dWfc"] = np.zeros((Cc, H), dt)
            grads["dbfc"] = np.zeros(Cc, dt)
    gs = _Grads(*[_p(grads.get(k)) for k in ("dEmb", "dW", "dU", "dBv", "dWfc", "dbfc")])
    rc = _fn("model_step", precise)(C.byref(cfg), C.byref(prm), _p(g), B, maxlen, _p(x), _p(labels),
                                    _p(loss_rows), _p(GO), _p(dGO), _p(pool),
                                    C.byref(gs) if want_grads else None)
    assert rc == N, f"model_step failed: {rc}"
    return dict(N=N, loss=loss_rows, graph_out=GO, dgraph_out=dGO, msg_pool=pool, grads=grads)
