"""Python view of the host runtime (include/cavs_session.h, libcavs_host.so).

Mirrors the reference's Session: construct with an optimisation bitmask, feed the
graph placeholder (host int32 parent arrays), vertex inputs and labels, run a step,
read results back.  All compute happens in the C++ runtime and the HIP backend;
nothing here falls back to the CPU.
"""
import ctypes as C
import os

import numpy as np

from . import hip

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libcavs_host.so")

OPT_FUSION, OPT_BATCHING, OPT_STREAMMING = 1, 2, 4
MODEL = {"treelstm": 0, "lstm": 1, "treefc": 2}
LOSS = {"softmax": 0, "root_sq": 1, "sum_abs": 2}
PAIR = {"reference": 0, "rowid": 1}


class _Config(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("model", "loss", "pairing", "opt", "V", "E", "H", "C", "act",
                                      "use_bias", "use_x", "device", "fused_round_rows", "split_backward_rounds",
                                      "schedule_mode", "plan_cache", "tail_rows", "graph_replay", "head_chunks")]


_lib = None


def lib():
    global _lib
    if _lib is None:
        hip.lib()  # the backend must be present; there is no CPU path
        if not os.path.exists(LIB_PATH):
            raise hip.CavsError(f"{LIB_PATH} is missing: build it with `python -m cavs_amd.build`")
        l = C.CDLL(LIB_PATH)
        l.cavs_session_error.restype = C.c_char_p
        l.cavs_session_stream.restype = C.c_void_p
        l.cavs_session_stream.argtypes = [C.c_void_p]
        P, I, Z, F = C.c_void_p, C.c_int, C.c_size_t, C.c_float
        sigs = {
            "cavs_session_create": [C.POINTER(_Config), C.POINTER(P)],
            "cavs_session_destroy": [P],
            "cavs_session_set_param": [P, C.c_char_p, P, Z],
            "cavs_session_get_param": [P, C.c_char_p, P, Z],
            "cavs_session_get_grad": [P, C.c_char_p, P, Z],
            "cavs_session_step": [P, P, I, I, P, P, I, I, F],
            "cavs_session_sync": [P],
            "cavs_session_fetch": [P, C.c_char_p, P, Z],
            "cavs_session_total_length": [P],
            "cavs_session_schedule_trace": [P, P, I],
            "cavs_schedule_trace": [P, I, I, I, I, P, I],
            "cavs_schedule_index_lists": [P, I, I, I, I, I, P, P, P, P, P, P, P],
            "cavs_schedule_tail_lists": [P, I, I, I, I, I, I, I, P, P, P, P, P, P, P, P, P],
            "cavs_schedule_trace_from_lists": [I, I, I, I, P, I, P, P, P, P, I, P, I],
            "cavs_session_timing": [P, C.c_char_p, C.POINTER(F)],
            "cavs_session_counter": [P, C.c_char_p, C.POINTER(C.c_double)],
            "cavs_session_profile": [P, I],
            "cavs_session_profile_read": [P, C.c_char_p, C.POINTER(C.c_double), C.POINTER(C.c_double)],
        }
        for k, a in sigs.items():
            fn = getattr(l, k)
            fn.argtypes, fn.restype = a, I
        _lib = l
    return _lib


def _check(rc, what):
    if rc != 0:
        raise hip.CavsError(f"{what} -> {rc}: {lib().cavs_session_error().decode()}")


def _parse_trace(out):
    pos = [3]

    def take_list():
        k = int(out[pos[0]])
        v = out[pos[0] + 1: pos[0] + 1 + k].tolist()
        pos[0] += 1 + k
        return v

    def take_round():
        off = int(out[pos[0]])
        pos[0] += 1
        ex = take_list()
        g0, g1, s0, s1 = take_list(), take_list(), take_list(), take_list()
        return dict(offset=off, exec=ex, gather=[g0, g1], scatter=[s0, s1], gather_init=take_list())

    N, rf, rb = int(out[0]), int(out[1]), int(out[2])
    fwd = [take_round() for _ in range(rf)]
    bwd = [take_round() for _ in range(rb)]
    t2j = out[pos[0]: pos[0] + N].tolist()
    pos[0] += N
    return dict(N=N, fwd=fwd, bwd=bwd, tids_to_jobids=t2j, round2offset=take_list())


def schedule_trace(graph, batching=True, with_backward=True):
    """Host-only: the production scheduler's rounds and index lists for a graph feed."""
    g = np.ascontiguousarray(graph, np.int32)
    B, maxlen = g.shape
    cap = 64 + 40 * g.size
    out = np.zeros(cap, np.int32)
    n = lib().cavs_schedule_trace(g.ctypes.data, B, maxlen, int(batching), int(with_backward),
                                  out.ctypes.data, cap)
    if n < 0:
        out = np.zeros(-n, np.int32)
        n = lib().cavs_schedule_trace(g.ctypes.data, B, maxlen, int(batching), int(with_backward),
                                      out.ctypes.data, -n)
    if n == 0:
        raise hip.CavsError("graph feed rejected: " + lib().cavs_session_error().decode())
    return _parse_trace(out)


def index_lists(graph, nchild, pairing="reference", fused_limit=1 << 30):
    """Host-only: the index lists a step's kernels consume, as the host scheduler builds them.
    Returns dict(N, t2j, pair, child, roots, kid, orphans); kid / orphans are None when the
    batch's message flow is not a forest."""
    g = np.ascontiguousarray(graph, np.int32)
    B, maxlen = g.shape
    cap = B * maxlen
    t2j, pair, orph = (np.zeros(cap, np.int32) for _ in range(3))
    child, kid = np.zeros(nchild * cap, np.int32), np.zeros(nchild * cap, np.int32)
    roots, n_orph = np.zeros(B, np.int32), C.c_int(0)
    N = lib().cavs_schedule_index_lists(g.ctypes.data, B, maxlen, nchild, PAIR[pairing], fused_limit, t2j.ctypes.data,
                                        pair.ctypes.data, child.ctypes.data, roots.ctypes.data, kid.ctypes.data,
                                        orph.ctypes.data, C.addressof(n_orph))
    if N <= 0:
        raise hip.CavsError("graph feed rejected: " + lib().cavs_session_error().decode())
    forest = n_orph.value >= 0
    return dict(N=N, t2j=t2j[:N], pair=pair[:N], child=child[: nchild * N], roots=roots,
                kid=kid[: nchild * N] if forest else None, orphans=orph[: n_orph.value] if forest else None)


def tail_lists(graph, pairing="reference", fused_limit=1 << 30, rows_limit=32, groups=8, max_lists=32):
    """Host-only: how the rounds near the roots of a batch of binary trees are dealt to the groups of the
    tail launches.  None when no suffix of the rounds can be dealt within the limits; else
    dict(first, M, lists_max, tiles_max, nrounds [groups], start / count / flags and bstart / bcount /
    bflags [groups, M], rows)."""
    g = np.ascontiguousarray(graph, np.int32)
    B, maxlen = g.shape
    meta, nrounds = np.zeros(4, np.int32), np.zeros(groups, np.int32)
    arr = [np.zeros(groups * max_lists, np.int32) for _ in range(6)]
    rows = np.zeros(B * maxlen, np.int32)
    n = lib().cavs_schedule_tail_lists(g.ctypes.data, B, maxlen, PAIR[pairing], fused_limit, rows_limit, groups, max_lists,
                                       meta.ctypes.data, nrounds.ctypes.data, *[a.ctypes.data for a in arr], rows.ctypes.data)
    if n < 0:
        raise hip.CavsError("graph feed rejected: " + lib().cavs_session_error().decode())
    if n == 0:
        return None
    M = int(meta[1])
    names = ("start", "count", "flags", "bstart", "bcount", "bflags")
    out = dict(first=int(meta[0]), M=M, lists_max=int(meta[2]), tiles_max=int(meta[3]), nrounds=nrounds, rows=rows[:n])
    out.update({k: a[: groups * M].reshape(groups, M) for k, a in zip(names, arr)})
    return out


def trace_from_lists(B, maxlen, nchild, round2offset, t2j, pair, child, roots, with_backward=True):
    """Host-only: the inverse of index_lists -- the complete schedule the lists describe."""
    I32 = lambda a: np.ascontiguousarray(a, np.int32)
    r2o, t2j, pair, child, roots = I32(round2offset), I32(t2j), I32(pair), I32(child), I32(roots)
    N, R = len(t2j), len(r2o) - 1
    cap = 64 + 40 * B * maxlen
    out = np.zeros(cap, np.int32)
    n = lib().cavs_schedule_trace_from_lists(B, maxlen, N, nchild, r2o.ctypes.data, R, t2j.ctypes.data, pair.ctypes.data,
                                             child.ctypes.data, roots.ctypes.data, int(with_backward), out.ctypes.data, cap)
    assert n > 0, n
    return _parse_trace(out)


class Session:
    """One model bound to the device.  `opt` is the reference's bitmask
    (OPT_BATCHING selects the level-wise batch scheduler)."""

    def __init__(self, model, *, H, E=0, V=0, C_=0, loss="softmax", pairing="reference",
                 opt=OPT_BATCHING, act=0, use_bias=False, use_x=False, device=0, fused_round_rows=0,
                 split_backward_rounds=False, schedule="host", plan_cache=0, tail_rows=0, graph_replay=False, head_chunks=0):
        self.model, self.H, self.E, self.V, self.C, self.loss = model, H, (H if model == "lstm" else E), V, C_, loss
        self.mw = H if model == "treefc" else 2 * H
        cfg = _Config(MODEL[model], LOSS[loss], PAIR[pairing], opt, V, E, H, C_, int(act), int(use_bias),
                      int(use_x), device, int(fused_round_rows), int(split_backward_rounds),
                      {"host": 0, "device": 1}[schedule], int(plan_cache), int(tail_rows), int(graph_replay), int(head_chunks))
        self._h = C.c_void_p()
        _check(lib().cavs_session_create(C.byref(cfg), C.byref(self._h)), "cavs_session_create")
        self._keep = None

    def close(self):
        if self._h:
            lib().cavs_session_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_params(self, params):
        for k, v in params.items():
            a = np.ascontiguousarray(v, np.float32)
            _check(lib().cavs_session_set_param(self._h, k.encode(), a.ctypes.data, a.size), f"set_param({k})")

    def param(self, name, shape):
        a = np.zeros(shape, np.float32)
        _check(lib().cavs_session_get_param(self._h, name.encode(), a.ctypes.data, a.size), f"get_param({name})")
        return a

    def grad(self, name, shape):
        a = np.zeros(shape, np.float32)
        _check(lib().cavs_session_get_grad(self._h, name.encode(), a.ctypes.data, a.size), f"get_grad({name})")
        return a

    def step(self, graph, x=None, labels=None, backward=True, lr=0.0):
        """x / labels: numpy arrays (host feeds) or torch CUDA tensors (already in HBM)."""
        g = np.ascontiguousarray(graph, np.int32)
        B, maxlen = g.shape
        on_device = hasattr(x, "data_ptr") or hasattr(labels, "data_ptr")

        def addr(a):
            if a is None:
                return None
            if hasattr(a, "data_ptr"):
                return a.data_ptr()
            return a.ctypes.data

        if not on_device:
            x = None if x is None else np.ascontiguousarray(x, np.float32)
            labels = None if labels is None else np.ascontiguousarray(labels, np.float32)
        self._keep = (g, x, labels)
        _check(lib().cavs_session_step(self._h, g.ctypes.data, B, maxlen, addr(x), addr(labels), int(on_device),
                                       int(backward), float(lr)), "cavs_session_step")

    def sync(self):
        _check(lib().cavs_session_sync(self._h), "cavs_session_sync")

    @property
    def N(self):
        return lib().cavs_session_total_length(self._h)

    def fetch(self, what):
        N, H = self.N, self.H
        shape = {"loss": (N if self.loss == "softmax" else 1,), "graph_out": (N, H), "dgraph_out": (N, H),
                 "msg_pool": (N, self.mw)}[what]
        a = np.zeros(shape, np.float32)
        _check(lib().cavs_session_fetch(self._h, what.encode(), a.ctypes.data, a.size), f"fetch({what})")
        return a

    def grads(self):
        H, E, V, Cc = self.H, self.E, self.V, self.C
        if self.model == "treelstm":
            out = dict(dEmb=self.grad("Emb", (V, E)), dW=self.grad("W", (E, 4 * H)), dU=self.grad("U", (4 * H * H,)),
                       dBv=self.grad("Bv", (4 * H,)))
        elif self.model == "lstm":
            out = dict(dEmb=self.grad("Emb", (V, H)), dW=self.grad("W", (8 * H * H,)), dBv=self.grad("Bv", (4 * H,)))
        else:
            out = dict(dW=self.grad("W", (2 * H, H)))
            try:
                out["dBv"] = self.grad("Bv", (H,))
            except hip.CavsError:
                pass
        if self.loss == "softmax":
            out["dWfc"] = self.grad("Wfc", (Cc, H))
            out["dbfc"] = self.grad("bfc", (Cc,))
        return out

    def schedule_trace(self):
        cap = 64 + 48 * max(self.N, 1)
        out = np.zeros(cap, np.int32)
        n = lib().cavs_session_schedule_trace(self._h, out.ctypes.data, cap)
        if n < 0:
            out = np.zeros(-n, np.int32)
            n = lib().cavs_session_schedule_trace(self._h, out.ctypes.data, -n)
        return _parse_trace(out)

    def timing(self, name):
        ms = C.c_float()
        _check(lib().cavs_session_timing(self._h, name.encode(), C.byref(ms)), f"timing({name})")
        return ms.value

    def counter(self, key):
        v = C.c_double()
        _check(lib().cavs_session_counter(self._h, key.encode(), C.byref(v)), f"counter({key})")
        return v.value

    def profile(self, enable):
        _check(lib().cavs_session_profile(self._h, int(enable)), "cavs_session_profile")

    def profile_read(self, kernel_class):
        """(total device ms, launches) of a kernel class since profile(True)"""
        t, n = C.c_double(), C.c_double()
        _check(lib().cavs_session_profile_read(self._h, kernel_class.encode(), C.byref(t), C.byref(n)),
               "cavs_session_profile_read")
        return t.value, n.value

    @property
    def stream(self):
        return lib().cavs_session_stream(self._h)
