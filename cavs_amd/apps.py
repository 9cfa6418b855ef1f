"""Python handle on the benchmark applications written against the C++ front end
(cavs_amd/host/apps/models.cc -> libcavs_apps.so): declare a program with Sym /
GraphSupport, open a Session(opt), run steps, read values and gradients back."""
import ctypes as C
import os

import numpy as np

from . import hip, session

_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
_apps = None
_host = None


def libs():
    global _apps, _host
    if _apps is None:
        hip.lib()
        _host = C.CDLL(os.path.join(_DIR, "libcavs_host.so"), mode=C.RTLD_GLOBAL)
        path = os.path.join(_DIR, "libcavs_apps.so")
        if not os.path.exists(path):
            raise hip.CavsError(f"{path} is missing: build it with `python -m cavs_amd.build`")
        a = C.CDLL(path)
        a.cavs_app_create.argtypes = [C.c_char_p] + [C.c_int] * 7 + [C.c_float]
        a.cavs_app_set_param.argtypes = [C.c_char_p, C.c_void_p, C.c_size_t]
        a.cavs_app_configure.argtypes = [C.c_int, C.c_int]
        a.cavs_app_step.argtypes = [C.c_void_p] * 4 + [C.c_int, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t]
        a.cavs_app_step.restype = C.c_long
        a.cavs_app_read_param.argtypes = [C.c_char_p, C.c_int, C.c_void_p, C.c_size_t]
        a.cavs_app_read_param.restype = C.c_long
        a.cavs_app_read.argtypes = [C.c_char_p, C.c_void_p, C.c_size_t]
        a.cavs_app_read.restype = C.c_long
        a.cavs_app_var_size.argtypes = [C.c_char_p]
        a.cavs_app_var_size.restype = C.c_long
        _host.C_DumpGraph.restype = C.c_size_t
        _host.C_DumpGraph.argtypes = [C.c_char_p, C.c_size_t]
        _host.C_DumpFusedGraph.restype = C.c_size_t
        _host.C_DumpFusedGraph.argtypes = [C.c_char_p, C.c_size_t]
        _host.C_LastError.restype = C.c_char_p
        _apps = a
    return _apps, _host


class App:
    """model: treelstm | lstm | treefc | treefc_x | treelstm2 | treegate | cell<seed>.  opt: OPT_* bitmask, or -1 to only
    declare the program (no device)."""

    def __init__(self, model, *, B, maxlen, H, E=0, V=0, C_=0, opt=session.OPT_BATCHING, lr=0.0, clip=0.0,
                 pairing="reference", allow_fused=True, iters=1):
        a, _ = libs()
        self.model, self.B, self.maxlen, self.H, self.E, self.V, self.C = model, B, maxlen, H, E, V, C_
        a.cavs_app_set_clip(C.c_float(clip))
        a.cavs_app_set_iters(int(iters))
        rc = a.cavs_app_create(model.encode(), B, maxlen, V, E, H, C_, opt, lr)
        if rc != 0:
            raise hip.CavsError(f"cavs_app_create({model}) -> {rc}")
        if opt >= 0:
            a.cavs_app_configure(session.PAIR[pairing], int(allow_fused))

    def dump(self):
        _, h = libs()
        n = h.C_DumpGraph(None, 0)
        buf = C.create_string_buffer(n)
        h.C_DumpGraph(buf, n)
        return buf.value.decode()

    def dump_fused(self):
        """The programs after the OPT_FUSION pass, with the generated kernel sources."""
        _, h = libs()
        n = h.C_DumpFusedGraph(None, 0)
        buf = C.create_string_buffer(n)
        h.C_DumpFusedGraph(buf, n)
        return buf.value.decode()

    def set_params(self, params):
        a, _ = libs()
        for k, v in params.items():
            arr = np.ascontiguousarray(v, np.float32)
            rc = a.cavs_app_set_param(k.encode(), arr.ctypes.data, arr.size)
            if rc != 0:
                raise hip.CavsError(f"set_param({k}) -> {rc}")

    def _placeholder(self, packed, width=1):
        buf = np.zeros(self.B * self.maxlen * width, np.float32)
        if packed is not None:
            p = np.ascontiguousarray(packed, np.float32).ravel()
            buf[: p.size] = p
        return buf

    def step(self, graph, x=None, labels=None, train=True, root_mask=None, fetch=True):
        """One Session::Run.  fetch=False (training only) requests just the optimizer symbol, as the
        reference apps' loops do, and reads nothing back."""
        a, _ = libs()
        g = np.ascontiguousarray(graph, np.int32)
        xw = self.H if self.model == "treefc_x" else 1
        if self.model == "treefc":  # the reference Tree-FC app reads no vertex input and no labels
            x = labels = None
        elif self.model == "treefc_x":
            labels = None
        xb, lb = self._placeholder(x, xw), self._placeholder(labels)
        mb = self._placeholder(root_mask, self.H) if self.model == "treefc_x" else np.zeros(1, np.float32)
        if train and not fetch:
            n = a.cavs_app_step(g.ctypes.data, xb.ctypes.data, lb.ctypes.data, mb.ctypes.data, 1, None, 0, None, 0)
            if n < 0:
                raise hip.CavsError(f"cavs_app_step -> {n}")
            return None
        cap = self.B * self.maxlen
        loss = np.zeros(cap, np.float32)
        go = np.zeros(cap * self.H, np.float32)
        n = a.cavs_app_step(g.ctypes.data, xb.ctypes.data, lb.ctypes.data, mb.ctypes.data, int(train),
                            loss.ctypes.data, loss.size, go.ctypes.data, go.size)
        if n < 0:
            raise hip.CavsError(f"cavs_app_step -> {n}")
        nl = n if not self.model.startswith("treefc") else 1  # (the Tree-FC apps end in one scalar loss)
        return loss[:nl].copy(), go[: n * self.H].reshape(n, self.H).copy()

    def grad(self, name, shape, grad=True):
        a, _ = libs()
        out = np.zeros(shape, np.float32)
        n = a.cavs_app_read_param(name.encode(), int(grad), out.ctypes.data, out.size)
        if n != out.size:
            raise hip.CavsError(f"read_param({name}) -> {n}, expected {out.size}")
        return out

    def var_size(self, name):
        """Element count of a parameter (the seeded cell<seed> family sizes its weights by the seed)."""
        a, _ = libs()
        n = a.cavs_app_var_size(name.encode())
        if n < 0:
            raise hip.CavsError(f"var_size({name}) -> {n}")
        return int(n)

    def read(self, edge, n):
        a, _ = libs()
        out = np.zeros(n, np.float32)
        got = a.cavs_app_read(edge.encode(), out.ctypes.data, out.size)
        if got != n:
            raise hip.CavsError(f"read({edge}) -> {got}")
        return out

    @property
    def fused(self):
        a, _ = libs()
        return bool(a.cavs_app_uses_fused_path())

    @property
    def fused_kind(self):
        """0: F runs op by op; 1: on the hand-written round kernels; 2: on kernels generated for it."""
        a, _ = libs()
        return int(a.cavs_app_uses_fused_path())

    @property
    def generated_kernels(self):
        """Kernels the OPT_FUSION pass generated for the programs compiled so far."""
        a, _ = libs()
        return int(a.cavs_app_generated_kernels())

    def close(self):
        a, _ = libs()
        a.cavs_app_destroy()
