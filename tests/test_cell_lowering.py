"""Lowering of a vertex function of the general shape onto generated kernels, the parts that need
no device: what the analysis of F accepts and refuses, how it cuts a function of several stages
into a chain of cells, and the elementwise part of the backward function it derives for every cell
-- compiled for the host in double and held against central differences of the generated forward
part (a wrong sign, a dropped term or a swapped operand of the derivation fails this)."""
import ctypes as C
import os
import re
import subprocess
import tempfile

import numpy as np
import pytest

from cavs_amd import apps


def _dump(what):
    _, h = apps.libs()
    h.C_DumpCell.restype = C.c_size_t
    h.C_DumpCell.argtypes = [C.c_char_p, C.c_size_t, C.c_int]
    n = h.C_DumpCell(None, 0, what)
    buf = C.create_string_buffer(n)
    h.C_DumpCell(buf, n, what)
    return buf.value.decode()


def _declare(model, H=64):
    return apps.App(model, B=3, maxlen=8, H=H, E=8, V=20, C_=4, opt=-1)


HARNESS = r"""
#include <math.h>
#include <string.h>
#define float double
%s
#undef float
extern "C" {
int sizes(int *s) { s[0] = sizeof(FwdIn) / 8; s[1] = sizeof(FwdOut) / 8; s[2] = sizeof(BwdIn) / 8; s[3] = sizeof(BwdOut) / 8; return 0; }
void fwd(const double *in, double *out) { FwdIn i; FwdOut o; memcpy(&i, in, sizeof i); cell_forward(i, o); memcpy(out, &o, sizeof o); }
void bwd(const double *in, double *out) { BwdIn i; BwdOut o; memcpy(&i, in, sizeof i); cell_backward(i, o); memcpy(out, &o, sizeof o); }
}
"""


# the seeded family cell<seed> (cavs_amd/host/apps/models.cc: RandomCell): bits 0-2 choose the number of
# children, state blocks and gates, the higher ones each gate's left operand and activation
CELL_SEEDS = [(i & 7) | (((i * 2654435761) >> 7 & 0x1FFF) << 3) for i in range(16)]


# members of the family with two or three stages of products (bits 16-17), which run as chains of cells
CHAIN_SEEDS = [(1 + i % 2) << 16 | (i * 5 + 3) & 7 | (((i * 2246822519) >> 9 & 0x1FFF) << 3) for i in range(10)]
FD_MODELS = ["treelstm", "treelstm2", "treegate", "lstm", "treefc", "treefc_x", "treegru", "treedeep"] + [f"cell{s}" for s in CELL_SEEDS + CHAIN_SEEDS]


@pytest.mark.parametrize("model", FD_MODELS)
def test_derived_backward_part_equals_central_differences_of_the_forward_part(model, tmp_path):
    """Every cell of the chain F is cut into (one cell for a function of one stage)."""
    a = _declare(model)
    srcs = [_dump(0)]
    stages = int(re.search(r"// stages=(\d+)", srcs[0]).group(1))
    srcs += [_dump(10 * st) for st in range(1, stages)]
    a.close()
    want_stages = {"treegru": 2, "treedeep": 3}.get(model, 1 + (int(model[4:]) >> 16 & 3) if model.startswith("cell") else 1)
    assert stages == want_stages
    for st, src in enumerate(srcs):
        _held_to_central_differences(src, tmp_path / str(st))


def _held_to_central_differences(src, tmp_path):
    tmp_path.mkdir()
    dims = {k: int(v) for k, v in re.findall(r"(\w+)=(\d+)", [l for l in src.splitlines() if l.startswith("// H=")][0])}
    K, S, SI, NX, XD, NP, NB, ND, NSV = (dims[k] for k in ("K", "S", "SI", "NX", "XD", "NP", "NB", "ND", "NSV"))
    prod_col = [int(c) for c in re.findall(r"// product \d+ dcol (\d+)", src)]
    bias_col = [int(c) for c in re.findall(r"// bias \d+ dcol (\d+)", src)]
    assert len(prod_col) == NP and len(bias_col) == NB
    cc = tmp_path / "cell.cc"
    cc.write_text(HARNESS % src)
    so = tmp_path / "cell.so"
    subprocess.run(["g++", "-O1", "-shared", "-fPIC", "-o", str(so), str(cc)], check=True)
    lib = C.CDLL(str(so))
    sz = (C.c_int * 4)()
    lib.sizes(sz)
    nxm, nbm, nsvm, xdm = max(1, NX), max(1, NB), max(1, NSV), max(1, XD)
    assert list(sz) == [nxm + NP + nbm + K * SI + xdm, S + 1 + nsvm, S + 1 + nsvm + K * SI, ND + K * SI]
    dp = C.POINTER(C.c_double)

    def fwd(x):
        out = np.zeros(sz[1])
        lib.fwd(np.ascontiguousarray(x).ctypes.data_as(dp), out.ctypes.data_as(dp))
        return out

    rng = np.random.default_rng(5)
    for _ in range(20):
        x = rng.normal(0, 0.8, sz[0])
        seed = rng.normal(0, 1, S + 1)  # d st[0..S), d ret
        out = fwd(x)
        bin_ = np.concatenate([seed, out[S + 1:], x[nxm + NP + nbm:nxm + NP + nbm + K * SI]])
        bout = np.zeros(sz[3])
        lib.bwd(bin_.ctypes.data_as(dp), bout.ctypes.data_as(dp))
        num = np.zeros(sz[0])
        eps = 1e-6
        for i in range(sz[0]):
            e = np.zeros(sz[0])
            e[i] = eps
            num[i] = (seed @ (fwd(x + e)[: S + 1] - fwd(x - e)[: S + 1])) / (2 * eps)
        want = np.zeros(sz[0])
        for i in range(NX):
            want[i] = bout[i]
        for p in range(NP):
            want[nxm + p] = bout[prod_col[p]]
        for i in range(NB):
            want[nxm + NP + i] = bout[bias_col[i]]
        want[nxm + NP + nbm:nxm + NP + nbm + K * SI] = bout[ND:]
        live = np.ones(sz[0], bool)
        live[nxm + NP + nbm + K * SI:] = False  # the pulled vertex input is a feed: no gradient is derived for it
        np.testing.assert_allclose(want[live], num[live], rtol=1e-6, atol=1e-8)


def test_the_reference_tree_lstm_keeps_six_values_and_six_gradient_blocks_per_vertex():
    """The same as the hand-written kernels keep: the five gates and tanh(c); d(x W) in four blocks
    plus the two forget gates' own."""
    a = _declare("treelstm")
    src = _dump(0)
    dev = _dump(1)
    a.close()
    assert "NX=4 XD=0 NP=5 NB=4 ND=6 NSV=6" in src
    assert "#define CELL_NA 3" in dev and "#define CELL_NT 5" in dev and "#define CELL_DS_MASK 2" in dev
    assert dev.count("__builtin_amdgcn_mfma_f32_16x16x4f32") == 10  # five per direction and k step


def test_what_is_not_of_the_general_shape_says_why():
    a = _declare("treelstm", H=40)
    assert "multiple of 32" in _dump(1)
    a.close()


def test_a_tree_gru_is_cut_into_two_cells():
    """The candidate's product reads r * (h_l + h_r), which depends on the products behind r: the
    first cell writes [r * hs, z, z * hs] per vertex, the second gathers that row as the state of
    its one child, multiplies its first block and writes h."""
    a = _declare("treegru")
    first, second, none = _dump(0), _dump(10), _dump(20)
    dev = _dump(11)
    a.close()
    assert "// stages=2" in first and "K=2 S=3 SI=1 NX=3 XD=0 NP=2 NB=2" in first
    assert "// stages=2" in second and "K=1 S=1 SI=3 NX=3 XD=0 NP=1 NB=1" in second
    assert "no such stage" in none
    assert "#define CELL_HAS_RET 1" in dev and "#define CELL_K 1" in dev
