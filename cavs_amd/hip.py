"""ctypes binding of the C ABI declared in include/cavs_hip.h.

The library is loaded from cavs_amd/lib; there is no CPU fallback: if the shared
object is missing, loading raises.  Device buffers are plain integers (device
addresses), typically `torch.Tensor.data_ptr()`; streams are raw hipStream_t
handles (`torch.cuda.current_stream().cuda_stream`).
"""
import ctypes as C
import os
import re

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libcavs_hip.so")
HEADER = os.path.join(os.path.dirname(_PKG), "include", "cavs_hip.h")


class CavsError(RuntimeError):
    pass


_lib = None

_P, _I, _F, _Z = C.c_void_p, C.c_int, C.c_float, C.c_size_t


class Task(C.Structure):
    """cavs_task: one job of cavs_run_tasks"""
    _fields_ = [("kind", _I), ("f0", _F), ("n0", C.c_longlong), ("n1", C.c_longlong), ("n2", C.c_longlong),
                ("p0", _P), ("p1", _P), ("p2", _P), ("p3", _P), ("p4", _P), ("p5", _P), ("p6", _P), ("p7", _P)]


TASK_TRANSPOSE, TASK_ZERO_ROWS, TASK_SGD, TASK_EMBED_SGD, TASK_SUM_PARTS, TASK_BLOCKS_SGD, TASK_PACK_T, TASK_SGD_PACK = 0, 1, 2, 3, 4, 5, 6, 7
TASK_TREELSTM_GATES_ROWS = 8
TASK_SGD_TRANSPOSE = 9
TASK_GUARD = 10


class GemmDesc(C.Structure):
    """cavs_gemm_desc: one product of cavs_sgemm_group"""
    _fields_ = [("transA", _I), ("transB", _I), ("M", _I), ("N", _I), ("K", _I), ("alpha", _F), ("beta", _F),
                ("A", _P), ("lda", _I), ("B", _P), ("ldb", _I), ("C", _P), ("ldc", _I),
                ("zero_kind", _I), ("zero_rows", _I), ("zero_col", _I)]


GEMM_C_UNUSED, GEMM_A_ZERO, GEMM_B_ZERO = 1, 2, 3


# name -> argtypes (every function returns int unless listed in _RESTYPE)
_SIGS = {
    "cavs_init": [_I],
    "cavs_device_name": [C.c_char_p, _Z],
    "cavs_malloc": [C.POINTER(_P), _Z],
    "cavs_free": [_P],
    "cavs_host_alloc": [C.POINTER(_P), _Z],
    "cavs_host_free": [_P],
    "cavs_memcpy_h2d": [_P, _P, _Z, _P],
    "cavs_memcpy_d2h": [_P, _P, _Z, _P],
    "cavs_memcpy_d2d": [_P, _P, _Z, _P],
    "cavs_zero": [_P, _Z, _P],
    "cavs_fill": [_P, _F, _Z, _P],
    "cavs_stream_create": [C.POINTER(_P)],
    "cavs_stream_destroy": [_P],
    "cavs_stream_sync": [_P],
    "cavs_event_create": [C.POINTER(_P)],
    "cavs_event_destroy": [_P],
    "cavs_event_record": [_P, _P],
    "cavs_stream_wait_event": [_P, _P],
    "cavs_graph_capture_begin": [_P],
    "cavs_graph_capture_end": [_P, C.POINTER(_P)],
    "cavs_graph_launch": [_P, _P],
    "cavs_graph_destroy": [_P],
    "cavs_event_sync": [_P],
    "cavs_event_elapsed_ms": [C.POINTER(_F), _P, _P],
    "cavs_gather_rows": [_P, _I, _P, _I, _P, _I, _I, _P],
    "cavs_scatter_rows": [_P, _I, _P, _P, _I, _I, _I, _P],
    "cavs_zero_rows": [_P, _I, _I, _I, _P],
    "cavs_copy_rows": [_P, _I, _P, _I, _I, _I, _P],
    "cavs_add_rows": [_P, _I, _P, _I, _I, _I, _P],
    "cavs_gather_children": [_P, _P, _P, _P, _I, _I, _I, _P],
    "cavs_sgemm": [_I, _I, _I, _I, _I, _F, _P, _I, _P, _I, _F, _P, _I, _P],
    "cavs_sgemm_addrows": [_I, _I, _I, _I, _I, _P, _I, _P, _I, _P, _I, _I, _P, _I, _P, _Z, _P],
    "cavs_sgemm_group": [_I, C.POINTER(GemmDesc), _P, _Z, _P],
    "cavs_sgemm_group_beside": [_I, C.POINTER(GemmDesc), _P, _Z, _P],
    "cavs_sgemm_group_embed_bwd": [_I, C.POINTER(GemmDesc), _I, _P, _P, _P, _Z, _P],
    "cavs_sgemm_splitk": [_I, _I, _I, _I, _I, _F, _P, _I, _P, _I, _F, _P, _I, _P, _Z, _P],
    "cavs_sgemm_splitk_static": [_I, _I, _I, _I, _I, _F, _P, _I, _P, _I, _F, _P, _I, _P],
    "cavs_colsum": [_P, _P, _I, _I, _I, _I, _P],
    "cavs_embed_fwd": [_P, _I, _P, _P, _I, _I, _P],
    "cavs_embed_pull_fwd": [_P, _I, _P, _P, _P, _P, _I, _I, _P],
    "cavs_embed_pull_sgemm": [_P, _I, _P, _I, _P, _P, _P, _P, _I, _I, _P, _I, _I, _I, _I, _P],
    "cavs_embed_bwd": [_P, _P, _P, _I, _I, _I, _P],
    "cavs_bias_add_rows": [_P, _P, _P, _I, _I, _P],
    "cavs_softmax_xent": [_P, _P, _P, _P, _I, _I, _P],
    "cavs_softmax_xent_part": [_P, _P, _P, _P, _I, _I, _I, _P],
    "cavs_sgd": [_P, _P, _F, _Z, _P],
    "cavs_ew_binary": [_I, _P, _P, _Z, _P, _Z, _Z, _I, _P],
    "cavs_ew_unary": [_I, _P, _P, _Z, _I, _P],
    "cavs_scale": [_P, _P, _F, _Z, _P],
    "cavs_treelstm_gates_fwd": [_P, _I, _P, _P, _P, _P, _P, _P, _I, _I, _P],
    "cavs_treelstm_gates_fwd_scatter": [_P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _P],
    "cavs_treelstm_gates_bwd": [_P, _P, _P, _P, _P, _I, _P, _P, _I, _I, _P],
    "cavs_lstm_gates_fwd": [_P, _I, _P, _P, _P, _P, _P, _I, _I, _P],
    "cavs_lstm_gates_bwd": [_P, _P, _P, _P, _P, _I, _P, _I, _I, _P],
    "cavs_treefc_fwd": [_P, _P, _P, _P, _I, _I, _I, _P],
    "cavs_treefc_bwd": [_P, _P, _P, _P, _I, _I, _I, _P],
    "cavs_treelstm_round_fwd": [_P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _P],
    "cavs_treelstm_round_fwd_packed": [_P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _P],
    "cavs_treelstm_round_leaves_fwd": [_P, _P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _P],
    "cavs_treelstm_round_bwd_gates": [_P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _I, _I, _P],
    "cavs_treelstm_round_bwd_children": [_P, _I, _P, _P, _P, _P, _I, _I, _P],
    "cavs_treelstm_round_bwd_children_gates": [_P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P],
    "cavs_treelstm_bwd_gates_rows": [_P, _I, _P, _P, _P, _P, _P, _I, _P, _P, _I, _I, _P],
    "cavs_treelstm_round_bwd_children_gates_packed": [_P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P],
    "cavs_tail_probe": [_P, _I, _I, _P],
    "cavs_treelstm_tail_fwd": [_P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _P, _I, _I, _P],
    "cavs_treelstm_tail_bwd": [_P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _I, _P, _P, _P, _P, _I, _I, _P, _I, _I, _P],
    "cavs_transpose": [_P, _P, _I, _I, _P],
    "cavs_lstm_round_fwd": [_P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _I, _I, _P],
    "cavs_lstm_round_fwd_packed": [_P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _I, _I, _P],
    "cavs_lstm_round_leaves_fwd": [_P, _P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _P],
    "cavs_lstm_round_bwd_gates": [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _P],
    "cavs_treefc_round_fwd": [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _P],
    "cavs_treefc_round_leaves_fwd": [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _P],
    "cavs_treefc_round_bwd": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _P],
    "cavs_round_bwd_children": [_P, _I, _I, _P, _I, _I, _P, _P, _I, _I, _I, _P],
    "cavs_lstm_round_bwd_children_gates": [_P, _I, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P],
    "cavs_lstm_round_bwd_children_gates_packed": [_P, _I, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P],
    "cavs_lstm_bwd_gates_rows": [_P, _I, _P, _P, _P, _P, _P, _I, _P, _I, _I, _P],
    "cavs_treefc_round_bwd_children_act": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P],
    "cavs_treefc_bwd_rows": [_P, _I, _P, _P, _P, _P, _I, _I, _P],
    "cavs_profile_arm": [_P, _P],
    "cavs_profile_disarm": [_P],
    "cavs_fc_softmax_xent": [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _Z, _I, _I, _I, _P],
    "cavs_run_tasks": [_I, C.POINTER(Task), _P],
    "cavs_sgd_multi": [_I, _P, _P, _P, _F, _P],
    "cavs_clip_grads": [_I, _P, _P, _F, _P, _Z, _P],
    "cavs_embed_sgd": [_P, _P, _P, _I, _I, _F, _P, _I, _P],
    "cavs_embed_zero_rows": [_P, _P, _I, _I, _P],
    "cavs_colsum_blocks": [_P, _P, _I, _I, _I, _I, _P, _P, _Z, _P],
    "cavs_fused_compile": [C.c_char_p, C.c_char_p, C.POINTER(_P)],
    "cavs_fused_launch": [_P, C.POINTER(_P), _I, C.POINTER(_P), _I, C.POINTER(_I), C.POINTER(_I), _I, _P],
    "cavs_fused_release": [_P],
    "cavs_cell_compile": [C.c_char_p, C.POINTER(_P)],
    "cavs_cell_launch": [_P, _I, C.c_uint, C.c_uint, C.c_uint, C.c_uint, _P, C.c_size_t, _P],
    "cavs_cell_release": [_P],
    "cavs_schedule_frontier": [_P, _I, _P, _P, _P, _P, _P, _P, _P],
    "cavs_schedule_arena": [_P, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, C.c_long, _P, _P, _Z, _P],
}
# measurement aids of cavs_amd.kernel_bench (cavs_amd/csrc/bench_probes.h): exported, not part of include/cavs_hip.h
_BENCH_SIGS = {"cavs_mfma_probe": [_P, _Z, _I, C.POINTER(C.c_double), _P]}
_RESTYPE = {"cavs_last_error": C.c_char_p, "cavs_abi_version": _I, "cavs_sgemm_splitk_workspace": _Z,
            "cavs_fc_softmax_xent_workspace": _Z, "cavs_colsum_blocks_workspace": _Z,
            "cavs_clip_grads_workspace": _Z, "cavs_sgemm_group_workspace": _Z, "cavs_fc_softmax_xent_parts": _I,
            "cavs_colsum_parts": _I, "cavs_round_packed_ok": _I, "cavs_lstm_round_packed_ok": _I,
            "cavs_tail_rounds_ok": _I, "cavs_tail_max_rounds": _I, "cavs_tail_max_groups": _I, "cavs_tail_sync_bytes": _Z,
            "cavs_sgemm_splitk_static_max_bytes": _Z,
            "cavs_schedule_arena_scratch": _Z}
_NOCHECK = {"cavs_last_error": [], "cavs_abi_version": [], "cavs_sgemm_splitk_workspace": [_I, _I, _I],
            "cavs_fc_softmax_xent_workspace": [_I, _I, _I], "cavs_colsum_blocks_workspace": [_I, _I, _I],
            "cavs_clip_grads_workspace": [_I], "cavs_sgemm_group_workspace": [_I, C.POINTER(GemmDesc)],
            "cavs_fc_softmax_xent_parts": [_I], "cavs_colsum_parts": [_I], "cavs_round_packed_ok": [_I, _I],
            "cavs_lstm_round_packed_ok": [_I, _I], "cavs_sgemm_splitk_static_max_bytes": [],
            "cavs_tail_rounds_ok": [_I, _I], "cavs_tail_max_rounds": [], "cavs_tail_max_groups": [], "cavs_tail_sync_bytes": [],
            "cavs_schedule_arena_scratch": [_I, _I]}

EW_BINARY = dict(add=0, sub=1, mul=2, div=3, sigmoid_grad=4, tanh_grad=5, relu_grad=6, equal=7)
EW_UNARY = dict(assign=0, neg=1, abs=2, square=3, sigmoid=4, tanh=5, relu=6)


def declared_symbols():
    """extern "C" function names declared in include/cavs_hip.h"""
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cavs_[a-z0-9_]+)\s*\(", text)))


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise CavsError(f"{LIB_PATH} is missing: build it with `python -m cavs_amd.build` "
                            "(there is no CPU fallback)")
        # PyTorch ships its own HIP runtime; a process that uses both must load PyTorch's first,
        # or the two runtimes each try to own the device and the second one finds none
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        l = C.CDLL(LIB_PATH)
        for name, args in list(_SIGS.items()) + list(_BENCH_SIGS.items()):
            fn = getattr(l, name)
            fn.argtypes, fn.restype = args, _I
        for name, args in _NOCHECK.items():
            fn = getattr(l, name)
            fn.argtypes, fn.restype = args, _RESTYPE[name]
        _lib = l
    return _lib


def call(name, *args):
    """Calls an int-returning entry point and raises CavsError on failure."""
    rc = getattr(lib(), name)(*args)
    if rc != 0:
        raise CavsError(f"{name} -> {rc}: {lib().cavs_last_error().decode()}")


def ptr(t):
    """device address of a torch tensor (or None / int passthrough)"""
    if t is None:
        return None
    if isinstance(t, int):
        return t
    return t.data_ptr()
