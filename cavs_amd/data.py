"""Batch readers of the benchmark applications (include/cavs/apps/readers.h, built into
libcavs_apps.so): the parse-tree reader of apps/paper/tree-lstm-cavs.cc:30-103 and the
token-stream loader of apps/paper/seq-lstm-cavs-varLength.cc:27-66.  Host memory only.

The arrays they return are the feeds of Session.step / App.step: `graph` [batch, maxlen]
int32 parent arrays (-1 = root and padding), `x` and `labels` float32.
"""
import ctypes as C

import numpy as np

from . import apps, hip

_ready = False


def _lib():
    global _ready
    a, _ = apps.libs()
    if not _ready:
        a.cavs_reader_last_error.restype = C.c_char_p
        a.cavs_tree_reader_open.argtypes = [C.c_char_p, C.c_char_p, C.c_char_p, C.POINTER(C.c_void_p)]
        a.cavs_tree_reader_next.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        a.cavs_tree_reader_close.argtypes = [C.c_void_p]
        a.cavs_ptb_reader_load.argtypes = [C.c_char_p, C.c_int, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_int)]
        a.cavs_ptb_reader_batch.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        a.cavs_ptb_reader_close.argtypes = [C.c_void_p]
        _ready = True
    return a


def _check(a, rc):
    if rc != 0:
        raise hip.CavsError(a.cavs_reader_last_error().decode())


class TreeReader:
    """sents_idx.txt / labels.txt / parents.txt, one sample per line.  max_vertices and
    max_words are MAX_DEPENDENCY and MAX_LEN of tree-lstm-cavs.cc:22-23."""

    def __init__(self, input_path, label_path, graph_path, *, batch, max_vertices=111, max_words=56):
        self._a = _lib()
        self._h = C.c_void_p()
        self.batch, self.max_vertices, self.max_words = batch, max_vertices, max_words
        _check(self._a, self._a.cavs_tree_reader_open(str(input_path).encode(), str(label_path).encode(),
                                                      str(graph_path).encode(), C.byref(self._h)))

    def next_batch(self, pack_inputs=False):
        """-> (graph [batch, max_vertices] int32, input [batch*max_vertices] float32, label likewise).
        pack_inputs=False is the reference's layout (sample i at i*max_vertices); True packs the
        word ids by global vertex id, the order the vertex function pulls them in."""
        n = self.batch * self.max_vertices
        graph = np.empty(n, np.int32)
        inp = np.empty(n, np.float32)
        lab = np.empty(n, np.float32)
        _check(self._a, self._a.cavs_tree_reader_next(self._h, self.batch, self.max_vertices, self.max_words,
                                                      int(pack_inputs), graph.ctypes.data, inp.ctypes.data, lab.ctypes.data))
        return graph.reshape(self.batch, self.max_vertices), inp, lab

    def close(self):
        if self._h:
            self._a.cavs_tree_reader_close(self._h)
            self._h = C.c_void_p()

    __del__ = close


class PtbReader:
    """One sentence of token ids per line; batches of `batch` sentences, the incomplete last one
    dropped.  max_length is MAX_LENGTH of seq-lstm-cavs-varLength.cc:25."""

    def __init__(self, path, *, batch, max_length=83):
        self._a = _lib()
        self._h = C.c_void_p()
        self.batch, self.max_length = batch, max_length
        n = C.c_int()
        _check(self._a, self._a.cavs_ptb_reader_load(str(path).encode(), batch, max_length, C.byref(self._h), C.byref(n)))
        self.n_batches = n.value

    def __len__(self):
        return self.n_batches

    def batch_at(self, k):
        """-> (graph [batch, max_length] int32, input [batch*max_length] float32, label likewise)"""
        n = self.batch * self.max_length
        graph = np.empty(n, np.int32)
        inp = np.empty(n, np.float32)
        lab = np.empty(n, np.float32)
        _check(self._a, self._a.cavs_ptb_reader_batch(self._h, k, graph.ctypes.data, inp.ctypes.data, lab.ctypes.data))
        return graph.reshape(self.batch, self.max_length), inp, lab

    def close(self):
        if self._h:
            self._a.cavs_ptb_reader_close(self._h)
            self._h = C.c_void_p()

    __del__ = close
