"""CPU restatement of the reference's two batch readers, in plain Python.

Test infrastructure: imported only by tests/.  The product package never imports it.

tree_next_batch follows Reader::next_batch of apps/paper/tree-lstm-cavs.cc:37-71 (with
process_data :75-83 and process_graph :86-96); ptb_load follows load() of
apps/paper/seq-lstm-cavs-varLength.cc:27-66.  Pinned by tests/test_readers.py against
arrays written out by hand from the fixture files and against the hand-derived schedule
of the two-sample batch (leaves 0,1 -> root 2; (0,1)->3, (2,3)->4).
"""
import numpy as np


def _ints(line):
    out = []
    for tok in line.split():
        try:
            out.append(int(tok))
        except ValueError:
            break
    return out


class TreeFiles:
    """The three line streams with the reference's end-of-file behaviour: a read that runs
    into the end sets `eof`; the next batch loop iteration then starts all three over."""

    def __init__(self, input_path, label_path, graph_path):
        self.lines = [open(p).read().split("\n") for p in (input_path, label_path, graph_path)]
        # a final newline leaves one empty trailing element: the read that returns it is the
        # one that hits the end of the file
        self.pos = [0, 0, 0]
        self.eof = False

    def rewind(self):
        self.pos = [0, 0, 0]
        self.eof = False

    def getline(self, k):
        lines, p = self.lines[k], self.pos[k]
        if p >= len(lines):
            if k == 0:
                self.eof = True
            return ""
        self.pos[k] = p + 1
        if p == len(lines) - 1 and k == 0:
            self.eof = True  # last line has no newline after it: reading it touches the end
        return lines[p]


def tree_next_batch(files, batch, max_vertices, max_words, pack_inputs=False):
    total = batch * max_vertices
    inp = np.zeros(total, np.float32)          # :38
    lab = np.full(total, -1, np.float32)       # :39
    graph = np.full(total, -1, np.int32)       # :40
    i = label_length = vertices = 0
    while i < batch:                           # :43
        if files.eof:                          # :44-51
            files.rewind()
        s = files.getline(0)                   # :54
        if len(s) == 0:                        # :55
            continue
        ls, gs = files.getline(1), files.getline(2)   # :56-57
        parents = [v - 1 for v in _ints(gs)]   # :91 (val - 1)
        assert parents[-1] == -1               # :95
        assert max_vertices >= len(parents)    # :60
        words = _ints(s)
        assert max_words >= len(words)         # :63
        labels = _ints(ls)
        assert max_vertices >= len(labels)     # :66
        graph[i * max_vertices:i * max_vertices + len(parents)] = parents   # :59
        base = vertices if pack_inputs else i * max_vertices                # :62
        inp[base:base + len(words)] = words
        lab[label_length:label_length + len(labels)] = labels               # :65
        label_length += len(labels)            # :67
        vertices += len(parents)
        i += 1                                 # :68
    return graph.reshape(batch, max_vertices), inp, lab


def ptb_load(path, batch, max_length):
    lines = open(path).read().split("\n")
    if lines and lines[-1] == "":
        lines.pop()  # the text after the last newline is not a line
    out, pos = [], 0
    while True:
        inp = np.full(batch * max_length, -1, np.float32)    # :36
        lab = np.full(batch * max_length, -1, np.float32)    # :37
        graph = np.full(batch * max_length, -1, np.int32)    # :38
        outer, end = 0, False
        for sample in range(batch):                          # :40
            if pos >= len(lines):                            # :41-44
                end = True
                break
            toks = []
            for t in lines[pos].split():                     # :46-51
                try:
                    toks.append(float(t))
                except ValueError:
                    break
            pos += 1
            inp[outer:outer + len(toks)] = toks
            if len(toks) > 1:
                lab[outer:outer + len(toks) - 1] = toks[1:]  # :52
            for j in range(1, len(toks)):                    # :53-55
                graph[j - 1 + sample * max_length] = j
            outer += len(toks)                               # :56
        if end:                                              # :59-60
            break
        out.append((graph.reshape(batch, max_length), inp, lab))
    return out
