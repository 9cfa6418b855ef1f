"""Portable seeded generators for the synthetic workloads.

The reference's apps read SST / PTB files from hard-coded paths that are not in
the repository (apps/paper/tree-lstm-cavs.cc:26-28, seq-lstm-cavs.cc:21), so the
workloads are synthesised.  Everything derives from splitmix64 so that the same
seed gives the same batch on any platform and numpy version.

Wire formats follow the reference's feeds:
  * graph  : int32 [B, maxlen], entry j = local parent of vertex j, first -1 marks
             the root and the end of the sample (cavs/midend/graph_scheduler.cc:35-43)
  * vertex inputs and labels: float32, packed by global vertex id
             (apps/paper/seq-lstm-cavs-varLength.cc:38-56)
"""
import math

import numpy as np

_M64 = (1 << 64) - 1


class SplitMix64:
    def __init__(self, seed):
        self.s = seed & _M64

    def next(self):
        self.s = (self.s + 0x9E3779B97F4A7C15) & _M64
        z = self.s
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
        return z ^ (z >> 31)

    def uniform(self):
        """float in [0,1) with a 24-bit mantissa"""
        return (self.next() >> 40) / float(1 << 24)

    def randint(self, lo, hi):
        """integer uniform over lo..hi inclusive"""
        return lo + self.next() % (hi - lo + 1)

    def normal(self):
        u1 = max(self.uniform(), 2.0 ** -24)
        u2 = self.uniform()
        return math.sqrt(-2.0 * math.log(u1)) * math.cos(2.0 * math.pi * u2)

    def bulk_u64(self, n):
        """n draws, vectorised; advances the state by n"""
        with np.errstate(over="ignore"):
            idx = np.arange(1, n + 1, dtype=np.uint64)
            z = np.uint64(self.s) + idx * np.uint64(0x9E3779B97F4A7C15)
            self.s = int(z[-1]) if n else self.s
            z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
            z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
            return z ^ (z >> np.uint64(31))

    def bulk_uniform(self, n, lo=0.0, hi=1.0):
        u = (self.bulk_u64(n) >> np.uint64(40)).astype(np.float64) / float(1 << 24)
        return (lo + (hi - lo) * u).astype(np.float32)

    def bulk_normal(self, n, mean=0.0, sd=1.0):
        m = (n + 1) // 2
        u1 = np.maximum(self.bulk_uniform(m).astype(np.float64), 2.0 ** -24)
        u2 = self.bulk_uniform(m).astype(np.float64)
        r = np.sqrt(-2.0 * np.log(u1))
        z = np.concatenate([r * np.cos(2 * np.pi * u2), r * np.sin(2 * np.pi * u2)])[:n]
        return (mean + sd * z).astype(np.float32)


def random_binary_tree(rng, leaves):
    """Parent array of a full binary tree with `leaves` leaves and a uniformly
    random bracketing (recursive uniform split).  Vertices: leaves 0..L-1 left to
    right, then internal vertices in post-order, so the root is the last vertex,
    which is what LoadGraph requires (graph_scheduler.cc:39)."""
    n = 2 * leaves - 1
    parent = [-1] * n
    next_id = [leaves]

    def build(lo, hi):  # returns the vertex id of the subtree over leaves lo..hi-1
        if hi - lo == 1:
            return lo
        k = rng.randint(1, hi - lo - 1)
        left = build(lo, lo + k)
        right = build(lo + k, hi)
        me = next_id[0]
        next_id[0] += 1
        parent[left] = me
        parent[right] = me
        return me

    build(0, leaves)
    return parent


def pack_graph(parents_list, maxlen):
    B = len(parents_list)
    g = np.full((B, maxlen), -1, dtype=np.int32)
    for i, p in enumerate(parents_list):
        assert len(p) <= maxlen and p[-1] == -1
        g[i, : len(p)] = p
    return g


def chain(length):
    """apps/paper/seq-lstm-cavs.cc:118: vertex k's parent is k+1, last is the root"""
    return list(range(1, length)) + [-1]


def tree_batch(seed, B, leaf_lo, leaf_hi, maxlen=None, leaf_dist="uniform"):
    rng = SplitMix64(seed)
    trees, leaves = [], []
    for _ in range(B):
        if leaf_dist == "uniform":
            L = rng.randint(leaf_lo, leaf_hi)
        else:  # clipped normal (mean, sd) given as leaf_dist=("normal", mean, sd)
            _, mean, sd = leaf_dist
            L = int(min(max(round(mean + sd * rng.normal()), leaf_lo), leaf_hi))
        leaves.append(L)
        trees.append(random_binary_tree(rng, L))
    if maxlen is None:
        maxlen = 2 * leaf_hi - 1
    return pack_graph(trees, maxlen), leaves, rng


def chain_batch(seed, B, len_lo, len_hi, maxlen=None):
    rng = SplitMix64(seed)
    lens = [rng.randint(len_lo, len_hi) for _ in range(B)]
    if maxlen is None:
        maxlen = len_hi
    return pack_graph([chain(n) for n in lens], maxlen), lens, rng


def zipf_ids(rng, n, vocab, s=1.1):
    """inverse-CDF Zipf(s) over 0..vocab-1"""
    w = 1.0 / np.power(np.arange(1, vocab + 1, dtype=np.float64), s)
    cdf = np.cumsum(w) / np.sum(w)
    u = rng.bulk_uniform(n).astype(np.float64)
    return np.minimum(np.searchsorted(cdf, u), vocab - 1).astype(np.float32)


def total_length(graph):
    return int(sum(int(np.argmax(row == -1)) + 1 for row in graph))


# --------------------------------------------------------------------------- configs
def make_workload(name, seed=None, scale=1.0, B=None):
    """The five benchmark configurations.  Returns a dict with
    model, dims, graph, x, labels and params (float32 numpy arrays)."""
    H_scale = scale
    if name == "C1":  # chain LSTM, fixed length 20
        seed = 1001 if seed is None else seed
        B = B or 16
        V, H, T, C = 1000, max(4, int(128 * H_scale)), 20, 1000
        graph, lens, rng = chain_batch(seed, B, T, T, T)
        N = sum(lens)
        x = np.floor(rng.bulk_uniform(N) * V).astype(np.float32)
        # label = next token within the sample (seq-lstm-cavs-varLength.cc:50)
        labels = np.empty(N, np.float32)
        o = 0
        for n in lens:
            labels[o : o + n - 1] = x[o + 1 : o + n]
            labels[o + n - 1] = x[o]
            o += n
        model, E = "lstm", H
    elif name == "C4":  # variable-length LSTM
        seed = 4004 if seed is None else seed
        B = B or 128
        V, H, C = 10000, max(4, int(512 * H_scale)), 10000
        graph, lens, rng = chain_batch(seed, B, 10, 100, 100)
        N = sum(lens)
        x = zipf_ids(rng, N, V)
        labels = np.empty(N, np.float32)
        o = 0
        for n in lens:
            labels[o : o + n - 1] = x[o + 1 : o + n]
            labels[o + n - 1] = x[o]
            o += n
        model, E = "lstm", H
    elif name == "C2":  # Tree-FC
        seed = 2002 if seed is None else seed
        B = B or 64
        H = max(4, int(256 * H_scale))
        graph, leaves, rng = tree_batch(seed, B, 2, 64, 127)
        N = sum(2 * l - 1 for l in leaves)
        x = np.zeros((N, H), np.float32)
        o = 0
        for l in leaves:  # N(0,1) inputs for leaves, zeros for internal vertices
            x[o : o + l] = rng.bulk_normal(l * H).reshape(l, H)
            o += 2 * l - 1
        labels = np.zeros(N, np.float32)
        model, E, V, C = "treefc", H, 0, 0
    elif name in ("C3", "C5"):
        if name == "C3":
            seed = 3003 if seed is None else seed
            B = B or 64
            V, E, H, C = 21701, max(4, int(300 * H_scale)), max(4, int(512 * H_scale)), 5
            graph, leaves, rng = tree_batch(seed, B, 2, 56, 111, ("normal", 19.0, 9.0))
        else:
            seed = 5005 if seed is None else seed
            B = B or 256
            V, E, H, C = 21701, max(4, int(1024 * H_scale)), max(4, int(1024 * H_scale)), 5
            graph, leaves, rng = tree_batch(seed, B, 32, 256, 511)
        N = sum(2 * l - 1 for l in leaves)
        x = np.zeros(N, np.float32)
        o = 0
        for l in leaves:  # word ids for leaves, 0 for internal (tree-lstm-cavs.cc:38)
            x[o : o + l] = np.floor(rng.bulk_uniform(l) * V)
            o += 2 * l - 1
        labels = np.floor(rng.bulk_uniform(N) * C).astype(np.float32)
        model = "treelstm"
    else:
        raise ValueError(name)

    p = {}
    if model == "treelstm":
        p["Emb"] = rng.bulk_normal(V * E, 0.0, 0.1).reshape(V, E)
        p["W"] = rng.bulk_uniform(E * 4 * H, -0.1, 0.1).reshape(E, 4 * H)
        p["U"] = rng.bulk_uniform(4 * H * H, -0.1, 0.1)
        p["Bv"] = np.zeros(4 * H, np.float32)
    elif model == "lstm":
        p["Emb"] = rng.bulk_uniform(V * H, -0.1, 0.1).reshape(V, H)
        p["W"] = rng.bulk_uniform(8 * H * H, -0.1, 0.1)
        p["Bv"] = np.zeros(4 * H, np.float32)
    else:
        p["W"] = rng.bulk_uniform(2 * H * H, -0.1, 0.1).reshape(2 * H, H)
        p["Bv"] = np.zeros(H, np.float32)
    if C:
        p["Wfc"] = rng.bulk_uniform(C * H, -0.1, 0.1).reshape(C, H)
        p["bfc"] = np.zeros(C, np.float32)
    return dict(name=name, model=model, B=B, V=V, E=E, H=H, C=C, N=N, graph=graph, x=x,
                labels=labels, params=p, seed=seed)
