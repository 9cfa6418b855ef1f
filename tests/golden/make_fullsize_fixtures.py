"""Writes tests/golden/fullsize_C4.npz and fullsize_C5.npz: what the CPU checker, evaluated in
double precision, produces for one training step of the benchmark configurations C4 (variable-length
LSTM, 128 sequences, H = 512, 10000-way head) and C5 (256 trees of up to 511 vertices, E = H = 1024)
at their full sizes.  The checker needs minutes for these, so the GPU suite does not run it; it
compares the GPU step with what is recorded here.

Per tensor (loss, graph_out, dgraph_out and every parameter gradient): its shape, its Euclidean
norm, its sum, and 512 entries at fixed pseudo-random positions (their flat indices are stored
with them), all as float64.

Run from the repository root:  python tests/golden/make_fullsize_fixtures.py [C4] [C5]
"""
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "oracle"))

SAMPLES = 512


def sample_positions(name, size):
    """fixed positions: a multiplicative hash of the tensor's name seeds a splitmix stream"""
    from cavs_amd import synth

    seed = sum((i + 1) * ord(c) for i, c in enumerate(name)) + 977 * (size % 65521)
    r = synth.SplitMix64(seed)
    k = min(SAMPLES, size)
    return np.unique(np.minimum((r.bulk_uniform(k) * size).astype(np.int64), size - 1))


def summarise(tensors):
    out = {}
    for name, t in tensors.items():
        flat = np.asarray(t, np.float64).ravel()
        idx = sample_positions(name, flat.size)
        out[name + ".shape"] = np.asarray(np.shape(t), np.int64)
        out[name + ".norm"] = np.float64(np.sqrt((flat * flat).sum()))
        out[name + ".sum"] = np.float64(flat.sum())
        out[name + ".absmax"] = np.float64(np.abs(flat).max())
        out[name + ".idx"] = idx
        out[name + ".val"] = flat[idx]
    return out


def main(names):
    import pyoracle
    from cavs_amd import synth

    for name in names:
        w = synth.make_workload(name)
        t0 = time.time()
        want = pyoracle.model_step(w["model"], w["graph"], w["x"], w["labels"], w["params"], H=w["H"], E=w["E"], V=w["V"], Cc=w["C"],
                                   loss="softmax", pairing="reference", precise=True, threads=os.cpu_count() or 1)
        tensors = dict(loss=want["loss"], graph_out=want["graph_out"], dgraph_out=want["dgraph_out"])
        tensors.update(want["grads"])
        out = summarise(tensors)
        out["N"] = np.int64(want["N"])
        path = os.path.join(ROOT, "tests", "golden", f"fullsize_{name}.npz")
        np.savez_compressed(path, **out)
        print(f"{name}: N = {want['N']}, {time.time() - t0:.0f} s, {os.path.getsize(path)} bytes -> {path}", flush=True)


if __name__ == "__main__":
    main(sys.argv[1:] or ["C4", "C5"])
