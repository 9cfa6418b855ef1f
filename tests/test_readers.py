"""The batch readers either side of the path (include/cavs/apps/readers.h): parse-tree
corpora as apps/paper/tree-lstm-cavs.cc:30-103 reads them, token streams as
apps/paper/seq-lstm-cavs-varLength.cc:27-66 loads them.

Pins: the arrays below are written out by hand from the fixture files in
tests/golden/ (three trees, six token lines); the first two trees are the two-sample
batch whose schedule is derived by hand in tests/golden/sched_kat.json, so reader ->
scheduler is checked end to end; then the C++ readers are compared with the plain
Python restatement (oracle/readers.py) over generated files.  Host only: no GPU."""
import json
import os

import numpy as np
import pytest

import readers as oracle_readers
from cavs_amd import data, hip, session

HERE = os.path.dirname(os.path.abspath(__file__))
SST = [os.path.join(HERE, "golden", "sst_tiny", f) for f in ("sents_idx.txt", "labels.txt", "parents.txt")]
PTB = os.path.join(HERE, "golden", "ptb_tiny.txt")


def test_tree_reader_known_answer():
    r = data.TreeReader(*SST, batch=2, max_vertices=5, max_words=3)
    graph, inp, lab = r.next_batch()
    assert graph.tolist() == [[2, 2, -1, -1, -1], [3, 3, 4, 4, -1]]          # parents minus one
    assert inp.tolist() == [7, 9, 0, 0, 0, 3, 4, 5, 0, 0]                    # sample i at i*max_vertices
    assert lab.tolist() == [1, 2, 3, 0, 4, 2, 1, 3, -1, -1]                  # packed back to back
    # the graph feed is the hand-derived two-tree batch: same rounds and index lists
    kat = [c for c in json.load(open(os.path.join(HERE, "golden", "sched_kat.json")))["cases"]
           if c["name"] == "two_trees_root_not_last"][0]
    tr = session.schedule_trace(graph)
    for k in ("N", "round2offset", "tids_to_jobids", "fwd", "bwd"):
        assert tr[k] == kat[k], k
    r.close()


def test_tree_reader_packs_inputs_by_vertex_id():
    r = data.TreeReader(*SST, batch=2, max_vertices=5, max_words=3)
    _, inp, _ = r.next_batch(pack_inputs=True)
    assert inp.tolist() == [7, 9, 0, 3, 4, 5, 0, 0, 0, 0]  # sample 1 starts at vertex 3


def test_tree_reader_starts_over_at_the_end_and_skips_empty_lines():
    r = data.TreeReader(*SST, batch=2, max_vertices=9, max_words=5)
    r.next_batch()
    graph, inp, lab = r.next_batch()  # third tree, then the first again
    assert graph.tolist() == [[5, 5, 6, 7, 8, 6, 7, 8, -1], [2, 2, -1, -1, -1, -1, -1, -1, -1]]
    assert inp.tolist() == [11, 12, 13, 14, 15, 0, 0, 0, 0, 7, 9, 0, 0, 0, 0, 0, 0, 0]
    assert lab.tolist() == [2] * 9 + [1, 2, 3] + [-1] * 6
    graph, _, _ = r.next_batch()
    assert graph[0, :5].tolist() == [3, 3, 4, 4, -1] and graph[1, :9].tolist() == [5, 5, 6, 7, 8, 6, 7, 8, -1]


def test_tree_reader_errors_are_reported_not_fatal(tmp_path):
    with pytest.raises(hip.CavsError, match="cannot open"):
        data.TreeReader(str(tmp_path / "nope"), SST[1], SST[2], batch=1)
    r = data.TreeReader(*SST, batch=2, max_vertices=4, max_words=3)
    with pytest.raises(hip.CavsError, match="5 vertices, limit 4"):
        r.next_batch()
    r = data.TreeReader(*SST, batch=1, max_vertices=5, max_words=1)
    with pytest.raises(hip.CavsError, match="2 words"):
        r.next_batch()
    bad = tmp_path / "parents.txt"
    bad.write_text("0 1 1\n")  # root first
    r = data.TreeReader(SST[0], SST[1], str(bad), batch=1, max_vertices=5, max_words=3)
    with pytest.raises(hip.CavsError, match="root"):
        r.next_batch()
    empty = tmp_path / "empty.txt"
    empty.write_text("\n\n")
    r = data.TreeReader(str(empty), SST[1], SST[2], batch=1, max_vertices=5, max_words=3)
    with pytest.raises(hip.CavsError, match="no sample"):
        r.next_batch()


def _write_corpus(tmp_path, seed, n_samples, trailing_newline):
    from cavs_amd import synth

    rng = np.random.default_rng(seed)
    sents, labels, parents = [], [], []
    for s in range(n_samples):
        leaves = int(rng.integers(2, 9))
        g = synth.tree_batch(seed * 100 + s, 1, leaves, leaves)[0][0]
        par = [int(p) + 1 for p in g[:2 * leaves - 1]]
        parents.append(" ".join(map(str, par)))
        sents.append(" ".join(str(int(v)) for v in rng.integers(0, 50, leaves)))
        labels.append(" ".join(str(int(v)) for v in rng.integers(0, 5, 2 * leaves - 1)))
        if rng.random() < 0.3:
            sents.append("")  # stray empty line in the word file only
    end = "\n" if trailing_newline else ""
    paths = []
    for name, lines in (("s.txt", sents), ("l.txt", labels), ("p.txt", parents)):
        p = tmp_path / name
        p.write_text("\n".join(lines) + end)
        paths.append(str(p))
    return paths


@pytest.mark.parametrize("seed,trailing", [(1, True), (2, False), (3, True)])
@pytest.mark.parametrize("batch", [1, 3, 4])
def test_tree_reader_matches_restatement(tmp_path, seed, trailing, batch):
    paths = _write_corpus(tmp_path, seed, 7, trailing)
    r = data.TreeReader(*paths, batch=batch, max_vertices=15, max_words=8)
    files = oracle_readers.TreeFiles(*paths)
    for it in range(6):  # 6 batches of up to 4 out of 7 samples: wraps around several times
        pack = bool(it % 2)
        got = r.next_batch(pack_inputs=pack)
        want = oracle_readers.tree_next_batch(files, batch, 15, 8, pack_inputs=pack)
        for g, w, what in zip(got, want, ("graph", "input", "label")):
            assert np.array_equal(g, w), (it, what)


def test_ptb_reader_known_answer():
    r = data.PtbReader(PTB, batch=2, max_length=5)
    assert len(r) == 3  # six lines, one of them empty
    graph, inp, lab = r.batch_at(0)
    assert graph.tolist() == [[1, 2, 3, -1, -1], [1, -1, -1, -1, -1]]   # chain j -> j+1, last vertex is the root
    assert inp.tolist() == [5, 6, 7, 8, 9, 10, -1, -1, -1, -1]          # packed back to back
    assert lab.tolist() == [6, 7, 8, -1, 10, -1, -1, -1, -1, -1]        # next token of the same sentence
    graph, inp, lab = r.batch_at(1)  # an empty line is a sentence without tokens
    assert graph.tolist() == [[-1] * 5, [1, 2, -1, -1, -1]]
    assert inp.tolist() == [1, 2, 3] + [-1] * 7 and lab.tolist() == [2, 3] + [-1] * 8
    graph, inp, lab = r.batch_at(2)
    assert graph.tolist() == [[1, 2, 3, 4, -1], [1, -1, -1, -1, -1]]
    assert inp.tolist() == [4, 5, 6, 7, 8, 20, 21, -1, -1, -1]
    assert lab.tolist() == [5, 6, 7, 8, -1, 21, -1, -1, -1, -1]
    with pytest.raises(hip.CavsError, match="batch 3 of 3"):
        r.batch_at(3)


def test_ptb_reader_drops_the_incomplete_batch_and_checks_lengths():
    assert len(data.PtbReader(PTB, batch=4, max_length=5)) == 1
    assert len(data.PtbReader(PTB, batch=6, max_length=5)) == 1
    assert len(data.PtbReader(PTB, batch=7, max_length=5)) == 0
    with pytest.raises(hip.CavsError, match="more than 4 tokens"):
        data.PtbReader(PTB, batch=2, max_length=4)
    with pytest.raises(hip.CavsError, match="cannot open"):
        data.PtbReader(PTB + ".missing", batch=2)


@pytest.mark.parametrize("batch", [1, 2, 3, 5])
def test_ptb_reader_matches_restatement(tmp_path, batch):
    rng = np.random.default_rng(batch)
    lines = [" ".join(str(int(v)) for v in rng.integers(0, 1000, int(rng.integers(1, 12)))) for _ in range(11)]
    p = tmp_path / "ptb.txt"
    p.write_text("\n".join(lines) + "\n")
    want = oracle_readers.ptb_load(str(p), batch, 12)
    r = data.PtbReader(str(p), batch=batch, max_length=12)
    assert len(r) == len(want) == 11 // batch
    for k, w in enumerate(want):
        for g, ww, what in zip(r.batch_at(k), w, ("graph", "input", "label")):
            assert np.array_equal(g, ww), (k, what)
    # every graph row is a chain the scheduler accepts: one vertex per round and sample
    tr = session.schedule_trace(r.batch_at(0)[0])
    assert tr["N"] == int((r.batch_at(0)[1] >= 0).sum())


def test_library_exports_every_declared_reader_symbol():
    import re

    from cavs_amd import apps

    header = os.path.join(os.path.dirname(HERE), "include", "cavs", "apps", "readers.h")
    names = sorted(set(re.findall(r"\b(cavs_\w+)\s*\(", open(header).read())))
    assert len(names) == 7, names
    a, _ = apps.libs()
    assert not [n for n in names if not hasattr(a, n)]
