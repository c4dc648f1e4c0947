"""Pins the CPU restatement of the draft-side expansion (oracle/draft_oracle.py) by checks that
do not repeat its formulas: float64 log-softmax, a full sort, and ground-truth parent pointers
tracked separately from the parents table (mlx_eagle.py:97-213)."""
import numpy as np
import pytest

from oracle import draft_oracle, tree_oracle


def test_logsoftmax_topk_against_float64():
    rng = np.random.default_rng(0)
    for V, k in ((50, 4), (1000, 8), (152064, 8)):
        logits = rng.normal(0, 2.0, (3, V)).astype(np.float16)
        x = logits.astype(np.float64)
        ref = x - (np.log(np.exp(x - x.max(1, keepdims=True)).sum(1, keepdims=True)) + x.max(1, keepdims=True))
        for mode in (0, 1):
            idx, sc = draft_oracle.logsoftmax_topk(logits, k, mode)
            assert idx.shape == (3, k) and sc.dtype == np.float16
            for r in range(3):
                got = sc[r].astype(np.float64)
                want = ref[r][idx[r]]
                # two fp16 roundings on the way (mode 0: lse and the difference; mode 1: p and log p)
                assert np.all(np.abs(got - want) <= 2.5 * np.spacing(np.abs(want).astype(np.float16)).astype(np.float64))
                assert np.all(np.diff(got) <= 0)                      # best first
                # nothing outside the selection beats the last selected entry by more than rounding
                rest = np.delete(ref[r], idx[r])
                assert rest.max() <= want.min() + 0.05
                if mode == 0:                                         # exact order on the logits
                    order = sorted(range(V), key=lambda j: (-float(logits[r, j]), j))[:k]
                    assert list(idx[r]) == order
                else:                                                 # ties in fp16: lowest index first
                    for a in range(k - 1):
                        if sc[r, a] == sc[r, a + 1]:
                            assert idx[r, a] < idx[r, a + 1]


def test_logsoftmax_mode1_orders_by_the_fp16_score():
    # two logits whose fp16 log-probabilities coincide: the lower index comes first even though
    # its logit is the smaller one
    V = 4096
    logits = np.full((1, V), -4.0, np.float16)
    logits[0, 100] = np.float16(3.002)
    logits[0, 7] = np.float16(3.0)
    idx, sc = draft_oracle.logsoftmax_topk(logits, 2, 1)
    if sc[0, 0] == sc[0, 1]:
        assert list(idx[0]) == [7, 100]
    idx0, _ = draft_oracle.logsoftmax_topk(logits, 2, 0)
    assert list(idx0[0]) == [100, 7]


def test_tree_level_brute_force():
    rng = np.random.default_rng(1)
    for k in (2, 4, 8):
        for trial in range(20):
            # coarse scores so that exact ties occur
            tsc = (-rng.integers(1, 30, (k, k)) / 4).astype(np.float16)
            tsc = -np.sort(-tsc, axis=1)
            tidx = rng.integers(0, 1000, (k, k)).astype(np.int32)
            cur = (-rng.integers(1, 30, k) / 4).astype(np.float16)
            ids, sc, out_ids, cu, cs = draft_oracle.tree_level(tidx, tsc, cur, k)
            flat = [(float(np.float16(np.float32(tsc[r, c]) + np.float32(cur[r]))), r * k + c)
                    for r in range(k) for c in range(k)]
            best = sorted(flat, key=lambda t: (-t[0], t[1]))[:k]
            assert [b[1] for b in best] == list(cs)
            assert [b[0] for b in best] == [float(v) for v in sc]
            assert list(out_ids) == [b[1] // k for b in best]
            assert list(ids) == [int(tidx.reshape(-1)[b[1]]) for b in best]


@pytest.mark.parametrize("depth,k,total", [(1, 8, 7), (3, 8, 31), (5, 8, 31), (4, 4, 15), (8, 8, 31)])
def test_parents_and_masks_against_ground_truth(monkeypatch, depth, k, total):
    """Random logits in place of the draft model; the true parent of every candidate is tracked
    here from the selections alone, and must agree with the parents table, with the mask rows
    every forward receives, and with the ancestor matrix process_draft_tree builds."""
    rng = np.random.default_rng(depth * 100 + k)
    V, offset = 300, 11
    seen = []

    def fake_forward(args, weights, inv, sc, ids, positions, mask, cache, write_offset):
        seen.append(dict(ids=np.array(ids), positions=np.array(positions), mask=np.array(mask),
                         write_offset=write_offset))
        return rng.normal(0, 2.0, (len(ids), V)).astype(np.float16)

    monkeypatch.setattr(draft_oracle, "draft_forward", fake_forward)
    t0 = rng.choice(V, k, replace=False).astype(np.int32)
    p0 = -np.sort(rng.uniform(1, 6, k)).astype(np.float16)
    parents, tokens, scores = draft_oracle.generate_draft_tree(None, None, None, 1.0, t0, p0, None,
                                                               offset, depth, k)
    C = k + k * k * depth
    assert parents.shape == (1 + k * depth,) and tokens.shape == (C,) and scores.shape == (C,)
    # ground truth from the selections: inputs[i][r] = flat id of the r-th input node of level i
    true_parent = {f: None for f in range(k)}
    inputs = [list(range(k))]
    for i in range(depth):
        base = k + k * k * i
        for r in range(k):
            for c in range(k):
                true_parent[base + k * r + c] = inputs[i][r]
        block = [(float(scores[base + j]), j) for j in range(k * k)]
        sel = [j for _, j in sorted(block, key=lambda t: (-t[0], t[1]))[:k]]
        inputs.append([base + j for j in sel])
        # the cumulative score of a child never exceeds its parent's
        for j in range(k * k):
            assert scores[base + j] <= scores[inputs[i][j // k]]

    def ancestors(f):
        out = set()
        while f is not None:
            out.add(f)
            f = true_parent[f]
        return out

    for f in range(C):
        row = parents[f // k]
        assert (row == 0) == (true_parent[f] is None)
        if true_parent[f] is not None:
            assert int(row) - 1 == true_parent[f]
    assert len(seen) == depth
    for i, call in enumerate(seen):
        assert call["write_offset"] == offset + k * i
        assert np.all(call["positions"] == offset + i)
        assert list(call["ids"]) == [int(tokens[f]) for f in inputs[i]]
        m = call["mask"]
        assert m.shape == (k, offset + k * (i + 1)) and np.all(m[:, :offset] == 0)
        for r in range(k):
            anc = ancestors(inputs[i][r])
            for lvl in range(i + 1):
                for q in range(k):
                    vis = m[r, offset + k * lvl + q] == 0
                    assert vis == (inputs[lvl][q] in anc)
    # the tree process_draft_tree lays out has the same ancestor sets
    pos, midx, toks, anc = tree_oracle.process_draft_tree(scores, tokens, parents, 5, k, total)
    sel = sorted(sorted(range(C), key=lambda f: (-float(scores[f]), f))[:total])
    for a, f in enumerate(sel):
        want = {0} | {1 + sel.index(g) for g in ancestors(f)}
        assert set(np.nonzero(anc[a + 1])[0]) == want
        assert pos[a + 1] == len(want) - 1
