"""Device-side tree construction, path extraction, greedy acceptance and KV compaction
against the integer oracle: bit-exact."""
import json
import os

import numpy as np
import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import _lib, eagle, ops, synth
from mlx_eagle_spec_decoding_tree_amd.cache import KVCache
from oracle import tree_oracle as to
from test_oracle_tree import simulate_draft
from util import to_dev

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def dev_process(dev, scores, tokens, parents_list, root, k, V):
    return eagle.process_draft_tree_device(
        to_dev(scores, dev), to_dev(tokens, dev), to_dev(parents_list.view(np.int32), dev),
        torch.tensor([root], dtype=torch.int32, device=dev), k, V)


@pytest.mark.parametrize("depth", [0, 1, 3, 5])
@pytest.mark.parametrize("V", [7, 15, 23, 31])
def test_process_and_post_process_bit_exact(dev, depth, V):
    rng = np.random.default_rng(depth * 37 + V)
    for trial in range(12):
        scores, tokens, parents_list, _ = simulate_draft(rng, depth, tie_levels=(4 if trial % 2 else None))
        if V > scores.size:
            pytest.skip("fewer candidates than requested nodes")
        pos_w, midx_w, toks_w, anc_w = to.process_draft_tree(scores, tokens, parents_list, np.array([[9]]), 8, V)
        pos, midx, toks, bits = dev_process(dev, scores, tokens, parents_list, 9, 8, V)
        assert np.array_equal(pos.cpu().numpy(), pos_w)
        assert np.array_equal(midx.cpu().numpy(), midx_w)
        assert np.array_equal(toks.cpu().numpy(), toks_w[0])
        assert np.array_equal(bits.cpu().numpy().view(np.uint32), to.mask_bits(anc_w))
        ri_w = to.post_process_draft_tree(pos_w, V, midx_w)
        ri = eagle.post_process_draft_tree(pos, V, midx).cpu().numpy()
        assert ri.shape == ri_w.shape and np.array_equal(ri, ri_w)


@pytest.mark.parametrize("n_nan", [1, 33, 150, 200])
def test_nan_scores_leave_a_well_formed_tree(dev, n_nan):
    """More NaN scores than tree slots: the device picks exactly V candidates (NaN ranks as
    -inf, ties by index) and equals the oracle bit for bit; nothing outside the outputs is
    written (the tokens after the tree and a second call on clean scores are intact)."""
    rng = np.random.default_rng(n_nan)
    V = 31
    scores, tokens, parents_list, _ = simulate_draft(rng, 3)
    clean = scores.copy()
    bad = rng.choice(scores.size, size=min(n_nan, scores.size), replace=False)
    scores[bad] = np.nan
    for sc in (scores, clean):
        pos_w, midx_w, toks_w, anc_w = to.process_draft_tree(sc, tokens, parents_list, np.array([[9]]), 8, V)
        pos, midx, toks, bits = dev_process(dev, sc, tokens, parents_list, 9, 8, V)
        assert np.array_equal(pos.cpu().numpy(), pos_w)
        assert np.array_equal(midx.cpu().numpy(), midx_w)
        assert np.array_equal(toks.cpu().numpy(), toks_w[0])
        assert np.array_equal(bits.cpu().numpy().view(np.uint32), to.mask_bits(anc_w))


@pytest.mark.parametrize("depth,V", [(5, 39), (5, 63), (3, 32), (7, 47)])
def test_trees_above_32_tokens_bit_exact(dev, depth, V):
    """Up to 64 tree slots (the reference's default is 39 nodes at depth 5, mlx_eagle.py:390,510):
    two mask words per row, 64 x 64 retrieve matrix."""
    rng = np.random.default_rng(depth * 41 + V)
    for trial in range(8):
        scores, tokens, parents_list, _ = simulate_draft(rng, depth, tie_levels=(4 if trial % 2 else None))
        pos_w, midx_w, toks_w, anc_w = to.process_draft_tree(scores, tokens, parents_list, np.array([[9]]), 8, V)
        pos, midx, toks, bits = dev_process(dev, scores, tokens, parents_list, 9, 8, V)
        assert tuple(bits.shape) == (V + 1, 2)
        assert np.array_equal(pos.cpu().numpy(), pos_w)
        assert np.array_equal(midx.cpu().numpy(), midx_w)
        assert np.array_equal(toks.cpu().numpy(), toks_w[0])
        assert np.array_equal(bits.cpu().numpy().view(np.uint32), to.mask_bits(anc_w))
        assert np.array_equal(eagle.bits_to_mask(bits).float().cpu().numpy() == 0, anc_w)
        ri_w = to.post_process_draft_tree(pos_w, V, midx_w)
        ri = eagle.post_process_draft_tree(pos, V, midx).cpu().numpy()
        assert ri.shape == ri_w.shape and np.array_equal(ri, ri_w)


def test_reference_signature_process_draft_tree(dev):
    """List-of-levels inputs and the (position_ids, mask_index, draft_tokens[1,T], bf16 mask) tuple."""
    rng = np.random.default_rng(5)
    depth, k, V = 3, 8, 31
    scores, tokens, parents_list, _ = simulate_draft(rng, depth)
    sl = [to_dev(scores[:8], dev).reshape(1, 1, 8)] + [to_dev(scores[8 + 64 * i: 72 + 64 * i], dev).reshape(1, 8, 8) for i in range(depth)]
    tl = [to_dev(tokens[:8], dev).reshape(1, 1, 8)] + [to_dev(tokens[8 + 64 * i: 72 + 64 * i], dev).reshape(1, 8, 8) for i in range(depth)]
    pl = [to_dev(parents_list[:1].view(np.int32), dev)] + [to_dev(parents_list[1 + 8 * i: 9 + 8 * i].view(np.int32), dev) for i in range(depth)]
    pos, midx, toks, mask = eagle.process_draft_tree(sl, tl, pl, torch.tensor([[4]], device=dev), k, V)
    pos_w, midx_w, toks_w, anc_w = to.process_draft_tree(scores, tokens, parents_list, np.array([[4]]), k, V)
    assert tuple(toks.shape) == (1, V + 1) and mask.dtype == torch.bfloat16 and tuple(mask.shape) == (V + 1, V + 1)
    assert np.array_equal(pos.cpu().numpy(), pos_w) and np.array_equal(midx.cpu().numpy(), midx_w)
    assert np.array_equal((mask.float().cpu().numpy() == 0), anc_w)
    assert np.array_equal(np.isneginf(mask.float().cpu().numpy()), ~anc_w)


def test_reference_fixture_on_device(dev):
    fx = json.load(open(os.path.join(HERE, "golden", "tree_fixture.json")))
    pos = torch.tensor(fx["tree_position_ids"], dtype=torch.int32, device=dev)
    midx = torch.tensor(fx["mask_index"], dtype=torch.int32, device=dev)
    ri = eagle.post_process_draft_tree(pos, fx["total_tokens"], midx)
    assert ri.cpu().tolist() == fx["retrieve_indices"]
    T, V = 8, 40000
    tokens = torch.arange(100, 100 + T, dtype=torch.int32, device=dev)
    path = fx["retrieve_indices"][fx["correct_draft_index"]]
    logits = torch.full((T, V), -1.0, dtype=torch.float16, device=dev)
    for a, b in zip(path[:-1], path[1:]):
        logits[a, 100 + b] = 1.0
    logits[path[-1], 33894] = 1.0
    cand = tokens[ri.long()]                       # -1 wraps to the last node as in the reference
    best, al, row = eagle.evaluate_posterior_greedy(logits[ri.long()], cand)
    assert int(al) == fx["expected_accept_length"] and int(best) == fx["expected_best_candidate"]
    assert int(ops.argmax_rows(row[None])[0]) == 33894


def test_greedy_accept_kernel_bit_exact(dev):
    rng = np.random.default_rng(21)
    L = _lib.lib()
    for trial in range(150):
        T = int(rng.integers(2, 65))
        parents = synth.random_tree(rng, T, max_depth=6 if T > 32 else 4, max_children=6 if T > 32 else 4)
        depth, anc = to.tree_from_parents(parents)
        ri_w = to.post_process_draft_tree(depth, T - 1, parents)
        tokens = rng.integers(0, 5, T).astype(np.int32)
        am = rng.integers(0, 5, T).astype(np.int32)
        best, al, bonus = to.greedy_accept(am, tokens, ri_w)
        full, shape = eagle.post_process_draft_tree_device(to_dev(depth, dev), T - 1, to_dev(parents, dev))
        result = torch.zeros(68, dtype=torch.int32, device=dev)
        acc_t = torch.zeros(64, dtype=torch.int32, device=dev)
        am_d, tok_d = to_dev(am, dev), to_dev(tokens, dev)
        rc = L.eagle_greedy_accept(am_d.data_ptr(), tok_d.data_ptr(), full.data_ptr(),
                                   shape.data_ptr(), T, result.data_ptr(), acc_t.data_ptr(), None)
        assert rc == 0
        torch.cuda.synchronize()
        r = result.cpu().numpy()
        assert (r[0], r[1], r[2], r[3]) == (best, al, bonus, am[bonus])
        assert np.array_equal(r[4:4 + al], ri_w[best, 1:1 + al])
        assert np.array_equal(acc_t.cpu().numpy()[:al], tokens[ri_w[best, 1:1 + al] % T])


def test_padding_quirk_on_device(dev):
    L = _lib.lib()
    ri = np.full((64, 64), -1, np.int32)
    ri[0, :5] = [0, 1, 2, 4, 6]
    ri[1, :6] = [0, 1, 2, 3, 5, 7]
    tokens = np.arange(8, dtype=np.int32)
    am = np.array([1, 2, 4, 9, 6, 9, 7, 9], np.int32)
    result = torch.zeros(68, dtype=torch.int32, device=dev)
    acc_t = torch.zeros(64, dtype=torch.int32, device=dev)
    shape = torch.tensor([2, 6], dtype=torch.int32, device=dev)
    am_d, tok_d, ri_d = to_dev(am, dev), to_dev(tokens, dev), to_dev(ri, dev)
    rc = L.eagle_greedy_accept(am_d.data_ptr(), tok_d.data_ptr(), ri_d.data_ptr(),
                               shape.data_ptr(), 8, result.data_ptr(), acc_t.data_ptr(), None)
    assert rc == 0
    r = result.cpu().numpy()
    assert tuple(r[:3]) == (0, 5, 7) and list(r[4:9]) == [1, 2, 4, 6, -1]
    assert list(acc_t.cpu().numpy()[:5]) == [1, 2, 4, 6, 7]


@pytest.mark.parametrize("idx", [[1, 2, 3], [2, 5, 9], [3], [1, 4], [-1, 5], [], list(range(1, 32))])
def test_accept_candidate_matches_oracle(dev, idx):
    rng = np.random.default_rng(len(idx))
    G, cap, hd, P, layers = 2, 96, 64, 20, 3
    caches, refs = [], []
    for _ in range(layers):
        c = KVCache(G, hd, cap, dev)
        k = rng.normal(size=(G, cap, hd)).astype(np.float16)
        v = rng.normal(size=(G, cap, hd)).astype(np.float16)
        c.keys[0].copy_(to_dev(k, dev)); c.values[0].copy_(to_dev(v, dev))
        c.offset = P + 32
        caches.append(c); refs.append((k.copy(), v.copy()))
    eagle.accept_candidate(caches, torch.tensor(idx, dtype=torch.int32, device=dev), len(idx), P)
    for c, (k, v) in zip(caches, refs):
        new = to.accept_candidate(k, v, np.array(idx, int), len(idx), P)
        assert c.offset == new
        assert np.array_equal(c.keys[0].cpu().numpy().view(np.uint16), k.view(np.uint16))
        assert np.array_equal(c.values[0].cpu().numpy().view(np.uint16), v.view(np.uint16))


def test_topk_and_search_sorted_mirror(dev):
    x = torch.tensor([1.0, 3.0, 3.0, 2.0, 3.0], dtype=torch.float16, device=dev)
    idx, vals = eagle.topk(x, 3)
    assert idx.tolist() == [1, 2, 4] and vals.tolist() == [3.0, 3.0, 3.0]
    rng = np.random.default_rng(0)
    for n in (7, 15, 23, 31):
        arr = np.sort(rng.choice(200, n, replace=False)).astype(np.int64)
        tgt = rng.choice(arr, 12)
        got = eagle.search_sorted(torch.from_numpy(arr).to(dev), torch.from_numpy(tgt).to(dev))
        assert np.array_equal(got.cpu().numpy(), to.search_sorted(arr, tgt))
