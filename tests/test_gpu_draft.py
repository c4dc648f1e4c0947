"""Draft-side tree expansion on the GPU against oracle/draft_oracle.py (mlx_eagle.py:97-213,
379-463, 503-606).  Float stages within the stated tolerances; every integer stage bit-exact on
identical inputs."""
import numpy as np
import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import eagle, llama, ops, synth
from mlx_eagle_spec_decoding_tree_amd.cache import make_prompt_cache
from oracle import draft_oracle, oracle, tree_oracle
from util import MODEL_TOL, TOL, rel_err, to_dev

pytestmark = pytest.mark.gpu

ULP = 2.0 ** -7          # fp16 spacing of log-probabilities in [-16, -8)


def check_topk(logits, k, mode, idx, sc):
    """GPU (idx, sc) against the oracle: the scores agree to two fp16 ulps, the order is
    descending with ties by index, and where the oracle's ranking has a clear margin (to the
    neighbours inside the selection and to the best entry outside it) the indices are equal."""
    R, V = logits.shape
    oidx, osc = draft_oracle.logsoftmax_topk(logits, k, mode)
    x = logits.astype(np.float64)
    lse = np.log(np.exp(x - x.max(1, keepdims=True)).sum(1, keepdims=True)) + x.max(1, keepdims=True)
    exact = x - lse
    for r in range(R):
        assert len(set(idx[r])) == k and idx[r].min() >= 0 and idx[r].max() < V
        got = sc[r].astype(np.float64)
        assert np.all(np.abs(got - exact[r][idx[r]]) <= 2.5 * ULP * np.maximum(1, np.abs(got) / 8))
        assert np.all(np.diff(got) <= 0)
        for a in range(k - 1):
            if sc[r, a] == sc[r, a + 1] and mode == 1:
                assert idx[r, a] < idx[r, a + 1]
        rest = np.delete(exact[r], idx[r])
        assert rest.max() <= exact[r][idx[r]].min() + 4 * ULP
        order = np.argsort(-exact[r], kind="stable")
        gaps = -np.diff(exact[r][order[:k + 1]])
        if gaps.min() > 6 * ULP:
            assert list(idx[r]) == list(oidx[r]) == list(order[:k])
            assert np.all(np.abs(got - osc[r].astype(np.float64)) <= 2 * ULP)


@pytest.mark.parametrize("R,V,k", [(8, 152064, 8), (1, 152064, 8), (8, 128256, 8), (8, 1000, 8),
                                   (5, 4097, 4), (3, 12, 8), (32, 5000, 1)])
@pytest.mark.parametrize("mode", [0, 1])
def test_logsoftmax_topk(dev, R, V, k, mode):
    print(f"topk R={R} V={V} k={k} mode={mode}", flush=True)
    rng = np.random.default_rng(R + V + k + mode)
    logits = rng.normal(0, 2.0, (R, V)).astype(np.float16)
    idx, sc = ops.logsoftmax_topk(to_dev(logits, dev), k, mode)
    check_topk(logits, k, mode, idx.cpu().numpy(), sc.cpu().numpy())


def test_logsoftmax_topk_row_index_and_ties(dev):
    rng = np.random.default_rng(3)
    V, k = 9000, 8
    logits = rng.normal(0, 1.0, (8, V)).astype(np.float16)
    # exact ties among the largest logits, on both sides of a chunk boundary
    logits[2, [4090, 4100, 17, 8999]] = np.float16(7.0)
    logits[2, [5, 4095, 4096]] = np.float16(6.5)
    d = to_dev(logits, dev)
    rows = torch.tensor([2, 5], dtype=torch.int32, device=dev)
    for mode in (0, 1):
        idx, sc = ops.logsoftmax_topk(d, k, mode, row_index=rows)
        idx, sc = idx.cpu().numpy(), sc.cpu().numpy()
        assert list(idx[0][:7]) == [17, 4090, 4100, 8999, 5, 4095, 4096]
        check_topk(logits[[2, 5]], k, mode, idx, sc)
        full_i, full_s = ops.logsoftmax_topk(d, k, mode)
        assert np.array_equal(full_i.cpu().numpy()[[2, 5]], idx)
        assert np.array_equal(full_s.cpu().numpy()[[2, 5]], sc)


@pytest.mark.parametrize("k,depth", [(8, 1), (8, 3), (8, 5), (8, 8), (4, 6), (2, 3)])
def test_draft_tree_levels_bit_exact(dev, k, depth):
    """init + every level on the device against the oracle's bookkeeping on the same per-level
    top-k (coarse scores, so exact ties are frequent)."""
    rng = np.random.default_rng(10 * k + depth)
    t0 = rng.integers(0, 50000, k).astype(np.int32)
    p0 = (-np.sort(rng.integers(1, 40, k)) / 8).astype(np.float16)
    b = eagle._level_buffers(k, depth, dev)
    eagle.draft_tree_init(to_dev(t0, dev), to_dev(p0, dev), k, b)
    # oracle state
    cur_ids, cur = t0.copy(), p0.copy()
    parents = [np.zeros(1, np.uint32), np.arange(k, dtype=np.uint32) + 1]
    tokens, scores = [t0], [p0]
    mask = np.zeros((k, k * depth), bool)
    mask[:, :k] = np.eye(k, dtype=bool)
    for i in range(depth):
        tidx = rng.integers(0, 50000, (k, k)).astype(np.int32)
        tsc = (-np.sort(rng.integers(1, 40, (k, k)), axis=1) / 8).astype(np.float16)
        got_mask = b["mask_words"].cpu().numpy().view(np.uint32).astype(np.uint64)
        got_bits = got_mask[:, 0] | (got_mask[:, 1] << np.uint64(32))
        want_bits = (mask.astype(np.uint64) << np.arange(k * depth, dtype=np.uint64)[None]).sum(1)
        assert np.array_equal(got_bits, want_bits), i
        assert np.array_equal(b["cur_ids"].cpu().numpy(), cur_ids)
        assert np.array_equal(b["cur_scores"].cpu().numpy(), cur)
        eagle.draft_tree_level(to_dev(tidx, dev), to_dev(tsc, dev), i, k, depth, b)
        cur_ids, cur, out_ids, cu, cs = draft_oracle.tree_level(tidx, tsc, cur, k)
        tokens.append(tidx.reshape(-1)); scores.append(cu.reshape(-1))
        if i + 1 < depth:
            parents.append((cs + (1 + k * k * i + k)).astype(np.uint32))
            mask = mask[out_ids]
            mask[:, k * (i + 1): k * (i + 2)] = np.eye(k, dtype=bool)
        assert np.array_equal(b["out_ids"].cpu().numpy(), out_ids)
        assert np.array_equal(b["topk_cs_index"].cpu().numpy(), cs)
    assert np.array_equal(b["parents"].cpu().numpy().view(np.uint32), np.concatenate(parents))
    assert np.array_equal(b["saved_tokens"].cpu().numpy(), np.concatenate(tokens))
    assert np.array_equal(b["saved_scores"].cpu().numpy(), np.concatenate(scores))


@pytest.mark.parametrize("H,G,hd,P,T,Tk", [(14, 2, 64, 512, 8, 8), (14, 2, 64, 515, 8, 24),
                                           (14, 2, 64, 100, 8, 40), (14, 2, 64, 7, 8, 64),
                                           (32, 8, 128, 1000, 8, 33), (4, 2, 64, 0, 8, 16),
                                           (28, 4, 128, 2048, 32, 32), (8, 8, 128, 31, 5, 64)])
def test_draft_attention(dev, H, G, hd, P, T, Tk):
    """T queries, Tk masked rows after the prefix, random visibility (own row always visible)."""
    print(f"draft attn H={H} G={G} hd={hd} P={P} T={T} Tk={Tk}", flush=True)
    rng = np.random.default_rng(H + P + T + Tk)
    cap = P + Tk + 9
    q = synth.make_x(rng, H, T, hd)
    k = synth.make_x(rng, G, cap, hd)
    v = synth.make_x(rng, G, cap, hd)
    k[:, P + Tk:] = np.nan
    v[:, P + Tk:] = np.nan
    vis = rng.random((T, Tk)) < 0.4
    vis[np.arange(T), Tk - T + np.arange(T)] = True
    if P == 0:
        vis[:, 0] = True
    mask = np.concatenate([np.zeros((T, P), np.float16),
                           np.where(vis, np.float16(0), np.float16(-np.inf))], axis=1)
    scale = hd ** -0.5
    want = oracle.tree_attention(q, k, v, mask, scale, S=P + Tk)
    want_t = np.ascontiguousarray(want.transpose(1, 0, 2)).reshape(T, H * hd)
    words = ops.mask_to_words(to_dev(vis, dev))
    len_dev = torch.tensor([P], dtype=torch.int32, device=dev)
    for max_len in (P + Tk, cap):
        got = ops.draft_attention(to_dev(q, dev), to_dev(k, dev), to_dev(v, dev), words, len_dev, Tk,
                                  scale, max_len=max_len).cpu().numpy()
        assert np.isfinite(got.astype(np.float32)).all()
        assert rel_err(got, want_t) <= TOL
    if T == Tk and Tk <= 32:
        # the one-word form gives the same bits
        one = ops.tree_attention(to_dev(q, dev), to_dev(k, dev), to_dev(v, dev),
                                 words[:, 0].contiguous(), len_dev, scale, max_len=cap).cpu().numpy()
        assert np.array_equal(one, got)


def tiny_pair(dev, same, seed=0, vocab=1024, **kw):
    targs = synth.tiny(layers=2, hidden=256, inter=512, heads=4, kv_heads=2, head_dim=64, vocab=vocab, **kw)
    tw = synth.make_model_weights(targs, seed=seed)
    if same:
        dargs, dw = targs, tw
    else:
        dargs = synth.tiny(layers=1, hidden=128, inter=256, heads=2, kv_heads=1, head_dim=64, vocab=vocab)
        dw = synth.make_model_weights(dargs, seed=seed + 7)
    return (targs, tw, llama.Model.from_numpy(targs, tw, dev)), (dargs, dw, llama.Model.from_numpy(dargs, dw, dev))


def test_causal_pass_matches_oracle(dev):
    """mask=None: causal over the new tokens, chunked above 32 (the prompt pass)."""
    (args, w, model), _ = tiny_pair(dev, same=True)
    rng = np.random.default_rng(4)
    ids = rng.integers(0, args.vocab_size, 75).astype(np.int32)
    inv, sc = synth.inv_freqs(args)
    side = draft_oracle.Side(args, w, inv, sc, 128)
    want = side.causal(ids[:70])
    want2 = side.causal(ids[70:])
    cache = make_prompt_cache(model, capacity=128)
    got = model(to_dev(ids[:70].astype(np.int64), dev)[None], cache=cache)[0].cpu().numpy()
    assert cache[0].offset == 70
    got2 = model(to_dev(ids[70:].astype(np.int64), dev)[None], cache=cache)[0].cpu().numpy()
    assert got.shape == want.shape and got2.shape == want2.shape
    assert rel_err(got, want) <= MODEL_TOL and rel_err(got2, want2) <= MODEL_TOL
    assert np.mean(got.argmax(-1) == want.argmax(-1)) > 0.9


@pytest.mark.parametrize("depth", [3, 5])
def test_generate_draft_tree_matches_oracle(dev, depth):
    k = 8
    (args, w, model), _ = tiny_pair(dev, same=True, seed=2)
    rng = np.random.default_rng(depth)
    P = 45
    ids = rng.integers(0, args.vocab_size, P).astype(np.int32)
    inv, sc = synth.inv_freqs(args)
    side = draft_oracle.Side(args, w, inv, sc, 160)
    lg = side.causal(ids)
    cache = make_prompt_cache(model, capacity=160)
    glg = model(to_dev(ids.astype(np.int64), dev)[None], cache=cache)[0]
    t0, p0 = ops.logsoftmax_topk(glg[-1:].contiguous(), k, 0)
    check_topk(lg[-1:], k, 0, t0.cpu().numpy(), p0.cpu().numpy())
    parents_list, toks_list, scores_list = eagle.generate_draft_tree(t0, p0[..., None], model, cache,
                                                                    depth=depth, k=k)
    assert cache[0].offset == P + k * depth
    assert [tuple(t.shape) for t in parents_list] == [(1,)] + [(k,)] * depth
    assert [tuple(t.shape) for t in toks_list] == [(1, 1, k)] + [(1, k, k)] * depth
    assert [tuple(t.shape) for t in scores_list] == [(1, 1, k)] + [(1, k, k)] * depth
    forced = [(toks_list[i + 1].cpu().numpy(), scores_list[i + 1].cpu().numpy()) for i in range(depth)]
    trace = []
    parents, tokens, scores = draft_oracle.generate_draft_tree(
        args, w, inv, sc, t0.cpu().numpy()[0], p0.cpu().numpy()[0], side.cache, P, depth, k,
        trace=trace, forced=forced)
    # integer bookkeeping: bit-exact on the same per-level float results
    assert np.array_equal(torch.cat([p.flatten() for p in parents_list]).cpu().numpy().astype(np.uint32), parents)
    assert np.array_equal(torch.cat([t.flatten() for t in toks_list]).cpu().numpy(), tokens)
    assert np.array_equal(torch.cat([s.flatten() for s in scores_list]).cpu().numpy(), scores)
    # float stage: the oracle's own per-level results under the same selections
    for i, tr in enumerate(trace):
        cu_oracle = (tr["topk_score"].astype(np.float32) + tr["cur_scores"].astype(np.float32)[:, None])
        got_cu = forced[i][1].reshape(k, k).astype(np.float32)
        same = forced[i][0].reshape(k, k) == tr["topk_index"]
        assert same.mean() > 0.8, i
        assert np.all(np.abs(got_cu - cu_oracle)[same] <= 0.05 + 8 * ULP * i), i
    # the KV rows the expansion wrote
    for (ok, ov), c in zip(side.cache, cache):
        assert rel_err(c.keys[0, :, :P + k * depth].cpu().numpy(), ok[:, :P + k * depth]) <= MODEL_TOL
        assert rel_err(c.values[0, :, :P + k * depth].cpu().numpy(), ov[:, :P + k * depth]) <= MODEL_TOL


def assert_greedy_stream(model, prompt, stream, dev, tol=0.06):
    """Every token of `stream` is the target's argmax given the prompt and the tokens before it,
    up to `tol` in logit units: the verification pass and a one-token pass round differently, so
    at a near-tie they may pick different maxima (then both are valid greedy streams)."""
    cache = make_prompt_cache(model, capacity=len(prompt) + len(stream) + 8)
    logits = model(to_dev(prompt.astype(np.int64), dev)[None], cache=cache)[0, -1].float()
    exact = 0
    for i, tok in enumerate(stream):
        deficit = float(logits.max() - logits[tok])
        assert deficit <= tol, (i, tok, int(logits.argmax()), deficit)
        exact += int(logits.argmax()) == tok
        logits = model(torch.tensor([[tok]], dtype=torch.int64, device=dev), cache=cache)[0, -1].float()
    assert exact >= len(stream) - 2      # near-ties are rare
    return exact


@pytest.mark.parametrize("same", [True, False])
def test_generate_step_stream_equals_target_greedy(dev, same):
    """Whatever the drafter proposes, the emitted stream is the target's own greedy stream; with
    the target as its own drafter nearly every level is accepted."""
    (targs, tw, target), (dargs, dw, draft) = tiny_pair(dev, same=same, seed=5)
    rng = np.random.default_rng(8)
    prompt = rng.integers(0, targs.vocab_size, 40).astype(np.int32)
    res = eagle.generate_step(to_dev(prompt.astype(np.int64), dev), target, draft, k=8, depth=3,
                              verify_num_tokens=31, max_tokens=64, N=6)
    n = res["n"]
    assert n == len(res["tokens"]) == sum(1 + s[0] for s in res["steps"])
    assert_greedy_stream(target, prompt, [res["first"]] + res["tokens"], dev)
    if same:
        assert res["mean_tokens_per_step"] >= 3.0
    for al, best, acc, y in res["steps"]:
        assert len(acc) == al and len(y) == al + 1


def test_generate_step_with_the_reference_default_tree(dev):
    """depth 5, 39 draft nodes (the reference's defaults, mlx_eagle.py:509-510): a tree of 40 tokens
    on the module path (tiled GEMMs for 40 rows, attention in two pieces of query rows inside one
    launch pair); the emitted stream is the target's greedy stream."""
    (targs, tw, target), (dargs, dw, draft) = tiny_pair(dev, same=True, seed=6)
    rng = np.random.default_rng(9)
    prompt = rng.integers(0, targs.vocab_size, 40).astype(np.int32)
    res = eagle.generate_step(to_dev(prompt.astype(np.int64), dev), target, draft, max_tokens=48, N=5)
    assert res["n"] == len(res["tokens"]) == sum(1 + s[0] for s in res["steps"])
    assert_greedy_stream(target, prompt, [res["first"]] + res["tokens"], dev)
    assert res["mean_tokens_per_step"] >= 3.0
    with pytest.raises(NotImplementedError):
        eagle.generate_step(to_dev(prompt.astype(np.int64), dev), target, draft, verify_num_tokens=64)
    with pytest.raises(NotImplementedError):
        eagle.TreeVerifier(target, make_prompt_cache(target, capacity=128), total_tokens=64)


def test_generate_step_matches_oracle_loop(dev):
    (targs, tw, target), (dargs, dw, draft) = tiny_pair(dev, same=False, seed=11)
    rng = np.random.default_rng(12)
    prompt = rng.integers(0, targs.vocab_size, 36).astype(np.int32)
    k, depth, V, N = 8, 3, 31, 3
    res = eagle.generate_step(to_dev(prompt.astype(np.int64), dev), target, draft, k=k, depth=depth,
                              verify_num_tokens=V, max_tokens=64, N=N)
    ti, ts = synth.inv_freqs(targs)
    di, ds = synth.inv_freqs(dargs)
    base = draft_oracle.Side(targs, tw, ti, ts, 200)
    dr = draft_oracle.Side(dargs, dw, di, ds, 200)
    want = draft_oracle.generate(base, dr, prompt, k, depth, V, 64, N)
    assert res["first"] == want["first"]
    assert res["tokens"] == want["tokens"]
    assert [s[0] for s in res["steps"]] == [s[0] for s in want["steps"]]


@pytest.mark.parametrize("same", [True, False])
@pytest.mark.parametrize("graph", [False, True])
def test_device_loop_equals_host_loop(dev, same, graph):
    """SpeculativeDecoder (state on the device, optionally one HIP graph per step) emits the
    stream of the host-driven generate_step, which is the target's greedy stream."""
    from mlx_eagle_spec_decoding_tree_amd import spec

    print(f"device loop same={same} graph={graph}", flush=True)
    (targs, tw, target), (dargs, dw, draft) = tiny_pair(dev, same=same, seed=5)
    rng = np.random.default_rng(8)
    prompt = rng.integers(0, targs.vocab_size, 40).astype(np.int32)
    N = 6
    host = eagle.generate_step(to_dev(prompt.astype(np.int64), dev), target, draft, k=8, depth=3,
                               verify_num_tokens=31, max_tokens=10 ** 6, N=N)
    # fresh models: the fused passes re-point the layers' tensors
    (_, _, target2), (_, _, draft2) = tiny_pair(dev, same=same, seed=5)
    dec = spec.SpeculativeDecoder(target2, draft2, capacity=256, k=8, depth=3, verify_num_tokens=31)
    first = dec.prefill(to_dev(prompt.astype(np.int64), dev))
    if graph:
        dec.capture()
    tokens = dec.generate(N)
    assert first == host["first"]
    assert_greedy_stream(target, prompt, [first] + tokens, dev)
    if tokens != host["tokens"]:          # only possible after a near-tie: then both are greedy streams
        assert_greedy_stream(target, prompt, [host["first"]] + host["tokens"], dev)
    assert int(dec.verifier.len_dev.item()) == len(prompt) + len(tokens)
    if same:
        assert len(tokens) >= 3 * N
    # a second run continues the stream
    more = dec.generate(2)
    assert more[:len(tokens)] == tokens and len(more) > len(tokens)
    assert_greedy_stream(target, prompt, [first] + more, dev)
    # a new prompt starts from empty caches, with the graphs already captured
    prompt2 = rng.integers(0, targs.vocab_size, 33).astype(np.int32)
    first2 = dec.prefill(to_dev(prompt2.astype(np.int64), dev))
    tokens2 = dec.generate(3)
    assert_greedy_stream(target, prompt2, [first2] + tokens2, dev)


def test_device_loop_refuses_to_overrun_the_caches(dev):
    from mlx_eagle_spec_decoding_tree_amd import spec

    (targs, tw, target), (dargs, dw, draft) = tiny_pair(dev, same=False, seed=5)
    prompt = np.random.default_rng(1).integers(0, targs.vocab_size, 40).astype(np.int64)
    dec = spec.SpeculativeDecoder(target, draft, capacity=128, k=8, depth=3, verify_num_tokens=31)
    dec.prefill(to_dev(prompt, dev))
    dec.generate(5)                       # 40 + 5 * 5 + 32 <= 128
    with pytest.raises(ValueError, match="too small"):
        dec.generate(10)
    with pytest.raises(ValueError):
        spec.SpeculativeDecoder(target, draft, capacity=128, k=8, depth=9)
    with pytest.raises(ValueError):
        spec.SpeculativeDecoder(target, draft, capacity=128, k=8, depth=3, verify_num_tokens=64)


@pytest.mark.parametrize("n,chunk,graphs", [(75, 512, True), (200, 64, False), (32, 512, True),
                                            (1100, 2048, True), (1300, 1024, False)])
def test_chunked_prompt_pass_matches_oracle(dev, n, chunk, graphs):
    """spec.CausalPrefill: linear layers over the whole chunk (tiled GEMM form above 32 rows),
    attention per 32-row piece; cache rows and the last token's logits against the oracle."""
    from mlx_eagle_spec_decoding_tree_amd import spec

    (args, w, model), _ = tiny_pair(dev, same=True, seed=3)
    rng = np.random.default_rng(n)
    ids = rng.integers(0, args.vocab_size, n).astype(np.int32)
    inv, sc = synth.inv_freqs(args)
    cap = max(320, n + 120)
    side = draft_oracle.Side(args, w, inv, sc, cap)
    want = side.causal(ids)
    cache = make_prompt_cache(model, capacity=cap)
    pre = spec.CausalPrefill(model, cache, head=True, chunk=chunk, graphs=graphs)
    got = pre(to_dev(ids, dev)).cpu().numpy()
    assert cache[0].offset == n and int(cache[0].len_dev.item()) == n
    assert got.shape == (1, args.vocab_size)
    assert rel_err(got, want[-1:]) <= MODEL_TOL
    assert got.argmax() == want[-1].argmax() or np.sort(want[-1])[-1] - np.sort(want[-1])[-2] < 0.05
    for (ok, ov), c in zip(side.cache, cache):
        assert rel_err(c.keys[0, :, :n].cpu().numpy(), ok[:, :n]) <= MODEL_TOL
        assert rel_err(c.values[0, :, :n].cpu().numpy(), ov[:, :n]) <= MODEL_TOL
    # a second call continues from the cache
    more = rng.integers(0, args.vocab_size, 40).astype(np.int32)
    want2 = side.causal(more)
    got2 = pre(to_dev(more, dev)).cpu().numpy()
    assert cache[0].offset == n + 40
    assert rel_err(got2, want2[-1:]) <= MODEL_TOL


def test_device_loop_depth_five(dev):
    """Depth 5: 40 expansion rows, so the draft attention uses both mask words."""
    from mlx_eagle_spec_decoding_tree_amd import spec

    (targs, tw, target), (dargs, dw, draft) = tiny_pair(dev, same=True, seed=21)
    rng = np.random.default_rng(22)
    prompt = rng.integers(0, targs.vocab_size, 50).astype(np.int32)
    dec = spec.SpeculativeDecoder(target, draft, capacity=256, k=8, depth=5, verify_num_tokens=31)
    first = dec.prefill(to_dev(prompt.astype(np.int64), dev))
    dec.capture()
    tokens = dec.generate(5)
    (_, _, ref), _ = tiny_pair(dev, same=True, seed=21)
    assert_greedy_stream(ref, prompt, [first] + tokens, dev)
    assert len(tokens) >= 3 * 5                       # two drafted tokens and the bonus per step


def test_draft_attention_random_shapes(dev):
    """Seeded sweep over query counts, masked-row counts, prefix lengths and head layouts."""
    rng = np.random.default_rng(2024)
    for case in range(24):
        hd = int(rng.choice([64, 128]))
        G = int(rng.choice([1, 2, 4, 8]))
        rep = int(rng.choice([1, 2, 4, 7, 8]))
        H = G * rep
        T = int(rng.integers(1, 33))
        Tk = int(rng.integers(T, 65))
        P = int(rng.choice([0, 1, 31, 32, 33, 63, 64, 65, 200, 517]))
        cap = P + Tk + int(rng.integers(0, 40))
        print(f"case {case}: H={H} G={G} hd={hd} T={T} Tk={Tk} P={P} cap={cap}", flush=True)
        q = synth.make_x(rng, H, T, hd)
        k = synth.make_x(rng, G, cap, hd)
        v = synth.make_x(rng, G, cap, hd)
        k[:, P + Tk:] = np.nan
        v[:, P + Tk:] = np.nan
        vis = rng.random((T, Tk)) < 0.5
        vis[np.arange(T), Tk - T + np.arange(T)] = True
        mask = np.concatenate([np.zeros((T, P), np.float16),
                               np.where(vis, np.float16(0), np.float16(-np.inf))], axis=1)
        want = oracle.tree_attention(q, k, v, mask, hd ** -0.5, S=P + Tk)
        want_t = np.ascontiguousarray(want.transpose(1, 0, 2)).reshape(T, H * hd)
        got = ops.draft_attention(to_dev(q, dev), to_dev(k, dev), to_dev(v, dev),
                                  ops.mask_to_words(to_dev(vis, dev)),
                                  torch.tensor([P], dtype=torch.int32, device=dev), Tk, hd ** -0.5,
                                  max_len=cap).cpu().numpy()
        assert np.isfinite(got.astype(np.float32)).all(), case
        assert rel_err(got, want_t) <= TOL, case


def test_causal_attention_pieces(dev):
    """All 32-row pieces of a chunk in one launch pair against per-piece causal attention."""
    rng = np.random.default_rng(77)
    for (H, G, hd, P, R) in ((4, 2, 64, 0, 64), (14, 2, 64, 100, 96), (32, 8, 128, 37, 160), (8, 8, 128, 500, 32)):
        print(f"chunk attention H={H} G={G} hd={hd} P={P} R={R}", flush=True)
        cap = P + R + 5
        q = synth.make_x(rng, H, R, hd)
        k = synth.make_x(rng, G, cap, hd)
        v = synth.make_x(rng, G, cap, hd)
        k[:, P + R:] = np.nan
        v[:, P + R:] = np.nan
        mask = np.zeros((R, P + R), np.float16)
        mask[:, P:] = np.where(np.tril(np.ones((R, R), bool)), np.float16(0), np.float16(-np.inf))
        want = oracle.tree_attention(q, k, v, mask, hd ** -0.5, S=P + R)
        want_t = np.ascontiguousarray(want.transpose(1, 0, 2)).reshape(R, H * hd)
        piece_len = torch.tensor([P + 32 * j for j in range(R // 32)], dtype=torch.int32, device=dev)
        got = ops.causal_attention(to_dev(q, dev), to_dev(k, dev), to_dev(v, dev), piece_len, hd ** -0.5,
                                   max_len=cap).cpu().numpy()
        assert np.isfinite(got.astype(np.float32)).all()
        assert rel_err(got, want_t) <= TOL
