"""Trees of 33..64 tokens (the reference's default is 39 draft nodes, mlx_eagle.py:390,510) on the
fused verification step and the device loop: attention in pieces of 32 query rows inside one
launch pair, the projections as tiled GEMMs."""
import numpy as np
import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import eagle, ops, spec, synth
from mlx_eagle_spec_decoding_tree_amd.cache import make_prompt_cache
from oracle import model_oracle, oracle, tree_oracle
from test_gpu_draft import assert_greedy_stream, tiny_pair
from test_gpu_model import CONFIGS, build, margins, run_verifier
from util import MODEL_TOL, TOL, rel_err, to_dev

pytestmark = pytest.mark.gpu


def test_attention_of_up_to_64_queries(dev):
    """One launch pair for 33..64 queries: against the oracle, and bit for bit against the
    32-query form called once per piece of rows."""
    rng = np.random.default_rng(4040)
    for case in range(16):
        hd = int(rng.choice([64, 128]))
        G = int(rng.choice([1, 2, 4, 8]))
        rep = int(rng.choice([1, 2, 4, 7, 8]))
        H = G * rep
        T = int(rng.choice([33, 40, 47, 63, 64])) if case < 12 else int(rng.integers(1, 33))
        Tk = T if case % 2 == 0 else int(rng.integers(T, 65))
        P = int(rng.choice([0, 1, 31, 33, 64, 200, 517, 1030]))
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
        qd, kd, vd = to_dev(q, dev), to_dev(k, dev), to_dev(v, dev)
        words = ops.mask_to_words(to_dev(vis, dev))
        len_dev = torch.tensor([P], dtype=torch.int32, device=dev)
        got = ops.draft_attention(qd, kd, vd, words, len_dev, Tk, hd ** -0.5, max_len=cap)
        assert np.isfinite(got.float().cpu().numpy()).all(), case
        assert rel_err(got.cpu().numpy(), want_t) <= TOL, case
        for t0 in range(0, T, 32):
            t1 = min(T, t0 + 32)
            piece = ops.draft_attention(qd[:, t0:t1].contiguous(), kd, vd, words[t0:t1].contiguous(), len_dev,
                                        Tk, hd ** -0.5, max_len=cap)
            assert torch.equal(piece, got[t0:t1]), (case, t0)
        if Tk == T:
            tree = ops.tree_attention(qd, kd, vd, words, len_dev, hd ** -0.5, max_len=cap)
            assert torch.equal(tree, got), case


def test_wide_attention_refusals(dev):
    L = __import__("mlx_eagle_spec_decoding_tree_amd._lib", fromlist=["lib"]).lib()
    assert L.eagle_tree_attention_wide_workspace_bytes(65, 4, 64, 128) == 0
    assert (L.eagle_tree_attention_wide_workspace_bytes(64, 4, 64, 128)
            == 2 * L.eagle_tree_attention_workspace_bytes(4, 64, 128))
    assert (L.eagle_tree_attention_wide_workspace_bytes(32, 4, 64, 128)
            == L.eagle_tree_attention_workspace_bytes(4, 64, 128))
    q = torch.zeros((4, 65, 64), dtype=torch.float16, device=dev)
    kc = torch.zeros((2, 200, 64), dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        ops.draft_attention(q, kc, kc, torch.zeros((65, 2), dtype=torch.int32, device=dev),
                            torch.zeros(1, dtype=torch.int32, device=dev), 64, 0.125)
    with pytest.raises(ValueError):
        ops.tree_attention(q[:, :40].contiguous(), kc, kc, torch.zeros((39, 2), dtype=torch.int32, device=dev),
                           torch.zeros(1, dtype=torch.int32, device=dev), 0.125)


@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("T", [40, 64, 33])
def test_fused_step_of_a_wide_tree(dev, name, T):
    """The fused step on a tree above 32 tokens against the module path (same GEMM kernels per
    projection, so close but another launch shape for the fused ones) and against the oracle;
    integer stages bit-exact on the device's own argmax; graph replays equal the eager run."""
    P = 200
    print(f"wide step {name} T={T}", flush=True)
    s = build(dev, name, P, T, seed=3)
    s2 = build(dev, name, P, T, seed=3)
    tree_mask = to_dev(tree_oracle.additive_mask(s2["anc"]), dev).to(torch.bfloat16)
    ref_logits = eagle.tree_decoding(to_dev(s2["tokens"][None], dev), tree_mask, to_dev(s2["depth"], dev),
                                     s2["model"], s2["cache"])[0]
    ver = run_verifier(s, dev, graph=False)
    assert ver.wide and tuple(ver.mask_bits.shape) == (T, 2)
    assert ver.slab == eagle.slab_plan(s["model"], T)       # the library's choice, as for 32 tokens
    ver.step()
    torch.cuda.synchronize()
    assert rel_err(ver.logits.cpu().numpy(), ref_logits.cpu().numpy()) <= TOL
    want = model_oracle.verify_step(s["args"], s["weights"], s["inv"], s["sc"], s["tokens"], s["depth"],
                                    s["parents"], s["anc"], s["ocache"], P)
    # logits after two layers: the whole-pass bound (the errors of the layers' matmuls add up)
    assert rel_err(ver.logits.cpu().numpy(), want["logits"]) <= MODEL_TOL
    am = ver.node_argmax.cpu().numpy()
    assert np.array_equal(am, oracle.argmax_rows(ver.logits.cpu().numpy()))
    ri = tree_oracle.post_process_draft_tree(s["depth"], T - 1, s["parents"])
    best, al, bonus = tree_oracle.greedy_accept(am, s["tokens"], ri)
    r = ver.result.cpu().numpy()
    assert (r[0], r[1], r[2], r[3]) == (best, al, bonus, am[bonus])
    err = np.abs(ver.logits.cpu().numpy().astype(np.float32) - want["logits"].astype(np.float32)).max()
    if (margins(want["logits"]) > 2 * err).all():
        assert (best, al, am[bonus]) == (want["best"], want["accept_length"], want["next_token"])
    # the cache after compaction: the oracle's rows when the decisions agree
    if (best, al) == (want["best"], want["accept_length"]):
        for c, (ok, ov) in zip(s["cache"], s["ocache"]):
            assert rel_err(c.keys[0, :, P:P + al + 1].cpu().numpy(), ok[:, P:P + al + 1]) <= MODEL_TOL
            assert rel_err(c.values[0, :, P:P + al + 1].cpu().numpy(), ov[:, P:P + al + 1]) <= MODEL_TOL
    assert ver.sync_host_offsets() == P + al + 1

    # captured graph: every replay on the same inputs gives the eager bits
    s3 = build(dev, name, P, T, seed=3)
    g = run_verifier(s3, dev, graph=True)
    for rep in range(3):
        g.len_dev.fill_(P)
        g._budget.reset(P)
        g.step()
        torch.cuda.synchronize()
        assert torch.equal(g.logits, ver.logits), rep
        assert torch.equal(g.result, ver.result), rep
        torch.zeros(1 << 20, device=dev).sum().item()     # eager work between the replays


def test_wide_tree_refuses_the_32_row_options(dev):
    s = build(dev, "qwen_like", 50, 40, seed=1)
    with pytest.raises(ValueError):
        eagle.TreeVerifier(s["model"], s["cache"], total_tokens=39, fuse=False)
    with pytest.raises(NotImplementedError):
        eagle.TreeVerifier(s["model"], s["cache"], total_tokens=64)


@pytest.mark.parametrize("same", [True, False])
@pytest.mark.parametrize("graph", [False, True])
def test_device_loop_with_the_reference_default_tree(dev, same, graph):
    """k 8, depth 5, 39 draft nodes (mlx_eagle.py:509-510) with the state on the device: the
    stream of the host-driven loop, which is the target's greedy stream."""
    print(f"wide device loop same={same} graph={graph}", flush=True)
    (targs, tw, target), (dargs, dw, draft) = tiny_pair(dev, same=same, seed=6)
    rng = np.random.default_rng(9)
    prompt = rng.integers(0, targs.vocab_size, 40).astype(np.int32)
    N = 5
    host = eagle.generate_step(to_dev(prompt.astype(np.int64), dev), target, draft, max_tokens=10 ** 6, N=N)
    (_, _, target2), (_, _, draft2) = tiny_pair(dev, same=same, seed=6)
    dec = spec.SpeculativeDecoder(target2, draft2, capacity=256, k=8, depth=5, verify_num_tokens=39)
    assert dec.verifier.wide
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
    more = dec.generate(2)
    assert more[:len(tokens)] == tokens and len(more) > len(tokens)
    assert_greedy_stream(target, prompt, [first] + more, dev)
    with pytest.raises(ValueError):
        spec.SpeculativeDecoder(target2, draft2, capacity=256, k=8, depth=5, verify_num_tokens=64)
