"""Parity at the sizes the benchmark configurations name, through the C ABI:
the projection shapes of a Qwen2.5-7B-shaped model at M in {1, 8, 16, 24, 32} (streaming and slab
forms of the matmul), one decoder layer of that width over a 2048-token prefix, and the
whole 28-layer verification step with the error followed through the layers for both forms of
the matmul and both weight-rounding modes of the oracle."""
import numpy as np
import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import eagle, llama, ops, synth
from mlx_eagle_spec_decoding_tree_amd.cache import make_prompt_cache
from oracle import model_oracle, oracle, tree_oracle
from util import TOL, layer_to_dev, rel_err, to_dev

pytestmark = pytest.mark.gpu

# (name, N, K) of the second benchmark configuration
CFG2 = [("q_o", 3584, 3584), ("k_v", 512, 3584), ("gate_up", 18944, 3584), ("down", 3584, 18944),
        ("lm_head", 152064, 3584)]
ROWS = (1, 8, 16, 24, 32)


@pytest.mark.parametrize("name,N,K", CFG2)
def test_cfg2_projection_shapes(dev, name, N, K):
    """Single-matmul value distributions (scales U(0.005, 0.02), biases -8 s + noise), seed 42."""
    rng = np.random.default_rng(42)
    layer = synth.make_qlinear(rng, N, K)
    d = layer_to_dev(layer, dev)
    for M in ROWS:
        print(f"cfg2 {name} {K}->{N} M={M}", flush=True)
        x = synth.make_x(rng, M, K)
        xd = to_dev(x, dev)
        want = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"])
        got = ops.quantized_matmul(xd, d["weight"], d["scales"], d["biases"])
        torch.cuda.synchronize()
        assert rel_err(got.cpu().numpy(), want) <= TOL, f"streaming form {name} M={M}"
        s = ops.slab_steps(M, N, K)
        if s:
            part = ops.quantized_matmul_slabs(xd, d["weight"], d["scales"], d["biases"], s)
            got = ops.slab_sum(part, ops.slab_count(K, s), M, N)
            torch.cuda.synchronize()
            assert rel_err(got.cpu().numpy(), want) <= TOL, f"slab form {name} M={M}"


def setup_step(dev, args, layers, seed, P, T):
    weights = synth.make_model_weights(args, seed=seed, layers=layers)
    if layers is not None:
        args.num_hidden_layers = layers
    model = llama.Model.from_numpy(args, weights, dev)
    rng = np.random.default_rng(seed + 1)
    G, hd = args.num_key_value_heads, args.head_dim
    cap = P + T + 32
    cache = make_prompt_cache(model, capacity=cap)
    ocache = model_oracle.new_cache(args, cap)
    for c, (ok, ov) in zip(cache, ocache):
        k = rng.standard_normal((G, P, hd), dtype=np.float32).astype(np.float16)
        v = rng.standard_normal((G, P, hd), dtype=np.float32).astype(np.float16)
        c.keys[0, :, :P].copy_(to_dev(k, dev))
        c.values[0, :, :P].copy_(to_dev(v, dev))
        c.offset = P
        ok[:, :P] = k
        ov[:, :P] = v
    cache[0].sync_len()
    parents = synth.random_tree(rng, T)
    depth, anc, bits = synth.tree_arrays(parents)
    tokens = rng.integers(0, args.vocab_size, T).astype(np.int32)
    inv, sc = synth.inv_freqs(args)
    return dict(args=args, weights=weights, model=model, cache=cache, ocache=ocache, parents=parents,
                depth=depth, anc=anc, bits=bits, tokens=tokens, inv=inv, sc=sc, P=P, T=T, cap=cap)


def run_verifier(dev, s, slab_plan, taps=None):
    """One eager step from cache length P; returns (logits, result, K rows, V rows of layer 0)."""
    P, T = s["P"], s["T"]
    for c in s["cache"]:
        c.offset = P
    s["cache"][0].sync_len()
    ver = eagle.TreeVerifier(s["model"], s["cache"], total_tokens=T - 1, max_len=s["cap"],
                             slab_plan=slab_plan, compact=False)
    ver.set_tree(to_dev(s["tokens"], dev), to_dev(s["depth"].astype(np.int32), dev),
                 to_dev(s["parents"], dev), to_dev(s["bits"].view(np.int32), dev))
    hidden = {}
    ver.forward(tap=(lambda i, h: hidden.__setitem__(i + 1, h.clone()) if i + 1 in taps else None)
                if taps else None)
    torch.cuda.synchronize()
    return ver, {k: v.cpu().numpy() for k, v in hidden.items()}


def test_one_layer_at_7b_width(dev):
    """hidden 3584, intermediate 18944, 28 / 4 heads of 128, 2048-token prefix, 32 tree rows: the
    residual stream after the layer, the appended K / V rows and the logits, with the slab plan
    the library picks and with the streaming kernel everywhere."""
    P, T = 2048, 32
    s = setup_step(dev, synth.qwen25_7b(), 1, 5, P, T)
    mask = np.concatenate([np.zeros((T, P), np.float16), tree_oracle.additive_mask(s["anc"])], axis=1)
    want_h = {}
    want = model_oracle.tree_forward(s["args"], s["weights"], s["inv"], s["sc"], s["tokens"], s["depth"] + P,
                                     mask, s["ocache"], P, tap=lambda i, h: want_h.__setitem__(i + 1, h.copy()))
    ok, ov = s["ocache"][0]
    for plan in (None, {}):
        print(f"7B-width layer, slab plan {plan}", flush=True)
        ver, hid = run_verifier(dev, s, plan, taps={1})
        assert (plan is None) == bool(ver.slab["qkv"] and ver.slab["o"] and ver.slab["down"])
        assert rel_err(hid[1], want_h[1]) <= TOL
        c = s["cache"][0]
        assert rel_err(c.keys[0, :, P:P + T].cpu().numpy(), ok[:, P:P + T]) <= TOL
        assert rel_err(c.values[0, :, P:P + T].cpu().numpy(), ov[:, P:P + T]) <= TOL
        assert rel_err(ver.logits.cpu().numpy(), want) <= TOL


def test_one_layer_at_7b_width_with_the_default_tree(dev):
    """The same layer on a tree of 40 tokens (the reference's default of 39 draft nodes,
    mlx_eagle.py:390,510): 64-row partial tiles in the slab form, gate|up and the vocabulary
    projection as two passes of 32 rows, attention in two pieces of query rows."""
    P, T = 2048, 40
    s = setup_step(dev, synth.qwen25_7b(), 1, 6, P, T)
    mask = np.concatenate([np.zeros((T, P), np.float16), tree_oracle.additive_mask(s["anc"])], axis=1)
    want_h = {}
    want = model_oracle.tree_forward(s["args"], s["weights"], s["inv"], s["sc"], s["tokens"], s["depth"] + P,
                                     mask, s["ocache"], P, tap=lambda i, h: want_h.__setitem__(i + 1, h.copy()))
    ok, ov = s["ocache"][0]
    for plan in (None, {}):
        print(f"7B-width layer, 40 tree tokens, slab plan {plan}", flush=True)
        ver, hid = run_verifier(dev, s, plan, taps={1})
        assert ver.wide and (plan is None) == bool(ver.slab["qkv"] and ver.slab["o"] and ver.slab["down"])
        assert rel_err(hid[1], want_h[1]) <= TOL
        c = s["cache"][0]
        assert rel_err(c.keys[0, :, P:P + T].cpu().numpy(), ok[:, P:P + T]) <= TOL
        assert rel_err(c.values[0, :, P:P + T].cpu().numpy(), ov[:, P:P + T]) <= TOL
        assert rel_err(ver.logits.cpu().numpy(), want) <= TOL


# Bound for the residual stream and the logits after all 28 layers.  Every operator meets
# TOL on its own output (the tests above and those of the operators); through 28 layers the
# rounding differences of 197 matmuls add up.  The test below prints how the error grows and
# which part of it is the fp16 rounding of the weights in the slab form of the matmul.
FULL_DEPTH_TOL = 6e-2


def test_cfg4_error_growth_and_acceptance(dev):
    """The whole verification step of the Qwen2.5-7B-shaped target (28 layers, 2048-token prefix,
    32 tree rows): max error over RMS of the residual stream after layers 1, 2, 4, 8, 16, 28 for
    the default slab plan and for the streaming kernel everywhere, against the oracle with fp32
    weights and with weights rounded to fp16; then the accept decision and every node argmax
    with a clear margin must equal the oracle's."""
    P, T = 2048, 32
    taps = {1, 2, 4, 8, 16, 28}
    s = setup_step(dev, synth.qwen25_7b(), None, 1234, P, T)
    oracle_runs = {}
    for mode in (False, True):
        hid = {}
        oc = [(k.copy(), v.copy()) for k, v in s["ocache"]]
        with oracle.weight_rounding(mode):
            out = model_oracle.verify_step(s["args"], s["weights"], s["inv"], s["sc"], s["tokens"], s["depth"],
                                           s["parents"], s["anc"], oc, P,
                                           tap=lambda i, h: hid.__setitem__(i + 1, h.copy()) if i + 1 in taps else None)
        oracle_runs[mode] = (out, hid)
    print("layer  " + "  ".join(f"{n:>22s}" for n in ("slab plan vs fp32 w", "slab plan vs fp16 w",
                                                         "streaming vs fp32 w", "streaming vs fp16 w")), flush=True)
    curves = {}
    vers = {}
    for pname, plan in (("slab", None), ("streaming", {})):
        ver, hid = run_verifier(dev, s, plan, taps=taps)
        vers[pname] = (ver.logits.cpu().numpy(), ver.result.cpu().numpy().copy(), ver.node_argmax.cpu().numpy())
        for mode in (False, True):
            curves[(pname, mode)] = {n: rel_err(hid[n], oracle_runs[mode][1][n]) for n in sorted(taps)}
    for n in sorted(taps):
        print(f"{n:5d}  " + "  ".join(f"{curves[k][n]:22.4f}" for k in (("slab", False), ("slab", True),
                                                                          ("streaming", False), ("streaming", True))),
              flush=True)
    for pname, (logits, result, node_argmax) in vers.items():
        want = oracle_runs[False][0]
        wl = want["logits"].astype(np.float32)
        abs_err = float(np.abs(logits.astype(np.float32) - wl).max())
        err = abs_err / float(np.sqrt(np.mean(wl * wl)))
        srt = np.sort(wl, axis=-1)
        clear = (srt[:, -1] - srt[:, -2]) > 2 * abs_err
        print(f"{pname}: logits err/rms {err:.4f}, argmax equal {int((node_argmax == want['node_argmax']).sum())}/32, "
              f"clear margins {int(clear.sum())}", flush=True)
        assert np.isfinite(logits).all()
        assert curves[(pname, False)][1] <= TOL
        assert curves[(pname, False)][28] <= FULL_DEPTH_TOL
        assert err <= FULL_DEPTH_TOL
        assert clear.sum() >= 16
        assert np.array_equal(node_argmax[clear], want["node_argmax"][clear])
        assert (result[0], result[1], result[3]) == (want["best"], want["accept_length"], want["next_token"])
