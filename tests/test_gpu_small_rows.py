"""The small-row products with norm, residual add and SwiGLU folded in (csrc/smallpass.hip) vs the
CPU oracle's separate operators, through the C ABI; and the drafter's pass object with them
against the same object with one launch per operator."""
import numpy as np
import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import llama, ops, spec, synth
from mlx_eagle_spec_decoding_tree_amd.cache import make_prompt_cache
from oracle import oracle
from util import MODEL_TOL, TOL, layer_to_dev, rel_err, to_dev

pytestmark = pytest.mark.gpu

EPS = 1e-6


def q(x, L):
    return oracle.qmm(x, L["weight"], L["scales"], L["biases"], L.get("bias"))


def close(got, want, what=""):
    """Whole-output bound plus an elementwise one in units of the output's RMS (a rounding flip of
    an fp16 intermediate moves single elements by an ulp or two of their own size)."""
    g64, w64 = got.astype(np.float64), want.astype(np.float64)
    assert np.isfinite(g64).all(), what
    rms = np.sqrt(np.mean(w64 * w64))
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(w64), 2.0 ** -14))) - 10)
    assert np.all(np.abs(g64 - w64) <= TOL * rms + 2 * ulp), what
    assert np.sqrt(np.mean((g64 - w64) ** 2)) <= 0.1 * TOL * rms, what


def dev_args(layer, dev):
    d = layer_to_dev(layer, dev)
    return (d["weight"], d["scales"], d["biases"]), d.get("bias")


# K: one chunk, the drafter's hidden size, the limit of the four-wave form; then eight and sixteen waves
@pytest.mark.parametrize("N,K", [(16, 128), (1152, 896), (896, 896), (272, 1280), (896, 4864), (48, 1408),
                                 (2048, 5120), (32, 2560), (16, 3072), (48, 6144)])
@pytest.mark.parametrize("T", [1, 8, 13, 16])
def test_plain_and_residual_forms(dev, T, N, K):
    print(f"small rows T={T} N={N} K={K}", flush=True)
    assert ops.small_supported(T, N, K)
    rng = np.random.default_rng(T + N + K)
    for bias in (False, True):
        layer = synth.make_qlinear(rng, N, K, bias=bias, gain=1.0)
        x = synth.make_x(rng, T, K)
        w, b = dev_args(layer, dev)
        want = q(x, layer)
        got = ops.quantized_matmul_small(to_dev(x, dev), *w, bias=b)
        close(got.cpu().numpy(), want, "plain")
        r = synth.make_x(rng, T, N)
        h = to_dev(r, dev)
        out = ops.quantized_matmul_small(to_dev(x, dev), *w, bias=b, out=h, residual=h)     # in place
        assert out is h
        close(h.cpu().numpy(), oracle.add(r, want), "residual")


def test_known_answers(dev):
    """One-hot x rows give the dequantised weight column exactly (pins the nibble order, the
    operand layout and the subnormal expansion: fp16(s q + b) with a single rounding), on both
    the four-wave and the eight-wave kernel; s = 1/8, b = 0 with small integer x is an exact integer
    product."""
    rng = np.random.default_rng(3)
    for N, K in ((96, 1024), (64, 2560), (32, 896)):
        layer = synth.make_qlinear(rng, N, K)
        cols = rng.choice(K, size=16, replace=False)
        x = np.zeros((16, K), np.float16)
        x[np.arange(16), cols] = 1.0
        w, _ = dev_args(layer, dev)
        got = ops.quantized_matmul_small(to_dev(x, dev), *w).cpu().numpy()
        qv = synth.unpack_nibbles(layer["weight"])[:, cols].astype(np.float32)
        s = layer["scales"].astype(np.float32)[:, cols // 64]
        b = layer["biases"].astype(np.float32)[:, cols // 64]
        assert np.array_equal(got, (s * qv + b).astype(np.float16).T)
        layer["scales"][:] = np.float16(0.125)
        layer["biases"][:] = np.float16(0)
        xi = rng.integers(-3, 4, size=(8, K)).astype(np.float16)
        w, _ = dev_args(layer, dev)
        got = ops.quantized_matmul_small(to_dev(xi, dev), *w).cpu().numpy()
        want = xi.astype(np.float64) @ synth.unpack_nibbles(layer["weight"]).astype(np.float64).T / 8
        assert np.array_equal(got.astype(np.float64), want.astype(np.float16).astype(np.float64))


@pytest.mark.parametrize("N,K", [(1152, 896), (16, 128), (512, 1280), (256, 384), (64, 1664), (4608, 3584),
                                 (32, 5120)])
@pytest.mark.parametrize("T", [1, 8, 16])
def test_norm_folded_in(dev, T, N, K):
    """RMSNorm(x) . W^T + bias against the oracle's norm followed by its product."""
    rng = np.random.default_rng(T * 7 + N + K)
    layer = synth.make_qlinear(rng, N, K, bias=True, gain=1.0)
    x = (synth.make_x(rng, T, K).astype(np.float32) * rng.uniform(0.2, 5.0, (T, 1))).astype(np.float16)
    nw = (1.0 + rng.normal(0, 0.1, K)).astype(np.float16)
    w, b = dev_args(layer, dev)
    got = ops.quantized_matmul_small(to_dev(x, dev), *w, bias=b, norm_weight=to_dev(nw, dev), eps=EPS)
    close(got.cpu().numpy(), q(oracle.rmsnorm(x, nw, EPS), layer))


@pytest.mark.parametrize("I,K,bias", [(4864, 896, False), (16, 128, True), (272, 1280, True), (1536, 512, False),
                                      (48, 2560, True), (8960, 1536, False)])
@pytest.mark.parametrize("T", [1, 8, 16])
def test_swiglu_with_norm(dev, T, I, K, bias):
    """silu(g) * u over RMSNorm(x), gate|up interleaved in 16-row tiles, with and without the norm."""
    rng = np.random.default_rng(T + I + K)
    g = synth.make_qlinear(rng, I, K, bias=bias, gain=1.0)
    u = synth.make_qlinear(rng, I, K, bias=bias, gain=1.0)
    x = synth.make_x(rng, T, K)
    nw = (1.0 + rng.normal(0, 0.1, K)).astype(np.float16)
    gd, ud = layer_to_dev(g, dev), layer_to_dev(u, dev)
    keys = ["weight", "scales", "biases"] + (["bias"] if bias else [])
    inter = {k: ops.interleave_gate_up(gd[k], ud[k]) for k in keys}
    for norm in (True, False):
        xn = oracle.rmsnorm(x, nw, EPS) if norm else x
        want = oracle.silu_mul(q(xn, g), q(xn, u))
        got = ops.quantized_matmul_small(to_dev(x, dev), inter["weight"], inter["scales"], inter["biases"],
                                         bias=inter.get("bias"), swiglu=True,
                                         norm_weight=to_dev(nw, dev) if norm else None, eps=EPS)
        assert tuple(got.shape) == (T, I)
        close(got.cpu().numpy(), want, norm)


def test_refusals(dev):
    assert not ops.small_supported(17, 896, 896)                       # rows
    assert not ops.small_supported(8, 896, 900)
    assert not ops.small_supported(8, 896, 6272)                       # x does not fit the waves of a workgroup
    assert not ops.small_supported(8, 896, 18944)
    assert not ops.small_supported(8, 48, 896, swiglu=True)            # whole (gate, up) tile pairs
    rng = np.random.default_rng(1)
    layer = synth.make_qlinear(rng, 64, 256)
    w, _ = dev_args(layer, dev)
    x = to_dev(synth.make_x(rng, 4, 256), dev)
    with pytest.raises(Exception):
        ops.quantized_matmul_small(x, *w, out=x[:, :64])               # x aliasing out / stride
    with pytest.raises(ValueError):
        ops.quantized_matmul_small(x, *w, residual=torch.zeros(4, 32, dtype=torch.float16, device=dev))


@pytest.mark.parametrize("shape", ["drafter", "tiny"])
def test_pass_object_with_and_without(dev, shape):
    """spec.DecoderPass over the same tokens, cache and masks with the folded small-row products
    and with one launch per operator: logits and the KV rows written agree to the whole-model
    bound, the argmax of every row is the same, and a HIP graph of the folded form replays to
    the same bits."""
    if shape == "drafter":
        args = synth.tiny(layers=3, hidden=896, inter=4864, heads=14, kv_heads=2, head_dim=64, vocab=2048)
    else:
        args = synth.tiny(layers=2, hidden=128, inter=256, heads=2, kv_heads=1, head_dim=64, vocab=1024)
    w = synth.make_model_weights(args, seed=11)
    rng = np.random.default_rng(3)
    P, T = 37, 8
    prompt = rng.integers(0, args.vocab_size, P).astype(np.int64)
    toks = to_dev(rng.integers(0, args.vocab_size, T).astype(np.int32), dev)
    pos = to_dev((P + np.arange(T) % 3).astype(np.int32), dev)
    # row t sees itself and a few earlier rows of the pass
    words = np.zeros((T, 2), np.uint32)
    for t in range(T):
        words[t, 0] = (1 << t) | (1 if t % 2 else 0) | ((1 << (t - 1)) if t > 2 else 0)
    words = to_dev(words.view(np.int32), dev)
    outs = {}
    for folded in (False, True):
        model = llama.Model.from_numpy(args, w, dev)
        cache = make_prompt_cache(model, capacity=128)
        model(to_dev(prompt, dev)[None], cache=cache)
        p = spec.DecoderPass(model, cache, T, folded=folded)
        assert p.folded == folded
        wl = torch.tensor([P], dtype=torch.int32, device=dev)
        logits = p.forward(toks, pos, wl, wl, words, T).clone()
        torch.cuda.synchronize()
        if folded:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                p.forward(toks, pos, wl, wl, words, T)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                p.forward(toks, pos, wl, wl, words, T)
            for _ in range(3):
                p.logits.zero_()
                g.replay()
                torch.cuda.synchronize()
                assert torch.equal(p.logits, logits)
        outs[folded] = (logits.cpu().numpy(), [c.keys[0, :, :P + T].cpu().numpy() for c in cache],
                        [c.values[0, :, :P + T].cpu().numpy() for c in cache])
    a, b = outs[False], outs[True]
    assert rel_err(b[0], a[0]) <= MODEL_TOL
    assert np.array_equal(a[0].argmax(-1), b[0].argmax(-1))
    for x, y in zip(a[1] + a[2], b[1] + b[2]):
        assert rel_err(y, x) <= MODEL_TOL


def test_pass_object_falls_back(dev):
    """Shapes or weights the small-row form does not take: the pass object keeps one launch per
    operator by itself and refuses the form when asked for it."""
    args = synth.tiny(layers=1, hidden=192, inter=256, heads=3, kv_heads=1, head_dim=64, vocab=512)   # 192: not a multiple of 128
    model = llama.Model.from_numpy(args, synth.make_model_weights(args, seed=2), dev)
    cache = make_prompt_cache(model, capacity=64)
    assert not spec.DecoderPass(model, cache, 8).folded
    with pytest.raises(ValueError):
        spec.DecoderPass(model, cache, 8, folded=True)
    args = synth.tiny(layers=1, hidden=128, inter=256, heads=2, kv_heads=1, head_dim=64, vocab=512)
    model = llama.Model.from_numpy(args, synth.make_model_weights(args, seed=2), dev)
    cache = make_prompt_cache(model, capacity=64)
    assert spec.DecoderPass(model, cache, 8).folded
    sc = model.model.layers[0].mlp.down_proj.scales
    sc[0, 0] = 0.25                                                    # scale * 2^18 no longer a finite fp16
    assert not spec.DecoderPass(model, cache, 8).folded


@pytest.mark.parametrize("T,D,H,G,hd,bias", [(8, 896, 14, 2, 64, True), (8, 128, 2, 1, 64, False),
                                             (3, 256, 4, 2, 64, True), (16, 1024, 8, 2, 128, True),
                                             (8, 2048, 32, 8, 64, False), (5, 384, 3, 3, 32, True)])
def test_qkv_with_rotation_and_append(dev, T, D, H, G, hd, bias):
    """Norm + q|k|v + rope + cache append in one launch against the same small-row product followed
    by the separate rope / append launch: the same q and new K rows (to the last bit but for rounding
    ties of the rotation), identical V rows, and nothing else in the caches touched; rows past the capacity are dropped (their q rows too, as there)."""
    rng = np.random.default_rng(T + D + H)
    W = (H + 2 * G) * hd
    layer = synth.make_qlinear(rng, W, D, bias=bias, gain=1.0)
    (w, sc, bi), b = dev_args(layer, dev)
    x = to_dev(synth.make_x(rng, T, D), dev)
    nw = to_dev((1.0 + rng.normal(0, 0.1, D)).astype(np.float16), dev)
    args = synth.ModelArgs(head_dim=hd, hidden_size=hd * H, num_attention_heads=H, rope_theta=1e4)
    inv, scaling = synth.inv_freqs(args)
    pos = to_dev(rng.integers(0, 500, T).astype(np.int32), dev)
    cs = ops.rope_table(pos, to_dev(inv, dev), scaling)
    for cap, P in ((64, 11), (40, 40 - T + 2)):
        wl = torch.tensor([P], dtype=torch.int32, device=dev)
        f16 = dict(dtype=torch.float16, device=dev)
        outs = []
        for fused in (False, True):
            q_rot = torch.full((H, T, hd), 5.0, **f16)
            kc = torch.full((G, cap, hd), 7.0, **f16)
            vc = torch.full((G, cap, hd), 7.0, **f16)
            if fused:
                ops.qkv_rope_small(x, w, sc, bi, b, cs, q_rot, kc, vc, wl, H, G, hd, norm_weight=nw, eps=EPS)
            else:
                qkv = ops.quantized_matmul_small(x, w, sc, bi, bias=b, norm_weight=nw, eps=EPS)
                ops.rope_kv_append(qkv, qkv[:, H * hd:], qkv[:, (H + G) * hd:], pos, to_dev(inv, dev), scaling,
                                   q_rot, kc, vc, wl, H, G, hd, row_stride=W, rope_cs=cs)
            torch.cuda.synchronize()
            outs.append((q_rot, kc, vc))
        for a, bb in zip(*outs):
            # the two kernels contract the rotation's multiply-adds differently: a last-bit fp32
            # difference can land on an fp16 rounding tie (seen: one element in 16 K)
            a32, b32 = a.float(), bb.float()
            ulp = torch.exp2(torch.floor(torch.log2(a32.abs().clamp_min(2.0 ** -14))) - 10)
            assert bool(((a32 - b32).abs() <= ulp).all())
            assert int((a != bb).sum()) <= max(1, a.numel() // 2000)
        assert torch.equal(outs[0][2], outs[1][2])                   # v rows are not rotated
        assert (outs[1][1][:, :P] == 7.0).all() and (outs[1][1][:, P + T:] == 7.0).all()
