"""Slab form of the 4-bit group-64 matmul for up to 64 rows: fp32 partial sums per K slab,
added by the consumer (plain sum, RMSNorm, rotary embedding + KV append), and the verification
step built on it."""
import numpy as np
import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import eagle, ops, synth
from oracle import model_oracle, oracle, tree_oracle
from test_gpu_model import build, margins, run_verifier
from util import TOL, close_fp16, layer_to_dev, rel_err, to_dev

pytestmark = pytest.mark.gpu


def ordered_sum_f16(partial, slabs, M):
    """fp16 of the fp32 sum in slab order, as the consumers form it."""
    acc = torch.zeros_like(partial[0, :M])
    for z in range(slabs):
        acc = acc + partial[z, :M]
    return acc.half()


@pytest.mark.parametrize("M,N,K,steps,bias", [(32, 512, 512, 8, True), (32, 4608, 3584, 8, True),
                                              (31, 3584, 3584, 16, False), (17, 200, 1536, 8, True),
                                              (1, 128, 1024, 8, False), (8, 136, 2048, 24, False),
                                              (32, 3584, 18944, 32, False), (24, 1000, 4096, 32, True),
                                              (32, 3584, 18944, 48, False), (32, 256, 4096, 64, True),
                                              (13, 136, 1536, 16, False),
                                              # K a multiple of 128 only: partial last chunk, 4-byte scale fetches
                                              (8, 1152, 896, 8, True), (8, 896, 4864, 8, False), (32, 896, 4864, 32, False),
                                              (32, 200, 128, 8, True), (5, 128, 640, 8, False), (32, 264, 1920, 16, True),
                                              # 33..64 rows: 64-row partial tiles
                                              (40, 4608, 3584, 8, True), (64, 3584, 3584, 8, False),
                                              (33, 200, 1536, 8, True), (40, 3584, 18944, 32, False),
                                              (64, 1000, 4096, 16, True), (47, 136, 1024, 24, False),
                                              (40, 1152, 896, 8, True), (64, 896, 4864, 32, False),
                                              (50, 264, 1920, 16, True), (64, 128, 128, 8, False)])
def test_slab_partials_match_oracle(dev, M, N, K, steps, bias):
    print(f"slab M={M} N={N} K={K} steps={steps}", flush=True)
    rng = np.random.default_rng(M + N + K + steps)
    layer = synth.make_qlinear(rng, N, K, bias=bias)
    x = synth.make_x(rng, M, K)
    want = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"], layer.get("bias"))
    d = layer_to_dev(layer, dev)
    slabs = ops.slab_count(K, steps)
    assert slabs == -(-(K // 64) // steps)
    partial = torch.full((slabs, ops.slab_rows(M), N), float("nan"), dtype=torch.float32, device=dev)
    ops.quantized_matmul_slabs(to_dev(x, dev), d["weight"], d["scales"], d["biases"], steps, partial=partial)
    assert torch.isfinite(partial[:, :M]).all()
    assert torch.isnan(partial[:, M:]).all(), "rows past M must stay untouched"
    got = ops.slab_sum(partial, slabs, M, N, bias=d.get("bias"))
    assert rel_err(got.cpu().numpy(), want) <= TOL
    # the sum is taken in slab order in fp32, rounded once, then the fp16 bias is added
    ref = ordered_sum_f16(partial, slabs, M)
    if bias:
        ref = ref + d["bias"]
    assert torch.equal(got, ref)
    # and agrees with the streaming kernel to the rounding of the expanded weights
    stream = ops.quantized_matmul(to_dev(x, dev), d["weight"], d["scales"], d["biases"], bias=d.get("bias"))
    assert rel_err(got.cpu().numpy(), stream.cpu().numpy()) <= TOL


@pytest.mark.parametrize("M,I,K,bias", [(40, 18944, 3584, True), (64, 14336, 4096, False), (33, 16, 128, True),
                                        (32, 18944, 3584, True), (8, 4864, 896, True), (64, 272, 1920, False),
                                        (47, 2432, 896, True), (1, 64, 512, False), (64, 4112, 1024, True)])
def test_slab_form_with_swiglu(dev, M, I, K, bias):
    """gate|up + SwiGLU on the slab kernel (one slab over all of K, 64-row tiles above 32 rows,
    four to eight waves per workgroup by the row count of the weights): every projection is
    within TOL of its own RMS, so silu(g) * u is within the propagated bound of the oracle's
    qmm -> silu_mul (as for the GEMM form); against the streaming kernel's SwiGLU form too."""
    print(f"slab swiglu M={M} I={I} K={K}", flush=True)
    rng = np.random.default_rng(M + I + K)
    g = synth.make_qlinear(rng, I, K, bias=bias, gain=1.0)
    u = synth.make_qlinear(rng, I, K, bias=bias, gain=1.0)
    x = synth.make_x(rng, M, K)
    og = oracle.qmm(x, g["weight"], g["scales"], g["biases"], g.get("bias"))
    ou = oracle.qmm(x, u["weight"], u["scales"], u["biases"], u.get("bias"))
    want = oracle.silu_mul(og, ou)
    gd, ud = layer_to_dev(g, dev), layer_to_dev(u, dev)
    keys = ["weight", "scales", "biases"] + (["bias"] if bias else [])
    inter = {k: ops.interleave_gate_up(gd[k], ud[k]) for k in keys}
    xd = to_dev(x, dev)
    out = torch.full((M + 1, I), float("nan"), dtype=torch.float16, device=dev)
    ops.quantized_matmul_swiglu_slab(xd, inter["weight"], inter["scales"], inter["biases"], bias=inter.get("bias"),
                                     out=out[:M])
    got = out.cpu().numpy()
    assert np.isnan(got[M].astype(np.float32)).all()                # nothing written past the rows
    g64, u64 = og.astype(np.float64), ou.astype(np.float64)
    rms_g, rms_u = np.sqrt(np.mean(g64 * g64)), np.sqrt(np.mean(u64 * u64))
    w64, got64 = want.astype(np.float64), got[:M].astype(np.float64)
    assert np.isfinite(got64).all()
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(w64), 2.0 ** -14))) - 10)
    bound = TOL * (1.1 * np.abs(u64) * rms_g + np.abs(g64 / (1 + np.exp(-g64))) * rms_u) + 2 * ulp
    assert np.all(np.abs(got64 - w64) <= bound)
    assert np.sqrt(np.mean((got64 - w64) ** 2)) <= 0.25 * TOL * np.sqrt(np.mean(w64 * w64))
    # the dispatcher sends 33..64 rows here
    auto = ops.quantized_matmul_swiglu(xd, inter["weight"], inter["scales"], inter["biases"], bias=inter.get("bias"))
    if M > 32:
        assert torch.equal(auto, out[:M])
    else:
        close_fp16(auto.cpu().numpy(), got[:M], "streaming form")


def test_slab_swiglu_refusals(dev):
    from mlx_eagle_spec_decoding_tree_amd import _lib
    L = _lib.lib()
    assert L.eagle_qmm_slab_swiglu_supported(64, 37888, 3584) == 1 and L.eagle_qmm_slab_swiglu_supported(65, 64, 128) == 0
    assert L.eagle_qmm_slab_swiglu_supported(8, 48, 128) == 0 and L.eagle_qmm_slab_swiglu_supported(8, 64, 192) == 0
    x = torch.zeros((8, 192), dtype=torch.float16, device=dev)
    w = torch.zeros((64, 24), dtype=torch.int32, device=dev)
    s = torch.zeros((64, 3), dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        ops.quantized_matmul_swiglu_slab(x, w, s, s)


def test_slab_form_integer_exact(dev):
    """Integer-valued x, scales 1 and integer biases: every product and sum is exact."""
    rng = np.random.default_rng(6)
    M, N, K = 32, 256, 1024
    w = rng.integers(0, 1 << 32, size=(N, K // 8), dtype=np.uint32)
    s = np.ones((N, K // 64), np.float16)
    b = rng.integers(-8, 1, (N, K // 64)).astype(np.float16)
    x = rng.integers(-2, 3, (M, K)).astype(np.float16)
    q = synth.unpack_nibbles(w).astype(np.int64)
    wd = q + np.repeat(b.astype(np.int64), 64, axis=1)
    want = x.astype(np.int64) @ wd.T
    partial = ops.quantized_matmul_slabs(to_dev(x, dev), to_dev(w, dev), to_dev(s, dev), to_dev(b, dev), 8)
    got = ops.slab_sum(partial, 2, M, N).cpu().numpy()
    assert np.array_equal(got.astype(np.int64), want)


def test_slab_form_rejects_bad_arguments(dev):
    x = torch.zeros((32, 896), dtype=torch.float16, device=dev)
    w = torch.zeros((64, 112), dtype=torch.int32, device=dev)
    s = torch.zeros((64, 14), dtype=torch.float16, device=dev)
    assert ops.slab_count(832, 8) == 0 and ops.slab_count(1024, 12) == 0 and ops.slab_count(1024, 4104) == 0
    assert ops.slab_count(896, 8) == 2
    with pytest.raises(ValueError):
        ops.quantized_matmul_slabs(x[:, :832].contiguous(), w[:, :104].contiguous(), s[:, :13].contiguous(),
                                   s[:, :13].contiguous(), 8)          # K not a multiple of 128
    x = torch.zeros((65, 1024), dtype=torch.float16, device=dev)
    w = torch.zeros((64, 128), dtype=torch.int32, device=dev)
    s = torch.zeros((64, 16), dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        ops.quantized_matmul_slabs(x, w, s, s, 8)                      # more than 64 rows
    with pytest.raises(ValueError):
        ops.quantized_matmul_slabs(x[:8], w, s, s, 8, partial=torch.zeros(100, device=dev))
    with pytest.raises(ValueError):                                    # 33 rows need 64-row tiles
        ops.quantized_matmul_slabs(x[:33], w, s, s, 8, partial=torch.zeros(2 * 32 * 64, device=dev))


@pytest.mark.parametrize("T,D,slabs,residual", [(32, 3584, 7, True), (5, 512, 1, True), (32, 1024, 10, False),
                                                (17, 4096, 8, True), (40, 3584, 7, True), (64, 1024, 10, False),
                                                (33, 4096, 3, True)])
def test_rms_norm_of_slabs_equals_norm_of_their_sum(dev, T, D, slabs, residual):
    g = torch.Generator(device="cpu").manual_seed(T + D + slabs)
    partial = torch.randn((slabs, ops.slab_rows(T), D), generator=g).to(dev)
    weight = (1 + 0.1 * torch.randn(D, generator=g)).half().to(dev)
    res = torch.randn((T, D), generator=g).half().to(dev) if residual else None
    x = ops.slab_sum(partial, slabs, T, D)
    assert torch.equal(x, ordered_sum_f16(partial, slabs, T))
    if residual:
        h_want, y_want = ops.rms_norm(x, weight, 1e-6, residual=res)
        h_got, y_got = ops.rms_norm_slabs(partial, slabs, weight, 1e-6, T, residual=res)
        assert torch.equal(h_got, h_want)
    else:
        y_want = ops.rms_norm(x, weight, 1e-6)
        y_got = ops.rms_norm_slabs(partial, slabs, weight, 1e-6, T)
    assert torch.equal(y_got, y_want)


@pytest.mark.parametrize("T,H,G,hd,slabs,bias", [(32, 28, 4, 128, 7, True), (9, 4, 2, 64, 2, False),
                                                 (32, 8, 8, 128, 8, False), (40, 28, 4, 128, 7, True),
                                                 (64, 4, 2, 64, 2, False), (33, 8, 8, 128, 3, True)])
def test_rope_append_of_slabs_equals_rope_append_of_their_sum(dev, T, H, G, hd, slabs, bias):
    g = torch.Generator(device="cpu").manual_seed(T + H + hd)
    N = (H + 2 * G) * hd
    partial = torch.randn((slabs, ops.slab_rows(T), N), generator=g).to(dev)
    b = torch.randn(N, generator=g).half().to(dev) if bias else None
    P, cap = 50, 128
    len_dev = torch.tensor([P], dtype=torch.int32, device=dev)
    pos = (P + torch.arange(T, dtype=torch.int32)).to(dev)
    inv = ops.default_inv_freqs(hd, 1e6, device=dev)
    cs = ops.rope_table(pos, inv, 1.0)
    qkv = ops.slab_sum(partial, slabs, T, N, bias=b)
    outs = []
    for form in ("plain", "slabs"):
        q_rot = torch.zeros((H, T, hd), dtype=torch.float16, device=dev)
        kc = torch.zeros((G, cap, hd), dtype=torch.float16, device=dev)
        vc = torch.zeros((G, cap, hd), dtype=torch.float16, device=dev)
        if form == "plain":
            ops.rope_kv_append(qkv, qkv[:, H * hd:], qkv[:, (H + G) * hd:], pos, inv, 1.0, q_rot, kc, vc,
                               len_dev, H, G, hd, row_stride=N, rope_cs=cs)
        else:
            ops.rope_kv_append_slabs(partial, slabs, b, cs, q_rot, kc, vc, len_dev, T, H, G, hd)
        outs.append((q_rot, kc, vc))
    # the same sums and the same formula; the compiler may round the rotated value once (a
    # mixed-precision fma straight to fp16) in one kernel and twice in the other, which shows
    # as a last-bit difference in about one value in 10^5
    for a, c in zip(*outs):
        diff = (a.float() - c.float()).abs()
        assert (diff > 0).sum().item() <= max(2, a.numel() // 20000)
        assert (diff <= 2.0 ** -10 * a.float().abs().clamp(min=2.0 ** -14)).all()
    assert torch.equal(outs[0][2], outs[1][2])           # values are copied, not rotated
    assert outs[1][1][:, P:P + T].abs().sum() > 0 and outs[1][1][:, :P].abs().sum() == 0


SLAB_MODEL = dict(layers=2, hidden=1024, inter=1536, heads=8, kv_heads=2, head_dim=128, vocab=640,
                  attention_bias=True, tie=False)


@pytest.mark.parametrize("plan", [dict(qkv=8, o=8, down=8), dict(qkv=16, o=0, down=24), dict(qkv=0, o=8, down=0)])
def test_step_with_slab_projections(dev, plan, monkeypatch):
    import test_gpu_model
    monkeypatch.setitem(test_gpu_model.CONFIGS, "slab_model", SLAB_MODEL)
    P, T = 150, 32
    s = build(dev, "slab_model", P, T, seed=11)
    ver = run_verifier(s, dev, graph=False, slab_plan=plan)
    assert ver.slab == plan
    ver.step()
    torch.cuda.synchronize()
    want = model_oracle.verify_step(s["args"], s["weights"], s["inv"], s["sc"], s["tokens"], s["depth"],
                                    s["parents"], s["anc"], s["ocache"], P)
    got = ver.logits.cpu().numpy()
    assert rel_err(got, want["logits"]) <= TOL
    for c, (ok, ov) in zip(s["cache"], s["ocache"]):
        assert rel_err(c.keys[0, :, P:P + T].cpu().numpy(), ok[:, P:P + T]) <= TOL
        assert rel_err(c.values[0, :, P:P + T].cpu().numpy(), ov[:, P:P + T]) <= TOL
    am = ver.node_argmax.cpu().numpy()
    assert np.array_equal(am, oracle.argmax_rows(got))
    ri = tree_oracle.post_process_draft_tree(s["depth"], T - 1, s["parents"])
    best, al, bonus = tree_oracle.greedy_accept(am, s["tokens"], ri)
    r = ver.result.cpu().numpy()
    assert (r[0], r[1], r[2], r[3]) == (best, al, bonus, am[bonus])
    err = np.abs(got.astype(np.float32) - want["logits"].astype(np.float32)).max()
    if (margins(want["logits"]) > 2 * err).all():
        assert (best, al, am[bonus]) == (want["best"], want["accept_length"], want["next_token"])
    # against the same step on the streaming kernel, and a captured graph against the eager step
    s2 = build(dev, "slab_model", P, T, seed=11)
    base = run_verifier(s2, dev, graph=False, slab_plan={})
    assert base.slab == dict(qkv=0, o=0, down=0)
    base.step()
    torch.cuda.synchronize()
    assert rel_err(got, base.logits.cpu().numpy()) <= TOL
    s3 = build(dev, "slab_model", P, T, seed=11)
    cap = run_verifier(s3, dev, graph=True, slab_plan=plan)
    for _ in range(2):
        cap.len_dev.fill_(P)
        cap.step()
        torch.cuda.synchronize()
        assert torch.equal(cap.logits, ver.logits)


def test_full_size_properties(dev):
    """The down projection of the 7B shape (3584 x 18944, 32 rows), too large for the CPU checker
    in a test: rows are independent (bit for bit), the slab length only changes the fp32
    summation order, and the product is linear in x."""
    g = torch.Generator(device="cpu").manual_seed(21)
    N, K, M = 3584, 18944, 32
    w = torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 8), dtype=torch.int32, generator=g).to(dev)
    s = (torch.rand(N, K // 64, generator=g) * 0.0015 + 0.0005).half().to(dev)
    b = (-7.5 * s.float() + 1e-4 * torch.randn(N, K // 64, generator=g).to(dev)).half()
    x = torch.randn(M, K, generator=g).half().to(dev)
    slabs = ops.slab_count(K, 32)
    full = ops.slab_sum(ops.quantized_matmul_slabs(x, w, s, b, 32), slabs, M, N)
    assert torch.isfinite(full).all()
    # row 5 alone, and rows 3..12 alone, give the same bits as inside the batch of 32
    one = ops.slab_sum(ops.quantized_matmul_slabs(x[5:6].contiguous(), w, s, b, 32), slabs, 1, N)
    assert torch.equal(one[0], full[5])
    some = ops.slab_sum(ops.quantized_matmul_slabs(x[3:13].contiguous(), w, s, b, 32), slabs, 10, N)
    assert torch.equal(some, full[3:13])
    # another slab length: same products, another order of the fp32 sums
    other = ops.slab_sum(ops.quantized_matmul_slabs(x, w, s, b, 16), ops.slab_count(K, 16), M, N)
    rms = full.float().pow(2).mean().sqrt()
    assert (other.float() - full.float()).abs().max() <= 2e-3 * rms
    # the streaming kernel (exact weights, fp32 accumulation) within the stated tolerance
    stream = ops.quantized_matmul(x, w, s, b)
    assert (stream.float() - full.float()).abs().max() <= TOL * rms
    # linear in x: f(x) + f(y) = f(x + y) up to the fp16 roundings of x + y and of the three results
    y = torch.randn(M, K, generator=g).half().to(dev)
    xy = (x.float() + y.float()).half()
    f_y = ops.slab_sum(ops.quantized_matmul_slabs(y, w, s, b, 32), slabs, M, N)
    f_xy = ops.slab_sum(ops.quantized_matmul_slabs(xy, w, s, b, 32), slabs, M, N)
    assert (f_xy.float() - full.float() - f_y.float()).abs().max() <= TOL * f_xy.float().pow(2).mean().sqrt()


@pytest.mark.parametrize("graph", [False, True])
def test_device_loop_with_slab_projections(dev, graph):
    """The device-resident loop with q|k|v, o and down of both models on the slab kernel emits
    the target's greedy stream."""
    from mlx_eagle_spec_decoding_tree_amd import llama, spec
    from test_gpu_draft import assert_greedy_stream

    targs = synth.tiny(layers=2, hidden=512, inter=1024, heads=4, kv_heads=2, head_dim=128, vocab=1024,
                       attention_bias=True)
    dargs = synth.tiny(layers=1, hidden=512, inter=512, heads=8, kv_heads=2, head_dim=64, vocab=1024)
    tw = synth.make_model_weights(targs, seed=31)
    dw = synth.make_model_weights(dargs, seed=32)
    target, draft = llama.Model.from_numpy(targs, tw, dev), llama.Model.from_numpy(dargs, dw, dev)
    rng = np.random.default_rng(33)
    prompt = rng.integers(0, 1024, 45).astype(np.int32)
    plan = dict(qkv=8, o=8, down=8)
    dec = spec.SpeculativeDecoder(target, draft, capacity=256, k=8, depth=3, verify_num_tokens=31,
                                  slab_plan=plan, draft_slab_plan=plan)
    assert dec.verifier.slab == plan and dec.draft.slab == plan
    first = dec.prefill(to_dev(prompt.astype(np.int64), dev))
    if graph:
        dec.capture()
    tokens = dec.generate(5)
    assert len(tokens) >= 5
    reference = llama.Model.from_numpy(targs, tw, dev)
    assert_greedy_stream(reference, prompt, [first] + tokens, dev)
