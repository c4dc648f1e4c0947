"""The matmul with x resident in registers (csrc/resident.hip) vs the CPU oracle, through the
C ABI: plain and SwiGLU forms, ragged rows, edge shapes, and the cfg2 shapes it serves."""
import numpy as np
import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import _lib, ops, synth
from oracle import oracle
from util import TOL, layer_to_dev, rel_err, to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("N,K", [(8, 512), (40, 1024), (136, 1536), (512, 3584), (8192, 2048),
                                 (3584, 3584), (4608, 3584)])
@pytest.mark.parametrize("M", [1, 8, 17, 32])
def test_plain_form(dev, M, N, K):
    print(f"resident qmm M={M} N={N} K={K}", flush=True)
    assert ops.resident_supported(M, N, K)
    rng = np.random.default_rng(N + K + M)
    bias = (N // 8) % 2 == 1
    layer = synth.make_qlinear(rng, N, K, bias=bias)
    x = synth.make_x(rng, M, K)
    want = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"], layer.get("bias"))
    d = layer_to_dev(layer, dev)
    got = ops.quantized_matmul_resident(to_dev(x, dev), d["weight"], d["scales"], d["biases"],
                                        bias=d.get("bias"))
    torch.cuda.synchronize()
    assert rel_err(got.cpu().numpy(), want) <= TOL


def test_known_answers(dev):
    """One-hot x rows give the dequantised weight column exactly (pins the nibble order and the
    subnormal expansion: fp16(s q + b) with a single rounding); s = 1/8, b = 0 with integer x is
    an exact integer matmul."""
    rng = np.random.default_rng(3)
    N, K = 96, 1024
    layer = synth.make_qlinear(rng, N, K)
    cols = rng.choice(K, size=32, replace=False)
    x = np.zeros((32, K), np.float16)
    x[np.arange(32), cols] = 1.0
    d = layer_to_dev(layer, dev)
    got = ops.quantized_matmul_resident(to_dev(x, dev), d["weight"], d["scales"], d["biases"]).cpu().numpy()
    q = synth.unpack_nibbles(layer["weight"])[:, cols].astype(np.float32)
    s = layer["scales"].astype(np.float32)[:, cols // 64]
    b = layer["biases"].astype(np.float32)[:, cols // 64]
    want = (s * q + b).astype(np.float16).T
    assert np.array_equal(got, want)
    layer["scales"][:] = np.float16(0.125)
    layer["biases"][:] = np.float16(0)
    xi = rng.integers(-3, 4, size=(8, K)).astype(np.float16)
    d = layer_to_dev(layer, dev)
    got = ops.quantized_matmul_resident(to_dev(xi, dev), d["weight"], d["scales"], d["biases"]).cpu().numpy()
    want = xi.astype(np.float64) @ synth.unpack_nibbles(layer["weight"]).astype(np.float64).T / 8
    assert np.array_equal(got.astype(np.float64), want.astype(np.float16).astype(np.float64))


@pytest.mark.parametrize("I,K,bias", [(16, 512, False), (48, 1024, True), (272, 1536, True), (18944, 3584, True)])
def test_swiglu_form(dev, I, K, bias):
    for M in (1, 8, 17, 32):
        print(f"resident swiglu I={I} K={K} M={M}", flush=True)
        rng = np.random.default_rng(I + K + M)
        g = synth.make_qlinear(rng, I, K, bias=bias, gain=1.0)
        u = synth.make_qlinear(rng, I, K, bias=bias, gain=1.0)
        x = synth.make_x(rng, M, K)
        want = oracle.silu_mul(oracle.qmm(x, g["weight"], g["scales"], g["biases"], g.get("bias")),
                               oracle.qmm(x, u["weight"], u["scales"], u["biases"], u.get("bias")))
        gd, ud = layer_to_dev(g, dev), layer_to_dev(u, dev)
        keys = ["weight", "scales", "biases"] + (["bias"] if bias else [])
        inter = {k: ops.interleave_gate_up(gd[k], ud[k]) for k in keys}
        got = ops.quantized_matmul_resident(to_dev(x, dev), inter["weight"], inter["scales"], inter["biases"],
                                            bias=inter.get("bias"), swiglu=True)
        torch.cuda.synchronize()
        assert tuple(got.shape) == (M, I)
        # The product of two rounded values: where |g| and |u| are several sigma, one fp16 ulp of
        # g (the sum lands on the other side of a rounding boundary) moves the output by more
        # than 2e-2 of the output RMS (seen: g 2.986 vs 2.984, u 3.33, output 9.48 vs 9.46 with an
        # RMS of 0.6).  So the bound is the QMM one plus two fp16 ulps of the expected value, and
        # the RMS error, which no single element dominates, has to stay 10 times below the bound.
        g64, w64 = got.cpu().numpy().astype(np.float64), want.astype(np.float64)
        rms = np.sqrt(np.mean(w64 * w64))
        ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(w64), 2.0 ** -14))) - 10)
        assert np.all(np.abs(g64 - w64) <= TOL * rms + 2 * ulp)
        assert np.sqrt(np.mean((g64 - w64) ** 2)) <= 0.1 * TOL * rms


def test_rejects_what_it_does_not_take(dev):
    assert not ops.resident_supported(8, 64, 4096)
    assert not ops.resident_supported(8, 64, 896)
    assert not ops.resident_supported(33, 64, 512)
    x = torch.zeros((8, 4096), dtype=torch.float16, device=dev)
    w = torch.zeros((64, 512), dtype=torch.int32, device=dev)
    s = torch.zeros((64, 64), dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        ops.quantized_matmul_resident(x, w, s, s)


@pytest.mark.parametrize("N,K", [(8, 512), (40, 1024), (3584, 3584), (512, 3584), (3584, 18944), (8192, 2048)])
def test_vector_alu_matvec(dev, N, K):
    """The M = 1 product on the vector ALU (csrc/qmv.hip) against the oracle."""
    print(f"qmv N={N} K={K}", flush=True)
    rng = np.random.default_rng(N + K)
    layer = synth.make_qlinear(rng, N, K, bias=(N % 16 == 8))
    x = synth.make_x(rng, 1, K)
    want = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"], layer.get("bias"))
    d = layer_to_dev(layer, dev)
    got = ops.quantized_matvec(to_dev(x, dev), d["weight"], d["scales"], d["biases"], bias=d.get("bias"))
    torch.cuda.synchronize()
    assert tuple(got.shape) == (1, N)
    assert rel_err(got.cpu().numpy(), want) <= TOL


def chain_case(dev, M, D, I, seed, bias):
    rng = np.random.default_rng(seed)
    o = synth.make_qlinear(rng, D, D, gain=1.0)
    g = synth.make_qlinear(rng, I, D, bias=bias, gain=1.0)
    u = synth.make_qlinear(rng, I, D, bias=bias, gain=1.0)
    attn = synth.make_x(rng, M, D)
    h = synth.make_x(rng, M, D)
    nw = (1.0 + rng.normal(0, 0.02, D)).astype(np.float16)
    eps = 1e-6
    od, gd, ud = layer_to_dev(o, dev), layer_to_dev(g, dev), layer_to_dev(u, dev)
    # the product that precedes the norm, as K slabs (the o projection of the step)
    partial = ops.quantized_matmul_slabs(to_dev(attn, dev), od["weight"], od["scales"], od["biases"], 8)
    slabs = ops.slab_count(D, 8)
    o16 = ops.slab_sum(partial, slabs, M, D).cpu().numpy()
    h2 = oracle.add(h, o16)
    xn = oracle.rmsnorm(h2, nw, eps)
    want = oracle.silu_mul(oracle.qmm(xn, g["weight"], g["scales"], g["biases"], g.get("bias")),
                           oracle.qmm(xn, u["weight"], u["scales"], u["biases"], u.get("bias")))
    keys = ["weight", "scales", "biases"] + (["bias"] if bias else [])
    inter = {k: ops.interleave_gate_up(gd[k], ud[k]) for k in keys}
    return dict(partial=partial, slabs=slabs, h=to_dev(h, dev), nw=to_dev(nw, dev), eps=eps, inter=inter,
                h2=h2, want=want, M=M, D=D, I=I)


def run_chain(dev, c, scratch, err, spin=None):
    h = c["h"].clone()
    act = torch.full((c["M"], c["I"]), float("nan"), dtype=torch.float16, device=dev)
    kw = {} if spin is None else {"spin_ticks": spin}
    ops.norm_mlp_in(c["partial"], c["slabs"], h, c["nw"], c["eps"], c["inter"]["weight"], c["inter"]["scales"],
                    c["inter"]["biases"], c["inter"].get("bias"), act, scratch, err, **kw)
    torch.cuda.synchronize()
    return h, act


def check_swiglu(got, want):
    g64, w64 = got.astype(np.float64), want.astype(np.float64)
    rms = np.sqrt(np.mean(w64 * w64))
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(w64), 2.0 ** -14))) - 10)
    assert np.all(np.abs(g64 - w64) <= TOL * rms + 2 * ulp)
    assert np.sqrt(np.mean((g64 - w64) ** 2)) <= 0.1 * TOL * rms


@pytest.mark.parametrize("M,D,I,bias", [(32, 512, 256, False), (8, 1024, 1536, True), (17, 1536, 4864, True),
                                        (32, 3584, 18944, False)])
def test_norm_and_mlp_in_one_launch(dev, M, D, I, bias):
    """Residual add + sums of squares, grid barrier, RMSNorm + gate|up + SwiGLU in one launch of
    a resident grid, against the oracle's separate operators; three launches in a row on the same
    scratch (the barrier counters only grow).  The new h is bit-identical to the separate
    kernels' (same slab sums, same rounding)."""
    print(f"chain M={M} D={D} I={I}", flush=True)
    assert ops.norm_mlp_in_supported(M, D, I)
    c = chain_case(dev, M, D, I, seed=M + D + I, bias=bias)
    scratch, err = ops.norm_mlp_in_scratch(dev)
    for rep in range(3):
        h, act = run_chain(dev, c, scratch, err)
        assert int(err.item()) == 0
        assert np.array_equal(h.cpu().numpy(), c["h2"])
        check_swiglu(act.cpu().numpy(), c["want"])


def test_grid_barrier_gives_up_and_recovers(dev):
    """The bounded wait of the in-kernel barrier, forced from the host: with a limit of one tick
    (10 ns) workgroups give up, the error word is set, the launch still ends normally; after
    the scratch and the error word are zeroed the next launch is correct."""
    c = chain_case(dev, 32, 1024, 1536, seed=77, bias=False)
    scratch, err = ops.norm_mlp_in_scratch(dev)
    run_chain(dev, c, scratch, err, spin=1)
    assert int(err.item()) == 1
    scratch.zero_()
    err.zero_()
    h, act = run_chain(dev, c, scratch, err)
    assert int(err.item()) == 0
    assert np.array_equal(h.cpu().numpy(), c["h2"])
    check_swiglu(act.cpu().numpy(), c["want"])


def test_verifier_with_the_chained_launch(dev):
    """TreeVerifier(chain=True): the whole step with norm + gate|up as one resident-grid launch
    per layer against the oracle, replayed as a HIP graph (every replay equal to the first, the
    barrier never gives up)."""
    import test_gpu_model as tm
    from mlx_eagle_spec_decoding_tree_amd import eagle
    from oracle import model_oracle
    P, T = 200, 32
    s = tm.build(dev, "llama_like_tied", P, T, seed=9)
    want = model_oracle.verify_step(s["args"], s["weights"], s["inv"], s["sc"], s["tokens"], s["depth"],
                                    s["parents"], s["anc"], s["ocache"], P)
    ver = tm.run_verifier(s, dev, graph=True, chain=True, compact=False)
    assert ver.chain and ver.slab["o"]
    outs = []
    for rep in range(3):
        ver.len_dev.fill_(P)
        ver.step()
        torch.cuda.synchronize()
        outs.append(ver.logits.clone())
        assert not ver.chain_error()
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    assert rel_err(outs[0].cpu().numpy(), want["logits"]) <= TOL
    r = ver.result.cpu().numpy()
    am = ver.node_argmax.cpu().numpy()
    assert np.array_equal(am, oracle.argmax_rows(outs[0].cpu().numpy()))
    with pytest.raises(ValueError):
        s2 = tm.build(dev, "qwen_like", 40, 8, seed=1)        # hidden 256: the chained launch does not take it
        eagle.TreeVerifier(s2["model"], s2["cache"], total_tokens=7, chain=True)


def test_verifier_with_resident_gate_up(dev):
    """TreeVerifier(resident_gate_up=True): gate|up + SwiGLU of every layer through the kernel with
    x resident in registers, the whole step against the oracle and against the default form; a
    model whose hidden size the kernel does not take is refused."""
    import test_gpu_model as tm
    from mlx_eagle_spec_decoding_tree_amd import eagle
    from oracle import model_oracle
    P, T = 200, 32
    s = tm.build(dev, "llama_like_tied", P, T, seed=9)          # hidden 512
    want = model_oracle.verify_step(s["args"], s["weights"], s["inv"], s["sc"], s["tokens"], s["depth"],
                                    s["parents"], s["anc"], s["ocache"], P)
    ver = tm.run_verifier(s, dev, graph=True, resident_gate_up=True, compact=False)
    assert ver.resident_gate_up
    ver.len_dev.fill_(P)
    ver.step()
    torch.cuda.synchronize()
    got = ver.logits.cpu().numpy()
    assert rel_err(got, want["logits"]) <= TOL
    assert np.array_equal(ver.node_argmax.cpu().numpy(), oracle.argmax_rows(got))
    s1 = tm.build(dev, "llama_like_tied", P, T, seed=9)
    plain = tm.run_verifier(s1, dev, graph=False, compact=False)
    assert not plain.resident_gate_up
    plain.step()
    torch.cuda.synchronize()
    assert rel_err(got, plain.logits.cpu().numpy()) <= TOL
    with pytest.raises(ValueError):
        s2 = tm.build(dev, "qwen_like", 40, 8, seed=1)          # hidden 256
        eagle.TreeVerifier(s2["model"], s2["cache"], total_tokens=7, resident_gate_up=True)
