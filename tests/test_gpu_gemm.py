"""Many-row form of the 4-bit group-64 matmul (the prompt pass) against the oracle."""
import numpy as np
import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import ops, synth
from oracle import oracle
from util import TOL, close_fp16, layer_to_dev, rel_err, to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,N,K,bias", [(512, 1152, 896, True), (512, 896, 4864, False), (33, 64, 64, True),
                                        (128, 128, 128, False), (129, 200, 192, True), (300, 4096, 1024, False),
                                        (512, 3584, 3584, True), (64, 1000, 640, False)])
def test_gemm_form_matches_oracle(dev, M, N, K, bias):
    print(f"gemm M={M} N={N} K={K}", flush=True)
    rng = np.random.default_rng(M + N + K)
    layer = synth.make_qlinear(rng, N, K, bias=bias)
    x = synth.make_x(rng, M, K)
    want = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"], layer.get("bias"))
    d = layer_to_dev(layer, dev)
    got = ops.quantized_matmul(to_dev(x, dev), d["weight"], d["scales"], d["biases"], bias=d.get("bias"),
                               gemm=True)
    got = got.cpu().numpy()
    assert got.shape == (M, N) and np.isfinite(got.astype(np.float32)).all()
    assert rel_err(got, want) <= TOL
    # rows are independent: the first 32 rows agree with the streaming kernel to rounding of the weights
    small = ops.quantized_matmul(to_dev(x[:32], dev), d["weight"], d["scales"], d["biases"],
                                 bias=d.get("bias")).cpu().numpy()
    assert rel_err(got[:32], small) <= TOL


def test_gemm_form_integer_exact(dev):
    """Integer-valued x, scales 1 and integer biases: every product and sum is exact in fp16/fp32."""
    rng = np.random.default_rng(5)
    M, N, K = 96, 192, 128
    w = rng.integers(0, 1 << 32, size=(N, K // 8), dtype=np.uint32)
    s = np.ones((N, K // 64), np.float16)
    b = rng.integers(-8, 1, (N, K // 64)).astype(np.float16)
    x = rng.integers(-2, 3, (M, K)).astype(np.float16)
    q = synth.unpack_nibbles(w).astype(np.int64)
    wd = q + np.repeat(b.astype(np.int64), 64, axis=1)
    want = x.astype(np.int64) @ wd.T
    got = ops.quantized_matmul(to_dev(x, dev), to_dev(w, dev), to_dev(s, dev), to_dev(b, dev)).cpu().numpy()
    assert np.array_equal(got.astype(np.int64), want)


def test_gemm_form_rejects_bad_shapes(dev):
    x = torch.zeros((64, 96), dtype=torch.float16, device=dev)
    w = torch.zeros((64, 12), dtype=torch.int32, device=dev)
    s = torch.zeros((64, 1), dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        ops.quantized_matmul(x, w, s, s)


def test_gemm_form_random_shapes(dev):
    """Seeded sweep: ragged row counts, N down to one tile, K with and without the vector
    scale loads (multiples of 512 or not), every block shape."""
    rng = np.random.default_rng(99)
    for case in range(14):
        M = int(rng.integers(1, 700))
        N = 8 * int(rng.integers(1, 700))
        K = 64 * int(rng.integers(1, 40))
        bias = bool(rng.integers(0, 2))
        print(f"case {case}: M={M} N={N} K={K} bias={bias}", flush=True)
        layer = synth.make_qlinear(rng, N, K, bias=bias)
        x = synth.make_x(rng, M, K)
        want = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"], layer.get("bias"))
        d = layer_to_dev(layer, dev)
        out = torch.full((M + 1, N), float("nan"), dtype=torch.float16, device=dev)
        ops.quantized_matmul(to_dev(x, dev), d["weight"], d["scales"], d["biases"], bias=d.get("bias"),
                             out=out[:M], gemm=True)
        got = out.cpu().numpy()
        assert np.isnan(got[M].astype(np.float32)).all(), case          # nothing written past the rows
        assert np.isfinite(got[:M].astype(np.float32)).all(), case
        assert rel_err(got[:M], want) <= TOL, case


@pytest.mark.parametrize("M,I,K,bias", [(33, 16, 64, True), (64, 48, 128, False), (100, 272, 256, True),
                                        (512, 2432, 896, False), (300, 1024, 1024, True), (129, 14336, 4096, False)])
def test_gemm_form_with_swiglu(dev, M, I, K, bias):
    """gate|up of a prompt chunk with the activation in the GEMM's epilogue (tile-interleaved rows):
    equal, bit for bit, to the GEMM over the concatenated rows followed by silu_mul wherever both
    pick the same block shape, within tolerance of the oracle's qmm -> silu_mul always."""
    print(f"gemm swiglu M={M} I={I} K={K}", flush=True)
    rng = np.random.default_rng(M + I + K)
    g = synth.make_qlinear(rng, I, K, bias=bias, gain=1.0)
    u = synth.make_qlinear(rng, I, K, bias=bias, gain=1.0)
    x = synth.make_x(rng, M, K)
    rows = rng.choice(M, size=min(M, 40), replace=False)             # the oracle on a sample of the rows
    og = oracle.qmm(x[rows], g["weight"], g["scales"], g["biases"], g.get("bias"))
    ou = oracle.qmm(x[rows], u["weight"], u["scales"], u["biases"], u.get("bias"))
    want = oracle.silu_mul(og, ou)
    gd, ud = layer_to_dev(g, dev), layer_to_dev(u, dev)
    keys = ["weight", "scales", "biases"] + (["bias"] if bias else [])
    inter = {k: ops.interleave_gate_up(gd[k], ud[k]) for k in keys}
    cat = {k: torch.cat([gd[k], ud[k]]).contiguous() for k in keys}
    xd = to_dev(x, dev)
    got = ops.quantized_matmul_swiglu(xd, inter["weight"], inter["scales"], inter["biases"], bias=inter.get("bias"),
                                      gemm=True)
    two = ops.silu_mul(ops.quantized_matmul(xd, cat["weight"], cat["scales"], cat["biases"], bias=cat.get("bias"),
                                            gemm=True))
    torch.cuda.synchronize()
    assert tuple(got.shape) == (M, I)
    # Against the oracle: each projection is within TOL of its own RMS (the bound of the plain form);
    # through silu(g) * u an error dg moves the result by u silu'(g) dg (|silu'| <= 1.1) and du by
    # silu(g) du, plus the two fp16 roundings of the epilogue.  The RMS error stays a fraction of TOL.
    g64, u64 = og.astype(np.float64), ou.astype(np.float64)
    rms_g, rms_u = np.sqrt(np.mean(g64 * g64)), np.sqrt(np.mean(u64 * u64))
    w64, got64 = want.astype(np.float64), got.cpu().numpy()[rows].astype(np.float64)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(w64), 2.0 ** -14))) - 10)
    bound = TOL * (1.1 * np.abs(u64) * rms_g + np.abs(g64 / (1 + np.exp(-g64))) * rms_u) + 2 * ulp
    assert np.all(np.abs(got64 - w64) <= bound)
    assert np.sqrt(np.mean((got64 - w64) ** 2)) <= 0.25 * TOL * np.sqrt(np.mean(w64 * w64))
    # against the plain form followed by silu_mul (same roundings, possibly another block shape)
    close_fp16(got.cpu().numpy(), two.cpu().numpy(), "two launches")
    with pytest.raises(Exception):
        ops.quantized_matmul_swiglu(xd, inter["weight"][:24], inter["scales"][:24], inter["biases"][:24])
