"""The tiled weight layout (`ops.tile_weights`) and the slab products that read it, through the
C ABI: the re-layout against a numpy statement of it, the partial sums against the row-major form
(bit for bit: same arithmetic, different addresses) and the oracle, the expansion through fp16
subnormals against fp16(s q + b), and gate|up + SwiGLU against the oracle."""
import numpy as np
import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import _lib, ops, synth
from oracle import oracle
from util import TOL, close_fp16, layer_to_dev, rel_err, to_dev

pytestmark = pytest.mark.gpu


def tile_numpy(w, s, b):
    """wt[tile][group][lane] = words 4 (lane / 32) .. + 3 of the group for row 32 tile + lane % 32;
    sbt[tile][chunk][lane] = eight scales (lanes 0..31) or biases (32..63) of that row."""
    N, KW = w.shape
    G = KW // 8
    wt = w.reshape(N // 32, 32, G, 2, 4).transpose(0, 2, 3, 1, 4).reshape(N // 32, G, 64, 4)
    s8 = s.reshape(N // 32, 32, G // 8, 8).transpose(0, 2, 1, 3)
    b8 = b.reshape(N // 32, 32, G // 8, 8).transpose(0, 2, 1, 3)
    return np.ascontiguousarray(wt), np.ascontiguousarray(np.concatenate([s8, b8], axis=2))


@pytest.mark.parametrize("N,K", [(32, 512), (4608, 3584), (3584, 18944), (96, 1024)])
def test_layout(dev, N, K):
    rng = np.random.default_rng(N + K)
    layer = synth.make_qlinear(rng, N, K)
    d = layer_to_dev(layer, dev)
    t = ops.tile_weights(d["weight"], d["scales"], d["biases"])
    wt, sbt = tile_numpy(layer["weight"], layer["scales"], layer["biases"])
    assert np.array_equal(t.wt.cpu().numpy().view(np.uint32), wt)
    assert np.array_equal(t.sbt.cpu().numpy(), sbt)
    assert t.small and (t.N, t.K) == (N, K)


@pytest.mark.parametrize("M,N,K,steps", [(32, 4608, 3584, 8), (32, 3584, 3584, 8), (32, 3584, 18944, 32),
                                         (17, 96, 1536, 8), (1, 128, 1024, 16), (24, 4096, 14336, 32),
                                         (8, 6144, 4096, 8), (32, 160, 512, 8),
                                         # 33..64 rows: 64-row partial tiles
                                         (40, 4608, 3584, 8), (64, 3584, 18944, 32), (33, 96, 1024, 8)])
def test_partial_sums(dev, M, N, K, steps):
    print(f"tiled slab M={M} N={N} K={K} steps={steps}", flush=True)
    rng = np.random.default_rng(M + N + K)
    layer = synth.make_qlinear(rng, N, K)
    x = synth.make_x(rng, M, K)
    want = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"])
    d = layer_to_dev(layer, dev)
    xd = to_dev(x, dev)
    slabs = ops.slab_count(K, steps)
    t = ops.tile_weights(d["weight"], d["scales"], d["biases"])
    plain = ops.quantized_matmul_slabs(xd, d["weight"], d["scales"], d["biases"], steps)
    for small in (False, True):
        t.small = small
        part = torch.full((slabs, ops.slab_rows(M), N), float("nan"), dtype=torch.float32, device=dev)
        ops.quantized_matmul_slabs(xd, d["weight"], d["scales"], d["biases"], steps, partial=part, tiled=t)
        assert torch.isfinite(part[:, :M]).all() and torch.isnan(part[:, M:]).all()
        if not small:
            assert torch.equal(part[:, :M], plain[:, :M]), "same arithmetic as the row-major form"
        got = ops.slab_sum(part, slabs, M, N)
        assert rel_err(got.cpu().numpy(), want) <= TOL, f"small_scales={small}"


def test_subnormal_expansion_is_one_rounding(dev):
    """One-hot x rows give the dequantised weight column: with small scales exactly
    fp16(s q + b), a single rounding (pins the nibble order of the tiled layout and the
    expansion)."""
    rng = np.random.default_rng(11)
    N, K, M = 160, 1024, 32
    layer = synth.make_qlinear(rng, N, K)
    d = layer_to_dev(layer, dev)
    t = ops.tile_weights(d["weight"], d["scales"], d["biases"])
    assert t.small
    cols = rng.choice(K, size=M, replace=False)
    x = np.zeros((M, K), np.float16)
    x[np.arange(M), cols] = 1.0
    part = ops.quantized_matmul_slabs(to_dev(x, dev), d["weight"], d["scales"], d["biases"], 16, tiled=t)
    got = ops.slab_sum(part, ops.slab_count(K, 16), M, N).cpu().numpy()
    qv = synth.unpack_nibbles(layer["weight"])[:, cols].astype(np.float32)
    s = layer["scales"].astype(np.float32)[:, cols // 64]
    b = layer["biases"].astype(np.float32)[:, cols // 64]
    assert np.array_equal(got, (s * qv + b).astype(np.float16).T)


def test_large_scales_take_the_other_expansion(dev):
    rng = np.random.default_rng(12)
    N, K, M = 64, 512, 8
    layer = synth.make_qlinear(rng, N, K)
    layer["scales"][3, 2] = np.float16(0.07)
    d = layer_to_dev(layer, dev)
    t = ops.tile_weights(d["weight"], d["scales"], d["biases"])
    assert not t.small
    x = synth.make_x(rng, M, K)
    part = ops.quantized_matmul_slabs(to_dev(x, dev), d["weight"], d["scales"], d["biases"], 8, tiled=t)
    got = ops.slab_sum(part, 1, M, N).cpu().numpy()
    assert rel_err(got, oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"])) <= TOL


@pytest.mark.parametrize("M,I,K,bias", [(32, 18944, 3584, True), (32, 14336, 4096, False), (8, 4864, 1024, True),
                                        (1, 64, 512, False), (27, 272, 1536, True), (40, 18944, 3584, True),
                                        (64, 14336, 4096, False), (47, 272, 1536, True)])
def test_swiglu(dev, M, I, K, bias):
    print(f"tiled swiglu M={M} I={I} K={K}", flush=True)
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
    t = ops.tile_weights(inter["weight"], inter["scales"], inter["biases"])
    xd = to_dev(x, dev)
    plain = ops.quantized_matmul_swiglu_slab(xd, inter["weight"], inter["scales"], inter["biases"],
                                             bias=inter.get("bias"))
    for small in (False, True):
        t.small = small
        out = torch.full((M + 1, I), float("nan"), dtype=torch.float16, device=dev)
        ops.quantized_matmul_swiglu(xd, inter["weight"], inter["scales"], inter["biases"], bias=inter.get("bias"),
                                    out=out[:M], tiled=t)
        got = out.cpu().numpy()
        assert np.isnan(got[M].astype(np.float32)).all()
        if not small and (K not in (3584, 4096) or M > 32):
            # (those two K sizes run two waves per weight tile, which add their halves of K at the end)
            assert torch.equal(out[:M], plain)
        else:
            close_fp16(got[:M], plain.cpu().numpy(), "against the row-major form")
        g64, u64 = og.astype(np.float64), ou.astype(np.float64)
        rms_g, rms_u = np.sqrt(np.mean(g64 * g64)), np.sqrt(np.mean(u64 * u64))
        w64, got64 = want.astype(np.float64), got[:M].astype(np.float64)
        ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(w64), 2.0 ** -14))) - 10)
        bound = TOL * (1.1 * np.abs(u64) * rms_g + np.abs(g64 / (1 + np.exp(-g64))) * rms_u) + 2 * ulp
        assert np.all(np.abs(got64 - w64) <= bound), f"small_scales={small}"
        assert np.sqrt(np.mean((got64 - w64) ** 2)) <= 0.25 * TOL * np.sqrt(np.mean(w64 * w64))


def test_refusals(dev):
    L = _lib.lib()
    assert L.eagle_qmm_tiled_supported(64, 4608, 3584) == 1 and L.eagle_qmm_tiled_supported(65, 4608, 3584) == 0
    assert L.eagle_qmm_tiled_supported(8, 1152, 896) == 0 and L.eagle_qmm_tiled_supported(8, 48, 512) == 0
    assert L.eagle_qmm_tiled_sb_bytes(4608, 3584) == 4608 * 56 * 4 and L.eagle_qmm_tiled_sb_bytes(48, 512) == 0
    rng = np.random.default_rng(1)
    layer = synth.make_qlinear(rng, 48, 512)
    d = layer_to_dev(layer, dev)
    with pytest.raises(ValueError):
        ops.tile_weights(d["weight"], d["scales"], d["biases"])
    layer = synth.make_qlinear(rng, 64, 512)
    d = layer_to_dev(layer, dev)
    t = ops.tile_weights(d["weight"], d["scales"], d["biases"])
    x = torch.zeros((8, 1024), dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        ops.quantized_matmul_slabs(x, d["weight"], d["scales"], d["biases"], 8, tiled=t)


@pytest.mark.parametrize("M,N,K,bias", [(32, 20 * 32 * 2 + 96, 1024, True), (8, 640, 512, False), (1, 32, 512, True),
                                        (31, 16 * 32 + 32, 1536, False), (32, 152064, 3584, False),
                                        (32, 128256, 4096, False), (8, 152064, 3584, True)])
def test_whole_product_from_the_tiled_layout(dev, M, N, K, bias):
    """`quantized_matmul_tiled` (the vocabulary projection's form: whole K per workgroup, fp16 out)
    against the oracle, with both expansions; workgroups with fewer tiles than they own and rows
    beyond M must leave the rest of `out` alone."""
    print(f"tiled whole product M={M} N={N} K={K} bias={bias}", flush=True)
    rng = np.random.default_rng(M + N + K)
    layer = synth.make_qlinear(rng, N, K, bias=bias)
    x = synth.make_x(rng, M, K)
    want = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"], layer.get("bias"))
    d = layer_to_dev(layer, dev)
    t = ops.tile_weights(d["weight"], d["scales"], d["biases"])
    assert ops.rows_tiled_supported(M, N, K)
    for small in (True, False):
        t.small = small
        out = torch.full((M + 1, N), float("nan"), dtype=torch.float16, device=dev)
        ops.quantized_matmul_tiled(to_dev(x, dev), t, bias=d.get("bias"), out=out[:M])
        torch.cuda.synchronize()
        assert torch.isnan(out[M:]).all()
        assert rel_err(out[:M].cpu().numpy(), want) <= TOL, f"small={small}"


def test_whole_product_one_hot_and_two_passes(dev):
    """One-hot rows give fp16(s q + b) exactly (nibble order and single rounding of this kernel's
    expansion); 40 rows run as two passes and agree with the oracle."""
    rng = np.random.default_rng(21)
    N, K, M = 672, 1024, 32
    layer = synth.make_qlinear(rng, N, K)
    d = layer_to_dev(layer, dev)
    t = ops.tile_weights(d["weight"], d["scales"], d["biases"])
    assert t.small
    cols = rng.choice(K, size=M, replace=False)
    x = np.zeros((M, K), np.float16)
    x[np.arange(M), cols] = 1.0
    got = ops.quantized_matmul_tiled(to_dev(x, dev), t).cpu().numpy()
    qv = synth.unpack_nibbles(layer["weight"])[:, cols].astype(np.float32)
    s = layer["scales"].astype(np.float32)[:, cols // 64]
    b = layer["biases"].astype(np.float32)[:, cols // 64]
    assert np.array_equal(got, (s * qv + b).astype(np.float16).T)
    x = synth.make_x(rng, 40, K)
    got = ops.quantized_matmul_tiled(to_dev(x, dev), t).cpu().numpy()
    assert rel_err(got, oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"])) <= TOL


def test_whole_product_refusals(dev):
    L = _lib.lib()
    assert L.eagle_qmm_rows_tiled_supported(32, 152064, 3584) == 1
    assert L.eagle_qmm_rows_tiled_supported(33, 152064, 3584) == 0
    assert L.eagle_qmm_rows_tiled_supported(8, 152064, 896) == 0 and L.eagle_qmm_rows_tiled_supported(8, 48, 512) == 0
    rng = np.random.default_rng(2)
    layer = synth.make_qlinear(rng, 64, 512)
    d = layer_to_dev(layer, dev)
    t = ops.tile_weights(d["weight"], d["scales"], d["biases"])
    with pytest.raises(ValueError):
        ops.quantized_matmul_tiled(torch.zeros((8, 1024), dtype=torch.float16, device=dev), t)
    with pytest.raises(ValueError):
        ops.quantized_matmul_tiled(torch.zeros((65, 512), dtype=torch.float16, device=dev), t)
    x = torch.zeros((8, 512), dtype=torch.float16, device=dev)
    assert L.eagle_qmm_rows_tiled_w4g64_f16(x.data_ptr(), t.wt.data_ptr(), t.sbt.data_ptr(), None, x.data_ptr(),
                                            8, 64, 512, 1, None) == 4          # in place
    assert L.eagle_qmm_rows_tiled_w4g64_f16(x.data_ptr(), None, t.sbt.data_ptr(), None, x.data_ptr(),
                                            8, 64, 512, 1, None) == 1
