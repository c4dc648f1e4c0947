"""HIP quantised matmul vs the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import _lib, ops, synth
from oracle import oracle
from util import TOL, layer_to_dev, rel_err, to_dev

pytestmark = pytest.mark.gpu


def shape_for(M, N, K, nw, phases, ranges, wide=False):
    """A forced launch shape: `nw` streaming waves per workgroup, each owning `phases` column
    units in turn (the K slabs follow from both), `ranges` workgroups per slab, `wide`:
    256-column units at M > 16; None if it cannot be launched."""
    wide = wide and M > 16
    cw = 256 if M <= 16 or wide else 128
    nt = 1 if M <= 16 else 2
    units = -(-K // cw)
    per_slab = nw * phases
    splits = -(-units // per_slab)
    tiles = -(-N // 16)
    if nw > (10 if wide else 14) or phases > 8 or per_slab * (splits - 1) >= units or ranges > tiles or splits > 64:
        return None
    lds = 2 * nw * 4096 + (32768 if nt == 1 else (16384 if wide else 8192))
    if phases > 1:
        lds += -(-(-(-tiles // ranges)) // 4) * 4 * nt * 1024
    if lds > 160 * 1024:
        return None
    return (nw, phases, splits, ranges, cw)


def run_case(dev, M, N, K, seed=0, bias=False, tuned=None):
    rng = np.random.default_rng(seed)
    layer = synth.make_qlinear(rng, N, K, bias=bias)
    x = synth.make_x(rng, M, K)
    want = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"], layer.get("bias"))
    d = layer_to_dev(layer, dev)
    got = ops.quantized_matmul(to_dev(x, dev), d["weight"], d["scales"], d["biases"],
                               bias=d.get("bias"), tuned=tuned)
    torch.cuda.synchronize()
    err = rel_err(got.cpu().numpy(), want)
    assert err <= TOL, f"M={M} N={N} K={K} tuned={tuned}: rel err {err:.3e}"
    return err


@pytest.mark.parametrize("M", [1, 2, 7, 8, 16, 17, 24, 32])
def test_cfg1_shape_all_m(dev, M):
    print(f"qmm cfg1 M={M}", flush=True)
    run_case(dev, M, 8192, 2048, seed=42)


@pytest.mark.parametrize("nw,phases", [(1, 1), (2, 1), (3, 2), (5, 3), (7, 1), (7, 2), (13, 1), (14, 1), (14, 2),
                                       (2, 7), (4, 8)])
@pytest.mark.parametrize("ranges", [1, 7, 96])
@pytest.mark.parametrize("M", [8, 32])
def test_forced_launch_shapes(dev, nw, phases, ranges, M):
    N, K = 1536, 3584
    tuned = shape_for(M, N, K, nw, phases, ranges)
    if tuned is None:
        pytest.skip("shape cannot be launched")
    print(f"qmm tuned={tuned} M={M}", flush=True)
    run_case(dev, M, N, K, seed=nw * 100 + ranges + phases, tuned=tuned)


@pytest.mark.parametrize("nw,phases", [(1, 1), (2, 1), (3, 2), (5, 3), (7, 1), (7, 2), (10, 1), (10, 2), (4, 4)])
@pytest.mark.parametrize("ranges", [1, 7, 96])
@pytest.mark.parametrize("M", [17, 32])
def test_forced_launch_shapes_wide_units(dev, nw, phases, ranges, M):
    """M > 16 with 256-column units (the form picked for K > 3584 and for very many tiles)."""
    N, K = 1536, 3584
    tuned = shape_for(M, N, K, nw, phases, ranges, wide=True)
    if tuned is None:
        pytest.skip("shape cannot be launched")
    print(f"qmm tuned={tuned} M={M}", flush=True)
    run_case(dev, M, N, K, seed=nw * 100 + ranges + phases, tuned=tuned, bias=(nw & 1) == 1)


@pytest.mark.parametrize("N,K", [(8, 64), (8, 128), (24, 192), (40, 896), (136, 2944), (512, 3584),
                                 (64, 18944)])
def test_edge_shapes(dev, N, K):
    for M in (1, 5, 32):
        print(f"qmm edge N={N} K={K} M={M}", flush=True)
        run_case(dev, M, N, K, seed=N + K + M)
        for cfg in ((1, 1, 1), (3, 2, 2), (14, 1, 3), (2, 3, 1)):
            for wide in (False, True):
                tuned = shape_for(M, N, K, *cfg, wide=wide)
                if tuned is not None and (wide is False or M > 16):
                    run_case(dev, M, N, K, seed=N + K + M, tuned=tuned)


def test_bias_and_leading_dims(dev):
    rng = np.random.default_rng(3)
    layer = synth.make_qlinear(rng, 512, 896, bias=True)
    x = synth.make_x(rng, 1, 8, 896)
    want = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"], layer["bias"])
    d = layer_to_dev(layer, dev)
    got = ops.quantized_matmul(to_dev(x, dev), d["weight"], d["scales"], d["biases"], bias=d["bias"])
    assert tuple(got.shape) == (1, 8, 512)
    assert rel_err(got.cpu().numpy(), want) <= TOL
    lst = ops.matmul(to_dev(x, dev), d["weight"], d["scales"], d["biases"], 64)
    assert isinstance(lst, list) and len(lst) == 1


def test_one_hot_rows_reproduce_dequantised_columns(dev):
    """x = e_k picks column k of dequant(W): pins nibble order and group indexing exactly."""
    rng = np.random.default_rng(5)
    N, K = 64, 256
    layer = synth.make_qlinear(rng, N, K)
    wd = synth.dequantize(layer, np.float32)
    d = layer_to_dev(layer, dev)
    for k0 in range(0, K, 32):
        x = np.zeros((32, K), np.float16)
        for m in range(32):
            x[m, k0 + m] = 1.0
        got = ops.quantized_matmul(to_dev(x, dev), d["weight"], d["scales"], d["biases"]).cpu().numpy()
        want = wd[:, k0:k0 + 32].T.astype(np.float16)
        np.testing.assert_allclose(got.astype(np.float32), want.astype(np.float32), rtol=0, atol=2e-3)


def test_deterministic_split_k(dev):
    rng = np.random.default_rng(9)
    layer = synth.make_qlinear(rng, 512, 3584)
    x = to_dev(synth.make_x(rng, 32, 3584), dev)
    d = layer_to_dev(layer, dev)
    tuned = shape_for(32, 512, 3584, 2, 2, 5)
    assert tuned[2] == 7
    ref = ops.quantized_matmul(x, d["weight"], d["scales"], d["biases"], tuned=tuned)
    for _ in range(5):
        again = ops.quantized_matmul(x, d["weight"], d["scales"], d["biases"], tuned=tuned)
        assert torch.equal(ref, again)


def test_plan_covers_benchmark_shapes(dev):
    for M in (1, 8, 16, 24, 32):
        for N, K in ((3584, 3584), (512, 3584), (18944, 3584), (3584, 18944), (152064, 3584),
                     (8192, 2048), (896, 896), (128, 896), (4864, 896), (896, 4864),
                     (4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336), (128256, 4096)):
            nw, phases, splits, ranges, cw = ops.qmm_plan(M, N, K)
            assert cw == 256 if M <= 16 else cw in (128, 256)
            assert nw * phases * splits * cw >= K > nw * phases * (splits - 1) * cw
            assert 1 <= nw <= (14 if M <= 16 or cw == 128 else 10) and 1 <= ranges <= -(-N // 16)


def test_argument_errors(dev):
    x = torch.zeros(33, 128, dtype=torch.float16, device=dev)
    w = torch.zeros(8, 16, dtype=torch.int32, device=dev)
    s = torch.zeros(8, 2, dtype=torch.float16, device=dev)
    # more than 32 rows go to the tiled GEMM form; the streaming kernel itself refuses them
    assert tuple(ops.quantized_matmul(x, w, s, s).shape) == (33, 8)
    with pytest.raises(ValueError):
        ops.quantized_matmul(x, w, s, s, tuned=(1, 1, 1, 1))
    with pytest.raises(ValueError):
        ops.quantized_matmul(x[:8], w, s, s, group_size=32)
    with pytest.raises(ValueError):
        ops.quantized_matmul(x[:8], w, s, s, bits=8)


@pytest.mark.parametrize("I,K,bias", [(16, 64, False), (48, 128, True), (272, 256, True), (4864, 896, False),
                                      (18944, 3584, True), (1024, 7168, False)])
def test_swiglu_form_equals_separate_launches(dev, I, K, bias):
    """gate|up in tile-interleaved rows with the activation in the matmul's epilogue: bit-identical
    to the concatenated launch followed by silu_mul (same launch shape, so the same fp32 sums), and
    within tolerance of the oracle's qmm -> silu_mul."""
    for M in (1, 8, 16, 17, 32):
        if not ops.swiglu_supported(M, I, K):
            continue
        print(f"qmm swiglu I={I} K={K} M={M}", flush=True)
        rng = np.random.default_rng(I + K + M)
        g = synth.make_qlinear(rng, I, K, bias=bias, gain=1.0)
        u = synth.make_qlinear(rng, I, K, bias=bias, gain=1.0)
        x = synth.make_x(rng, M, K)
        want = oracle.silu_mul(oracle.qmm(x, g["weight"], g["scales"], g["biases"], g.get("bias")),
                               oracle.qmm(x, u["weight"], u["scales"], u["biases"], u.get("bias")))
        gd, ud = layer_to_dev(g, dev), layer_to_dev(u, dev)
        keys = ["weight", "scales", "biases"] + (["bias"] if bias else [])
        inter = {k: ops.interleave_gate_up(gd[k], ud[k]) for k in keys}
        cat = {k: torch.cat([gd[k], ud[k]]).contiguous() for k in keys}
        xd = to_dev(x, dev)
        got = ops.quantized_matmul_swiglu(xd, inter["weight"], inter["scales"], inter["biases"],
                                          bias=inter.get("bias"))
        two = ops.silu_mul(ops.quantized_matmul(xd, cat["weight"], cat["scales"], cat["biases"],
                                                bias=cat.get("bias")))
        torch.cuda.synchronize()
        assert tuple(got.shape) == (M, I)
        if M == 1 and ops.qmv_preferred(2 * I, K):
            # one row of the concatenated launch goes to the vector-ALU kernel (another order
            # of the fp32 sums): the tolerance applies, not bit equality
            assert rel_err(got.cpu().numpy(), two.cpu().numpy().astype(np.float64)) <= TOL
        else:
            assert torch.equal(got, two), f"I={I} K={K} M={M}: swiglu form differs from matmul + silu_mul"
        assert rel_err(got.cpu().numpy(), want) <= TOL


def test_swiglu_form_with_k_slabs(dev):
    """Shapes whose launch uses K slabs: the last workgroup of a tile range applies the activation."""
    rng = np.random.default_rng(1)
    for M, I, K in ((8, 32, 8192), (32, 48, 7168), (17, 1024, 3584)):
        assert ops.qmm_plan(M, 2 * I, K)[2] > 1
        g = synth.make_qlinear(rng, I, K, bias=True, gain=1.0)
        u = synth.make_qlinear(rng, I, K, bias=True, gain=1.0)
        x = synth.make_x(rng, M, K)
        want = oracle.silu_mul(oracle.qmm(x, g["weight"], g["scales"], g["biases"], g["bias"]),
                               oracle.qmm(x, u["weight"], u["scales"], u["biases"], u["bias"]))
        gd, ud = layer_to_dev(g, dev), layer_to_dev(u, dev)
        inter = {k: ops.interleave_gate_up(gd[k], ud[k]) for k in ("weight", "scales", "biases", "bias")}
        cat = {k: torch.cat([gd[k], ud[k]]).contiguous() for k in ("weight", "scales", "biases", "bias")}
        xd = to_dev(x, dev)
        got = ops.quantized_matmul_swiglu(xd, inter["weight"], inter["scales"], inter["biases"], bias=inter["bias"])
        two = ops.silu_mul(ops.quantized_matmul(xd, cat["weight"], cat["scales"], cat["biases"], bias=cat["bias"]))
        torch.cuda.synchronize()
        assert torch.equal(got, two), f"M={M} I={I} K={K}"
        assert rel_err(got.cpu().numpy(), want) <= TOL


@pytest.mark.parametrize("N,K", [(3584, 3584), (512, 3584), (8192, 2048), (40, 512), (136, 4096)])
@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8])
def test_vector_alu_rows(dev, M, N, K):
    """The vector-ALU kernel for 1..8 rows of x (the expanded nibbles of a packed word shared by
    the rows) against the oracle, with a bias; rows past M are neither read nor written."""
    rng = np.random.default_rng(M * 7 + N + K)
    layer = synth.make_qlinear(rng, N, K, bias=True)
    x = synth.make_x(rng, M, K)
    want = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"], layer["bias"])
    d = layer_to_dev(layer, dev)
    out = torch.full((M + 1, N), float("nan"), dtype=torch.float16, device=dev)
    ops.quantized_matvec(to_dev(x, dev), d["weight"], d["scales"], d["biases"], bias=d["bias"], out=out[:M])
    got = out.cpu().numpy()
    assert np.isnan(got[M].astype(np.float32)).all()
    assert rel_err(got[:M], want) <= TOL


def test_vector_alu_rows_refusals(dev):
    from mlx_eagle_spec_decoding_tree_amd import _lib
    L = _lib.lib()
    assert L.eagle_qmv_rows_supported(8, 3584, 3584) == 1 and L.eagle_qmv_rows_supported(9, 3584, 3584) == 0
    assert L.eagle_qmv_rows_supported(1, 3584, 18944) == 1 and L.eagle_qmv_rows_supported(4, 3584, 18944) == 0   # x beyond LDS
    assert L.eagle_qmv_rows_supported(2, 64, 896) == 0
