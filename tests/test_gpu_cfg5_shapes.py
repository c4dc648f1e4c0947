"""Parity at the shapes of the fifth benchmark configuration (mlx_eagle.py:620-681: a
Qwen2.5-0.5B-shaped drafter under a Llama-3-8B-shaped target), through the C ABI:
every projection of the target at 8 and 32 rows in the streaming, slab and SwiGLU forms, every
projection of the drafter at 8 rows through the small-row forms it runs in the loop, and one
decoder layer of each width against the oracle's tree forward."""
import numpy as np
import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import ops, synth
from oracle import model_oracle, oracle, tree_oracle
from test_gpu_fullsize import run_verifier, setup_step
from util import TOL, close_fp16, layer_to_dev, rel_err, to_dev

pytestmark = pytest.mark.gpu

EPS = 1e-5

# (name, N, K) of the Llama-3-8B-shaped target: q|k|v fused, o, down, the vocabulary projection
TARGET = [("qkv", 6144, 4096), ("o", 4096, 4096), ("down", 4096, 14336), ("lm_head", 128256, 4096)]
# the drafter (hidden 896, 14 / 2 heads of 64, intermediate 4864): q|k|v fused, o, down, the tied head
DRAFTER = [("qkv", 1152, 896), ("o", 896, 896), ("down", 896, 4864), ("head", 152064, 896)]


def q(x, L):
    return oracle.qmm(x, L["weight"], L["scales"], L["biases"], L.get("bias"))


@pytest.mark.parametrize("name,N,K", TARGET)
def test_target_projections(dev, name, N, K):
    rng = np.random.default_rng(N + K)
    layer = synth.make_qlinear(rng, N, K)
    d = layer_to_dev(layer, dev)
    for M in (8, 32):
        print(f"cfg5 target {name} {K}->{N} M={M}", flush=True)
        x = synth.make_x(rng, M, K)
        xd = to_dev(x, dev)
        want = q(x, layer)
        got = ops.quantized_matmul(xd, d["weight"], d["scales"], d["biases"])
        torch.cuda.synchronize()
        assert rel_err(got.cpu().numpy(), want) <= TOL, f"streaming form {name} M={M}"
        s = ops.slab_steps(M, N, K)
        assert bool(s) == (name != "lm_head")
        if s:
            part = ops.quantized_matmul_slabs(xd, d["weight"], d["scales"], d["biases"], s)
            got = ops.slab_sum(part, ops.slab_count(K, s), M, N)
            torch.cuda.synchronize()
            assert rel_err(got.cpu().numpy(), want) <= TOL, f"slab form {name} M={M}"


def test_target_gate_up_with_swiglu(dev):
    """4096 -> 2 x 14336 with the SwiGLU epilogue: the form the library picks and the slab form."""
    I, K = 14336, 4096
    rng = np.random.default_rng(5)
    g = synth.make_qlinear(rng, I, K, gain=1.0)
    u = synth.make_qlinear(rng, I, K, gain=1.0)
    gd, ud = layer_to_dev(g, dev), layer_to_dev(u, dev)
    inter = {k: ops.interleave_gate_up(gd[k], ud[k]) for k in ("weight", "scales", "biases")}
    for M in (8, 32):
        print(f"cfg5 target gate|up M={M}", flush=True)
        x = synth.make_x(rng, M, K)
        xd = to_dev(x, dev)
        want = oracle.silu_mul(q(x, g), q(x, u))
        got = ops.quantized_matmul_swiglu(xd, inter["weight"], inter["scales"], inter["biases"])
        torch.cuda.synchronize()
        close_fp16(got.cpu().numpy(), want, f"library's choice, M={M}")
        got = ops.quantized_matmul_swiglu_slab(xd, inter["weight"], inter["scales"], inter["biases"])
        torch.cuda.synchronize()
        close_fp16(got.cpu().numpy(), want, f"slab form, M={M}")


@pytest.mark.parametrize("name,N,K", DRAFTER)
def test_drafter_projections(dev, name, N, K):
    """8 rows, as the drafter's passes run them: the streaming kernel for the tied head, the
    small-row kernel with the norm in its load (q|k|v) or the residual in its store (o, down)."""
    rng = np.random.default_rng(N + K)
    M = 8
    layer = synth.make_qlinear(rng, N, K, bias=(name == "qkv"), gain=1.0)
    d = layer_to_dev(layer, dev)
    x = synth.make_x(rng, M, K)
    xd = to_dev(x, dev)
    print(f"cfg5 drafter {name} {K}->{N}", flush=True)
    got = ops.quantized_matmul(xd, d["weight"], d["scales"], d["biases"], bias=d.get("bias"))
    torch.cuda.synchronize()
    assert rel_err(got.cpu().numpy(), q(x, layer)) <= TOL
    if name == "head":
        return
    assert ops.small_supported(M, N, K)
    if name == "qkv":
        nw = (1.0 + rng.normal(0, 0.1, K)).astype(np.float16)
        got = ops.quantized_matmul_small(xd, d["weight"], d["scales"], d["biases"], bias=d["bias"],
                                         norm_weight=to_dev(nw, dev), eps=EPS)
        want = q(oracle.rmsnorm(x, nw, EPS), layer)
    else:
        r = synth.make_x(rng, M, N)
        got = ops.quantized_matmul_small(xd, d["weight"], d["scales"], d["biases"], residual=to_dev(r, dev))
        want = oracle.add(r, q(x, layer))
    torch.cuda.synchronize()
    close_fp16(got.cpu().numpy(), want, name)


def test_drafter_gate_up_with_norm_and_swiglu(dev):
    I, K, M = 4864, 896, 8
    rng = np.random.default_rng(9)
    g = synth.make_qlinear(rng, I, K, gain=1.0)
    u = synth.make_qlinear(rng, I, K, gain=1.0)
    gd, ud = layer_to_dev(g, dev), layer_to_dev(u, dev)
    inter = {k: ops.interleave_gate_up(gd[k], ud[k]) for k in ("weight", "scales", "biases")}
    x = synth.make_x(rng, M, K)
    nw = (1.0 + rng.normal(0, 0.1, K)).astype(np.float16)
    xn = oracle.rmsnorm(x, nw, EPS)
    want = oracle.silu_mul(q(xn, g), q(xn, u))
    got = ops.quantized_matmul_small(to_dev(x, dev), inter["weight"], inter["scales"], inter["biases"],
                                     swiglu=True, norm_weight=to_dev(nw, dev), eps=EPS)
    torch.cuda.synchronize()
    close_fp16(got.cpu().numpy(), want)


@pytest.mark.parametrize("shape", ["llama3_8b", "qwen25_05b"])
def test_one_layer_at_cfg5_widths(dev, shape):
    """One decoder layer of the target's width (4096, 32 / 8 heads of 128, theta 5e5, 32 tree rows
    behind a 512-token prefix) and of the drafter's (896, 14 / 2 heads of 64, q|k|v biases, tied
    head, 8 rows): residual stream, appended K / V rows and logits against the oracle."""
    args = getattr(synth, shape)()
    P, T = 512, (32 if shape == "llama3_8b" else 8)
    s = setup_step(dev, args, 1, 21, P, T)
    mask = np.concatenate([np.zeros((T, P), np.float16), tree_oracle.additive_mask(s["anc"])], axis=1)
    want_h = {}
    want = model_oracle.tree_forward(s["args"], s["weights"], s["inv"], s["sc"], s["tokens"], s["depth"] + P,
                                     mask, s["ocache"], P, tap=lambda i, h: want_h.__setitem__(i + 1, h.copy()))
    ok, ov = s["ocache"][0]
    print(f"{shape}-width layer", flush=True)
    ver, hid = run_verifier(dev, s, None, taps={1})
    assert rel_err(hid[1], want_h[1]) <= TOL
    c = s["cache"][0]
    assert rel_err(c.keys[0, :, P:P + T].cpu().numpy(), ok[:, P:P + T]) <= TOL
    assert rel_err(c.values[0, :, P:P + T].cpu().numpy(), ov[:, P:P + T]) <= TOL
    assert rel_err(ver.logits.cpu().numpy(), want) <= TOL
