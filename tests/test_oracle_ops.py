"""Pins the float oracle (oracle/eagle_oracle.c) against closed forms in float64,
known-answer cases and independent library routines (torch, transformers).  CPU only."""
import numpy as np
import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import synth
from oracle import oracle, tree_oracle
from util import TOL, rel_err


# ----------------------------------------------------------------------------- QMM
def qmm_f64(x, layer, bias=None):
    """out[m,n] = sum_k x[m,k] * (s[n,k/64] q[n,k] + b[n,k/64]), q = (w >> 4(k%8)) & 15."""
    wd = synth.dequantize(layer, np.float64)
    out = x.astype(np.float64) @ wd.T
    return out if bias is None else out + bias.astype(np.float64)


@pytest.mark.parametrize("M,N,K", [(1, 8, 64), (2, 8, 128), (8, 64, 896), (32, 128, 2048), (5, 24, 192)])
def test_qmm_closed_form(M, N, K):
    rng = np.random.default_rng(M * N + K)
    layer = synth.make_qlinear(rng, N, K, bias=True)
    x = synth.make_x(rng, M, K)
    got = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"])
    want = qmm_f64(x, layer)
    assert rel_err(got, want) <= 2e-3           # fp32 accumulation + one fp16 rounding
    got_b = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"], layer["bias"])
    assert rel_err(got_b, qmm_f64(x, layer, layer["bias"])) <= 3e-3


def test_qmm_one_hot_pins_nibble_order_and_groups():
    """x = e_k returns column k of the dequantised matrix: a wrong nibble order, word
    order or group index fails here."""
    rng = np.random.default_rng(1)
    N, K = 16, 256
    q = rng.integers(0, 16, size=(N, K)).astype(np.uint8)
    layer = {"weight": synth.pack_nibbles(q),
             "scales": rng.uniform(0.5, 2.0, (N, K // 64)).astype(np.float16),
             "biases": rng.uniform(-1, 1, (N, K // 64)).astype(np.float16)}
    assert np.array_equal(synth.unpack_nibbles(layer["weight"]), q)
    # explicit bit formula for a few entries
    for n, k in [(0, 0), (3, 7), (5, 8), (15, 255), (9, 77)]:
        assert q[n, k] == (int(layer["weight"][n, k // 8]) >> (4 * (k % 8))) & 15
    x = np.eye(K, dtype=np.float16)[:32]
    for k0 in range(0, K, 32):
        xs = np.roll(x, k0, axis=1)
        got = oracle.qmm(xs, layer["weight"], layer["scales"], layer["biases"]).astype(np.float32)
        s = layer["scales"].astype(np.float32)[:, (k0 // 64)]
        b = layer["biases"].astype(np.float32)[:, (k0 // 64)]
        want = (s[None, :] * q[:, k0:k0 + 32].T.astype(np.float32) + b[None, :]).astype(np.float16)
        np.testing.assert_array_equal(got, want.astype(np.float32))


def test_qmm_integer_exact_and_zero_weights():
    rng = np.random.default_rng(2)
    N, K, M = 24, 192, 4
    q = rng.integers(0, 16, size=(N, K)).astype(np.uint8)
    ones = np.ones((N, K // 64), np.float16)
    zeros = np.zeros((N, K // 64), np.float16)
    x = rng.integers(-3, 4, size=(M, K)).astype(np.float16)
    got = oracle.qmm(x, synth.pack_nibbles(q), ones, zeros)
    want = x.astype(np.int64) @ q.T.astype(np.int64)          # s = 1, b = 0: exact integers
    np.testing.assert_array_equal(got.astype(np.int64), want)
    b = rng.uniform(-1, 1, (N, K // 64)).astype(np.float16)
    got0 = oracle.qmm(x, np.zeros((N, K // 8), np.uint32), ones, b)   # q = 0: b * sum_group(x)
    xs = x.astype(np.float64).reshape(M, K // 64, 64).sum(-1)
    assert rel_err(got0, xs @ b.astype(np.float64).T) <= 2e-3


def test_qmm_matches_torch_matmul_on_dequantised_weights():
    rng = np.random.default_rng(3)
    layer = synth.make_qlinear(rng, 256, 3584)
    x = synth.make_x(rng, 8, 3584)
    wd = torch.from_numpy(synth.dequantize(layer, np.float32))
    want = (torch.from_numpy(x.astype(np.float32)) @ wd.T).numpy()
    assert rel_err(oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"]), want) <= 2e-3


def test_qmm_with_rounded_weights_is_the_closed_form_on_fp16_weights():
    """The oracle's second mode (weights rounded to fp16 before the product, as the reference's
    Metal kernel holds them): float64 product over fp16(s q + b); off again after the block."""
    rng = np.random.default_rng(4)
    layer = synth.make_qlinear(rng, 64, 1024)
    x = synth.make_x(rng, 8, 1024)
    w16 = synth.dequantize(layer, np.float32).astype(np.float16).astype(np.float64)
    want = x.astype(np.float64) @ w16.T
    plain = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"])
    with oracle.weight_rounding():
        got = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"])
    assert rel_err(got, want) <= 1.2e-3          # one fp16 rounding of the output
    # the two modes differ by what the rounding of the weights is worth, and no more
    assert 0 < rel_err(got, plain.astype(np.float64)) <= 5e-3
    again = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"])
    assert np.array_equal(again, plain)


def test_embed_is_qmm_with_one_hot_rows():
    rng = np.random.default_rng(4)
    V, D = 64, 128
    layer = synth.make_qlinear(rng, V, D)
    ids = rng.integers(0, V, 10).astype(np.int32)
    got = oracle.embed(ids, layer["weight"], layer["scales"], layer["biases"])
    wd = synth.dequantize(layer, np.float32)                  # fp32 s*q + b
    np.testing.assert_array_equal(got, wd[ids].astype(np.float16))


# ----------------------------------------------------------------------------- RoPE
def rope_f64(x, pos, inv, scale):
    B, H, L, hd = x.shape
    half = hd // 2
    theta = (np.float32(scale) * inv).astype(np.float32)[None, None, :] * pos.astype(np.float32)[:, :, None]
    theta = theta.astype(np.float32).astype(np.float64)[:, None]          # [B,1,L,half]
    x1, x2 = x[..., :half].astype(np.float64), x[..., half:].astype(np.float64)
    return np.concatenate([x1 * np.cos(theta) - x2 * np.sin(theta),
                           x1 * np.sin(theta) + x2 * np.cos(theta)], axis=-1)


@pytest.mark.parametrize("hd,theta", [(128, 1e6), (64, 5e5), (32, 1e4)])
def test_rope_closed_form(hd, theta):
    rng = np.random.default_rng(hd)
    B, H, L = 2, 3, 9
    x = synth.make_x(rng, B, H, L, hd)
    pos = rng.integers(0, 5000, (B, L)).astype(np.int32)
    inv, sc = synth.inv_freqs(synth.ModelArgs(head_dim=hd, hidden_size=hd * H, num_attention_heads=H,
                                              rope_theta=theta))
    got = oracle.rope_arrayed(x, pos, inv, sc)
    assert rel_err(got, rope_f64(x, pos, inv, sc)) <= 1e-3
    # inverse-frequency table: 2 ** (-log2(theta) * 2i / hd) == theta ** (-2i / hd)
    np.testing.assert_allclose(inv, theta ** (-np.arange(0, hd, 2) / hd), rtol=2e-6)
    assert inv[0] == 1.0


def test_rope_permutation_invariant_of_the_reference_self_check():
    """mlx_arrayed_rope_kernel.py:186-216: positions perm+OFFSET on x == contiguous positions
    on the inversely re-ordered x, permuted back (bit-exact, it is the same arithmetic)."""
    rng = np.random.default_rng(42)
    B, H, L, hd, OFFSET = 3, 5, 31, 64, 467
    x = synth.make_x(rng, B, H, L, hd)
    perm = np.stack([rng.permutation(L) for _ in range(B)]).astype(np.int32)
    inv = synth.inv_freqs(synth.ModelArgs(head_dim=hd, hidden_size=hd * H, num_attention_heads=H,
                                          rope_theta=5e5))[0]
    a = oracle.rope_arrayed(x, perm + OFFSET, inv)
    rev = np.argsort(perm, axis=1)
    xr = np.take_along_axis(x, rev[:, None, :, None], axis=2)
    cont = np.ascontiguousarray(np.broadcast_to(np.arange(L, dtype=np.int32)[None] + OFFSET, (B, L)))
    b = np.take_along_axis(oracle.rope_arrayed(xr, cont, inv), perm[:, None, :, None], axis=2)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))


def test_rope_matches_transformers_rotate_half():
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
    rng = np.random.default_rng(7)
    B, H, L, hd = 1, 4, 12, 64
    x = synth.make_x(rng, B, H, L, hd)
    pos = rng.integers(0, 3000, (B, L)).astype(np.int32)
    inv = synth.inv_freqs(synth.ModelArgs(head_dim=hd, hidden_size=hd * H, num_attention_heads=H,
                                          rope_theta=1e6))[0]
    freqs = torch.from_numpy(pos.astype(np.float64))[:, :, None] * torch.from_numpy(inv.astype(np.float64))[None, None]
    emb = torch.cat([freqs, freqs], dim=-1)
    xt = torch.from_numpy(x.astype(np.float64))
    want, _ = apply_rotary_pos_emb(xt, xt, emb.cos(), emb.sin())
    assert rel_err(oracle.rope_arrayed(x, pos, inv), want.numpy()) <= 1e-3


# ----------------------------------------------------------------------------- attention
@pytest.mark.parametrize("H,G,hd,P,T", [(8, 2, 64, 37, 8), (4, 4, 32, 0, 5), (14, 2, 64, 100, 32)])
def test_tree_attention_matches_torch_sdpa(H, G, hd, P, T):
    rng = np.random.default_rng(H + P)
    S = P + T
    q, k, v = synth.make_x(rng, H, T, hd), synth.make_x(rng, G, S + 3, hd), synth.make_x(rng, G, S + 3, hd)
    depth, anc = tree_oracle.tree_from_parents(synth.random_tree(rng, T))
    mask = np.concatenate([np.zeros((T, P), np.float16), tree_oracle.additive_mask(anc)], axis=1)
    got = oracle.tree_attention(q, k, v, mask, hd ** -0.5, S=S)
    f = lambda a: torch.from_numpy(a.astype(np.float32))
    want = torch.nn.functional.scaled_dot_product_attention(
        f(q)[None], f(k[:, :S])[None], f(v[:, :S])[None], attn_mask=f(mask)[None, None],
        scale=hd ** -0.5, enable_gqa=True)[0].numpy()
    assert rel_err(got, want) <= 2e-3


def test_tree_attention_equals_causal_attention_over_each_path():
    """The invariant behind mlx_eagle_tests.py:83-170: node i sees prefix + path(root..i)."""
    rng = np.random.default_rng(9)
    H, G, hd, P, T = 4, 2, 32, 11, 16
    q, k, v = synth.make_x(rng, H, T, hd), synth.make_x(rng, G, P + T, hd), synth.make_x(rng, G, P + T, hd)
    parents = synth.random_tree(rng, T)
    depth, anc = tree_oracle.tree_from_parents(parents)
    mask = np.concatenate([np.zeros((T, P), np.float16), tree_oracle.additive_mask(anc)], axis=1)
    tree = oracle.tree_attention(q, k, v, mask, hd ** -0.5)
    for i in range(T):
        path = [j for j in range(T) if anc[i, j]]
        rows = list(range(P)) + [P + j for j in path]
        ks, vs = np.ascontiguousarray(k[:, rows]), np.ascontiguousarray(v[:, rows])
        one = oracle.tree_attention(np.ascontiguousarray(q[:, i:i + 1]), ks, vs,
                                    np.zeros((1, len(rows)), np.float16), hd ** -0.5)
        assert rel_err(tree[:, i], one[:, 0]) <= 2e-3


# ----------------------------------------------------------------------------- norms etc.
def test_rmsnorm_silu_add_argmax():
    rng = np.random.default_rng(11)
    x = synth.make_x(rng, 7, 896)
    w = (1 + rng.normal(0, 0.02, 896)).astype(np.float16)
    xt = torch.from_numpy(x.astype(np.float64))
    want = torch.from_numpy(w.astype(np.float64)) * xt * torch.rsqrt(xt.pow(2).mean(-1, keepdim=True) + 1e-6)
    assert rel_err(oracle.rmsnorm(x, w, 1e-6), want.numpy()) <= 1e-3
    g, u = (3 * synth.make_x(rng, 5, 64).astype(np.float32)).astype(np.float16), synth.make_x(rng, 5, 64)
    gt, ut = torch.from_numpy(g.astype(np.float64)), torch.from_numpy(u.astype(np.float64))
    assert rel_err(oracle.silu_mul(g, u), (torch.nn.functional.silu(gt) * ut).numpy()) <= 6e-3   # two fp16 roundings
    np.testing.assert_array_equal(oracle.add(g, u), (g.astype(np.float32) + u.astype(np.float32)).astype(np.float16))
    lg = rng.normal(size=(6, 999)).astype(np.float16)
    lg[2, [5, 700]] = lg[2].max()                                   # tie -> first index
    assert np.array_equal(oracle.argmax_rows(lg), np.argmax(lg.astype(np.float32), axis=-1))
    assert oracle.argmax_rows(lg)[2] == min(5, int(np.argmax(lg[2].astype(np.float32))))


# ----------------------------------------------------------------------------- rope tables
def _hf_inv_freq(rope_type, theta, hd, scaling, max_pos, seq_len=None):
    from transformers import LlamaConfig
    from transformers.modeling_rope_utils import ROPE_INIT_FUNCTIONS

    params = dict(scaling, rope_type=rope_type, rope_theta=theta)
    cfg = LlamaConfig(hidden_size=hd * 4, num_attention_heads=4, head_dim=hd,
                      max_position_embeddings=max_pos, rope_parameters=params)
    inv, att = ROPE_INIT_FUNCTIONS[rope_type](cfg, "cpu", seq_len=seq_len)
    assert att == 1.0
    return inv.numpy()


@pytest.mark.parametrize("hd,theta,factor,old_len", [(64, 5e5, 32.0, 8192), (128, 5e5, 8.0, 8192),
                                                      (128, 1e6, 4.0, 4096)])
def test_llama3_inv_freq_table_against_transformers(hd, theta, factor, old_len):
    """The table the reference takes from 1 / fast_rope._freqs (mlx_llama.py:114-116), pinned
    against transformers' _compute_llama3_parameters to fp32 rounding; all three bands
    (kept, interpolated, slowed) are populated."""
    scaling = {"factor": factor, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
               "original_max_position_embeddings": old_len}
    args = synth.ModelArgs(model_type="llama", hidden_size=hd * 4, num_attention_heads=4, head_dim=hd,
                           rope_theta=theta, max_position_embeddings=131072,
                           rope_scaling=dict(scaling, rope_type="llama3"))
    inv, scale = synth.inv_freqs(args)
    want = _hf_inv_freq("llama3", theta, hd, scaling, 131072)
    assert scale == 1.0 and inv.dtype == np.float32
    assert np.allclose(inv, want, rtol=4e-6, atol=0), np.max(np.abs(inv / want - 1))
    plain, _ = synth.inv_freqs(synth.ModelArgs(hidden_size=hd * 4, num_attention_heads=4, head_dim=hd,
                                               rope_theta=theta))
    ratio = plain / inv
    assert (np.isclose(ratio, 1.0, rtol=1e-5)).any() and (np.isclose(ratio, factor, rtol=1e-5)).any()
    assert ((ratio > 1.001) & (ratio < factor * 0.999)).any()


def test_dynamic_inv_freq_table_against_transformers():
    scaling = {"factor": 2.0}
    args = synth.ModelArgs(hidden_size=512, num_attention_heads=4, head_dim=128, rope_theta=1e4,
                           max_position_embeddings=2048, rope_scaling={"factor": 2.0, "type": "dynamic"})
    plain, _ = synth.inv_freqs(synth.ModelArgs(hidden_size=512, num_attention_heads=4, head_dim=128,
                                               rope_theta=1e4))
    inv, scale = synth.inv_freqs(args)
    assert scale == 1.0 and np.allclose(inv, plain, rtol=2e-6)       # within max_position_embeddings
    for L in (2048, 3000, 8192):
        got, _ = synth.inv_freqs(args, seq_len=L)
        want = _hf_inv_freq("dynamic", 1e4, 128, scaling, 2048, seq_len=L)
        assert np.allclose(got, want, rtol=2e-5), (L, np.max(np.abs(got / want - 1)))
