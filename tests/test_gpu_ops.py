"""HIP element-wise / row-wise operators and tree attention vs the CPU oracle."""
import numpy as np
import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import ops, synth
from oracle import oracle, tree_oracle
from util import TOL, layer_to_dev, rel_err, to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,H,L,hd,theta", [(1, 28, 32, 128, 1e6), (1, 4, 32, 128, 1e6),
                                            (2, 3, 17, 64, 5e5), (1, 2, 5, 48, 1e4)])
def test_rope_arrayed(dev, B, H, L, hd, theta):
    print(f"rope B={B} H={H} L={L} hd={hd}", flush=True)
    rng = np.random.default_rng(B * 100 + H)
    x = synth.make_x(rng, B, H, L, hd)
    pos = rng.integers(0, 4096, size=(B, L)).astype(np.int32)
    args = synth.ModelArgs(head_dim=hd, hidden_size=hd * H, num_attention_heads=H, rope_theta=theta)
    inv, sc = synth.inv_freqs(args)
    want = oracle.rope_arrayed(x, pos, inv, sc)
    got = ops.arrayed_rope(to_dev(x, dev), to_dev(pos, dev), to_dev(inv, dev), sc).cpu().numpy()
    assert rel_err(got, want) <= TOL
    # sin/cos differ by at most a few fp32 ulp, so almost every output is bit-identical
    assert np.mean(got.view(np.uint16) != want.view(np.uint16)) < 5e-3
    got2 = ops.rope_positions(to_dev(x, dev), to_dev(pos, dev), to_dev(inv, dev), sc).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), got2.view(np.uint16))


def test_rope_permutation_invariant(dev):
    """The reference's own self-check (mlx_arrayed_rope_kernel.py:186-216): RoPE at
    positions perm+OFFSET equals contiguous RoPE of the inversely re-ordered input,
    permuted back."""
    rng = np.random.default_rng(42)
    B, H, L, hd, OFFSET = 3, 5, 49, 64, 467
    x = synth.make_x(rng, B, H, L, hd)
    perm = np.stack([rng.permutation(L) for _ in range(B)]).astype(np.int32)
    inv = synth.inv_freqs(synth.ModelArgs(head_dim=hd, hidden_size=hd * H, num_attention_heads=H,
                                          rope_theta=5e5))[0]
    got = ops.arrayed_rope(to_dev(x, dev), to_dev(perm + OFFSET, dev), to_dev(inv, dev)).cpu().numpy()
    rev = np.argsort(perm, axis=1)
    xr = np.take_along_axis(x, rev[:, None, :, None], axis=2)
    contiguous = np.broadcast_to(np.arange(L, dtype=np.int32)[None] + OFFSET, (B, L))
    ref = ops.arrayed_rope(to_dev(xr, dev), to_dev(np.ascontiguousarray(contiguous), dev),
                           to_dev(inv, dev)).cpu().numpy()
    ref = np.take_along_axis(ref, perm[:, None, :, None], axis=2)
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("T,D", [(32, 3584), (8, 896), (1, 4096), (5, 64)])
def test_rmsnorm(dev, T, D):
    rng = np.random.default_rng(T + D)
    x = synth.make_x(rng, T, D)
    r = synth.make_x(rng, T, D)
    w = (1 + rng.normal(0, 0.02, D)).astype(np.float16)
    want = oracle.rmsnorm(x, w, 1e-6)
    got = ops.rms_norm(to_dev(x, dev), to_dev(w, dev), 1e-6).cpu().numpy()
    assert rel_err(got, want) <= 2e-3
    assert np.mean(got.view(np.uint16) != want.view(np.uint16)) < 1e-2
    h_want = oracle.add(x, r)
    n_want = oracle.rmsnorm(h_want, w, 1e-6)
    h, n = ops.rms_norm(to_dev(x, dev), to_dev(w, dev), 1e-6, residual=to_dev(r, dev))
    assert np.array_equal(h.cpu().numpy().view(np.uint16), h_want.view(np.uint16))
    assert rel_err(n.cpu().numpy(), n_want) <= 2e-3


def test_silu_mul_and_add(dev):
    rng = np.random.default_rng(1)
    g = (synth.make_x(rng, 32, 18944).astype(np.float32) * 3).astype(np.float16)
    u = synth.make_x(rng, 32, 18944)
    want = oracle.silu_mul(g, u)
    got = ops.silu_mul(to_dev(g, dev), to_dev(u, dev)).cpu().numpy()
    assert rel_err(got, want) <= 2e-3
    assert np.mean(got.view(np.uint16) != want.view(np.uint16)) < 1e-2
    fused = np.concatenate([g, u], axis=1)
    got2 = ops.silu_mul(to_dev(fused, dev)).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), got2.view(np.uint16))
    a = ops.add(to_dev(g, dev), to_dev(u, dev)).cpu().numpy()
    assert np.array_equal(a.view(np.uint16), oracle.add(g, u).view(np.uint16))


def test_embed_bit_exact(dev):
    rng = np.random.default_rng(2)
    layer = synth.make_qlinear(rng, 1000, 896)
    ids = rng.integers(0, 1000, size=(1, 32)).astype(np.int32)
    want = oracle.embed(ids, layer["weight"], layer["scales"], layer["biases"])
    d = layer_to_dev(layer, dev)
    got = ops.embed(to_dev(ids, dev), d["weight"], d["scales"], d["biases"]).cpu().numpy()
    assert got.shape == (1, 32, 896)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("R,V", [(32, 152064), (8, 128256), (3, 1000), (1, 7)])
def test_argmax_rows_bit_exact(dev, R, V):
    rng = np.random.default_rng(R + V)
    logits = (rng.normal(0, 3, size=(R, V))).astype(np.float16)
    # force ties at the maximum: the lowest index must win
    for r in range(R):
        top = logits[r].max()
        idx = rng.integers(0, V, size=3)
        logits[r, idx] = top
    want = oracle.argmax_rows(logits)
    assert np.array_equal(want, np.argmax(logits.astype(np.float32), axis=-1))
    got = ops.argmax_rows(to_dev(logits, dev)).cpu().numpy()
    assert np.array_equal(got, want)


def make_attention_case(rng, H, G, hd, P, T, cap):
    q = synth.make_x(rng, H, T, hd)
    k = synth.make_x(rng, G, cap, hd)
    v = synth.make_x(rng, G, cap, hd)
    parents = synth.random_tree(rng, T, max_depth=4, max_children=4)
    depth, anc = tree_oracle.tree_from_parents(parents)
    return q, k, v, depth, anc


@pytest.mark.parametrize("H,G,hd,P,T", [(28, 4, 128, 1024, 32), (28, 4, 128, 2048, 32),
                                        (14, 2, 64, 515, 32), (32, 8, 128, 100, 8),
                                        (4, 2, 64, 0, 16), (8, 8, 128, 31, 24)])
def test_tree_attention(dev, H, G, hd, P, T):
    print(f"attn H={H} G={G} hd={hd} P={P} T={T}", flush=True)
    rng = np.random.default_rng(H + P + T)
    cap = P + T + 13
    q, k, v, depth, anc = make_attention_case(rng, H, G, hd, P, T, cap)
    # rows past P+T hold NaN: they must never be read into the result
    k[:, P + T:] = np.nan
    v[:, P + T:] = np.nan
    mask = np.concatenate([np.zeros((T, P), np.float16), tree_oracle.additive_mask(anc)], axis=1)
    scale = hd ** -0.5
    want = oracle.tree_attention(q, k, v, mask, scale, S=P + T)          # [H,T,hd]
    want_t = np.ascontiguousarray(want.transpose(1, 0, 2)).reshape(T, H * hd)
    bits = to_dev(tree_oracle.mask_bits(anc).view(np.int32), dev)
    len_dev = torch.tensor([P], dtype=torch.int32, device=dev)
    got = ops.tree_attention(to_dev(q, dev), to_dev(k, dev), to_dev(v, dev), bits, len_dev, scale,
                             max_len=P + T).cpu().numpy()
    assert np.isfinite(got.astype(np.float32)).all()
    assert rel_err(got, want_t) <= TOL
    # larger bound for the grid than the live length (graph-replay use)
    got2 = ops.tree_attention(to_dev(q, dev), to_dev(k, dev), to_dev(v, dev), bits, len_dev, scale,
                              max_len=cap).cpu().numpy()
    assert rel_err(got2, want_t) <= TOL


def test_sdpa_signature(dev):
    rng = np.random.default_rng(11)
    H, G, hd, P, T = 8, 2, 64, 40, 8
    q, k, v, depth, anc = make_attention_case(rng, H, G, hd, P, T, P + T)
    mask = np.concatenate([np.zeros((T, P), np.float16), tree_oracle.additive_mask(anc)], axis=1)
    want = oracle.tree_attention(q, k, v, mask, hd ** -0.5)
    got = ops.scaled_dot_product_attention(to_dev(q[None], dev), to_dev(k[None], dev),
                                           to_dev(v[None], dev), scale=hd ** -0.5,
                                           mask=to_dev(mask[None, None], dev))
    assert tuple(got.shape) == (1, H, T, hd)
    assert rel_err(got[0].cpu().numpy(), want) <= TOL


@pytest.mark.parametrize("H,G,hd,T", [(28, 4, 128, 32), (14, 2, 64, 17), (4, 4, 64, 1)])
def test_rope_kv_append_from_table(dev, H, G, hd, T):
    """Angles from the per-step cos/sin table instead of sincos in the launch: the values are
    copies, the rotated q and k agree to one fp16 ulp in at most a handful of elements (the two
    sincos evaluations may differ in the last fp32 bit)."""
    rng = np.random.default_rng(H + T)
    P, cap = 77, 77 + T + 5
    W = (H + 2 * G) * hd
    qkv = to_dev(synth.make_x(rng, T, W), dev)
    pos = to_dev((P + rng.integers(0, 9, size=T)).astype(np.int32), dev)
    inv = ops.default_inv_freqs(hd, 1000000.0, device=dev)
    len_dev = torch.tensor([P], dtype=torch.int32, device=dev)
    outs = []
    for table in (False, True):
        k = torch.zeros((G, cap, hd), dtype=torch.float16, device=dev)
        v = torch.zeros_like(k)
        q = torch.empty((H, T, hd), dtype=torch.float16, device=dev)
        cs = ops.rope_table(pos, inv, 0.5) if table else None
        ops.rope_kv_append(qkv, qkv[:, H * hd:], qkv[:, (H + G) * hd:], pos, inv, 0.5, q, k, v, len_dev, H, G, hd,
                           row_stride=W, rope_cs=cs)
        torch.cuda.synchronize()
        outs.append((q, k, v))
    (q0, k0, v0), (q1, k1, v1) = outs
    assert torch.equal(v0, v1)
    for a, b in ((q0, q1), (k0, k1)):
        d = (a.float() - b.float()).abs()
        assert int((d > 0).sum()) <= max(1, a.numel() // 10000)
        assert float(d.max()) <= 2.0 ** -10 * float(a.float().abs().max())
