"""Seeded synthetic inputs for every benchmark configuration.

numpy `default_rng(seed)` (PCG64) is platform-stable, so the generator code is
what ships, not data: the same call yields the same arrays for the HIP path and
for the CPU checker.  Value distributions follow the benchmark configuration
text: packed uint4 uniform in 0..15, scales ~ U(0.005, 0.02) fp16,
biases = fp16(-8*scale + N(0, 1e-3)), activations ~ N(0, 1) fp16.
"""
from dataclasses import dataclass, field
from typing import Dict, Optional

import numpy as np


@dataclass
class ModelArgs:
    """Same fields as the reference's ModelArgs (mlx_llama.py:21-58)."""
    model_type: str = "qwen2"
    hidden_size: int = 3584
    num_hidden_layers: int = 28
    intermediate_size: int = 18944
    num_attention_heads: int = 28
    rms_norm_eps: float = 1e-6
    vocab_size: int = 152064
    head_dim: Optional[int] = None
    max_position_embeddings: Optional[int] = None
    num_key_value_heads: Optional[int] = None
    attention_bias: bool = False
    mlp_bias: bool = False
    rope_theta: float = 10000.0
    rope_traditional: bool = False
    rope_scaling: Optional[Dict] = None
    tie_word_embeddings: bool = True
    group_size: int = 64
    bits: int = 4

    def __post_init__(self):
        if self.num_key_value_heads is None:
            self.num_key_value_heads = self.num_attention_heads
        if self.head_dim is None:
            self.head_dim = self.hidden_size // self.num_attention_heads
        if self.rope_scaling:
            if "factor" not in self.rope_scaling:
                raise ValueError("rope_scaling must contain 'factor'")
            rope_type = self.rope_scaling.get("type") or self.rope_scaling.get("rope_type")
            if rope_type is None:
                raise ValueError("rope_scaling must contain either 'type' or 'rope_type'")
            if rope_type not in ("linear", "dynamic", "llama3"):
                raise ValueError("rope_scaling 'type' supports 'linear', 'dynamic' or 'llama3'")


def qwen25_7b():
    return ModelArgs(model_type="qwen2", hidden_size=3584, num_hidden_layers=28,
                     intermediate_size=18944, num_attention_heads=28, num_key_value_heads=4,
                     head_dim=128, vocab_size=152064, rms_norm_eps=1e-6, rope_theta=1e6,
                     attention_bias=True, tie_word_embeddings=False)


def qwen25_05b():
    return ModelArgs(model_type="qwen2", hidden_size=896, num_hidden_layers=24,
                     intermediate_size=4864, num_attention_heads=14, num_key_value_heads=2,
                     head_dim=64, vocab_size=152064, rms_norm_eps=1e-6, rope_theta=1e6,
                     attention_bias=True, tie_word_embeddings=True)


def llama3_8b():
    return ModelArgs(model_type="llama", hidden_size=4096, num_hidden_layers=32,
                     intermediate_size=14336, num_attention_heads=32, num_key_value_heads=8,
                     head_dim=128, vocab_size=128256, rms_norm_eps=1e-5, rope_theta=5e5,
                     attention_bias=False, tie_word_embeddings=False)


def tiny(layers=2, hidden=256, inter=512, heads=4, kv_heads=2, head_dim=64, vocab=1024,
         attention_bias=True, tie=False, theta=1e6):
    return ModelArgs(model_type="qwen2", hidden_size=hidden, num_hidden_layers=layers,
                     intermediate_size=inter, num_attention_heads=heads,
                     num_key_value_heads=kv_heads, head_dim=head_dim, vocab_size=vocab,
                     rms_norm_eps=1e-6, rope_theta=theta, attention_bias=attention_bias,
                     tie_word_embeddings=tie)


def make_qlinear(rng, N, K, bias=False, gain=None):
    """Random 4-bit group-64 linear layer in the packed layout
    (weight uint32 [N, K/8], nibble i of a word = element 8*word + i).

    gain=None: the single-matmul benchmark distribution (scales ~ U(0.005, 0.02),
    biases = -8*scale + N(0, 1e-3)); the dequantised weights then have mean -0.5*scale
    and rms 0.061, which is what a lone matmul is measured with.
    gain=g: the same shapes of distribution rescaled for whole-model use: zero-mean
    weights (biases = -7.5*scale + small noise) of rms g / sqrt(K), so that activations
    stay O(1) through dozens of layers instead of overflowing fp16 in the first MLP."""
    assert K % 64 == 0
    w = rng.integers(0, 1 << 32, size=(N, K // 8), dtype=np.uint32)
    s32 = rng.uniform(0.005, 0.02, size=(N, K // 64))
    noise = rng.normal(0.0, 1e-3, size=s32.shape)
    if gain is None:
        s = s32.astype(np.float16)
        b = (-8.0 * s.astype(np.float32) + noise.astype(np.float32)).astype(np.float16)
    else:
        f = gain / (0.0610 * np.sqrt(K))
        s = (s32 * f).astype(np.float16)
        b = (-7.5 * s.astype(np.float32) + (noise * f).astype(np.float32)).astype(np.float16)
    out = {"weight": w, "scales": s, "biases": b}
    if bias:
        out["bias"] = rng.normal(0.0, 0.02, size=(N,)).astype(np.float16)
    return out


def unpack_nibbles(w):
    """uint32 [N, K/8] -> uint8 [N, K] (element 8*j+i = bits 4i..4i+3 of word j)."""
    N, K8 = w.shape
    sh = (np.arange(8, dtype=np.uint32) * 4)[None, None, :]
    return ((w[:, :, None] >> sh) & np.uint32(15)).astype(np.uint8).reshape(N, K8 * 8)


def pack_nibbles(q):
    """uint8 [N, K] with values 0..15 -> uint32 [N, K/8]."""
    N, K = q.shape
    q = q.reshape(N, K // 8, 8).astype(np.uint32)
    sh = (np.arange(8, dtype=np.uint32) * 4)[None, None, :]
    return (q << sh).sum(axis=2, dtype=np.uint64).astype(np.uint32)


def dequantize(layer, dtype=np.float64):
    q = unpack_nibbles(layer["weight"]).astype(dtype)
    s = np.repeat(layer["scales"].astype(dtype), 64, axis=1)
    b = np.repeat(layer["biases"].astype(dtype), 64, axis=1)
    return s * q + b


def make_x(rng, *shape):
    return rng.normal(0.0, 1.0, size=shape).astype(np.float16)


def make_model_weights(args: ModelArgs, seed=42, layers=None, gain=1.0):
    """All tensors of a random-init quantised decoder as a flat dict of numpy
    arrays keyed like an MLX-community checkpoint
    (`model.layers.3.self_attn.q_proj.weight` / `.scales` / `.biases` / `.bias`)."""
    rng = np.random.default_rng(seed)
    D, I, V = args.hidden_size, args.intermediate_size, args.vocab_size
    H, G, hd = args.num_attention_heads, args.num_key_value_heads, args.head_dim
    out = {}

    def put(prefix, layer):
        for k, v in layer.items():
            out[f"{prefix}.{k}"] = v

    put("model.embed_tokens", make_qlinear(rng, V, D, gain=gain))
    n_layers = args.num_hidden_layers if layers is None else layers
    for i in range(n_layers):
        p = f"model.layers.{i}"
        put(f"{p}.self_attn.q_proj", make_qlinear(rng, H * hd, D, args.attention_bias, gain=gain))
        put(f"{p}.self_attn.k_proj", make_qlinear(rng, G * hd, D, args.attention_bias, gain=gain))
        put(f"{p}.self_attn.v_proj", make_qlinear(rng, G * hd, D, args.attention_bias, gain=gain))
        put(f"{p}.self_attn.o_proj", make_qlinear(rng, D, H * hd, gain=gain))
        put(f"{p}.mlp.gate_proj", make_qlinear(rng, I, D, args.mlp_bias, gain=gain))
        put(f"{p}.mlp.up_proj", make_qlinear(rng, I, D, args.mlp_bias, gain=gain))
        put(f"{p}.mlp.down_proj", make_qlinear(rng, D, I, args.mlp_bias, gain=gain))
        out[f"{p}.input_layernorm.weight"] = (1.0 + rng.normal(0, 0.02, D)).astype(np.float16)
        out[f"{p}.post_attention_layernorm.weight"] = (1.0 + rng.normal(0, 0.02, D)).astype(np.float16)
    out["model.norm.weight"] = (1.0 + rng.normal(0, 0.02, D)).astype(np.float16)
    if not args.tie_word_embeddings:
        put("lm_head", make_qlinear(rng, V, D, gain=gain))
    return out


def inv_freqs(args: ModelArgs, seq_len=None):
    """fp32 inverse-frequency table and scaling factor of the rotary embedding
    (mlx_llama.py:98-116).

    default / linear: inv_freq[i] = 2 ** (-log2(theta) * 2i / head_dim), scaling factor
    1 / factor for linear (:105-113).
    llama3: the table of the Llama-3.1 rule, 1 / fast_rope._freqs in the reference (:114-116):
    pairs whose wavelength exceeds original_max_position_embeddings / low_freq_factor are slowed
    by `factor`, those below original_max_position_embeddings / high_freq_factor are kept, and
    the band between is interpolated in the frequency.
    dynamic: the NTK rule, theta * (factor * L / max_pos - (factor - 1)) ** (hd / (hd - 2)) with
    L = max(seq_len, max_position_embeddings); up to max_position_embeddings tokens (seq_len None)
    this is the default table."""
    rope_type = "default"
    rs = args.rope_scaling
    if rs is not None:
        rope_type = rs.get("type") or rs.get("rope_type", "default")
    if rope_type not in ("default", "linear", "llama3", "dynamic"):
        raise NotImplementedError(f"rope type {rope_type!r}")
    hd = args.head_dim
    theta = float(args.rope_theta)
    if rope_type == "dynamic":
        max_pos = args.max_position_embeddings
        if not max_pos:
            raise ValueError("dynamic rope scaling needs max_position_embeddings")
        L = max(int(seq_len or max_pos), int(max_pos))
        theta = theta * ((rs["factor"] * L / max_pos) - (rs["factor"] - 1)) ** (hd / (hd - 2))
    expo = (-np.log2(np.float32(theta)) * np.arange(0, hd, 2, dtype=np.float32)
            / np.float32(hd)).astype(np.float32)
    inv = np.exp2(expo).astype(np.float32)
    if rope_type == "llama3":
        factor = np.float32(rs["factor"])
        low = np.float32(rs.get("low_freq_factor", 1.0))
        high = np.float32(rs.get("high_freq_factor", 4.0))
        old_len = np.float32(rs.get("original_max_position_embeddings", 8192))
        wavelen = (np.float32(2 * np.pi) / inv).astype(np.float32)
        slowed = np.where(wavelen > old_len / low, inv / factor, inv).astype(np.float32)
        smooth = ((old_len / wavelen - low) / (high - low)).astype(np.float32)
        mixed = ((1 - smooth) * slowed / factor + smooth * slowed).astype(np.float32)
        medium = ~(wavelen < old_len / high) & ~(wavelen > old_len / low)
        inv = np.where(medium, mixed, slowed).astype(np.float32)
    scale = 1.0 / rs["factor"] if rope_type == "linear" else 1.0
    return inv, float(scale)


def random_tree(rng, n_nodes=32, max_depth=4, max_children=4):
    """Parents (node ids, for nodes 1..n-1) of a random tree with topologically
    sorted ids, depth <= max_depth, at most max_children children per node."""
    depth = [0]
    children = [0]
    parents = []
    for node in range(1, n_nodes):
        ok = [p for p in range(node) if depth[p] < max_depth and children[p] < max_children]
        p = int(ok[rng.integers(len(ok))])
        parents.append(p)
        children[p] += 1
        children.append(0)
        depth.append(depth[p] + 1)
    return np.array(parents, np.int32)


def tree_arrays(parents):
    """(depth [T] int32, ancestor-or-self visibility [T,T] bool, row bitmasks [T] uint32, or
    [T,2] (low word, high word) above 32 tokens) of the tree given by `parents` (as returned by
    random_tree)."""
    T = len(parents) + 1
    depth = np.zeros(T, np.int32)
    vis = np.eye(T, dtype=bool)
    for node in range(1, T):
        p = int(parents[node - 1])
        depth[node] = depth[p] + 1
        vis[node] |= vis[p]
    rows = (vis.astype(np.uint64) << np.arange(T, dtype=np.uint64)[None, :]).sum(1)
    if T <= 32:
        return depth, vis, rows.astype(np.uint32)
    bits = np.stack([rows & np.uint64(0xFFFFFFFF), rows >> np.uint64(32)], axis=1).astype(np.uint32)
    return depth, vis, bits
