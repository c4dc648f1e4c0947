"""The launch sequence of one decoder layer (mlx_llama.py:121-196, 214-215, 231-249) on static
buffers, shared by every pass object: the tree-verification step (`eagle.TreeVerifier`), the
drafter's small passes (`spec.DecoderPass`) and the prompt chunks (`spec.ChunkPass`).

A pass object `p` provides
  model, args, cache, T (rows of the pass),
  h, hn, qkv, q_rot, rope_cs, attn, o, gate_up, act, down   (fp16 buffers; rope_cs fp32),
  qkv_w, gu_w            per-layer fused (weight, scales, biases, bias) tuples (`fuse_projections`),
  swiglu                 gate|up interleaved with SwiGLU in the matmul's epilogue,
  slab                   {"qkv": s, "o": s, "down": s}: K steps per slab, 0 = streaming / GEMM kernel,
  partial                fp32 buffer for the slab form (when any of the three is set),
  tiled                  (optional) {"qkv", "o", "down", "gu"}: per-layer `ops.TiledWeights` copies.
"""
from . import ops


def emit_layer(p, i, write_len, attend, positions=None):
    """Enqueue layer i of pass `p` on the current stream.  On entry p.hn holds the normed input
    and p.h the residual stream; on exit p.hn holds the input of the next layer (or of the final
    head: normed with `model.norm`) and p.h the updated residual stream.

    write_len: device int32, cache row at which the T new K / V rows are written.
    attend(at, c): enqueue attention of p.q_rot over cache `c` into p.attn.
    positions: int32 [T] for the rope launch that reads them (None: only the table p.rope_cs)."""
    m, args, T = p.model, p.args, p.T
    H, G, hd = args.num_attention_heads, args.num_key_value_heads, args.head_dim
    W = (H + 2 * G) * hd
    layers = m.model.layers
    layer = layers[i]
    at, mlp, c = layer.self_attn, layer.mlp, p.cache[i]
    slab = p.slab
    tiled = getattr(p, "tiled", None) or {"qkv": None, "o": None, "down": None, "gu": None}

    def tl(name):
        return tiled[name][i] if tiled[name] else None

    w, sc, bi, b = p.qkv_w[i]
    q_lin, k_lin, v_lin = p.qkv, p.qkv[:, H * hd:], p.qkv[:, (H + G) * hd:]
    if slab["qkv"]:
        s = slab["qkv"]
        ops.quantized_matmul_slabs(p.hn, w, sc, bi, s, partial=p.partial, tiled=tl("qkv"))
        ops.rope_kv_append_slabs(p.partial, ops.slab_count(args.hidden_size, s), b, p.rope_cs, p.q_rot,
                                 c.keys[0], c.values[0], write_len, T, H, G, hd)
        attend(at, c)
    else:
        ops.quantized_matmul(p.hn, w, sc, bi, bias=b, out=p.qkv)
        ops.rope_kv_append(q_lin, k_lin, v_lin, positions, at._inv_freqs, at._scaling_factor, p.q_rot,
                           c.keys[0], c.values[0], write_len, H, G, hd, row_stride=W, rope_cs=p.rope_cs)
        attend(at, c)

    if slab["o"]:
        s = slab["o"]
        ops.quantized_matmul_slabs(p.attn, at.o_proj.weight, at.o_proj.scales, at.o_proj.biases, s,
                                   partial=p.partial, tiled=tl("o"))
        ops.rms_norm_slabs(p.partial, ops.slab_count(H * hd, s), layer.post_attention_layernorm.weight,
                           args.rms_norm_eps, T, residual=p.h, out=p.hn, h_out=p.h)
    else:
        ops.quantized_matmul(p.attn, at.o_proj.weight, at.o_proj.scales, at.o_proj.biases,
                             bias=at.o_proj.bias, out=p.o)
        ops.rms_norm(p.o, layer.post_attention_layernorm.weight, args.rms_norm_eps, residual=p.h,
                     out=p.hn, h_out=p.h)
    w, sc, bi, b = p.gu_w[i]
    if p.swiglu:
        ops.quantized_matmul_swiglu(p.hn, w, sc, bi, bias=b, out=p.act, tiled=tl("gu"))
    else:
        ops.quantized_matmul(p.hn, w, sc, bi, bias=b, out=p.gate_up)
        ops.silu_mul(p.gate_up, None, out=p.act)

    nxt = layers[i + 1].input_layernorm.weight if i + 1 < len(layers) else m.model.norm.weight
    if slab["down"]:
        s = slab["down"]
        ops.quantized_matmul_slabs(p.act, mlp.down_proj.weight, mlp.down_proj.scales, mlp.down_proj.biases, s,
                                   partial=p.partial, tiled=tl("down"))
        ops.rms_norm_slabs(p.partial, ops.slab_count(args.intermediate_size, s), nxt, args.rms_norm_eps, T,
                           residual=p.h, out=p.hn, h_out=p.h)
    else:
        ops.quantized_matmul(p.act, mlp.down_proj.weight, mlp.down_proj.scales, mlp.down_proj.biases,
                             bias=mlp.down_proj.bias, out=p.down)
        ops.rms_norm(p.down, nxt, args.rms_norm_eps, residual=p.h, out=p.hn, h_out=p.h)
