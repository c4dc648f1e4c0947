"""CPU restatement of the target-model tree-verification forward.

TEST INFRASTRUCTURE ONLY.  Composes the C operators of eagle_oracle.c in the
operator order of the reference graph (mlx_llama.py:121-196, 214-215, 231-249,
265-313), rounding to fp16 wherever the reference materialises an fp16 tensor.

`weights` is the flat dict produced by synth.make_model_weights (numpy arrays
keyed like an MLX-community checkpoint).
"""
import numpy as np

from . import oracle, tree_oracle


def _lin(weights, prefix, x):
    return oracle.qmm(x, weights[f"{prefix}.weight"], weights[f"{prefix}.scales"],
                      weights[f"{prefix}.biases"], weights.get(f"{prefix}.bias"))


def new_cache(args, capacity, layers=None):
    n = args.num_hidden_layers if layers is None else layers
    shape = (args.num_key_value_heads, capacity, args.head_dim)
    return [(np.zeros(shape, np.float16), np.zeros(shape, np.float16)) for _ in range(n)]


def tree_forward(args, weights, inv_freq, rope_scale, token_ids, positions, mask, cache, offset,
                 layers=None, return_hidden=False, tap=None):
    """Logits [T, V] of T tree tokens appended at `offset`.

    token_ids [T] int, positions [T] int (absolute), mask [T, offset+T] additive fp16,
    cache: list of (keys, values) [G, capacity, hd] modified in place (rows offset..offset+T-1).
    tap(i, h): called with the residual stream [T, D] after decoder layer i (tests).
    """
    T = len(token_ids)
    H, G, hd = args.num_attention_heads, args.num_key_value_heads, args.head_dim
    n_layers = args.num_hidden_layers if layers is None else layers
    scale = hd ** -0.5
    h = oracle.embed(np.asarray(token_ids, np.int32), weights["model.embed_tokens.weight"],
                     weights["model.embed_tokens.scales"], weights["model.embed_tokens.biases"])
    pos = np.asarray(positions, np.int32)[None]
    for i in range(n_layers):
        p = f"model.layers.{i}"
        xn = oracle.rmsnorm(h, weights[f"{p}.input_layernorm.weight"], args.rms_norm_eps)
        q = _lin(weights, f"{p}.self_attn.q_proj", xn).reshape(T, H, hd).transpose(1, 0, 2)
        k = _lin(weights, f"{p}.self_attn.k_proj", xn).reshape(T, G, hd).transpose(1, 0, 2)
        v = _lin(weights, f"{p}.self_attn.v_proj", xn).reshape(T, G, hd).transpose(1, 0, 2)
        q = oracle.rope_arrayed(np.ascontiguousarray(q)[None], pos, inv_freq, rope_scale)[0]
        k = oracle.rope_arrayed(np.ascontiguousarray(k)[None], pos, inv_freq, rope_scale)[0]
        keys, values = cache[i]
        keys[:, offset:offset + T] = k
        values[:, offset:offset + T] = v
        att = oracle.tree_attention(q, keys, values, mask, scale, S=offset + T)     # [H,T,hd]
        att = np.ascontiguousarray(att.transpose(1, 0, 2)).reshape(T, H * hd)
        h = oracle.add(h, _lin(weights, f"{p}.self_attn.o_proj", att))
        xn = oracle.rmsnorm(h, weights[f"{p}.post_attention_layernorm.weight"], args.rms_norm_eps)
        act = oracle.silu_mul(_lin(weights, f"{p}.mlp.gate_proj", xn),
                              _lin(weights, f"{p}.mlp.up_proj", xn))
        h = oracle.add(h, _lin(weights, f"{p}.mlp.down_proj", act))
        if tap is not None:
            tap(i, h)
    hn = oracle.rmsnorm(h, weights["model.norm.weight"], args.rms_norm_eps)
    if return_hidden:
        return hn
    head = "model.embed_tokens" if args.tie_word_embeddings else "lm_head"
    return oracle.qmm(hn, weights[f"{head}.weight"], weights[f"{head}.scales"],
                      weights[f"{head}.biases"])


def verify_step(args, weights, inv_freq, rope_scale, draft_tokens, tree_position_ids, mask_index,
                anc, cache, offset, layers=None, tap=None):
    """Full verification step: forward, per-node argmax, greedy acceptance, KV compaction.
    Returns dict(logits, node_argmax, retrieve_indices, best, accept_length, bonus_node,
    next_token, accept_indices, new_offset)."""
    T = len(draft_tokens)
    mask = np.concatenate([np.zeros((T, offset), np.float16), tree_oracle.additive_mask(anc)], axis=1)
    logits = tree_forward(args, weights, inv_freq, rope_scale, draft_tokens,
                          np.asarray(tree_position_ids) + offset, mask, cache, offset, layers, tap=tap)
    node_argmax = oracle.argmax_rows(logits)
    ri = tree_oracle.post_process_draft_tree(tree_position_ids, T - 1, mask_index)
    best, al, bonus = tree_oracle.greedy_accept(node_argmax, draft_tokens, ri)
    accept_indices = ri[best, 1:1 + al]
    new_offset = offset
    for keys, values in cache:
        new_offset = tree_oracle.accept_candidate(keys, values, accept_indices, al, offset)
    return dict(logits=logits, node_argmax=node_argmax, retrieve_indices=ri, best=best,
                accept_length=al, bonus_node=bonus, next_token=int(node_argmax[bonus]),
                accept_indices=accept_indices, new_offset=new_offset)
