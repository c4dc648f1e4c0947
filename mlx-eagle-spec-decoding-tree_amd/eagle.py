"""Tree speculative-decoding step: the reference's function names, argument order
and return tuples (mlx_eagle.py:24-93, 217-376) on torch tensors, plus
`TreeVerifier`, the same step as one HIP-graph replay with no host round trip.

All index work runs in the single-workgroup kernels of csrc/tree.hip; the
float work in the kernels of qmm / ops / attn.
"""
import math

import torch

from . import _lib, ops
from .layer import emit_layer

MAXT = 32            # tree tokens per matmul launch and per mask word; larger trees: two of each
TREE_SLOTS = 64      # tree tokens the tree-layout kernels, the module path and the fused step take


def _ptr(t):
    return None if t is None else t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def topk(x, k, axis=-1, stable=False):
    """(indices, values) of the k largest entries, descending; equal values keep the
    lowest index first.  The reference's non-stable branch (mlx_eagle.py:30-32) leaves
    that order to argpartition; here both branches are stable."""
    vals, idx = torch.sort(x.float(), dim=axis, descending=True, stable=True)
    idx = idx.narrow(axis, 0, k)
    return idx, torch.gather(x, axis, idx)


def search_sorted(arr, target, left=True):
    """Vectorised binary search with ceil(log2(n)) steps on uint32 bounds
    (mlx_eagle.py:61-93).  int64 holds the uint32 values."""
    n = arr.numel()
    tgt = target.to(torch.int64) & 0xFFFFFFFF
    low = torch.zeros_like(tgt)
    high = torch.full_like(tgt, n)
    a = arr.to(torch.int64) & 0xFFFFFFFF
    for _ in range(int(math.ceil(math.log2(n))) if n > 1 else 0):
        mid = (low + high) // 2
        inside = mid < n
        vals = a[torch.clamp(mid, max=n - 1)]
        if left:
            lt = (vals < tgt) & inside
            ge = (vals >= tgt) & inside
        else:
            lt = (vals <= tgt) & inside
            ge = (vals > tgt) & inside
        low = torch.where(lt, mid + 1, low)
        high = torch.where(ge, mid, high)
    return low


def bits_to_mask(bits, dtype=torch.bfloat16):
    """[T] int32 row bitmasks (or [T,2]: low and high word of trees above 32 tokens) -> [T,T]
    additive mask (0 where visible, -inf elsewhere)."""
    T = bits.shape[0]
    b = bits.to(torch.int64) & 0xFFFFFFFF
    if bits.dim() == 2:
        b = b[:, 0] | (b[:, 1] << 32)
    vis = ((b[:, None] >> torch.arange(T, device=bits.device)[None, :]) & 1).bool()
    zero = torch.zeros((), dtype=dtype, device=bits.device)
    return torch.where(vis, zero, torch.full((), -math.inf, dtype=dtype, device=bits.device))


def _level_buffers(k, depth, dev):
    C = k + k * k * depth
    return dict(
        saved_scores=torch.zeros(C, dtype=torch.float16, device=dev),
        saved_tokens=torch.zeros(C, dtype=torch.int32, device=dev),
        parents=torch.zeros(1 + k * depth, dtype=torch.int32, device=dev),
        cur_scores=torch.zeros(k, dtype=torch.float16, device=dev),
        cur_ids=torch.zeros(k, dtype=torch.int32, device=dev),
        mask_words=torch.zeros((k, 2), dtype=torch.int32, device=dev),
        out_ids=torch.zeros(k, dtype=torch.int32, device=dev),
        topk_cs_index=torch.zeros(k, dtype=torch.int32, device=dev))


def draft_tree_init(topk_index, topk_score, k, b):
    """State of the expansion before its first level, in the buffers of `_level_buffers`."""
    rc = _lib.lib().eagle_draft_tree_init(_ptr(topk_index), _ptr(topk_score), k, _ptr(b["saved_scores"]),
                                          _ptr(b["saved_tokens"]), _ptr(b["parents"]),
                                          _ptr(b["cur_scores"]), _ptr(b["cur_ids"]),
                                          _ptr(b["mask_words"]), _stream())
    _lib.check(rc, "draft_tree_init")


def draft_tree_level(topk_index, topk_score, level, k, depth, b):
    """One level of the expansion on the buffers of `_level_buffers` (no host round trip)."""
    rc = _lib.lib().eagle_draft_tree_level(_ptr(topk_index), _ptr(topk_score), level, k, depth,
                                           _ptr(b["saved_scores"]), _ptr(b["saved_tokens"]),
                                           _ptr(b["parents"]), _ptr(b["cur_scores"]), _ptr(b["cur_ids"]),
                                           _ptr(b["mask_words"]), _ptr(b["out_ids"]),
                                           _ptr(b["topk_cs_index"]), _stream())
    _lib.check(rc, "draft_tree_level")


def process_generate_tree_iteration(logits, current_scores, k=8, tokenizer=None):
    """mlx_eagle.py:97-115.  logits [1,k,V] fp16, current_scores [1,k,1] fp16 ->
    (next_input_ids [1,k], next_scores [1,k,1], out_ids [k], topk_index [1,k,k],
    cu_scores [1,k,k], topk_cs_index [k])."""
    dev = logits.device
    V = logits.shape[-1]
    idx, score = ops.logsoftmax_topk(logits.reshape(-1, V), k, mode=1)
    b = _level_buffers(k, 1, dev)
    b["cur_scores"].copy_(current_scores.reshape(-1).to(torch.float16))
    draft_tree_level(idx, score, 0, k, 1, b)
    cu = b["saved_scores"][k:].reshape(1, k, k)
    return (b["cur_ids"][None], b["cur_scores"].reshape(1, k, 1), b["out_ids"],
            idx.reshape(1, k, k), cu, b["topk_cs_index"])


def generate_draft_tree(topk_index, topk_p, draft_model, cache, depth=5, k=8, tokenizer=None):
    """mlx_eagle.py:118-213: `depth` draft forwards of k tokens, all k at one position, each seeing
    the prefix, its ancestors' rows and its own.  topk_index [1,k], topk_p [1,k,1] ->
    (parents_list, saved_topk_indices, saved_cu_scores) as lists of per-level tensors."""
    dev = topk_index.device
    offset = cache[0].offset
    current_input_ids = topk_index.to(torch.int32)
    scores = topk_p.to(torch.float16)
    ninf = float("-inf")
    mask = torch.full((1, 1, k, offset + depth * k), ninf, dtype=torch.bfloat16, device=dev)
    mask[..., :offset] = 0
    eye = torch.full((k, k), ninf, dtype=torch.bfloat16, device=dev)
    eye.fill_diagonal_(0)
    saved_topk_indices = [current_input_ids[:, None]]
    saved_cu_scores = [scores.transpose(1, 2)]
    parents_list = [torch.zeros(1, dtype=torch.int32, device=dev)]
    topk_cs_index = torch.arange(k, dtype=torch.int32, device=dev)
    for i in range(depth):
        bias = 1 + k * k * max(0, i - 1) + (k if i > 0 else 0)
        parents_list.append(topk_cs_index + bias)
        mask[..., offset + i * k: offset + (i + 1) * k] = eye
        logits = draft_model(current_input_ids, cache, position_ids=offset + i, flat_rope=True,
                             mask=mask[..., : offset + (i + 1) * k])
        (current_input_ids, scores, out_ids, topk_index, cu_scores,
         topk_cs_index) = process_generate_tree_iteration(logits, scores, k=k)
        saved_topk_indices.append(topk_index)
        saved_cu_scores.append(cu_scores)
        mask = mask[..., out_ids.long(), :]
    return parents_list, saved_topk_indices, saved_cu_scores


def process_draft_tree_device(scores, tokens, parents_list, sampled_token_id, k, total_tokens,
                              out=None):
    """Device-only form: flat fp16 scores [C], int32 tokens [C], parents [C/k] ->
    (tree_position_ids [T], mask_index [V], draft_tokens [T], tree_mask_bits [T]), int32."""
    dev = scores.device
    T = total_tokens + 1
    C = scores.numel()
    if out is None:
        out = (torch.empty(T, dtype=torch.int32, device=dev),
               torch.empty(total_tokens, dtype=torch.int32, device=dev),
               torch.empty(T, dtype=torch.int32, device=dev),
               torch.empty(T if T <= 32 else (T, 2), dtype=torch.int32, device=dev))
    pos, midx, toks, bits = out
    rc = _lib.lib().eagle_process_draft_tree(
        _ptr(scores), _ptr(tokens), _ptr(parents_list), _ptr(sampled_token_id), C, k,
        total_tokens, _ptr(pos), _ptr(midx), _ptr(toks), _ptr(bits), _stream())
    _lib.check(rc, "process_draft_tree")
    return out


def process_draft_tree(scores_list, ss_token, parents_list, sampled_token_id, k, total_tokens):
    """mlx_eagle.py:217-250.  Lists of per-level tensors in, and
    (tree_position_ids [T], mask_index [V], draft_tokens [1,T], tree_mask [T,T] bf16) out."""
    scores = torch.cat([s.reshape(s.shape[0], -1) for s in scores_list], dim=1).flatten()
    tokens = torch.cat([t.reshape(t.shape[0], -1) for t in ss_token], dim=1).flatten()
    parents = torch.cat([p.flatten() for p in parents_list], dim=0)
    pos, midx, toks, bits = process_draft_tree_device(
        scores.to(torch.float16).contiguous(), tokens.to(torch.int32).contiguous(),
        parents.to(torch.int32).contiguous(),
        sampled_token_id.to(torch.int32).reshape(-1)[:1].contiguous(), k, total_tokens)
    return pos, midx, toks[None], bits_to_mask(bits)


def post_process_draft_tree_device(tree_position_ids, total_tokens, mask_index, out=None):
    """retrieve_indices [64,64] (-1 padded) and shape [2] = {leaf_num, max_depth+1}, on device."""
    dev = tree_position_ids.device
    if out is None:
        out = (torch.empty((TREE_SLOTS, TREE_SLOTS), dtype=torch.int32, device=dev),
               torch.empty(2, dtype=torch.int32, device=dev))
    rc = _lib.lib().eagle_post_process_draft_tree(_ptr(tree_position_ids), _ptr(mask_index),
                                                  total_tokens, _ptr(out[0]), _ptr(out[1]),
                                                  _stream())
    _lib.check(rc, "post_process_draft_tree")
    return out


def post_process_draft_tree(tree_position_ids, total_tokens, mask_index):
    """mlx_eagle.py:254-295: retrieve_indices [leaf_num, max_depth+1]; like the reference
    this form synchronises with the host (to learn the shape)."""
    full, shape = post_process_draft_tree_device(tree_position_ids.to(torch.int32).contiguous(),
                                                 total_tokens,
                                                 mask_index.to(torch.int32).contiguous())
    leaf_num, cols = (int(v) for v in shape.tolist())
    return full[:leaf_num, :cols].contiguous()


def evaluate_posterior_greedy(logits, candidates):
    """mlx_eagle.py:311-326.  logits [n_leaves, cols, vocab], candidates [n_leaves, cols]."""
    am = ops.argmax_rows(logits[:, :-1].contiguous())
    posterior = (candidates[:, 1:].to(torch.int32) == am).to(torch.int32)
    lens = torch.cumprod(posterior, dim=1).sum(dim=1)
    accept_length = lens.max()
    # first maximum (torch.argmax does not promise it): smallest index reaching the max
    first = torch.nonzero(lens == accept_length)[0, 0]
    best = torch.where(accept_length == 0, torch.zeros_like(first), first).to(torch.int32)
    return best, accept_length, logits[best.long(), accept_length.long()]


def tree_decoding(token_ids, tree_mask, tree_position_ids, base_model, cache):
    """mlx_eagle.py:329-346."""
    offset = cache[0].offset
    T = tree_mask.shape[0]
    mask = torch.zeros((1, 1, T, offset), dtype=tree_mask.dtype, device=tree_mask.device)
    mask = torch.cat((mask, tree_mask[None, None]), dim=-1)
    return base_model(token_ids, cache, position_ids=tree_position_ids[None] + offset, mask=mask)


def accept_candidate(cache, accept_indices, accept_length, offset):
    """mlx_eagle.py:349-376: for every layer move rows offset+accept_indices to
    offset+1.., then set every cache length to offset + accept_length + 1."""
    accept_length = int(accept_length)
    if accept_length > 0:
        dev = cache[0].keys.device
        acc = torch.zeros(4 + TREE_SLOTS, dtype=torch.int32, device=dev)
        acc[1] = accept_length
        acc[4:4 + accept_length] = accept_indices.to(torch.int32).reshape(-1)[:accept_length]
        len_dev = torch.tensor([offset], dtype=torch.int32, device=dev)
        ptrs = torch.tensor([c.keys.data_ptr() for c in cache] + [c.values.data_ptr() for c in cache],
                            dtype=torch.int64, device=dev)
        G, cap, hd = cache[0].keys.shape[1:]
        rc = _lib.lib().eagle_kv_compact_f16(_ptr(ptrs), ptrs.numel(), _ptr(acc), _ptr(len_dev),
                                             G, hd, cap, _stream())
        _lib.check(rc, "accept_candidate")
    for c in cache:
        c.offset = offset + accept_length + 1


def _check_tree_size(verify_num_tokens):
    """The tree kernels lay a tree out in 64 slots (root + 63 nodes), which covers the reference's
    default of 39 nodes (mlx_eagle.py:390,510): above 32 tokens the matmuls run as two passes of
    32 rows and attention over two mask words per query in pieces of 32 queries."""
    if verify_num_tokens + 1 > TREE_SLOTS:
        raise NotImplementedError(
            f"verify_num_tokens={verify_num_tokens}: this build verifies at most {TREE_SLOTS - 1} draft nodes "
            f"per step (a tree of {TREE_SLOTS} tokens)")


def spec_step(y, base_model, draft_model, base_cache, draft_cache, offset=None, accept_length=0,
              k=8, depth=5, verify_num_tokens=39, tokenizer=None):
    """mlx_eagle.py:379-463 up to its first return (same defaults; at most 63 draft nodes): the draft forward of the tokens accepted
    last step, the level-0 top-k, the expansion, the tree layout and the target forward.
    y [1, accept_length + 1] int.  Returns (tree_position_ids, mask_index, draft_tokens,
    base_logits, base_offset, draft_offset)."""
    _check_tree_size(verify_num_tokens)
    base_offset = base_cache[0].offset
    draft_offset = draft_cache[0].offset + 1 + accept_length
    _y = y
    if accept_length > 0:
        pad_size = 8 - accept_length - 1
        if pad_size < 0:
            raise ValueError("accept_length above 7")
        y = torch.cat((y, torch.zeros((1, pad_size), dtype=y.dtype, device=y.device)), dim=-1)
    draft_logits = draft_model(y, cache=draft_cache)
    for c in draft_cache:
        c.offset = draft_offset
    row = torch.tensor([accept_length], dtype=torch.int32, device=y.device)
    topk_index, topk_p = ops.logsoftmax_topk(draft_logits[0], k, mode=0, row_index=row)
    out_parents, out_tokens, out_scores = generate_draft_tree(
        topk_index=topk_index, topk_p=topk_p[..., None], draft_model=draft_model, cache=draft_cache,
        depth=depth, k=k)
    tree_position_ids, mask_index, draft_tokens, tree_mask = process_draft_tree(
        scores_list=out_scores, ss_token=out_tokens, parents_list=out_parents,
        sampled_token_id=_y[:, -1:], k=k, total_tokens=verify_num_tokens)
    base_logits = tree_decoding(token_ids=draft_tokens, tree_mask=tree_mask, base_model=base_model,
                                cache=base_cache, tree_position_ids=tree_position_ids)
    return tree_position_ids, mask_index, draft_tokens, base_logits, base_offset, draft_offset


def generate_step(prompt, base_model, draft_model, prefill_step_size=512, k=8, depth=5,
                  verify_num_tokens=39, max_tokens=128, tokenizer=None, N=20, capacity=None):
    """mlx_eagle.py:503-606, greedy.  prompt: 1-D int tensor on the models' device.  Instead of
    printing, returns dict(tokens: every generated token in order, first: the token sampled
    from the prompt, steps: per step (accept_length, best_candidate, accept_indices, y), n,
    mean_tokens_per_step)."""
    from .cache import make_prompt_cache

    _check_tree_size(verify_num_tokens)
    y = prompt.reshape(-1).to(torch.int64)
    if capacity is None:
        capacity = y.numel() + max_tokens + N + k * depth + TREE_SLOTS + 16
    base_cache = make_prompt_cache(base_model, capacity=capacity)
    draft_cache = make_prompt_cache(draft_model, capacity=capacity)
    while y.numel() > prefill_step_size:
        draft_model(y[:prefill_step_size][None], cache=draft_cache)
        base_model(y[:prefill_step_size][None], cache=base_cache)
        y = y[prefill_step_size:]
    draft_model(y[None], cache=draft_cache)
    base_logits = base_model(y[None], cache=base_cache)
    y = ops.argmax_rows(base_logits[0, -1:].contiguous()).reshape(1, 1).to(torch.int64)
    first = int(y.item())
    tokens, steps = [], []
    n = 0
    accept_length = 0
    i = -1
    for i in range(N):
        if n >= max_tokens:
            break
        (tree_position_ids, mask_index, draft_tokens, base_logits, base_offset,
         draft_offset) = spec_step(y, base_model, draft_model, base_cache, draft_cache,
                                   accept_length=accept_length, k=k, depth=depth,
                                   verify_num_tokens=verify_num_tokens)
        retrieve_indices = post_process_draft_tree(tree_position_ids, verify_num_tokens, mask_index)
        ri = retrieve_indices.long()                  # -1 wraps to the last node (mlx_eagle.py:582)
        candidates = draft_tokens[0, ri]
        best, al, sample_p = evaluate_posterior_greedy(base_logits[0, ri], candidates)
        accept_length = int(al.item())
        best = int(best.item())
        accept_indices = retrieve_indices[best, 1:1 + accept_length]
        accepted_tokens = candidates[best, 1:1 + accept_length]
        accept_candidate(base_cache, accept_indices, accept_length, base_offset)
        for c in draft_cache:
            c.offset = draft_offset
        next_token = ops.argmax_rows(sample_p[None].contiguous()).reshape(1)
        y = torch.cat((accepted_tokens.to(torch.int64), next_token.to(torch.int64)))[None]
        n += 1 + accept_length
        tokens.extend(int(t) for t in y[0].tolist())
        steps.append((accept_length, best, [int(v) for v in accept_indices.tolist()],
                      [int(v) for v in y[0].tolist()]))
    return dict(tokens=tokens, first=first, steps=steps, n=n,
                mean_tokens_per_step=n / max(1, len(steps)))


def fuse_projections(model, swiglu):
    """Lay q/k/v and gate/up of every layer out as one matrix each (rows concatenated) and
    re-point the layers' tensors at row blocks of it, so that one matmul launch serves
    the three (two) projections; memory use is unchanged."""
    # one fused layout per model, shared by every pass object built on it
    done = getattr(model, "_fused_projections", None)
    if done is None:
        done = model._fused_projections = {}
    if swiglu in done:
        return done[swiglu]
    qkv_w, gu_w = [], []

    def interleave(lins):
        g, u = lins
        fused = [ops.interleave_gate_up(getattr(g, k), getattr(u, k))
                 for k in ("weight", "scales", "biases")]
        bias = None
        if g.bias is not None or u.bias is not None:
            z = torch.zeros(g.weight.shape[0], dtype=torch.float16, device=g.weight.device)
            bias = ops.interleave_gate_up(g.bias if g.bias is not None else z,
                                          u.bias if u.bias is not None else z)
        return (*fused, bias)

    def fuse(lins):
        parts = [[l.weight, l.scales, l.biases] for l in lins]
        fused = [torch.cat([p[k] for p in parts], dim=0).contiguous() for k in range(3)]
        bias = None
        if any(l.bias is not None for l in lins):
            bias = torch.cat([l.bias if l.bias is not None
                              else torch.zeros(l.weight.shape[0], dtype=torch.float16,
                                               device=l.weight.device) for l in lins]).contiguous()
        row = 0
        for l in lins:
            n = l.weight.shape[0]
            l.weight, l.scales, l.biases = (f[row:row + n] for f in fused)
            if l.bias is not None:
                l.bias = bias[row:row + n]
            row += n
        return (*fused, bias)

    other = done.get(not swiglu)
    for layer in model.model.layers:
        at, mlp = layer.self_attn, layer.mlp
        if other is None:
            qkv_w.append(fuse([at.q_proj, at.k_proj, at.v_proj]))
        if swiglu:
            # a tile-interleaved copy: the layers keep their own tensors for the module path
            gu_w.append(interleave([mlp.gate_proj, mlp.up_proj]))
        else:
            gu_w.append(fuse([mlp.gate_proj, mlp.up_proj]))
    if other is not None:
        qkv_w = other[0]
    done[swiglu] = (qkv_w, gu_w)
    return qkv_w, gu_w


def tiled_projections(model, qkv_w, gu_w, plan, swiglu):
    """`ops.TiledWeights` copies of the projections a pass of up to 32 rows runs through the slab
    kernels: q|k|v, o and down where `plan` sends them there, and the interleaved gate|up when
    the SwiGLU form is on.  {"qkv": [...], "o": [...], "down": [...], "gu": [...]} with one entry
    per layer (None where the shape is not taken); one set per model, shared by its pass objects."""
    done = getattr(model, "_tiled_projections", None)
    if done is None:
        done = model._tiled_projections = {}
    key = (bool(plan["qkv"]), bool(plan["o"]), bool(plan["down"]), bool(swiglu))
    if key in done:
        return done[key]

    def tile(w, sc, bi):
        n, k = w.shape[0], w.shape[1] * 8
        return ops.tile_weights(w, sc, bi) if ops.tiled_supported(32, n, k) else None

    out = {"qkv": [], "o": [], "down": [], "gu": []}
    for i, layer in enumerate(model.model.layers):
        at, mlp = layer.self_attn, layer.mlp
        out["qkv"].append(tile(*qkv_w[i][:3]) if plan["qkv"] else None)
        out["o"].append(tile(at.o_proj.weight, at.o_proj.scales, at.o_proj.biases) if plan["o"] else None)
        out["down"].append(tile(mlp.down_proj.weight, mlp.down_proj.scales, mlp.down_proj.biases)
                           if plan["down"] else None)
        out["gu"].append(tile(*gu_w[i][:3]) if swiglu else None)
    done[key] = out
    return out


def tiled_head(model):
    """`ops.TiledWeights` copy of the vocabulary projection (the tied embedding or `lm_head`,
    mlx_llama.py:309-312) where the whole-K form on the tiled layout takes it and the matrix has
    enough rows to give every compute unit a workgroup of that form; None otherwise.  One copy
    per model."""
    if not hasattr(model, "_tiled_head"):
        head = model.model.embed_tokens if model.args.tie_word_embeddings else model.lm_head
        n, k = head.weight.shape[0], head.weight.shape[1] * 8
        ok = ops.rows_tiled_supported(32, n, k) and n >= 32 * 16 * 128
        model._tiled_head = ops.tile_weights(head.weight, head.scales, head.biases) if ok else None
    return model._tiled_head


def slab_plan(model, T, forced=None, fused=True):
    """K steps per slab for the q|k|v, o and down projections of a pass of T rows (0: streaming
    kernel): the library's choice per shape, or `forced` ({"qkv": s, "o": s, "down": s}).  The
    slab form leaves the product as partial sums for its consumer to add, so it needs the fused
    pass (table-driven rope launch after q|k|v, norm with the residual after o and down),
    K % 512 == 0, and projections without a bias for o and down."""
    args = model.args
    D, I = args.hidden_size, args.intermediate_size
    H, G, hd = args.num_attention_heads, args.num_key_value_heads, args.head_dim
    layer = model.model.layers[0]
    shapes = {"qkv": ((H + 2 * G) * hd, D), "o": (D, H * hd), "down": (D, I)}
    plan = {}
    for name, (n, k) in shapes.items():
        s = ops.slab_steps(T, n, k) if forced is None else int(forced.get(name, 0))
        ok = fused and s > 0 and ops.slab_count(k, s) > 0
        if name == "o":
            ok = ok and layer.self_attn.o_proj.bias is None
        if name == "down":
            ok = ok and layer.mlp.down_proj.bias is None
        plan[name] = s if ok else 0
    return plan


def slab_partial_buffer(model, plan, T=MAXT):
    """fp32 buffer large enough for the partial sums of any projection in `plan` of a pass of T rows."""
    args = model.args
    D, I = args.hidden_size, args.intermediate_size
    H, G, hd = args.num_attention_heads, args.num_key_value_heads, args.head_dim
    need = max([1] + [ops.slab_count(k, plan[name]) * ops.slab_rows(T) * n
                      for name, n, k in (("qkv", (H + 2 * G) * hd, D), ("o", D, H * hd), ("down", D, I))
                      if plan[name]])
    return torch.empty(need, dtype=torch.float32, device=model.device)


class LengthBudget:
    """Host-side upper bound of a cache length that lives on the device.  A step appends
    `rows_per_step` rows and keeps at most that many; `reserve` is called before every step
    and reads the true length back (`read_length()`, one device-to-host copy) only when the
    bound has reached the capacity.  Raises ValueError when a step would not fit."""

    def __init__(self, capacity, rows_per_step, length=0):
        self.capacity, self.rows, self.bound = int(capacity), int(rows_per_step), int(length)

    def reset(self, length):
        self.bound = int(length)

    def reserve(self, read_length):
        if self.bound + self.rows > self.capacity:
            self.bound = int(read_length())
            if self.bound + self.rows > self.capacity:
                raise ValueError(f"KV caches of {self.capacity} rows have no room for {self.rows} more rows "
                                 f"at length {self.bound}")
        self.bound += self.rows


class TreeVerifier:
    """One target-model tree-verification step with static buffers, so that it can be
    captured once in a HIP graph and replayed: embedding, all decoder layers, final norm,
    output head, per-node argmax, greedy acceptance and KV compaction.  Inputs are written
    into `tokens`, `tree_position_ids`, `mask_index` and `mask_bits`; results appear in
    `logits`, `node_argmax`, `result` (best, accept_length, bonus_node, next_token,
    accept_indices...) and `accepted_tokens`; the cache length advances on the device.
    Same kernels and operator order as Model.__call__ + the host functions above."""

    def __init__(self, model, cache, total_tokens=31, max_len=None, compact=True, fuse=True,
                 swiglu=True, slab_plan=None, tiled=None):
        """slab_plan: {"qkv": s, "o": s, "down": s}, K steps per slab for the projections that go
        through the slab form of the matmul (their consumer adds the slabs), 0 for the
        streaming kernel; None: the library's choice for this shape.
        tiled: the slab products (and gate|up + SwiGLU) read a copy of their weights in the tiled
        layout (`ops.tile_weights`; doubles the memory of those matrices).  None: on for the fused
        step."""
        args = model.args
        self.model, self.cache, self.args = model, cache, args
        if total_tokens + 1 > TREE_SLOTS:
            raise NotImplementedError(f"the verification step takes at most {TREE_SLOTS} tree tokens "
                                      f"(total_tokens <= {TREE_SLOTS - 1})")
        self.V = total_tokens
        self.T = T = total_tokens + 1
        # above 32 tree tokens: q|k|v, o and down in the slab form with 64-row partial tiles, the
        # other matmuls in two passes of the 32-row streaming kernel, two mask words per token and
        # attention in pieces of 32 query rows (one launch pair)
        self.wide = T > MAXT
        if self.wide and not fuse:
            raise ValueError(f"a tree of more than {MAXT} tokens runs with the fused projections only")
        dev = model.device
        self.dev = dev
        D, I = args.hidden_size, args.intermediate_size
        H, G, hd = args.num_attention_heads, args.num_key_value_heads, args.head_dim
        self.capacity = cache[0].capacity
        self.max_len = max_len or self.capacity
        self.compact = compact
        self.fuse = fuse
        # gate|up with the SwiGLU epilogue when the matmul covers the shape in one K slab
        self.swiglu = bool(fuse and swiglu and ops.swiglu_supported(T, I, D))
        if fuse:
            self._fuse_projections()
        self.slab = self._slab_plan(slab_plan)
        if tiled and not fuse:
            raise ValueError("the tiled weight layout serves the fused step")
        self.tiled = None
        self.head_tiled = None
        if (tiled or tiled is None) and fuse:
            self.tiled = tiled_projections(model, self.qkv_w, self.gu_w, self.slab, self.swiglu)
            self.head_tiled = tiled_head(model)
        i32 = dict(dtype=torch.int32, device=dev)
        f16 = dict(dtype=torch.float16, device=dev)
        self.tokens = torch.zeros(T, **i32)
        self.tree_position_ids = torch.zeros(T, **i32)
        self.mask_index = torch.zeros(total_tokens, **i32)
        self.mask_bits = torch.zeros((T, 2) if self.wide else T, **i32)
        self.positions = torch.zeros(T, **i32)
        self.retrieve = torch.zeros((TREE_SLOTS, TREE_SLOTS), **i32)
        self.shape = torch.zeros(2, **i32)
        self.node_argmax = torch.zeros(T, **i32)
        self.result = torch.zeros(4 + TREE_SLOTS, **i32)
        self.accepted_tokens = torch.zeros(TREE_SLOTS, **i32)
        self.h = torch.empty((T, D), **f16)
        self.hn = torch.empty((T, D), **f16)
        # q | k | v of a token side by side: one fused projection writes all three
        self.qkv = torch.empty((T, (H + 2 * G) * hd), **f16)
        self.q = torch.empty((T, H * hd), **f16)
        self.k = torch.empty((T, G * hd), **f16)
        self.v = torch.empty((T, G * hd), **f16)
        self.q_rot = torch.empty((H, T, hd), **f16)
        self.rope_cs = torch.empty((T, hd // 2, 2), dtype=torch.float32, device=dev)
        self.attn = torch.empty((T, H * hd), **f16)
        self.o = torch.empty((T, D), **f16)
        self.gate_up = torch.empty((T, 2 * I), **f16)        # gate | up of a token side by side
        self.gate = torch.empty((T, I), **f16)
        self.up = torch.empty((T, I), **f16)
        self.act = torch.empty((T, I), **f16)
        self.down = torch.empty((T, D), **f16)
        self.logits = torch.empty((T, args.vocab_size), **f16)
        self.partial = slab_partial_buffer(model, self.slab, T)
        self.len_dev = cache[0].len_dev
        self.cache_ptrs = torch.tensor([c.keys.data_ptr() for c in cache]
                                       + [c.values.data_ptr() for c in cache],
                                       dtype=torch.int64, device=dev)
        self.graph = None
        # host-side upper bound of the device cache length (a step adds at most T rows); step()
        # refreshes it from the device before it could pass the capacity
        self._budget = LengthBudget(self.capacity, T, max(c.offset for c in cache))
        # the captured graph holds raw addresses of these tensors: keep them alive with it
        self._graph_keepalive = None
        # size every workspace before any capture
        L = _lib.lib()
        head = model.lm_head if not args.tie_word_embeddings else model.model.embed_tokens
        # (a tree above 32 tokens goes through the 32-row matmul kernel in two passes)
        need = max(L.eagle_qmm_workspace_bytes(rows, n, k) for n, k in
                   ((H * hd, D), (G * hd, D), ((H + 2 * G) * hd, D), (D, H * hd), (I, D), (2 * I, D),
                    (D, I), (head.weight.shape[0], D))
                   for rows in ((T,) if not self.wide else (MAXT, T - MAXT)))
        ops.workspace("qmm", need, dev)
        ops.workspace("attn", L.eagle_tree_attention_wide_workspace_bytes(T, H, hd, self.max_len), dev)
        ops.workspace("argmax", L.eagle_argmax_workspace_bytes(T, args.vocab_size), dev)

    def _fuse_projections(self):
        self.qkv_w, self.gu_w = fuse_projections(self.model, self.swiglu)

    def _slab_plan(self, forced):
        return slab_plan(self.model, self.T, forced, fused=self.fuse)

    def qmm_launches(self):
        """(weight, scales, biases, bias, x, out, form, tiled) of every quantised matmul of one
        step, in order; `form` is True for the launches that go through `quantized_matmul_swiglu`,
        the K steps per slab for those that go through `quantized_matmul_slabs` (into
        `self.partial`), "rows" for `quantized_matmul_tiled` (the vocabulary projection on the
        tiled layout), False for `quantized_matmul`; `tiled` the `ops.TiledWeights` copy the first
        three forms read, or None."""
        m = self.model
        out = []
        for i, layer in enumerate(m.model.layers):
            at, mlp = layer.self_attn, layer.mlp
            if self.fuse:
                out.append((*self.qkv_w[i], self.hn, self.qkv, self.slab["qkv"] or False, self._tiled("qkv", i)))
            else:
                for lin, o in ((at.q_proj, self.q), (at.k_proj, self.k), (at.v_proj, self.v)):
                    out.append((lin.weight, lin.scales, lin.biases, lin.bias, self.hn, o, False, None))
            out.append((at.o_proj.weight, at.o_proj.scales, at.o_proj.biases, at.o_proj.bias,
                        self.attn, self.o, self.slab["o"] or False, self._tiled("o", i)))
            if self.fuse:
                out.append((*self.gu_w[i], self.hn, self.act if self.swiglu else self.gate_up,
                            self.swiglu, self._tiled("gu", i)))
            else:
                for lin, o in ((mlp.gate_proj, self.gate), (mlp.up_proj, self.up)):
                    out.append((lin.weight, lin.scales, lin.biases, lin.bias, self.hn, o, False, None))
            out.append((mlp.down_proj.weight, mlp.down_proj.scales, mlp.down_proj.biases,
                        mlp.down_proj.bias, self.act, self.down, self.slab["down"] or False,
                        self._tiled("down", i)))
        head = m.model.embed_tokens if self.args.tie_word_embeddings else m.lm_head
        out.append((head.weight, head.scales, head.biases, None, self.hn, self.logits,
                    "rows" if self.head_tiled is not None else False, self.head_tiled))
        return out

    def _tiled(self, name, i):
        return self.tiled[name][i] if self.tiled else None

    def set_tree(self, tokens, tree_position_ids, mask_index, mask_bits):
        self.tokens.copy_(tokens.reshape(-1))
        self.tree_position_ids.copy_(tree_position_ids.reshape(-1))
        self.mask_index.copy_(mask_index.reshape(-1))
        self.mask_bits.copy_(mask_bits.reshape(self.mask_bits.shape))

    def forward(self, tap=None):
        """Enqueue the whole step on the current stream (no synchronisation).  tap(i, h):
        called after decoder layer i with the residual stream `self.h` (eager runs only: tests
        that follow the error through the layers)."""
        L = _lib.lib()
        m = self.model
        args = self.args
        T = self.T
        H, G, hd = args.num_attention_heads, args.num_key_value_heads, args.head_dim
        st = _stream()
        _lib.check(L.eagle_tree_positions(_ptr(self.tree_position_ids), _ptr(self.len_dev),
                                          _ptr(self.positions), T, st), "tree_positions")
        post_process_draft_tree_device(self.tree_position_ids, self.V, self.mask_index,
                                       out=(self.retrieve, self.shape))
        emb = m.model.embed_tokens
        ops.embed(self.tokens, emb.weight, emb.scales, emb.biases, out=self.h)
        layers = m.model.layers
        ops.rms_norm(self.h, layers[0].input_layernorm.weight, args.rms_norm_eps, out=self.hn)
        if self.fuse:   # one cos/sin table per step: the positions are the same in every layer
            at0 = layers[0].self_attn
            ops.rope_table(self.positions, at0._inv_freqs, at0._scaling_factor, out=self.rope_cs)

        def attend(at, c):
            ops.tree_attention(self.q_rot, c.keys[0], c.values[0], self.mask_bits, self.len_dev, at.scale,
                               max_len=self.max_len, out=self.attn)

        for i, layer in enumerate(layers):
            if self.fuse:
                emit_layer(self, i, self.len_dev, attend, positions=self.positions)
            else:
                self._layer_one_launch_per_projection(i, layer)
            if tap is not None:
                tap(i, self.h)
        if self.head_tiled is not None:
            ops.quantized_matmul_tiled(self.hn, self.head_tiled, out=self.logits)
        else:
            head = m.model.embed_tokens if args.tie_word_embeddings else m.lm_head
            ops.quantized_matmul(self.hn, head.weight, head.scales, head.biases, out=self.logits)
        ops.argmax_rows(self.logits, out=self.node_argmax)
        _lib.check(L.eagle_greedy_accept(_ptr(self.node_argmax), _ptr(self.tokens),
                                         _ptr(self.retrieve), _ptr(self.shape), T,
                                         _ptr(self.result), _ptr(self.accepted_tokens), st),
                   "greedy_accept")
        if self.compact:
            c0 = self.cache[0]
            _lib.check(L.eagle_kv_compact_f16(_ptr(self.cache_ptrs), self.cache_ptrs.numel(),
                                              _ptr(self.result), _ptr(self.len_dev), G, hd,
                                              c0.capacity, st), "kv_compact")

    def _layer_one_launch_per_projection(self, i, layer):
        """fuse=False: the kernels and launch shapes of the module path (one launch per
        projection), on the static buffers."""
        m, args, T = self.model, self.args, self.T
        H, G, hd = args.num_attention_heads, args.num_key_value_heads, args.head_dim
        layers = m.model.layers
        at, mlp, c = layer.self_attn, layer.mlp, self.cache[i]
        for lin, out in ((at.q_proj, self.q), (at.k_proj, self.k), (at.v_proj, self.v)):
            ops.quantized_matmul(self.hn, lin.weight, lin.scales, lin.biases, bias=lin.bias, out=out)
        ops.rope_kv_append(self.q, self.k, self.v, self.positions, at._inv_freqs, at._scaling_factor,
                           self.q_rot, c.keys[0], c.values[0], self.len_dev, H, G, hd)
        ops.tree_attention(self.q_rot, c.keys[0], c.values[0], self.mask_bits, self.len_dev, at.scale,
                           max_len=self.max_len, out=self.attn)
        ops.quantized_matmul(self.attn, at.o_proj.weight, at.o_proj.scales, at.o_proj.biases,
                             bias=at.o_proj.bias, out=self.o)
        ops.rms_norm(self.o, layer.post_attention_layernorm.weight, args.rms_norm_eps, residual=self.h,
                     out=self.hn, h_out=self.h)
        ops.quantized_matmul(self.hn, mlp.gate_proj.weight, mlp.gate_proj.scales, mlp.gate_proj.biases,
                             bias=mlp.gate_proj.bias, out=self.gate)
        ops.quantized_matmul(self.hn, mlp.up_proj.weight, mlp.up_proj.scales, mlp.up_proj.biases,
                             bias=mlp.up_proj.bias, out=self.up)
        ops.silu_mul(self.gate, self.up, out=self.act)
        nxt = layers[i + 1].input_layernorm.weight if i + 1 < len(layers) else m.model.norm.weight
        ops.quantized_matmul(self.act, mlp.down_proj.weight, mlp.down_proj.scales, mlp.down_proj.biases,
                             bias=mlp.down_proj.bias, out=self.down)
        ops.rms_norm(self.down, nxt, args.rms_norm_eps, residual=self.h, out=self.hn, h_out=self.h)

    def capture(self):
        """Record forward() into a HIP graph (after one eager warm-up on a side stream)."""
        saved_len = self.len_dev.clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self.forward()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.len_dev.copy_(saved_len)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.forward()
        self.len_dev.copy_(saved_len)
        torch.cuda.synchronize()
        self._graph_keepalive = ([c.keys for c in self.cache], [c.values for c in self.cache],
                                 self.qkv_w if self.fuse else None, self.gu_w if self.fuse else None,
                                 self.model)
        self._budget.reset(int(saved_len.item()))
        return self

    def step(self):
        """Run one verification step (graph replay when captured).  The cache length lives on
        the device; the host keeps an upper bound (a step appends T rows and keeps at most T of
        them) and reads the true length back only when that bound reaches the capacity.
        Raises ValueError instead of running a step that the caches have no room for."""
        self._budget.reserve(lambda: self.len_dev.item())
        if self.graph is not None:
            self.graph.replay()
        else:
            self.forward()

    def sync_host_offsets(self):
        """Bring the host-side cache offsets in line with the device length (one D2H copy)."""
        n = int(self.len_dev.item())
        for c in self.cache:
            c.offset = n
        self._budget.reset(n)
        return n
