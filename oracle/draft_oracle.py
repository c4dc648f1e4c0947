"""CPU restatement of the draft-side tree expansion and of the outer speculative loop.

TEST INFRASTRUCTURE ONLY: nothing outside tests/, the smoke check and the benchmark's CPU
baseline may import this module.

Follows mlx_eagle.py:97-213 (process_generate_tree_iteration, generate_draft_tree), :379-463
(spec_step) and :503-606 (generate_step).  Integer results are exact restatements.  The float
parts (log-softmax in fp16, fp16 cumulative scores) round to fp16 wherever the reference
materialises an fp16 tensor; what MLX does inside softmax / logsumexp on fp16 inputs (the width
of its accumulator) cannot be checked here (MLX is not available), so those two are
"parity unpinned" beyond the fp16 rounding of their results.  Pinned by tests: the top-k against
a full stable sort, log-probabilities against float64 log-softmax, the parents / mask
bookkeeping against ground-truth parent pointers tracked separately.

Ordering rule everywhere: larger score first, equal scores lowest flat index first (the
reference's non-stable top-k leaves ties to argpartition, mlx_eagle.py:30-32).
"""
import numpy as np

from . import model_oracle, oracle, tree_oracle


def topk_desc(x, k):
    """Indices of the k largest entries of a 1-D array, descending, ties lowest index first."""
    order = np.argsort(-x.astype(np.float64), kind="stable")
    return order[:k]


def logsoftmax_topk(logits, k, mode):
    """logits [R,V] fp16 -> (index [R,k] int32, score [R,k] fp16).
    mode 0: mlx_eagle.py:410-412 (top-k of the logits, then logit - logsumexp in fp16);
    mode 1: mlx_eagle.py:103-104 (log(softmax(logits)) in fp16, then top-k of that)."""
    logits = np.asarray(logits, np.float16)
    R, V = logits.shape
    idx = np.empty((R, k), np.int32)
    sc = np.empty((R, k), np.float16)
    for r in range(R):
        x = logits[r].astype(np.float32)
        m = x.max()
        e = np.exp(x - m, dtype=np.float32)
        s = np.float32(e.sum(dtype=np.float64))
        if mode == 0:
            lse16 = np.float16(m + np.log(s, dtype=np.float32))
            top = topk_desc(x, k)
            idx[r] = top
            sc[r] = (logits[r][top].astype(np.float32) - np.float32(lse16)).astype(np.float16)
        else:
            p16 = (e / s).astype(np.float16)
            with np.errstate(divide="ignore"):
                lp = np.log(p16.astype(np.float32)).astype(np.float16)
            top = topk_desc(lp, k)
            idx[r] = top
            sc[r] = lp[top]
    return idx, sc


def tree_level(topk_index, topk_score, cur_scores, k):
    """process_generate_tree_iteration after its per-row top-k (mlx_eagle.py:106-115).
    topk_index, topk_score [k,k]; cur_scores [k] fp16.  Returns (next_input_ids [k],
    next_scores [k] fp16, out_ids [k], cu_scores [k,k] fp16, topk_cs_index [k])."""
    topk_score = np.asarray(topk_score, np.float16)
    cur = np.asarray(cur_scores, np.float16).reshape(k, 1)
    cu = (topk_score.astype(np.float32) + cur.astype(np.float32)).astype(np.float16)   # fp16 add
    cs = topk_desc(cu.reshape(-1), k).astype(np.int32)
    out_ids = cs // k
    return (np.asarray(topk_index, np.int32).reshape(-1)[cs], cu.reshape(-1)[cs], out_ids, cu, cs)


def draft_forward(args, weights, inv_freq, rope_scale, ids, positions, mask, cache, write_offset):
    return model_oracle.tree_forward(args, weights, inv_freq, rope_scale, ids, positions, mask, cache,
                                     write_offset)


def generate_draft_tree(args, weights, inv_freq, rope_scale, topk_index, topk_p, cache, offset,
                        depth, k, trace=None, forced=None):
    """mlx_eagle.py:118-213.  topk_index [k] int, topk_p [k] fp16; cache rows >= offset are
    overwritten.  Returns (parents [1 + k*depth] uint32, tokens [k + k*k*depth] int32,
    scores [same] fp16) in the flat layout process_draft_tree concatenates them to.
    trace: list that receives every level's inputs and float results.  forced: per level
    (topk_index [k,k], cu_scores [k,k]) to use instead of this function's own float results,
    so that the integer bookkeeping can be compared on identical inputs."""
    ids = np.asarray(topk_index, np.int32).copy()
    scores = np.asarray(topk_p, np.float16).copy()
    ninf = np.float16(-np.inf)
    mask = np.full((k, offset + depth * k), ninf, np.float16)
    mask[:, :offset] = 0
    eye = np.where(np.eye(k, dtype=bool), np.float16(0), ninf)
    saved_tokens = [ids.copy()]
    saved_scores = [scores.copy()]
    parents = [np.zeros(1, np.uint32)]
    cs = np.arange(k, dtype=np.uint32)
    for i in range(depth):
        bias = 1 + k * k * max(0, i - 1) + (k if i > 0 else 0)                      # :158-161
        parents.append((cs + bias).astype(np.uint32))
        mask[:, offset + i * k: offset + (i + 1) * k] = eye                          # :171
        logits = draft_forward(args, weights, inv_freq, rope_scale, ids,
                               np.full(k, offset + i, np.int32),                     # flat_rope
                               np.ascontiguousarray(mask[:, : offset + (i + 1) * k]), cache,
                               offset + i * k)
        tidx, tsc = logsoftmax_topk(logits, k, mode=1)
        if trace is not None:
            trace.append(dict(logits=logits, input_ids=ids.copy(), cur_scores=scores.copy(),
                              mask=mask[:, offset: offset + (i + 1) * k].copy(), topk_index=tidx,
                              topk_score=tsc))
        ids, scores, out_ids, cu, cs = tree_level(tidx, tsc, scores, k)
        if forced is not None:
            tidx = np.asarray(forced[i][0], np.int32).reshape(k, k)
            cu = np.asarray(forced[i][1], np.float16).reshape(k, k)
            cs = topk_desc(cu.reshape(-1), k).astype(np.int32)
            ids, scores, out_ids = tidx.reshape(-1)[cs], cu.reshape(-1)[cs], cs // k
        saved_tokens.append(tidx.reshape(-1))
        saved_scores.append(cu.reshape(-1))
        mask = mask[out_ids]                                                         # :207
    return (np.concatenate(parents), np.concatenate(saved_tokens).astype(np.int32),
            np.concatenate(saved_scores).astype(np.float16))


def causal_forward(args, weights, inv_freq, rope_scale, ids, cache, offset, chunk=32):
    """Causal pass over `ids` appended at `offset` (mask=None in the reference,
    mlx_llama.py:275-276), in pieces of `chunk` tokens.  Returns logits [len(ids), V]."""
    out = []
    ids = np.asarray(ids, np.int32)
    for s in range(0, len(ids), chunk):
        part = ids[s:s + chunk]
        L = len(part)
        off = offset + s
        mask = np.zeros((L, off + L), np.float16)
        mask[:, off:] = np.where(np.tril(np.ones((L, L), bool)), np.float16(0), np.float16(-np.inf))
        out.append(model_oracle.tree_forward(args, weights, inv_freq, rope_scale, part,
                                             off + np.arange(L, dtype=np.int32), mask, cache, off))
    return np.concatenate(out, axis=0)


class Side:
    """One model of the loop: arguments, weights, rotary table, cache and its length."""

    def __init__(self, args, weights, inv_freq, rope_scale, capacity):
        self.args, self.weights, self.inv, self.sc = args, weights, inv_freq, rope_scale
        self.cache = model_oracle.new_cache(args, capacity)
        self.offset = 0

    def causal(self, ids):
        logits = causal_forward(self.args, self.weights, self.inv, self.sc, ids, self.cache, self.offset)
        self.offset += len(ids)
        return logits


def spec_step(base, draft, y, accept_length, k, depth, verify_num_tokens, trace=None):
    """mlx_eagle.py:379-463 (to the first return) + :571-597.  y: the tokens accepted last step
    followed by the bonus token.  Returns dict(accept_length, best, accept_indices, y, ...)."""
    base_offset = base.offset
    draft_offset = draft.offset + 1 + accept_length
    y = np.asarray(y, np.int32)
    yy = y
    if accept_length > 0:
        yy = np.concatenate([y, np.zeros(8 - accept_length - 1, np.int32)])            # :400-403
    draft_logits = draft.causal(yy)
    draft.offset = draft_offset                                                       # :405-406
    tidx, tsc = logsoftmax_topk(draft_logits[accept_length:accept_length + 1], k, mode=0)
    parents, tokens, scores = generate_draft_tree(draft.args, draft.weights, draft.inv, draft.sc,
                                                  tidx[0], tsc[0], draft.cache, draft_offset, depth, k,
                                                  trace=trace)
    pos, midx, toks, anc = tree_oracle.process_draft_tree(scores, tokens, parents, int(y[-1]), k,
                                                          verify_num_tokens)
    toks = toks[0]
    res = model_oracle.verify_step(base.args, base.weights, base.inv, base.sc, toks, pos, midx, anc,
                                   base.cache, base_offset)
    base.offset = res["new_offset"]
    al = res["accept_length"]
    ri = res["retrieve_indices"]
    accepted = [int(toks[j]) for j in ri[res["best"], 1:1 + al]]                      # -1 wraps
    new_y = accepted + [res["next_token"]]
    return dict(accept_length=al, best=res["best"], accept_indices=[int(v) for v in res["accept_indices"]],
                y=new_y, level0=(tidx[0], tsc[0]), parents=parents, tokens=tokens, scores=scores,
                draft_tokens=toks, tree_position_ids=pos, mask_index=midx, logits=res["logits"])


def generate(base, draft, prompt, k, depth, verify_num_tokens, max_tokens, N):
    """mlx_eagle.py:503-606: prefill both models, then up to N speculative steps."""
    prompt = np.asarray(prompt, np.int32)
    draft.causal(prompt)
    logits = base.causal(prompt)
    y = [int(oracle.argmax_rows(logits[-1:])[0])]
    first = y[0]
    tokens, steps = [], []
    n, al = 0, 0
    for _ in range(N):
        if n >= max_tokens:
            break
        r = spec_step(base, draft, y, al, k, depth, verify_num_tokens)
        al, y = r["accept_length"], r["y"]
        n += 1 + al
        tokens.extend(y)
        steps.append((al, r["best"], r["accept_indices"], list(y)))
    return dict(tokens=tokens, first=first, steps=steps, n=n)
