"""CPU restatement of the integer / index logic of the EAGLE-2 tree step.

TEST INFRASTRUCTURE ONLY (checker for the device kernels and host mirror).

Everything here is exact integer work, written with explicit loops on numpy
arrays.  Each function cites the reference lines whose semantics it restates,
including the quirks that bit-exact parity has to reproduce.

Parity pins: the 8-node fixture of the reference test (mlx_eagle_tests.py:80,
97-113,124-126) and brute force with explicit parent pointers on random trees
(tests/test_oracle_tree.py).
"""
import math

import numpy as np


def topk(x, k, stable=False):
    """Top-k of a 1-D array, values descending; equal values keep the lowest
    index first.  mlx_eagle.py:24-58.  The reference's non-stable branch leaves
    the order of equal values to argpartition; this build fixes "lowest index
    first" for both branches, so `stable` only documents the caller's intent.
    A NaN score ranks as -inf (where MLX's argsort puts NaN is unpinned; an fp16 overflow
    in a drafter can produce them, and the tree must stay well formed).
    Returns (indices int64, values)."""
    x = np.asarray(x)
    key = x.astype(np.float64)
    key = np.where(np.isnan(key), -np.inf, key)
    order = np.argsort(-key, kind="stable")[:k]
    return order, x[order]


def search_sorted(arr, target):
    """Left binary search with a fixed ceil(log2(n)) step count on uint32
    bounds, as mlx_eagle.py:61-93 (left=True branch)."""
    arr = np.asarray(arr)
    target = np.asarray(target).astype(np.uint32)
    n = arr.size
    low = np.zeros(target.shape, np.uint32)
    high = np.full(target.shape, n, np.uint32)
    steps = int(math.ceil(math.log2(n))) if n > 1 else 0
    for _ in range(steps):
        mid = (low + high) // np.uint32(2)
        # A read at index n happens only once low == high == n, i.e. for a target
        # above every element.  On the tree path that is the wrapped "parent - 1" of
        # a root child, whose result the caller discards (mlx_eagle.py:237), so the
        # out-of-range read is treated as "not less" and low stays n.
        vals = arr[np.minimum(mid, n - 1)].astype(np.uint32)
        lt = vals < target
        lt = np.where(mid >= n, False, lt)
        ge = np.where(mid >= n, False, ~lt)
        low = np.where(lt, mid + np.uint32(1), low)
        high = np.where(ge, mid, high)
    return low


def process_draft_tree(scores, tokens, parents_list, sampled_token_id, k, total_tokens):
    """Select the `total_tokens` best draft candidates and lay out the tree.

    scores  [C]   cumulative log-probs of all candidates, flat (C = k + k*k*depth)
    tokens  [C]   their token ids
    parents_list [C // k]  per table row: 0 for the root's children, else the
                  parent's flat candidate id + 1
    Returns (tree_position_ids [T], mask_index [V], draft_tokens [1,T],
             tree_mask bool [T,T]) with T = V + 1 = total_tokens + 1.
    mlx_eagle.py:217-250."""
    scores = np.asarray(scores).reshape(-1)
    tokens = np.asarray(tokens).reshape(-1)
    parents_list = np.asarray(parents_list).reshape(-1).astype(np.uint32)
    V = total_tokens
    sel, _ = topk(scores, V, stable=True)                      # :229
    sel = np.sort(sel)                                         # :230
    draft_tokens = np.concatenate([np.asarray(sampled_token_id).reshape(1), tokens[sel]])  # :232-233
    draft_parents = parents_list[sel // k]                     # :235
    mask_index = search_sorted(sel, draft_parents - np.uint32(1))   # :236 (uint32 wrap for roots)
    mask_index = np.where(draft_parents == 0, -1, mask_index.astype(np.int64)) + 1   # :237
    T = V + 1
    anc = np.eye(T, dtype=bool)                                # :239
    for i in range(V):                                         # :242-243
        anc[i + 1] = anc[i + 1] | anc[mask_index[i]]
    tree_position_ids = anc.sum(1) - 1                         # :245
    return (tree_position_ids.astype(np.int32), mask_index.astype(np.int32),
            draft_tokens.astype(np.int32)[None], anc)


def additive_mask(anc, dtype=np.float16):
    """{0, -inf} additive form of a boolean visibility matrix (mlx_eagle.py:248)."""
    return np.where(anc, 0.0, -np.inf).astype(dtype)


def post_process_draft_tree(tree_position_ids, total_tokens, mask_index):
    """Root-to-leaf node paths, one row per leaf in ascending node id, padded
    with -1 on the right to max depth + 1 columns.  mlx_eagle.py:254-295."""
    depth = [int(v) for v in np.asarray(tree_position_ids).reshape(-1)]
    parent = [int(v) for v in np.asarray(mask_index).reshape(-1)]
    max_depth = max(depth) + 1                                 # :269
    inner = set(parent)                                        # :270
    leaf_num = total_tokens - (len(inner) - 1)                 # :271-272
    rows = [[-1] * max_depth for _ in range(leaf_num)]
    r = 0
    for node in range(total_tokens + 1):                       # :280
        if node in inner:
            continue
        cur = node
        for col in range(depth[node], -1, -1):                 # :286-289
            rows[r][col] = cur
            cur = parent[-1] if cur == 0 else parent[cur - 1]
        r += 1
    return np.array(rows, dtype=np.int32).reshape(leaf_num, max_depth)


def greedy_accept(node_argmax, draft_tokens, retrieve_indices):
    """Longest greedily accepted root-to-leaf path.

    node_argmax [T]  argmax token of the target logits at each tree node
    draft_tokens [T] token of each tree node (node 0 = last sampled token)
    retrieve_indices [n_leaves, cols]  paths, -1 padded
    A -1 entry is used as a gather index and therefore selects node T-1
    (mlx_eagle.py:582,584); the comparison, cumulative product, max and the
    "first best, 0 when nothing matched" rule follow mlx_eagle.py:316-326.
    Returns (best, accept_length, bonus_node) where bonus_node is the node whose
    logits give the next token (:326,596)."""
    node_argmax = np.asarray(node_argmax).reshape(-1)
    draft_tokens = np.asarray(draft_tokens).reshape(-1)
    ri = np.asarray(retrieve_indices)
    T = draft_tokens.size
    n_leaves, cols = ri.shape
    lengths = []
    for r in range(n_leaves):
        n = 0
        for j in range(cols - 1):
            prev_node = ri[r, j] % T
            next_node = ri[r, j + 1] % T
            if draft_tokens[next_node] == node_argmax[prev_node]:
                n += 1
            else:
                break
        lengths.append(n)
    accept_length = max(lengths)
    best = 0 if accept_length == 0 else lengths.index(accept_length)
    bonus_node = int(ri[best, accept_length]) % T
    return best, accept_length, bonus_node


def evaluate_posterior_greedy(logits, candidates):
    """Array form of mlx_eagle.py:311-326.  logits [n_leaves, cols, vocab],
    candidates [n_leaves, cols].  Returns (best, accept_length, logits_row)."""
    logits = np.asarray(logits)
    candidates = np.asarray(candidates)
    am = np.argmax(logits[:, :-1].astype(np.float32), axis=-1)      # first maximum
    post = (candidates[:, 1:] == am).astype(np.int32)
    lens = np.cumprod(post, axis=1).sum(axis=1)
    accept_length = int(lens.max())
    best = 0 if accept_length == 0 else int(np.argmax(lens))
    return best, accept_length, logits[best, accept_length]


def accept_candidate(keys, values, accept_indices, accept_length, offset):
    """KV compaction of one layer, in place: rows offset+accept_indices move to
    offset+1 .. offset+accept_length (gather first, then scatter); returns the
    new cache length.  keys/values [G, cap, hd].  mlx_eagle.py:349-376."""
    if accept_length > 0:
        idx = offset + np.asarray(accept_indices).reshape(-1)[:accept_length]
        for buf in (keys, values):
            picked = buf[:, idx].copy()
            buf[:, offset + 1: offset + accept_length + 1] = picked
    return offset + accept_length + 1


# --- helpers used by the tests and the synthetic-tree generator -----------------

def tree_from_parents(parents):
    """(tree_position_ids [T], ancestor-or-self bool [T,T]) from parent node ids."""
    T = len(parents) + 1
    anc = np.eye(T, dtype=bool)
    for i, p in enumerate(parents):
        anc[i + 1] |= anc[p]
    return (anc.sum(1) - 1).astype(np.int32), anc


def mask_bits(anc):
    """Row bitmasks (bit j of word i set iff node j is visible to node i): [T] uint32 for trees
    of at most 32 tokens, [T, 2] (low word, high word) up to 64."""
    T = anc.shape[0]
    assert T <= 64
    rows = [sum(1 << j for j in range(T) if anc[i, j]) for i in range(T)]
    if T <= 32:
        return np.array(rows, np.uint64).astype(np.uint32)
    return np.array([[r & 0xFFFFFFFF, r >> 32] for r in rows], np.uint64).astype(np.uint32)
