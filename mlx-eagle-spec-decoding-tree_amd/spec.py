"""The whole speculative step of the reference loop (mlx_eagle.py:379-463, 571-599) enqueued on
one stream with static buffers and all loop state on the device: draft pass over the tokens
accepted last step, level-0 top-k, `depth` expansion passes with their bookkeeping, tree layout,
target verification, greedy acceptance, KV compaction, state update.  Captured once as a HIP
graph, N steps are N replays and one device-to-host copy of the emitted tokens at the end (the
reference synchronises at least five times per step).

Differences from the host-driven functions of eagle.py, both invisible in the results: the
draft pass over the accepted tokens always has 8 rows (the reference pads to 8 only when
something was accepted, mlx_eagle.py:400-408; row `accept_length` of a causal pass does not
depend on the rows after it), and the expansion masks travel as two 32-bit words per query.
"""
import torch

from . import _lib, ops
from .layer import emit_layer
from .eagle import (TREE_SLOTS, TreeVerifier, _level_buffers, _ptr, _stream, draft_tree_init, draft_tree_level,
                    fuse_projections, process_draft_tree_device, slab_partial_buffer)
from .eagle import slab_plan as eagle_slab_plan

Y_LEN = 8
MAX_CHUNK = 2048     # rows of one causal prompt pass (EAGLE_MAX_CHUNK)


class DecoderPass:
    """One pass of T <= 32 rows through a decoder with static buffers: tokens -> logits [T,V].
    The rows are written to the cache at *write_len; query t sees the *attn_len rows before
    them and, of the Tk rows from there on, those its two mask words select."""

    def __init__(self, model, cache, T, max_len=None, swiglu=True, slab_plan=None, folded=None):
        """folded: the small-row form of the products with norm, residual add and SwiGLU folded in
        (`ops.quantized_matmul_small`: four launches per layer besides rope and attention);
        None = wherever the library takes the shapes and the weights."""
        args = model.args
        self.model, self.cache, self.args, self.T = model, cache, args, T
        dev = model.device
        self.slab = eagle_slab_plan(model, T, slab_plan)
        self.partial = slab_partial_buffer(model, self.slab)
        D, I = args.hidden_size, args.intermediate_size
        H, G, hd = args.num_attention_heads, args.num_key_value_heads, args.head_dim
        self.max_len = max_len or cache[0].capacity
        self.swiglu = bool(swiglu and ops.swiglu_supported(T, I, D))
        self.qkv_w, self.gu_w = fuse_projections(model, self.swiglu)
        f16 = dict(dtype=torch.float16, device=dev)
        self.h = torch.empty((T, D), **f16)
        self.hn = torch.empty((T, D), **f16)
        self.qkv = torch.empty((T, (H + 2 * G) * hd), **f16)
        self.q_rot = torch.empty((H, T, hd), **f16)
        self.rope_cs = torch.empty((T, hd // 2, 2), dtype=torch.float32, device=dev)
        self.attn = torch.empty((T, H * hd), **f16)
        self.o = torch.empty((T, D), **f16)
        self.gate_up = torch.empty((T, 2 * I), **f16)
        self.act = torch.empty((T, I), **f16)
        self.down = torch.empty((T, D), **f16)
        self.logits = torch.empty((T, args.vocab_size), **f16)
        W = (H + 2 * G) * hd
        can_fold = self.swiglu and ops.small_supported(T, W, D, norm=True) \
            and ops.small_supported(T, D, H * hd) and ops.small_supported(T, 2 * I, D, norm=True, swiglu=True) \
            and ops.small_supported(T, D, I) and self._scales_within(ops.SMALL_SCALE_LIMIT)
        if folded and not can_fold:
            raise ValueError("the small-row form does not take these shapes or weights")
        self.folded = can_fold if folded is None else bool(folded)
        # within the folded form: rotation and cache append in the q|k|v launch
        self.rope_folded = self.folded and ops.qkv_rope_small_supported(T, D, H, G, hd)
        L = _lib.lib()
        head = model.lm_head if not args.tie_word_embeddings else model.model.embed_tokens
        need = max(L.eagle_qmm_workspace_bytes(T, n, k) for n, k in
                   (((H + 2 * G) * hd, D), (D, H * hd), (2 * I, D), (D, I), (head.weight.shape[0], D)))
        ops.workspace("qmm", need, dev)
        ops.workspace("attn", L.eagle_tree_attention_workspace_bytes(H, hd, self.max_len), dev)
        ops.workspace("topk", L.eagle_logsoftmax_topk_workspace_bytes(T, args.vocab_size), dev)

    def _scales_within(self, limit):
        """Every quantisation scale of the layers' matrices is below `limit` in magnitude."""
        worst = 0.0
        for i, layer in enumerate(self.model.model.layers):
            for sc in (self.qkv_w[i][1], layer.self_attn.o_proj.scales, self.gu_w[i][1], layer.mlp.down_proj.scales):
                worst = max(worst, float(sc.abs().max()))
        return worst < limit

    def forward(self, tokens, positions, write_len, attn_len, mask_words, Tk, head=True):
        """head=False: stop after the last layer (a pass that is only run for its KV rows)."""
        m, args = self.model, self.args
        H, G, hd = args.num_attention_heads, args.num_key_value_heads, args.head_dim
        W = (H + 2 * G) * hd
        emb = m.model.embed_tokens
        ops.embed(tokens, emb.weight, emb.scales, emb.biases, out=self.h)
        layers = m.model.layers
        at0 = layers[0].self_attn
        ops.rope_table(positions, at0._inv_freqs, at0._scaling_factor, out=self.rope_cs)
        def attend(at, c):
            ops.draft_attention(self.q_rot, c.keys[0], c.values[0], mask_words, attn_len, Tk, at.scale,
                                max_len=self.max_len, out=self.attn)

        if self.folded:
            # per layer: q|k|v with the input norm folded in, rope + cache append, attention, o with
            # the residual, gate|up with the post-attention norm and SwiGLU, down with the residual
            q_lin, k_lin, v_lin = self.qkv, self.qkv[:, H * hd:], self.qkv[:, (H + G) * hd:]
            eps = args.rms_norm_eps
            for i, layer in enumerate(layers):
                at, mlp, c = layer.self_attn, layer.mlp, self.cache[i]
                w, sc, bi, b = self.qkv_w[i]
                if self.rope_folded:
                    ops.qkv_rope_small(self.h, w, sc, bi, b, self.rope_cs, self.q_rot, c.keys[0], c.values[0],
                                       write_len, H, G, hd, norm_weight=layer.input_layernorm.weight, eps=eps)
                else:
                    ops.quantized_matmul_small(self.h, w, sc, bi, bias=b, out=self.qkv,
                                               norm_weight=layer.input_layernorm.weight, eps=eps)
                    ops.rope_kv_append(q_lin, k_lin, v_lin, positions, at._inv_freqs, at._scaling_factor,
                                       self.q_rot, c.keys[0], c.values[0], write_len, H, G, hd, row_stride=W,
                                       rope_cs=self.rope_cs)
                attend(at, c)
                o = at.o_proj
                ops.quantized_matmul_small(self.attn, o.weight, o.scales, o.biases, bias=o.bias, out=self.h,
                                           residual=self.h)
                w, sc, bi, b = self.gu_w[i]
                ops.quantized_matmul_small(self.h, w, sc, bi, bias=b, out=self.act,
                                           norm_weight=layer.post_attention_layernorm.weight, eps=eps, swiglu=True)
                d = mlp.down_proj
                ops.quantized_matmul_small(self.act, d.weight, d.scales, d.biases, bias=d.bias, out=self.h,
                                           residual=self.h)
            ops.rms_norm(self.h, m.model.norm.weight, eps, out=self.hn)
        else:
            ops.rms_norm(self.h, layers[0].input_layernorm.weight, args.rms_norm_eps, out=self.hn)
            for i in range(len(layers)):
                emit_layer(self, i, write_len, attend, positions=positions)
        if not head:
            return None
        head = m.model.embed_tokens if args.tie_word_embeddings else m.lm_head
        ops.quantized_matmul(self.hn, head.weight, head.scales, head.biases, out=self.logits)
        return self.logits


class ChunkPass:
    """A causal pass of R rows (a multiple of 32, at most 2048) through a decoder: the linear
    layers see all R rows at once (the tiled GEMM form of the matmul above 32 rows), so do rope
    and the cache append; attention runs per piece of 32 rows (all pieces in one launch), every
    piece seeing the cache rows before it and its own rows causally.  Rows are appended at the cache length, which advances by R."""

    PIECE = 32

    def __init__(self, model, cache, R, max_len=None, head=True):
        args = model.args
        self.model, self.cache, self.args, self.R, self.head = model, cache, args, R, head
        dev = model.device
        P = self.PIECE
        if R % P or R < P or R > MAX_CHUNK:
            raise ValueError(f"rows must be a multiple of 32 between 32 and {MAX_CHUNK}")
        self.pieces = R // P
        D, I = args.hidden_size, args.intermediate_size
        H, G, hd = args.num_attention_heads, args.num_key_value_heads, args.head_dim
        self.max_len = max_len or cache[0].capacity
        self.T = R
        # above 32 rows: the tiled GEMM form everywhere, gate|up with the SwiGLU epilogue
        self.swiglu = bool(ops.swiglu_supported(R, args.intermediate_size, args.hidden_size))
        self.qkv_w, self.gu_w = fuse_projections(model, self.swiglu)
        self.slab = {"qkv": 0, "o": 0, "down": 0}
        f16 = dict(dtype=torch.float16, device=dev)
        i32 = dict(dtype=torch.int32, device=dev)
        self.tokens = torch.zeros(R, **i32)
        self.h = torch.empty((R, D), **f16)
        self.hn = torch.empty((R, D), **f16)
        self.qkv = torch.empty((R, (H + 2 * G) * hd), **f16)
        self.q_rot = torch.empty((H, R, hd), **f16)
        self.rope_cs = torch.empty((R, hd // 2, 2), dtype=torch.float32, device=dev)
        self.attn = torch.empty((R, H * hd), **f16)
        self.o = torch.empty((R, D), **f16)
        self.gate_up = torch.empty((R, 2 * I), **f16)
        self.act = torch.empty((R, I), **f16)
        self.down = torch.empty((R, D), **f16)
        self.logits = torch.empty((P, args.vocab_size), **f16)      # of the last piece only
        self.piece_off = (torch.arange(self.pieces, **i32) * P).contiguous()
        self.piece_len = torch.zeros(self.pieces, **i32)
        self.arange = torch.arange(P, **i32)
        self.positions = torch.zeros(R, **i32)
        self.len_dev = cache[0].len_dev
        L = _lib.lib()
        hw = model.lm_head if not args.tie_word_embeddings else model.model.embed_tokens
        ops.workspace("qmm", L.eagle_qmm_workspace_bytes(P, hw.weight.shape[0], D), dev)
        ops.workspace("attn_chunk", L.eagle_causal_attention_workspace_bytes(R, H, hd, self.max_len), dev)
        self.graph = None

    def enqueue(self):
        L = _lib.lib()
        st = _stream()
        m, args, P = self.model, self.args, self.PIECE
        H, G, hd = args.num_attention_heads, args.num_key_value_heads, args.head_dim
        W = (H + 2 * G) * hd
        layers = m.model.layers
        at0 = layers[0].self_attn
        # cache length, positions and rotary table of every piece, once for all layers
        _lib.check(L.eagle_tree_positions(_ptr(self.piece_off), _ptr(self.len_dev), _ptr(self.piece_len),
                                          self.pieces, st), "piece lengths")
        for j in range(self.pieces):
            pos = self.positions[j * P:(j + 1) * P]
            _lib.check(L.eagle_tree_positions(_ptr(self.arange), _ptr(self.piece_len[j:j + 1]), _ptr(pos),
                                              P, st), "positions")
        ops.rope_table(self.positions, at0._inv_freqs, at0._scaling_factor, out=self.rope_cs)
        emb = m.model.embed_tokens
        ops.embed(self.tokens, emb.weight, emb.scales, emb.biases, out=self.h)
        ops.rms_norm(self.h, layers[0].input_layernorm.weight, args.rms_norm_eps, out=self.hn)
        # all rows at once through the linear layers, the rotation and the cache append; then
        # attention with one 32-row piece per workgroup column
        def attend(at, c):
            ops.causal_attention(self.q_rot, c.keys[0], c.values[0], self.piece_len, at.scale,
                                 max_len=self.max_len, out=self.attn)

        for i in range(len(layers)):
            emit_layer(self, i, self.len_dev, attend)
        if self.head:
            hw = m.model.embed_tokens if args.tie_word_embeddings else m.lm_head
            ops.quantized_matmul(self.hn[self.R - P:], hw.weight, hw.scales, hw.biases, out=self.logits)
        _lib.check(L.eagle_advance_len(_ptr(self.len_dev), self.R, st), "advance_len")

    def capture(self):
        saved = self.len_dev.clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self.enqueue()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.len_dev.copy_(saved)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.enqueue()
        self.len_dev.copy_(saved)
        torch.cuda.synchronize()
        return self

    def run(self):
        if self.graph is not None:
            self.graph.replay()
        else:
            self.enqueue()


class CausalPrefill:
    """The prompt pass (mlx_eagle.py:522-533) as causal passes of up to `chunk` rows (512, the
    reference's prefill_step_size), each one HIP-graph replay; a last piece that is not a
    multiple of 32 is padded (its extra rows land beyond the cache length and no real row sees
    them).  One captured pass per distinct row count."""

    def __init__(self, model, cache, max_len=None, head=True, chunk=512, graphs=True):
        self.model, self.cache, self.head, self.max_len = model, cache, head, max_len
        self.chunk, self.graphs = chunk, graphs
        self.passes = {}

    def _pass(self, R, capture=True):
        p = self.passes.get(R)
        if p is None:
            p = self.passes[R] = ChunkPass(self.model, self.cache, R, max_len=self.max_len, head=self.head)
        if capture and self.graphs and p.graph is None:
            p.capture()
        return p

    def prepare(self, n, capture=True):
        """Build (and, with capture, record) the passes a prompt of n tokens needs.  Several
        models sharing the workspaces should all be built before any of them is captured, so
        that no workspace is outgrown after an address went into a graph."""
        while n > 0:
            R = min(self.chunk, (n + 31) // 32 * 32)
            self._pass(R, capture)
            n -= R
        return self

    def __call__(self, ids):
        """Append the tokens `ids` (1-D) to the cache; returns the logits row of the last one
        ([1,V] view of a static buffer) when the pass has a head."""
        ids = ids.reshape(-1).to(torch.int32)
        n = ids.numel()
        start = self.cache[0].offset
        if start + (n + 31) // 32 * 32 > self.cache[0].capacity:
            raise ValueError("KV cache too small for the padded prompt pass")
        self.cache[0].sync_len()
        s, last = 0, None
        while s < n:
            R = min(self.chunk, (n - s + 31) // 32 * 32)
            p = self._pass(R)
            part = ids[s:s + R]
            p.tokens.zero_()
            p.tokens[:part.numel()] = part
            p.run()
            last, last_rows = p, part.numel()
            s += R
        for c in self.cache:
            c.offset = start + n
        self.cache[0].sync_len()
        if not self.head:
            return None
        row = last_rows - (last.R - ChunkPass.PIECE) - 1     # within the last piece
        if row < 0:
            raise RuntimeError("the last token does not lie in the last piece")
        return last.logits[row:row + 1]


class SpeculativeDecoder:
    """Greedy tree-speculative generation with the step on the device.

        dec = SpeculativeDecoder(base_model, draft_model, capacity=..., k=8, depth=3,
                                 verify_num_tokens=31)
        dec.prefill(prompt)          # both models, chunked causal passes; first token
        dec.capture()                # optional: one HIP graph per step
        tokens = dec.generate(n_steps)
    """

    def __init__(self, base_model, draft_model, capacity, k=8, depth=3, verify_num_tokens=31,
                 max_out=8192, slab_plan=None, draft_slab_plan=None, draft_folded=None,
                 prefill_step_size=MAX_CHUNK):
        from .cache import make_prompt_cache

        if k != Y_LEN:
            raise ValueError("the step is laid out for k = 8 candidates per node")
        if verify_num_tokens + 1 > TREE_SLOTS or k * depth > 64 or depth + 2 > Y_LEN:
            raise ValueError(f"tree does not fit: at most {TREE_SLOTS - 1} draft nodes, k * depth <= 64, "
                             "depth <= 6")
        if k + k * k * depth < verify_num_tokens:
            raise ValueError("fewer candidates than draft nodes")
        self.base_model, self.draft_model = base_model, draft_model
        self.k, self.depth, self.V = k, depth, verify_num_tokens
        self.capacity = capacity
        dev = base_model.device
        self.dev = dev
        self.base_cache = make_prompt_cache(base_model, capacity=capacity)
        self.draft_cache = make_prompt_cache(draft_model, capacity=capacity)
        self.verifier = TreeVerifier(base_model, self.base_cache, total_tokens=verify_num_tokens,
                                     max_len=capacity, slab_plan=slab_plan)
        self.draft = DecoderPass(draft_model, self.draft_cache, k, max_len=capacity, slab_plan=draft_slab_plan,
                                 folded=draft_folded)
        i32 = dict(dtype=torch.int32, device=dev)
        self.y = torch.zeros(Y_LEN, **i32)
        self.root_token = torch.zeros(1, **i32)
        self.draft_len = self.draft_cache[0].len_dev
        self.expand_len = torch.zeros(1, **i32)
        self.write_len = torch.zeros(1, **i32)
        self.positions = torch.zeros(k, **i32)
        self.arange = torch.arange(k, **i32)
        self.levels = torch.arange(depth, **i32)[:, None].repeat(1, k).contiguous()
        causal = torch.tril(torch.ones((k, k), dtype=torch.bool, device=dev))
        self.causal_words = ops.mask_to_words(causal)
        self.topk_index = torch.zeros((k, k), **i32)
        self.topk_score = torch.zeros((k, k), dtype=torch.float16, device=dev)
        self.buf = _level_buffers(k, depth, dev)
        self.out_tokens = torch.zeros(max_out, **i32)
        self.out_count = torch.zeros(1, **i32)
        self.max_out = max_out
        self.graph = None
        self.first = None
        self._prefill = None
        # Rows per prompt pass (mlx_eagle.py:505, where the default is 512).  The result does not
        # depend on it; the matmuls of a pass run faster with more rows (2048-token prompt, both
        # models of the loop benchmark: 54.0 / 45.2 / 39.8 ms at 512 / 1024 / 2048 rows per pass).
        self.prefill_step_size = min(int(prefill_step_size), MAX_CHUNK)

    def prepare(self, prompt_len=0):
        """Build and capture the prompt passes for a prompt of this length (done by the first
        prefill otherwise)."""
        if self._prefill is None:
            self._prefill = (CausalPrefill(self.draft_model, self.draft_cache, self.capacity, head=False,
                                           chunk=self.prefill_step_size),
                             CausalPrefill(self.base_model, self.base_cache, self.capacity,
                                           chunk=self.prefill_step_size))
        if prompt_len:
            for p in self._prefill:
                p.prepare(prompt_len, capture=False)     # every workspace at its final size first
            for p in self._prefill:
                p.prepare(prompt_len)
        return self

    def prefill(self, prompt):
        """mlx_eagle.py:522-535: both models read the prompt; the first token is the target's
        argmax at its last position."""
        self.prepare(prompt.numel())
        for cache in (self.base_cache, self.draft_cache):     # a new sequence: empty caches
            for c in cache:
                c.offset = 0
            cache[0].sync_len()
        self._prefill[0](prompt)
        first = ops.argmax_rows(self._prefill[1](prompt))
        self.y.zero_()
        self.y[:1] = first
        self.root_token.copy_(first)
        self.verifier.result.zero_()            # accept_length 0
        self.out_count.zero_()
        self.base_cache[0].sync_len()
        self.draft_cache[0].sync_len()
        self.first = int(first.item())
        self._bound = self.base_cache[0].offset
        return self.first

    def enqueue_step(self):
        L = _lib.lib()
        st = _stream()
        k, depth, ver, d, b = self.k, self.depth, self.verifier, self.draft, self.buf
        accept = ver.result
        # draft pass over the accepted tokens and the bonus token (mlx_eagle.py:400-408)
        _lib.check(L.eagle_tree_positions(_ptr(self.arange), _ptr(self.draft_len), _ptr(self.positions),
                                          k, st), "positions")
        logits = d.forward(self.y, self.positions, self.draft_len, self.draft_len, self.causal_words, k)
        _lib.check(L.eagle_spec_begin(_ptr(self.draft_len), _ptr(accept), _ptr(self.expand_len),
                                      _ptr(self.write_len), st), "spec_begin")
        # level 0: the k most likely continuations of the bonus token (mlx_eagle.py:410-412)
        ops.logsoftmax_topk(logits, k, 0, row_index=accept[1:2],
                            out=(self.topk_index[:1], self.topk_score[:1]))
        draft_tree_init(self.topk_index, self.topk_score, k, b)
        for i in range(depth):
            _lib.check(L.eagle_tree_positions(_ptr(self.levels[i]), _ptr(self.expand_len),
                                              _ptr(self.positions), k, st), "positions")
            logits = d.forward(b["cur_ids"], self.positions, self.write_len, self.expand_len,
                               b["mask_words"], k * (i + 1))
            ops.logsoftmax_topk(logits, k, 1, out=(self.topk_index, self.topk_score))
            draft_tree_level(self.topk_index, self.topk_score, i, k, depth, b)
            _lib.check(L.eagle_advance_len(_ptr(self.write_len), k, st), "advance_len")
        process_draft_tree_device(b["saved_scores"], b["saved_tokens"], b["parents"], self.root_token, k,
                                  self.V, out=(ver.tree_position_ids, ver.mask_index, ver.tokens,
                                               ver.mask_bits))
        ver.forward()        # target pass, argmax, acceptance, KV compaction, target length
        _lib.check(L.eagle_spec_update(_ptr(accept), _ptr(ver.accepted_tokens), _ptr(self.y), Y_LEN,
                                       _ptr(self.draft_len), _ptr(self.expand_len),
                                       _ptr(self.root_token), _ptr(self.out_tokens),
                                       _ptr(self.out_count), self.max_out, st), "spec_update")

    def _state(self):
        return [self.y, self.root_token, self.draft_len, self.verifier.len_dev, self.verifier.result,
                self.out_count, self.out_tokens]

    def capture(self):
        """Record one step into a HIP graph (after an eager run on a side stream); the loop
        state is restored afterwards, cache rows written meanwhile lie beyond the lengths."""
        saved = [t.clone() for t in self._state()]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self.enqueue_step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        for t, s in zip(self._state(), saved):
            t.copy_(s)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.enqueue_step()
        for t, s in zip(self._state(), saved):
            t.copy_(s)
        torch.cuda.synchronize()
        return self

    def step(self):
        if self.graph is not None:
            self.graph.replay()
        else:
            self.enqueue_step()

    def generate(self, n_steps):
        """Run n_steps speculative steps; returns the emitted tokens (without the first one).
        The caches must have room for n_steps * (depth + 2) + max(8 * (depth + 1), tree tokens)
        more rows."""
        # upper bound of the rows either cache can hold after these steps (the lengths live on
        # the device; a step adds at most depth + 2 tokens and writes up to 8 * (depth + 1) draft
        # rows or the tree's rows beyond the length)
        self._bound += n_steps * (self.depth + 2)
        if self._bound + max(Y_LEN * (self.depth + 1), self.verifier.T) > self.capacity:
            self._bound -= n_steps * (self.depth + 2)
            raise ValueError(f"KV caches of {self.capacity} rows are too small for {n_steps} more steps")
        for _ in range(n_steps):
            self.step()
        n = int(self.out_count.item())
        return self.out_tokens[:min(n, self.max_out)].tolist()
