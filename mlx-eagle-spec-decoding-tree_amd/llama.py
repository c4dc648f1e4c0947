"""Llama / Qwen2 decoder with the tree-decoding arguments of the reference model
(mlx_llama.py:21-323): `Model(inputs, cache, mask, position_ids, flat_rope)`.

Same module tree and the same operator boundaries as the reference, so that the
fp16 roundings fall in the same places; every operator runs as a HIP kernel
behind the C ABI.  `patch_model(model, kernel)` is the plug-in seam of
mlx_model_fwd_bench.py:43-86.

The kernels serve at most 32 rows per linear layer.  Passes without a mask are causal
(mlx_llama.py:275-276); longer ones (the prompt) run as consecutive 32-token passes.
"""
from functools import reduce

import numpy as np
import torch

from . import ops
from .synth import ModelArgs, inv_freqs


CAUSAL_CHUNK = 32


class Module:
    """Minimal module base: attribute containers that can be walked and patched."""

    def children(self):
        for name, value in vars(self).items():
            if isinstance(value, Module):
                yield name, value, None
            elif isinstance(value, (list, tuple)):
                for i, v in enumerate(value):
                    if isinstance(v, Module):
                        yield name, v, i

    def named_modules(self, prefix=""):
        yield prefix, self
        for name, child, idx in self.children():
            path = f"{prefix}.{name}" if prefix else name
            if idx is not None:
                path = f"{path}.{idx}"
            yield from child.named_modules(path)

    def replace_modules(self, fn):
        """Depth-first: replace every child m by fn(path, m) when fn returns a new module."""
        def walk(mod, prefix):
            for name, child, idx in list(mod.children()):
                path = f"{prefix}.{name}" if prefix else name
                if idx is not None:
                    path = f"{path}.{idx}"
                new = fn(path, child)
                if new is not child:
                    if idx is None:
                        setattr(mod, name, new)
                    else:
                        getattr(mod, name)[idx] = new
                else:
                    walk(child, path)
        walk(self, "")


class QuantizedLinear(Module):
    """4-bit group-64 linear layer in the MLX layout (weight uint32 [N, K/8],
    scales / biases fp16 [N, K/64], optional fp16 bias [N])."""

    def __init__(self, weight, scales, biases, bias=None, group_size=64, bits=4):
        self.weight, self.scales, self.biases = weight, scales, biases
        self.bias = bias
        self.group_size, self.bits = group_size, bits

    def __call__(self, x):
        return ops.quantized_matmul(x, self.weight, self.scales, self.biases,
                                    group_size=self.group_size, bits=self.bits, bias=self.bias)


class QuantizedEmbedding(Module):
    def __init__(self, weight, scales, biases, group_size=64, bits=4):
        self.weight, self.scales, self.biases = weight, scales, biases
        self.group_size, self.bits = group_size, bits

    def __call__(self, ids):
        return ops.embed(ids, self.weight, self.scales, self.biases)

    def as_linear(self, x):
        """Tied output head: the embedding matrix used as a linear layer (mlx_llama.py:310)."""
        return ops.quantized_matmul(x, self.weight, self.scales, self.biases,
                                    group_size=self.group_size, bits=self.bits)


class RMSNorm(Module):
    def __init__(self, weight, eps):
        self.weight, self.eps = weight, eps

    def __call__(self, x):
        return ops.rms_norm(x, self.weight, self.eps)


class Attention(Module):
    """mlx_llama.py:60-196."""

    def __init__(self, args: ModelArgs, layer, device):
        self.n_heads = args.num_attention_heads
        self.n_kv_heads = args.num_key_value_heads
        self.head_dim = args.head_dim
        self.scale = self.head_dim ** -0.5
        self.q_proj, self.k_proj = layer["q_proj"], layer["k_proj"]
        self.v_proj, self.o_proj = layer["v_proj"], layer["o_proj"]
        inv, scaling = inv_freqs(args)
        self._inv_freqs = torch.from_numpy(inv).to(device)
        self._scaling_factor = scaling

    def __call__(self, x, mask=None, cache=None, position_ids=None, flat_rope=False):
        B, L, D = x.shape
        queries, keys, values = self.q_proj(x), self.k_proj(x), self.v_proj(x)
        queries = queries.reshape(B, L, self.n_heads, -1).transpose(1, 2).contiguous()
        keys = keys.reshape(B, L, self.n_kv_heads, -1).transpose(1, 2).contiguous()
        values = values.reshape(B, L, self.n_kv_heads, -1).transpose(1, 2).contiguous()
        if cache is None:
            raise NotImplementedError("the tree path always runs with a KV cache")
        if isinstance(position_ids, torch.Tensor):
            pos = position_ids.to(torch.int32).reshape(B, L)
        else:
            # scalar offset (mlx_llama.py:163-172); flat_rope gives every token the same one
            start = cache.offset if position_ids is None else int(position_ids)
            step = 0 if flat_rope else 1
            pos = (start + step * torch.arange(L, dtype=torch.int32, device=x.device)).expand(B, L)
        queries = ops.rope_positions(queries, pos, self._inv_freqs, self._scaling_factor)
        keys = ops.rope_positions(keys, pos, self._inv_freqs, self._scaling_factor)
        keys, values = cache.update_and_fetch(keys, values)
        output = ops.scaled_dot_product_attention(queries, keys, values, cache=cache,
                                                  scale=self.scale, mask=mask)
        output = output.transpose(1, 2).reshape(B, L, -1)
        return self.o_proj(output)


class MLP(Module):
    def __init__(self, layer):
        self.gate_proj, self.down_proj, self.up_proj = layer["gate_proj"], layer["down_proj"], layer["up_proj"]

    def __call__(self, x):
        return self.down_proj(ops.silu_mul(self.gate_proj(x), self.up_proj(x)))


class TransformerBlock(Module):
    def __init__(self, args, layer, device):
        self.self_attn = Attention(args, layer, device)
        self.mlp = MLP(layer)
        self.input_layernorm = RMSNorm(layer["input_layernorm"], args.rms_norm_eps)
        self.post_attention_layernorm = RMSNorm(layer["post_attention_layernorm"], args.rms_norm_eps)

    def __call__(self, x, mask=None, cache=None, position_ids=None, flat_rope=False):
        r = self.self_attn(self.input_layernorm(x), mask, cache, position_ids=position_ids,
                           flat_rope=flat_rope)
        h = ops.add(x, r)
        r = self.mlp(self.post_attention_layernorm(h))
        return ops.add(h, r)


class LlamaModel(Module):
    def __init__(self, args, tensors, device):
        self.args = args
        self.embed_tokens = QuantizedEmbedding(*_qtuple(tensors, "model.embed_tokens")[:3])
        self.layers = []
        for i in range(args.num_hidden_layers):
            p = f"model.layers.{i}"
            layer = {
                "q_proj": _qlinear(tensors, f"{p}.self_attn.q_proj"),
                "k_proj": _qlinear(tensors, f"{p}.self_attn.k_proj"),
                "v_proj": _qlinear(tensors, f"{p}.self_attn.v_proj"),
                "o_proj": _qlinear(tensors, f"{p}.self_attn.o_proj"),
                "gate_proj": _qlinear(tensors, f"{p}.mlp.gate_proj"),
                "up_proj": _qlinear(tensors, f"{p}.mlp.up_proj"),
                "down_proj": _qlinear(tensors, f"{p}.mlp.down_proj"),
                "input_layernorm": tensors[f"{p}.input_layernorm.weight"],
                "post_attention_layernorm": tensors[f"{p}.post_attention_layernorm.weight"],
            }
            self.layers.append(TransformerBlock(args, layer, device))
        self.norm = RMSNorm(tensors["model.norm.weight"], args.rms_norm_eps)

    def __call__(self, inputs, cache=None, mask=None, position_ids=None, flat_rope=False):
        if cache is None:
            raise NotImplementedError("the tree path always runs with a KV cache")
        L = inputs.shape[1]
        h = self.embed_tokens(inputs)
        if mask is None:
            # causal over the new tokens, everything in the cache visible (mlx_llama.py:275-276)
            offset = cache[0].offset
            mask = torch.zeros((1, 1, L, offset + L), dtype=h.dtype, device=h.device)
            mask[..., offset:] = torch.triu(
                torch.full((L, L), float("-inf"), dtype=h.dtype, device=h.device), diagonal=1)
        mask = mask.to(h.dtype)                                    # mlx_llama.py:278
        for layer, c in zip(self.layers, cache):
            h = layer(h, mask, cache=c, position_ids=position_ids, flat_rope=flat_rope)
        return self.norm(h)


class Model(Module):
    """mlx_llama.py:289-323."""

    def __init__(self, args: ModelArgs, tensors, device):
        self.args = args
        self.model_type = args.model_type
        self.device = device
        self.model = LlamaModel(args, tensors, device)
        if not args.tie_word_embeddings:
            self.lm_head = _qlinear(tensors, "lm_head")

    @classmethod
    def from_numpy(cls, args, weights, device):
        """weights: flat dict of numpy arrays keyed like an MLX-community checkpoint."""
        tensors = {}
        for k, v in weights.items():
            if v.dtype == np.uint32:
                v = v.view(np.int32)
            tensors[k] = torch.from_numpy(np.ascontiguousarray(v)).to(device)
        return cls(args, tensors, device)

    def __call__(self, inputs, cache=None, mask=None, position_ids=None, flat_rope=False):
        if mask is None and inputs.shape[1] > CAUSAL_CHUNK:
            # a long causal pass (prompt prefill, mlx_eagle.py:522-533) as consecutive passes of
            # at most 32 tokens: the kernels of this path take at most 32 rows
            if position_ids is not None or flat_rope:
                raise NotImplementedError("chunked causal passes take their positions from the cache")
            parts = [self(inputs[:, s:s + CAUSAL_CHUNK], cache)
                     for s in range(0, inputs.shape[1], CAUSAL_CHUNK)]
            return torch.cat(parts, dim=1)
        out = self.model(inputs, cache, mask=mask, position_ids=position_ids, flat_rope=flat_rope)
        if self.args.tie_word_embeddings:
            return self.model.embed_tokens.as_linear(out)
        return self.lm_head(out)

    @property
    def layers(self):
        return self.model.layers


def _qtuple(tensors, prefix):
    return (tensors[f"{prefix}.weight"], tensors[f"{prefix}.scales"], tensors[f"{prefix}.biases"],
            tensors.get(f"{prefix}.bias"))


def _qlinear(tensors, prefix):
    w, s, b, bias = _qtuple(tensors, prefix)
    return QuantizedLinear(w, s, b, bias)


def patch_model(model, kernel):
    """Replace every QuantizedLinear leaf by a layer that calls
    `kernel(x, weight, scales, biases, group_size)` for 8/16/24/32 rows and adds the
    bias afterwards; other row counts use the built-in path
    (mlx_model_fwd_bench.py:43-86)."""

    class NewQuantizedLinear(QuantizedLinear):
        def __init__(self, q):
            super().__init__(q.weight, q.scales, q.biases, q.bias, q.group_size, q.bits)

        def __call__(self, x):
            B = reduce(lambda a, b: a * b, x.shape[:-1], 1)
            if B in (8, 16, 24, 32):
                assert (x.shape[-1] % 128) == 0
                y = kernel(x, self.weight, self.scales, self.biases, self.group_size)
                if self.bias is not None:
                    y = ops.add(y, self.bias.expand_as(y).contiguous())
                return y
            return super().__call__(x)

    def swap(path, m):
        if type(m) is QuantizedLinear:
            return NewQuantizedLinear(m)
        return m

    model.replace_modules(swap)
    return model
