"""KV cache with the semantics the tree path relies on from mlx_lm's KVCache
(call sites: mlx_llama.py:178, mlx_eagle.py:139,336,369-376,393-394): buffers
`keys`, `values` [1, n_kv, capacity, head_dim], an integer `offset`,
`update_and_fetch` that appends at `offset`, and plain assignment to `offset`
to rewind.

The buffers are preallocated (no growth steps) and the length also lives in a
device scalar `len_dev`, so that kernels replayed from a HIP graph read the
current length from memory instead of from a launch argument.
"""
import torch


class KVCache:
    def __init__(self, n_kv_heads, head_dim, capacity, device, len_dev=None):
        self.keys = torch.zeros((1, n_kv_heads, capacity, head_dim), dtype=torch.float16, device=device)
        self.values = torch.zeros_like(self.keys)
        self.capacity = capacity
        self._offset = 0
        # one device scalar may be shared by every layer of a model
        self.len_dev = len_dev if len_dev is not None else torch.zeros(1, dtype=torch.int32, device=device)

    @property
    def offset(self):
        return self._offset

    @offset.setter
    def offset(self, value):
        self._offset = int(value)

    def sync_len(self):
        """Push the host offset to the device scalar (one tiny H2D copy)."""
        self.len_dev.fill_(self._offset)

    def update_and_fetch(self, keys, values):
        """Append [1, n_kv, L, hd] at `offset`; return views of the first offset+L rows."""
        L = keys.shape[2]
        end = self._offset + L
        if end > self.capacity:
            raise ValueError(f"KV cache capacity {self.capacity} exceeded ({end})")
        self.keys[:, :, self._offset:end] = keys
        self.values[:, :, self._offset:end] = values
        self._offset = end
        return self.keys[:, :, :end], self.values[:, :, :end]

    @property
    def state(self):
        return self.keys, self.values


def make_prompt_cache(model, capacity=4096):
    """One cache per layer (mlx_eagle.py:518-519); all layers share one device length."""
    args = model.args
    dev = model.device
    len_dev = torch.zeros(1, dtype=torch.int32, device=dev)
    return [KVCache(args.num_key_value_heads, args.head_dim, capacity, dev, len_dev)
            for _ in range(args.num_hidden_layers)]
