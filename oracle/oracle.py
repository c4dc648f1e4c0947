"""ctypes front end of the CPU checker (oracle/eagle_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke check and the
cpu_baseline leg of bench.py.  The shipped package never imports this module.

All half-precision tensors are numpy float16 arrays (C-contiguous).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force=False):
    """Compile liboracle.so with the committed Makefile."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True, capture_output=True)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _h(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.float16, a.dtype
    return a


class weight_rounding:
    """Context manager: inside it `qmm` rounds every dequantised weight to fp16 before the
    product, as the reference's Metal kernel holds them
    (kernels/progression/simd_no_swizzle_cast.metal:82-84); outside it s*q + b stays in fp32."""

    def __init__(self, on=True):
        self.on = bool(on)

    def __enter__(self):
        lib().orc_set_weight_rounding(ctypes.c_int(int(self.on)))
        return self

    def __exit__(self, *exc):
        lib().orc_set_weight_rounding(ctypes.c_int(0))
        return False


def qmm(x, w, scales, biases, bias=None):
    """out[..., N] = x[..., K] . dequant(w)[N, K]^T  (4 bit, group 64), fp16."""
    x = _h(x)
    w = np.ascontiguousarray(w)
    assert w.dtype == np.uint32
    scales, biases = _h(scales), _h(biases)
    K = x.shape[-1]
    N = w.shape[0]
    assert w.shape[1] * 8 == K and scales.shape == (N, K // 64) == biases.shape
    M = x.size // K
    out = np.empty((M, N), np.float16)
    bp = _p(_h(bias)) if bias is not None else None
    rc = lib().orc_qmm_w4g64(_p(x), _p(w), _p(scales), _p(biases), bp, _p(out),
                             ctypes.c_int(M), ctypes.c_int(N), ctypes.c_int(K))
    assert rc == 0, rc
    return out.reshape(*x.shape[:-1], N)


def embed(ids, w, scales, biases):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    V, D8 = w.shape
    D = D8 * 8
    out = np.empty((ids.size, D), np.float16)
    rc = lib().orc_embed_w4g64(_p(ids), _p(np.ascontiguousarray(w)), _p(_h(scales)),
                               _p(_h(biases)), _p(out), ctypes.c_int(ids.size),
                               ctypes.c_int(D), ctypes.c_int(V))
    assert rc == 0, rc
    return out.reshape(*ids.shape, D)


def rope_arrayed(x, positions, inv_freqs, scaling_factor=1.0):
    """x [B,H,L,hd] fp16, positions [B,L] int, inv_freqs [hd/2] fp32."""
    x = _h(x)
    B, H, L, hd = x.shape
    pos = np.ascontiguousarray(positions, dtype=np.int32).reshape(B, L)
    inv = np.ascontiguousarray(inv_freqs, dtype=np.float32)
    assert inv.shape == (hd // 2,)
    out = np.empty_like(x)
    rc = lib().orc_rope_arrayed(_p(x), _p(pos), _p(inv), ctypes.c_float(scaling_factor),
                                _p(out), *(ctypes.c_int(v) for v in (B, H, L, hd)))
    assert rc == 0, rc
    return out


def tree_attention(q, k, v, mask, scale, S=None):
    """q [H,T,hd]; k, v [G,cap,hd] (first S rows used); mask [T,S] additive fp16."""
    q, k, v, mask = _h(q), _h(k), _h(v), _h(mask)
    H, T, hd = q.shape
    G, cap, _ = k.shape
    if S is None:
        S = cap
    assert mask.shape == (T, S) and v.shape == k.shape
    out = np.empty_like(q)
    rc = lib().orc_tree_attention(_p(q), _p(k), _p(v), _p(mask), _p(out),
                                  ctypes.c_int(H), ctypes.c_int(G), ctypes.c_int(T),
                                  ctypes.c_int(S), ctypes.c_int(hd), ctypes.c_long(cap),
                                  ctypes.c_float(scale))
    assert rc == 0, rc
    return out


def rmsnorm(x, w, eps):
    x, w = _h(x), _h(w)
    D = x.shape[-1]
    out = np.empty_like(x)
    lib().orc_rmsnorm(_p(x), _p(w), ctypes.c_float(eps), _p(out),
                      ctypes.c_int(x.size // D), ctypes.c_int(D))
    return out


def silu_mul(g, u):
    g, u = _h(g), _h(u)
    out = np.empty_like(g)
    lib().orc_silu_mul(_p(g), _p(u), _p(out), ctypes.c_long(g.size))
    return out


def add(a, b):
    a, b = _h(a), _h(b)
    out = np.empty_like(a)
    lib().orc_add(_p(a), _p(b), _p(out), ctypes.c_long(a.size))
    return out


def argmax_rows(logits):
    logits = _h(logits)
    V = logits.shape[-1]
    R = logits.size // V
    out = np.empty(R, np.int32)
    lib().orc_argmax_rows(_p(logits), _p(out), ctypes.c_int(R), ctypes.c_long(V))
    return out.reshape(logits.shape[:-1])
