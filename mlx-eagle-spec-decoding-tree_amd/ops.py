"""Operator front end: reference call signatures on torch tensors, executed by the
HIP kernels of libeagle_mi355x.so through its C ABI.

torch only supplies device memory and the current stream.  There is no eager
or CPU fallback: every function raises if the library is missing or the tensor
is not on a GPU.
"""
from functools import reduce

import torch

from . import _lib

_WS = {}        # (device index, tag) -> workspace tensor
_RETIRED = []   # outgrown workspaces, kept allocated (see workspace())


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


def _need_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("eagle ops need GPU tensors (there is no CPU path)")


def _f16(t, name):
    if t.dtype != torch.float16:
        raise TypeError(f"{name} must be float16, got {t.dtype}")
    return t.contiguous()


def workspace(tag, nbytes, device):
    """A zero-initialised device buffer that persists between calls (and across
    HIP-graph replays).  It only grows; growing is not graph-capture safe, so
    capture callers size it first."""
    key = (device.index, tag)
    buf = _WS.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None:
            # a captured graph may still hold the old address, and beginning the next capture
            # returns every free block to the driver (torch.cuda.graph empties the allocator's
            # cache): a replay would then write to unmapped memory.  Outgrown buffers therefore
            # stay allocated until the process ends.
            _RETIRED.append(buf)
        buf = torch.zeros(max(int(nbytes), 1 << 16), dtype=torch.uint8, device=device)
        _WS[key] = buf
    return buf


ROW_PASS = 32        # rows of x the streaming kernel takes per launch


def as_packed_u32(w_q):
    """MLX packs into uint32; torch has weak uint32 support, so int32 storage of
    the same bits is accepted too."""
    if w_q.dtype not in (torch.uint32, torch.int32):
        raise TypeError(f"packed weights must be uint32/int32, got {w_q.dtype}")
    return w_q.contiguous()


def quantized_matmul(x, w_q, scales, biases, transpose=True, group_size=64, bits=4, bias=None,
                     out=None, tuned=None, gemm=None):
    """`mx.quantized_matmul(x, w, scales, biases, transpose=True, group_size=64, bits=4)`
    (any leading dims, flattened as qmm_kernel.py:99-100,136): the streaming kernel for 1..32
    rows of x, two passes of it for 33..64 rows (a tree above 32 tokens; faster there than the
    GEMM's few long-running workgroups: 21 against 31 us for 40 x 4608 x 3584, 44 against 185 us
    for 40 x 3584 x 18944), a tiled GEMM above that.
    `bias` ([N] fp16) is added after rounding, as the patched linear layer does
    (mlx_model_fwd_bench.py:70-71).  `tuned` forces a launch shape of the streaming kernel,
    `gemm=True` the tiled GEMM whatever the row count."""
    if not transpose:
        raise ValueError("only transpose=True (x @ dequant(w).T) is implemented")
    _need_cuda(x, w_q, scales, biases, bias)
    x = _f16(x, "x")
    w_q = as_packed_u32(w_q)
    scales, biases = _f16(scales, "scales"), _f16(biases, "biases")
    *lead, K = x.shape
    M = reduce(lambda a, b: a * b, lead, 1)
    N = w_q.shape[0]
    if w_q.shape[1] * 8 != K or tuple(scales.shape) != (N, K // 64) or tuple(biases.shape) != (N, K // 64):
        raise ValueError(f"shape mismatch: x {tuple(x.shape)}, w {tuple(w_q.shape)}, "
                         f"scales {tuple(scales.shape)}, biases {tuple(biases.shape)}")
    if bias is not None:
        bias = _f16(bias, "bias")
        if tuple(bias.shape) != (N,):
            raise ValueError("bias must have shape [N]")
    if out is None:
        out = torch.empty((*lead, N), dtype=torch.float16, device=x.device)
    L = _lib.lib()
    if M > 32 and tuned is not None:
        raise ValueError("launch shapes can be forced for at most 32 rows")
    if ROW_PASS < M <= 2 * ROW_PASS and not gemm:
        x2, out2 = x.reshape(M, K), out.view(M, N)
        for r0 in range(0, M, ROW_PASS):
            quantized_matmul(x2[r0:r0 + ROW_PASS], w_q, scales, biases, group_size=group_size, bits=bits,
                             bias=bias, out=out2[r0:r0 + ROW_PASS])
        return out
    if M > 32 or gemm:
        # many rows (the prompt pass): the tiled GEMM form
        rc = L.eagle_qmm_gemm_w4g64_f16(_ptr(x), _ptr(w_q), _ptr(scales), _ptr(biases), _ptr(bias),
                                        _ptr(out), M, N, K, group_size, bits, _stream())
        _lib.check(rc, "quantized_matmul")
        return out
    if tuned is None and M <= QMV_MAX_ROWS and qmv_preferred(N, K, M) and group_size == 64 and bits == 4:
        # one row (or the few rows `qmv_preferred` takes): the vector-ALU kernel, faster than a 16-row
        # matrix tile with most rows idle wherever the matrix has enough rows to fill the GPU with
        # short K
        rc = L.eagle_qmv_rows_w4g64_f16(_ptr(x), _ptr(w_q), _ptr(scales), _ptr(biases), _ptr(bias),
                                        _ptr(out), M, N, K, group_size, bits, _stream())
        _lib.check(rc, "quantized_matmul")
        return out
    if tuned is None:
        ws = workspace("qmm", L.eagle_qmm_workspace_bytes(M, N, K), x.device)
        rc = L.eagle_qmm_w4g64_f16(_ptr(x), _ptr(w_q), _ptr(scales), _ptr(biases), _ptr(bias),
                                   _ptr(out), M, N, K, group_size, bits, _ptr(ws), ws.numel(),
                                   _stream())
    else:
        # tuned = (nw, phases, splits, ranges[, unit_cols]): forced launch shape
        if group_size != 64 or bits != 4:
            raise ValueError("only group_size=64, bits=4 is supported")
        nw, phases, splits, ranges = (int(v) for v in tuned[:4])
        unit_cols = int(tuned[4]) if len(tuned) > 4 else 0
        need = L.eagle_qmm_workspace_bytes_tuned(M, N, splits)
        ws = workspace("qmm", need, x.device)
        rc = L.eagle_qmm_w4g64_f16_tuned(_ptr(x), _ptr(w_q), _ptr(scales), _ptr(biases),
                                         _ptr(bias), _ptr(out), M, N, K, nw, phases, splits, ranges,
                                         unit_cols, _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "quantized_matmul")
    return out


def slab_count(K, steps_per_slab):
    """K slabs of the slab form of the matmul; 0 when it does not take this K."""
    return _lib.lib().eagle_qmm_slab_count(int(K), int(steps_per_slab))


def slab_steps(M, N, K):
    """K steps per slab the library recommends for the slab form of this product, 0 where the
    streaming kernel is the faster form."""
    return _lib.lib().eagle_qmm_slab_steps(int(M), int(N), int(K))


def slab_rows(M):
    """Rows of a partial tile of the slab form for M rows of x."""
    if M < 1 or M > 64:
        raise ValueError("the slab form takes 1..64 rows")
    return 64 if M > 32 else 32


def quantized_matmul_slabs(x, w_q, scales, biases, steps_per_slab, partial=None, tiled=None):
    """The product for 1..64 rows as fp32 partial sums of K slabs, [slabs, R, N] with R = 32 up
    to 32 rows and 64 above (`slab_rows`): the result is fp16(partial.sum(0)) (+ bias), formed by
    `slab_sum`, `rms_norm_slabs` or `rope_kv_append_slabs`.  K % 128 == 0.
    tiled: the same matrix as `TiledWeights`; the kernel then reads that copy."""
    _need_cuda(x, w_q, scales, biases)
    x = _f16(x, "x")
    if tiled is not None and x.numel() // x.shape[-1] <= 64:
        return _matmul_slabs_tiled(x, tiled, steps_per_slab, partial)
    w_q = as_packed_u32(w_q)
    scales, biases = _f16(scales, "scales"), _f16(biases, "biases")
    *lead, K = x.shape
    M = reduce(lambda a, b: a * b, lead, 1)
    N = w_q.shape[0]
    if w_q.shape[1] * 8 != K or tuple(scales.shape) != (N, K // 64) or tuple(biases.shape) != (N, K // 64):
        raise ValueError(f"shape mismatch: x {tuple(x.shape)}, w {tuple(w_q.shape)}, "
                         f"scales {tuple(scales.shape)}, biases {tuple(biases.shape)}")
    slabs = slab_count(K, steps_per_slab)
    if slabs < 1:
        raise ValueError(f"the slab form does not take K = {K} with {steps_per_slab} steps per slab")
    R = slab_rows(M)
    if partial is None:
        partial = torch.empty((slabs, R, N), dtype=torch.float32, device=x.device)
    elif partial.dtype != torch.float32 or partial.numel() < slabs * R * N or not partial.is_contiguous():
        raise ValueError(f"partial must be a contiguous fp32 buffer of at least slabs * {R} * N elements")
    rc = _lib.lib().eagle_qmm_slab_partial_w4g64(_ptr(x), _ptr(w_q), _ptr(scales), _ptr(biases),
                                                 _ptr(partial), partial.numel() * 4, M, N, K, 64, 4,
                                                 int(steps_per_slab), _stream())
    _lib.check(rc, "quantized_matmul_slabs")
    return partial


def _matmul_slabs_tiled(x, tiled, steps_per_slab, partial):
    *lead, K = x.shape
    M = reduce(lambda a, b: a * b, lead, 1)
    N = tiled.N
    if K != tiled.K:
        raise ValueError(f"shape mismatch: x {tuple(x.shape)}, tiled weights [{N}, {tiled.K}]")
    slabs = slab_count(K, steps_per_slab)
    if slabs < 1:
        raise ValueError(f"the slab form does not take K = {K} with {steps_per_slab} steps per slab")
    R = slab_rows(M)
    if partial is None:
        partial = torch.empty((slabs, R, N), dtype=torch.float32, device=x.device)
    elif partial.dtype != torch.float32 or partial.numel() < slabs * R * N or not partial.is_contiguous():
        raise ValueError(f"partial must be a contiguous fp32 buffer of at least slabs * {R} * N elements")
    rc = _lib.lib().eagle_qmm_slab_partial_tiled_w4g64(_ptr(x), _ptr(tiled.wt), _ptr(tiled.sbt), _ptr(partial),
                                                       partial.numel() * 4, M, N, K, int(steps_per_slab),
                                                       int(tiled.small), _stream())
    _lib.check(rc, "quantized_matmul_slabs (tiled)")
    return partial


def slab_sum(partial, slabs, M, N, bias=None, out=None):
    """fp16(sum of the slabs, in slab order) (+ bias) -> [M, N]."""
    _need_cuda(partial, bias)
    if out is None:
        out = torch.empty((M, N), dtype=torch.float16, device=partial.device)
    rc = _lib.lib().eagle_slab_sum_f16(_ptr(partial), int(slabs), _ptr(bias), _ptr(out), M, N, _stream())
    _lib.check(rc, "slab_sum")
    return out


def qmm_plan(M, N, K):
    """The launch shape the library picks: (streaming waves, phases, K slabs, tile ranges,
    columns per unit)."""
    import ctypes
    plan = (ctypes.c_int * 5)()
    _lib.check(_lib.lib().eagle_qmm_plan(M, N, K, plan), "qmm_plan")
    return tuple(plan)


def interleave_gate_up(gate, up):
    """Rows of two [N, ...] tensors interleaved in 16-row tiles (gate 0..15, up 0..15, gate
    16..31, ...): the weight layout `quantized_matmul_swiglu` reads."""
    n = gate.shape[0]
    if up.shape != gate.shape or n % 16:
        raise ValueError("gate and up must have the same shape with rows a multiple of 16")
    g = gate.reshape(n // 16, 1, 16, *gate.shape[1:])
    u = up.reshape(n // 16, 1, 16, *up.shape[1:])
    return torch.cat([g, u], dim=1).reshape(2 * n, *gate.shape[1:]).contiguous()


def swiglu_supported(M, I, K):
    """True when the SwiGLU matmul covers this shape (whole (gate, up) tile pairs)."""
    return I % 16 == 0 and M >= 1 and K % 64 == 0


def rows_tiled_supported(M, N, K):
    """Whether `quantized_matmul_tiled` takes the shape (1..32 rows per pass, N % 32 == 0, K % 512 == 0)."""
    return bool(_lib.lib().eagle_qmm_rows_tiled_supported(int(M), int(N), int(K)))


def quantized_matmul_tiled(x, tiled, bias=None, out=None):
    """`quantized_matmul` of up to 32 rows (64: two passes) from the tiled copy of a matrix with
    very many rows (the vocabulary projection, mlx_llama.py:309-312): one workgroup per compute
    unit walks all of K over its share of the weight rows, so every compute unit reads x once.
    Agrees with `quantized_matmul` to the tolerance of the product (fp16 weights)."""
    _need_cuda(x, tiled.wt, tiled.sbt, bias)
    x = _f16(x, "x")
    *lead, K = x.shape
    M = reduce(lambda a, b: a * b, lead, 1)
    if K != tiled.K:
        raise ValueError(f"shape mismatch: x {tuple(x.shape)}, tiled weights [{tiled.N}, {tiled.K}]")
    if M < 1 or M > 64:
        raise ValueError("quantized_matmul_tiled takes 1..64 rows")
    if bias is not None:
        bias = _f16(bias, "bias")
        if tuple(bias.shape) != (tiled.N,):
            raise ValueError("bias must have shape [N]")
    if out is None:
        out = torch.empty((*lead, tiled.N), dtype=torch.float16, device=x.device)
    x2, o2 = x.reshape(M, K), out.view(M, tiled.N)
    L = _lib.lib()
    for r0 in range(0, M, 32):
        r1 = min(M, r0 + 32)
        rc = L.eagle_qmm_rows_tiled_w4g64_f16(_ptr(x2[r0:r1]), _ptr(tiled.wt), _ptr(tiled.sbt), _ptr(bias),
                                              _ptr(o2[r0:r1]), r1 - r0, tiled.N, K, int(tiled.small), _stream())
        _lib.check(rc, "quantized_matmul_tiled")
    return out


def quantized_matmul_swiglu_slab(x, w_q, scales, biases, bias=None, out=None):
    """`quantized_matmul_swiglu` for 1..64 rows on the slab kernel with one slab over all of K
    (each expanded weight feeds the matrix instructions of both 32-row tiles above 32 rows)."""
    _need_cuda(x, w_q, scales, biases, bias)
    x = _f16(x, "x")
    w_q = as_packed_u32(w_q)
    scales, biases = _f16(scales, "scales"), _f16(biases, "biases")
    *lead, K = x.shape
    M = reduce(lambda a, b: a * b, lead, 1)
    N = w_q.shape[0]
    if w_q.shape[1] * 8 != K or tuple(scales.shape) != (N, K // 64) or tuple(biases.shape) != (N, K // 64):
        raise ValueError(f"shape mismatch: x {tuple(x.shape)}, w {tuple(w_q.shape)}, "
                         f"scales {tuple(scales.shape)}, biases {tuple(biases.shape)}")
    if bias is not None:
        bias = _f16(bias, "bias")
        if tuple(bias.shape) != (N,):
            raise ValueError("bias must have shape [N]")
    if out is None:
        out = torch.empty((*lead, N // 2), dtype=torch.float16, device=x.device)
    rc = _lib.lib().eagle_qmm_slab_swiglu_w4g64_f16(_ptr(x), _ptr(w_q), _ptr(scales), _ptr(biases), _ptr(bias),
                                                    _ptr(out), M, N, K, 64, 4, _stream())
    _lib.check(rc, "quantized_matmul_swiglu_slab")
    return out


def quantized_matmul_swiglu(x, w_q, scales, biases, bias=None, out=None, gemm=None, tiled=None):
    """silu(x @ Wg.T) * (x @ Wu.T) (mlx_llama.py:214-215) in one launch: w_q / scales / biases
    / bias hold the gate and up projections interleaved by `interleave_gate_up`.  With more than
    one row on the streaming kernel the result equals `silu_mul(quantized_matmul(x, gate...),
    quantized_matmul(x, up...))` bit for bit; the other forms agree with it to the tolerance of
    the product.  33..64 rows run on the slab kernel with 64-row tiles
    (`quantized_matmul_swiglu_slab`), more rows as the tiled GEMM form with the same epilogue
    (`gemm=True`: that form whatever the row count).
    tiled: the interleaved matrix as `TiledWeights`; up to 64 rows then run the slab kernel on
    that copy."""
    _need_cuda(x, w_q, scales, biases, bias)
    x = _f16(x, "x")
    if tiled is not None and not gemm and x.numel() // x.shape[-1] <= 64:
        *lead, K = x.shape
        M = reduce(lambda a, b: a * b, lead, 1)
        if K != tiled.K:
            raise ValueError(f"shape mismatch: x {tuple(x.shape)}, tiled weights [{tiled.N}, {tiled.K}]")
        if bias is not None:
            bias = _f16(bias, "bias")
            if tuple(bias.shape) != (tiled.N,):
                raise ValueError("bias must have shape [N]")
        if out is None:
            out = torch.empty((*lead, tiled.N // 2), dtype=torch.float16, device=x.device)
        rc = _lib.lib().eagle_qmm_slab_swiglu_tiled_w4g64_f16(_ptr(x), _ptr(tiled.wt), _ptr(tiled.sbt), _ptr(bias),
                                                              _ptr(out), M, tiled.N, K, int(tiled.small), _stream())
        _lib.check(rc, "quantized_matmul_swiglu (tiled)")
        return out
    w_q = as_packed_u32(w_q)
    scales, biases = _f16(scales, "scales"), _f16(biases, "biases")
    *lead, K = x.shape
    M = reduce(lambda a, b: a * b, lead, 1)
    N = w_q.shape[0]
    if w_q.shape[1] * 8 != K or tuple(scales.shape) != (N, K // 64) or tuple(biases.shape) != (N, K // 64):
        raise ValueError(f"shape mismatch: x {tuple(x.shape)}, w {tuple(w_q.shape)}, "
                         f"scales {tuple(scales.shape)}, biases {tuple(biases.shape)}")
    if bias is not None:
        bias = _f16(bias, "bias")
        if tuple(bias.shape) != (N,):
            raise ValueError("bias must have shape [N]")
    if out is None:
        out = torch.empty((*lead, N // 2), dtype=torch.float16, device=x.device)
    L = _lib.lib()
    if not gemm and L.eagle_qmm_slab_swiglu_preferred(M, N, K):
        # the slab kernel with one slab over all of K: above 32 rows one launch with 64-row tiles
        # (35 us against 48..56 us for two passes of the 32-row kernel at the 7B shape), and from
        # 24 rows where its workgroups fill the GPU in one round (the 8B shape: 24 against 27 us)
        rc = L.eagle_qmm_slab_swiglu_w4g64_f16(_ptr(x), _ptr(w_q), _ptr(scales), _ptr(biases), _ptr(bias),
                                               _ptr(out), M, N, K, 64, 4, _stream())
        _lib.check(rc, "quantized_matmul_swiglu")
        return out
    if ROW_PASS < M <= 2 * ROW_PASS and not gemm:
        x2, out2 = x.reshape(M, K), out.view(M, N // 2)
        for r0 in range(0, M, ROW_PASS):
            quantized_matmul_swiglu(x2[r0:r0 + ROW_PASS], w_q, scales, biases, bias=bias,
                                    out=out2[r0:r0 + ROW_PASS])
        return out
    if M > 32 or gemm:
        # many rows (a prompt chunk): the tiled GEMM with the same epilogue
        rc = L.eagle_qmm_gemm_swiglu_w4g64_f16(_ptr(x), _ptr(w_q), _ptr(scales), _ptr(biases), _ptr(bias),
                                               _ptr(out), M, N, K, 64, 4, _stream())
        _lib.check(rc, "quantized_matmul_swiglu")
        return out
    ws = workspace("qmm", L.eagle_qmm_workspace_bytes(M, N, K), x.device)
    rc = L.eagle_qmm_swiglu_w4g64_f16(_ptr(x), _ptr(w_q), _ptr(scales), _ptr(biases), _ptr(bias),
                                      _ptr(out), M, N, K, 64, 4, _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "quantized_matmul_swiglu")
    return out


# |scale| below this: the kernels may expand nibbles through fp16 subnormals (scale * 2^20 is a
# finite fp16), three vector instructions fewer per packed word
TILED_SMALL_SCALE = 0.0624


class TiledWeights:
    """A 4-bit group-64 weight matrix [N, K] in the layout the 32-row slab kernels stream
    fastest (`tile_weights`): `wt` [N/32, K/64, 64, 4] int32, one contiguous 1 KB block per
    32-row tile and quantisation group in the order the lanes of a wave hold it, and `sbt`
    [N/32, K/512, 64, 8] fp16 with the scales of a tile's rows for eight groups in lanes 0..31
    and the biases in lanes 32..63.  `small` says that every |scale| is below TILED_SMALL_SCALE."""

    def __init__(self, wt, sbt, N, K, small):
        self.wt, self.sbt, self.N, self.K, self.small = wt, sbt, int(N), int(K), bool(small)


def tiled_supported(M, N, K):
    """True when the tiled forms (`quantized_matmul_slabs` / `quantized_matmul_swiglu` with
    `tiled=`) take this product: up to 64 rows, N a multiple of 32, K a multiple of 512."""
    return bool(_lib.lib().eagle_qmm_tiled_supported(int(M), int(N), int(K)))


def tile_weights(w_q, scales, biases):
    """Re-lay a weight matrix in the MLX layout (`w_q` [N, K/8] uint32, `scales`, `biases`
    [N, K/64] fp16) out as `TiledWeights` (one device launch; the inputs are left as they are)."""
    _need_cuda(w_q, scales, biases)
    w_q = as_packed_u32(w_q)
    scales, biases = _f16(scales, "scales"), _f16(biases, "biases")
    N, K = w_q.shape[0], w_q.shape[1] * 8
    L = _lib.lib()
    nsb = L.eagle_qmm_tiled_sb_bytes(N, K)
    if not nsb or tuple(scales.shape) != (N, K // 64) or tuple(biases.shape) != (N, K // 64):
        raise ValueError(f"the tiled layout takes N % 32 == 0 and K % 512 == 0, got [{N}, {K}]")
    wt = torch.empty((N // 32, K // 64, 64, 4), dtype=torch.int32, device=w_q.device)
    sbt = torch.empty((N // 32, K // 512, 64, 8), dtype=torch.float16, device=w_q.device)
    rc = L.eagle_qmm_tile_w4g64(_ptr(w_q), _ptr(scales), _ptr(biases), _ptr(wt), _ptr(sbt), N, K, 64, 4, _stream())
    _lib.check(rc, "tile_weights")
    small = bool(scales.abs().max().item() < TILED_SMALL_SCALE)
    return TiledWeights(wt, sbt, N, K, small)


SMALL_SCALE_LIMIT = 0.2499       # |scale| * 2^18 has to stay a finite fp16 (the small-row kernels)


def small_supported(T, N, K, norm=False, swiglu=False):
    """True when `quantized_matmul_small` takes this shape."""
    return bool(_lib.lib().eagle_qmm_small_supported(T, N, K, int(bool(norm)), int(bool(swiglu))))


def quantized_matmul_small(x, w_q, scales, biases, bias=None, out=None, norm_weight=None, eps=1e-6,
                           residual=None, swiglu=False):
    """The product for at most 16 rows with its neighbours folded in (mlx_llama.py:195-196,
    214-215, 225-249): RMSNorm of x before it (norm_weight), the residual added to it (residual;
    may be `out`), or SwiGLU over gate|up interleaved by `interleave_gate_up` (swiglu).  Every
    scale must be below SMALL_SCALE_LIMIT in magnitude; the caller checks that once per matrix."""
    _need_cuda(x, w_q, scales, biases, bias, norm_weight, residual)
    x = _f16(x, "x")
    w_q = as_packed_u32(w_q)
    scales, biases = _f16(scales, "scales"), _f16(biases, "biases")
    *lead, K = x.shape
    T = reduce(lambda a, b: a * b, lead, 1)
    N = w_q.shape[0]
    if w_q.shape[1] * 8 != K or tuple(scales.shape) != (N, K // 64) or tuple(biases.shape) != (N, K // 64):
        raise ValueError(f"shape mismatch: x {tuple(x.shape)}, w {tuple(w_q.shape)}, "
                         f"scales {tuple(scales.shape)}, biases {tuple(biases.shape)}")
    n_out = N // 2 if swiglu else N
    if bias is not None and tuple(_f16(bias, "bias").shape) != (N,):
        raise ValueError("bias must have shape [N]")
    if norm_weight is not None and tuple(_f16(norm_weight, "norm_weight").shape) != (K,):
        raise ValueError("norm_weight must have shape [K]")
    if out is None:
        out = torch.empty((*lead, n_out), dtype=torch.float16, device=x.device)
    if residual is not None and (tuple(residual.shape) != tuple(out.shape) or not residual.is_contiguous()):
        raise ValueError("residual must be contiguous with the shape of the result")
    rc = _lib.lib().eagle_qmm_small_w4g64_f16(
        _ptr(x), _ptr(norm_weight), float(eps), _ptr(w_q), _ptr(scales), _ptr(biases), _ptr(bias),
        _ptr(residual), _ptr(out), T, N, K, 64, 4, int(bool(swiglu)), _stream())
    _lib.check(rc, "quantized_matmul_small")
    return out


def qkv_rope_small_supported(T, D, H, G, hd):
    return bool(_lib.lib().eagle_qkv_rope_small_supported(T, D, H, G, hd))


def qkv_rope_small(x, w_q, scales, biases, bias, rope_cs, q_rot, k_cache, v_cache, cache_len_dev, H, G, hd,
                   norm_weight=None, eps=1e-6):
    """RMSNorm, fused q|k|v product, rotation of q and k with the (cos, sin) table and append of the
    new K / V rows at *cache_len_dev, in one launch (mlx_llama.py:136-183, 231-233).  x [T, D];
    q_rot [H, T, hd] is written; k_cache, v_cache [G, capacity, hd]."""
    _need_cuda(x, w_q, scales, biases, bias, rope_cs, q_rot, k_cache, v_cache, cache_len_dev, norm_weight)
    x = _f16(x, "x")
    T, D = x.shape
    w_q = as_packed_u32(w_q)
    if w_q.shape != ((H + 2 * G) * hd, D // 8) or tuple(q_rot.shape) != (H, T, hd) \
            or tuple(k_cache.shape[-3:]) != (G, k_cache.shape[-2], hd) or tuple(rope_cs.shape) != (T, hd // 2, 2):
        raise ValueError("shape mismatch")
    for t in (q_rot, k_cache, v_cache, rope_cs):
        if not t.is_contiguous():
            raise ValueError("non-contiguous buffer")
    rc = _lib.lib().eagle_qkv_rope_small_w4g64_f16(
        _ptr(x), _ptr(norm_weight), float(eps), _ptr(w_q), _ptr(_f16(scales, "scales")), _ptr(_f16(biases, "biases")),
        _ptr(bias), _ptr(rope_cs), _ptr(q_rot), _ptr(k_cache), _ptr(v_cache), _ptr(cache_len_dev), T, D, H, G, hd,
        k_cache.shape[-2], 64, 4, _stream())
    _lib.check(rc, "qkv_rope_small")
    return q_rot


# rows of x up to which `quantized_matmul` considers the vector-ALU kernel (`bench.py --small-m`
# has the measurements behind QMV_MAX_ROWS and `qmv_preferred`)
QMV_MAX_ROWS = 2


def qmv_preferred(N, K, M=1):
    """True where the vector-ALU kernel is the faster form for M rows of x.  Measured on the
    projection shapes of the 7B model, vector ALU against matrix tiles, us per launch:
      M = 1: 5.8 / 8.5 (3584 x 3584), 4.4 / 6.7 (512 x 3584), 12.6 / 16.1 (18944 x 3584), 5.3 / 7.1
             (8192 x 2048); a long K over few rows (3584 x 18944: 28.3 / 18.9) and the vocabulary
             projection (66.6 / 63.2) stay on the matrix kernel;
      M = 2: 7.2 / 8.5, 5.8 / 6.9, 16.3 / 15.9, 6.6 / 7.2: the vector ALU up to a few thousand rows;
      M = 4: 9.4 / 8.6, 8.4 / 7.0, 28.7 / 16.1, 8.9 / 7.3; M = 8: 15.1 / 8.7, 14.3 / 7.1, 44.2 / 16.1,
             14.2 / 7.4: matrix tiles everywhere (5 + 4 M vector instructions per packed word)."""
    if M > QMV_MAX_ROWS or not _lib.lib().eagle_qmv_rows_supported(M, N, K) or K > 4096:
        return False
    return N <= 65536 if M == 1 else N <= 16384


def quantized_matvec(x, w_q, scales, biases, bias=None, out=None):
    """One to eight rows of x times the quantised matrix on the vector ALU (no matrix
    instructions): the M = 1 case of `quantized_matmul` (mlx_model_fwd_bench.py:65-73) and the
    reference's batched vector form (qmv.py:226-241)."""
    _need_cuda(x, w_q, scales, biases, bias)
    x = _f16(x, "x")
    w_q = as_packed_u32(w_q)
    scales, biases = _f16(scales, "scales"), _f16(biases, "biases")
    K = x.shape[-1]
    N = w_q.shape[0]
    M = x.numel() // K
    if M < 1 or M > 8 or w_q.shape[1] * 8 != K or tuple(scales.shape) != (N, K // 64) \
            or tuple(biases.shape) != (N, K // 64):
        raise ValueError(f"shape mismatch: x {tuple(x.shape)}, w {tuple(w_q.shape)}, "
                         f"scales {tuple(scales.shape)}, biases {tuple(biases.shape)}")
    if bias is not None:
        bias = _f16(bias, "bias")
    if out is None:
        out = torch.empty((*x.shape[:-1], N), dtype=torch.float16, device=x.device)
    rc = _lib.lib().eagle_qmv_rows_w4g64_f16(_ptr(x), _ptr(w_q), _ptr(scales), _ptr(biases), _ptr(bias),
                                             _ptr(out), M, N, K, 64, 4, _stream())
    _lib.check(rc, "quantized_matvec")
    return out


def matmul(x, w, s, b, group_size, **_ignored):
    """Same contract as the reference's `qmm_kernel.matmul` (qmm_kernel.py:84-164):
    returns a one-element list.  The Metal tuning keywords are accepted and ignored."""
    return [quantized_matmul(x, w, s, b, group_size=group_size, bits=4)]


def default_inv_freqs(head_dim, base=10000.0, device=None):
    """inv_freq[i] = 2 ** (-log2(base) * 2i / head_dim) in fp32 (mlx_llama.py:109-113)."""
    expo = -torch.log2(torch.tensor(float(base), dtype=torch.float32)) * \
        torch.arange(0, head_dim, 2, dtype=torch.float32) / float(head_dim)
    return torch.exp2(expo).to(device)


def arrayed_rope(x, positions, inv_freqs=None, scaling_factor=1.0, base=10000.0):
    """RoPE with a position per (batch, token).  x [B,H,L,hd] fp16, positions [B,L]
    (or [L] for B=1) integer.  Same semantics as `rope_positions`
    (mlx_arrayed_rope_kernel.py:46-152)."""
    _need_cuda(x, positions)
    x = _f16(x, "x")
    if x.dim() != 4:
        raise ValueError("x must be [B, H, L, head_dim]")
    B, H, L, hd = x.shape
    pos = positions.to(torch.int32).contiguous()
    if pos.numel() != B * L:
        raise ValueError(f"positions must hold B*L = {B * L} entries")
    if inv_freqs is None:
        inv_freqs = default_inv_freqs(hd, base, x.device)
    inv = inv_freqs.to(device=x.device, dtype=torch.float32).contiguous()
    if inv.numel() != hd // 2:
        raise ValueError("inv_freqs must have head_dim/2 entries")
    out = torch.empty_like(x)
    rc = _lib.lib().eagle_rope_arrayed_f16(_ptr(x), _ptr(pos), _ptr(inv), float(scaling_factor),
                                           _ptr(out), B, H, L, hd, _stream())
    _lib.check(rc, "arrayed_rope")
    return out


def rope_positions(inp, offsets, inv_freqs, scaling_factor, verbose=False):
    """Reference name and argument order (mlx_arrayed_rope_kernel.py:47-53)."""
    return arrayed_rope(inp, offsets, inv_freqs, scaling_factor)


def rope_kv_append(q_lin, k_lin, v_lin, positions, inv_freqs, scaling_factor, q_out, k_cache,
                   v_cache, cache_len_dev, H, G, hd, row_stride=0, rope_cs=None):
    """Rotate q and k at `positions`, write q as [H,T,hd] and append k, v to the caches.
    row_stride > 0: q_lin, k_lin, v_lin are column blocks of one [T,row_stride] matrix.
    rope_cs: the `rope_table` of these positions (then positions / inv_freqs are not read)."""
    T = q_lin.shape[0]
    if rope_cs is not None:
        rc = _lib.lib().eagle_rope_kv_append_table_f16(
            _ptr(q_lin), _ptr(k_lin), _ptr(v_lin), _ptr(rope_cs), _ptr(q_out), _ptr(k_cache),
            _ptr(v_cache), _ptr(cache_len_dev), T, H, G, hd, k_cache.shape[1], int(row_stride), _stream())
        _lib.check(rc, "rope_kv_append")
        return
    rc = _lib.lib().eagle_rope_kv_append_f16(
        _ptr(q_lin), _ptr(k_lin), _ptr(v_lin), _ptr(positions), _ptr(inv_freqs),
        float(scaling_factor), _ptr(q_out), _ptr(k_cache), _ptr(v_cache), _ptr(cache_len_dev),
        T, H, G, hd, k_cache.shape[1], int(row_stride), _stream())
    _lib.check(rc, "rope_kv_append")


def rope_kv_append_slabs(partial, slabs, bias, rope_cs, q_out, k_cache, v_cache, cache_len_dev, T, H, G, hd):
    """`rope_kv_append` (table form) of the fused q|k|v projection held as
    [slabs, slab_rows(T), (H+2G) hd] fp32 partial sums; `bias` is the projection's fp16 bias or None."""
    rc = _lib.lib().eagle_rope_kv_append_slabs_f16(
        _ptr(partial), int(slabs), _ptr(bias), _ptr(rope_cs), _ptr(q_out), _ptr(k_cache), _ptr(v_cache),
        _ptr(cache_len_dev), T, H, G, hd, k_cache.shape[1], _stream())
    _lib.check(rc, "rope_kv_append_slabs")


def mask_to_bits(tree_mask):
    """[T,T] additive ({0,-inf}) or boolean visibility matrix -> [T] int32 row bitmasks."""
    m = tree_mask
    vis = m if m.dtype == torch.bool else (m == 0)
    T = vis.shape[-1]
    if vis.shape[-2] != T or T > 32:
        raise ValueError("tree mask must be [T,T] with T <= 32")
    weights = (torch.ones(T, dtype=torch.int64, device=vis.device) << torch.arange(T, device=vis.device))
    bits = (vis.reshape(T, T).to(torch.int64) * weights[None, :]).sum(1)
    bits = torch.where(bits >= 2 ** 31, bits - 2 ** 32, bits)   # bit 31 -> sign bit of int32
    return bits.to(torch.int32)


def tree_attention(q, k_cache, v_cache, tree_mask_bits, cache_len_dev, scale, max_len=None,
                   out=None):
    """q [H,T,hd]; k_cache, v_cache [G,capacity,hd] holding *cache_len_dev prefix rows
    followed by the T tree rows; tree_mask_bits [T] int32, or [T,2] (`mask_to_words`) for
    trees of up to 64 tokens.  Returns [T, H*hd]."""
    _need_cuda(q, k_cache, v_cache, tree_mask_bits, cache_len_dev)
    H, T, hd = q.shape
    G, cap, _ = k_cache.shape
    if max_len is None:
        max_len = cap
    if out is None:
        out = torch.empty((T, H * hd), dtype=torch.float16, device=q.device)
    L = _lib.lib()
    if tree_mask_bits.dim() == 2:
        if tree_mask_bits.shape != (T, 2):
            raise ValueError("two mask words per tree token")
        ws = workspace("attn", L.eagle_tree_attention_wide_workspace_bytes(T, H, hd, max_len), q.device)
        rc = L.eagle_tree_attention_wide_f16(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(tree_mask_bits),
                                             _ptr(cache_len_dev), _ptr(out), T, T, H, G, hd, cap, max_len,
                                             float(scale), _ptr(ws), ws.numel(), _stream())
        _lib.check(rc, "tree_attention")
        return out
    need = L.eagle_tree_attention_workspace_bytes(H, hd, max_len)
    ws = workspace("attn", need, q.device)
    rc = L.eagle_tree_attention_f16(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(tree_mask_bits),
                                    _ptr(cache_len_dev), _ptr(out), T, H, G, hd, cap, max_len,
                                    float(scale), _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "tree_attention")
    return out


def rope_table(positions, inv_freqs, scaling_factor=1.0, out=None):
    """fp32 [T, hd/2, 2] table of (cos, sin)(positions[t] * scaling_factor * inv_freqs[i]) for
    the rope launches; the angles are those of `arrayed_rope`."""
    _need_cuda(positions, inv_freqs)
    T, half = positions.numel(), inv_freqs.numel()
    if out is None:
        out = torch.empty((T, half, 2), dtype=torch.float32, device=positions.device)
    rc = _lib.lib().eagle_rope_table_f32(_ptr(positions), _ptr(inv_freqs), float(scaling_factor),
                                         T, half, _ptr(out), _stream())
    _lib.check(rc, "rope_table")
    return out


def mask_to_words(mask):
    """[T,Tk] additive ({0,-inf}) or boolean visibility matrix, Tk <= 64 -> [T,2] int32: bit
    (j % 32) of word j // 32 says whether query t sees masked row j."""
    vis = mask if mask.dtype == torch.bool else (mask == 0)
    T, Tk = vis.shape
    if Tk > 64:
        raise ValueError("at most 64 masked rows")
    v = torch.zeros((T, 64), dtype=torch.int64, device=vis.device)
    v[:, :Tk] = vis.to(torch.int64)
    weights = torch.ones(32, dtype=torch.int64, device=vis.device) << torch.arange(32, device=vis.device)
    words = (v.reshape(T, 2, 32) * weights[None, None, :]).sum(2)
    words = torch.where(words >= 2 ** 31, words - 2 ** 32, words)
    return words.to(torch.int32).contiguous()


def draft_attention(q, k_cache, v_cache, mask_words, cache_len_dev, Tk, scale, max_len=None, out=None):
    """q [H,T,hd]; k_cache, v_cache [G,capacity,hd] holding *cache_len_dev prefix rows followed
    by Tk <= 64 rows that query t sees according to mask_words [T,2].  Returns [T, H*hd].
    More than 32 (up to 64) queries go in pieces of 32 rows through one launch pair."""
    _need_cuda(q, k_cache, v_cache, mask_words, cache_len_dev)
    H, T, hd = q.shape
    G, cap, _ = k_cache.shape
    if max_len is None:
        max_len = cap
    if out is None:
        out = torch.empty((T, H * hd), dtype=torch.float16, device=q.device)
    L = _lib.lib()
    if T > 32:
        ws = workspace("attn", L.eagle_tree_attention_wide_workspace_bytes(T, H, hd, max_len), q.device)
        rc = L.eagle_tree_attention_wide_f16(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(mask_words),
                                             _ptr(cache_len_dev), _ptr(out), T, int(Tk), H, G, hd, cap,
                                             max_len, float(scale), _ptr(ws), ws.numel(), _stream())
        _lib.check(rc, "draft_attention")
        return out
    need = L.eagle_tree_attention_workspace_bytes(H, hd, max_len)
    ws = workspace("attn", need, q.device)
    rc = L.eagle_draft_attention_f16(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(mask_words),
                                     _ptr(cache_len_dev), _ptr(out), T, int(Tk), H, G, hd, cap, max_len,
                                     float(scale), _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "draft_attention")
    return out


def scaled_dot_product_attention(queries, keys, values, cache=None, scale=None, mask=None):
    """Drop-in for the call at mlx_llama.py:185-192 on the tree and draft paths:
    queries [1,H,T,hd] with T <= 64 (32 query rows per launch set), keys/values [1,G,S,hd],
    mask [1,1,T,S] additive.  Only
    the last min(S, 64) columns of the mask are looked at: every earlier column has to be zero
    (a prefix that all queries see), which holds for the verification mask
    (mlx_eagle.py:337-338), the expansion masks up to depth 8 (mlx_eagle.py:143-171) and causal
    masks of up to 32 new tokens.  Returns [1,H,T,hd]."""
    _need_cuda(queries, keys, values, mask)
    B, H, T, hd = queries.shape
    if B != 1:
        raise ValueError("batch size 1 only")
    G, S = keys.shape[1], keys.shape[2]
    if scale is None:
        scale = hd ** -0.5
    if mask is None:
        raise ValueError("the tree path always passes a mask")
    Tk = min(S, 64)
    P = S - Tk
    words = mask_to_words(mask.reshape(T, S)[:, P:])
    len_dev = torch.tensor([P], dtype=torch.int32, device=queries.device)
    if cache is not None and keys.data_ptr() == cache.keys.data_ptr():
        k_buf, v_buf = cache.keys[0], cache.values[0]        # the fetched views alias the cache
    else:
        k_buf, v_buf = _f16(keys[0], "k"), _f16(values[0], "v")
    q = _f16(queries[0], "q")
    if T > 64:
        raise ValueError("at most 64 query rows")
    # more than 32 queries (a tree of up to 64 tokens) go in pieces of 32 query rows, each with
    # its own mask rows over the same keys, inside the one launch pair
    out = draft_attention(q, k_buf, v_buf, words, len_dev, Tk, scale, max_len=S)
    return out.reshape(T, H, hd).permute(1, 0, 2).unsqueeze(0).contiguous()


def causal_attention(q, k_cache, v_cache, piece_len_dev, scale, max_len=None, out=None):
    """Causal attention of a prompt chunk in pieces of 32 rows, one launch pair for all pieces:
    q [H,R,hd] (R a multiple of 32); piece j sits at cache rows piece_len_dev[j] .. +31.
    Returns [R, H*hd]."""
    _need_cuda(q, k_cache, v_cache, piece_len_dev)
    H, R, hd = q.shape
    G, cap, _ = k_cache.shape
    if max_len is None:
        max_len = cap
    if out is None:
        out = torch.empty((R, H * hd), dtype=torch.float16, device=q.device)
    L = _lib.lib()
    ws = workspace("attn_chunk", L.eagle_causal_attention_workspace_bytes(R, H, hd, max_len), q.device)
    rc = L.eagle_causal_attention_f16(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(piece_len_dev), _ptr(out),
                                      R, H, G, hd, cap, max_len, float(scale), _ptr(ws), ws.numel(),
                                      _stream())
    _lib.check(rc, "causal_attention")
    return out


def logsoftmax_topk(logits, k, mode, row_index=None, out=None):
    """The k most likely tokens per row of fp16 logits [R,V] (or the rows row_index selects)
    and their fp16 log-probabilities, best first, ties lowest index first.  mode 0: the level-0
    form of mlx_eagle.py:410-412; mode 1: the form of mlx_eagle.py:103-104.
    Returns (index [R,k] int32, score [R,k] fp16)."""
    _need_cuda(logits, row_index)
    logits = _f16(logits, "logits")
    V = logits.shape[-1]
    R = row_index.numel() if row_index is not None else logits.numel() // V
    if out is None:
        out = (torch.empty((R, k), dtype=torch.int32, device=logits.device),
               torch.empty((R, k), dtype=torch.float16, device=logits.device))
    L = _lib.lib()
    ws = workspace("topk", L.eagle_logsoftmax_topk_workspace_bytes(R, V), logits.device)
    rc = L.eagle_logsoftmax_topk_f16(_ptr(logits), _ptr(row_index), R, V, int(k), int(mode),
                                     _ptr(out[0]), _ptr(out[1]), _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "logsoftmax_topk")
    return out


def rms_norm(x, weight, eps, residual=None, out=None, h_out=None):
    """`mx.fast.rms_norm(x, weight, eps)`; with `residual` returns (h, norm(h)),
    h = fp16(x + residual) (h_out may alias residual for an in-place update)."""
    _need_cuda(x, weight, residual)
    x = _f16(x, "x")
    D = x.shape[-1]
    T = x.numel() // D
    if out is None:
        out = torch.empty_like(x)
    h = None
    if residual is not None:
        h = h_out if h_out is not None else torch.empty_like(x)
    rc = _lib.lib().eagle_rmsnorm_f16(_ptr(x), _ptr(residual), _ptr(_f16(weight, "weight")),
                                      float(eps), _ptr(h), _ptr(out), T, D, _stream())
    _lib.check(rc, "rms_norm")
    return out if residual is None else (h, out)


def rms_norm_slabs(partial, slabs, weight, eps, T, residual=None, out=None, h_out=None):
    """`rms_norm` of x = fp16(sum of the slabs) held as [slabs, slab_rows(T), D] fp32 partial sums."""
    _need_cuda(partial, weight, residual)
    D = weight.shape[-1]
    if out is None:
        out = torch.empty((T, D), dtype=torch.float16, device=partial.device)
    h = None
    if residual is not None:
        h = h_out if h_out is not None else torch.empty((T, D), dtype=torch.float16, device=partial.device)
    rc = _lib.lib().eagle_rmsnorm_slabs_f16(_ptr(partial), int(slabs), _ptr(residual),
                                            _ptr(_f16(weight, "weight")), float(eps), _ptr(h), _ptr(out),
                                            T, D, _stream())
    _lib.check(rc, "rms_norm_slabs")
    return out if residual is None else (h, out)


def silu_mul(gate, up=None, out=None):
    """fp16(fp16(silu(gate)) * up); with up=None, `gate` is the fused [T, 2*I] tensor."""
    _need_cuda(gate, up)
    gate = _f16(gate, "gate")
    if up is None:
        I = gate.shape[-1] // 2
    else:
        up = _f16(up, "up")
        I = gate.shape[-1]
    T = gate.numel() // gate.shape[-1]
    if out is None:
        out = torch.empty((*gate.shape[:-1], I), dtype=torch.float16, device=gate.device)
    rc = _lib.lib().eagle_silu_mul_f16(_ptr(gate), _ptr(up), _ptr(out), T, I, _stream())
    _lib.check(rc, "silu_mul")
    return out


def add(a, b):
    _need_cuda(a, b)
    a, b = _f16(a, "a"), _f16(b, "b")
    out = torch.empty_like(a)
    rc = _lib.lib().eagle_add_f16(_ptr(a), _ptr(b), _ptr(out), a.numel(), _stream())
    _lib.check(rc, "add")
    return out


def embed(ids, w_q, scales, biases, out=None):
    """Quantised embedding lookup: ids [...] int -> [..., D] fp16."""
    _need_cuda(ids, w_q, scales, biases)
    w_q = as_packed_u32(w_q)
    V, D = w_q.shape[0], w_q.shape[1] * 8
    ids32 = ids.to(torch.int32).contiguous()
    if out is None:
        out = torch.empty((*ids.shape, D), dtype=torch.float16, device=ids.device)
    rc = _lib.lib().eagle_embed_w4g64_f16(_ptr(ids32), _ptr(w_q), _ptr(_f16(scales, "scales")),
                                          _ptr(_f16(biases, "biases")), _ptr(out), ids32.numel(),
                                          D, V, _stream())
    _lib.check(rc, "embed")
    return out


def argmax_rows(logits, out=None):
    """argmax over the last axis, lowest index among equal maxima; int32."""
    _need_cuda(logits)
    logits = _f16(logits, "logits")
    V = logits.shape[-1]
    R = logits.numel() // V
    if out is None:
        out = torch.empty(logits.shape[:-1], dtype=torch.int32, device=logits.device)
    L = _lib.lib()
    ws = workspace("argmax", L.eagle_argmax_workspace_bytes(R, V), logits.device)
    rc = L.eagle_argmax_rows_f16(_ptr(logits), _ptr(out), R, V, _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "argmax_rows")
    return out
