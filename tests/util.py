"""Shared helpers of the test-suite."""
import numpy as np
import torch

TOL = 2e-2   # max |err| <= TOL * RMS(reference output): the bound stated for fp16 QMM / RoPE / attention
# Outputs of a whole multi-layer pass (cache rows of the second layer, logits): every operator
# meets TOL on its own output, but the inputs of the later operators already differ by the
# earlier ones' rounding, so the errors of the 7 matmuls per layer add up.  Measured on the
# two-layer test models: up to 0.024; at 7B width 0.005 after one layer and 0.034 after 28
# (tests/test_gpu_fullsize.py follows the growth).
MODEL_TOL = 2 * TOL


def to_dev(a, dev):
    """numpy -> torch on the device; uint32 travels as int32 bits."""
    if isinstance(a, np.ndarray) and a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).to(dev)
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def rel_err(got, want):
    """max |got - want| / RMS(want), computed in float64."""
    g = np.asarray(got, dtype=np.float64)
    w = np.asarray(want, dtype=np.float64)
    rms = np.sqrt(np.mean(w * w))
    return float(np.max(np.abs(g - w)) / max(rms, 1e-30))


def layer_to_dev(layer, dev):
    return {k: to_dev(v, dev) for k, v in layer.items()}


def close_fp16(got, want, what="", rms_frac=0.1):
    """Bound for fp16 results that are themselves products of rounded fp16 values (SwiGLU): every
    element within TOL * RMS + 2 ulp of its own size (a rounding flip of an intermediate moves a
    large element by an ulp or two), and the RMS error within rms_frac * TOL * RMS."""
    g64, w64 = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert np.isfinite(g64).all(), what
    rms = np.sqrt(np.mean(w64 * w64))
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(w64), 2.0 ** -14))) - 10)
    assert np.all(np.abs(g64 - w64) <= TOL * rms + 2 * ulp), what
    assert np.sqrt(np.mean((g64 - w64) ** 2)) <= rms_frac * TOL * rms, what
