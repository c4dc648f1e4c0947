"""The matmul entry point that allocates nothing (its split-K workspace is a fixed device
array owned by the library) against the entry point that takes a workspace, through the C ABI:
bit-identical results on two calls in a row, the second with a smaller input, and a clear
error for a shape whose workspace does not fit the array."""
import numpy as np
import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import _lib, ops, synth
from oracle import oracle
from util import TOL, layer_to_dev, rel_err, to_dev

pytestmark = pytest.mark.gpu


def both(dev, M, N, K, seed):
    L = _lib.lib()
    rng = np.random.default_rng(seed)
    layer = synth.make_qlinear(rng, N, K, bias=True)
    x = synth.make_x(rng, M, K)
    d = layer_to_dev(layer, dev)
    xd = to_dev(x, dev)
    want = torch.empty((M, N), dtype=torch.float16, device=dev)
    got = torch.full((M, N), float("nan"), dtype=torch.float16, device=dev)
    ws = ops.workspace("qmm", L.eagle_qmm_workspace_bytes(M, N, K), dev)
    st = torch.cuda.current_stream().cuda_stream
    rc = L.eagle_qmm_w4g64_f16(xd.data_ptr(), d["weight"].data_ptr(), d["scales"].data_ptr(),
                               d["biases"].data_ptr(), d["bias"].data_ptr(), want.data_ptr(), M, N, K, 64, 4,
                               ws.data_ptr(), ws.numel(), st)
    assert rc == 0
    free0 = torch.cuda.mem_get_info()[0]
    rc = L.eagle_qmm_w4g64_f16_noalloc(xd.data_ptr(), d["weight"].data_ptr(), d["scales"].data_ptr(),
                                       d["biases"].data_ptr(), d["bias"].data_ptr(), got.data_ptr(), M, N, K,
                                       64, 4, st)
    assert rc == 0, _lib.status_string(rc)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0          # nothing was allocated by the call
    assert torch.equal(got, want)
    ref = oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"], layer["bias"])
    assert rel_err(got.cpu().numpy(), ref) <= TOL
    return ops.qmm_plan(M, N, K)[2]


def test_two_calls_in_a_row_the_second_smaller(dev):
    print("no-alloc matmul: 32 x 3584 x 18944, then 8 x 512 x 7168, then 32 x 512 x 3584", flush=True)
    assert both(dev, 32, 3584, 18944, seed=1) > 1          # K slabs: partial sums and counters in the array
    assert both(dev, 8, 512, 7168, seed=2) > 1             # a smaller product on the array the first one used
    both(dev, 32, 512, 3584, seed=3)
    both(dev, 17, 8192, 2048, seed=4)


def test_rejects_a_shape_beyond_the_array(dev):
    L = _lib.lib()
    assert L.eagle_qmm_noalloc_scratch_bytes() == 8 << 20
    # find a shape whose workspace is larger than the array
    M, N, K = 32, 65536, 16384
    assert ops.qmm_plan(M, N, K)[2] > 1 and L.eagle_qmm_workspace_bytes(M, N, K) > (8 << 20)
    x = torch.zeros((M, K), dtype=torch.float16, device=dev)
    w = torch.zeros((N, K // 8), dtype=torch.int32, device=dev)
    s = torch.zeros((N, K // 64), dtype=torch.float16, device=dev)
    out = torch.empty((M, N), dtype=torch.float16, device=dev)
    rc = L.eagle_qmm_w4g64_f16_noalloc(x.data_ptr(), w.data_ptr(), s.data_ptr(), s.data_ptr(), None,
                                       out.data_ptr(), M, N, K, 64, 4, torch.cuda.current_stream().cuda_stream)
    assert rc == 5 and "workspace" in _lib.status_string(rc).lower()
    rc = L.eagle_qmm_w4g64_f16_noalloc(x.data_ptr(), w.data_ptr(), s.data_ptr(), s.data_ptr(), None,
                                       out.data_ptr(), M, N, K, 32, 4, torch.cuda.current_stream().cuda_stream)
    assert rc == 4
