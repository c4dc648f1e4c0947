"""CPU-only checks of the C-ABI library: it loads, exports every symbol the header
declares, and rejects bad arguments on the host before any device work."""
import ctypes
import os
import re

import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import _lib, ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "eagle_mi355x.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(eagle_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
    # and the Python binding knows each of them
    assert set(names) == set(_lib.SIGNATURES), set(names) ^ set(_lib.SIGNATURES)


def test_status_strings_and_version():
    L = _lib.lib()
    assert L.eagle_abi_version() == 1
    assert L.eagle_status_string(0) == b"ok"
    for rc in range(1, 8):
        assert len(L.eagle_status_string(rc)) > 3


def test_qmm_argument_errors_are_detected_on_the_host():
    L = _lib.lib()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)
    p = (p + 15) & ~15
    call = lambda **kw: L.eagle_qmm_w4g64_f16(kw.get("x", p), kw.get("w", p), kw.get("s", p), kw.get("b", p),
                                              None, kw.get("out", p), kw.get("M", 8), kw.get("N", 64),
                                              kw.get("K", 128), kw.get("gs", 64), kw.get("bits", 4),
                                              None, 0, None)
    assert call(x=None) == 1                       # EAGLE_ERR_NULL
    assert call(out=None) == 1
    assert call(M=0) == 2 and call(M=33) == 2      # EAGLE_ERR_SHAPE
    assert call(K=100) == 2 and call(N=12) == 2 and call(K=1024 * 1024) == 2
    assert call(x=p + 2) == 3                      # EAGLE_ERR_ALIGN
    assert call(gs=32) == 4 and call(bits=8) == 4  # EAGLE_ERR_UNSUPPORTED
    # a K-split launch needs a workspace
    assert L.eagle_qmm_w4g64_f16(p, p, p, p, None, p, 32, 512, 3584, 64, 4, None, 0, None) == 5
    assert L.eagle_qmm_workspace_bytes(32, 512, 3584) > 65536
    assert L.eagle_qmm_workspace_bytes(8, 152064, 3584) == 65536


def test_other_entry_points_reject_bad_arguments():
    L = _lib.lib()
    buf = (ctypes.c_char * 4096)()
    p = (ctypes.addressof(buf) + 15) & ~15
    assert L.eagle_rope_arrayed_f16(None, p, p, 1.0, p, 1, 1, 1, 64, None) == 1
    assert L.eagle_rope_arrayed_f16(p, p, p, 1.0, p, 1, 1, 1, 63, None) == 2
    assert L.eagle_rope_kv_append_f16(p, p, p, p, p, 1.0, p, p, p, p, 33, 4, 2, 64, 100, 0, None) == 2
    assert L.eagle_rope_kv_append_f16(p, p, p, p, p, 1.0, p, p, p, p, 8, 4, 2, 64, 100, 100, None) == 2
    assert L.eagle_tree_attention_f16(p, p, p, p, p, p, 32, 28, 4, 96, 4096, 2080, 0.1, p, 1 << 30, None) == 2
    assert L.eagle_tree_attention_f16(p, p, p, p, p, p, 32, 28, 4, 128, 4096, 2080, 0.1, None, 0, None) == 5
    assert L.eagle_rmsnorm_f16(p, None, p, 1e-6, None, p, 4, 100, None) == 2
    assert L.eagle_rmsnorm_f16(p, p, p, 1e-6, None, p, 4, 128, None) == 1      # residual needs h_out
    assert L.eagle_silu_mul_f16(p, None, p, 4, 12, None) == 2
    assert L.eagle_add_f16(p, p, p + 2, 16, None) == 3
    assert L.eagle_embed_w4g64_f16(p, p, p, p, p, 4, 100, 10, None) == 2
    assert L.eagle_argmax_rows_f16(p, p, 4, 1000, None, 0, None) == 5
    assert L.eagle_process_draft_tree(p, p, p, p, 200, 8, 64, p, p, p, p, None) == 2    # total must be < 64
    assert L.eagle_process_draft_tree(p, p, p, p, 2000, 8, 31, p, p, p, p, None) == 2   # too many candidates
    assert L.eagle_post_process_draft_tree(p, p, 0, p, p, None) == 2
    assert L.eagle_greedy_accept(p, p, p, p, 65, p, p, None) == 2
    assert L.eagle_kv_compact_f16(None, 4, p, p, 4, 128, 100, None) == 1
    assert L.eagle_tree_positions(p, p, p, 0, None) == 2


def test_plan_is_consistent_for_benchmark_shapes():
    for M in (1, 8, 16, 24, 32):
        for N, K in ((3584, 3584), (512, 3584), (18944, 3584), (3584, 18944), (152064, 3584),
                     (8192, 2048), (896, 896), (128, 896), (4864, 896), (896, 4864), (151936, 896),
                     (4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336), (128256, 4096)):
            nw, phases, splits, ranges, cw = ops.qmm_plan(M, N, K)
            assert cw == 256 if M <= 16 else cw in (128, 256)
            assert nw * phases * splits * cw >= K > nw * phases * (splits - 1) * cw
            assert 1 <= nw <= (14 if M <= 16 or cw == 128 else 10) and 1 <= phases <= 2
            assert 1 <= ranges <= -(-N // 16)
            assert ranges * splits <= 1024


def test_ops_refuse_cpu_tensors():
    x = torch.zeros(8, 128, dtype=torch.float16)
    w = torch.zeros(8, 16, dtype=torch.int32)
    s = torch.zeros(8, 2, dtype=torch.float16)
    with pytest.raises(RuntimeError):
        ops.quantized_matmul(x, w, s, s)
    with pytest.raises(RuntimeError):
        ops.arrayed_rope(torch.zeros(1, 1, 2, 64, dtype=torch.float16), torch.zeros(1, 2, dtype=torch.int32))


def test_mask_bit_helpers_round_trip():
    from mlx_eagle_spec_decoding_tree_amd import eagle
    vis = torch.tril(torch.ones(32, 32, dtype=torch.bool))
    bits = ops.mask_to_bits(vis)
    assert bits.dtype == torch.int32 and bits[0].item() == 1 and bits[31].item() == -1
    back = eagle.bits_to_mask(bits, torch.float32)
    assert torch.equal(back == 0, vis)
    assert torch.equal(ops.mask_to_bits(back), bits)


def test_outgrown_workspaces_stay_allocated():
    """A captured graph may hold a workspace address, and beginning a later capture hands every
    free block back to the driver: a workspace that is outgrown must not be released."""
    import torch
    from mlx_eagle_spec_decoding_tree_amd import ops

    cpu = torch.device("cpu")
    a = ops.workspace("test_outgrown", 100_000, cpu)
    assert ops.workspace("test_outgrown", 50_000, cpu) is a          # large enough: reused
    b = ops.workspace("test_outgrown", 300_000, cpu)
    assert b is not a and b.numel() >= 300_000
    assert any(t is a for t in ops._RETIRED)


def test_draft_side_entry_points_reject_bad_arguments():
    L = _lib.lib()
    buf = (ctypes.c_char * 4096)()
    p = (ctypes.addressof(buf) + 15) & ~15
    big = 1 << 30
    # draft attention: T <= 32 queries, Tk <= 64 masked rows
    assert L.eagle_draft_attention_f16(p, p, p, None, p, p, 8, 24, 14, 2, 64, 4096, 2048, 0.1, p, big, None) == 1
    assert L.eagle_draft_attention_f16(p, p, p, p, p, p, 33, 24, 14, 2, 64, 4096, 2048, 0.1, p, big, None) == 2
    assert L.eagle_draft_attention_f16(p, p, p, p, p, p, 8, 65, 14, 2, 64, 4096, 2048, 0.1, p, big, None) == 2
    assert L.eagle_draft_attention_f16(p, p, p, p, p, p, 8, 24, 14, 2, 64, 4096, 8192, 0.1, p, big, None) == 2
    assert L.eagle_draft_attention_f16(p, p, p, p, p, p, 8, 24, 14, 2, 64, 4096, 2048, 0.1, None, 0, None) == 5
    # causal chunk attention: rows a multiple of 32, at most 2048; a positive scale
    assert L.eagle_causal_attention_f16(p, p, p, p, p, 48, 14, 2, 64, 4096, 2048, 0.1, p, big, None) == 2
    assert L.eagle_causal_attention_f16(p, p, p, p, p, 2080, 14, 2, 64, 4096, 2048, 0.1, p, big, None) == 2
    assert L.eagle_causal_attention_f16(p, p, p, p, p, 64, 14, 2, 64, 4096, 2048, 0.0, p, big, None) == 2
    assert L.eagle_draft_attention_f16(p, p, p, p, p, p, 8, 24, 14, 2, 64, 4096, 2048, -0.1, p, big, None) == 2
    assert L.eagle_causal_attention_f16(p, p, p, p, p, 512, 14, 2, 64, 4096, 2048, 0.1, p, 1024, None) == 5
    assert (L.eagle_causal_attention_workspace_bytes(512, 14, 64, 2048)
            == 16 * L.eagle_tree_attention_workspace_bytes(14, 64, 2048))
    # log-softmax + top-k: k <= 8, k <= V, modes 0 and 1
    assert L.eagle_logsoftmax_topk_f16(None, None, 8, 1000, 8, 0, p, p, p, big, None) == 1
    assert L.eagle_logsoftmax_topk_f16(p, None, 8, 1000, 9, 0, p, p, p, big, None) == 2
    assert L.eagle_logsoftmax_topk_f16(p, None, 8, 4, 8, 0, p, p, p, big, None) == 2
    assert L.eagle_logsoftmax_topk_f16(p, None, 33, 1000, 8, 0, p, p, p, big, None) == 2
    assert L.eagle_logsoftmax_topk_f16(p, None, 8, 1000, 8, 2, p, p, p, big, None) == 4
    assert L.eagle_logsoftmax_topk_f16(p, None, 8, 152064, 8, 1, p, p, p, 1024, None) == 5
    assert L.eagle_logsoftmax_topk_workspace_bytes(8, 152064) == 8 * 38 * 18 * 4
    # tree bookkeeping: k <= 8, k * depth <= 64, level < depth
    assert L.eagle_draft_tree_init(p, p, 9, p, p, p, p, p, p, None) == 2
    assert L.eagle_draft_tree_init(p, None, 8, p, p, p, p, p, p, None) == 1
    assert L.eagle_draft_tree_level(p, p, 3, 8, 3, p, p, p, p, p, p, p, p, None) == 2
    assert L.eagle_draft_tree_level(p, p, 0, 8, 9, p, p, p, p, p, p, p, p, None) == 2
    assert L.eagle_draft_tree_level(p, p, 0, 8, 3, p, p, p, p, p, p, None, p, None) == 1
    assert L.eagle_spec_begin(p, None, p, p, None) == 1
    assert L.eagle_spec_update(p, p, p, 0, p, p, p, p, p, 16, None) == 2
    assert L.eagle_spec_update(p, p, p, 8, p, p, p, p, p, 0, None) == 2
    # many-row matmul
    assert L.eagle_qmm_gemm_w4g64_f16(p, p, p, p, None, None, 512, 128, 128, 64, 4, None) == 1
    assert L.eagle_qmm_gemm_w4g64_f16(p, p, p, p, None, p, 512, 100, 128, 64, 4, None) == 2
    assert L.eagle_qmm_gemm_w4g64_f16(p, p, p, p, None, p, 512, 128, 100, 64, 4, None) == 2
    assert L.eagle_qmm_gemm_w4g64_f16(p, p, p, p, None, p, 512, 128, 128, 32, 4, None) == 4
    assert L.eagle_qmm_gemm_w4g64_f16(p + 2, p, p, p, None, p, 512, 128, 128, 64, 4, None) == 3


def test_slab_form_entry_points_reject_bad_arguments():
    L = _lib.lib()
    buf = (ctypes.c_char * 4096)()
    p = (ctypes.addressof(buf) + 15) & ~15
    big = 1 << 30
    assert L.eagle_qmm_slab_count(3584, 8) == 7 and L.eagle_qmm_slab_count(18944, 32) == 10
    assert L.eagle_qmm_slab_count(896, 8) == 2 and L.eagle_qmm_slab_count(4864, 32) == 3
    assert L.eagle_qmm_slab_count(832, 8) == 0 and L.eagle_qmm_slab_count(1024, 12) == 0
    assert L.eagle_qmm_slab_partial_bytes(4608, 3584, 8) == 7 * 32 * 4608 * 4
    # the library's choice: the small projections of the 7B / 8B models, not gate|up or the head
    assert L.eagle_qmm_slab_steps(32, 4608, 3584) == 8 and L.eagle_qmm_slab_steps(32, 3584, 18944) == 32
    assert L.eagle_qmm_slab_steps(8, 4096, 4096) == 8 and L.eagle_qmm_slab_steps(32, 4096, 14336) == 32
    assert L.eagle_qmm_slab_steps(32, 37888, 3584) == 0 and L.eagle_qmm_slab_steps(32, 152064, 3584) == 0
    assert L.eagle_qmm_slab_steps(32, 1152, 896) == 0 and L.eagle_qmm_slab_steps(65, 4608, 3584) == 0
    # 33..64 rows (a tree above 32 tokens): the same choice, partial tiles of 64 rows
    assert L.eagle_qmm_slab_steps(40, 4608, 3584) == 8 and L.eagle_qmm_slab_steps(64, 3584, 18944) == 32
    assert L.eagle_qmm_slab_partial_bytes_rows(32, 4608, 3584, 8) == 7 * 32 * 4608 * 4
    assert L.eagle_qmm_slab_partial_bytes_rows(33, 4608, 3584, 8) == 7 * 64 * 4608 * 4
    assert L.eagle_qmm_slab_partial_bytes_rows(65, 4608, 3584, 8) == 0
    call = lambda **kw: L.eagle_qmm_slab_partial_w4g64(
        kw.get("x", p), p, p, p, kw.get("partial", p), kw.get("bytes", big), kw.get("M", 32), kw.get("N", 128),
        kw.get("K", 1024), kw.get("gs", 64), kw.get("bits", 4), kw.get("steps", 8), None)
    assert call(x=None) == 1 and call(partial=None) == 1
    assert call(M=65) == 2 and call(N=100) == 2 and call(K=832) == 2 and call(steps=12) == 2
    assert call(M=33, bytes=2 * 32 * 128 * 4) == 5
    assert call(x=p + 2) == 3
    assert call(gs=32) == 4
    assert call(bytes=1024) == 5
    assert L.eagle_slab_sum_f16(p, 0, None, p, 8, 128, None) == 2
    assert L.eagle_slab_sum_f16(p, 2, None, p, 65, 128, None) == 2
    assert L.eagle_slab_sum_f16(p, 2, p + 2, p, 8, 128, None) == 3
    assert L.eagle_rmsnorm_slabs_f16(p, 2, None, p, 1e-6, None, p, 65, 128, None) == 2
    assert L.eagle_rmsnorm_slabs_f16(p, 0, None, p, 1e-6, None, p, 8, 128, None) == 2
    assert L.eagle_rmsnorm_slabs_f16(p, 2, p, p, 1e-6, None, p, 8, 128, None) == 1     # residual needs h_out
    assert L.eagle_rope_kv_append_slabs_f16(p, 2, None, p, p, p, p, p, 65, 4, 2, 64, 100, None) == 2
    assert L.eagle_rope_kv_append_slabs_f16(p, 2, None, p, p, p, p, p, 8, 4, 3, 64, 100, None) == 2
    assert L.eagle_rope_kv_append_slabs_f16(p, 2, p + 2, p, p, p, p, p, 8, 4, 2, 64, 100, None) == 3
    assert L.eagle_rope_kv_append_slabs_f16(None, 2, None, p, p, p, p, p, 8, 4, 2, 64, 100, None) == 1


def test_length_budget_bounds_the_device_length():
    """The verifier's host-side bound of the device cache length: no read-back while the bound
    is below the capacity, one read-back when it reaches it, ValueError when the true length
    leaves no room for a step."""
    from mlx_eagle_spec_decoding_tree_amd.eagle import LengthBudget
    reads = []
    true_len = [100]

    def read():
        reads.append(true_len[0])
        return true_len[0]

    b = LengthBudget(capacity=200, rows_per_step=32, length=100)
    for _ in range(3):                       # bound 100 -> 196: fits without asking the device
        b.reserve(read)
        true_len[0] += 1                     # the device really keeps one row per step
    assert reads == []
    b.reserve(read)                          # bound 196 + 32 > 200: read back 103, fits again
    assert reads == [103] and b.bound == 135
    true_len[0] = 170
    b.reset(170)
    with pytest.raises(ValueError):
        b.reserve(read)                      # 170 + 32 > 200
    assert reads == [103, 170]
    b.reset(168)
    true_len[0] = 168
    b.reserve(read)                          # 168 + 32 == 200 still fits


def test_build_fails_on_registers_spilled_to_scratch_memory():
    """The build reads the compiler's per-kernel resource report: a kernel outside the allowed
    list with a non-zero scratch size is an error, one on the list is reported, none is fine."""
    from mlx_eagle_spec_decoding_tree_amd import build
    remark = ("a.hip:7:1: remark: Function Name: {n} [-Rpass-analysis=kernel-resource-usage]\n"
              "a.hip:7:1: remark:     VGPRs: 128 [-Rpass-analysis=kernel-resource-usage]\n"
              "a.hip:7:1: remark:     ScratchSize [bytes/lane]: {b} [-Rpass-analysis=kernel-resource-usage]\n")
    clean = "_ZN12_GLOBAL__N_121qmm_burst_w4g64_kernelILi5ELb1ELb1ELi7ELi7EEEvPKDF16_"
    listed = "_ZN12_GLOBAL__N_121qmm_gemm_w4g64_kernelILi2ELi4ELi4ELi1ELb0EEEvPKDF16_PKjS2_S2_S2_PDF16_iii"
    rep = build.scratch_report(remark.format(n=clean, b=0) + remark.format(n=listed, b=8))
    assert rep == {clean: 0, listed: 8}
    allowed = build.check_scratch(rep)
    assert list(allowed) == [listed] and allowed[listed][0] == 8
    with pytest.raises(RuntimeError, match="spilled to scratch"):
        build.check_scratch(build.scratch_report(remark.format(n=clean, b=48)))
    # the drafter's down projection (sixteen waves, one tile, no norm) is not on the list
    small = "_ZN12_GLOBAL__N_116qmm_small_kernelILi16ELi2ELi0ELb0EEEvNS_9SmallArgsE"
    with pytest.raises(RuntimeError):
        build.check_scratch({small: 4})


def test_gemm_refuses_an_x_beyond_32_bit_indexing():
    """The many-row matmul indexes x with 32 bits: M * K >= 2^31 is a shape error on the host."""
    L = _lib.lib()
    buf = (ctypes.c_char * 4096)()
    p = (ctypes.addressof(buf) + 15) & ~15
    assert L.eagle_qmm_gemm_w4g64_f16(p, p, p, p, None, p, 1 << 20, 64, 2048, 64, 4, None) == 2
    assert L.eagle_qmm_gemm_w4g64_f16(None, p, p, p, None, p, 64, 64, 2048, 64, 4, None) == 1
