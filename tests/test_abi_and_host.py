"""No-GPU checks: the C-ABI library loads and exports every symbol include/fdattn.h declares,
argument errors are reported without touching the device, and the host-side logic
(rope table, sequence bookkeeping, argument validation) behaves."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import fastdeploy_amd as fd
from fastdeploy_amd import _lib, ops
from fastdeploy_amd import synthetic as syn

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = open(os.path.join(ROOT, "include", "fdattn.h")).read()


def declared_symbols():
    return re.findall(r"FDATTN_API\s+[\w\s\*]+?\b(fdattn_\w+)\s*\(", HEADER)


def test_header_declares_the_entry_points():
    names = declared_symbols()
    for n in ["fdattn_write_cache_kv", "fdattn_decode_attention", "fdattn_decode_attention_sparse",
              "fdattn_splitkv_combine", "fdattn_sqattn_select", "fdattn_append_attention_prefill",
              "fdattn_version", "fdattn_last_error"]:
        assert n in names
    assert len(names) == len(set(names))


def test_library_exports_every_declared_symbol_and_binding_covers_them():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in declared_symbols():
        assert hasattr(lib, n), "libfdattn.so does not export %s" % n
        assert n in _lib.SIGNATURES, "ctypes binding misses %s" % n
    assert set(_lib.SIGNATURES) == set(declared_symbols())


def test_binding_argument_counts_match_the_header():
    for name, (_, args) in _lib.SIGNATURES.items():
        m = re.search(r"FDATTN_API[^;(]*?\b%s\s*\(([^;]*?)\)\s*;" % name, HEADER, re.S)
        assert m, name
        params = [p for p in m.group(1).replace("\n", " ").split(",") if p.strip() and p.strip() != "void"]
        assert len(params) == len(args), "%s: header has %d parameters, binding %d" % (name, len(params), len(args))


def test_version_and_argument_errors_need_no_gpu():
    lib = _lib.lib()
    assert lib.fdattn_version().decode().startswith("fdattn ")
    # NULL pointers / bad shapes are rejected before any device call
    rc = lib.fdattn_write_cache_kv(*([None] * 13), 1, 1, 32, 8, 128, 64, 1, 1, 0, 1, 1, None)
    assert rc == -1 and b"NULL" in lib.fdattn_last_error()
    one = ctypes.c_void_p(16)
    rc = lib.fdattn_write_cache_kv(*([one] * 13), 1, 1, 32, 7, 128, 64, 1, 1, 8, 1, 1, None)
    assert rc == -2 and b"shape" in lib.fdattn_last_error()
    rc = lib.fdattn_write_cache_kv(*([one] * 13), 1, 1, 32, 8, 128, 64, 1, 1, 8, 1, 9, None)
    assert rc == -3
    rc = lib.fdattn_decode_attention(*([None] * 10), 0, 1, 32, 8, 128, 64, 1, 1, 1, 0.1, None)
    assert rc == -1
    rc = lib.fdattn_decode_attention(*([one] * 10), 16, 4, 32, 8, 128, 64, 64, 64, 1, 0.1, None)
    assert rc == -4 and b"workspace" in lib.fdattn_last_error()          # 16-byte workspace
    rc = lib.fdattn_decode_attention(*([one] * 10), 1 << 30, 4, 32, 8, 128, 64, 64, 64, 9, 0.1, None)
    assert rc == -3
    rc = lib.fdattn_sqattn_select(*([one] * 10), 0, 2, 32, 8, 128, 64, 8, 8, 4, 2, None)
    assert rc == -4
    rc = lib.fdattn_append_attention_prefill(*([None] * 11), 1, 1, 1, 32, 8, 128, 64, 1, 1, 1, 0.1, None)
    assert rc == -1
    # the one-call step refuses what its decode rows cannot be given before it writes anything: five tokens per
    # decode row with 4 query heads per KV head (20 rows > 16), the same together with the block selector,
    # the selector for rows of two tokens at a head size its MFMA path does not cover
    big = 1 << 40
    for extras, hd in ((_lib.StepExtras(None, None, None, 0.0, 0, 0, 5), 128), (_lib.StepExtras(None, None, None, 0.0, 0, 4, 5), 128),
                       (_lib.StepExtras(None, None, None, 0.0, 0, 4, 2), 64)):
        rc = lib.fdattn_append_attention_ex(*([one] * 14), big, 4, 2, 0, 32, 8, hd, 64, 8, 16, 64, 0, 1, 0.1,
                                            ctypes.addressof(extras), None)
        assert rc == -2 and (b"decode_tokens" in lib.fdattn_last_error() or b"sqattn_top_k" in lib.fdattn_last_error())
    # a list per token: the decode side runs over batch x decode_tokens rows, and the workspace is sized for those
    per_token = _lib.StepExtras(None, None, None, 0.0, 0, 4, 3, 1)
    fits_the_batch = lib.fdattn_append_attention_workspace_bytes_ex(4, 2, 32, 8, 128, 8, 1)
    assert lib.fdattn_append_attention_workspace_bytes_ex(4, 6, 32, 8, 128, 8, 1) > fits_the_batch
    rc = lib.fdattn_append_attention_ex(*([one] * 14), fits_the_batch, 4, 2, 0, 32, 8, 128, 64, 8, 16, 64, 0, 1, 0.1,
                                        ctypes.addressof(per_token), None)
    assert rc == -4 and b"sqattn_per_token" in lib.fdattn_last_error()
    assert lib.fdattn_decode_workspace_bytes(64, 32, 8, 128, 72) >= 64 * 8 * 3 * 2080
    # at least 16 partial rows (head_dim + 2 floats) per output row at any shape; a batch of fewer (sequence, KV head)
    # pairs than the GPU has CUs gets room for the up to 64 key splits that put a workgroup on each of them
    assert lib.fdattn_decode_workspace_bytes(64, 32, 8, 64, 72) >= 64 * 32 * 16 * 66 * 4
    assert lib.fdattn_decode_workspace_bytes(1, 8, 2, 256, 300) >= 1 * 8 * 64 * 258 * 4
    assert lib.fdattn_decode_workspace_bytes(2, 8, 2, 256, 300) < 2 * (1 * 8 * 64 * 258 * 4 + 256)
    assert lib.fdattn_decode_uses_mfma(32, 8, 128, 64, 1) == 1 and lib.fdattn_decode_uses_mfma(32, 8, 64, 64, 1) == 0
    with pytest.raises(ValueError):
        _lib.check(-2, "x")
    with pytest.raises(_lib.FdattnError):
        _lib.check(700, "x")


def test_dynamic_formats_in_the_argument_checks_and_the_host_helpers():
    """The formats with one scale per stored row: names, what odd head sizes and unknown format numbers answer
    (before any device call), the decode kernel choice and the size of their wire form."""
    lib = _lib.lib()
    one = ctypes.c_void_p(16)
    assert ops._quant("cache_int8_dynamic") == 3 and ops._quant("cache_fp8_dynamic") == 4
    assert ops.is_dynamic("cache_fp8_dynamic") and not ops.is_dynamic("cache_fp8")
    assert ops.byte_format("cache_int8_dynamic") == ops.CACHE_INT8 and ops.byte_format(4) == ops.CACHE_FP8
    assert lib.fdattn_decode_uses_mfma(32, 8, 128, 64, 3) == 1 and lib.fdattn_decode_uses_mfma(32, 8, 128, 64, 4) == 1
    # 1 .. 8 query heads per KV head run on the MFMA decode kernel; more, or a ragged ratio, do not
    assert [lib.fdattn_decode_uses_mfma(g * 8, 8, 128, 64, 1) for g in (1, 2, 5, 8, 9)] == [1, 1, 1, 1, 0]
    assert lib.fdattn_decode_uses_mfma(36, 8, 128, 64, 1) == 0
    # the workspace of two row sets (5 .. 8 heads) is twice that of one
    assert lib.fdattn_decode_workspace_bytes(1, 64, 8, 128, 2048) > lib.fdattn_decode_workspace_bytes(1, 32, 8, 128, 2048)
    rc = lib.fdattn_write_cache_kv(*([one] * 13), 1, 1, 4, 2, 96, 64, 1, 1, 8, 1, 3, None)    # 96 / 16 = 6 threads a row
    assert rc == -2 and b"dynamic" in lib.fdattn_last_error()
    rc = lib.fdattn_sqattn_select(*([one] * 10), 1 << 30, 2, 32, 8, 128, 64, 8, 8, 4, 7, None)
    assert rc == -3 and b"unknown" in lib.fdattn_last_error()
    # wire form: the scales section grows with the pages instead of holding 2 x hkv x head_dim floats
    stat, dyn = lib.fdattn_kv_wire_bytes_for(130, 8, 128, 64, 1), lib.fdattn_kv_wire_bytes_for(130, 8, 128, 64, 3)
    assert stat == lib.fdattn_kv_wire_bytes(130, 8, 128, 64)
    assert dyn - stat == 3 * 2 * 8 * 64 * 4 - 2 * 8 * 128 * 4
    assert lib.fdattn_kv_wire_bytes_for(130, 8, 128, 64, 7) == 0
    case = syn.decode_case(batch=2, ctx=[70, 3], quant="cache_int8_dynamic")
    assert case["cache_k_scale"].shape == (case["key_cache"].shape[0], 8, 64)
    with pytest.raises(ValueError, match="CUDA/HIP"):      # (shape checks come after the device checks)
        fd.decode_attention(case["q"], case["key_cache"], case["value_cache"], case["cache_k_scale"],
                            case["cache_v_scale"], case["block_tables"], case["seq_lens_decoder"], num_heads=32,
                            cache_quant_type="cache_int8_dynamic")


def test_per_block_formats_in_the_argument_checks_and_the_host_helpers():
    """The formats with one scale per (block, KV head) tile: names, shapes of the scale caches, kernel choice, the
    writer's head-size rule and the size of their wire form - all before any device call."""
    lib = _lib.lib()
    one = ctypes.c_void_p(16)
    assert ops._quant("cache_int8_block") == 5 and ops._quant("cache_fp8_block") == 6
    assert ops.is_blockwise(5) and ops.is_blockwise("cache_fp8_block") and not ops.is_blockwise("cache_fp8_dynamic")
    assert ops.is_dynamic(5) and ops.is_dynamic(6)        # their scales live in scale caches, too
    assert ops.byte_format(5) == ops.CACHE_INT8 and ops.byte_format("cache_fp8_block") == ops.CACHE_FP8
    assert ops.scale_cache_shape(5, 40, 8, 64) == (40, 8) and ops.scale_cache_shape(3, 40, 8, 64) == (40, 8, 64)
    assert lib.fdattn_decode_uses_mfma(32, 8, 128, 64, 5) == 1 and lib.fdattn_decode_uses_mfma(32, 8, 128, 64, 6) == 1
    rc = lib.fdattn_write_cache_kv(*([one] * 13), 1, 1, 4, 2, 96, 64, 1, 1, 8, 1, 6, None)    # 96 / 16 = 6 threads a row
    assert rc == -2 and b"per-block" in lib.fdattn_last_error()
    stat, blk = lib.fdattn_kv_wire_bytes_for(130, 8, 128, 64, 1), lib.fdattn_kv_wire_bytes_for(130, 8, 128, 64, 5)
    assert blk - stat == (256 + 3 * 2 * 8 * 4 + 255) // 256 * 256 - (256 + 2 * 8 * 128 * 4)
    case = syn.decode_case(batch=2, ctx=[70, 3], quant="cache_fp8_block")
    pool = case["key_cache"].shape[0]
    assert case["cache_k_scale"].shape == (pool, 8) and case["cache_v_scale"].shape == (pool, 8)
    # every tile that holds a token carries max-abs / 448: its largest code is the format's largest
    bt, k8 = case["block_tables"], case["key_cache"]
    for b, blocks in ((0, 2), (1, 1)):
        for j in range(blocks):
            assert ((k8[int(bt[b, j])] & 0x7F).amax((1, 2)) == 0x7E).all()


def test_ops_reject_cpu_tensors_and_bad_dtypes():
    case = syn.decode_case(batch=2, ctx=64)
    with pytest.raises(ValueError, match="CUDA/HIP"):
        fd.decode_attention(case["q"], case["key_cache"], case["value_cache"], case["cache_k_scale"],
                            case["cache_v_scale"], case["block_tables"], case["seq_lens_decoder"], num_heads=32)
    with pytest.raises(ValueError):
        ops._quant("cache_int4")


def test_sequence_bookkeeping():
    enc = torch.tensor([0, 5, 0, 0], dtype=torch.int32)
    dec = torch.tensor([7, 0, 0, 100], dtype=torch.int32)
    tt = ops.seq_lens_this_time_of(enc, dec)
    assert tt.tolist() == [1, 5, 0, 1] and tt.dtype == torch.int32
    assert ops.cu_seqlens_of(tt).tolist() == [0, 1, 6, 6, 7]


def test_synthetic_workloads_are_seeded_and_well_formed():
    a = syn.decode_case(batch=4, ctx=1024, pool_blocks=64, seed=3)
    b = syn.decode_case(batch=4, ctx=1024, pool_blocks=64, seed=3)
    assert torch.equal(a["key_cache"], b["key_cache"]) and torch.equal(a["block_tables"], b["block_tables"])
    assert sorted(a["block_tables"].flatten().tolist()) == list(range(64))         # a permutation of the pool
    k = a["key_cache"].view(torch.int8)
    assert int(k.abs().max()) == 127                                               # scale = max-abs / 127
    c = syn.decode_case(batch=3, ctx=(100, 200), seed=1, extra_blocks=3)
    assert all(100 <= n <= 200 for n in c["seq_lens_decoder"].tolist())
    assert int((c["block_tables"] >= 0).sum()) == sum((n + 63) // 64 for n in c["seq_lens_decoder"].tolist())
    assert syn.decode_kv_bytes([4096] * 64) == 536870912
    assert syn.prefill_flops(8192, 2048) * 2 == 618508845056      # 4 * 128 * 32 * 2 * sum_i (8192 + i + 1), i < 2048
    w = syn.write_case(num_seqs=5, max_pos=300, chunk=3)
    assert w["cu_seqlens_q"].tolist() == [0, 3, 6, 9, 12, 15] and w["qkv"].shape == (15, 48 * 128)


def test_decode_workspace_covers_every_list_length_up_to_the_table_width():
    """The sparse entry point cuts lists of min(max_kept, max_blocks) units, and the chunk count is not monotonic in
    the list length (213 units may be cut into more chunks than 257): the workspace documented for max_blocks must
    hold the partials of every shorter list too.  Sizes only - no GPU needed."""
    lib = _lib.lib()
    for batch, hq, hkv, max_blocks in ((1, 32, 8, 257), (1, 32, 8, 33), (2, 64, 8, 300), (3, 32, 8, 2048), (7, 8, 8, 100)):
        full = lib.fdattn_decode_workspace_bytes(batch, hq, hkv, 128, max_blocks)
        for max_kept in range(1, max_blocks + 1):
            need = lib.fdattn_decode_workspace_bytes(batch, hq, hkv, 128, max_kept)
            assert need <= full, "batch %d max_blocks %d: lists of %d units need %d B > %d B" % (batch, max_blocks, max_kept, need, full)
    # the chunk count a launch uses never exceeds what the workspace was sized with
    for max_blocks in (33, 213, 257):
        chunks = [lib.fdattn_decode_chunks_per_sequence(1, 8, u) for u in range(1, max_blocks + 1)]
        sets = 1
        assert lib.fdattn_decode_workspace_bytes(1, 32, 8, 128, max_blocks) >= 8 * max(chunks) * sets * (4 * 128 + 8) * 4


def test_noalloc_decode_refuses_oversized_shapes_without_touching_the_device():
    lib = _lib.lib()
    one = ctypes.c_void_p(256)
    assert lib.fdattn_decode_noalloc_scratch_bytes() == 16 << 20
    assert lib.fdattn_decode_workspace_bytes(9000, 32, 8, 128, 72) > lib.fdattn_decode_noalloc_scratch_bytes()
    rc = lib.fdattn_decode_attention_noalloc(*([one] * 7), None, one, 9000, 32, 8, 128, 64, 72, 6000, 1, 0.1, None)
    assert rc == -4 and b"static scratch" in lib.fdattn_last_error()
    rc = lib.fdattn_decode_attention_noalloc(*([None] * 9), 4, 32, 8, 128, 64, 72, 6000, 1, 0.1, None)
    assert rc == -1


def test_sequence_book_and_backend_check_lengths_against_max_position():
    from fastdeploy_amd import BlockPool, SequenceBook
    book = SequenceBook(BlockPool(16, 64, 2, 8), device="cpu", max_position=100)
    meta = book.schedule({0: 90})
    assert meta.max_len_after == 90
    book.commit()
    with pytest.raises(ValueError, match="max_position"):
        book.schedule({0: 11})
    meta = book.schedule({0: 10, 1: 3})
    assert meta.max_len_after == 100 and meta.seq_lens_encoder.tolist() == [10, 3]


def test_pool_create_reports_bad_and_absurd_shapes():
    lib = _lib.lib()
    assert not lib.fdattn_pool_create(0, 64, 1, 1) and b"bad shape" in lib.fdattn_last_error()
    # a table no host could hold: an error return, nothing unwinds through the C ABI
    assert not lib.fdattn_pool_create(1, 64, 0x7fffffff, 0x7fffffff)
    assert b"out of host memory" in lib.fdattn_last_error()


def test_register_plan_parser_reads_both_ends_of_a_register_range():
    """The build fails when the compiler's own allocation reaches the accumulation registers that prefill_v2.hip
    addresses by name; the check reads the device assembly, where a tuple `a[28:43]` starts below the limit of 32 and
    ends above it."""
    from fastdeploy_amd.build import highest_agpr
    assert highest_agpr("\tv_accvgpr_write_b32 a[28:43], v1") == 43
    assert highest_agpr("\tv_mfma_f32_32x32x16_f16 a[0:15], v[2:5], v[6:9], a[0:15]") == 15
    assert highest_agpr("\tv_accvgpr_read_b32 v3, a31") == 31
    assert highest_agpr("\tv_accvgpr_read_b32 v3, a7 ; was a[100:131]") == 7
    assert highest_agpr("\tv_add_f32 v1, v2, v3") == -1
    assert highest_agpr("\tds_read_b128 v[28:31], v40 offset:32") == -1
    assert highest_agpr("\tv_accvgpr_mov_b32 a[33], a2") == 33
