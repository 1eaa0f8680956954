"""SQAttn selector (bit-exact indices) and append/prefill attention on the GPU against the oracle."""
import numpy as np
import pytest
import torch

import fastdeploy_amd as fd
from conftest import bf16_close, bits, np_of
from fastdeploy_amd import synthetic as syn
from fastdeploy_amd.ops import (CACHE_FP8, CACHE_FP8_BLOCK, CACHE_FP8_DYNAMIC, CACHE_INT8, CACHE_INT8_BLOCK,
                                CACHE_INT8_DYNAMIC, is_dynamic)

ALL_FORMATS = [CACHE_INT8, CACHE_FP8, CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC, CACHE_INT8_BLOCK, CACHE_FP8_BLOCK]

pytestmark = pytest.mark.gpu


def oracle_select(oracle, case, top_k):
    s = oracle.sqattn_block_scores(bits(case["q"]), np_of(case["key_cache"]), np_of(case["cache_k_scale"]),
                                   np_of(case["block_tables"]), np_of(case["seq_lens_decoder"]), case["hq"],
                                   case["hkv"], case["d"], case["quant"])
    kept, cnt = oracle.topk_select(s, np_of(case["seq_lens_decoder"]), case["bs"], top_k)
    return s, kept, cnt


@pytest.mark.parametrize("impl", ["auto", "exact"])
@pytest.mark.parametrize("quant", ALL_FORMATS)
def test_selector_indices_bit_exact(oracle, quant, impl):
    for seed in range(2):
        case = syn.decode_case(batch=3, ctx=[4096, 3000, 64 * 20 + 1], quant=quant, seed=seed, salient=0.05)
        dev = syn.to_device(case, "cuda")
        for k in (8, 17):
            kept, cnt, sc = fd.sqattn_select(dev["q"], dev["key_cache"], dev["cache_k_scale"], dev["block_tables"],
                                             dev["seq_lens_decoder"], num_heads=32, top_k=k, cache_quant_type=quant,
                                             return_scores=True, impl=impl)
            s, okept, ocnt = oracle_select(oracle, case, k)
            assert np.array_equal(np_of(cnt), ocnt)
            assert np.array_equal(np_of(kept), okept)
            if impl == "exact":
                assert np.array_equal(np_of(sc), s.astype(np.float32))
            else:   # the MFMA scores the selection starts from: close to the fp64 ones, -inf in the same places
                got = np_of(sc).astype(np.float64)
                fin = np.isfinite(s)
                assert np.array_equal(np.isfinite(got), fin)
                assert np.abs(got[fin] - s[fin]).max() <= 2e-3 * np.abs(s[fin]).max()


@pytest.mark.parametrize("impl", ["auto", "exact"])
@pytest.mark.parametrize("quant", ALL_FORMATS)
def test_selector_ties_near_ties_and_short_sequences(oracle, quant, impl):
    case = syn.decode_case(batch=2, ctx=[64 * 12, 100], quant=quant, seed=3)
    bt = case["block_tables"]
    dyn = is_dynamic(quant)
    # identical K pages (and, for the dynamic formats, scale rows) -> identical scores -> the lower block index must win
    for j in (5, 7, 9):
        case["key_cache"][int(bt[0, j])] = case["key_cache"][int(bt[0, 2])]
        if dyn:
            case["cache_k_scale"][int(bt[0, j])] = case["cache_k_scale"][int(bt[0, 2])]
    # near ties: copies that differ by one code step in one channel of every token
    for j, ch in ((3, 0), (10, 77)):
        page = case["key_cache"][int(bt[0, 2])].clone()
        page[:, :, ch] = torch.where((page[:, :, ch] & 0x7F) < 0x70, page[:, :, ch] + 1, page[:, :, ch])
        case["key_cache"][int(bt[0, j])] = page
        if dyn:
            case["cache_k_scale"][int(bt[0, j])] = case["cache_k_scale"][int(bt[0, 2])]
    dev = syn.to_device(case, "cuda")
    for k in (1, 2, 3, 4, 5, 6, 7, 11, 12, 64):
        kept, cnt = fd.sqattn_select(dev["q"], dev["key_cache"], dev["cache_k_scale"], dev["block_tables"],
                                     dev["seq_lens_decoder"], num_heads=32, top_k=k, cache_quant_type=quant, impl=impl)
        _, okept, ocnt = oracle_select(oracle, case, k)
        assert np.array_equal(np_of(kept), okept) and np.array_equal(np_of(cnt), ocnt), k


@pytest.mark.parametrize("quant", ALL_FORMATS)
@pytest.mark.parametrize("group", [1, 3, 5, 8])
def test_selector_other_group_sizes(oracle, group, quant):
    """1 .. 8 query heads per KV head on the fast path (MFMA scores + exact resolution): indices bit for bit as the
    oracle's and as the all-fp64 path's, including planted ties."""
    hkv = 2
    hq = group * hkv
    case = syn.decode_case(batch=3, ctx=[64 * 40, 64 * 17 + 9, 100], quant=quant, seed=50 + group, salient=0.1,
                           hq=hq, hkv=hkv)
    bt = case["block_tables"]
    for j in (6, 11):   # identical pages -> identical scores -> the lower index wins
        case["key_cache"][int(bt[0, j])] = case["key_cache"][int(bt[0, 2])]
        if is_dynamic(quant):
            case["cache_k_scale"][int(bt[0, j])] = case["cache_k_scale"][int(bt[0, 2])]
    dev = syn.to_device(case, "cuda")
    for k in (1, 5, 16):
        _, okept, ocnt = oracle_select(oracle, case, k)
        for impl in ("auto", "exact"):
            kept, cnt = fd.sqattn_select(dev["q"], dev["key_cache"], dev["cache_k_scale"], dev["block_tables"],
                                         dev["seq_lens_decoder"], num_heads=hq, top_k=k, cache_quant_type=quant, impl=impl)
            assert np.array_equal(np_of(kept), okept) and np.array_equal(np_of(cnt), ocnt), (k, impl)


@pytest.mark.parametrize("quant", ALL_FORMATS)
@pytest.mark.parametrize("hq,hkv,d,bs", [(8, 4, 64, 16), (8, 2, 64, 64), (16, 4, 128, 32), (32, 8, 128, 16), (8, 8, 128, 128),
                                         (8, 4, 256, 64), (4, 2, 256, 8), (6, 2, 128, 24), (8, 1, 64, 48), (14, 2, 128, 256)])
def test_selector_other_shapes_on_the_mfma_path(oracle, hq, hkv, d, bs, quant):
    """head_dim 64 / 128 / 256 at block sizes 8 .. 256 (two that are no powers of two): block scores and bounds from the
    fp16-MFMA decode kernel's K half, classification, fp64 re-scoring of the undecided blocks.  Kept indices bit for bit
    as the oracle's and as the all-fp64 path's - ragged lengths with partial last blocks, planted ties (identical
    pages: the lower index wins) - and the MFMA scores close to the fp64 ones, -inf in the same places."""
    from fastdeploy_amd import _lib
    assert _lib.lib().fdattn_sqattn_path(hq, hkv, d, bs, 2048) == (1 if (d, bs) == (128, 64) else 2)
    nb = 40
    lens = [bs * nb, bs * 17 + max(bs // 3, 1), max(bs // 2, 1), bs * 29 - 1]
    case = syn.decode_case(batch=len(lens), ctx=lens, quant=quant, seed=d + bs + hq, salient=0.1, hq=hq, hkv=hkv, d=d, bs=bs,
                           max_blocks=nb + 1)
    bt = case["block_tables"]
    for j in (6, 11):
        case["key_cache"][int(bt[0, j])] = case["key_cache"][int(bt[0, 2])]
        if is_dynamic(quant):
            case["cache_k_scale"][int(bt[0, j])] = case["cache_k_scale"][int(bt[0, 2])]
    dev = syn.to_device(case, "cuda")
    for k in (1, 7, 16):
        s, okept, ocnt = oracle_select(oracle, case, k)
        for impl in ("auto", "exact"):
            kept, cnt, sc = fd.sqattn_select(dev["q"], dev["key_cache"], dev["cache_k_scale"], dev["block_tables"],
                                             dev["seq_lens_decoder"], num_heads=hq, top_k=k, cache_quant_type=quant, impl=impl,
                                             return_scores=True)
            assert np.array_equal(np_of(cnt), ocnt), (k, impl)
            assert np.array_equal(np_of(kept), okept), (k, impl)
            if impl == "auto":
                got = np_of(sc).astype(np.float64)
                fin = np.isfinite(s)
                assert np.array_equal(np.isfinite(got), fin)
                assert np.abs(got[fin] - s[fin]).max() <= 1e-3 * np.abs(s[fin]).max()


@pytest.mark.parametrize("quant", ALL_FORMATS)
@pytest.mark.parametrize("hq,hkv,d,bs", [(8, 2, 64, 64), (32, 8, 128, 16), (8, 4, 256, 32), (4, 4, 128, 8), (16, 2, 64, 128)])
def test_selector_other_shapes_empty_and_tiny_sequences(oracle, hq, hkv, d, bs, quant):
    """The fp16-MFMA scoring pass on sequences of 0, 1, one block, one block and a token, and a few blocks, with top_k
    below, at and beyond the number of blocks (a wavefront's walk then starts past its split's end, or ends one tile
    past it): indices as the oracle's, on the MFMA path and on the all-fp64 one."""
    lens = [0, 1, bs, bs + 1, 5 * bs - 1, 7 * bs]
    case = syn.decode_case(batch=len(lens), ctx=lens, quant=quant, seed=3, hq=hq, hkv=hkv, d=d, bs=bs, max_blocks=9, extra_blocks=2)
    dev = syn.to_device(case, "cuda")
    for k in (1, 3, 100):
        _, okept, ocnt = oracle_select(oracle, case, k)
        for impl in ("auto", "exact"):
            kept, cnt = fd.sqattn_select(dev["q"], dev["key_cache"], dev["cache_k_scale"], dev["block_tables"],
                                         dev["seq_lens_decoder"], num_heads=hq, top_k=k, cache_quant_type=quant, impl=impl)
            assert np.array_equal(np_of(cnt), ocnt) and np.array_equal(np_of(kept), okept), (k, impl)


@pytest.mark.parametrize("quant,hq,hkv,d", [(CACHE_FP8, 32, 8, 128), (CACHE_INT8_DYNAMIC, 32, 8, 128), (CACHE_INT8, 8, 1, 256)])
def test_selector_4096_blocks_of_16_tokens(oracle, quant, hq, hkv, d):
    """65,536 tokens at block_size 16: the most blocks the fp16-MFMA selector takes (two splits of 2048 blocks at least:
    a scoring workgroup keeps a split's maxima in LDS), with a shorter sequence beside it; at head_dim 256 with eight
    query heads per KV head the resolve kernel's LDS is at its largest."""
    from fastdeploy_amd import _lib
    assert _lib.lib().fdattn_sqattn_path(hq, hkv, d, 16, 4096) == 2
    case = syn.decode_case(batch=2, ctx=[16 * 4096, 16 * 3000 + 5], quant=quant, seed=6, device="cuda", salient=0.05, hq=hq, hkv=hkv,
                           d=d, bs=16, max_blocks=4096, row_log2=(-6, 0))
    for k in (1, 300):
        kept, cnt = fd.sqattn_select(case["q"], case["key_cache"], case["cache_k_scale"], case["block_tables"],
                                     case["seq_lens_decoder"], num_heads=hq, top_k=k, cache_quant_type=quant)
        torch.cuda.synchronize()
        _, okept, ocnt = oracle_select(oracle, syn.to_device(case, "cpu"), k)
        assert np.array_equal(np_of(cnt), ocnt) and np.array_equal(np_of(kept), okept), k


def test_selector_longest_sequences_of_the_fast_path_and_beyond(oracle):
    """2048 blocks per sequence (131,072 tokens) is the most the int8 / fp8-MFMA scoring pass takes; one block more goes
    to the fp16-MFMA pass, whose resolve kernel holds 4096 blocks in LDS (262,144 tokens: the selector's limit, also
    on the all-fp64 path).  All against the oracle."""
    from fastdeploy_amd import _lib
    assert [_lib.lib().fdattn_sqattn_path(32, 8, 128, 64, n) for n in (2048, 2049, 4096)] == [1, 2, 2]
    for ctx in (64 * 2048, 64 * 2049 + 5, 64 * 4096):
        case = syn.decode_case(batch=1, ctx=ctx, quant=CACHE_INT8, seed=4, device="cuda", direct_bytes=True)
        kept, cnt = fd.sqattn_select(case["q"], case["key_cache"], case["cache_k_scale"], case["block_tables"],
                                     case["seq_lens_decoder"], num_heads=32, top_k=100, cache_quant_type=CACHE_INT8)
        torch.cuda.synchronize()
        _, okept, ocnt = oracle_select(oracle, syn.to_device(case, "cpu"), 100)
        assert np.array_equal(np_of(cnt), ocnt) and np.array_equal(np_of(kept), okept), ctx


@pytest.mark.parametrize("quant", [CACHE_FP8, CACHE_FP8_DYNAMIC, CACHE_FP8_BLOCK])
def test_selector_config4_shape_indices_bit_exact(oracle, quant):
    """batch 16, ctx 32768, fp8 KV, top-64 of 512 blocks per KV head, 5 % salient blocks (scaled x4):
    the full-size launch against the oracle (per-channel scales, and one scale per stored row)."""
    # (dynamic format: row scales up to 2^6 apart with the largest rows at unit scale, where the absolute part of
    # the output tolerance applies; the fp8 weights of the decode kernel carry 16 significant bits)
    case = syn.decode_case(batch=16, ctx=32768, quant=quant, seed=0, device="cuda", salient=0.05, row_log2=(-6, 0))
    kept, cnt = fd.sqattn_select(case["q"], case["key_cache"], case["cache_k_scale"], case["block_tables"],
                                 case["seq_lens_decoder"], num_heads=32, top_k=64, cache_quant_type=quant)
    torch.cuda.synchronize()
    cpu = syn.to_device(case, "cpu")
    _, okept, ocnt = oracle_select(oracle, cpu, 64)
    assert np.array_equal(np_of(cnt), ocnt)
    assert np.array_equal(np_of(kept), okept)
    # and the sparse decode over the kept blocks equals the oracle's
    out = fd.decode_attention_sparse(case["q"], case["key_cache"], case["value_cache"], case["cache_k_scale"],
                                     case["cache_v_scale"], case["block_tables"], case["seq_lens_decoder"],
                                     kept_blocks=kept, kept_counts=cnt, num_heads=32, cache_quant_type=quant)
    want = oracle.decode_attention(bits(cpu["q"]), np_of(cpu["key_cache"]), np_of(cpu["value_cache"]),
                                   np_of(cpu["cache_k_scale"]), np_of(cpu["cache_v_scale"]), np_of(cpu["block_tables"]),
                                   np_of(cpu["seq_lens_decoder"]), 32, 8, 128, quant, kept_blocks=okept, kept_counts=ocnt)
    ok, mx, bad = bf16_close(bits(out), want)
    assert ok, "%d out of tolerance, max %.4g" % (bad, mx)


@pytest.mark.parametrize("d,bs,batch,quant", [(64, 64, 16, CACHE_FP8), (128, 16, 8, CACHE_FP8), (256, 64, 4, CACHE_FP8_DYNAMIC),
                                              (128, 32, 4, CACHE_INT8_BLOCK)])
def test_selector_full_size_at_the_other_shapes(oracle, d, bs, batch, quant):
    """configs[3]'s sequences (32768 tokens, 32 query / 8 KV heads, an eighth of the blocks kept, 5 % salient blocks) at
    head_dim 64 / 128 / 256 and block sizes 16 / 32 / 64: the fp16-MFMA scoring pass at its full launch shape (several
    key splits per pair, 512 .. 2048 blocks per sequence), indices bit for bit as the oracle's; then the decode over
    the kept blocks against the oracle's."""
    from fastdeploy_amd import _lib
    mb = 32768 // bs
    top_k = mb // 8
    assert _lib.lib().fdattn_sqattn_path(32, 8, d, bs, mb) == 2
    case = syn.decode_case(batch=batch, ctx=32768, quant=quant, seed=1, device="cuda", salient=0.05, row_log2=(-6, 0), d=d, bs=bs,
                           max_blocks=mb)
    kept, cnt = fd.sqattn_select(case["q"], case["key_cache"], case["cache_k_scale"], case["block_tables"],
                                 case["seq_lens_decoder"], num_heads=32, top_k=top_k, cache_quant_type=quant)
    torch.cuda.synchronize()
    cpu = syn.to_device(case, "cpu")
    _, okept, ocnt = oracle_select(oracle, cpu, top_k)
    assert np.array_equal(np_of(cnt), ocnt)
    assert np.array_equal(np_of(kept), okept)
    out = fd.decode_attention_sparse(case["q"], case["key_cache"], case["value_cache"], case["cache_k_scale"],
                                     case["cache_v_scale"], case["block_tables"], case["seq_lens_decoder"],
                                     kept_blocks=kept, kept_counts=cnt, num_heads=32, cache_quant_type=quant)
    want = oracle.decode_attention(bits(cpu["q"]), np_of(cpu["key_cache"]), np_of(cpu["value_cache"]),
                                   np_of(cpu["cache_k_scale"]), np_of(cpu["cache_v_scale"]), np_of(cpu["block_tables"]),
                                   np_of(cpu["seq_lens_decoder"]), 32, 8, d, quant, kept_blocks=okept, kept_counts=ocnt)
    ok, mx, bad = bf16_close(bits(out), want)
    assert ok, "%d out of tolerance, max %.4g" % (bad, mx)


def _prefill_case(seed, prefix, chunks, quant=CACHE_INT8):
    batch = len(chunks)
    # the dynamic formats: the stored rows differ in scale by up to 2^6 and reach twice unit scale (dequantised
    # magnitudes up to ~ 9); the kernel's validated range is |V^| <= 8 or so (fp16 softmax weights)
    base = syn.decode_case(batch=batch, ctx=prefix, quant=quant, seed=seed, extra_blocks=4, row_log2=(-5, 1))
    g = torch.Generator().manual_seed(seed + 100)
    T = sum(chunks)
    base["q_new"] = torch.randn((T, 32 * 128), generator=g).to(torch.bfloat16)
    base["k_new"] = torch.randn((T, 8 * 128), generator=g).to(torch.bfloat16)
    base["v_new"] = torch.randn((T, 8 * 128), generator=g).to(torch.bfloat16)
    base["cu_seqlens_q"] = torch.tensor([0] + list(np.cumsum(chunks)), dtype=torch.int32)
    return base


@pytest.mark.parametrize("impl", ["generic", "auto"])
@pytest.mark.parametrize("quant", ALL_FORMATS)
def test_prefill_small(oracle, impl, quant):
    c = _prefill_case(1, [200, 64, 0, 333], [70, 128, 5, 1], quant)
    dev = syn.to_device(c, "cuda")
    out = fd.append_attention_prefill(dev["q_new"], dev["k_new"], dev["v_new"], dev["key_cache"], dev["value_cache"],
                                      dev["cache_k_scale"], dev["cache_v_scale"], dev["block_tables"],
                                      dev["seq_lens_decoder"], dev["cu_seqlens_q"], num_heads=32, max_chunk=128,
                                      cache_quant_type=quant, impl=impl)
    want = oracle.append_attention_prefill(bits(c["q_new"]), bits(c["k_new"]), bits(c["v_new"]), np_of(c["key_cache"]),
                                           np_of(c["value_cache"]), np_of(c["cache_k_scale"]), np_of(c["cache_v_scale"]),
                                           np_of(c["block_tables"]), np_of(c["seq_lens_decoder"]), np_of(c["cu_seqlens_q"]),
                                           32, 8, 128, quant)
    ok, mx, bad = bf16_close(bits(out), want)
    assert ok, "%d out of tolerance, max %.4g" % (bad, mx)


@pytest.mark.parametrize("quant", ALL_FORMATS)
def test_prefill_ragged_edges(oracle, quant):
    """Prefix lengths around the tile size, chunks around the workgroup size, an empty prefix."""
    c = _prefill_case(2, [0, 63, 64, 65, 1000, 129], [129, 128, 1, 127, 257, 64], quant)
    dev = syn.to_device(c, "cuda")
    out = fd.append_attention_prefill(dev["q_new"], dev["k_new"], dev["v_new"], dev["key_cache"], dev["value_cache"],
                                      dev["cache_k_scale"], dev["cache_v_scale"], dev["block_tables"],
                                      dev["seq_lens_decoder"], dev["cu_seqlens_q"], num_heads=32, max_chunk=257,
                                      cache_quant_type=quant)
    want = oracle.append_attention_prefill(bits(c["q_new"]), bits(c["k_new"]), bits(c["v_new"]), np_of(c["key_cache"]),
                                           np_of(c["value_cache"]), np_of(c["cache_k_scale"]), np_of(c["cache_v_scale"]),
                                           np_of(c["block_tables"]), np_of(c["seq_lens_decoder"]), np_of(c["cu_seqlens_q"]),
                                           32, 8, 128, quant)
    ok, mx, bad = bf16_close(bits(out), want)
    assert ok, "%d out of tolerance, max %.4g" % (bad, mx)


@pytest.mark.parametrize("quant", ALL_FORMATS)
def test_prefill_long_chunks_on_no_or_short_prefixes(oracle, quant):
    """Chunks of many key tiles, where most of the walk is over the chunk's own keys: whole tiles below a
    wavefront's diagonal, the diagonal tiles themselves, a chunk that ends inside a tile, and the switch from the
    cached prefix to the chunk one, two and three tiles into the walk - alone and shared by three key splits."""
    c = _prefill_case(5, [0, 64, 130, 192, 0], [1000, 515, 389, 256, 770], quant)
    dev = syn.to_device(c, "cuda")
    want = oracle.append_attention_prefill(bits(c["q_new"]), bits(c["k_new"]), bits(c["v_new"]), np_of(c["key_cache"]),
                                           np_of(c["value_cache"]), np_of(c["cache_k_scale"]), np_of(c["cache_v_scale"]),
                                           np_of(c["block_tables"]), np_of(c["seq_lens_decoder"]), np_of(c["cu_seqlens_q"]),
                                           32, 8, 128, quant)
    for splits in (1, 3):
        out = fd.append_attention_prefill(dev["q_new"], dev["k_new"], dev["v_new"], dev["key_cache"], dev["value_cache"],
                                          dev["cache_k_scale"], dev["cache_v_scale"], dev["block_tables"],
                                          dev["seq_lens_decoder"], dev["cu_seqlens_q"], num_heads=32, max_chunk=1000,
                                          cache_quant_type=quant, num_splits=splits)
        ok, mx, bad = bf16_close(bits(out), want)
        assert ok, "%d splits: %d out of tolerance, max %.4g" % (splits, bad, mx)


@pytest.mark.parametrize("quant", ALL_FORMATS)
def test_prefill_short_chunks_share_a_workgroup_per_kv_head(oracle, quant):
    """Chunks short enough that all query heads of a KV head fit one workgroup's query columns (speculative
    steps, tails of prompts): 1 .. 32 tokens with 4 heads per KV head, up to 64 with the 8-wavefront workgroup,
    ragged rows, an empty prefix, and key splits on a long prefix - against the oracle."""
    for prefix, chunks, mc, splits in (([200, 64, 0, 333, 1000], [4, 32, 5, 1, 17], 32, None),
                                       ([64 * 9 + 3, 0, 129], [64, 33, 2], 64, None),
                                       ([64 * 200 + 7], [8], 8, 8), ([64 * 70, 5], [3, 2], 3, 4)):
        c = _prefill_case(sum(chunks) + len(prefix), prefix, chunks, quant)
        dev = syn.to_device(c, "cuda")
        out = fd.append_attention_prefill(dev["q_new"], dev["k_new"], dev["v_new"], dev["key_cache"], dev["value_cache"],
                                          dev["cache_k_scale"], dev["cache_v_scale"], dev["block_tables"],
                                          dev["seq_lens_decoder"], dev["cu_seqlens_q"], num_heads=32, max_chunk=mc,
                                          cache_quant_type=quant, num_splits=splits)
        torch.cuda.synchronize()
        want = oracle.append_attention_prefill(bits(c["q_new"]), bits(c["k_new"]), bits(c["v_new"]), np_of(c["key_cache"]),
                                               np_of(c["value_cache"]), np_of(c["cache_k_scale"]), np_of(c["cache_v_scale"]),
                                               np_of(c["block_tables"]), np_of(c["seq_lens_decoder"]), np_of(c["cu_seqlens_q"]),
                                               32, 8, 128, quant)
        ok, mx, bad = bf16_close(bits(out), want)
        assert ok, "prefix %r chunks %r splits %r: %d out of tolerance, max %.4g" % (prefix, chunks, splits, bad, mx)


def _run_prefill_vs_oracle(oracle, c, quant, max_chunk):
    dev = syn.to_device(c, "cuda")
    out = fd.append_attention_prefill(dev["q_new"], dev["k_new"], dev["v_new"], dev["key_cache"], dev["value_cache"],
                                      dev["cache_k_scale"], dev["cache_v_scale"], dev["block_tables"],
                                      dev["seq_lens_decoder"], dev["cu_seqlens_q"], num_heads=32, max_chunk=max_chunk,
                                      cache_quant_type=quant)
    want = oracle.append_attention_prefill(bits(c["q_new"]), bits(c["k_new"]), bits(c["v_new"]), np_of(c["key_cache"]),
                                           np_of(c["value_cache"]), np_of(c["cache_k_scale"]), np_of(c["cache_v_scale"]),
                                           np_of(c["block_tables"]), np_of(c["seq_lens_decoder"]), np_of(c["cu_seqlens_q"]),
                                           32, 8, 128, quant)
    ok, mx, bad = bf16_close(bits(out), want)
    assert ok, "%d out of tolerance, max %.4g" % (bad, mx)


@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_FP8])
@pytest.mark.parametrize("order", ["ascending", "descending"])
def test_prefill_scores_trending_along_the_prefix(oracle, quant, order):
    """Keys whose score grows (or falls) steadily from block to block: the running maximum is raised
    again and again (or never after the first tile), the case the deferred rescaling has to get right.
    Sharp softmax on top: q is scaled up."""
    c = _prefill_case(3, [1536, 700], [260, 90], quant)
    bt, kc = c["block_tables"], c["key_cache"]
    sgn = torch.where(torch.arange(128) % 3 == 0, -1, 1)
    top = 120 if quant == CACHE_INT8 else 0x6e  # int8 magnitude / e4m3 code of 240
    for b, n in enumerate(c["seq_lens_decoder"].tolist()):
        nb = (n + 63) // 64
        for j in range(nb):
            frac = (j + 1) / nb if order == "ascending" else (nb - j) / nb
            if quant == CACHE_INT8:
                mag = int(round(top * frac))
                row = (sgn * mag).to(torch.int8).view(torch.uint8)
            else:
                code = max(1, int(round(top * frac)))          # e4m3 codes are monotonic in magnitude
                row = torch.where(sgn < 0, code | 0x80, code).to(torch.uint8)
            kc[int(bt[b, j])] = row                              # every head, every token of the block
    c["q_new"] = (c["q_new"].float().abs() * sgn.repeat(32).float() * 1.5).to(torch.bfloat16)
    _run_prefill_vs_oracle(oracle, c, quant, 260)


@pytest.mark.parametrize("fill", [127, -127, 0])
def test_prefill_constant_value_bytes(oracle, fill):
    """V bytes all equal: the output is fill * v_scale whatever the weights are - exactly the case where the
    kernel's byte offset (it stages b + 128) must cancel against the weight sum."""
    c = _prefill_case(4, [2048, 65], [300, 20], CACHE_INT8)
    c["value_cache"][:] = torch.tensor(fill, dtype=torch.int8).view(torch.uint8)
    c["v_new"] = torch.zeros_like(c["v_new"])
    _run_prefill_vs_oracle(oracle, c, CACHE_INT8, 300)


def _moment_case(seed, prefix, chunk, kind, sk, sv, sq):
    """One sequence whose cached K and V are drawn with a given shape and size - Gaussian, uniform or +-1 ("binary":
    every code at full scale) times sk / sv - and quantised to int8 with max-abs / 127 per-channel scales; q ~ N(0, sq)."""
    c = syn.decode_case(batch=1, ctx=prefix, quant=CACHE_INT8, seed=seed, extra_blocks=2, direct_bytes=True)
    g = torch.Generator().manual_seed(seed)
    shp = c["key_cache"].shape
    draw = {"gauss": lambda: torch.randn(shp, generator=g),
            "uniform": lambda: torch.rand(shp, generator=g) * 2 - 1,
            "binary": lambda: torch.randint(0, 2, shp, generator=g).float() * 2 - 1}[kind]
    k, v = draw() * sk, draw() * sv
    ks, vs = k.abs().amax(dim=(0, 2)) / 127.0, v.abs().amax(dim=(0, 2)) / 127.0
    c["key_cache"] = torch.clamp(torch.round(k / ks[None, :, None, :]), -127, 127).to(torch.int8).view(torch.uint8)
    c["value_cache"] = torch.clamp(torch.round(v / vs[None, :, None, :]), -127, 127).to(torch.int8).view(torch.uint8)
    c["cache_k_scale"], c["cache_v_scale"] = ks.contiguous().float(), vs.contiguous().float()
    c["q_new"] = (torch.randn((chunk, 32 * 128), generator=g) * sq).to(torch.bfloat16)
    c["k_new"] = (torch.randn((chunk, 8 * 128), generator=g) * sk).to(torch.bfloat16)
    c["v_new"] = (torch.randn((chunk, 8 * 128), generator=g) * sv).to(torch.bfloat16)
    c["cu_seqlens_q"] = torch.tensor([0, chunk], dtype=torch.int32)
    return c


@pytest.mark.parametrize("kind,sk,sv,sq", [("gauss", 1, 1, 1), ("gauss", 2, 2, 1), ("gauss", 4, 4, 1), ("gauss", 8, 8, 0.25),
                                           ("uniform", 5, 8, 0.3), ("uniform", 5, 8, 1), ("binary", 2, 4, 0.5),
                                           ("binary", 4, 8, 0.5)])
def test_prefill_second_term_of_q_follows_the_tiles(oracle, kind, sk, sv, sq):
    """The kernel for head_dim 128 / block_size 64 takes q * k_scale as one fp16 term for the tiles of the steady state
    whose measured magnitudes (with the queries' norm) keep the rounding's effect below a tenth of the tolerance, and
    as two terms elsewhere.  Long prefixes (the steady state) on both sides of that test - score sizes x value sizes
    from 1 (quantised unit-scale activations: one term) to 70, distributions with every ratio of mean magnitude to
    root mean square; computed with one term everywhere, the cases (gauss 4 4 1), (gauss 8 8 .25), (uniform 5 8 1)
    and (binary 4 8 .5) leave the tolerance.  Every case against the oracle."""
    c = _moment_case(3, 4096, 256, kind, sk, sv, sq)
    _run_prefill_vs_oracle(oracle, c, CACHE_INT8, 256)


def _config5_rows():
    """Rows of configs[4] checked against the oracle: in both sequences the first and last query of every 64-query
    wavefront (= every edge of a 64-key tile of the chunk), their neighbours, and every 7th row: 782 of 4096."""
    rows = set()
    for base in (0, 2048):
        for i in range(0, 2048, 64):
            rows.update({base + i, base + i + 1, base + i + 62, base + i + 63})
        rows.update(range(base, base + 2048, 7))
    return np.array(sorted(rows), np.int32)


@pytest.mark.parametrize("quant,quantised", [(CACHE_INT8, True), (CACHE_INT8, False), (CACHE_INT8_DYNAMIC, True)])
def test_prefill_config5_shape_against_the_oracle(oracle, quant, quantised):
    """batch 2, 2048 new tokens on 8192 cached (int8 paged), causal: the full-size launch against the oracle on 782
    rows (every tile edge, both sequences).  quantised: the prefix is N(0,1) activations quantised with max-abs / 127
    scales, as the config states; otherwise uniform random bytes (a wider, flatter distribution of dequantised values)."""
    g = torch.Generator(device="cuda").manual_seed(0)
    c = syn.decode_case(batch=2, ctx=8192, seed=0, device="cuda", direct_bytes=not quantised, extra_blocks=8, quant=quant,
                        row_log2=(-5, 1))
    T = 2 * 2048
    c["q_new"] = torch.randn((T, 32 * 128), generator=g, device="cuda").to(torch.bfloat16)
    c["k_new"] = torch.randn((T, 8 * 128), generator=g, device="cuda").to(torch.bfloat16)
    c["v_new"] = torch.randn((T, 8 * 128), generator=g, device="cuda").to(torch.bfloat16)
    cu = torch.tensor([0, 2048, 4096], dtype=torch.int32, device="cuda")
    args = (c["q_new"], c["k_new"], c["v_new"], c["key_cache"], c["value_cache"], c["cache_k_scale"],
            c["cache_v_scale"], c["block_tables"], c["seq_lens_decoder"], cu)
    out = fd.append_attention_prefill(*args, num_heads=32, max_chunk=2048, cache_quant_type=quant)
    torch.cuda.synchronize()
    ids = _config5_rows()
    assert len(ids) >= 512
    want = oracle.append_attention_prefill(bits(c["q_new"]), bits(c["k_new"]), bits(c["v_new"]), np_of(c["key_cache"]),
                                           np_of(c["value_cache"]), np_of(c["cache_k_scale"]), np_of(c["cache_v_scale"]),
                                           np_of(c["block_tables"]), np_of(c["seq_lens_decoder"]), np_of(cu),
                                           32, 8, 128, quant, token_ids=ids)
    ok, mx, bad = bf16_close(bits(out)[ids], want[ids])
    assert ok, "%d of %d elements out of tolerance, max %.4g" % (bad, want[ids].size, mx)
    if quant == CACHE_INT8 and quantised:
        # an extra look at every row: the shape-agnostic GPU kernel agrees within twice the tolerance (each is within
        # it of the truth); not a substitute for the rows above
        ref = fd.append_attention_prefill(*args, num_heads=32, max_chunk=2048, impl="generic", cache_quant_type=quant)
        ok, mx, bad = bf16_close(bits(out), bits(ref), 4e-3, 2e-2)
        assert ok, "%d out of tolerance, max %.4g" % (bad, mx)


def _large_magnitude_case(seed, prefix, chunks, quant, vmax, kmax=5.0):
    """Uniform random cache bytes with scales that put the largest dequantised K at kmax and V at vmax (every channel /
    row between half of that and all of it): flat, wide value distributions far from quantised N(0,1)."""
    from fastdeploy_amd.ops import byte_format, is_dynamic
    c = syn.decode_case(batch=len(chunks), ctx=prefix, quant=quant, seed=seed, extra_blocks=3, direct_bytes=True)
    g = torch.Generator().manual_seed(seed + 7)
    top = 127.0 if byte_format(quant) == CACHE_INT8 else 448.0
    for name, mag in (("cache_k_scale", kmax), ("cache_v_scale", vmax)):
        c[name] = ((torch.rand(c[name].shape, generator=g) * 0.5 + 0.5) * (mag / top)).to(torch.float32)
    T = sum(chunks)
    c["q_new"] = torch.randn((T, 32 * 128), generator=g).to(torch.bfloat16)
    c["k_new"] = (torch.randn((T, 8 * 128), generator=g) * (kmax / 4.0)).to(torch.bfloat16)
    c["v_new"] = ((torch.rand((T, 8 * 128), generator=g) * 2 - 1) * vmax).to(torch.bfloat16)
    c["cu_seqlens_q"] = torch.tensor([0] + list(np.cumsum(chunks)), dtype=torch.int32)
    return c


@pytest.mark.parametrize("impl", ["auto", "tiles"])
@pytest.mark.parametrize("vmax", [5.0, 8.0])
@pytest.mark.parametrize("quant", ALL_FORMATS)
def test_prefill_large_magnitudes_short_and_long_rows(oracle, quant, vmax, impl):
    """The regime a single fp16 term for q * k_scale does not survive: uniform random int8 / fp8 bytes, dequantised K
    up to 5 and V up to 5 and 8 (the chunk's own V as wide), rows that see 1 .. 64 keys (prefixes of 0 .. 62 tokens
    under short chunks), and long rows in the same regime.  Both MFMA kernels (the hand-scheduled one of this shape and
    the one for any block size), every format, against the oracle.

    The softmax weights enter the P.V products in fp16 (11 significant bits), which leaves an output off by up to
    2^-11 * sum_j p_j |v_j|; tiles whose values may exceed 6 - by their scales, or by the chunk's own V - take the
    weights as two fp16 terms instead (22 bits).  Outputs that are small sums of large terms - a row of four keys
    with values near +-8 and weights near 1/2 - are what needs it.  The stated tolerance, at both magnitudes."""
    for seed, prefix, chunks in ((21, [0, 1, 5, 31, 62, 0, 17], [64, 63, 40, 33, 2, 1, 9]),
                                 (22, [700, 2500, 64], [100, 70, 256])):
        c = _large_magnitude_case(seed, prefix, chunks, quant, vmax)
        dev = syn.to_device(c, "cuda")
        out = fd.append_attention_prefill(dev["q_new"], dev["k_new"], dev["v_new"], dev["key_cache"], dev["value_cache"],
                                          dev["cache_k_scale"], dev["cache_v_scale"], dev["block_tables"],
                                          dev["seq_lens_decoder"], dev["cu_seqlens_q"], num_heads=32,
                                          max_chunk=max(chunks), cache_quant_type=quant, impl=impl)
        torch.cuda.synchronize()
        want = oracle.append_attention_prefill(bits(c["q_new"]), bits(c["k_new"]), bits(c["v_new"]), np_of(c["key_cache"]),
                                               np_of(c["value_cache"]), np_of(c["cache_k_scale"]), np_of(c["cache_v_scale"]),
                                               np_of(c["block_tables"]), np_of(c["seq_lens_decoder"]), np_of(c["cu_seqlens_q"]),
                                               32, 8, 128, quant)
        ok, mx, bad = bf16_close(bits(out), want)
        assert ok, "prefix %r chunks %r: %d of %d out of tolerance, max %.4g" % (prefix, chunks, bad, want.size, mx)


@pytest.mark.parametrize("quant", ALL_FORMATS)
def test_prefill_key_splits(oracle, quant):
    """Every query tile's keys shared by 2 .. 8 workgroups (partials + merge) against the oracle and against the
    unsplit kernel: one sequence's chunk on a long prefix (what the split is for), shares that end inside the
    prefix, start in the chunk or are empty, a ragged batch, and no prefix at all."""
    from fastdeploy_amd.ops import prefill_auto_splits
    assert prefill_auto_splits(1, 32, 512) >= 2 and prefill_auto_splits(64, 32, 2048) == 1
    for prefix, chunks, splits in (([64 * 70 + 17], [300], None), ([64 * 300], [130], 8), ([0, 4500, 64], [129, 5, 256], 4),
                                   ([0, 0], [40, 200], 3)):
        c = _prefill_case(len(chunks) * 7 + (splits or 0), prefix, chunks, quant)
        dev = syn.to_device(c, "cuda")
        args = (dev["q_new"], dev["k_new"], dev["v_new"], dev["key_cache"], dev["value_cache"], dev["cache_k_scale"],
                dev["cache_v_scale"], dev["block_tables"], dev["seq_lens_decoder"], dev["cu_seqlens_q"])
        out = fd.append_attention_prefill(*args, num_heads=32, max_chunk=max(chunks), cache_quant_type=quant, num_splits=splits)
        one = fd.append_attention_prefill(*args, num_heads=32, max_chunk=max(chunks), cache_quant_type=quant, num_splits=1)
        torch.cuda.synchronize()
        want = oracle.append_attention_prefill(bits(c["q_new"]), bits(c["k_new"]), bits(c["v_new"]), np_of(c["key_cache"]),
                                               np_of(c["value_cache"]), np_of(c["cache_k_scale"]), np_of(c["cache_v_scale"]),
                                               np_of(c["block_tables"]), np_of(c["seq_lens_decoder"]), np_of(c["cu_seqlens_q"]),
                                               32, 8, 128, quant)
        ok, mx, bad = bf16_close(bits(out), want)
        assert ok, "splits %r: %d out of tolerance, max %.4g" % (splits, bad, mx)
        ok, mx, bad = bf16_close(bits(one), want)
        assert ok, "unsplit: %d out of tolerance, max %.4g" % (bad, mx)


@pytest.mark.parametrize("hq,hkv,d,bs,quant", [
    (12, 1, 128, 64, CACHE_INT8),            # 12 query heads on one KV head: sets of 8 and 4, one token per group
    (6, 2, 96, 32, CACHE_FP8),               # 3 per KV head: groups of two tokens, 6 of the 8 rows in use
    (4, 4, 256, 128, CACHE_INT8_DYNAMIC),    # 1 per KV head: groups of eight tokens; a V row takes the whole wavefront
    (10, 2, 16, 8, CACHE_FP8_DYNAMIC),       # 5 per KV head: one token per group, 5 rows; 16 V rows per pass
    (8, 4, 20, 16, CACHE_INT8),              # head_dim not a multiple of 16: 4-byte K words
])
def test_prefill_shape_agnostic_kernel_shapes(oracle, hq, hkv, d, bs, quant):
    """The shape-agnostic prefill kernel at shapes that exercise its layout arithmetic: 1 .. 12 query heads per KV
    head (1, 2 or 8 tokens per workgroup, row sets partly empty), chunks that are not multiples of the token group,
    prefixes of zero, one and several 64-key groups, a prefix that ends inside a group."""
    prefix, chunks = [0, 1, 3 * bs + 5, 200, 64], [9, 1, 70, 13, 130]
    c = syn.decode_case(batch=len(chunks), ctx=prefix, quant=quant, seed=91, extra_blocks=20, hq=hq, hkv=hkv, d=d, bs=bs,
                        row_log2=(-3, 1))
    g = torch.Generator().manual_seed(92)
    T = sum(chunks)
    q = torch.randn((T, hq * d), generator=g).to(torch.bfloat16)
    k = torch.randn((T, hkv * d), generator=g).to(torch.bfloat16)
    v = torch.randn((T, hkv * d), generator=g).to(torch.bfloat16)
    cu = torch.tensor([0] + list(np.cumsum(chunks)), dtype=torch.int32)
    dev = syn.to_device(c, "cuda")
    out = fd.append_attention_prefill(q.cuda(), k.cuda(), v.cuda(), dev["key_cache"], dev["value_cache"],
                                      dev["cache_k_scale"], dev["cache_v_scale"], dev["block_tables"],
                                      dev["seq_lens_decoder"], cu.cuda(), num_heads=hq, max_chunk=max(chunks),
                                      cache_quant_type=quant, impl="generic")
    want = oracle.append_attention_prefill(bits(q), bits(k), bits(v), np_of(c["key_cache"]), np_of(c["value_cache"]),
                                           np_of(c["cache_k_scale"]), np_of(c["cache_v_scale"]), np_of(c["block_tables"]),
                                           np_of(c["seq_lens_decoder"]), np_of(cu), hq, hkv, d, quant)
    ok, mx, bad = bf16_close(bits(out), want)
    assert ok, "%d out of tolerance, max %.4g" % (bad, mx)


@pytest.mark.parametrize("hq,hkv,d,bs,quant,impl", [
    (8, 2, 64, 64, CACHE_INT8, "auto"),            # head_dim 64: half a 16-byte chunk row per thread
    (8, 2, 64, 16, CACHE_FP8_DYNAMIC, "auto"),     # a 32-key tile spans two blocks
    (6, 2, 256, 64, CACHE_FP8, "auto"),            # head_dim 256: two chunks per thread, 8 output blocks
    (4, 4, 256, 128, CACHE_INT8_DYNAMIC, "auto"),  # blocks of four tiles
    (8, 8, 256, 8, CACHE_INT8_BLOCK, "auto"),      # four blocks per tile, one scale per (block, head)
    (12, 4, 128, 16, CACHE_FP8_BLOCK, "auto"),     # head_dim 128 off the block size of the hand-scheduled kernel
    (10, 2, 128, 48, CACHE_INT8, "auto"),          # a block size that no tile boundary respects; 5 heads per KV head
    (32, 8, 128, 64, CACHE_INT8, "tiles"),         # the other MFMA kernel's own shape, on this one
    (32, 8, 128, 64, CACHE_FP8_DYNAMIC, "tiles"),
])
def test_prefill_mfma_kernel_of_the_other_shapes(oracle, hq, hkv, d, bs, quant, impl):
    """The MFMA append-attention kernel for head_dim 64 / 128 / 256 at any block size against the oracle: prefixes of
    zero, one key, whole and partial tiles and blocks, chunks of one token, of less than a wavefront's 32 queries, of
    several workgroups' worth, and chunks that end inside a tile."""
    prefix, chunks = [0, 1, 3 * bs + 5, 200, 64, 31, 700], [9, 1, 70, 13, 300, 33, 129]
    c = syn.decode_case(batch=len(chunks), ctx=prefix, quant=quant, seed=93, extra_blocks=20, hq=hq, hkv=hkv, d=d, bs=bs,
                        row_log2=(-3, 1))
    g = torch.Generator().manual_seed(94)
    T = sum(chunks)
    q = torch.randn((T, hq * d), generator=g).to(torch.bfloat16)
    k = torch.randn((T, hkv * d), generator=g).to(torch.bfloat16)
    v = torch.randn((T, hkv * d), generator=g).to(torch.bfloat16)
    cu = torch.tensor([0] + list(np.cumsum(chunks)), dtype=torch.int32)
    dev = syn.to_device(c, "cuda")
    out = fd.append_attention_prefill(q.cuda(), k.cuda(), v.cuda(), dev["key_cache"], dev["value_cache"],
                                      dev["cache_k_scale"], dev["cache_v_scale"], dev["block_tables"],
                                      dev["seq_lens_decoder"], cu.cuda(), num_heads=hq, max_chunk=max(chunks),
                                      cache_quant_type=quant, impl=impl, num_splits=1)
    want = oracle.append_attention_prefill(bits(q), bits(k), bits(v), np_of(c["key_cache"]), np_of(c["value_cache"]),
                                           np_of(c["cache_k_scale"]), np_of(c["cache_v_scale"]), np_of(c["block_tables"]),
                                           np_of(c["seq_lens_decoder"]), np_of(cu), hq, hkv, d, quant)
    ok, mx, bad = bf16_close(bits(out), want)
    assert ok, "%d out of tolerance, max %.4g" % (bad, mx)


def test_selector_random_shapes_against_the_oracle(oracle):
    """60 seeded random cases: 1 .. 8 query heads per KV head, 1 .. 3 KV heads, the six cache formats, lengths that
    favour zero and block boundaries, table rows wider than needed, top_k 1 .. 39: kept indices and counts exact."""
    rng = np.random.default_rng(11)
    for it in range(60):
        group, hkv, quant = int(rng.integers(1, 9)), int(rng.integers(1, 4)), int(rng.integers(1, 7))
        hq, batch = group * hkv, int(rng.integers(1, 6))
        lens = [[0, 64 * int(rng.integers(0, 60)), int(rng.integers(1, 6000))][int(rng.integers(0, 3))] for _ in range(batch)]
        if not any(lens):
            lens[0] = 130
        mb = max(lens) // 64 + 1 + int(rng.integers(0, 3))
        top_k = int(rng.integers(1, 40))
        c = syn.decode_case(batch=batch, ctx=lens, quant=quant, seed=3000 + it, extra_blocks=2, hq=hq, hkv=hkv,
                            max_blocks=mb, row_log2=(-4, 2), salient=0.05)
        what = "case %d: group %d hkv %d quant %d lens %r mb %d top_k %d" % (it, group, hkv, quant, lens, mb, top_k)
        dev = syn.to_device(c, "cuda")
        kept, cnt = fd.sqattn_select(dev["q"], dev["key_cache"], dev["cache_k_scale"], dev["block_tables"],
                                     dev["seq_lens_decoder"], num_heads=hq, top_k=top_k, cache_quant_type=quant)
        sc = oracle.sqattn_block_scores(bits(c["q"]), np_of(c["key_cache"]), np_of(c["cache_k_scale"]),
                                        np_of(c["block_tables"]), np_of(c["seq_lens_decoder"]), hq, hkv, 128, quant)
        wk, wc = oracle.topk_select(sc, np_of(c["seq_lens_decoder"]), 64, top_k)
        assert np.array_equal(np_of(cnt), wc) and np.array_equal(np_of(kept), wk), what


def test_prefill_random_shapes_against_the_oracle(oracle):
    """40 seeded random launches of the MFMA kernel: 1 / 2 / 3 / 4 / 8 query heads per KV head, 1 .. 3 KV heads, the
    six formats, 1 .. 4 sequences with short (packed), medium or long chunks on prefixes of zero, whole blocks or
    anything, key splits chosen by the library or forced to 1 .. 8."""
    rng = np.random.default_rng(12)
    for it in range(40):
        group, hkv, quant = [1, 2, 3, 4, 8][int(rng.integers(0, 5))], int(rng.integers(1, 4)), int(rng.integers(1, 7))
        hq, batch, kind = group * hkv, int(rng.integers(1, 5)), int(rng.integers(0, 3))
        hi = [max(2, 256 // group // 2), 400, 700][kind]
        chunks = [int(rng.integers(100 if kind == 2 else 1, hi)) for _ in range(batch)]
        prefix = [[0, 64 * int(rng.integers(0, 30)), int(rng.integers(1, 2500))][int(rng.integers(0, 3))] for _ in range(batch)]
        c = syn.decode_case(batch=batch, ctx=prefix, quant=quant, seed=4000 + it, extra_blocks=12, hq=hq, hkv=hkv,
                            row_log2=(-5, 1))
        g = torch.Generator().manual_seed(4000 + it)
        T = sum(chunks)
        q = torch.randn((T, hq * 128), generator=g).to(torch.bfloat16)
        k = torch.randn((T, hkv * 128), generator=g).to(torch.bfloat16)
        v = torch.randn((T, hkv * 128), generator=g).to(torch.bfloat16)
        cu = torch.tensor([0] + list(np.cumsum(chunks)), dtype=torch.int32)
        ns = [None, 1, 2, 3, 5, 8][int(rng.integers(0, 6))]
        what = "case %d: group %d hkv %d quant %d chunks %r prefix %r splits %r" % (it, group, hkv, quant, chunks, prefix, ns)
        dev = syn.to_device(c, "cuda")
        out = fd.append_attention_prefill(q.cuda(), k.cuda(), v.cuda(), dev["key_cache"], dev["value_cache"],
                                          dev["cache_k_scale"], dev["cache_v_scale"], dev["block_tables"],
                                          dev["seq_lens_decoder"], cu.cuda(), num_heads=hq, max_chunk=max(chunks),
                                          cache_quant_type=quant, num_splits=ns)
        want = oracle.append_attention_prefill(bits(q), bits(k), bits(v), np_of(c["key_cache"]), np_of(c["value_cache"]),
                                               np_of(c["cache_k_scale"]), np_of(c["cache_v_scale"]), np_of(c["block_tables"]),
                                               np_of(c["seq_lens_decoder"]), np_of(cu), hq, hkv, 128, quant)
        ok, mx, bad = bf16_close(bits(out), want)
        assert ok, "%s: %d out of tolerance, max %.4g" % (what, bad, mx)
