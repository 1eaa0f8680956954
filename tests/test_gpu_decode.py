"""Decode attention on the GPU against the CPU oracle (bf16 outputs within 2e-3 abs OR 1e-2 rel)."""
import numpy as np
import pytest
import torch

import fastdeploy_amd as fd
from conftest import bf16_close, bits, np_of
from fastdeploy_amd import synthetic as syn
from fastdeploy_amd.ops import (CACHE_FP8, CACHE_FP8_BLOCK, CACHE_FP8_DYNAMIC, CACHE_INT8, CACHE_INT8_BLOCK,
                                CACHE_INT8_DYNAMIC)

ALL_FORMATS = [CACHE_INT8, CACHE_FP8, CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC, CACHE_INT8_BLOCK, CACHE_FP8_BLOCK]

pytestmark = pytest.mark.gpu

ATOL, RTOL = 2e-3, 1e-2     # the path's stated tolerance for bf16 attention outputs


def oracle_decode(oracle, case, **kw):
    return oracle.decode_attention(bits(case["q"]), np_of(case["key_cache"]), np_of(case["value_cache"]),
                                   np_of(case["cache_k_scale"]), np_of(case["cache_v_scale"]),
                                   np_of(case["block_tables"]), np_of(case["seq_lens_decoder"]), case["hq"],
                                   case["hkv"], case["d"], case["quant"], **kw)


def gpu_decode(case, impl="auto", **kw):
    dev = syn.to_device(case, "cuda")
    out = fd.decode_attention(dev["q"], dev["key_cache"], dev["value_cache"], dev["cache_k_scale"], dev["cache_v_scale"],
                              dev["block_tables"], dev["seq_lens_decoder"], num_heads=case["hq"],
                              cache_quant_type=case["quant"], impl=impl, **kw)
    torch.cuda.synchronize()
    return bits(out)


def check(got, want, what=""):
    ok, mx, bad = bf16_close(got, want, ATOL, RTOL)
    assert ok, "%s: %d elements out of tolerance, max abs diff %.4g" % (what, bad, mx)


@pytest.mark.parametrize("impl", ["generic", "tiles", "auto"])
@pytest.mark.parametrize("quant", ALL_FORMATS)
def test_decode_config1(oracle, impl, quant):
    """batch 4, 32/8 heads, head_dim 128, ctx 1024, 64 physical blocks in a random permutation."""
    for seed in range(3):
        case = syn.decode_case(batch=4, ctx=1024, pool_blocks=64, quant=quant, seed=seed)
        check(gpu_decode(case, impl), oracle_decode(oracle, case), "cfg1 seed %d" % seed)


@pytest.mark.parametrize("impl", ["generic", "tiles", "auto"])
@pytest.mark.parametrize("quant", ALL_FORMATS)
def test_decode_ragged_and_edge_lengths(oracle, impl, quant):
    lens = [1, 2, 63, 64, 65, 127, 128, 129, 700, 0, 1000, 31]
    case = syn.decode_case(batch=len(lens), ctx=lens, quant=quant, seed=5, extra_blocks=7, max_blocks=20)
    got, want = gpu_decode(case, impl), oracle_decode(oracle, case)
    check(got, want, "ragged")
    assert not got.reshape(len(lens), -1)[9].any()          # kv_len 0 -> zeros


@pytest.mark.parametrize("impl", ["generic", "tiles", "auto"])
def test_decode_peaked_and_flat_softmax(oracle, impl):
    """A query aligned with one key (one dominant weight) and constant keys (uniform weights)."""
    case = syn.decode_case(batch=2, ctx=900, seed=6)
    q = case["q"].view(2, 32, 128)
    blk = int(case["block_tables"][0, 3])
    krow = case["key_cache"][blk, :, 17, :].view(torch.int8).float() * case["cache_k_scale"]
    q[0] = (krow * 2.0).repeat_interleave(4, 0).to(torch.bfloat16)
    case["key_cache"][case["block_tables"][1, :15].long()] = 5
    check(gpu_decode(case, impl), oracle_decode(oracle, case), "peaked/flat")


@pytest.mark.parametrize("impl", ["generic", "tiles", "auto"])
def test_decode_this_time_adds_to_kv_len(oracle, impl):
    case = syn.decode_case(batch=3, ctx=[100, 64, 257], seed=7)
    dev = syn.to_device(case, "cuda")
    dec = dev["seq_lens_decoder"] - 1
    one = torch.ones_like(dec)
    out = fd.decode_attention(dev["q"], dev["key_cache"], dev["value_cache"], dev["cache_k_scale"], dev["cache_v_scale"],
                              dev["block_tables"], dec, one, num_heads=32, impl=impl)
    check(bits(out), oracle_decode(oracle, case), "this_time")


@pytest.mark.parametrize("impl", ["generic", "tiles", "auto"])
@pytest.mark.parametrize("quant", [CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC])
def test_decode_dynamic_formats_with_widely_different_row_scales(oracle, impl, quant):
    """One scale per stored row; the rows of one block differ in scale by up to 2^16 for V and 2^12 for K, and the
    slots past a sequence's end hold NaN scales.  The dequantised magnitudes stay at the scale the absolute part of
    the tolerance is meant for (|V| up to about 8)."""
    case = syn.decode_case(batch=5, ctx=[1, 64, 200, 1000, 2500], quant=quant, seed=12, extra_blocks=3)
    g = torch.Generator().manual_seed(5)
    for name, lo, hi in (("cache_k_scale", -6, 0), ("cache_v_scale", -12, -2)):
        sc = case[name]
        mult = torch.exp2(torch.randint(lo, hi + 1, sc.shape, generator=g).float())
        case[name] = torch.where(sc.isnan(), sc, sc * mult)
    check(gpu_decode(case, impl), oracle_decode(oracle, case), "row scales")


@pytest.mark.parametrize("impl", ["tiles", "auto"])
@pytest.mark.parametrize("quant", [CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC])
def test_decode_dynamic_formats_with_vanishing_units(oracle, impl, quant):
    """A query aligned with one key so strongly that the weights of whole blocks fall to the bottom of the fp32
    range (where the reciprocal of a block's heaviest weight x scale product overflows): those blocks must drop
    out, not poison the row."""
    # logit gaps from ~30 to ~500 (and 4 x to 16 x smaller for the heads whose key row has a smaller scale): for
    # some of them the heaviest weight of a block lands in the band just above the smallest fp32 numbers
    gains = [3.0, 5.0, 7.0, 8.5, 10.0, 12.0, 16.0, 24.0, 34.0, 48.0]
    case = syn.decode_case(batch=len(gains), ctx=64 * 12 + 5, quant=quant, seed=21, row_log2=(-2, 0))
    q = case["q"].view(len(gains), 32, 128)
    for b, gain in enumerate(gains):
        blk = int(case["block_tables"][b, 3 + b % 5])
        k8 = case["key_cache"][blk, :, 7 + b, :]
        kf = (k8.view(torch.int8) if quant == CACHE_INT8_DYNAMIC else k8.view(torch.float8_e4m3fn)).float()
        krow = kf * case["cache_k_scale"][blk, :, 7 + b][:, None]
        q[b] = (krow * gain).repeat_interleave(4, 0).to(torch.bfloat16)
    got, want = gpu_decode(case, impl), oracle_decode(oracle, case)
    assert np.isfinite(oracle.bf16_to_f32(got)).all()
    check(got, want, "vanishing units")


@pytest.mark.parametrize("quant", ALL_FORMATS)
@pytest.mark.parametrize("group", [1, 2, 3, 5, 7, 8])
def test_decode_other_group_sizes_on_the_mfma_kernel(oracle, group, quant):
    """1 .. 8 query heads per KV head (head_dim 128, block 64) run on the MFMA kernel: groups up to 4 in one set of
    MFMA rows with the unused head rows zero, 5 .. 8 in two sets sharing every K / V operand.  Ragged lengths, a
    multi-chunk launch (partials + merge kernel) and a sparse call, each against the oracle."""
    hkv = 4
    hq = group * hkv
    assert fd.decode_uses_mfma(hq, hkv, 128, 64, quant)
    lens = [1, 63, 64, 65, 700, 0, 1500, 31]
    case = syn.decode_case(batch=len(lens), ctx=lens, quant=quant, seed=30 + group, extra_blocks=3, hq=hq, hkv=hkv)
    got, want = gpu_decode(case), oracle_decode(oracle, case)
    check(got, want, "group %d ragged" % group)
    assert not got.reshape(len(lens), -1)[5].any()
    # few long sequences: several chunks per list
    case = syn.decode_case(batch=2, ctx=[64 * 150 - 3, 64 * 90], quant=quant, seed=40 + group, hq=hq, hkv=hkv,
                           direct_bytes=True)
    from fastdeploy_amd import _lib
    assert _lib.lib().fdattn_decode_chunks_per_sequence(2, hkv, 150) > 1
    check(gpu_decode(case), oracle_decode(oracle, case), "group %d chunks" % group)
    # sparse
    rng = np.random.default_rng(group)
    kept = np.full((2, hkv, 9), -1, np.int32)
    cnt = np.zeros((2, hkv), np.int32)
    for b, nb in enumerate((150, 90)):
        for h in range(hkv):
            k = int(rng.integers(1, 10))
            kept[b, h, :k] = np.sort(rng.choice(nb, k, replace=False))
            cnt[b, h] = k
    dev = syn.to_device(case, "cuda")
    out = fd.decode_attention_sparse(dev["q"], dev["key_cache"], dev["value_cache"], dev["cache_k_scale"],
                                     dev["cache_v_scale"], dev["block_tables"], dev["seq_lens_decoder"],
                                     kept_blocks=torch.from_numpy(kept).cuda(), kept_counts=torch.from_numpy(cnt).cuda(),
                                     num_heads=hq, cache_quant_type=quant)
    check(bits(out), oracle_decode(oracle, case, kept_blocks=kept, kept_counts=cnt), "group %d sparse" % group)


def test_decode_random_shapes_against_the_oracle(oracle):
    """40 seeded random cases: batch 1 .. 9, 1 .. 8 query heads per KV head, 1 .. 4 KV heads, any of the six cache
    formats, lengths that favour block boundaries and zero, dense or sparse lists - the MFMA kernel against the oracle."""
    rng = np.random.default_rng(2024)
    for it in range(40):
        group, hkv = int(rng.integers(1, 9)), int(rng.integers(1, 5))
        hq, quant = group * hkv, ALL_FORMATS[int(rng.integers(0, len(ALL_FORMATS)))]
        batch = int(rng.integers(1, 10))
        lens = []
        for _ in range(batch):
            kind = int(rng.integers(0, 5))
            base = int(rng.integers(0, 40)) * 64
            lens.append([0, base, base + 1, base + 63, int(rng.integers(1, 2600))][kind])
        if not any(lens):
            lens[0] = 65
        mb = max(max(lens) // 64 + 1, 1) + int(rng.integers(0, 3))
        case = syn.decode_case(batch=batch, ctx=lens, quant=quant, seed=1000 + it, extra_blocks=2, hq=hq, hkv=hkv,
                               max_blocks=mb, row_log2=(-4, 0))
        assert fd.decode_uses_mfma(hq, hkv, 128, 64, quant)
        what = "case %d: group %d hkv %d quant %d lens %r" % (it, group, hkv, quant, lens)
        if it % 3 == 2:   # sparse: random ascending subsets, some empty
            mk = int(rng.integers(1, 8))
            kept = np.full((batch, hkv, mk), -1, np.int32)
            cnt = np.zeros((batch, hkv), np.int32)
            for b in range(batch):
                nb = (lens[b] + 63) // 64
                for h in range(hkv):
                    k = int(rng.integers(0, min(mk, nb) + 1))
                    kept[b, h, :k] = np.sort(rng.choice(nb, k, replace=False)) if k else []
                    cnt[b, h] = k
            dev = syn.to_device(case, "cuda")
            out = fd.decode_attention_sparse(dev["q"], dev["key_cache"], dev["value_cache"], dev["cache_k_scale"],
                                             dev["cache_v_scale"], dev["block_tables"], dev["seq_lens_decoder"],
                                             kept_blocks=torch.from_numpy(kept).cuda(), kept_counts=torch.from_numpy(cnt).cuda(),
                                             num_heads=hq, cache_quant_type=quant)
            check(bits(out), oracle_decode(oracle, case, kept_blocks=kept, kept_counts=cnt), what + " sparse")
        else:
            check(gpu_decode(case), oracle_decode(oracle, case), what)


def test_decode_generic_other_shapes(oracle):
    """Shapes outside the MFMA kernel: head_dim 64, group 2, block_size 16."""
    case = syn.decode_case(batch=3, ctx=[50, 200, 333], seed=8, hq=8, hkv=4, d=64, bs=16)
    got = gpu_decode(case)
    want = oracle.decode_attention(bits(case["q"]), np_of(case["key_cache"]), np_of(case["value_cache"]),
                                   np_of(case["cache_k_scale"]), np_of(case["cache_v_scale"]),
                                   np_of(case["block_tables"]), np_of(case["seq_lens_decoder"]), 8, 4, 64, CACHE_INT8)
    check(got, want, "d64 g2 bs16")


@pytest.mark.parametrize("hq,hkv,d,bs,quant", [
    (12, 1, 128, 64, CACHE_INT8),            # 12 query heads on one KV head: two sets of heads per KV head
    (40, 2, 96, 32, CACHE_FP8),              # 20 per KV head (sets of 8, 8, 4); 24 lanes per V row, 16 lanes idle
    (6, 2, 256, 128, CACHE_INT8_DYNAMIC),    # a V row takes the whole wavefront; blocks of two 64-token groups
    (5, 5, 16, 8, CACHE_FP8_DYNAMIC),        # 16 V rows per pass; blocks smaller than a token group
    (16, 2, 20, 64, CACHE_INT8),             # head_dim not a multiple of 16: 4-byte K words
])
@pytest.mark.parametrize("impl", ["generic", "auto"])
def test_decode_shape_agnostic_kernel_shapes(oracle, impl, hq, hkv, d, bs, quant):
    """The shape-agnostic kernel at shapes that exercise its layout arithmetic: more query heads per KV head than a
    workgroup serves, head sizes whose V rows take 5 .. 64 lanes, blocks above and below 64 tokens; dense and sparse.
    ("auto" hands the first and the third shape to the fp16-MFMA kernel.)"""
    lens = [0, 1, bs - 1, bs, bs + 1, 5 * bs + 3, 700]
    case = syn.decode_case(batch=len(lens), ctx=lens, seed=77, hq=hq, hkv=hkv, d=d, bs=bs, quant=quant, row_log2=(-3, 1))
    assert not fd.decode_uses_mfma(hq, hkv, d, bs, quant)
    want = oracle.decode_attention(bits(case["q"]), np_of(case["key_cache"]), np_of(case["value_cache"]),
                                   np_of(case["cache_k_scale"]), np_of(case["cache_v_scale"]),
                                   np_of(case["block_tables"]), np_of(case["seq_lens_decoder"]), hq, hkv, d, quant)
    check(gpu_decode(case, impl), want, "dense")
    rng = np.random.default_rng(5)
    mk = 4
    kept = np.full((len(lens), hkv, mk), -1, np.int32)
    cnt = np.zeros((len(lens), hkv), np.int32)
    for b, n in enumerate(lens):
        nb = (n + bs - 1) // bs
        for h in range(hkv):
            k = int(rng.integers(0, min(mk, nb) + 1))
            kept[b, h, :k] = np.sort(rng.choice(nb, k, replace=False)) if k else []
            cnt[b, h] = k
    dev = syn.to_device(case, "cuda")
    out = fd.decode_attention_sparse(dev["q"], dev["key_cache"], dev["value_cache"], dev["cache_k_scale"],
                                     dev["cache_v_scale"], dev["block_tables"], dev["seq_lens_decoder"],
                                     kept_blocks=torch.from_numpy(kept).cuda(), kept_counts=torch.from_numpy(cnt).cuda(),
                                     num_heads=hq, cache_quant_type=quant, impl=impl)
    want = oracle.decode_attention(bits(case["q"]), np_of(case["key_cache"]), np_of(case["value_cache"]),
                                   np_of(case["cache_k_scale"]), np_of(case["cache_v_scale"]),
                                   np_of(case["block_tables"]), np_of(case["seq_lens_decoder"]), hq, hkv, d, quant,
                                   kept_blocks=kept, kept_counts=cnt)
    check(bits(out), want, "sparse")


def _random_kept(rng, lens, hkv, bs, mk):
    kept = np.full((len(lens), hkv, mk), -1, np.int32)
    cnt = np.zeros((len(lens), hkv), np.int32)
    for b, n in enumerate(lens):
        nb = (n + bs - 1) // bs
        for h in range(hkv):
            k = int(rng.integers(0, min(mk, nb) + 1))
            kept[b, h, :k] = np.sort(rng.choice(nb, k, replace=False)) if k else []
            cnt[b, h] = k
    return kept, cnt


@pytest.mark.parametrize("quant", ALL_FORMATS)
@pytest.mark.parametrize("hq,hkv,d,bs", [
    (32, 8, 128, 64),    # the int8-MFMA kernel's own shape, on this kernel by name
    (8, 4, 64, 16),      # tiles of two blocks
    (6, 2, 256, 128),    # blocks of four tiles
    (40, 2, 64, 32),     # 20 query heads per KV head: a set of 16 and a set of 4 on workgroups of their own; a tile is a block
    (16, 2, 128, 48),    # a block size that is no power of two: tiles straddle blocks at changing offsets
    (5, 5, 64, 8),       # one query head per KV head; tiles of four blocks
    (32, 8, 256, 64),
])
def test_decode_mfma_kernel_of_the_other_shapes(oracle, hq, hkv, d, bs, quant):
    """The fp16-MFMA decode kernel (head_dim 64 / 128 / 256, any block size, up to 64 query heads per KV head) against
    the oracle: lengths around tile and block edges and zero, dense and over random lists of kept blocks, every
    format; and it is what the dispatch picks where the int8-MFMA kernel does not apply."""
    lens = [0, 1, bs - 1, bs, bs + 1, 5 * bs + 3, 700, 33, 2049]
    case = syn.decode_case(batch=len(lens), ctx=lens, seed=77 + d + bs, hq=hq, hkv=hkv, d=d, bs=bs, quant=quant,
                           row_log2=(-3, 1))
    want = oracle_decode(oracle, case)
    got = gpu_decode(case, "tiles")
    check(got, want, "dense")
    assert not got.reshape(len(lens), -1)[0].any()          # kv_len 0 -> zeros
    if not fd.decode_uses_mfma(hq, hkv, d, bs, quant):
        assert np.array_equal(gpu_decode(case, "auto"), got)
    kept, cnt = _random_kept(np.random.default_rng(5), lens, hkv, bs, 5)
    kept[6, 0, :2] = [0, (700 - 1) // bs]                   # includes the partial last block
    kept[6, 0, 2:] = -1
    cnt[6, 0] = 2
    dev = syn.to_device(case, "cuda")
    out = fd.decode_attention_sparse(dev["q"], dev["key_cache"], dev["value_cache"], dev["cache_k_scale"],
                                     dev["cache_v_scale"], dev["block_tables"], dev["seq_lens_decoder"],
                                     kept_blocks=torch.from_numpy(kept).cuda(), kept_counts=torch.from_numpy(cnt).cuda(),
                                     num_heads=hq, cache_quant_type=quant, impl="tiles")
    check(bits(out), oracle_decode(oracle, case, kept_blocks=kept, kept_counts=cnt), "sparse")


@pytest.mark.parametrize("d,batch", [(64, 90), (128, 60), (256, 30)])
def test_decode_mfma_kernel_of_the_other_shapes_unsplit(oracle, d, batch):
    """Batches that fill the GPU without key splits: the kernel then writes the output itself, no merge launch.
    Table entries inside a sequence that name no block (-1) are outside the oracle's contract; the kernel drops their
    keys as the vector-ALU kernel does, and the two are compared with each other there."""
    rng = np.random.default_rng(d)
    lens = [int(x) for x in rng.integers(1, 400, batch)]
    lens[3] = 0
    case = syn.decode_case(batch=batch, ctx=lens, seed=d, hq=32, hkv=8, d=d, bs=64, quant=CACHE_FP8, max_blocks=8)
    got = gpu_decode(case, "tiles")
    check(got, oracle_decode(oracle, case), "unsplit d %d" % d)
    assert not got.reshape(batch, -1)[3].any()
    holes = [b for b in range(batch) if lens[b] > 130][:2]
    case["block_tables"][holes[0], 1] = -1
    case["block_tables"][holes[1], 0] = -1
    check(gpu_decode(case, "tiles"), gpu_decode(case, "generic"), "entries that name no block, d %d" % d)


@pytest.mark.parametrize("d,lens", [(64, [9000]), (128, [20000]), (128, [11000, 3]), (256, [13001])])
def test_decode_mfma_kernel_of_the_other_shapes_few_sequences(oracle, d, lens):
    """A batch of one or two long sequences splits its keys over more workgroups than the 16 partial results per row
    that every workspace holds (up to 64, in the workspace the library asks for at such a batch); with a workspace of
    only the smaller size the launch uses the splits that fit."""
    hq, hkv, bs = 8, 2, 64
    case = syn.decode_case(batch=len(lens), ctx=lens, seed=d + len(lens), hq=hq, hkv=hkv, d=d, bs=bs, quant=CACHE_INT8)
    want = oracle_decode(oracle, case)
    check(gpu_decode(case, "tiles"), want, "few sequences d %d" % d)
    nblk = case["block_tables"].shape[1]
    full = fd._lib.lib().fdattn_decode_workspace_bytes(len(lens), hq, hkv, d, nblk)
    small = len(lens) * hq * 16 * (d + 2) * 4
    assert full >= 2 * small
    dev = syn.to_device(case, "cuda")
    out = fd.decode_attention(dev["q"], dev["key_cache"], dev["value_cache"], dev["cache_k_scale"], dev["cache_v_scale"],
                              dev["block_tables"], dev["seq_lens_decoder"], num_heads=hq, cache_quant_type=CACHE_INT8,
                              impl="tiles", workspace=torch.empty(small, dtype=torch.uint8, device="cuda"))
    check(bits(out), want, "few sequences, workspace of 16 splits, d %d" % d)


@pytest.mark.parametrize("impl", ["generic", "tiles", "auto"])
@pytest.mark.parametrize("quant", ALL_FORMATS)
def test_sparse_decode(oracle, impl, quant):
    case = syn.decode_case(batch=3, ctx=[2000, 1500, 64 * 40 + 5], quant=quant, seed=9)
    rng = np.random.default_rng(1)
    kept = np.full((3, 8, 12), -1, np.int32)
    cnt = np.zeros((3, 8), np.int32)
    for b in range(3):
        nb = (int(case["seq_lens_decoder"][b]) + 63) // 64
        for h in range(8):
            k = int(rng.integers(1, 13))
            kept[b, h, :k] = np.sort(rng.choice(nb, k, replace=False))
            cnt[b, h] = k
    kept[2, 0, :3] = [0, 39, 40]      # includes the partial last block
    kept[2, 0, 3:] = -1
    cnt[2, 0] = 3
    dev = syn.to_device(case, "cuda")
    out = fd.decode_attention_sparse(dev["q"], dev["key_cache"], dev["value_cache"], dev["cache_k_scale"],
                                     dev["cache_v_scale"], dev["block_tables"], dev["seq_lens_decoder"],
                                     kept_blocks=torch.from_numpy(kept).cuda(), kept_counts=torch.from_numpy(cnt).cuda(),
                                     num_heads=32, cache_quant_type=quant, impl=impl)
    check(bits(out), oracle_decode(oracle, case, kept_blocks=kept, kept_counts=cnt), "sparse")


@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_FP8_DYNAMIC])
def test_per_token_block_lists_for_the_tokens_of_one_sequence(oracle, quant):
    """Block lists per draft TOKEN of a speculative step (the one-call step keeps one list per row): the selector and
    the sparse decode take every token as a row of its own whose table row repeats the sequence's - rows may name the
    same blocks, as sequences with a shared prefix do - and whose length ends at that token.  Four tokens per
    sequence, the last of them across a block boundary; lists and outputs against the oracle's on the same rows."""
    T, top_k = 4, 6
    # (dynamic format: the largest rows at unit scale, where the absolute part of the output tolerance applies)
    base = syn.decode_case(batch=3, ctx=[64 * 30 + 2, 64 * 17, 900], quant=quant, seed=21, salient=0.1, row_log2=(-6, 0))
    lens = np_of(base["seq_lens_decoder"])
    rows = [(b, int(lens[b]) - T + t + 1) for b in range(3) for t in range(T)]
    g = torch.Generator().manual_seed(5)
    case = dict(base)
    case["q"] = torch.randn((len(rows), 32 * 128), generator=g).to(torch.bfloat16)
    case["block_tables"] = base["block_tables"][[b for b, _ in rows]].contiguous()
    case["seq_lens_decoder"] = torch.tensor([n for _, n in rows], dtype=torch.int32)
    dev = syn.to_device(case, "cuda")
    kept, cnt = fd.sqattn_select(dev["q"], dev["key_cache"], dev["cache_k_scale"], dev["block_tables"],
                                 dev["seq_lens_decoder"], num_heads=32, top_k=top_k, cache_quant_type=quant)
    s = oracle.sqattn_block_scores(bits(case["q"]), np_of(case["key_cache"]), np_of(case["cache_k_scale"]),
                                   np_of(case["block_tables"]), np_of(case["seq_lens_decoder"]), 32, 8, 128, quant)
    okept, ocnt = oracle.topk_select(s, np_of(case["seq_lens_decoder"]), 64, top_k)
    assert np.array_equal(np_of(cnt), ocnt) and np.array_equal(np_of(kept), okept)
    assert any(not np.array_equal(okept[i], okept[i + 1]) for i in range(T - 1))   # the tokens' lists do differ
    out = fd.decode_attention_sparse(dev["q"], dev["key_cache"], dev["value_cache"], dev["cache_k_scale"],
                                     dev["cache_v_scale"], dev["block_tables"], dev["seq_lens_decoder"],
                                     kept_blocks=kept, kept_counts=cnt, num_heads=32, cache_quant_type=quant)
    check(bits(out), oracle_decode(oracle, case, kept_blocks=okept, kept_counts=ocnt), "per-token lists")


def test_splitkv_combine_entry_point(oracle):
    g = torch.Generator().manual_seed(0)
    po = torch.randn((37, 9, 128), generator=g)
    pm = torch.randn((37, 9), generator=g) * 4
    pl = torch.rand((37, 9), generator=g) * 50 + 1
    pm[3, 4:] = -float("inf")
    ns = torch.randint(1, 10, (37,), generator=g, dtype=torch.int32)
    for n in (None, ns):
        out = fd.splitkv_combine(po.cuda(), pm.cuda(), pl.cuda(), None if n is None else n.cuda())
        want = oracle.splitkv_combine(po.numpy(), pm.numpy(), pl.numpy(), None if n is None else n.numpy())
        check(bits(out), want, "combine")


def test_decode_rejects_bad_arguments():
    case = syn.to_device(syn.decode_case(batch=2, ctx=64), "cuda")
    with pytest.raises(ValueError):
        fd.decode_attention(case["q"][:, :-1].contiguous(), case["key_cache"], case["value_cache"], case["cache_k_scale"],
                            case["cache_v_scale"], case["block_tables"], case["seq_lens_decoder"], num_heads=32)
    with pytest.raises(ValueError):
        fd.decode_attention(case["q"], case["key_cache"], case["value_cache"], case["cache_k_scale"],
                            case["cache_v_scale"], case["block_tables"], case["seq_lens_decoder"], num_heads=32,
                            workspace=torch.empty(16, dtype=torch.uint8, device="cuda"))


def test_workspace_is_reusable_across_calls_and_shapes(oracle):
    """One workspace serves calls of different batch sizes, lengths and cache types back to back."""
    ws = fd.decode_workspace(12, 32, 8, 128, 64, "cuda")
    ws.fill_(0xAB)   # the kernels must not rely on its contents
    cases = [syn.decode_case(batch=12, ctx=[1, 2, 63, 64, 65, 127, 128, 129, 700, 0, 1000, 31], seed=5, max_blocks=20),
             syn.decode_case(batch=3, ctx=[4000, 64 * 17, 5], seed=6, max_blocks=64),
             syn.decode_case(batch=12, ctx=2048, seed=7, max_blocks=40, quant=CACHE_FP8)]
    for rep in range(3):
        for case in cases:
            got = gpu_decode(case, workspace=ws)
            check(got, oracle_decode(oracle, case), "reuse rep %d" % rep)


@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_FP8_DYNAMIC])
def test_decode_lists_of_up_to_256_blocks_in_one_chunk(oracle, quant):
    """64 sequences (512 (sequence, KV head) pairs: one chunk per list) of 8.2k to 16.4k tokens: lists of 129 .. 256
    blocks, the third and fourth entries per lane of the int8-MFMA kernel's unit table, go through one workgroup each
    with no partial and no merge launch; 257 blocks make two chunks.  The tables draw from a pool of 3,000 blocks, so
    sequences share blocks (as after a fork); against the oracle."""
    from fastdeploy_amd import _lib
    assert _lib.lib().fdattn_decode_chunks_per_sequence(64, 8, 256) == 1
    assert _lib.lib().fdattn_decode_chunks_per_sequence(64, 8, 257) == 2
    g = torch.Generator().manual_seed(11)
    base = syn.decode_case(batch=64, ctx=64, pool_blocks=3000, seed=3, quant=quant, direct_bytes=True, max_blocks=257)
    lens = torch.randint(64 * 128 + 1, 64 * 256 + 1, (64,), generator=g)
    lens[0], lens[1], lens[2] = 64 * 256, 64 * 128 + 1, 64 * 192 + 1   # the table's last entry, its 129th, its 193rd
    case = dict(base)
    case["seq_lens_decoder"] = lens.to(torch.int32)
    case["block_tables"] = torch.randint(0, 3000, (64, 257), generator=g).to(torch.int32)
    for mb in (256, 257):
        c = dict(case)
        c["block_tables"] = case["block_tables"][:, :mb].contiguous()
        check(gpu_decode(c), oracle_decode(oracle, c), "tables of %d entries" % mb)


@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_INT8_DYNAMIC])
def test_decode_config2_full_size(oracle, quant):
    """batch 64, ctx U[3584, 4608], int8 KV (per-channel scales, and one scale per stored row), block tables a random permutation over a 6000-block pool:
    the full-size launch against the oracle, plus two size-independent properties: the result does not
    depend on where the blocks sit in the pool, and it is the same whatever the split-KV chunking is
    (dense call == sparse call that keeps every block)."""
    g = torch.Generator().manual_seed(0)
    lens = torch.randint(3584, 4609, (64,), generator=g).tolist()
    case = syn.decode_case(batch=64, ctx=lens, pool_blocks=6000, seed=1, device="cuda", max_blocks=72, quant=quant)
    out = fd.decode_attention(case["q"], case["key_cache"], case["value_cache"], case["cache_k_scale"],
                              case["cache_v_scale"], case["block_tables"], case["seq_lens_decoder"], num_heads=32,
                              cache_quant_type=quant)
    torch.cuda.synchronize()
    cpu = syn.to_device(case, "cpu")
    check(bits(out), oracle_decode(oracle, cpu), "cfg2")
    # move every block somewhere else in the pool: bit-identical output
    perm = torch.randperm(6000, generator=torch.Generator().manual_seed(5)).cuda()
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(6000, device="cuda")
    bt2 = torch.where(case["block_tables"] >= 0, inv[case["block_tables"].clamp(min=0).long()].to(torch.int32), -1)
    dyn = quant == CACHE_INT8_DYNAMIC   # the scale caches move with their blocks
    ks2 = case["cache_k_scale"][perm].contiguous() if dyn else case["cache_k_scale"]
    vs2 = case["cache_v_scale"][perm].contiguous() if dyn else case["cache_v_scale"]
    out2 = fd.decode_attention(case["q"], case["key_cache"][perm], case["value_cache"][perm], ks2, vs2,
                               bt2.contiguous(), case["seq_lens_decoder"], num_heads=32, cache_quant_type=quant)
    assert torch.equal(out, out2)
    # keep-everything sparse call: same blocks, different chunk geometry -> same within a bf16 ulp of rounding noise
    nb = torch.tensor([(n + 63) // 64 for n in lens], dtype=torch.int32, device="cuda")
    kept = torch.arange(72, dtype=torch.int32, device="cuda")[None, None, :].repeat(64, 8, 1)
    kept = torch.where(kept < nb[:, None, None], kept, -1).contiguous()
    cnt = nb[:, None].repeat(1, 8).contiguous()
    out3 = fd.decode_attention_sparse(case["q"], case["key_cache"], case["value_cache"], case["cache_k_scale"],
                                      case["cache_v_scale"], case["block_tables"], case["seq_lens_decoder"],
                                      kept_blocks=kept, kept_counts=cnt, num_heads=32, cache_quant_type=quant)
    check(bits(out3), bits(out), "dense vs keep-all sparse")


@pytest.mark.parametrize("quant", ALL_FORMATS)
def test_decode_launch_shapes(oracle, quant):
    """The chunking follows the launch size (as few chunks per block list as fill the GPU's workgroup slots):
    long lists in a small batch are cut into several chunks of more than 64 units (second unit-table entry
    of a lane, partials, merge kernel), a single sequence into many short chunks, a large batch into one
    chunk per list.  Every shape against the oracle."""
    from fastdeploy_amd import _lib
    for batch, ctx, cpp in ((16, [20000 - 37 * i for i in range(16)], 4), (1, 64 * 300 - 11, 60), (70, 64 * 9 + 1, 1)):
        mb = (max(ctx) if isinstance(ctx, list) else ctx) // 64 + 1
        assert _lib.lib().fdattn_decode_chunks_per_sequence(batch, 8, mb) == cpp
        case = syn.decode_case(batch=batch, ctx=ctx, quant=quant, seed=batch, device="cuda", max_blocks=mb)
        out = fd.decode_attention(case["q"], case["key_cache"], case["value_cache"], case["cache_k_scale"],
                                  case["cache_v_scale"], case["block_tables"], case["seq_lens_decoder"], num_heads=32,
                                  cache_quant_type=quant)
        torch.cuda.synchronize()
        check(bits(out), oracle_decode(oracle, syn.to_device(case, "cpu")), "batch %d" % batch)


@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_FP8])
@pytest.mark.parametrize("batch,hq,hkv", [(64, 32, 8), (37, 32, 16), (33, 16, 16), (64, 24, 8)])
def test_decode_batches_of_single_chunk_lists(oracle, batch, hq, hkv, quant):
    """Batches of at least 512 (sequence, KV head) pairs: every list is one chunk, finished by its workgroup without
    partials.  Ragged lengths with empty sequences, equal lengths, an odd batch, lists of 1 .. 128 units (both
    unit-table entries of a lane), 1, 2, 3 and 4 query heads per KV head."""
    from fastdeploy_amd import _lib
    rng = np.random.default_rng(batch * 7 + hq)
    shapes = [("ragged", [int(x) for x in rng.integers(0, 1500, batch)], None),
              ("equal", [777] * batch, None),
              ("long and short", [64 * 128 - 3 if i % 5 == 0 else int(rng.integers(1, 200)) for i in range(batch)], 128)]
    for what, lens, mb in shapes:
        lens[3] = 0
        mb = mb or max(lens) // 64 + 2
        assert _lib.lib().fdattn_decode_chunks_per_sequence(batch, hkv, mb) == 1
        case = syn.decode_case(batch=batch, ctx=lens, quant=quant, seed=batch + len(what), hq=hq, hkv=hkv, max_blocks=mb,
                               extra_blocks=3)
        want = oracle_decode(oracle, case)
        got = gpu_decode(case)
        check(got, want, "single chunks, %s" % what)
        assert not got.reshape(batch, -1)[3].any()


def test_decode_one_very_long_sequence(oracle):
    """One sequence of 524,288 tokens (8,192 blocks, 1 GiB of K and V): 64 chunks of 128 units per KV head and the
    merge kernel over all of them."""
    from fastdeploy_amd import _lib
    ctx = 64 * 8192 - 9
    assert _lib.lib().fdattn_decode_chunks_per_sequence(1, 8, 8192) == 64
    case = syn.decode_case(batch=1, ctx=ctx, seed=3, device="cuda", direct_bytes=True)
    out = fd.decode_attention(case["q"], case["key_cache"], case["value_cache"], case["cache_k_scale"],
                              case["cache_v_scale"], case["block_tables"], case["seq_lens_decoder"], num_heads=32)
    torch.cuda.synchronize()
    check(bits(out), oracle_decode(oracle, syn.to_device(case, "cpu")), "524k tokens")


def test_write_then_decode_config3_full_size(oracle):
    """256 new tokens (bf16 qkv ~ N(0,1)), RoPE theta 500000 at positions U{0..8191}, int8 write into the
    block-tabled slots, then decode over ctx = pos + 1: cache bytes bit-exact, outputs within tolerance."""
    case = syn.write_case(num_seqs=256, max_pos=8192, seed=2, blocks_per_seq=128)
    # the prior cache contents are random bytes: use scales that keep the logits moderate
    dev = syn.to_device(case, "cuda")
    out = fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                              dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                              (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                              num_heads=32, kv_num_heads=8, max_chunk=0)
    torch.cuda.synchronize()
    kc, vc = np_of(case["key_cache"]).copy(), np_of(case["value_cache"]).copy()
    q, _, _ = oracle.write_cache_kv(bits(case["qkv"]), kc, vc, np_of(case["cache_k_scale"]), np_of(case["cache_v_scale"]),
                                    np_of(case["rope_cos"]), np_of(case["rope_sin"]), np_of(case["block_tables"]),
                                    np_of(case["seq_lens_decoder"]), np_of(case["cu_seqlens_q"]), 32, 8, 128, 1, CACHE_INT8,
                                    want_kv_out=False)
    assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc)
    want = oracle.decode_attention(q, kc, vc, np_of(case["cache_k_scale"]), np_of(case["cache_v_scale"]),
                                   np_of(case["block_tables"]), np_of(case["seq_lens_decoder"]) + 1, 32, 8, 128, CACHE_INT8)
    check(bits(out), want, "cfg3")


@pytest.mark.parametrize("seqs,hq,hkv,d,bs,mb", [
    (48, 32, 8, 128, 64, 34),     # the int8-MFMA decode kernel
    (12, 16, 4, 64, 16, 136),     # the fp16-MFMA decode kernel with key splits and the merge launch
    (80, 8, 4, 256, 64, 34),      # the same with one split: no merge launch
])
def test_decode_step_replays_from_a_hip_graph(seqs, hq, hkv, d, bs, mb):
    """One decode step of a layer (cache write + decode attention + the length update) captured in a HIP
    graph and replayed with eager work and synchronisations between the replays: every replay must equal
    the same step run eagerly on a copy of the state (outputs and cache bytes, bit for bit).  The path
    allocates nothing of its own and clears nothing with memsets, which is what makes it capturable."""
    case = syn.write_case(num_seqs=seqs, max_pos=2048, seed=5, blocks_per_seq=mb, hq=hq, hkv=hkv, d=d, bs=bs)
    dev = syn.to_device(case, "cuda")
    eag = {k: (v.clone() if isinstance(v, torch.Tensor) else v) for k, v in dev.items()}
    rot_g, rot_e = (dev["rope_cos"], dev["rope_sin"]), (eag["rope_cos"], eag["rope_sin"])
    ws_g = fd.append_attention_workspace(seqs, seqs, hq, hkv, d, mb)
    ws_e = fd.append_attention_workspace(seqs, seqs, hq, hkv, d, mb)

    def step(c, rot, ws):
        out = fd.append_attention(c["qkv"], c["key_cache"], c["value_cache"], c["seq_lens_encoder"],
                                  c["seq_lens_decoder"], c["seq_lens_this_time"], c["block_tables"], rot,
                                  c["cache_k_scale"], c["cache_v_scale"], num_heads=hq, kv_num_heads=hkv, max_chunk=0,
                                  workspace=ws)
        c["seq_lens_decoder"].add_(1)
        return out

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):            # warm-up outside the capture, on a throw-away copy
        tmp = {k: (v.clone() if isinstance(v, torch.Tensor) else v) for k, v in dev.items()}
        step(tmp, rot_g, ws_g)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g = step(dev, rot_g, ws_g)
    # the capture itself runs nothing: state is still the initial one
    gen = torch.Generator(device="cuda").manual_seed(11)
    for r in range(4):
        new_qkv = torch.randn(dev["qkv"].shape, generator=gen, device="cuda").to(torch.bfloat16)
        dev["qkv"].copy_(new_qkv)            # eager work between the replays
        eag["qkv"].copy_(new_qkv)
        torch.cuda.synchronize()
        graph.replay()
        want = step(eag, rot_e, ws_e)
        torch.cuda.synchronize()
        assert torch.equal(out_g, want), "replay %d: outputs differ" % r
        assert torch.equal(dev["key_cache"], eag["key_cache"]) and torch.equal(dev["value_cache"], eag["value_cache"]), r
        assert torch.equal(dev["seq_lens_decoder"], eag["seq_lens_decoder"])
