"""Cache writer on the GPU against the CPU oracle: cache bytes and rotated Q/K bit-exact."""
import numpy as np
import pytest
import torch

import fastdeploy_amd as fd
from conftest import bits, np_of
from fastdeploy_amd import synthetic as syn
from fastdeploy_amd.ops import (CACHE_FP8, CACHE_FP8_BLOCK, CACHE_FP8_DYNAMIC, CACHE_INT8, CACHE_INT8_BLOCK,
                                CACHE_INT8_DYNAMIC, is_dynamic)

ALL_FORMATS = [CACHE_INT8, CACHE_FP8, CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC, CACHE_INT8_BLOCK, CACHE_FP8_BLOCK]

pytestmark = pytest.mark.gpu


def _run_both(oracle, case, want_kv=True, rope=True):
    dev = syn.to_device(case, "cuda")
    rot = (dev["rope_cos"], dev["rope_sin"]) if rope else None
    q, k, v = fd.write_cache_kv(
        dev["qkv"], dev["key_cache"], dev["value_cache"], dev["cache_k_scale"], dev["cache_v_scale"],
        dev["block_tables"], dev["seq_lens_encoder"], dev["seq_lens_decoder"], dev["seq_lens_this_time"],
        dev["cu_seqlens_q"], rot, num_heads=case["hq"], kv_num_heads=case["hkv"], rope_style=case["rope_style"],
        cache_quant_type=case["quant"], want_kv_out=want_kv)
    torch.cuda.synchronize()
    kc, vc = np_of(case["key_cache"]).copy(), np_of(case["value_cache"]).copy()
    ks, vs = np_of(case["cache_k_scale"]).copy(), np_of(case["cache_v_scale"]).copy()  # the dynamic formats store into them
    oq, ok, ov = oracle.write_cache_kv(
        bits(case["qkv"]), kc, vc, ks, vs,
        np_of(case["rope_cos"]) if rope else None, np_of(case["rope_sin"]) if rope else None,
        np_of(case["block_tables"]), np_of(case["seq_lens_decoder"]), np_of(case["cu_seqlens_q"]), case["hq"],
        case["hkv"], case["d"], 1 if case["rope_style"] == "neox" else 0, case["quant"], want_kv)
    assert np.array_equal(np_of(dev["key_cache"]), kc), "key cache bytes differ"
    assert np.array_equal(np_of(dev["value_cache"]), vc), "value cache bytes differ"
    if is_dynamic(case["quant"]):
        assert np.array_equal(np_of(dev["cache_k_scale"]).view(np.uint32), ks.view(np.uint32)), "K scale cache differs"
        assert np.array_equal(np_of(dev["cache_v_scale"]).view(np.uint32), vs.view(np.uint32)), "V scale cache differs"
    assert np.array_equal(bits(q), oq), "rotated Q differs"
    if want_kv:
        assert np.array_equal(bits(k), ok) and np.array_equal(bits(v), ov)
    return dev


@pytest.mark.parametrize("quant", ALL_FORMATS)
@pytest.mark.parametrize("style", ["neox", "interleaved"])
def test_writer_bit_exact_small(oracle, quant, style):
    for seed in range(3):
        _run_both(oracle, syn.write_case(num_seqs=19, max_pos=1000, quant=quant, seed=seed, rope_style=style))


@pytest.mark.parametrize("quant", [CACHE_INT8_DYNAMIC, CACHE_INT8_BLOCK])
@pytest.mark.parametrize("chunk", [1, 40])
def test_writer_shared_scales_at_exact_ties(oracle, quant, chunk):
    """The formats whose rows share a scale quantise with the scale's reciprocal and fall back to the division next to
    a tie: V rows made of half-integers k + 1/2 (every one a tie under the scale 1 = 127 / 127, which the row's or
    tile's largest element, 127, sets; under the scale 1/2 every other one), without rotation so that K meets the same
    values.  Bytes and scales as the oracle's, bit for bit - rint's ties-to-even included."""
    case = syn.write_case(num_seqs=7, max_pos=300, quant=quant, seed=11, chunk=chunk)
    T, hq, hkv, d = case["qkv"].shape[0], case["hq"], case["hkv"], case["d"]
    g = torch.Generator().manual_seed(5)
    half = torch.randint(-126, 126, (T, (hq + 2 * hkv) * d), generator=g).float() + 0.5   # exact in bf16: 8 bits
    half[:, 0::d] = 127.0                                                                # every head's row: maximum 127
    rows = torch.arange(T) % 2 == 1
    half[rows] = half[rows] * 0.5                                                        # odd tokens: scale 1/2 (rows) / mixed tiles
    case["qkv"] = half.to(torch.bfloat16)
    assert torch.equal(case["qkv"].float(), half)
    _run_both(oracle, case, rope=False)


def test_writer_config3_shape_bit_exact(oracle):
    """256 new tokens, positions U{0..8191}, theta 500000, int8, block_size 64."""
    for seed in range(2):
        _run_both(oracle, syn.write_case(num_seqs=256, max_pos=8192, seed=seed, blocks_per_seq=128))


@pytest.mark.parametrize("quant", [CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC, CACHE_INT8_BLOCK, CACHE_FP8_BLOCK])
def test_writer_dynamic_formats_other_head_dims_and_odd_rows(oracle, quant):
    """One scale per stored row (or per tile) for head_dim 128 / 64 / 32 (8, 4, 2 threads share a row), rows of zeros and rows
    holding a NaN: bytes and scale caches bit for bit as the oracle's."""
    for d, hq, hkv in ((128, 8, 2), (64, 4, 2), (32, 2, 1)):
        case = syn.write_case(num_seqs=9, max_pos=400, quant=quant, seed=3 + d, hq=hq, hkv=hkv, d=d, chunk=4)
        x = case["qkv"].view(36, hq + 2 * hkv, d)
        x[3, hq] = 0                       # a K row of zeros: scale 1, bytes 0
        x[5, hq + hkv, 7] = float("nan")   # a NaN does not take part in the row's maximum
        x[7, hq + hkv + hkv - 1] *= 300.0  # a large row
        _run_both(oracle, case)


@pytest.mark.parametrize("quant", ALL_FORMATS)
def test_writer_chunks_ragged_and_no_rope(oracle, quant):
    case = syn.write_case(num_seqs=5, max_pos=700, quant=quant, seed=4, chunk=37)
    _run_both(oracle, case)
    _run_both(oracle, case, rope=False, want_kv=False)
    # ragged chunks incl. an empty sequence
    lens = torch.tensor([3, 0, 64, 1, 117], dtype=torch.int32)
    T = int(lens.sum())
    case["qkv"] = case["qkv"][:T].contiguous()
    case["seq_lens_this_time"] = lens
    case["seq_lens_encoder"] = lens
    case["cu_seqlens_q"] = torch.tensor([0, 3, 3, 67, 68, 185], dtype=torch.int32)
    case["seq_lens_decoder"] = torch.tensor([0, 5, 63, 640, 300], dtype=torch.int32)
    _run_both(oracle, case)


@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_FP8_DYNAMIC, CACHE_INT8_BLOCK])
def test_writer_more_tokens_than_one_grid_dimension_holds(oracle, quant):
    """66,000 new tokens in one call (a grid dimension holds 65,535 workgroups: the launch goes in slices): every
    byte, scale and rotated row as the oracle's."""
    case = syn.write_case(num_seqs=3, max_pos=22050, quant=quant, seed=17, hq=2, hkv=1, d=32, chunk=22000)
    assert case["qkv"].shape[0] == 66000
    _run_both(oracle, case)


@pytest.mark.parametrize("style", ["neox", "interleaved"])
@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_FP8])
def test_writer_epilogue_bit_exact(oracle, quant, style):
    """bias, RMS norm of Q and K heads, both, and each norm alone - in front of the rotation; every output
    bit for bit as the oracle's."""
    g = torch.Generator().manual_seed(8)
    for d, hq, hkv in ((128, 32, 8), (64, 4, 2), (32, 2, 1)):
        case = syn.write_case(num_seqs=11, max_pos=500, quant=quant, seed=d, rope_style=style, hq=hq, hkv=hkv, d=d,
                              chunk=3)
        dev = syn.to_device(case, "cuda")
        bias = (torch.randn(((hq + 2 * hkv) * d,), generator=g) * 0.5).to(torch.bfloat16)
        qw = torch.rand((d,), generator=g) + 0.5
        kw = torch.rand((d,), generator=g) + 0.5
        for use_bias, use_q, use_k, eps in ((1, 0, 0, 0.0), (0, 1, 1, 1e-6), (1, 1, 1, 1e-5), (0, 1, 0, 0.0), (1, 0, 1, 1e-6)):
            kc_d, vc_d = dev["key_cache"].clone(), dev["value_cache"].clone()
            q, k, v = fd.write_cache_kv(
                dev["qkv"], kc_d, vc_d, dev["cache_k_scale"], dev["cache_v_scale"], dev["block_tables"],
                dev["seq_lens_encoder"], dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["cu_seqlens_q"],
                (dev["rope_cos"], dev["rope_sin"]), num_heads=hq, kv_num_heads=hkv, rope_style=style,
                cache_quant_type=quant, want_kv_out=True, qkv_bias=bias.cuda() if use_bias else None,
                q_norm_weight=qw.cuda() if use_q else None, k_norm_weight=kw.cuda() if use_k else None, rms_norm_eps=eps)
            torch.cuda.synchronize()
            kc, vc = np_of(case["key_cache"]).copy(), np_of(case["value_cache"]).copy()
            oq, ok, ov = oracle.write_cache_kv(
                bits(case["qkv"]), kc, vc, np_of(case["cache_k_scale"]), np_of(case["cache_v_scale"]),
                np_of(case["rope_cos"]), np_of(case["rope_sin"]), np_of(case["block_tables"]),
                np_of(case["seq_lens_decoder"]), np_of(case["cu_seqlens_q"]), hq, hkv, d, 1 if style == "neox" else 0,
                quant, True, qkv_bias=bits(bias) if use_bias else None, q_norm_weight=np_of(qw) if use_q else None,
                k_norm_weight=np_of(kw) if use_k else None, rms_norm_eps=eps)
            what = "d=%d bias=%d qnorm=%d knorm=%d" % (d, use_bias, use_q, use_k)
            assert np.array_equal(bits(q), oq), what + ": Q"
            assert np.array_equal(bits(k), ok), what + ": K"
            assert np.array_equal(bits(v), ov), what + ": V"
            assert np.array_equal(np_of(kc_d), kc) and np.array_equal(np_of(vc_d), vc), what + ": cache bytes"
    with pytest.raises(ValueError):      # head_dim 96: six threads per head, no butterfly
        c96 = syn.to_device(syn.write_case(num_seqs=2, max_pos=64, hq=2, hkv=1, d=96), "cuda")
        fd.write_cache_kv(c96["qkv"], c96["key_cache"], c96["value_cache"], c96["cache_k_scale"], c96["cache_v_scale"],
                          c96["block_tables"], c96["seq_lens_encoder"], c96["seq_lens_decoder"], c96["seq_lens_this_time"],
                          c96["cu_seqlens_q"], None, num_heads=2, kv_num_heads=1,
                          q_norm_weight=torch.ones(96, device="cuda"))


def test_quantisers_exhaustive_over_bf16(oracle):
    """Every finite bf16 value through the int8 and fp8 quantisers at several scales, via V (no rotation)."""
    allbits = np.arange(65536, dtype=np.uint16)
    vals = torch.from_numpy(allbits.view(np.int16)).view(torch.bfloat16)
    vals = vals[torch.isfinite(vals.float())]
    n = vals.numel()
    T = (n + 1023) // 1024
    pad = torch.zeros(T * 1024 - n, dtype=torch.bfloat16)
    v = torch.cat([vals, pad]).view(T, 8 * 128)
    for quant in (CACHE_INT8, CACHE_FP8):
        case = syn.write_case(num_seqs=T, max_pos=64, quant=quant, seed=1, blocks_per_seq=1)
        case["qkv"][:, 32 * 128 + 8 * 128:] = v
        case["qkv"][:, 32 * 128:40 * 128] = v          # K too (rotated: still must match the oracle)
        sc = torch.tensor([1.0, 0.03125, 0.0314159, 4.0 / 127.0, 3.7e-3, 17.25, 0.5, 1e-2])
        case["cache_v_scale"] = sc[:, None].repeat(1, 128).contiguous()
        _run_both(oracle, case, want_kv=False)


def test_writer_rejects_bad_arguments():
    case = syn.to_device(syn.write_case(num_seqs=4, max_pos=128), "cuda")
    with pytest.raises(ValueError):
        fd.write_cache_kv(case["qkv"][:, :-1].contiguous(), case["key_cache"], case["value_cache"], case["cache_k_scale"],
                          case["cache_v_scale"], case["block_tables"], case["seq_lens_encoder"], case["seq_lens_decoder"],
                          num_heads=32, kv_num_heads=8)
    with pytest.raises(ValueError):
        fd.write_cache_kv(case["qkv"], case["key_cache"], case["value_cache"], case["cache_k_scale"],
                          case["cache_v_scale"], case["block_tables"], case["seq_lens_encoder"], case["seq_lens_decoder"],
                          num_heads=32, kv_num_heads=8, cache_quant_type="cache_int4")


@pytest.mark.parametrize("quant", [CACHE_INT8_BLOCK, CACHE_FP8_BLOCK])
@pytest.mark.parametrize("shape", [(128, 8, 2, 64), (32, 2, 1, 16), (64, 4, 4, 32)])
def test_writer_per_block_formats_call_after_call(oracle, quant, shape):
    """One scale per (block, KV head) tile, kept over a sequence of calls: ragged prefill chunks, decode steps whose
    rows outgrow the tiles' scales (earlier rows are requantised) and steps that do not, chunks crossing block
    boundaries, with and without the projection's epilogue.  After every call the caches and both scale caches are
    the oracle's bit for bit."""
    d, hq, hkv, bs = shape
    g = torch.Generator().manual_seed(d + quant)
    nseq, blocks = 5, 6
    pool = nseq * blocks
    from fastdeploy_amd.rope import rope_table
    cos, sin = rope_table(blocks * bs, d, 10000.0, "cpu")
    kc = torch.randint(0, 256, (pool, hkv, bs, d), generator=g, dtype=torch.uint8)
    vc = torch.randint(0, 256, (pool, hkv, bs, d), generator=g, dtype=torch.uint8)
    ks, vs = torch.full((pool, hkv), float("nan")), torch.full((pool, hkv), float("nan"))
    bt = torch.randperm(pool, generator=g).to(torch.int32).view(nseq, blocks)
    host = [np_of(t).copy() for t in (kc, vc, ks, vs)]
    dev = [t.cuda() for t in (kc, vc, ks, vs)]
    bias = (torch.randn(((hq + 2 * hkv) * d,), generator=g) * 0.5).to(torch.bfloat16)
    kw = torch.rand((d,), generator=g) + 0.5
    lens = [0] * nseq
    calls = [([bs + 3, 1, 0, 2 * bs, 7], 1.0, False), ([1] * nseq, 1.0, False), ([1] * nseq, 6.0, True),
             ([1, 0, 1, 1, 0], 0.2, False), ([bs - 5, 2, 3, bs, 1], 2.5, True), ([1] * nseq, 30.0, False),
             ([3, 3, 3, 3, 3], 0.01, False),
             # no more tokens than sequences, yet rows of several tokens: the one-launch path walks them
             ([3, 0, 0, 2, 0], 50.0, False), ([0, 2, 1, 0, 1], 0.3, True)]
    for new, mag, epilogue in calls:
        T = sum(new)
        qkv = (torch.randn((T, (hq + 2 * hkv) * d), generator=g) * mag).to(torch.bfloat16)
        this = torch.tensor(new, dtype=torch.int32)
        cu = torch.tensor([0] + list(np.cumsum(new)), dtype=torch.int32)
        dec = torch.tensor(lens, dtype=torch.int32)
        extra = dict(qkv_bias=bias.cuda(), k_norm_weight=kw.cuda(), rms_norm_eps=1e-6) if epilogue else {}
        q, k, v = fd.write_cache_kv(qkv.cuda(), dev[0], dev[1], dev[2], dev[3], bt.cuda(), this.cuda(), dec.cuda(),
                                    this.cuda(), cu.cuda(), (cos.cuda(), sin.cuda()), num_heads=hq, kv_num_heads=hkv,
                                    rope_style="neox", cache_quant_type=quant, want_kv_out=True, **extra)
        torch.cuda.synchronize()
        oextra = dict(qkv_bias=bits(bias), k_norm_weight=np_of(kw), rms_norm_eps=1e-6) if epilogue else {}
        oq, ok, ov = oracle.write_cache_kv(bits(qkv), host[0], host[1], host[2], host[3], np_of(cos), np_of(sin), np_of(bt),
                                           np_of(dec), np_of(cu), hq, hkv, d, 1, quant, True, **oextra)
        what = "after the call with %r x %g" % (new, mag)
        assert np.array_equal(bits(q), oq) and np.array_equal(bits(k), ok) and np.array_equal(bits(v), ov), what
        assert np.array_equal(np_of(dev[2]).view(np.uint32), host[2].view(np.uint32)), what + ": K scales"
        assert np.array_equal(np_of(dev[3]).view(np.uint32), host[3].view(np.uint32)), what + ": V scales"
        assert np.array_equal(np_of(dev[0]), host[0]), what + ": K bytes"
        assert np.array_equal(np_of(dev[1]), host[1]), what + ": V bytes"
        lens = [a + b for a, b in zip(lens, new)]


@pytest.mark.parametrize("quant", [CACHE_INT8_BLOCK, CACHE_FP8_BLOCK])
def test_writer_per_block_formats_after_rejected_drafts(oracle, quant):
    """A speculative step writes three tokens per sequence, two of them large, and only the first is accepted: the next
    step writes over the rejected rows.  A tile's scale only ever grows - it stays where the rejected rows put it, and
    the accepted row keeps the bytes of that grid - so the cache is a function of the CALLS, not of the accepted
    tokens: the oracle, given the same calls, must agree bit for bit after every one of them, and no scale may shrink."""
    d, hq, hkv, bs = 128, 8, 2, 64
    g = torch.Generator().manual_seed(17 + quant)
    nseq, blocks = 4, 3
    pool = nseq * blocks
    from fastdeploy_amd.rope import rope_table
    cos, sin = rope_table(blocks * bs, d, 10000.0, "cpu")
    kc = torch.zeros((pool, hkv, bs, d), dtype=torch.uint8)
    vc = torch.zeros((pool, hkv, bs, d), dtype=torch.uint8)
    ks, vs = torch.full((pool, hkv), float("nan")), torch.full((pool, hkv), float("nan"))
    bt = torch.randperm(pool, generator=g).to(torch.int32).view(nseq, blocks)
    host = [np_of(t).copy() for t in (kc, vc, ks, vs)]
    dev = [t.cuda() for t in (kc, vc, ks, vs)]
    lens = [bs - 2, 5, 0, bs + 1]          # drafts that cross a block boundary, sit inside a tile, open the first tile
    # (tokens per sequence, magnitude of each token of a row, tokens that stay)
    steps = [([5, 5, 5, 5], [1.0] * 5, 5),              # some history in every tile first (sequence 2: its first rows)
             ([3, 3, 3, 3], [1.0, 20.0, 40.0], 1),       # drafts 2 and 3 are large and rejected
             ([3, 3, 3, 3], [0.5, 0.5, 0.5], 3),         # written over them, small: the scale stays up
             ([1, 1, 1, 1], [0.0], 1),                   # a row of zeros
             ([2, 2, 2, 2], [60.0, 0.1], 0)]             # everything rejected
    for new, mags, keep in steps:
        T = sum(new)
        rows = torch.cat([torch.tensor(mags[:n]) for n in new])
        qkv = (torch.randn((T, (hq + 2 * hkv) * d), generator=g) * rows[:, None]).to(torch.bfloat16)
        this = torch.tensor(new, dtype=torch.int32)
        cu = torch.tensor([0] + list(np.cumsum(new)), dtype=torch.int32)
        dec = torch.tensor(lens, dtype=torch.int32)
        before = [np_of(dev[2]).copy(), np_of(dev[3]).copy()]
        fd.write_cache_kv(qkv.cuda(), dev[0], dev[1], dev[2], dev[3], bt.cuda(), this.cuda(), dec.cuda(), this.cuda(), cu.cuda(),
                          (cos.cuda(), sin.cuda()), num_heads=hq, kv_num_heads=hkv, rope_style="neox", cache_quant_type=quant)
        torch.cuda.synchronize()
        oracle.write_cache_kv(bits(qkv), host[0], host[1], host[2], host[3], np_of(cos), np_of(sin), np_of(bt), np_of(dec),
                              np_of(cu), hq, hkv, d, 1, quant, False)
        what = "after the step of %r tokens x %r of which %d stay" % (new, mags, keep)
        for i, name in ((2, "K scales"), (3, "V scales")):
            assert np.array_equal(np_of(dev[i]).view(np.uint32), host[i].view(np.uint32)), what + ": " + name
            was, now = before[i - 2], np_of(dev[i])
            assert np.all((now >= was) | np.isnan(was)), what + ": a scale shrank"
        assert np.array_equal(np_of(dev[0]), host[0]), what + ": K bytes"
        assert np.array_equal(np_of(dev[1]), host[1]), what + ": V bytes"
        lens = [a + keep for a in lens]


@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_FP8_DYNAMIC, CACHE_INT8_BLOCK])
def test_writer_tokens_past_the_rope_table_are_skipped_with_zeroed_rows(quant):
    """A token whose position lies outside the rotation table cannot be written: the caches (and scale caches) keep
    their bytes and its rows of q_out / k_out / v_out are zeros, not whatever the output buffers held."""
    case = syn.to_device(syn.write_case(num_seqs=6, max_pos=256, quant=quant, seed=9), "cuda")
    case["seq_lens_decoder"][1] = 256          # first position past the table
    case["seq_lens_decoder"][4] = 300
    before = {k: case[k].clone() for k in ("key_cache", "value_cache", "cache_k_scale", "cache_v_scale")}
    # the same step without the two rows gives the expected cache contents
    ref = {k: (v.clone() if isinstance(v, torch.Tensor) else v) for k, v in case.items()}
    ref["block_tables"] = case["block_tables"].clone()
    ref["block_tables"][[1, 4]] = -1
    ref["seq_lens_decoder"][[1, 4]] = 0
    torch.cuda.synchronize()
    outs = {}
    for name, c in (("got", case), ("ref", ref)):
        outs[name] = fd.write_cache_kv(c["qkv"], c["key_cache"], c["value_cache"], c["cache_k_scale"], c["cache_v_scale"],
                                       c["block_tables"], c["seq_lens_encoder"], c["seq_lens_decoder"],
                                       c["seq_lens_this_time"], c["cu_seqlens_q"], (c["rope_cos"], c["rope_sin"]),
                                       num_heads=32, kv_num_heads=8, cache_quant_type=quant, want_kv_out=True)
    torch.cuda.synchronize()
    for k in before:
        assert torch.equal(case[k].view(torch.uint8), ref[k].view(torch.uint8)), k
    for got, want in zip(outs["got"], outs["ref"]):
        assert not got[[1, 4]].any()
        keep = [0, 2, 3, 5]
        assert torch.equal(got[keep].view(torch.int16), want[keep].view(torch.int16))
