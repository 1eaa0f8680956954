"""Cache writer on the GPU against the CPU oracle: cache bytes and rotated Q/K bit-exact."""
import numpy as np
import pytest
import torch

import fastdeploy_amd as fd
from conftest import bits, np_of
from fastdeploy_amd import synthetic as syn
from fastdeploy_amd.ops import CACHE_FP8, CACHE_FP8_DYNAMIC, CACHE_INT8, CACHE_INT8_DYNAMIC, is_dynamic

ALL_FORMATS = [CACHE_INT8, CACHE_FP8, CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC]

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


def test_writer_config3_shape_bit_exact(oracle):
    """256 new tokens, positions U{0..8191}, theta 500000, int8, block_size 64."""
    for seed in range(2):
        _run_both(oracle, syn.write_case(num_seqs=256, max_pos=8192, seed=seed, blocks_per_seq=128))


@pytest.mark.parametrize("quant", [CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC])
def test_writer_dynamic_formats_other_head_dims_and_odd_rows(oracle, quant):
    """One scale per stored row for head_dim 128 / 64 / 32 (8, 4, 2 threads share a row), rows of zeros and rows
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


@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_FP8_DYNAMIC])
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
