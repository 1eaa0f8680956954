"""Pins the CPU oracle (oracle/fdattn_oracle.c) before anything is compared with it.

The reference holds no implementation or vector of this path, so each function is
pinned by what fixes it independently: torch's CPU casts (exhaustively), closed
forms, invariants, torch's CPU attention in fp64, brute force in numpy fp64, and
the adjacent known-answer vectors of the reference's own unit tests.
"""
import json
import math
import os

import numpy as np
import pytest
import torch

from conftest import bf16_close, bits, np_of
from fastdeploy_amd import synthetic as syn
from fastdeploy_amd.ops import CACHE_FP8, CACHE_FP8_DYNAMIC, CACHE_INT8, CACHE_INT8_DYNAMIC, is_dynamic
from fastdeploy_amd.rope import rope_table

def assert_is_bf16_of(got, want, extra=3e-4):
    """got (bf16 values as float) must be want (fp64) rounded to bf16, up to `extra` of fp32 arithmetic error:
    |got - want| <= |want| * 2^-8 (half a bf16 ulp just above a power of two) + extra."""
    d = np.abs(np.asarray(got, np.float64) - np.asarray(want, np.float64))
    lim = np.abs(np.asarray(want, np.float64)) * 2.0 ** -8 + extra
    assert (d <= lim).all(), "max excess %.3g at |want|=%.3g" % ((d - lim).max(), np.abs(want).ravel()[(d - lim).argmax()])


GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_function_vectors.json")))


# ------------------------------------------------------------------ scalars

def test_bf16_roundtrip_and_rne_match_torch(oracle):
    allbits = np.arange(65536, dtype=np.uint16)
    f = oracle.bf16_to_f32(allbits)
    t = torch.from_numpy(allbits.view(np.int16)).view(torch.bfloat16).float().numpy()
    assert np.array_equal(f.view(np.uint32), t.view(np.uint32))
    # RNE: random fp32 incl. exact ties, against torch's cast
    rng = np.random.default_rng(0)
    x = rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-20, 20, 200000).astype(np.float32)
    ties = ((rng.integers(0, 65536, 50000).astype(np.uint32) << 16) | 0x8000).view(np.float32)
    ties = ties[~np.isnan(ties)]          # NaN payloads are a convention, not a rounding question
    x = np.concatenate([x, ties, np.array([0.0, -0.0, np.inf, -np.inf, 3.3895314e38], np.float32)])
    got = oracle.f32_to_bf16(x)
    want = bits(torch.from_numpy(x).to(torch.bfloat16))
    assert np.array_equal(got, want)
    one = np.array([oracle.lib().fdo_f32_to_bf16(float(v)) for v in x[:2000]], dtype=np.uint16)
    assert np.array_equal(one, want[:2000])


def test_e4m3_decode_all_codes_match_torch(oracle):
    codes = np.arange(256, dtype=np.uint8)
    got = oracle.e4m3_to_f32(codes)
    want = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    ok = np.isnan(want) == np.isnan(got)
    assert ok.all()
    m = ~np.isnan(want)
    assert np.array_equal(got[m].view(np.uint32), want[m].view(np.uint32))


def test_e4m3_encode_exhaustive_over_bf16_and_midpoints(oracle):
    # every finite bf16 value, clamped to +-448 as the cache format says
    allbits = np.arange(65536, dtype=np.uint16)
    x = oracle.bf16_to_f32(allbits)
    x = x[np.isfinite(x)]
    # plus every midpoint between adjacent e4m3 values and its two fp32 neighbours (tie cases)
    grid = oracle.e4m3_to_f32(np.arange(0, 0x7F, dtype=np.uint8)).astype(np.float64)
    mid = ((grid[:-1] + grid[1:]) / 2).astype(np.float32)
    x = np.concatenate([x, mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(1e9)), -mid,
                        np.float32(1e-3) * np.random.default_rng(1).standard_normal(20000).astype(np.float32),
                        np.float32(100) * np.random.default_rng(2).standard_normal(20000).astype(np.float32)])
    got = oracle.f32_to_e4m3(x)
    want = torch.from_numpy(np.clip(x, -448, 448)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(got, want)


def test_int8_quant_closed_form_exhaustive(oracle):
    allbits = np.arange(65536, dtype=np.uint16)
    x = oracle.bf16_to_f32(allbits)
    x = x[np.isfinite(x)]
    for s in [1.0, 0.03125, 0.0314159, 4.0 / 127.0, 3.7e-3, 17.25]:
        s32 = np.float32(s)
        got = oracle.quant_int8(x, s32)
        want = np.clip(np.rint(x / s32), -127, 127).astype(np.int8)   # numpy: fp32 division, ties to even
        assert np.array_equal(got, want), s
        inside = np.abs(x / s32) <= 127
        err = np.abs(x[inside].astype(np.float64) - got[inside].astype(np.float64) * float(s32))
        assert (err <= float(s32) / 2 * (1 + 1e-6)).all()
    # the max-abs channel value maps to +-127 exactly
    for m in [0.5, 3.0, 4.46875, 1e-3]:
        s32 = np.float32(m) / np.float32(127.0)
        assert oracle.lib().fdo_quant_int8(float(np.float32(m)), float(s32)) == 127
        assert oracle.lib().fdo_quant_int8(float(np.float32(-m)), float(s32)) == -127


def test_softmax_known_answers_of_reference(oracle):
    g = GOLD["softmax"]
    x = np.array(g["input_2x3"], np.float32).reshape(2, 3)
    rows = np.stack([oracle.softmax_row(x[i]) for i in range(2)])
    assert np.allclose(rows.ravel(), g["expected_axis1"], atol=1e-6, rtol=1e-6)
    cols = np.stack([oracle.softmax_row(np.ascontiguousarray(x[:, j])) for j in range(3)], axis=1)
    assert np.allclose(cols.ravel(), g["expected_axis0"], atol=1e-6, rtol=1e-6)


# -------------------------------------------------------------- cache writer

def _write(oracle, case, want_kv=True):
    kc, vc = np_of(case["key_cache"]).copy(), np_of(case["value_cache"]).copy()
    q, k, v = oracle.write_cache_kv(
        bits(case["qkv"]), kc, vc, np_of(case["cache_k_scale"]), np_of(case["cache_v_scale"]),
        np_of(case["rope_cos"]), np_of(case["rope_sin"]), np_of(case["block_tables"]),
        np_of(case["seq_lens_decoder"]), np_of(case["cu_seqlens_q"]), case["hq"], case["hkv"], case["d"],
        1 if case["rope_style"] == "neox" else 0, case["quant"], want_kv)
    return q, k, v, kc, vc


def test_rope_table_closed_forms():
    cos, sin = rope_table(64, 128, 500000.0)
    assert cos.shape == (64, 64) and cos.dtype == torch.float32
    assert torch.all(cos[0] == 1) and torch.all(sin[0] == 0)
    assert torch.all(cos[:, 0] == torch.cos(torch.arange(64, dtype=torch.float64)).float())
    inv = 500000.0 ** (-2.0 * 63 / 128)
    assert abs(float(cos[17, 63]) - math.cos(17 * inv)) < 1e-7
    assert torch.allclose(cos ** 2 + sin ** 2, torch.ones_like(cos), atol=1e-6)


@pytest.mark.parametrize("style", ["neox", "interleaved"])
def test_writer_rope_against_complex_multiplication(oracle, style):
    case = syn.write_case(num_seqs=24, max_pos=512, seed=3, rope_style=style)
    q, k, v, kc, vc = _write(oracle, case)
    hq, hkv, d = case["hq"], case["hkv"], case["d"]
    x = case["qkv"].double().view(24, hq + 2 * hkv, d)
    pos = case["seq_lens_decoder"].long()
    ang = torch.arange(512, dtype=torch.float64)[:, None] * (500000.0 ** (-2.0 * torch.arange(d // 2, dtype=torch.float64) / d))[None]
    rot = torch.polar(torch.ones_like(ang), ang)[pos][:, None, :]                      # e^{i pos w_j}
    if style == "neox":
        z = torch.complex(x[..., : d // 2], x[..., d // 2:])
    else:
        z = torch.complex(x[..., 0::2], x[..., 1::2])
    zr = z * rot
    want = torch.empty_like(x)
    if style == "neox":
        want[..., : d // 2], want[..., d // 2:] = zr.real, zr.imag
    else:
        want[..., 0::2], want[..., 1::2] = zr.real, zr.imag
    got_q = torch.from_numpy(oracle.bf16_to_f32(q)).double().view(24, hq, d)
    assert torch.allclose(got_q, want[:, :hq], atol=2e-2, rtol=8e-3)                   # bf16 rounding of the output
    got_k = torch.from_numpy(oracle.bf16_to_f32(k)).double().view(24, hkv, d)
    assert torch.allclose(got_k, want[:, hq:hq + hkv], atol=2e-2, rtol=8e-3)
    # pair norms are preserved (checked on the fp64 side of the same rotation) and v passes through
    assert np.array_equal(v.reshape(24, hkv, d), bits(case["qkv"]).reshape(24, hq + 2 * hkv, d)[:, hq + hkv:])
    # cache bytes = quantised rotated K at the block-tabled slot, within half a step of the fp64 value
    ks = case["cache_k_scale"].double()
    bt = case["block_tables"]
    for b in range(24):
        p = int(pos[b])
        blk, slot = int(bt[b, p // 64]), p % 64
        got = torch.from_numpy(kc[blk, :, slot, :].view(np.int8).astype(np.float64))
        ideal = want[b, hq:hq + hkv] / ks
        assert (got - torch.clamp(ideal, -127, 127)).abs().max() <= 0.5 + 1e-3


def _write_ep(oracle, case, bias=None, qw=None, kw=None, eps=0.0, rope=True):
    kc, vc = np_of(case["key_cache"]).copy(), np_of(case["value_cache"]).copy()
    q, k, v = oracle.write_cache_kv(
        bits(case["qkv"]), kc, vc, np_of(case["cache_k_scale"]), np_of(case["cache_v_scale"]),
        np_of(case["rope_cos"]) if rope else None, np_of(case["rope_sin"]) if rope else None,
        np_of(case["block_tables"]), np_of(case["seq_lens_decoder"]), np_of(case["cu_seqlens_q"]), case["hq"],
        case["hkv"], case["d"], 1 if case["rope_style"] == "neox" else 0, case["quant"], True,
        qkv_bias=None if bias is None else bits(bias), q_norm_weight=qw, k_norm_weight=kw, rms_norm_eps=eps)
    return q, k, v, kc, vc


@pytest.mark.parametrize("style", ["neox", "interleaved"])
def test_writer_epilogue_bias_and_rms_norm(oracle, style):
    """The projection epilogue of the writer: the bias add is torch's bf16 add; the RMS norm agrees with
    an fp64 one; unit weights give heads of unit mean square; the norm forgets the input's scale; and the
    epilogue composes with the rotation (norm in front of the complex multiplication)."""
    case = syn.write_case(num_seqs=16, max_pos=300, seed=11, rope_style=style)
    hq, hkv, d = case["hq"], case["hkv"], case["d"]
    g = torch.Generator().manual_seed(1)
    bias = (torch.randn(((hq + 2 * hkv) * d,), generator=g) * 0.5).to(torch.bfloat16)
    # bias alone, no rotation: every output is torch's bf16 sum, V included
    q, k, v, kc, vc = _write_ep(oracle, case, bias=bias, rope=False)
    want = (case["qkv"] + bias[None]).view(16, hq + 2 * hkv, d)                        # bf16 + bf16 -> bf16 (RNE of the exact sum)
    assert np.array_equal(q.reshape(16, hq, d), bits(want[:, :hq]))
    assert np.array_equal(k.reshape(16, hkv, d), bits(want[:, hq:hq + hkv]))
    assert np.array_equal(v.reshape(16, hkv, d), bits(want[:, hq + hkv:]))
    # the V bytes are the quantised biased values
    pos = case["seq_lens_decoder"].long()
    bt = case["block_tables"]
    for b in range(16):
        blk, slot = int(bt[b, int(pos[b]) // 64]), int(pos[b]) % 64
        ideal = want[b, hq + hkv:].double() / case["cache_v_scale"].double()
        got = torch.from_numpy(vc[blk, :, slot, :].view(np.int8).astype(np.float64))
        assert (got - torch.clamp(ideal, -127, 127)).abs().max() <= 0.5 + 1e-6
    # norm (with bias), no rotation, against fp64
    qw = (torch.rand((d,), generator=g) + 0.5).numpy()
    kw = (torch.rand((d,), generator=g) + 0.5).numpy()
    eps = 1e-6
    q, k, v, _, _ = _write_ep(oracle, case, bias=bias, qw=qw, kw=kw, eps=eps, rope=False)
    x = want.double()
    rms = torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)
    nq = x[:, :hq] * rms[:, :hq] * torch.from_numpy(qw).double()
    nk = x[:, hq:hq + hkv] * rms[:, hq:hq + hkv] * torch.from_numpy(kw).double()
    gq = torch.from_numpy(oracle.bf16_to_f32(q)).double().view(16, hq, d)
    gk = torch.from_numpy(oracle.bf16_to_f32(k)).double().view(16, hkv, d)
    assert torch.allclose(gq, nq, atol=1e-6, rtol=2.0 ** -8) and torch.allclose(gk, nk, atol=1e-6, rtol=2.0 ** -8)
    assert np.array_equal(v.reshape(16, hkv, d), bits(want[:, hq + hkv:]))             # V is never normed
    # only K normed: Q stays the biased input
    q2, k2, _, _, _ = _write_ep(oracle, case, bias=bias, kw=kw, eps=eps, rope=False)
    assert np.array_equal(q2.reshape(16, hq, d), bits(want[:, :hq])) and np.array_equal(k2, k)
    # unit weights, eps 0: mean square 1 (up to bf16 rounding of the outputs); input scale is forgotten
    one = np.ones(d, np.float32)
    q3, _, _, _, _ = _write_ep(oracle, case, qw=one, kw=one, rope=False)
    ms = (torch.from_numpy(oracle.bf16_to_f32(q3)).double().view(16, hq, d) ** 2).mean(-1)
    assert (ms - 1).abs().max() < 5e-3
    scaled = dict(case)
    scaled["qkv"] = (case["qkv"].float() * 4.0).to(torch.bfloat16)                      # exact in bf16
    q4, k4, _, kc4, _ = _write_ep(oracle, scaled, qw=qw, kw=kw, eps=0.0)
    q5, k5, _, kc5, _ = _write_ep(oracle, case, qw=qw, kw=kw, eps=0.0)
    assert np.array_equal(q4, q5) and np.array_equal(k4, k5) and np.array_equal(kc4, kc5)   # x4 is exact at every step
    # with the rotation: the norm comes first (rotation keeps pair norms, so rotating the fp64 norm matches)
    ang = torch.arange(300, dtype=torch.float64)[:, None] * (500000.0 ** (-2.0 * torch.arange(d // 2, dtype=torch.float64) / d))[None]
    rot = torch.polar(torch.ones_like(ang), ang)[pos][:, None, :]
    xq = case["qkv"].double().view(16, hq + 2 * hkv, d)[:, :hq]
    nq = xq * torch.rsqrt((xq * xq).mean(-1, keepdim=True) + eps) * torch.from_numpy(qw).double()
    z = torch.complex(nq[..., : d // 2], nq[..., d // 2:]) if style == "neox" else torch.complex(nq[..., 0::2], nq[..., 1::2])
    zr = z * rot
    wq = torch.empty_like(nq)
    if style == "neox":
        wq[..., : d // 2], wq[..., d // 2:] = zr.real, zr.imag
    else:
        wq[..., 0::2], wq[..., 1::2] = zr.real, zr.imag
    q6, _, _, _, _ = _write_ep(oracle, case, qw=qw, kw=kw, eps=eps)
    g6 = torch.from_numpy(oracle.bf16_to_f32(q6)).double().view(16, hq, d)
    assert torch.allclose(g6, wq, atol=2e-2, rtol=8e-3)


def test_writer_position_zero_is_identity_and_untouched_slots_stay(oracle):
    case = syn.write_case(num_seqs=8, max_pos=256, seed=5)
    case["seq_lens_decoder"][:] = 0
    before_k = np_of(case["key_cache"]).copy()
    q, k, v, kc, vc = _write(oracle, case)
    hq, hkv, d = case["hq"], case["hkv"], case["d"]
    src = bits(case["qkv"]).reshape(8, hq + 2 * hkv, d)
    assert np.array_equal(q.reshape(8, hq, d), src[:, :hq])
    assert np.array_equal(k.reshape(8, hkv, d), src[:, hq:hq + hkv])
    changed = (kc != before_k)
    touched = np.zeros_like(changed)
    for b in range(8):
        touched[int(case["block_tables"][b, 0]), :, 0, :] = True
    assert not (changed & ~touched).any()
    want = syn.quantize_ref(case["qkv"].float().view(8, hq + 2 * hkv, d)[:, hq:hq + hkv], case["cache_k_scale"], CACHE_INT8)
    for b in range(8):
        assert np.array_equal(kc[int(case["block_tables"][b, 0]), :, 0, :], want[b].numpy())


def test_writer_relative_position_property(oracle):
    """<RoPE(q,p), RoPE(k,p')> depends only on p - p' (checked through the bf16 outputs)."""
    case = syn.write_case(num_seqs=2, max_pos=4096, seed=7)
    case["qkv"][1] = case["qkv"][0]
    case["seq_lens_decoder"][0], case["seq_lens_decoder"][1] = 100, 100
    q0, k0, *_ = _write(oracle, case)
    hq, hkv, d = case["hq"], case["hkv"], case["d"]
    base = float(oracle.bf16_to_f32(q0[0, :d]).astype(np.float64) @ oracle.bf16_to_f32(k0[0, :d]).astype(np.float64))
    case["seq_lens_decoder"][0], case["seq_lens_decoder"][1] = 3100, 3100
    q1, k1, *_ = _write(oracle, case)
    moved = float(oracle.bf16_to_f32(q1[0, :d]).astype(np.float64) @ oracle.bf16_to_f32(k1[0, :d]).astype(np.float64))
    assert abs(base - moved) < 0.35   # two bf16 roundings of 128-term dot products of N(0,1) data


@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_FP8])
def test_writer_bytes_match_torch_formulas(oracle, quant):
    """With no rotation the cache bytes must equal torch's x/scale -> round/clamp (-> e4m3 cast)."""
    case = syn.write_case(num_seqs=16, max_pos=300, seed=11, quant=quant, chunk=3)
    kc, vc = np_of(case["key_cache"]).copy(), np_of(case["value_cache"]).copy()
    hq, hkv, d = case["hq"], case["hkv"], case["d"]
    oracle.write_cache_kv(bits(case["qkv"]), kc, vc, np_of(case["cache_k_scale"]), np_of(case["cache_v_scale"]),
                          None, None, np_of(case["block_tables"]), np_of(case["seq_lens_decoder"]),
                          np_of(case["cu_seqlens_q"]), hq, hkv, d, 1, quant)
    x = case["qkv"].float().view(16, 3, hq + 2 * hkv, d)
    wk = syn.quantize_ref(x[:, :, hq:hq + hkv], case["cache_k_scale"], quant).numpy()
    wv = syn.quantize_ref(x[:, :, hq + hkv:], case["cache_v_scale"], quant).numpy()
    for b in range(16):
        for i in range(3):
            p = int(case["seq_lens_decoder"][b]) + i
            blk, slot = int(case["block_tables"][b, p // 64]), p % 64
            assert np.array_equal(kc[blk, :, slot], wk[b, i])
            assert np.array_equal(vc[blk, :, slot], wv[b, i])


@pytest.mark.parametrize("quant", [CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC])
def test_writer_dynamic_formats_scale_and_bytes(oracle, quant):
    """One scale per stored row.  Without rotation: scale = numpy's max-abs / 127 (/ 448) of the row and the bytes
    are torch's x / scale -> round / clamp (-> e4m3 cast); the row's largest element maps to the largest code.
    With rotation: the bytes are those of the (pinned) per-channel writer run with the row's scale in every channel."""
    fmt = CACHE_INT8 if quant == CACHE_INT8_DYNAMIC else CACHE_FP8
    qmax = np.float32(127.0 if fmt == CACHE_INT8 else 448.0)
    case = syn.write_case(num_seqs=6, max_pos=300, seed=21, quant=quant, chunk=2)
    hq, hkv, d = case["hq"], case["hkv"], case["d"]
    args = (np_of(case["block_tables"]), np_of(case["seq_lens_decoder"]), np_of(case["cu_seqlens_q"]), hq, hkv, d, 1)
    # a row of zeros and a row with a NaN among the inputs
    qkv = case["qkv"].clone().view(12, hq + 2 * hkv, d)
    qkv[0, hq + 1] = 0
    qkv[1, hq + hkv + 2, 5] = float("nan")
    qkv = qkv.view(12, -1)
    kc, vc = np_of(case["key_cache"]).copy(), np_of(case["value_cache"]).copy()
    ks, vs = np_of(case["cache_k_scale"]).copy(), np_of(case["cache_v_scale"]).copy()
    ks0, vs0 = ks.copy(), vs.copy()
    oracle.write_cache_kv(bits(qkv), kc, vc, ks, vs, None, None, *args, quant)
    x = qkv.float().view(6, 2, hq + 2 * hkv, d).numpy()
    touched = np.zeros(ks.shape, bool)
    for b in range(6):
        for i in range(2):
            p = int(case["seq_lens_decoder"][b]) + i
            blk, slot = int(case["block_tables"][b, p // 64]), p % 64
            touched[blk, :, slot] = True
            for h in range(hkv):
                for row, cache, sc in ((x[b, i, hq + h], kc, ks), (x[b, i, hq + hkv + h], vc, vs)):
                    m = np.nanmax(np.abs(row)).astype(np.float32)
                    want_s = np.float32(m / qmax) if m > 0 else np.float32(1.0)
                    assert sc[blk, h, slot] == want_s
                    wb = syn.quantize_ref(torch.from_numpy(row), float(want_s), quant).numpy()
                    assert np.array_equal(cache[blk, h, slot], wb)
                    if m > 0:  # the largest element takes the largest code
                        top = cache[blk, h, slot][np.nanargmax(np.abs(row))]
                        assert (int(np.int8(top)) in (-127, 127)) if fmt == CACHE_INT8 else (top & 0x7F) == 0x7E
    assert np.array_equal(ks[~touched], ks0[~touched]) and np.array_equal(vs[~touched], vs0[~touched])
    assert ks[int(case["block_tables"][0, int(case["seq_lens_decoder"][0]) // 64]), 1, int(case["seq_lens_decoder"][0]) % 64] == 1.0
    # with rotation: token by token against the per-channel writer carrying that row's scale
    rope = (np_of(case["rope_cos"]), np_of(case["rope_sin"]))
    kc, vc = np_of(case["key_cache"]).copy(), np_of(case["value_cache"]).copy()
    oracle.write_cache_kv(bits(case["qkv"]), kc, vc, ks, vs, *rope, *args, quant)
    for b in range(6):
        p = int(case["seq_lens_decoder"][b])
        blk, slot = int(case["block_tables"][b, p // 64]), p % 64
        kc2, vc2 = np_of(case["key_cache"]).copy(), np_of(case["value_cache"]).copy()
        sk = np.repeat(ks[blk, :, slot][:, None], d, 1).astype(np.float32)
        sv = np.repeat(vs[blk, :, slot][:, None], d, 1).astype(np.float32)
        oracle.write_cache_kv(bits(case["qkv"]), kc2, vc2, sk, sv, *rope, *args, fmt)
        assert np.array_equal(kc[blk, :, slot], kc2[blk, :, slot]) and np.array_equal(vc[blk, :, slot], vc2[blk, :, slot])
        k8 = kc[blk, :, slot].view(np.int8) if fmt == CACHE_INT8 else kc[blk, :, slot] & 0x7F
        assert (np.abs(k8.astype(np.int32)).max(-1) == (127 if fmt == CACHE_INT8 else 0x7E)).all()


# ------------------------------------------------------------ decode attention

def _gather_dense(case, b):
    """Dequantised [ctx, hkv, d] K and V of sequence b in fp64 via the block table."""
    n = int(case["seq_lens_decoder"][b])
    nb = (n + case["bs"] - 1) // case["bs"]
    idx = case["block_tables"][b, :nb].long()
    if is_dynamic(case["quant"]):  # one scale per stored row: [pool, hkv, bs]
        sk, sv = case["cache_k_scale"][idx][..., None], case["cache_v_scale"][idx][..., None]
    else:
        sk, sv = case["cache_k_scale"][:, None, :], case["cache_v_scale"][:, None, :]
    k = syn.dequantize_ref(case["key_cache"][idx], sk, case["quant"])
    v = syn.dequantize_ref(case["value_cache"][idx], sv, case["quant"])
    k = k.permute(0, 2, 1, 3).reshape(nb * case["bs"], case["hkv"], case["d"])[:n].double()
    v = v.permute(0, 2, 1, 3).reshape(nb * case["bs"], case["hkv"], case["d"])[:n].double()
    return k, v


def _sdpa_decode(case):
    hq, hkv, d = case["hq"], case["hkv"], case["d"]
    outs = []
    for b in range(case["batch"]):
        k, v = _gather_dense(case, b)
        q = case["q"][b].double().view(hq, 1, d)
        kk = k.permute(1, 0, 2).repeat_interleave(hq // hkv, 0)
        vv = v.permute(1, 0, 2).repeat_interleave(hq // hkv, 0)
        outs.append(torch.nn.functional.scaled_dot_product_attention(q, kk, vv).view(hq * d))
    return torch.stack(outs)


def _decode(oracle, case, **kw):
    return oracle.decode_attention(bits(case["q"]), np_of(case["key_cache"]), np_of(case["value_cache"]),
                                   np_of(case["cache_k_scale"]), np_of(case["cache_v_scale"]),
                                   np_of(case["block_tables"]), np_of(case["seq_lens_decoder"]), case["hq"],
                                   case["hkv"], case["d"], case["quant"], **kw)


@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_FP8])
def test_decode_matches_torch_sdpa_fp64(oracle, quant):
    case = syn.decode_case(batch=3, ctx=[1, 63, 330], quant=quant, seed=1, extra_blocks=5)
    got = oracle.bf16_to_f32(_decode(oracle, case)).astype(np.float64)
    want = _sdpa_decode(case).numpy()
    assert_is_bf16_of(got, want)


@pytest.mark.parametrize("quant", [CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC])
def test_decode_dynamic_formats_match_sdpa_and_the_per_channel_path(oracle, quant):
    """Scales per stored row: fp64 SDPA on the dequantised cache (rows scaled over 2^-3 .. 2^3); and when every row
    of a head carries one scale, the result of the per-channel path with that scale in every channel."""
    case = syn.decode_case(batch=3, ctx=[1, 63, 330], quant=quant, seed=1, extra_blocks=5)
    got = oracle.bf16_to_f32(_decode(oracle, case)).astype(np.float64)
    assert_is_bf16_of(got, _sdpa_decode(case).numpy())
    fmt = CACHE_INT8 if quant == CACHE_INT8_DYNAMIC else CACHE_FP8
    stat = syn.decode_case(batch=2, ctx=[200, 77], quant=fmt, seed=3, extra_blocks=2, direct_bytes=True)
    dyn = dict(stat)
    dyn["quant"] = quant
    pool = stat["key_cache"].shape[0]
    head_k, head_v = stat["cache_k_scale"][:, 0], stat["cache_v_scale"][:, 0]
    stat["cache_k_scale"] = head_k[:, None].repeat(1, 128).contiguous()
    stat["cache_v_scale"] = head_v[:, None].repeat(1, 128).contiguous()
    dyn["cache_k_scale"] = head_k[None, :, None].repeat(pool, 1, 64).contiguous()
    dyn["cache_v_scale"] = head_v[None, :, None].repeat(pool, 1, 64).contiguous()
    a, b = _decode(oracle, stat), _decode(oracle, dyn)
    ok, mx, bad = bf16_close(b, a, atol=1e-4, rtol=2 ** -7)
    assert ok, (mx, bad)
    # sparse lists read the same scale rows
    kept = np.full((2, 8, 4), -1, np.int32)
    kept[0, :, :3] = [0, 2, 3]
    kept[1, :, :2] = [0, 1]
    cnt = np.array([[3] * 8, [2] * 8], np.int32)
    a, b = _decode(oracle, stat, kept_blocks=kept, kept_counts=cnt), _decode(oracle, dyn, kept_blocks=kept, kept_counts=cnt)
    ok, mx, bad = bf16_close(b, a, atol=1e-4, rtol=2 ** -7)
    assert ok, (mx, bad)


def test_decode_config1_shape_and_block_table_permutation_invariance(oracle):
    case = syn.decode_case(batch=4, ctx=1024, pool_blocks=64, seed=0)
    a = _decode(oracle, case)
    want = _sdpa_decode(case).numpy()
    assert_is_bf16_of(oracle.bf16_to_f32(a), want)
    # move every physical block somewhere else: the result must not change by a bit
    g = torch.Generator().manual_seed(9)
    perm = torch.randperm(64, generator=g)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(64)
    moved = dict(case)
    moved["key_cache"] = case["key_cache"][perm]
    moved["value_cache"] = case["value_cache"][perm]
    moved["block_tables"] = inv[case["block_tables"].long()].to(torch.int32)
    assert np.array_equal(a, _decode(oracle, moved))


def test_decode_special_cases(oracle):
    # ctx 1: the output is the dequantised V row
    case = syn.decode_case(batch=2, ctx=1, seed=2)
    out = oracle.bf16_to_f32(_decode(oracle, case)).reshape(2, 32, 128)
    for b in range(2):
        _, v = _gather_dense(case, b)
        want = v[0].repeat_interleave(4, 0).float().to(torch.bfloat16).float().numpy()
        assert np.array_equal(out[b], want)
    # constant K: uniform weights, output = mean of V
    case = syn.decode_case(batch=1, ctx=200, seed=4)
    case["key_cache"][:] = 3
    out = oracle.bf16_to_f32(_decode(oracle, case)).reshape(32, 128).astype(np.float64)
    _, v = _gather_dense(case, 0)
    want = v.mean(0).repeat_interleave(4, 0).numpy()
    assert_is_bf16_of(out, want)
    # kv_len 0: zeros
    case["seq_lens_decoder"][:] = 0
    assert not _decode(oracle, case).any()


def test_sparse_decode_with_all_blocks_equals_dense_and_subset_equals_sdpa(oracle):
    case = syn.decode_case(batch=2, ctx=[500, 640], seed=6)
    dense = _decode(oracle, case)
    nb = [8, 10]
    kept = np.full((2, 8, 10), -1, np.int32)
    cnt = np.zeros((2, 8), np.int32)
    for b in range(2):
        kept[b, :, :nb[b]] = np.arange(nb[b])
        cnt[b] = nb[b]
    assert np.array_equal(dense, _decode(oracle, case, kept_blocks=kept, kept_counts=cnt))
    # a hand-built selection equals attention over the kept tokens only
    sel = [[0, 3, 7], [1, 2, 9]]
    kept = np.full((2, 8, 3), -1, np.int32)
    for b in range(2):
        kept[b, :, :] = sel[b]
    cnt[:] = 3
    got = oracle.bf16_to_f32(_decode(oracle, case, kept_blocks=kept, kept_counts=cnt)).astype(np.float64)
    for b in range(2):
        k, v = _gather_dense(case, b)
        n = k.shape[0]
        tok = torch.cat([torch.arange(j * 64, min(j * 64 + 64, n)) for j in sel[b]])
        q = case["q"][b].double().view(32, 1, 128)
        kk = k[tok].permute(1, 0, 2).repeat_interleave(4, 0)
        vv = v[tok].permute(1, 0, 2).repeat_interleave(4, 0)
        want = torch.nn.functional.scaled_dot_product_attention(q, kk, vv).view(-1).numpy()
        assert_is_bf16_of(got[b], want)


def test_splitkv_combine_is_split_count_invariant(oracle):
    rng = np.random.default_rng(3)
    n, d = 448, 128
    logits = rng.standard_normal((5, n)).astype(np.float64) * 3
    v = rng.standard_normal((n, d)).astype(np.float64)
    p = np.exp(logits - logits.max(1, keepdims=True))
    want = (p @ v) / p.sum(1, keepdims=True)
    for splits in [1, 2, 7, 64]:
        edges = np.linspace(0, n, splits + 1).astype(int)
        po = np.zeros((5, splits, d), np.float32)
        pm = np.full((5, splits), -np.inf, np.float32)
        pl = np.zeros((5, splits), np.float32)
        for s in range(splits):
            lo, hi = edges[s], edges[s + 1]
            if hi == lo:
                continue
            m = logits[:, lo:hi].max(1)
            e = np.exp(logits[:, lo:hi] - m[:, None])
            pm[:, s], pl[:, s], po[:, s] = m, e.sum(1), e @ v[lo:hi]
        got = oracle.bf16_to_f32(oracle.splitkv_combine(po, pm, pl)).astype(np.float64)
        assert_is_bf16_of(got, want)
    # num_splits masks the tail slots
    po2 = np.concatenate([po, np.full_like(po, 1e9)], 1)
    pm2 = np.concatenate([pm, np.full_like(pm, 50.0)], 1)
    pl2 = np.concatenate([pl, np.ones_like(pl)], 1)
    got2 = oracle.splitkv_combine(po2, pm2, pl2, np.full(5, 64, np.int32))
    assert np.array_equal(got2, oracle.splitkv_combine(po, pm, pl))


# ------------------------------------------------------------------ selector

@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_FP8])
def test_block_scores_brute_force_fp64(oracle, quant):
    case = syn.decode_case(batch=2, ctx=[200, 130], quant=quant, seed=8, salient=0.3)
    s = oracle.sqattn_block_scores(bits(case["q"]), np_of(case["key_cache"]), np_of(case["cache_k_scale"]),
                                   np_of(case["block_tables"]), np_of(case["seq_lens_decoder"]), 32, 8, 128, quant)
    qs = (case["q"].float().view(2, 8, 4, 128) * case["cache_k_scale"][None, :, None, :]).double()   # one fp32 rounding
    for b in range(2):
        n = int(case["seq_lens_decoder"][b])
        for j in range(case["block_tables"].shape[1]):
            if j * 64 >= n:
                assert np.all(s[b, :, j] == -np.inf)
                continue
            blk = int(case["block_tables"][b, j])
            k8 = case["key_cache"][blk]
            kv = (k8.view(torch.int8) if quant == CACHE_INT8 else k8.view(torch.float8_e4m3fn)).double()   # [8,64,128]
            kv = kv[:, : min(64, n - j * 64)]
            dots = torch.einsum("hgc,htc->hgt", qs[b], kv)
            want = dots.amax((1, 2)).numpy()
            assert np.allclose(s[b, :, j], want, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("quant", [CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC])
def test_block_scores_dynamic_formats_brute_force_fp64(oracle, quant):
    """One scale per stored row: the block score is the largest, over the block's tokens and the group's heads, of
    (row scale) x (q . K8) - here by einsum in fp64 over rows whose scales differ by up to 2^6."""
    case = syn.decode_case(batch=2, ctx=[200, 130], quant=quant, seed=8, salient=0.3)
    s = oracle.sqattn_block_scores(bits(case["q"]), np_of(case["key_cache"]), np_of(case["cache_k_scale"]),
                                   np_of(case["block_tables"]), np_of(case["seq_lens_decoder"]), 32, 8, 128, quant)
    q = case["q"].double().view(2, 8, 4, 128)
    for b in range(2):
        n = int(case["seq_lens_decoder"][b])
        for j in range(case["block_tables"].shape[1]):
            if j * 64 >= n:
                assert np.all(s[b, :, j] == -np.inf)
                continue
            blk = int(case["block_tables"][b, j])
            k8 = case["key_cache"][blk]
            kv = (k8.view(torch.int8) if quant == CACHE_INT8_DYNAMIC else k8.view(torch.float8_e4m3fn)).double()
            nt = min(64, n - j * 64)
            dots = torch.einsum("hgc,htc->hgt", q[b], kv[:, :nt]) * case["cache_k_scale"][blk, :, None, :nt].double()
            assert np.allclose(s[b, :, j], dots.amax((1, 2)).numpy(), rtol=1e-12, atol=1e-12)


def test_topk_tie_rule_sort_vectors_and_torch(oracle):
    # ties resolve to the lowest index (fastdeploy/vision/utils/utils.h:41-60)
    sc = np.array([[[1.0, 5.0, 5.0, 2.0, 5.0, 0.0, 2.0, -1.0]]])
    kept, cnt = oracle.topk_select(sc, np.array([8 * 64], np.int32), 64, 2)
    assert kept[0, 0].tolist() == [1, 2] and cnt[0, 0] == 2
    kept, cnt = oracle.topk_select(sc, np.array([8 * 64], np.int32), 64, 4)
    assert kept[0, 0].tolist() == [1, 2, 3, 4]
    # fewer blocks than k: all of them, -1 padded; a partial last block counts
    kept, cnt = oracle.topk_select(sc, np.array([2 * 64 + 1], np.int32), 64, 5)
    assert kept[0, 0].tolist() == [0, 1, 2, -1, -1] and cnt[0, 0] == 3
    # the reference's sort vectors: top-k = the last k of its ascending order
    g = GOLD["sort_dim2"]
    x = np.array(g["input_2x3x4"], np.float64).reshape(6, 4)
    asc = np.array(g["ascending_indices"]).reshape(6, 4)
    for r in range(6):
        for k in (1, 2, 3):
            kept, _ = oracle.topk_select(x[r].reshape(1, 1, 4), np.array([4 * 64], np.int32), 64, k)
            assert sorted(kept[0, 0].tolist()) == sorted(asc[r, 4 - k:].tolist())
    # random scores with planted duplicates against a stable argsort
    rng = np.random.default_rng(5)
    s = rng.standard_normal((3, 8, 512))
    s[:, :, 100:140] = s[:, :, 300:340]
    kept, cnt = oracle.topk_select(s, np.full(3, 512 * 64, np.int32), 64, 64)
    for b in range(3):
        for h in range(8):
            order = np.argsort(-s[b, h], kind="stable")[:64]
            assert kept[b, h].tolist() == sorted(order.tolist())
            tk = torch.topk(torch.from_numpy(s[b, h]), 64).values.min().item()
            assert s[b, h][kept[b, h]].min() == tk


# ------------------------------------------------------------------- prefill

def _prefill_case(seed, batch, prefix, chunk, quant=CACHE_INT8):
    base = syn.decode_case(batch=batch, ctx=prefix, quant=quant, seed=seed, extra_blocks=batch * ((max(chunk) if isinstance(chunk, list) else chunk) // 64 + 2))
    g = torch.Generator().manual_seed(seed + 100)
    chunks = chunk if isinstance(chunk, list) else [chunk] * batch
    T = sum(chunks)
    base["q_new"] = torch.randn((T, 32 * 128), generator=g).to(torch.bfloat16)
    base["k_new"] = torch.randn((T, 8 * 128), generator=g).to(torch.bfloat16)
    base["v_new"] = torch.randn((T, 8 * 128), generator=g).to(torch.bfloat16)
    base["cu_seqlens_q"] = torch.tensor([0] + list(np.cumsum(chunks)), dtype=torch.int32)
    return base


def _prefill(oracle, c, **kw):
    return oracle.append_attention_prefill(bits(c["q_new"]), bits(c["k_new"]), bits(c["v_new"]), np_of(c["key_cache"]),
                                           np_of(c["value_cache"]), np_of(c["cache_k_scale"]), np_of(c["cache_v_scale"]),
                                           np_of(c["block_tables"]), np_of(c["seq_lens_decoder"]), np_of(c["cu_seqlens_q"]),
                                           32, 8, 128, c["quant"], **kw)


@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_FP8])
def test_prefill_matches_dense_causal_sdpa(oracle, quant):
    c = _prefill_case(2, 2, [70, 129], [33, 20], quant)
    got = oracle.bf16_to_f32(_prefill(oracle, c)).astype(np.float64)
    cu = c["cu_seqlens_q"].tolist()
    for b in range(2):
        kp, vp = _gather_dense(c, b)
        n, p = cu[b + 1] - cu[b], kp.shape[0]
        k = torch.cat([kp, c["k_new"][cu[b]:cu[b + 1]].double().view(n, 8, 128)]).permute(1, 0, 2).repeat_interleave(4, 0)
        v = torch.cat([vp, c["v_new"][cu[b]:cu[b + 1]].double().view(n, 8, 128)]).permute(1, 0, 2).repeat_interleave(4, 0)
        q = c["q_new"][cu[b]:cu[b + 1]].double().view(n, 32, 128).permute(1, 0, 2)
        mask = torch.arange(p + n)[None, :] <= (p + torch.arange(n))[:, None]
        want = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask).permute(1, 0, 2).reshape(n, -1)
        assert_is_bf16_of(got[cu[b]:cu[b + 1]], want.numpy())


@pytest.mark.parametrize("quant", [CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC])
def test_prefill_dynamic_formats_match_dense_causal_sdpa(oracle, quant):
    c = _prefill_case(4, 2, [70, 129], [33, 20], quant)
    got = oracle.bf16_to_f32(_prefill(oracle, c)).astype(np.float64)
    cu = c["cu_seqlens_q"].tolist()
    for b in range(2):
        kp, vp = _gather_dense(c, b)
        n, p = cu[b + 1] - cu[b], kp.shape[0]
        k = torch.cat([kp, c["k_new"][cu[b]:cu[b + 1]].double().view(n, 8, 128)]).permute(1, 0, 2).repeat_interleave(4, 0)
        v = torch.cat([vp, c["v_new"][cu[b]:cu[b + 1]].double().view(n, 8, 128)]).permute(1, 0, 2).repeat_interleave(4, 0)
        q = c["q_new"][cu[b]:cu[b + 1]].double().view(n, 32, 128).permute(1, 0, 2)
        mask = torch.arange(p + n)[None, :] <= (p + torch.arange(n))[:, None]
        want = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask).permute(1, 0, 2).reshape(n, -1)
        assert_is_bf16_of(got[cu[b]:cu[b + 1]], want.numpy(), extra=1e-3)


def test_prefill_row_subset_and_one_token_chunk_equals_decode(oracle):
    c = _prefill_case(3, 2, [100, 64], [5, 7])
    full = _prefill(oracle, c)
    ids = np.array([0, 4, 6, 11], np.int32)
    part = _prefill(oracle, c, token_ids=ids)
    assert np.array_equal(part[ids], full[ids]) and not np.delete(part, ids, 0).any()
    # a 1-token chunk: append == decode over a cache that holds prefix + the new token
    w = syn.write_case(num_seqs=3, max_pos=256, seed=13)
    kc, vc = np_of(w["key_cache"]).copy(), np_of(w["value_cache"]).copy()
    q, k, v = oracle.write_cache_kv(bits(w["qkv"]), kc, vc, np_of(w["cache_k_scale"]), np_of(w["cache_v_scale"]),
                                    np_of(w["rope_cos"]), np_of(w["rope_sin"]), np_of(w["block_tables"]),
                                    np_of(w["seq_lens_decoder"]), np_of(w["cu_seqlens_q"]), 32, 8, 128, 1, CACHE_INT8)
    dec = oracle.decode_attention(q, kc, vc, np_of(w["cache_k_scale"]), np_of(w["cache_v_scale"]), np_of(w["block_tables"]),
                                  np_of(w["seq_lens_decoder"]) + 1, 32, 8, 128, CACHE_INT8)
    # for the append path the new token's K/V are the *bf16* rows; decode reads their int8 versions:
    # they agree to the quantisation step, so compare loosely but element-wise
    app = oracle.append_attention_prefill(q, k, v, kc, vc, np_of(w["cache_k_scale"]), np_of(w["cache_v_scale"]),
                                          np_of(w["block_tables"]), np_of(w["seq_lens_decoder"]), np_of(w["cu_seqlens_q"]),
                                          32, 8, 128, CACHE_INT8)
    a = oracle.bf16_to_f32(app).astype(np.float64)
    d_ = oracle.bf16_to_f32(dec).astype(np.float64)
    assert np.abs(a - d_).max() < 0.05 and np.abs(a - d_).mean() < 3e-3


def test_prefill_chunking_invariance(oracle):
    """One 48-token chunk == two 24-token chunks when the first one's K/V sit in the prefix as bf16.
    With a quantised prefix the second call reads int8 versions of chunk 1, so the check uses the
    part that is exactly invariant: the first chunk's rows."""
    c = _prefill_case(4, 1, [128], [48])
    one = _prefill(oracle, c)
    c2 = dict(c)
    c2["q_new"], c2["k_new"], c2["v_new"] = c["q_new"][:24], c["k_new"][:24], c["v_new"][:24]
    c2["cu_seqlens_q"] = torch.tensor([0, 24], dtype=torch.int32)
    first = _prefill(oracle, c2)
    assert np.array_equal(one[:24], first)
