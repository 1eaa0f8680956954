"""ctypes front end of the CPU oracle (oracle/fdattn_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg, never by the fastdeploy_amd package.  All arrays
are numpy; bf16 tensors travel as uint16 bit patterns.  Parity status and what
pins each function are stated in the header of fdattn_oracle.c.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libfdattn_oracle.so")

CACHE_INT8 = 1
CACHE_FP8 = 2
CACHE_INT8_DYNAMIC = 3   # one scale per stored row: scale caches float32 [num_blocks, hkv, bs]
CACHE_FP8_DYNAMIC = 4
DYNAMIC = (CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC)


def build(force=False):
    """Compile the oracle with gcc (seconds)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "libfdattn_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.fdo_bf16_to_f32.restype = ctypes.c_float
        _lib.fdo_bf16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.fdo_f32_to_bf16.restype = ctypes.c_uint16
        _lib.fdo_f32_to_bf16.argtypes = [ctypes.c_float]
        _lib.fdo_e4m3_to_f32.restype = ctypes.c_float
        _lib.fdo_e4m3_to_f32.argtypes = [ctypes.c_uint8]
        _lib.fdo_f32_to_e4m3.restype = ctypes.c_uint8
        _lib.fdo_f32_to_e4m3.argtypes = [ctypes.c_float]
        _lib.fdo_quant_int8.restype = ctypes.c_int8
        _lib.fdo_quant_int8.argtypes = [ctypes.c_float, ctypes.c_float]
        _lib.fdo_quant_fp8.restype = ctypes.c_uint8
        _lib.fdo_quant_fp8.argtypes = [ctypes.c_float, ctypes.c_float]
        _lib.fdo_row_scale.restype = ctypes.c_float
        _lib.fdo_row_scale.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    if a is None:
        return None
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


# ----------------------------------------------------------------- scalars

def bf16_to_f32(bits):
    """uint16 bit patterns -> float32 (exact)."""
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(x):
    """float32 -> bf16 bit patterns, round to nearest even (vectorised twin of fdo_f32_to_bf16)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + (0x7FFF + ((u >> 16) & 1))) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def f32_to_e4m3(x):
    f = np.vectorize(lambda v: lib().fdo_f32_to_e4m3(float(v)), otypes=[np.uint8])
    return f(np.asarray(x, dtype=np.float32))


def e4m3_to_f32(c):
    table = np.array([lib().fdo_e4m3_to_f32(i) for i in range(256)], dtype=np.float32)
    return table[np.asarray(c, dtype=np.uint8)]


def quant_int8(x, scale):
    f = np.vectorize(lambda v, s: lib().fdo_quant_int8(float(v), float(s)), otypes=[np.int8])
    return f(np.asarray(x, dtype=np.float32), np.asarray(scale, dtype=np.float32))


def row_scale(x, cache_type):
    """The scale the dynamic formats store for the row x (float32 [d])."""
    x = _c(x, np.float32)
    return float(lib().fdo_row_scale(_p(x), x.size, cache_type))


def softmax_row(x):
    x = _c(x, np.float32)
    y = np.empty_like(x)
    lib().fdo_softmax_row(_p(x), _p(y), ctypes.c_int(x.size))
    return y


# ------------------------------------------------------------ cache writer

def write_cache_kv(qkv, key_cache, value_cache, k_scale, v_scale, rope_cos, rope_sin,
                   block_tables, seq_lens_decoder, cu_seqlens_q, hq, hkv, d, rope_style,
                   cache_type, want_kv_out=True, qkv_bias=None, q_norm_weight=None, k_norm_weight=None,
                   rms_norm_eps=0.0):
    """Mutates key_cache / value_cache (uint8 [num_blocks,hkv,bs,d]) in place - and, for the dynamic
    formats, k_scale / v_scale (float32 [num_blocks,hkv,bs]), which receive the stored rows' scales.

    qkv_bias: uint16 bf16 patterns [(hq+2hkv)*d]; q_norm_weight / k_norm_weight: float32 [d].
    Returns (q_out, k_out, v_out) as uint16 bf16 patterns.
    """
    qkv = _c(qkv, np.uint16)
    T = qkv.shape[0]
    assert key_cache.dtype == np.uint8 and key_cache.flags.c_contiguous
    assert value_cache.dtype == np.uint8 and value_cache.flags.c_contiguous
    num_blocks, _, bs, _ = key_cache.shape
    if cache_type in DYNAMIC:
        for sc in (k_scale, v_scale):
            assert sc.dtype == np.float32 and sc.flags.c_contiguous and sc.shape == (num_blocks, hkv, bs)
    k_scale, v_scale = _c(k_scale, np.float32), _c(v_scale, np.float32)
    rope_cos, rope_sin = _c(rope_cos, np.float32), _c(rope_sin, np.float32)
    bt = _c(block_tables, np.int32)
    dec = _c(seq_lens_decoder, np.int32)
    cu = _c(cu_seqlens_q, np.int32)
    batch, mb = bt.shape
    q_out = np.zeros((T, hq * d), np.uint16)
    k_out = np.zeros((T, hkv * d), np.uint16) if want_kv_out else None
    v_out = np.zeros((T, hkv * d), np.uint16) if want_kv_out else None
    max_pos = rope_cos.shape[0] if rope_cos is not None else 0
    bias = _c(qkv_bias, np.uint16) if qkv_bias is not None else None
    qw = _c(q_norm_weight, np.float32) if q_norm_weight is not None else None
    kw = _c(k_norm_weight, np.float32) if k_norm_weight is not None else None
    rc = lib().fdo_write_cache_kv_ex(
        _p(qkv), _p(q_out), _p(k_out), _p(v_out), _p(key_cache), _p(value_cache), _p(k_scale),
        _p(v_scale), _p(rope_cos), _p(rope_sin), _p(bt), _p(dec), _p(cu), T, batch, hq, hkv, d,
        bs, mb, num_blocks, max_pos, rope_style, cache_type, _p(bias), _p(qw), _p(kw),
        ctypes.c_float(rms_norm_eps))
    if rc != 0:
        raise ValueError("fdo_write_cache_kv: bad position or block id (%d)" % rc)
    return q_out, k_out, v_out


# ------------------------------------------------------------------ decode

def decode_attention(q, key_cache, value_cache, k_scale, v_scale, block_tables, kv_lens, hq, hkv,
                     d, cache_type, sm_scale=None, kept_blocks=None, kept_counts=None):
    """q uint16 [batch, hq*d] -> out uint16 [batch, hq*d]."""
    q = _c(q, np.uint16)
    bt = _c(block_tables, np.int32)
    kv = _c(kv_lens, np.int32)
    batch, mb = bt.shape
    bs = key_cache.shape[2]
    k_scale, v_scale = _c(k_scale, np.float32), _c(v_scale, np.float32)
    kb = _c(kept_blocks, np.int32)
    kc = _c(kept_counts, np.int32)
    max_kept = kb.shape[-1] if kb is not None else 0
    out = np.zeros((batch, hq * d), np.uint16)
    if sm_scale is None:
        sm_scale = 1.0 / np.sqrt(d)
    lib().fdo_decode_attention(
        _p(q), _p(key_cache), _p(value_cache), _p(k_scale), _p(v_scale), _p(bt), _p(kv), _p(kb),
        _p(kc), max_kept, _p(out), batch, hq, hkv, d, bs, mb, cache_type,
        ctypes.c_float(sm_scale))
    return out


def splitkv_combine(part_o, part_m, part_l, num_splits=None):
    part_o, part_m, part_l = _c(part_o, np.float32), _c(part_m, np.float32), _c(part_l, np.float32)
    rows, ms, d = part_o.shape
    ns = _c(num_splits, np.int32)
    out = np.zeros((rows, d), np.uint16)
    lib().fdo_splitkv_combine(_p(part_o), _p(part_m), _p(part_l), _p(ns), _p(out), rows, ms, d)
    return out


# ---------------------------------------------------------------- selector

def sqattn_block_scores(q, key_cache, k_scale, block_tables, kv_lens, hq, hkv, d, cache_type):
    q = _c(q, np.uint16)
    bt = _c(block_tables, np.int32)
    kv = _c(kv_lens, np.int32)
    batch, mb = bt.shape
    bs = key_cache.shape[2]
    k_scale = _c(k_scale, np.float32)
    scores = np.zeros((batch, hkv, mb), np.float64)
    lib().fdo_sqattn_block_scores(_p(q), _p(key_cache), _p(k_scale), _p(bt), _p(kv), _p(scores),
                                  batch, hq, hkv, d, bs, mb, cache_type)
    return scores


def topk_select(scores, kv_lens, bs, top_k):
    scores = _c(scores, np.float64)
    batch, hkv, mb = scores.shape
    kv = _c(kv_lens, np.int32)
    kept = np.zeros((batch, hkv, top_k), np.int32)
    counts = np.zeros((batch, hkv), np.int32)
    lib().fdo_topk_select(_p(scores), _p(kv), _p(kept), _p(counts), batch, hkv, bs, mb, top_k)
    return kept, counts


# ----------------------------------------------------------------- prefill

def append_attention_prefill(q, k_new, v_new, key_cache, value_cache, k_scale, v_scale,
                             block_tables, seq_lens_decoder, cu_seqlens_q, hq, hkv, d, cache_type,
                             sm_scale=None, token_ids=None):
    q, k_new, v_new = _c(q, np.uint16), _c(k_new, np.uint16), _c(v_new, np.uint16)
    bt = _c(block_tables, np.int32)
    dec = _c(seq_lens_decoder, np.int32)
    cu = _c(cu_seqlens_q, np.int32)
    batch, mb = bt.shape
    bs = key_cache.shape[2]
    T = q.shape[0]
    k_scale, v_scale = _c(k_scale, np.float32), _c(v_scale, np.float32)
    ids = _c(token_ids, np.int32)
    out = np.zeros((T, hq * d), np.uint16)
    if sm_scale is None:
        sm_scale = 1.0 / np.sqrt(d)
    lib().fdo_append_attention_prefill(
        _p(q), _p(k_new), _p(v_new), _p(key_cache), _p(value_cache), _p(k_scale), _p(v_scale),
        _p(bt), _p(dec), _p(cu), _p(out), _p(ids), 0 if ids is None else ids.size, T, batch, hq,
        hkv, d, bs, mb, cache_type, ctypes.c_float(sm_scale))
    return out
