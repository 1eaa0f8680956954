"""Python op surface of the paged-KV attention path.

Argument names follow FastDeploy's attention operator surface (qkv, key_cache,
value_cache, cache_k_scale, cache_v_scale, block_tables, seq_lens_encoder,
seq_lens_decoder, seq_lens_this_time).  Tensors cross into the library as
(address, shape, dtype) triples, the same contract as the reference's
FDTensor.from_external_data (fastdeploy/pybind/fd_tensor.cc:248-286); work is
enqueued on torch's current stream and nothing synchronises, as the reference's
custom operators do on their input's stream
(fastdeploy/runtime/backends/paddle/ops/voxelize_op.cu:287-351).  Bad arguments
raise ValueError where the reference's operators PD_THROW
(fastdeploy/runtime/backends/paddle/ops/voxelize_op.cc:172).
"""
import ctypes
import math

import torch

from . import _lib

CACHE_INT8 = 1
CACHE_FP8 = 2
# the same byte formats with one scale per stored row (token, KV head), computed by the cache writer:
# the scale tensors are then float32 [num_blocks, kv_num_heads, block_size] and the writer fills them
CACHE_INT8_DYNAMIC = 3
CACHE_FP8_DYNAMIC = 4
# the same byte formats with one scale per (block, KV head) tile, kept by the cache writer at the largest magnitude
# stored in the tile: the scale tensors are float32 [num_blocks, kv_num_heads]
CACHE_INT8_BLOCK = 5
CACHE_FP8_BLOCK = 6
_QUANT = {"cache_int8": CACHE_INT8, "int8": CACHE_INT8, CACHE_INT8: CACHE_INT8,
          "cache_fp8": CACHE_FP8, "fp8": CACHE_FP8, "fp8_e4m3": CACHE_FP8, CACHE_FP8: CACHE_FP8,
          "cache_int8_dynamic": CACHE_INT8_DYNAMIC, CACHE_INT8_DYNAMIC: CACHE_INT8_DYNAMIC,
          "cache_fp8_dynamic": CACHE_FP8_DYNAMIC, CACHE_FP8_DYNAMIC: CACHE_FP8_DYNAMIC,
          "cache_int8_block": CACHE_INT8_BLOCK, CACHE_INT8_BLOCK: CACHE_INT8_BLOCK,
          "cache_fp8_block": CACHE_FP8_BLOCK, CACHE_FP8_BLOCK: CACHE_FP8_BLOCK}


def is_blockwise(cache_quant_type):
    """True for the formats that carry one scale per (block, KV head) tile."""
    return _QUANT.get(cache_quant_type) in (CACHE_INT8_BLOCK, CACHE_FP8_BLOCK)


def is_dynamic(cache_quant_type):
    """True for the formats whose scales the cache writer computes and stores in scale caches beside the rows:
    one per stored row, or one per tile (is_blockwise)."""
    return _QUANT.get(cache_quant_type) in (CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC, CACHE_INT8_BLOCK, CACHE_FP8_BLOCK)


def scale_cache_shape(cache_quant_type, num_blocks, kv_num_heads, block_size):
    """Shape of cache_k_scale / cache_v_scale for a format with scale caches."""
    if is_blockwise(cache_quant_type):
        return (num_blocks, kv_num_heads)
    return (num_blocks, kv_num_heads, block_size)


def byte_format(cache_quant_type):
    """CACHE_INT8 or CACHE_FP8: how the cache bytes of this format are encoded."""
    q = _QUANT[cache_quant_type]
    return {CACHE_INT8_DYNAMIC: CACHE_INT8, CACHE_FP8_DYNAMIC: CACHE_FP8,
            CACHE_INT8_BLOCK: CACHE_INT8, CACHE_FP8_BLOCK: CACHE_FP8}.get(q, q)


_ROPE = {"interleaved": 0, 0: 0, False: 0, "neox": 1, 1: 1, True: 1}


def _quant(t):
    if t not in _QUANT:
        raise ValueError("unknown cache_quant_type %r (cache_int8 | cache_fp8 | cache_int8_dynamic | cache_fp8_dynamic | "
                         "cache_int8_block | cache_fp8_block)" % (t,))
    return _QUANT[t]


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _chk(t, name, dtypes, ndim=None, optional=False):
    if t is None:
        if optional:
            return 0
        raise ValueError("%s is required" % name)
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise ValueError("%s must be a CUDA/HIP tensor" % name)
    if not isinstance(dtypes, (tuple, list)):
        dtypes = (dtypes,)
    if t.dtype not in dtypes:
        raise ValueError("%s has dtype %s, expected %s" % (name, t.dtype, "/".join(map(str, dtypes))))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)
    if ndim is not None and t.dim() != ndim:
        raise ValueError("%s must have %d dimensions, has shape %s" % (name, ndim, tuple(t.shape)))
    return t.data_ptr()


_CACHE_DT = (torch.int8, torch.uint8, torch.float8_e4m3fn)


def _cache_dims(key_cache, value_cache):
    if key_cache.shape != value_cache.shape:
        raise ValueError("key_cache %s and value_cache %s differ in shape" %
                         (tuple(key_cache.shape), tuple(value_cache.shape)))
    return key_cache.shape  # num_blocks, hkv, block_size, head_dim


def _scales(cache_k_scale, cache_v_scale, hkv, d, quant=CACHE_INT8, nb=0, bs=0):
    pk = _chk(cache_k_scale, "cache_k_scale", torch.float32)
    pv = _chk(cache_v_scale, "cache_v_scale", torch.float32)
    if is_blockwise(quant):
        if cache_k_scale.numel() != nb * hkv or cache_v_scale.numel() != nb * hkv:
            raise ValueError("the per-block formats' cache scales must hold num_blocks*kv_num_heads = %d values"
                             % (nb * hkv))
    elif is_dynamic(quant):
        if cache_k_scale.numel() != nb * hkv * bs or cache_v_scale.numel() != nb * hkv * bs:
            raise ValueError("the dynamic formats' cache scales must hold num_blocks*kv_num_heads*block_size = %d "
                             "values" % (nb * hkv * bs))
    elif cache_k_scale.numel() != hkv * d or cache_v_scale.numel() != hkv * d:
        raise ValueError("cache scales must hold kv_num_heads*head_dim = %d values" % (hkv * d))
    return pk, pv


def _extras(qkv_bias, q_norm_weight, k_norm_weight, rms_norm_eps, width, d, prefill_rows=0, sqattn_top_k=0,
            decode_tokens=0, sqattn_per_token=False):
    """fdattn_step_extras for the optional projection epilogue / prefill splits / block-sparse decode rows / decode
    rows of several tokens, or None"""
    if (qkv_bias is None and q_norm_weight is None and k_norm_weight is None and prefill_rows <= 0
            and sqattn_top_k <= 0 and decode_tokens <= 1):
        return None
    pb = _chk(qkv_bias, "qkv_bias", torch.bfloat16, 1, optional=True)
    if qkv_bias is not None and qkv_bias.numel() != width:
        raise ValueError("qkv_bias has %d entries, qkv %d columns" % (qkv_bias.numel(), width))
    pq = _chk(q_norm_weight, "q_norm_weight", torch.float32, 1, optional=True)
    pk = _chk(k_norm_weight, "k_norm_weight", torch.float32, 1, optional=True)
    for name, t in (("q_norm_weight", q_norm_weight), ("k_norm_weight", k_norm_weight)):
        if t is not None and t.numel() != d:
            raise ValueError("%s has %d entries, head_dim is %d" % (name, t.numel(), d))
    return _lib.StepExtras(pb or None, pq or None, pk or None, float(rms_norm_eps), int(prefill_rows), int(sqattn_top_k),
                           int(decode_tokens), 1 if sqattn_per_token else 0)


def prefill_auto_splits(rows, num_heads, max_chunk, kv_num_heads=None):
    """How many key splits fill the GPU when `rows` sequences bring at most max_chunk new tokens each (1..8)."""
    if kv_num_heads:
        return _lib.lib().fdattn_prefill_auto_splits_for(int(rows), int(num_heads), int(kv_num_heads), int(max_chunk))
    return _lib.lib().fdattn_prefill_auto_splits(int(rows), int(num_heads), int(max_chunk))


def seq_lens_this_time_of(seq_lens_encoder, seq_lens_decoder):
    """Tokens each sequence brings this step: its chunk length for a prefill row
    (seq_lens_encoder > 0), one for a decode row (seq_lens_decoder > 0), else none."""
    one = (seq_lens_decoder > 0).to(torch.int32)
    return torch.where(seq_lens_encoder > 0, seq_lens_encoder, one).to(torch.int32)


def cu_seqlens_of(seq_lens_this_time):
    cu = torch.zeros(seq_lens_this_time.numel() + 1, dtype=torch.int32, device=seq_lens_this_time.device)
    cu[1:] = torch.cumsum(seq_lens_this_time, 0)
    return cu


def write_cache_kv(qkv, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                   seq_lens_encoder, seq_lens_decoder, seq_lens_this_time=None, cu_seqlens_q=None,
                   rotary_embs=None, *, num_heads, kv_num_heads, rope_style="neox",
                   cache_quant_type="cache_int8", want_kv_out=False, qkv_bias=None, q_norm_weight=None,
                   k_norm_weight=None, rms_norm_eps=1e-6):
    """RoPE on Q/K, quantise K/V into their block-tabled cache slots (in place).

    rotary_embs = (cos, sin) float32 [max_pos, head_dim/2] from rope_table(), or None.
    The projection's epilogue, all optional: qkv_bias bf16 [(num_heads+2*kv_num_heads)*head_dim]
    (x = bf16(x + bias)), q_norm_weight / k_norm_weight float32 [head_dim] (RMS norm of every Q / K
    head before the rotation, with rms_norm_eps).
    Returns (q_out, k_out, v_out); k_out / v_out are None unless want_kv_out.
    """
    nb, hkv, bs, d = _cache_dims(key_cache, value_cache)
    if hkv != kv_num_heads:
        raise ValueError("cache holds %d KV heads, kv_num_heads=%d" % (hkv, kv_num_heads))
    p_qkv = _chk(qkv, "qkv", torch.bfloat16, 2)
    T = qkv.shape[0]
    if qkv.shape[1] != (num_heads + 2 * hkv) * d:
        raise ValueError("qkv has %d columns, expected (num_heads+2*kv_num_heads)*head_dim = %d" %
                         (qkv.shape[1], (num_heads + 2 * hkv) * d))
    p_kc = _chk(key_cache, "key_cache", _CACHE_DT, 4)
    p_vc = _chk(value_cache, "value_cache", _CACHE_DT, 4)
    p_ks, p_vs = _scales(cache_k_scale, cache_v_scale, hkv, d, cache_quant_type, nb, bs)
    p_bt = _chk(block_tables, "block_tables", torch.int32, 2)
    batch, mb = block_tables.shape
    p_dec = _chk(seq_lens_decoder, "seq_lens_decoder", torch.int32, 1)
    if seq_lens_decoder.numel() != batch:
        raise ValueError("seq_lens_decoder has %d entries, block_tables %d rows" % (seq_lens_decoder.numel(), batch))
    if cu_seqlens_q is None:
        if seq_lens_this_time is None:
            _chk(seq_lens_encoder, "seq_lens_encoder", torch.int32, 1)
            seq_lens_this_time = seq_lens_this_time_of(seq_lens_encoder, seq_lens_decoder)
        _chk(seq_lens_this_time, "seq_lens_this_time", torch.int32, 1)
        cu_seqlens_q = cu_seqlens_of(seq_lens_this_time)
    p_cu = _chk(cu_seqlens_q, "cu_seqlens_q", torch.int32, 1)
    if cu_seqlens_q.numel() != batch + 1:
        raise ValueError("cu_seqlens_q must have batch+1 entries")
    p_cos = p_sin = 0
    max_pos = 0
    if rotary_embs is not None:
        cos, sin = rotary_embs
        p_cos = _chk(cos, "rotary cos", torch.float32, 2)
        p_sin = _chk(sin, "rotary sin", torch.float32, 2)
        if cos.shape != sin.shape or cos.shape[1] != d // 2:
            raise ValueError("rotary table must be [max_pos, head_dim/2]")
        max_pos = cos.shape[0]
    if rope_style not in _ROPE:
        raise ValueError("unknown rope_style %r (neox | interleaved)" % (rope_style,))
    q_out = torch.empty((T, num_heads * d), dtype=torch.bfloat16, device=qkv.device)
    k_out = v_out = None
    if want_kv_out:
        k_out = torch.empty((T, hkv * d), dtype=torch.bfloat16, device=qkv.device)
        v_out = torch.empty((T, hkv * d), dtype=torch.bfloat16, device=qkv.device)
    ep = _extras(qkv_bias, q_norm_weight, k_norm_weight, rms_norm_eps, qkv.shape[1], d)
    rc = _lib.lib().fdattn_write_cache_kv_ex(
        p_qkv, q_out.data_ptr(), k_out.data_ptr() if want_kv_out else 0,
        v_out.data_ptr() if want_kv_out else 0, p_kc, p_vc, p_ks, p_vs, p_cos, p_sin, p_bt, p_dec,
        p_cu, T, batch, num_heads, hkv, d, bs, mb, nb, max_pos, _ROPE[rope_style],
        _quant(cache_quant_type), ctypes.addressof(ep) if ep is not None else None, _stream())
    _lib.check(rc, "write_cache_kv")
    return q_out, k_out, v_out


def decode_workspace(batch, num_heads, kv_num_heads, head_dim, max_blocks_per_seq, device="cuda"):
    """A workspace tensor large enough for decode_attention(_sparse) at these shapes."""
    n = _lib.lib().fdattn_decode_workspace_bytes(batch, num_heads, kv_num_heads, head_dim, max_blocks_per_seq)
    return torch.empty(n, dtype=torch.uint8, device=device)


def decode_uses_mfma(num_heads, kv_num_heads, head_dim, block_size, cache_quant_type="cache_int8"):
    """True if decode_attention runs these shapes on the MFMA kernel."""
    return bool(_lib.lib().fdattn_decode_uses_mfma(num_heads, kv_num_heads, head_dim, block_size,
                                                   _quant(cache_quant_type)))


def _decode_common(q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                   seq_lens_decoder, seq_lens_this_time, num_heads, out, workspace, cache_quant_type):
    nb, hkv, bs, d = _cache_dims(key_cache, value_cache)
    p_q = _chk(q, "q", torch.bfloat16)
    batch, mb = block_tables.shape
    if q.numel() != batch * num_heads * d:
        raise ValueError("q holds %d values, expected batch*num_heads*head_dim = %d" %
                         (q.numel(), batch * num_heads * d))
    p_kc = _chk(key_cache, "key_cache", _CACHE_DT, 4)
    p_vc = _chk(value_cache, "value_cache", _CACHE_DT, 4)
    p_ks, p_vs = _scales(cache_k_scale, cache_v_scale, hkv, d, cache_quant_type, nb, bs)
    p_bt = _chk(block_tables, "block_tables", torch.int32, 2)
    p_dec = _chk(seq_lens_decoder, "seq_lens_decoder", torch.int32, 1)
    p_tt = _chk(seq_lens_this_time, "seq_lens_this_time", torch.int32, 1, optional=True)
    if seq_lens_decoder.numel() != batch:
        raise ValueError("seq_lens_decoder has %d entries, block_tables %d rows" % (seq_lens_decoder.numel(), batch))
    if out is None:
        out = torch.empty((batch, num_heads * d), dtype=torch.bfloat16, device=q.device)
    p_out = _chk(out, "out", torch.bfloat16)
    if workspace is None:
        workspace = decode_workspace(batch, num_heads, hkv, d, mb, q.device)
    p_ws = _chk(workspace, "workspace", torch.uint8)
    return (p_q, p_kc, p_vc, p_ks, p_vs, p_bt, p_dec, p_tt), out, p_out, p_ws, workspace, \
        (batch, num_heads, hkv, d, bs, mb, nb)


def decode_attention(q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                     seq_lens_decoder, seq_lens_this_time=None, *, num_heads,
                     cache_quant_type="cache_int8", softmax_scale=None, out=None, workspace=None,
                     impl="auto"):
    """One query token per sequence against kv_len = seq_lens_decoder (+ seq_lens_this_time)
    cached tokens.  q bf16 [batch, num_heads*head_dim] -> out bf16 of the same shape.
    impl: "auto" (the int8-MFMA kernel at head_dim 128 / block_size 64, the fp16-MFMA kernel at head_dim 64 / 128 / 256
    with any block size, else the vector-ALU kernel), "tiles" (the second of these at any of its shapes) or "generic"
    (the last)."""
    ptrs, out, p_out, p_ws, workspace, dims = _decode_common(
        q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables, seq_lens_decoder,
        seq_lens_this_time, num_heads, out, workspace, cache_quant_type)
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(dims[3])
    if impl in ("generic", "tiles"):
        fn = _lib.lib().fdattn_decode_attention_generic if impl == "generic" else _lib.lib().fdattn_decode_attention_tiles
        rc = fn(*ptrs, 0, 0, 0, p_out, p_ws, workspace.numel(), *dims, _quant(cache_quant_type), scale, _stream())
    elif impl == "auto":
        rc = _lib.lib().fdattn_decode_attention(
            *ptrs, p_out, p_ws, workspace.numel(), *dims, _quant(cache_quant_type), scale, _stream())
    elif impl in ("partials", "merge"):   # the two kernels of the MFMA path, one at a time
        rc = _lib.lib().fdattn_decode_attention_stages(
            *ptrs, p_out, p_ws, workspace.numel(), *dims, _quant(cache_quant_type), scale,
            1 if impl == "partials" else 2, _stream())
    else:
        raise ValueError("impl must be auto, generic, tiles, partials or merge")
    _lib.check(rc, "decode_attention")
    return out


def decode_attention_noalloc(q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                             seq_lens_decoder, seq_lens_this_time=None, *, num_heads, out,
                             cache_quant_type="cache_int8", softmax_scale=None):
    """decode_attention through the entry point that allocates nothing: no workspace tensor, the split-KV
    partials live in the library's own 16 MiB device array (shared by every call on the GPU: calls that
    overlap there race).  `out` must be passed.  Shapes that need more scratch raise ValueError."""
    if out is None:
        raise ValueError("out is required")
    nb, hkv, bs, d = _cache_dims(key_cache, value_cache)
    p_q = _chk(q, "q", torch.bfloat16)
    batch, mb = block_tables.shape
    if q.numel() != batch * num_heads * d or out.numel() != q.numel():
        raise ValueError("q and out must hold batch*num_heads*head_dim = %d values" % (batch * num_heads * d))
    p_kc = _chk(key_cache, "key_cache", _CACHE_DT, 4)
    p_vc = _chk(value_cache, "value_cache", _CACHE_DT, 4)
    p_ks, p_vs = _scales(cache_k_scale, cache_v_scale, hkv, d, cache_quant_type, nb, bs)
    p_bt = _chk(block_tables, "block_tables", torch.int32, 2)
    p_dec = _chk(seq_lens_decoder, "seq_lens_decoder", torch.int32, 1)
    p_tt = _chk(seq_lens_this_time, "seq_lens_this_time", torch.int32, 1, optional=True)
    if seq_lens_decoder.numel() != batch:
        raise ValueError("seq_lens_decoder has %d entries, block_tables %d rows" % (seq_lens_decoder.numel(), batch))
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(d)
    rc = _lib.lib().fdattn_decode_attention_noalloc(
        p_q, p_kc, p_vc, p_ks, p_vs, p_bt, p_dec, p_tt, _chk(out, "out", torch.bfloat16), batch, num_heads, hkv, d,
        bs, mb, nb, _quant(cache_quant_type), scale, _stream())
    _lib.check(rc, "decode_attention_noalloc")
    return out


def decode_attention_sparse(q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                            seq_lens_decoder, seq_lens_this_time=None, *, kept_blocks, kept_counts,
                            num_heads, cache_quant_type="cache_int8", softmax_scale=None, out=None,
                            workspace=None, impl="auto"):
    """decode_attention restricted to kept_blocks int32 [batch, kv_num_heads, max_kept]
    (ascending logical block indices) / kept_counts int32 [batch, kv_num_heads]."""
    ptrs, out, p_out, p_ws, workspace, dims = _decode_common(
        q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables, seq_lens_decoder,
        seq_lens_this_time, num_heads, out, workspace, cache_quant_type)
    batch, _, hkv = dims[0], dims[1], dims[2]
    p_kb = _chk(kept_blocks, "kept_blocks", torch.int32, 3)
    p_kn = _chk(kept_counts, "kept_counts", torch.int32, 2)
    if kept_blocks.shape[:2] != (batch, hkv) or kept_counts.shape != (batch, hkv):
        raise ValueError("kept_blocks must be [batch, kv_num_heads, max_kept], kept_counts [batch, kv_num_heads]")
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(dims[3])
    if impl not in ("auto", "generic", "tiles"):
        raise ValueError("impl must be auto, generic or tiles")
    fn = {"auto": _lib.lib().fdattn_decode_attention_sparse, "generic": _lib.lib().fdattn_decode_attention_generic,
          "tiles": _lib.lib().fdattn_decode_attention_tiles}[impl]
    rc = fn(*ptrs, p_kb, p_kn, kept_blocks.shape[2], p_out, p_ws, workspace.numel(), *dims,
            _quant(cache_quant_type), scale, _stream())
    _lib.check(rc, "decode_attention_sparse")
    return out


def splitkv_combine(part_o, part_m, part_l, num_splits=None, out=None):
    """Merge split-KV partials: part_o f32 [rows, splits, d], part_m / part_l f32 [rows, splits]."""
    p_o = _chk(part_o, "part_o", torch.float32, 3)
    p_m = _chk(part_m, "part_m", torch.float32, 2)
    p_l = _chk(part_l, "part_l", torch.float32, 2)
    rows, ms, d = part_o.shape
    if part_m.shape != (rows, ms) or part_l.shape != (rows, ms):
        raise ValueError("part_m / part_l must be [rows, splits]")
    p_n = _chk(num_splits, "num_splits", torch.int32, 1, optional=True)
    if out is None:
        out = torch.empty((rows, d), dtype=torch.bfloat16, device=part_o.device)
    rc = _lib.lib().fdattn_splitkv_combine(p_o, p_m, p_l, p_n, _chk(out, "out", torch.bfloat16), rows, ms, d, _stream())
    _lib.check(rc, "splitkv_combine")
    return out


def sqattn_select(q, key_cache, cache_k_scale, block_tables, seq_lens_decoder, seq_lens_this_time=None, *,
                  num_heads, top_k, cache_quant_type="cache_fp8", return_scores=False, workspace=None, impl="auto"):
    """SQAttn block selection: per (sequence, KV head) the top_k blocks by block-max q.k score.
    Returns (kept_blocks int32 [batch, hkv, top_k], kept_counts int32 [batch, hkv][, scores f32])."""
    nb, hkv, bs, d = key_cache.shape
    p_q = _chk(q, "q", torch.bfloat16)
    p_kc = _chk(key_cache, "key_cache", _CACHE_DT, 4)
    p_ks = _chk(cache_k_scale, "cache_k_scale", torch.float32)
    p_bt = _chk(block_tables, "block_tables", torch.int32, 2)
    batch, mb = block_tables.shape
    p_dec = _chk(seq_lens_decoder, "seq_lens_decoder", torch.int32, 1)
    p_tt = _chk(seq_lens_this_time, "seq_lens_this_time", torch.int32, 1, optional=True)
    if q.numel() != batch * num_heads * d:
        raise ValueError("q holds %d values, expected %d" % (q.numel(), batch * num_heads * d))
    if top_k <= 0:
        raise ValueError("top_k must be positive")
    kept = torch.empty((batch, hkv, top_k), dtype=torch.int32, device=q.device)
    counts = torch.empty((batch, hkv), dtype=torch.int32, device=q.device)
    scores = torch.empty((batch, hkv, mb), dtype=torch.float32, device=q.device) if return_scores else None
    if workspace is None:
        n = _lib.lib().fdattn_sqattn_workspace_bytes(batch, hkv, mb)
        workspace = torch.empty(n, dtype=torch.uint8, device=q.device)
    fn = _lib.lib().fdattn_sqattn_select if impl == "auto" else _lib.lib().fdattn_sqattn_select_exact
    rc = fn(
        p_q, p_kc, p_ks, p_bt, p_dec, p_tt, scores.data_ptr() if return_scores else 0, kept.data_ptr(),
        counts.data_ptr(), _chk(workspace, "workspace", torch.uint8), workspace.numel(), batch, num_heads,
        hkv, d, bs, mb, nb, top_k, _quant(cache_quant_type), _stream())
    _lib.check(rc, "sqattn_select")
    return (kept, counts, scores) if return_scores else (kept, counts)


def append_attention_prefill(q, k_new, v_new, key_cache, value_cache, cache_k_scale, cache_v_scale,
                             block_tables, seq_lens_decoder, cu_seqlens_q, *, num_heads, max_chunk,
                             cache_quant_type="cache_int8", softmax_scale=None, out=None, impl="auto",
                             num_splits=None, workspace=None):
    """Chunked prefill: the chunk's tokens attend to the cached prefix (quantised pages)
    and causally to the chunk itself (bf16 k_new / v_new).
    num_splits: workgroups that share one query tile's keys (None: as many as fill the GPU when the
    batch's query tiles alone would not, 1: none); partials go to `workspace` (allocated if None).
    impl: "auto" (the MFMA kernel of the shape: head_dim 128 / block_size 64, or head_dim 64 / 128 / 256 at any
    block size; else the shape-agnostic kernel), "tiles" (the second of these at any of its shapes) or "generic"."""
    nb, hkv, bs, d = _cache_dims(key_cache, value_cache)
    p_q = _chk(q, "q", torch.bfloat16, 2)
    p_k = _chk(k_new, "k_new", torch.bfloat16, 2)
    p_v = _chk(v_new, "v_new", torch.bfloat16, 2)
    T = q.shape[0]
    if q.shape[1] != num_heads * d or k_new.shape != (T, hkv * d) or v_new.shape != (T, hkv * d):
        raise ValueError("q must be [T, num_heads*head_dim], k_new / v_new [T, kv_num_heads*head_dim]")
    p_kc = _chk(key_cache, "key_cache", _CACHE_DT, 4)
    p_vc = _chk(value_cache, "value_cache", _CACHE_DT, 4)
    p_ks, p_vs = _scales(cache_k_scale, cache_v_scale, hkv, d, cache_quant_type, nb, bs)
    p_bt = _chk(block_tables, "block_tables", torch.int32, 2)
    batch, mb = block_tables.shape
    p_dec = _chk(seq_lens_decoder, "seq_lens_decoder", torch.int32, 1)
    p_cu = _chk(cu_seqlens_q, "cu_seqlens_q", torch.int32, 1)
    if cu_seqlens_q.numel() != batch + 1:
        raise ValueError("cu_seqlens_q must have batch+1 entries")
    if out is None:
        out = torch.empty((T, num_heads * d), dtype=torch.bfloat16, device=q.device)
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(d)
    if impl == "auto":
        if num_splits is None:
            num_splits = prefill_auto_splits(batch, num_heads, max_chunk)
        p_ws = n_ws = 0
        if num_splits > 1:
            need = _lib.lib().fdattn_append_attention_prefill_split_workspace_bytes(T, num_heads, num_splits)
            if workspace is None:
                workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
            p_ws, n_ws = _chk(workspace, "workspace", torch.uint8), workspace.numel()
        rc = _lib.lib().fdattn_append_attention_prefill_split(
            p_q, p_k, p_v, p_kc, p_vc, p_ks, p_vs, p_bt, p_dec, p_cu, _chk(out, "out", torch.bfloat16), p_ws or None,
            n_ws, num_splits, T, batch, max_chunk, num_heads, hkv, d, bs, mb, nb, _quant(cache_quant_type), scale,
            _stream())
    else:
        if impl not in ("generic", "tiles"):
            raise ValueError("impl must be auto, generic or tiles")
        fn = _lib.lib().fdattn_append_attention_prefill_generic if impl == "generic" else _lib.lib().fdattn_append_attention_prefill_tiles
        rc = fn(
            p_q, p_k, p_v, p_kc, p_vc, p_ks, p_vs, p_bt, p_dec, p_cu, _chk(out, "out", torch.bfloat16), T, batch,
            max_chunk, num_heads, hkv, d, bs, mb, nb, _quant(cache_quant_type), scale, _stream())
    _lib.check(rc, "append_attention_prefill")
    return out


def append_attention_workspace_bytes(num_tokens, batch, num_heads, kv_heads, head_dim, max_blocks_per_seq,
                                     prefill_splits=1):
    return _lib.lib().fdattn_append_attention_workspace_bytes_ex(num_tokens, batch, num_heads, kv_heads, head_dim,
                                                                max_blocks_per_seq, prefill_splits)


def append_attention_workspace(num_tokens, batch, num_heads, kv_heads, head_dim, max_blocks_per_seq, device="cuda",
                               prefill_splits=1):
    """A workspace tensor large enough for append_attention at these shapes."""
    n = append_attention_workspace_bytes(num_tokens, batch, num_heads, kv_heads, head_dim, max_blocks_per_seq,
                                         prefill_splits)
    return torch.empty(n, dtype=torch.uint8, device=device)


def append_attention(qkv, key_cache, value_cache, seq_lens_encoder, seq_lens_decoder, seq_lens_this_time,
                     block_tables, rotary_embs, cache_k_scale, cache_v_scale, *, num_heads, kv_num_heads,
                     max_chunk, rope_style="neox", cache_quant_type="cache_int8", softmax_scale=None,
                     cu_seqlens_q=None, workspace=None, out=None, qkv_bias=None, q_norm_weight=None,
                     k_norm_weight=None, rms_norm_eps=1e-6, prefill_rows=None, sqattn_top_k=None,
                     decode_tokens=None, sqattn_per_token=False):
    """One attention step of a layer over a mixed batch (one call into the library):
    every new token is rotated and written to the cache, decode rows (one token,
    seq_lens_encoder == 0) attend to the cache, prefill rows (seq_lens_encoder > 0)
    to their cached prefix and causally to their own chunk; slots without a token
    are skipped.  max_chunk bounds the tokens of a prefill row (0: the step has none, decode only).
    qkv_bias / q_norm_weight / k_norm_weight / rms_norm_eps: the projection's epilogue, as in write_cache_kv.
    prefill_rows: how many sequences of the step have seq_lens_encoder > 0, if the host knows (None: unknown).  A
    promise, not a guess - the prefill pass then covers that many prefill rows only (no workgroups for decode rows),
    and when they alone would leave CUs idle every query tile is shared by prefill_auto_splits(prefill_rows,
    num_heads, max_chunk, kv_num_heads) workgroups (as many as a workspace passed in has room for).  Without it the
    prefill pass covers the whole batch, counts the prefill rows on the GPU and shares the query tiles as that count
    asks, given a workspace with room for the splits of a single prefill row (the one allocated here has it).
    sqattn_top_k: > 0 makes the decode rows block-sparse - the selector keeps that many blocks per (row, KV head),
    scored with the row's new query, and the decode attention reads only those (the MFMA selector at its shapes,
    the exact fp64 selector elsewhere).
    decode_tokens: > 1 makes rows with seq_lens_encoder 0 and up to that many tokens (speculative drafts) decode rows:
    token t attends to the cached tokens and the new ones up to itself, all read from the cache, in one decode pass
    (head_dim 64 / 128 / 256, decode_tokens x heads per KV head <= 16).  With sqattn_top_k such a row keeps one
    list of blocks per KV head, scored by all its tokens (the maximum over tokens and heads).
    sqattn_per_token: with sqattn_top_k and decode_tokens, every token of a decode row keeps a list of its own, scored
    with its own query over the keys it attends to (the step then runs its decode side over batch x decode_tokens
    rows of one token; a workspace passed in must be sized for that many sequences).
    Returns bf16 [num_tokens, num_heads*head_dim]."""
    nb, hkv, bs, d = _cache_dims(key_cache, value_cache)
    if hkv != kv_num_heads:
        raise ValueError("cache holds %d KV heads, kv_num_heads=%d" % (hkv, kv_num_heads))
    p_qkv = _chk(qkv, "qkv", torch.bfloat16, 2)
    T = qkv.shape[0]
    if qkv.shape[1] != (num_heads + 2 * hkv) * d:
        raise ValueError("qkv has %d columns, expected (num_heads+2*kv_num_heads)*head_dim = %d" %
                         (qkv.shape[1], (num_heads + 2 * hkv) * d))
    p_kc = _chk(key_cache, "key_cache", _CACHE_DT, 4)
    p_vc = _chk(value_cache, "value_cache", _CACHE_DT, 4)
    p_ks, p_vs = _scales(cache_k_scale, cache_v_scale, hkv, d, cache_quant_type, nb, bs)
    p_bt = _chk(block_tables, "block_tables", torch.int32, 2)
    batch, mb = block_tables.shape
    p_enc = _chk(seq_lens_encoder, "seq_lens_encoder", torch.int32, 1)
    p_dec = _chk(seq_lens_decoder, "seq_lens_decoder", torch.int32, 1)
    p_this = _chk(seq_lens_this_time, "seq_lens_this_time", torch.int32, 1)
    for name, t in (("seq_lens_encoder", seq_lens_encoder), ("seq_lens_decoder", seq_lens_decoder),
                    ("seq_lens_this_time", seq_lens_this_time)):
        if t.numel() != batch:
            raise ValueError("%s has %d entries, block_tables %d rows" % (name, t.numel(), batch))
    if cu_seqlens_q is None:
        cu_seqlens_q = cu_seqlens_of(seq_lens_this_time)
    p_cu = _chk(cu_seqlens_q, "cu_seqlens_q", torch.int32, 1)
    if cu_seqlens_q.numel() != batch + 1:
        raise ValueError("cu_seqlens_q must have batch+1 entries")
    p_cos = p_sin = 0
    max_pos = 0
    if rotary_embs is not None:
        cos, sin = rotary_embs
        p_cos = _chk(cos, "rotary cos", torch.float32, 2)
        p_sin = _chk(sin, "rotary sin", torch.float32, 2)
        if cos.shape != sin.shape or cos.shape[1] != d // 2:
            raise ValueError("rotary table must be [max_pos, head_dim/2]")
        max_pos = cos.shape[0]
    if rope_style not in _ROPE:
        raise ValueError("unknown rope_style %r (neox | interleaved)" % (rope_style,))
    if max_chunk < 0:
        raise ValueError("max_chunk must be >= 0")
    if out is None:
        out = torch.empty((T, num_heads * d), dtype=torch.bfloat16, device=qkv.device)
    elif out.numel() != T * num_heads * d:
        raise ValueError("out holds %d values, the step writes num_tokens*num_heads*head_dim = %d"
                         % (out.numel(), T * num_heads * d))
    splits = prefill_auto_splits(prefill_rows or 1, num_heads, max_chunk, hkv) if max_chunk > 0 else 1
    per_token = bool(sqattn_per_token) and (sqattn_top_k or 0) > 0 and (decode_tokens or 0) > 1
    need = _lib.lib().fdattn_append_attention_workspace_bytes_ex(T, batch * decode_tokens if per_token else batch,
                                                                 num_heads, hkv, d, mb, splits)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=qkv.device)
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(d)
    ep = _extras(qkv_bias, q_norm_weight, k_norm_weight, rms_norm_eps, qkv.shape[1], d, prefill_rows or 0,
                 sqattn_top_k or 0, decode_tokens or 0, per_token)
    rc = _lib.lib().fdattn_append_attention_ex(
        p_qkv, p_kc, p_vc, p_ks, p_vs, p_cos, p_sin, p_bt, p_enc, p_dec, p_this, p_cu,
        _chk(out, "out", torch.bfloat16), workspace.data_ptr(), workspace.numel() * workspace.element_size(),
        T, batch, max_chunk, num_heads, hkv, d, bs, mb, nb, max_pos, _ROPE[rope_style], _quant(cache_quant_type),
        scale, ctypes.addressof(ep) if ep is not None else None, _stream())
    _lib.check(rc, "append_attention")
    return out
