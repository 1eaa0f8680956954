"""KV pages of whole sequences to and from a contiguous, self-describing buffer (the layout is
stated in include/fdattn.h).  Device tensors in and out, like every op of this package; the
header can be read on the host with ``parse_header``."""
import struct

import torch

from . import _lib
from .ops import _CACHE_DT, _cache_dims, _chk, _quant, _scales, _stream, is_dynamic

MAGIC = 0x564B4446
HEADER_BYTES = 256


def wire_bytes(num_tokens, kv_num_heads, head_dim, block_size, cache_quant_type="cache_int8"):
    n = _lib.lib().fdattn_kv_wire_bytes_for(int(num_tokens), kv_num_heads, head_dim, block_size, _quant(cache_quant_type))
    if n == 0:
        raise ValueError("bad wire shape: num_tokens=%r kv_num_heads=%r head_dim=%r block_size=%r"
                         % (num_tokens, kv_num_heads, head_dim, block_size))
    return n


def wire_offsets(num_tokens, kv_num_heads, head_dim, block_size, cache_quant_type="cache_int8"):
    """Byte offset of every sequence in one packed buffer, and the buffer's size."""
    offs, total = [], 0
    for n in num_tokens:
        offs.append(total)
        total += wire_bytes(n, kv_num_heads, head_dim, block_size, cache_quant_type)
    return offs, total


def parse_header(raw):
    """The header of one sequence (``raw``: at least 64 bytes) as a dict; ValueError if it is not one."""
    raw = bytes(raw[:64])
    if len(raw) < 64:
        raise ValueError("a wire header has %d bytes, got %d" % (HEADER_BYTES, len(raw)))
    f = struct.unpack("<8I4Q", raw)
    if f[0] != MAGIC:
        raise ValueError("not a KV wire buffer (magic %#x)" % f[0])
    if f[1] != 1:
        raise ValueError("KV wire version %d is not supported" % f[1])
    keys = ("magic", "version", "cache_quant_type", "kv_num_heads", "head_dim", "block_size", "num_tokens",
            "num_pages", "scales_off", "sums_off", "pages_off", "total_bytes")
    return dict(zip(keys, f))


class WirePlan:
    """Host and device copies of a batch's token counts and buffer offsets, reusable across layers
    (every layer of a model exports the same sequences)."""

    def __init__(self, num_tokens, kv_num_heads, head_dim, block_size, device="cuda", cache_quant_type="cache_int8"):
        self.num_tokens = [int(n) for n in num_tokens]
        if any(n < 0 for n in self.num_tokens):
            raise ValueError("num_tokens must not be negative")
        self.shape = (kv_num_heads, head_dim, block_size)
        self.dynamic = is_dynamic(cache_quant_type)  # the two kinds of format differ in the size of the scales section
        self.offsets, self.total = wire_offsets(self.num_tokens, kv_num_heads, head_dim, block_size, cache_quant_type)
        self.num_tokens_dev = torch.tensor(self.num_tokens, dtype=torch.int32).to(device)
        self.offsets_dev = torch.tensor(self.offsets, dtype=torch.int64).to(device)


def _common(key_cache, value_cache, block_tables, num_tokens, cache_quant_type):
    _chk(key_cache, "key_cache", _CACHE_DT, 4)
    _chk(value_cache, "value_cache", _CACHE_DT, 4)
    nb, hkv, bs, d = _cache_dims(key_cache, value_cache)
    _chk(block_tables, "block_tables", torch.int32, 2)
    plan = num_tokens if isinstance(num_tokens, WirePlan) else WirePlan(num_tokens, hkv, d, bs, key_cache.device,
                                                                        cache_quant_type)
    if plan.dynamic != is_dynamic(cache_quant_type):
        raise ValueError("the plan was made for a %s format, cache_quant_type is %r"
                         % ("dynamic" if plan.dynamic else "per-channel", cache_quant_type))
    if plan.shape != (hkv, d, bs):
        raise ValueError("the plan was made for kv_num_heads, head_dim, block_size = %r, the cache has %r"
                         % (plan.shape, (hkv, d, bs)))
    if len(plan.num_tokens) != block_tables.shape[0]:
        raise ValueError("num_tokens has %d entries, block_tables %d rows"
                         % (len(plan.num_tokens), block_tables.shape[0]))
    return nb, hkv, bs, d, plan.num_tokens, plan.offsets, plan.total, plan.num_tokens_dev, plan.offsets_dev


def kv_export(key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables, num_tokens, *,
              cache_quant_type="cache_int8", wire=None):
    """Packs the first ``num_tokens[b]`` tokens of every row of ``block_tables`` into one buffer
    (``num_tokens``: a list of ints or a WirePlan).  Returns (wire uint8 tensor, list of byte offsets)."""
    nb, hkv, bs, d, num_tokens, offs, total, nt, of = _common(key_cache, value_cache, block_tables, num_tokens,
                                                              cache_quant_type)
    pk, pv = _scales(cache_k_scale, cache_v_scale, hkv, d, cache_quant_type, nb, bs)
    if wire is None:
        wire = torch.empty(total, dtype=torch.uint8, device=key_cache.device)
    _chk(wire, "wire", torch.uint8, 1)
    if wire.numel() < total:
        raise ValueError("wire holds %d bytes, %d needed" % (wire.numel(), total))
    rc = _lib.lib().fdattn_kv_export(key_cache.data_ptr(), value_cache.data_ptr(), pk, pv, block_tables.data_ptr(),
                                     nt.data_ptr(), of.data_ptr(), wire.data_ptr(), len(num_tokens),
                                     max(num_tokens, default=0), hkv, d, bs, block_tables.shape[1], nb,
                                     _quant(cache_quant_type), _stream())
    _lib.check(rc, "fdattn_kv_export")
    return wire, offs


def kv_import(wire, key_cache, value_cache, block_tables, num_tokens, *, cache_k_scale=None, cache_v_scale=None,
              cache_quant_type="cache_int8", status=None):
    """Scatters a buffer made by ``kv_export`` (same ``num_tokens``) into the blocks ``block_tables``
    names.  Returns the device status int32[2]: [0] error bits (0 = good), [1] tiles whose sum failed.
    The dynamic formats need cache_k_scale / cache_v_scale: the scale caches the rows' scales are stored into."""
    nb, hkv, bs, d, num_tokens, offs, total, nt, of = _common(key_cache, value_cache, block_tables, num_tokens,
                                                              cache_quant_type)
    _chk(wire, "wire", torch.uint8, 1)
    if wire.numel() < total:
        raise ValueError("wire holds %d bytes, %d needed" % (wire.numel(), total))
    pk = pv = 0
    if cache_k_scale is not None or cache_v_scale is not None or is_dynamic(cache_quant_type):
        pk, pv = _scales(cache_k_scale, cache_v_scale, hkv, d, cache_quant_type, nb, bs)
    if status is None:
        status = torch.zeros(2, dtype=torch.int32, device=key_cache.device)
    _chk(status, "status", torch.int32, 1)
    rc = _lib.lib().fdattn_kv_import(wire.data_ptr(), of.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(),
                                     pk or None, pv or None, block_tables.data_ptr(), nt.data_ptr(), status.data_ptr(),
                                     len(num_tokens), max(num_tokens, default=0), hkv, d, bs, block_tables.shape[1],
                                     nb, _quant(cache_quant_type), _stream())
    _lib.check(rc, "fdattn_kv_import")
    return status
