"""CPU restatement (numpy) of the KV wire format written by fdattn_kv_export and read by
fdattn_kv_import (layout: include/fdattn.h).

TEST INFRASTRUCTURE ONLY, like everything under oracle/.  The format has no counterpart in the
reference ("parity unpinned" against it); what pins this restatement is in
tests/test_kv_wire_oracle.py: the header re-read field by field with struct, every tile sum
recomputed from single bytes with Python integers, the zero rows, the section alignment, and the
export -> import round trip into other blocks.
"""
import struct

import numpy as np

MAGIC, VERSION, HEADER = 0x564B4446, 1, 256


def _up(x):
    return (x + 255) // 256 * 256


DYNAMIC = (3, 4)  # cache_quant_type values with one scale per stored row: scale caches [num_blocks, hkv, bs]


def layout(num_tokens, hkv, d, bs, quant=1):
    pages = -(-num_tokens // bs)
    scales_off = HEADER
    sums_off = _up(scales_off + (pages * 2 * hkv * bs if quant in DYNAMIC else 2 * hkv * d) * 4)
    pages_off = _up(sums_off + pages * 2 * hkv * 8)
    total = _up(pages_off + pages * 2 * hkv * bs * d)
    return pages, scales_off, sums_off, pages_off, total


def _tile_sums(body):
    """u64 [pages, 2, hkv]: sum of the little-endian 32-bit words of every (page, K|V, head) tile"""
    pages, _, hkv, bs, d = body.shape
    return body.reshape(pages, 2, hkv, bs * d).view("<u4").astype(np.uint64).sum(axis=-1)


def export_seq(key_cache, value_cache, k_scale, v_scale, table_row, num_tokens, quant):
    """One sequence's wire bytes (numpy uint8).  Caches: uint8 [num_blocks, hkv, bs, d]."""
    nb, hkv, bs, d = key_cache.shape
    pages, scales_off, sums_off, pages_off, total = layout(num_tokens, hkv, d, bs, quant)
    buf = np.zeros(total, np.uint8)
    buf[:64] = np.frombuffer(struct.pack("<8I4Q", MAGIC, VERSION, quant, hkv, d, bs, num_tokens, pages,
                                         scales_off, sums_off, pages_off, total), np.uint8)
    dyn = quant in DYNAMIC
    rows = np.zeros((pages, 2, hkv, bs), np.float32)  # dynamic formats: the stored rows' scales
    body = np.zeros((pages, 2, hkv, bs, d), np.uint8)
    for p in range(pages):
        valid = min(bs, num_tokens - p * bs)
        pb = int(table_row[p])
        if 0 <= pb < nb:
            body[p, 0, :, :valid] = key_cache[pb, :, :valid]
            body[p, 1, :, :valid] = value_cache[pb, :, :valid]
            if dyn:
                rows[p, 0, :, :valid] = k_scale[pb, :, :valid]
                rows[p, 1, :, :valid] = v_scale[pb, :, :valid]
    sc = rows.ravel() if dyn else np.concatenate([np.asarray(k_scale, np.float32).ravel(),
                                                  np.asarray(v_scale, np.float32).ravel()])
    buf[scales_off:scales_off + sc.nbytes] = sc.view(np.uint8)
    sums = _tile_sums(body)
    if dyn:  # a tile's sum covers its scale row, too
        sums = sums + rows.view("<u4").astype(np.uint64).sum(axis=-1)
    buf[sums_off:sums_off + sums.nbytes] = sums.astype("<u8").view(np.uint8).ravel()
    buf[pages_off:pages_off + body.nbytes] = body.ravel()
    return buf


def export_batch(key_cache, value_cache, k_scale, v_scale, block_tables, num_tokens, quant):
    return np.concatenate([export_seq(key_cache, value_cache, k_scale, v_scale, block_tables[b], int(n), quant)
                           for b, n in enumerate(num_tokens)] or [np.zeros(0, np.uint8)])


def import_seq(buf, key_cache, value_cache, table_row, num_tokens, quant, k_scale=None, v_scale=None):
    """Scatters one sequence into the caches in place; returns (error bits, tiles whose sum failed), the
    status words of fdattn_kv_import.  Dynamic formats: k_scale / v_scale are the scale caches, written here."""
    nb, hkv, bs, d = key_cache.shape
    dyn = quant in DYNAMIC
    pages, scales_off, sums_off, pages_off, total = layout(num_tokens, hkv, d, bs, quant)
    got = struct.unpack("<8I4Q", bytes(buf[:64]))
    want = (MAGIC, VERSION, quant, hkv, d, bs, num_tokens, pages, scales_off, sums_off, pages_off, total)
    bits = (1 if got[:2] != want[:2] else 0) | (2 if got[2:] != want[2:] else 0)
    if bits:
        return bits, 0
    if k_scale is not None and not dyn:
        sc = np.concatenate([np.asarray(k_scale, np.float32).ravel(), np.asarray(v_scale, np.float32).ravel()])
        if not np.array_equal(buf[scales_off:scales_off + sc.nbytes], sc.view(np.uint8)):
            bits |= 4
    body = buf[pages_off:pages_off + pages * 2 * hkv * bs * d].reshape(pages, 2, hkv, bs, d)
    sums = np.ascontiguousarray(buf[sums_off:sums_off + pages * 2 * hkv * 8]).view("<u8").reshape(pages, 2, hkv)
    real = _tile_sums(np.ascontiguousarray(body))
    if dyn:
        rows = np.ascontiguousarray(buf[scales_off:scales_off + pages * 2 * hkv * bs * 4]).view(np.float32).reshape(pages, 2, hkv, bs)
        real = real + rows.view("<u4").astype(np.uint64).sum(axis=-1)
    failed = int((real != sums).sum())
    if failed:
        bits |= 8
    for p in range(pages):
        pb = int(table_row[p])
        if 0 <= pb < nb:
            key_cache[pb], value_cache[pb] = body[p, 0], body[p, 1]
            if dyn:
                k_scale[pb], v_scale[pb] = rows[p, 0], rows[p, 1]
        else:
            bits |= 16
    return bits, failed
