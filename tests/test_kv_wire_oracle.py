"""Pins the numpy restatement of the KV wire format (oracle/kv_wire.py) without a GPU: the header is
re-read field by field with struct and with the package's own parser, tile sums are recomputed from
single bytes with Python integers, rows past the sequence are zero, sections are aligned, and
export -> import into other blocks reproduces the sequence's bytes.  Size arithmetic is checked
against the library's fdattn_kv_wire_bytes."""
import struct

import numpy as np
import pytest

from fastdeploy_amd import _lib
from fastdeploy_amd.kv_wire import parse_header, wire_bytes, wire_offsets
from oracle import kv_wire as ow


def case(seed, nb=12, hkv=2, bs=16, d=32):
    rng = np.random.default_rng(seed)
    kc = rng.integers(0, 256, (nb, hkv, bs, d), dtype=np.uint8)
    vc = rng.integers(0, 256, (nb, hkv, bs, d), dtype=np.uint8)
    ks = rng.random((hkv, d), dtype=np.float32) + 0.5
    vs = rng.random((hkv, d), dtype=np.float32) + 0.5
    return rng, kc, vc, ks, vs


@pytest.mark.parametrize("tokens", [0, 1, 15, 16, 17, 47, 64])
def test_layout_fields_sums_and_zero_rows(tokens):
    rng, kc, vc, ks, vs = case(tokens)
    nb, hkv, bs, d = kc.shape
    row = rng.permutation(nb)[:6].astype(np.int32)
    buf = ow.export_seq(kc, vc, ks, vs, row, tokens, 1)
    h = parse_header(buf.tobytes())
    pages = (tokens + bs - 1) // bs
    assert (h["cache_quant_type"], h["kv_num_heads"], h["head_dim"], h["block_size"]) == (1, hkv, d, bs)
    assert h["num_tokens"] == tokens and h["num_pages"] == pages and h["total_bytes"] == len(buf)
    assert h["scales_off"] == 256 and all(h[k] % 256 == 0 for k in ("sums_off", "pages_off", "total_bytes"))
    assert h["sums_off"] >= 256 + 2 * hkv * d * 4 and h["pages_off"] >= h["sums_off"] + pages * 2 * hkv * 8
    assert len(buf) == wire_bytes(tokens, hkv, d, bs)                      # the library's size arithmetic
    assert not buf[64:256].any()
    sc = np.frombuffer(buf[256:256 + 2 * hkv * d * 4].tobytes(), "<f4")
    assert np.array_equal(sc[:hkv * d], ks.ravel()) and np.array_equal(sc[hkv * d:], vs.ravel())
    raw = buf.tobytes()
    for p in range(pages):
        valid = min(bs, tokens - p * bs)
        for kv, cache in enumerate((kc, vc)):
            for hh in range(hkv):
                unit = (p * 2 + kv) * hkv + hh
                tile = raw[h["pages_off"] + unit * bs * d: h["pages_off"] + (unit + 1) * bs * d]
                want = cache[row[p], hh].copy()
                want[valid:] = 0
                assert tile == want.tobytes()
                s = sum(int.from_bytes(tile[i:i + 4], "little") for i in range(0, len(tile), 4))
                assert struct.unpack_from("<Q", raw, h["sums_off"] + 8 * unit)[0] == s


def test_round_trip_into_other_blocks_and_error_bits():
    rng, kc, vc, ks, vs = case(3)
    nb, hkv, bs, d = kc.shape
    tokens = 41
    src = np.array([7, 2, 9, 0, 0, 0], np.int32)
    dst = np.array([1, 11, 4, 0, 0, 0], np.int32)
    buf = ow.export_seq(kc, vc, ks, vs, src, tokens, 2)
    kc2, vc2 = np.zeros_like(kc), np.zeros_like(vc)
    assert ow.import_seq(buf, kc2, vc2, dst, tokens, 2, ks, vs) == (0, 0)
    for p in range(3):
        valid = min(bs, tokens - p * bs)
        assert np.array_equal(kc2[dst[p], :, :valid], kc[src[p], :, :valid])
        assert np.array_equal(vc2[dst[p], :, :valid], vc[src[p], :, :valid])
        assert not kc2[dst[p], :, valid:].any()
    untouched = [b for b in range(nb) if b not in dst[:3]]
    assert not kc2[untouched].any() and not vc2[untouched].any()
    # a second export of the imported sequence gives the same bytes: the wire form depends on content only
    assert np.array_equal(ow.export_seq(kc2, vc2, ks, vs, dst, tokens, 2), buf)
    # error bits
    k3, v3 = np.zeros_like(kc), np.zeros_like(vc)
    bad = buf.copy(); bad[0] ^= 1
    assert ow.import_seq(bad, k3, v3, dst, tokens, 2) == (1, 0) and not k3.any()
    assert ow.import_seq(buf, k3, v3, dst, tokens, 1) == (2, 0) and not k3.any()       # other quant type
    assert ow.import_seq(buf, k3, v3, dst, tokens + 1, 2) == (2, 0) and not k3.any()   # other length
    assert ow.import_seq(buf, k3, v3, dst, tokens, 2, ks * 2, vs)[0] == 4
    bad = buf.copy(); bad[parse_header(buf.tobytes())["pages_off"] + 5] ^= 0x40
    assert ow.import_seq(bad, k3, v3, dst, tokens, 2) == (8, 1)
    assert ow.import_seq(buf, k3, v3, np.array([1, 99, 4, 0, 0, 0], np.int32), tokens, 2)[0] == 16


@pytest.mark.parametrize("tokens", [0, 1, 16, 41])
def test_dynamic_formats_carry_their_scale_rows(tokens):
    """One scale per stored row: the scales section holds [pages][2][hkv][bs] floats (zero past the end), every
    tile's sum covers its scale row, and the import stores the rows into the scale caches of the new blocks."""
    rng, kc, vc, _, _ = case(40 + tokens)
    nb, hkv, bs, d = kc.shape
    ks = rng.random((nb, hkv, bs), dtype=np.float32) + 0.5
    vs = rng.random((nb, hkv, bs), dtype=np.float32) + 0.5
    src = rng.permutation(nb)[:6].astype(np.int32)
    buf = ow.export_seq(kc, vc, ks, vs, src, tokens, 3)
    h = parse_header(buf.tobytes())
    pages = (tokens + bs - 1) // bs
    assert h["cache_quant_type"] == 3 and h["num_pages"] == pages and h["total_bytes"] == len(buf)
    assert len(buf) == wire_bytes(tokens, hkv, d, bs, 3)
    assert h["sums_off"] >= 256 + pages * 2 * hkv * bs * 4 and h["sums_off"] % 256 == 0
    raw = buf.tobytes()
    for p in range(pages):
        valid = min(bs, tokens - p * bs)
        for kv, (cache, sc) in enumerate(((kc, ks), (vc, vs))):
            for hh in range(hkv):
                unit = (p * 2 + kv) * hkv + hh
                srow = raw[256 + unit * bs * 4: 256 + (unit + 1) * bs * 4]
                want = sc[src[p], hh].copy()
                want[valid:] = 0
                assert srow == want.tobytes()
                tile = raw[h["pages_off"] + unit * bs * d: h["pages_off"] + (unit + 1) * bs * d]
                s = sum(int.from_bytes(x[i:i + 4], "little") for x in (tile, srow) for i in range(0, len(x), 4))
                assert struct.unpack_from("<Q", raw, h["sums_off"] + 8 * unit)[0] == s
    # round trip into other blocks
    dst = np.array([b for b in range(nb) if b not in src[:pages]][:6], np.int32)
    kc2, vc2, ks2, vs2 = np.zeros_like(kc), np.zeros_like(vc), np.zeros_like(ks), np.zeros_like(vs)
    assert ow.import_seq(buf, kc2, vc2, dst, tokens, 3, ks2, vs2) == (0, 0)
    for p in range(pages):
        valid = min(bs, tokens - p * bs)
        assert np.array_equal(kc2[dst[p], :, :valid], kc[src[p], :, :valid])
        assert np.array_equal(ks2[dst[p], :, :valid], ks[src[p], :, :valid]) and not ks2[dst[p], :, valid:].any()
        assert np.array_equal(vs2[dst[p], :, :valid], vs[src[p], :, :valid])
    assert np.array_equal(ow.export_seq(kc2, vc2, ks2, vs2, dst, tokens, 3), buf)
    if pages:  # a flipped bit in a scale row fails that tile's sum
        bad = buf.copy(); bad[256 + 2] ^= 0x10
        assert ow.import_seq(bad, kc2, vc2, dst, tokens, 3, ks2, vs2) == (8, 1)
    assert ow.import_seq(buf, kc2, vc2, dst, tokens, 1, ks2, vs2)[0] == 2      # read as a per-channel format


def test_offsets_of_a_packed_batch():
    offs, total = wire_offsets([0, 5, 130], 8, 128, 64)
    sizes = [wire_bytes(n, 8, 128, 64) for n in (0, 5, 130)]
    assert offs == [0, sizes[0], sizes[0] + sizes[1]] and total == sum(sizes)
    assert sizes[0] == 256 + 8192 and all(o % 256 == 0 for o in offs)      # header + scales, no pages
    assert sizes[2] == ow.layout(130, 8, 128, 64)[4]
    assert _lib.lib().fdattn_kv_wire_bytes(-1, 8, 128, 64) == 0
    with pytest.raises(ValueError):
        wire_bytes(5, 0, 128, 64)
    with pytest.raises(ValueError):
        parse_header(b"\0" * 64)
