"""KV wire export / import on the GPU against the numpy restatement (oracle/kv_wire.py): wire bytes and
cache bytes bit-exact, status words equal, corruption and mismatches reported; at full size the
export -> import round trip keeps decode attention's output bit-identical."""
import numpy as np
import pytest
import torch

import fastdeploy_amd as fd
from conftest import np_of
from fastdeploy_amd import kv_wire
from fastdeploy_amd.ops import CACHE_FP8, CACHE_FP8_DYNAMIC, CACHE_INT8, CACHE_INT8_DYNAMIC
from oracle import kv_wire as ow

pytestmark = pytest.mark.gpu


def make(seed, nb, hkv, bs, d, batch, width):
    g = torch.Generator().manual_seed(seed)
    kc = torch.randint(0, 256, (nb, hkv, bs, d), generator=g, dtype=torch.uint8)
    vc = torch.randint(0, 256, (nb, hkv, bs, d), generator=g, dtype=torch.uint8)
    ks = torch.rand((hkv, d), generator=g) + 0.5
    vs = torch.rand((hkv, d), generator=g) + 0.5
    bt = torch.randperm(nb, generator=g)[:batch * width].to(torch.int32).view(batch, width).contiguous()
    return kc, vc, ks, vs, bt


@pytest.mark.parametrize("shape", [(8, 64, 128), (2, 16, 32), (3, 8, 48)])
def test_export_import_match_the_numpy_restatement(shape):
    hkv, bs, d = shape
    tokens = [0, 1, bs, bs + 1, 3 * bs - 1, 4 * bs]
    kc, vc, ks, vs, bt = make(1, 40, hkv, bs, d, len(tokens), 5)
    bt[2, 0] = -1                                            # a hole in a table: exports as zeros
    wire, offs = kv_wire.kv_export(kc.cuda(), vc.cuda(), ks.cuda(), vs.cuda(), bt.cuda(), tokens,
                                   cache_quant_type=CACHE_INT8)
    torch.cuda.synchronize()
    want = ow.export_batch(np_of(kc), np_of(vc), np_of(ks), np_of(vs), np_of(bt), tokens, CACHE_INT8)
    assert np.array_equal(np_of(wire), want)
    assert kv_wire.parse_header(np_of(wire)[offs[4]:offs[4] + 64].tobytes())["num_tokens"] == tokens[4]
    # import into other blocks of an empty cache
    g = torch.Generator().manual_seed(2)
    bt2 = (torch.randperm(40, generator=g)[:bt.numel()].to(torch.int32).view_as(bt)).contiguous()
    bt2[5, 1] = 40                                           # outside the pool: reported, not written
    kc2, vc2 = torch.zeros_like(kc).cuda(), torch.zeros_like(vc).cuda()
    st = kv_wire.kv_import(wire, kc2, vc2, bt2.cuda(), tokens, cache_k_scale=ks.cuda(), cache_v_scale=vs.cuda())
    torch.cuda.synchronize()
    kc_w, vc_w = np.zeros_like(np_of(kc)), np.zeros_like(np_of(vc))
    bits = 0
    for b, n in enumerate(tokens):
        r = ow.import_seq(want[offs[b]:], kc_w, vc_w, np_of(bt2)[b], n, CACHE_INT8, np_of(ks), np_of(vs))
        bits |= r[0]
    assert bits == 16 and st.tolist() == [16, 0]
    assert np.array_equal(np_of(kc2), kc_w) and np.array_equal(np_of(vc2), vc_w)


@pytest.mark.parametrize("shape", [(8, 64, 128), (2, 16, 32)])
def test_dynamic_formats_export_import_match_the_numpy_restatement(shape):
    """The formats with one scale per stored row: wire bytes (scale rows, sums over tile + row) and the imported
    caches and scale caches bit for bit as the restatement's; a flipped scale bit fails its tile's sum."""
    hkv, bs, d = shape
    tokens = [0, 1, bs, bs + 1, 3 * bs - 1, 4 * bs]
    kc, vc, _, _, bt = make(5, 40, hkv, bs, d, len(tokens), 5)
    g = torch.Generator().manual_seed(6)
    ks, vs = torch.rand((40, hkv, bs), generator=g) + 0.5, torch.rand((40, hkv, bs), generator=g) + 0.5
    bt[2, 0] = -1
    wire, offs = kv_wire.kv_export(kc.cuda(), vc.cuda(), ks.cuda(), vs.cuda(), bt.cuda(), tokens,
                                   cache_quant_type=CACHE_FP8_DYNAMIC)
    torch.cuda.synchronize()
    want = ow.export_batch(np_of(kc), np_of(vc), np_of(ks), np_of(vs), np_of(bt), tokens, CACHE_FP8_DYNAMIC)
    assert np.array_equal(np_of(wire), want)
    bt2 = (torch.randperm(40, generator=g)[:bt.numel()].to(torch.int32).view_as(bt)).contiguous()
    kc2, vc2 = torch.zeros_like(kc).cuda(), torch.zeros_like(vc).cuda()
    ks2, vs2 = torch.full_like(ks, 7.0).cuda(), torch.full_like(vs, 7.0).cuda()
    st = kv_wire.kv_import(wire, kc2, vc2, bt2.cuda(), tokens, cache_k_scale=ks2, cache_v_scale=vs2,
                           cache_quant_type=CACHE_FP8_DYNAMIC)
    torch.cuda.synchronize()
    kc_w, vc_w = np.zeros_like(np_of(kc)), np.zeros_like(np_of(vc))
    ks_w, vs_w = np.full_like(np_of(ks), 7.0), np.full_like(np_of(vs), 7.0)
    for b, n in enumerate(tokens):
        assert ow.import_seq(want[offs[b]:], kc_w, vc_w, np_of(bt2)[b], n, CACHE_FP8_DYNAMIC, ks_w, vs_w) == (0, 0)
    assert st.tolist() == [0, 0]
    assert np.array_equal(np_of(kc2), kc_w) and np.array_equal(np_of(vc2), vc_w)
    assert np.array_equal(np_of(ks2), ks_w) and np.array_equal(np_of(vs2), vs_w)
    bad = wire.clone()
    bad[offs[3] + 256 + 1] ^= 0x04                            # inside the first scale row of sequence 3
    st = kv_wire.kv_import(bad, kc2, vc2, bt2.cuda(), tokens, cache_k_scale=ks2, cache_v_scale=vs2,
                           cache_quant_type=CACHE_FP8_DYNAMIC)
    assert st.tolist() == [8, 1]
    with pytest.raises(ValueError):                           # the dynamic formats need somewhere to put the scales
        kv_wire.kv_import(wire, kc2, vc2, bt2.cuda(), tokens, cache_quant_type=CACHE_FP8_DYNAMIC)
    with pytest.raises(ValueError):                           # a plan sized for the per-channel formats
        kv_wire.kv_export(kc.cuda(), vc.cuda(), ks.cuda(), vs.cuda(), bt.cuda(),
                          kv_wire.WirePlan(tokens, hkv, d, bs), cache_quant_type=CACHE_FP8_DYNAMIC)


def test_import_reports_bad_buffers_and_leaves_the_cache_alone():
    hkv, bs, d = 8, 64, 128
    tokens = [100, 64]
    kc, vc, ks, vs, bt = make(4, 16, hkv, bs, d, 2, 2)
    dev = [t.cuda() for t in (kc, vc, ks, vs, bt)]
    wire, offs = kv_wire.kv_export(*dev, tokens, cache_quant_type=CACHE_FP8)
    hdr = kv_wire.parse_header(np_of(wire)[:64].tobytes())
    assert hdr["cache_quant_type"] == CACHE_FP8

    def run(w, toks=tokens, quant=CACHE_FP8, scales=(dev[2], dev[3])):
        k2, v2 = torch.zeros_like(dev[0]), torch.zeros_like(dev[1])
        st = kv_wire.kv_import(w, k2, v2, dev[4], toks, cache_k_scale=scales[0], cache_v_scale=scales[1],
                               cache_quant_type=quant)
        torch.cuda.synchronize()
        return st.tolist(), k2, v2

    st, k2, v2 = run(wire)
    assert st == [0, 0]
    bad = wire.clone(); bad[offs[1]] ^= 0xFF                 # second sequence: magic broken
    st, k2, v2 = run(bad)
    assert st == [1, 0]
    blocks1 = np_of(bt)[1, :1]
    assert not np_of(k2)[blocks1].any() and np_of(k2)[np_of(bt)[0, :2]].any()      # only the good sequence landed
    st, k2, _ = run(wire, quant=CACHE_INT8)
    assert st == [2, 0] and not np_of(k2).any()
    st, k2, _ = run(wire, toks=[100, 63])                    # a length the buffer was not made with
    assert st[0] & 2
    st, _, _ = run(wire, scales=(dev[2] * 2, dev[3]))
    assert st == [4, 0]
    bad = wire.clone()
    bad[hdr["pages_off"] + 3] ^= 1
    bad[hdr["pages_off"] + 9 * bs * d + 77] ^= 0x10
    st, _, _ = run(bad)
    assert st == [8, 2]
    with pytest.raises(ValueError):
        kv_wire.kv_import(wire[:1000], dev[0], dev[1], dev[4], tokens)
    with pytest.raises(ValueError):
        kv_wire.kv_export(*dev, [100, 64, 3])


def test_full_size_round_trip_keeps_decode_output():
    """configs[1]-shaped: 64 sequences of ~4k tokens leave one cache and enter another through the wire
    form; decode attention over the copy equals decode attention over the original bit for bit."""
    from fastdeploy_amd import synthetic as syn
    c = syn.decode_case(batch=64, ctx=(3584, 4608), seed=0, device="cuda")
    tokens = c["seq_lens_decoder"].cpu().tolist()
    wire, offs = kv_wire.kv_export(c["key_cache"], c["value_cache"], c["cache_k_scale"], c["cache_v_scale"],
                                   c["block_tables"], tokens)
    nb = c["key_cache"].shape[0]
    g = torch.Generator().manual_seed(5)
    remap = torch.randperm(nb, generator=g).to(torch.int32).cuda()
    bt2 = remap[c["block_tables"].clamp(min=0).long()].contiguous()
    kc2, vc2 = torch.zeros_like(c["key_cache"]), torch.zeros_like(c["value_cache"])
    st = kv_wire.kv_import(wire, kc2, vc2, bt2, tokens, cache_k_scale=c["cache_k_scale"],
                           cache_v_scale=c["cache_v_scale"])
    assert st.tolist() == [0, 0]
    a = fd.decode_attention(c["q"], c["key_cache"], c["value_cache"], c["cache_k_scale"], c["cache_v_scale"],
                            c["block_tables"], c["seq_lens_decoder"], num_heads=32)
    b = fd.decode_attention(c["q"], kc2, vc2, c["cache_k_scale"], c["cache_v_scale"], bt2, c["seq_lens_decoder"],
                            num_heads=32)
    torch.cuda.synchronize()
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    # a second export, from the copy, gives the same bytes
    wire2, _ = kv_wire.kv_export(kc2, vc2, c["cache_k_scale"], c["cache_v_scale"], bt2, tokens)
    assert torch.equal(wire, wire2)
