"""One attention step over a mixed batch (prefill rows, decode rows, idle slots in one call) against the
CPU oracle: cache bytes bit-exact, bf16 outputs within 2e-3 abs OR 1e-2 rel."""
import numpy as np
import pytest
import torch

import fastdeploy_amd as fd
from conftest import bf16_close, bits, np_of
from fastdeploy_amd.ops import (CACHE_FP8, CACHE_FP8_BLOCK, CACHE_FP8_DYNAMIC, CACHE_INT8, CACHE_INT8_BLOCK,
                                CACHE_INT8_DYNAMIC, append_attention_workspace_bytes, byte_format, cu_seqlens_of, is_dynamic, scale_cache_shape,
                                seq_lens_this_time_of)
from fastdeploy_amd.rope import rope_table

pytestmark = pytest.mark.gpu


def mixed_case(enc, dec, quant, seed, hq=32, hkv=8, d=128, bs=64, max_pos=4096, this=None):
    g = torch.Generator().manual_seed(seed)
    batch = len(enc)
    enc_t, dec_t = torch.tensor(enc, dtype=torch.int32), torch.tensor(dec, dtype=torch.int32)
    this = seq_lens_this_time_of(enc_t, dec_t) if this is None else torch.tensor(this, dtype=torch.int32)
    cu = cu_seqlens_of(this)
    T = int(cu[-1])
    mb = max((int(dec[b]) + int(this[b]) + bs - 1) // bs for b in range(batch)) + 1
    pool = batch * mb
    bt = torch.randperm(pool, generator=g).to(torch.int32).view(batch, mb).contiguous()
    kc = torch.randint(0, 256, (pool, hkv, bs, d), generator=g, dtype=torch.uint8)
    vc = torch.randint(0, 256, (pool, hkv, bs, d), generator=g, dtype=torch.uint8)
    if byte_format(quant) == CACHE_FP8:  # no NaN codes in the prior contents
        kc = torch.where((kc & 0x7F) == 0x7F, kc & 0xFE, kc)
        vc = torch.where((vc & 0x7F) == 0x7F, vc & 0xFE, vc)
    # The prior cache bytes are uniform over all codes - far heavier-tailed than quantised activations - so the
    # scales put the dequantised range at +-(1..1.5): the prefill kernel carries q*k_scale and the softmax weights
    # in fp16, and its error grows with the magnitude of the dequantised cache.
    qmax = 127.0 if byte_format(quant) == CACHE_INT8 else 448.0
    # one scale per stored row or per tile / per channel
    shape = scale_cache_shape(quant, pool, hkv, bs) if is_dynamic(quant) else (hkv, d)
    ks = ((torch.rand(shape, generator=g) * 0.5 + 1.0) / qmax).contiguous()
    vs = ((torch.rand(shape, generator=g) * 0.5 + 1.0) / qmax).contiguous()
    qkv = torch.randn((T, (hq + 2 * hkv) * d), generator=g).to(torch.bfloat16)
    cos, sin = rope_table(max_pos, d, 500000.0, "cpu")
    return dict(qkv=qkv, key_cache=kc, value_cache=vc, cache_k_scale=ks, cache_v_scale=vs, block_tables=bt,
                seq_lens_encoder=enc_t, seq_lens_decoder=dec_t, seq_lens_this_time=this, cu_seqlens_q=cu,
                rope_cos=cos, rope_sin=sin, T=T)


def oracle_step(oracle, c, quant, hq=32, hkv=8, d=128, decode_tokens=1, top_k=0, per_token=False, **epilogue):
    """The step composed from the oracle's pieces; returns (out bf16 bits [T, hq*d] with NaN-free rows only where
    a token exists, key cache, value cache).  For the dynamic formats the scale caches the step leaves behind are
    put into c["scales_after"].  top_k > 0: the decode rows are block-sparse - a row keeps one list per KV head, a
    block's score being the maximum over the row's tokens (each at its own length) and query heads - or, per_token, every
    token keeps its own list, scored by itself alone."""
    kc, vc = np_of(c["key_cache"]).copy(), np_of(c["value_cache"]).copy()
    ks, vs = np_of(c["cache_k_scale"]).copy(), np_of(c["cache_v_scale"]).copy()
    c["scales_after"] = (ks, vs)
    bt, dec, cu = np_of(c["block_tables"]), np_of(c["seq_lens_decoder"]), np_of(c["cu_seqlens_q"])
    enc, this = np_of(c["seq_lens_encoder"]), np_of(c["seq_lens_this_time"])
    q, k_new, v_new = oracle.write_cache_kv(bits(c["qkv"]), kc, vc, ks, vs, np_of(c["rope_cos"]), np_of(c["rope_sin"]),
                                            bt, dec, cu, hq, hkv, d, 1, quant, want_kv_out=True, **epilogue)
    out = np.zeros((c["T"], hq * d), np.uint16)
    # decode rows: every token (one; up to decode_tokens in a speculative step) attends to the cache up to itself
    drows = [(b, t) for b in range(len(enc)) if enc[b] == 0 and 1 <= this[b] <= decode_tokens for t in range(this[b])]
    if drows:
        qd = np.ascontiguousarray(q[[cu[b] + t for b, t in drows]])
        btd = np.ascontiguousarray(bt[[b for b, _ in drows]])
        kvl = np.array([dec[b] + t + 1 for b, t in drows], np.int32)
        kept = cnt = None
        if top_k > 0:
            sc = oracle.sqattn_block_scores(qd, kc, ks, btd, kvl, hq, hkv, d, quant)   # per token: [rows, hkv, max_blocks]
            for i in range(len(drows)):
                sc[i, :, (kvl[i] + 63) // 64:] = -np.inf   # blocks past a token's length are not scored by it
            kept = np.zeros((len(drows), hkv, top_k), np.int32)
            cnt = np.zeros((len(drows), hkv), np.int32)
            if per_token:
                kept, cnt = oracle.topk_select(sc, kvl, 64, top_k)
            for b in sorted(set(b for b, _ in drows)) if not per_token else ():
                idx = [i for i, (bb, _) in enumerate(drows) if bb == b]
                kb, cb = oracle.topk_select(sc[idx].max(axis=0, keepdims=True), kvl[idx[-1]:idx[-1] + 1], 64, top_k)
                kept[idx], cnt[idx] = kb, cb
        od = oracle.decode_attention(qd, kc, vc, ks, vs, btd, kvl, hq, hkv, d, quant, kept_blocks=kept, kept_counts=cnt)
        for i, (b, t) in enumerate(drows):
            out[cu[b] + t] = od[i]
    ptoks = np.array([t for b in range(len(enc)) if enc[b] > 0 for t in range(cu[b], cu[b + 1])], np.int32)
    if len(ptoks):
        op = oracle.append_attention_prefill(q, k_new, v_new, kc, vc, ks, vs, bt, dec, cu, hq, hkv, d, quant,
                                             token_ids=ptoks)
        out[ptoks] = op[ptoks]
    return out, kc, vc


@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_FP8, CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC, CACHE_INT8_BLOCK, CACHE_FP8_BLOCK])
def test_mixed_batch_step(oracle, quant):
    enc = [0, 150, 0, 0, 70, 0, 1, 300]
    dec = [700, 0, 0, 63, 200, 1, 0, 129]
    c = mixed_case(enc, dec, quant, seed=7)
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    out = fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                              dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                              (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                              num_heads=32, kv_num_heads=8, max_chunk=300, cache_quant_type=quant,
                              cu_seqlens_q=dev["cu_seqlens_q"])
    torch.cuda.synchronize()
    want, kc, vc = oracle_step(oracle, c, quant)
    assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc)
    if is_dynamic(quant):  # the writer stored the new rows' scales
        assert np.array_equal(np_of(dev["cache_k_scale"]), c["scales_after"][0])
        assert np.array_equal(np_of(dev["cache_v_scale"]), c["scales_after"][1])
        assert not np.array_equal(np_of(c["cache_k_scale"]), c["scales_after"][0])
    ok, mx, bad = bf16_close(bits(out), want)
    assert ok, "%d out of tolerance, max %.4g" % (bad, mx)


def test_mixed_batch_step_with_projection_epilogue(oracle):
    """qkv bias and the RMS norm of Q and K heads in front of the cache write, inside the one-call step."""
    enc, dec = [0, 90, 0, 33], [130, 64, 7, 0]
    c = mixed_case(enc, dec, CACHE_INT8, seed=12)
    g = torch.Generator().manual_seed(3)
    bias = (torch.randn((48 * 128,), generator=g) * 0.25).to(torch.bfloat16)
    qw, kw = torch.rand((128,), generator=g) + 0.5, torch.rand((128,), generator=g) + 0.5
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    out = fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                              dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                              (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                              num_heads=32, kv_num_heads=8, max_chunk=90, cu_seqlens_q=dev["cu_seqlens_q"],
                              qkv_bias=bias.cuda(), q_norm_weight=qw.cuda(), k_norm_weight=kw.cuda(), rms_norm_eps=1e-6)
    torch.cuda.synchronize()
    want, kc, vc = oracle_step(oracle, c, CACHE_INT8, qkv_bias=bits(bias), q_norm_weight=np_of(qw),
                               k_norm_weight=np_of(kw), rms_norm_eps=1e-6)
    assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc)
    ok, mx, bad = bf16_close(bits(out), want)
    assert ok, "%d out of tolerance, max %.4g" % (bad, mx)


def test_mixed_step_with_key_splits_for_the_prefill_row(oracle):
    """One prefill row on a long prefix among decode rows, the host saying so (prefill_rows=1): its query tiles'
    keys are shared by several workgroups; same cache bytes and outputs as the oracle."""
    enc, dec = [0, 200, 0, 0], [700, 4500, 64, 3000]
    c = mixed_case(enc, dec, CACHE_INT8, seed=15, max_pos=8192)
    assert fd.ops.prefill_auto_splits(1, 32, 200) > 1
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    out = fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                              dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                              (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                              num_heads=32, kv_num_heads=8, max_chunk=200, cu_seqlens_q=dev["cu_seqlens_q"], prefill_rows=1)
    torch.cuda.synchronize()
    want, kc, vc = oracle_step(oracle, c, CACHE_INT8)
    assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc)
    ok, mx, bad = bf16_close(bits(out), want)
    assert ok, "%d out of tolerance, max %.4g" % (bad, mx)
    # without the host's count the prefill kernel counts the prefill rows itself and splits the same way
    kc1, vc1 = c["key_cache"].cuda(), c["value_cache"].cuda()
    out1 = fd.append_attention(dev["qkv"], kc1, vc1, dev["seq_lens_encoder"], dev["seq_lens_decoder"],
                               dev["seq_lens_this_time"], dev["block_tables"], (dev["rope_cos"], dev["rope_sin"]),
                               dev["cache_k_scale"], dev["cache_v_scale"], num_heads=32, kv_num_heads=8, max_chunk=200,
                               cu_seqlens_q=dev["cu_seqlens_q"])
    assert np.array_equal(bits(out1), bits(out)), "counted on the GPU: not the splits of the host's count"
    # a workspace sized without the splits still works: as many splits as it holds (none)
    ws = fd.append_attention_workspace(c["T"], 4, 32, 8, 128, dev["block_tables"].shape[1])
    kc2, vc2 = c["key_cache"].cuda(), c["value_cache"].cuda()
    import ctypes
    from fastdeploy_amd import _lib
    ex = _lib.StepExtras(None, None, None, 0.0, 1)
    o2 = torch.empty_like(out)
    rc = _lib.lib().fdattn_append_attention_ex(
        dev["qkv"].data_ptr(), kc2.data_ptr(), vc2.data_ptr(), dev["cache_k_scale"].data_ptr(), dev["cache_v_scale"].data_ptr(),
        dev["rope_cos"].data_ptr(), dev["rope_sin"].data_ptr(), dev["block_tables"].data_ptr(), dev["seq_lens_encoder"].data_ptr(),
        dev["seq_lens_decoder"].data_ptr(), dev["seq_lens_this_time"].data_ptr(), dev["cu_seqlens_q"].data_ptr(), o2.data_ptr(),
        ws.data_ptr(), ws.numel(), c["T"], 4, 200, 32, 8, 128, 64, dev["block_tables"].shape[1], kc2.shape[0],
        dev["rope_cos"].shape[0], 1, CACHE_INT8, 1.0 / 128 ** 0.5, ctypes.addressof(ex), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == 0
    ok, mx, bad = bf16_close(bits(o2), want)
    assert ok, "small workspace: %d out of tolerance, max %.4g" % (bad, mx)


@pytest.mark.parametrize("top_k,tokens,rows,per_token", [(None, None, 1, False), (8, None, 1, False), (None, 2, 1, False),
                                                         (8, 3, 1, False), (None, None, None, False), (8, 2, None, False),
                                                         (8, 3, 1, True)])
def test_mixed_step_with_key_splits_replays_from_a_hip_graph(top_k, tokens, rows, per_token):
    """The mixed step with key splits (writer, decode + its merge - with top_k the block selector and the sparse
    decode instead -, prefill shares, prefill merge) captured in a HIP graph: every replay, with eager work and synchronisations in between, equals the eager step on a copy of the
    state bit for bit (outputs and cache bytes).  rows None: without the host's count of prefill rows (the prefill
    kernel counts them).  per_token: a block list per draft token (the token-as-row view is laid out by a kernel of
    the step, inside the graph)."""
    enc, dec = [0, 160, 0, 0, 0], [900, 4200, 63, 2100, 4600]
    # (tokens: three of the decode rows bring that many draft tokens - the decode kernel's several-token variant)
    c = mixed_case(enc, dec, CACHE_INT8, seed=21, max_pos=8192, this=[tokens, 160, 1, tokens, tokens] if tokens else None)
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    eag = {k: (v.clone() if isinstance(v, torch.Tensor) else v) for k, v in dev.items()}
    splits = fd.ops.prefill_auto_splits(1, 32, 160)
    assert splits > 1
    mb = dev["block_tables"].shape[1]
    seqs = 5 * tokens if per_token else 5   # (a list per token: the decode side runs over batch x decode_tokens rows)
    ws_g = fd.append_attention_workspace(c["T"], seqs, 32, 8, 128, mb, prefill_splits=splits)
    ws_e = fd.append_attention_workspace(c["T"], seqs, 32, 8, 128, mb, prefill_splits=splits)

    def step(s, ws):
        return fd.append_attention(s["qkv"], s["key_cache"], s["value_cache"], s["seq_lens_encoder"],
                                   s["seq_lens_decoder"], s["seq_lens_this_time"], s["block_tables"],
                                   (s["rope_cos"], s["rope_sin"]), s["cache_k_scale"], s["cache_v_scale"],
                                   num_heads=32, kv_num_heads=8, max_chunk=160, cu_seqlens_q=s["cu_seqlens_q"],
                                   prefill_rows=rows, workspace=ws, sqattn_top_k=top_k, decode_tokens=tokens,
                                   sqattn_per_token=per_token)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up outside the capture, on a throw-away copy
        tmp = {k: (v.clone() if isinstance(v, torch.Tensor) else v) for k, v in dev.items()}
        step(tmp, ws_g)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g = step(dev, ws_g)
    gen = torch.Generator(device="cuda").manual_seed(3)
    for r in range(3):
        new_qkv = torch.randn(dev["qkv"].shape, generator=gen, device="cuda").to(torch.bfloat16)
        dev["qkv"].copy_(new_qkv)  # eager work between the replays
        eag["qkv"].copy_(new_qkv)
        torch.cuda.synchronize()
        graph.replay()
        want = step(eag, ws_e)
        torch.cuda.synchronize()
        assert torch.equal(out_g, want), "replay %d: outputs differ" % r
        assert torch.equal(dev["key_cache"], eag["key_cache"]) and torch.equal(dev["value_cache"], eag["value_cache"]), r


def test_decode_only_and_prefill_only_steps_through_the_same_entry(oracle):
    # (the last case says that all its 3 sequences are prefill rows: the step then launches no decode pass)
    for enc, dec, mc, rows in (([0, 0, 0, 0], [5, 64, 1000, 0], 0, None), ([64, 1, 257, 0], [0, 0, 100, 0], 257, None),
                               ([64, 1, 257], [0, 0, 100], 257, 3)):
        c = mixed_case(enc, dec, CACHE_INT8, seed=9)
        dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
        ws = fd.append_attention_workspace(c["T"], len(enc), 32, 8, 128, dev["block_tables"].shape[1])
        out = fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                                  dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                                  (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                                  num_heads=32, kv_num_heads=8, max_chunk=mc, workspace=ws,
                                  cu_seqlens_q=dev["cu_seqlens_q"], prefill_rows=rows)
        torch.cuda.synchronize()
        want, kc, vc = oracle_step(oracle, c, CACHE_INT8)
        assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc)
        ok, mx, bad = bf16_close(bits(out), want)
        assert ok, "%d out of tolerance, max %.4g" % (bad, mx)


@pytest.mark.parametrize("d", [64, 96, 256])
def test_mixed_step_other_shapes(oracle, d):
    """2 query heads per KV head, block_size 16, head_dim 64 / 256 (decode and prefill rows on the MFMA kernels for
    any block size) and 96 (both on the vector-ALU kernels)."""
    hq, hkv, bs = 4, 2, 16
    c = mixed_case([0, 40, 0, 9], [33, 0, 0, 20], CACHE_INT8, seed=3, hq=hq, hkv=hkv, d=d, bs=bs, max_pos=256)
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    out = fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                              dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                              (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                              num_heads=hq, kv_num_heads=hkv, max_chunk=40)
    torch.cuda.synchronize()
    want, kc, vc = oracle_step(oracle, c, CACHE_INT8, hq, hkv, d)
    assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc)
    ok, mx, bad = bf16_close(bits(out), want)
    assert ok, "%d out of tolerance, max %.4g" % (bad, mx)


@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_FP8_BLOCK])
def test_mixed_step_other_shapes_many_rows(oracle, quant):
    """head_dim 256, block_size 32, 60 sequences x 4 KV heads: (sequence, KV head) pairs that fill the GPU's 256
    workgroup slots once, so the decode kernel takes one split and writes the step's output rows itself, between the
    rows of the prefill sequences."""
    hq, hkv, d, bs = 8, 4, 256, 32
    rng = np.random.default_rng(17)
    enc = [0] * 60
    dec = [int(x) for x in rng.integers(1, 300, 60)]
    for b in (4, 31, 59):
        enc[b], dec[b] = int(rng.integers(2, 50)), int(rng.integers(0, 100))
    dec[10] = 0
    c = mixed_case(enc, dec, quant, seed=9, hq=hq, hkv=hkv, d=d, bs=bs, max_pos=512)
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    out = fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                              dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                              (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                              num_heads=hq, kv_num_heads=hkv, max_chunk=50, cache_quant_type=quant,
                              cu_seqlens_q=dev["cu_seqlens_q"])
    torch.cuda.synchronize()
    want, kc, vc = oracle_step(oracle, c, quant, hq, hkv, d)
    assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc)
    ok, mx, bad = bf16_close(bits(out), want)
    assert ok, "%d out of tolerance, max %.4g" % (bad, mx)


@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_FP8_DYNAMIC])
@pytest.mark.parametrize("group", [2, 8])
def test_mixed_step_other_group_sizes(oracle, group, quant):
    """2 and 8 query heads per KV head (head_dim 128, block 64): the whole step stays on the MFMA kernels."""
    hkv = 4
    hq = group * hkv
    c = mixed_case([0, 150, 0, 0, 70, 1], [700, 0, 63, 200, 129, 0], quant, seed=40 + group, hq=hq, hkv=hkv)
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    out = fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                              dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                              (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                              num_heads=hq, kv_num_heads=hkv, max_chunk=150, cache_quant_type=quant,
                              cu_seqlens_q=dev["cu_seqlens_q"])
    torch.cuda.synchronize()
    want, kc, vc = oracle_step(oracle, c, quant, hq, hkv, 128)
    assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc)
    ok, mx, bad = bf16_close(bits(out), want)
    assert ok, "%d out of tolerance, max %.4g" % (bad, mx)


@pytest.mark.parametrize("quant", [CACHE_FP8, CACHE_INT8_DYNAMIC, CACHE_FP8_BLOCK])
def test_mixed_step_with_block_sparse_decode_rows(oracle, quant):
    """sqattn_top_k in the one-call step: every decode row selects its top-k blocks with its new query over the
    cache that already holds its new token, and attends to those only; prefill rows are untouched by it.  Against the
    oracle's pieces: writer, block scores + top-k, sparse decode, prefill."""
    enc, dec = [0, 90, 0, 0, 0, 0, 1], [64 * 30 + 5, 700, 63, 64 * 11, 64 * 3, 0, 0]   # + an idle slot, a 1-token prompt
    top_k = 6
    c = mixed_case(enc, dec, quant, seed=33, max_pos=4096)
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    out = fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                              dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                              (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                              num_heads=32, kv_num_heads=8, max_chunk=90, cache_quant_type=quant,
                              cu_seqlens_q=dev["cu_seqlens_q"], prefill_rows=2, sqattn_top_k=top_k)
    torch.cuda.synchronize()
    # the oracle's step, with the decode rows done sparsely
    kc, vc = np_of(c["key_cache"]).copy(), np_of(c["value_cache"]).copy()
    ks, vs = np_of(c["cache_k_scale"]).copy(), np_of(c["cache_v_scale"]).copy()
    bt, cu = np_of(c["block_tables"]), np_of(c["cu_seqlens_q"])
    decs, this = np_of(c["seq_lens_decoder"]), np_of(c["seq_lens_this_time"])
    q, k_new, v_new = oracle.write_cache_kv(bits(c["qkv"]), kc, vc, ks, vs, np_of(c["rope_cos"]), np_of(c["rope_sin"]),
                                            bt, decs, cu, 32, 8, 128, 1, quant, want_kv_out=True)
    assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc)
    want = np.zeros((c["T"], 32 * 128), np.uint16)
    drows = [b for b in range(len(enc)) if enc[b] == 0 and this[b] == 1]
    qd = np.ascontiguousarray(q[[cu[b] for b in drows]])
    btd, kvl = np.ascontiguousarray(bt[drows]), np.ascontiguousarray(decs[drows] + 1)
    sc = oracle.sqattn_block_scores(qd, kc, ks, btd, kvl, 32, 8, 128, quant)
    kept, cnt = oracle.topk_select(sc, kvl, 64, top_k)
    od = oracle.decode_attention(qd, kc, vc, ks, vs, btd, kvl, 32, 8, 128, quant, kept_blocks=kept, kept_counts=cnt)
    for i, b in enumerate(drows):
        want[cu[b]] = od[i]
    ptoks = np.concatenate([np.arange(cu[1], cu[2]), np.arange(cu[6], cu[7])]).astype(np.int32)
    op = oracle.append_attention_prefill(q, k_new, v_new, kc, vc, ks, vs, bt, decs, cu, 32, 8, 128, quant, token_ids=ptoks)
    want[ptoks] = op[ptoks]
    ok, mx, bad = bf16_close(bits(out), want)
    assert ok, "%d out of tolerance, max %.4g" % (bad, mx)
    # and it differs from the dense step where a row has more blocks than it keeps
    dense = fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                                dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                                (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                                num_heads=32, kv_num_heads=8, max_chunk=90, cache_quant_type=quant,
                                cu_seqlens_q=dev["cu_seqlens_q"], prefill_rows=2)
    assert not torch.equal(dense[0], out[0]) and torch.equal(dense[cu[1]:cu[2]], out[cu[1]:cu[2]])
    ok, mx, bad = bf16_close(bits(out[int(cu[4])]), bits(dense[int(cu[4])]))   # 4 blocks <= top_k: the row keeps them all
    assert ok


@pytest.mark.parametrize("quant,hq,hkv,d,bs", [
    (CACHE_INT8, 8, 4, 64, 16),            # the fp16-MFMA decode kernel over the lists, tiles of two blocks
    (CACHE_FP8_DYNAMIC, 16, 2, 256, 64),   # 8 query heads per KV head, the exact selector's most
    (CACHE_FP8, 6, 2, 96, 32),             # a head size only the vector-ALU kernels take
    (CACHE_FP8_BLOCK, 6, 2, 64, 32),
    (CACHE_INT8_DYNAMIC, 4, 4, 128, 128),
])
def test_mixed_step_with_block_sparse_decode_rows_other_shapes(oracle, quant, hq, hkv, d, bs):
    """sqattn_top_k in the one-call step outside the MFMA selector's shapes: the exact (fp64) selector picks the
    blocks of the step's decode rows, the decode kernels of the other shapes attend to them.  Against the oracle's
    pieces, as at the MFMA selector's shape: writer, block scores + top-k, sparse decode, prefill."""
    enc, dec = [0, 40, 0, 0, 0, 0, 1], [bs * 30 + 5, 300, bs - 1, bs * 11, bs * 3, 0, 0]   # + an idle slot, a 1-token prompt
    top_k = 6
    c = mixed_case(enc, dec, quant, seed=35, hq=hq, hkv=hkv, d=d, bs=bs, max_pos=4096)
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    kw = dict(num_heads=hq, kv_num_heads=hkv, max_chunk=40, cache_quant_type=quant, cu_seqlens_q=dev["cu_seqlens_q"])
    args = lambda: (dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"], dev["seq_lens_decoder"],
                    dev["seq_lens_this_time"], dev["block_tables"], (dev["rope_cos"], dev["rope_sin"]),
                    dev["cache_k_scale"], dev["cache_v_scale"])
    out = fd.append_attention(*args(), sqattn_top_k=top_k, **kw)
    torch.cuda.synchronize()
    kc, vc = np_of(c["key_cache"]).copy(), np_of(c["value_cache"]).copy()
    ks, vs = np_of(c["cache_k_scale"]).copy(), np_of(c["cache_v_scale"]).copy()
    bt, cu = np_of(c["block_tables"]), np_of(c["cu_seqlens_q"])
    decs, this = np_of(c["seq_lens_decoder"]), np_of(c["seq_lens_this_time"])
    q, k_new, v_new = oracle.write_cache_kv(bits(c["qkv"]), kc, vc, ks, vs, np_of(c["rope_cos"]), np_of(c["rope_sin"]),
                                            bt, decs, cu, hq, hkv, d, 1, quant, want_kv_out=True)
    assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc)
    want = np.zeros((c["T"], hq * d), np.uint16)
    drows = [b for b in range(len(enc)) if enc[b] == 0 and this[b] == 1]
    qd = np.ascontiguousarray(q[[cu[b] for b in drows]])
    btd, kvl = np.ascontiguousarray(bt[drows]), np.ascontiguousarray(decs[drows] + 1)
    sc = oracle.sqattn_block_scores(qd, kc, ks, btd, kvl, hq, hkv, d, quant)
    kept, cnt = oracle.topk_select(sc, kvl, bs, top_k)
    od = oracle.decode_attention(qd, kc, vc, ks, vs, btd, kvl, hq, hkv, d, quant, kept_blocks=kept, kept_counts=cnt)
    for i, b in enumerate(drows):
        want[cu[b]] = od[i]
    ptoks = np.concatenate([np.arange(cu[1], cu[2]), np.arange(cu[6], cu[7])]).astype(np.int32)
    op = oracle.append_attention_prefill(q, k_new, v_new, kc, vc, ks, vs, bt, decs, cu, hq, hkv, d, quant, token_ids=ptoks)
    want[ptoks] = op[ptoks]
    ok, mx, bad = bf16_close(bits(out), want)
    assert ok, "%d out of tolerance, max %.4g" % (bad, mx)
    # and it differs from the dense step where a row has more blocks than it keeps
    dense = fd.append_attention(*args(), **kw)
    assert not torch.equal(dense[cu[0]], out[cu[0]])


@pytest.mark.parametrize("quant,hq,hkv,tokens", [(CACHE_FP8, 32, 8, 2), (CACHE_INT8, 32, 8, 4), (CACHE_INT8_DYNAMIC, 16, 8, 3),
                                                 (CACHE_FP8_DYNAMIC, 8, 8, 5), (CACHE_FP8_BLOCK, 24, 8, 5), (CACHE_INT8_BLOCK, 32, 8, 3)])
def test_mixed_step_with_block_sparse_decode_rows_of_several_tokens(oracle, quant, hq, hkv, tokens):
    """sqattn_top_k and decode_tokens together: a decode row of several tokens keeps ONE list of blocks per KV head - a
    block's score is the maximum over the row's tokens, each over the keys it attends to, and query heads - and token t
    attends to the kept blocks' keys up to itself.  Against the oracle's pieces: its writer; block scores per token at
    that token's length, their maximum, the oracle's top-k at the row's length (indices must agree exactly, or the
    outputs would not); one sparse decode per token with the row's list.  Rows whose new tokens straddle a block
    boundary, a row on an empty cache, rows of fewer tokens, rows with no more blocks than are kept, a prefill row."""
    T, top_k = tokens, 5
    enc = [0, 50, 0, 0, 0, 0, 0, 0]
    dec = [64 * 20 + 7, 300, 64 * 9 - 1, 0, 64 * 31 - T + 1, 64 * 3, 64 * 12 + 30, 64 * 15]
    this = [T, 50, T, T, T, T, max(T - 1, 1), 1]
    c = mixed_case(enc, dec, quant, seed=70 + T, hq=hq, hkv=hkv, max_pos=4096, this=this)
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    out = fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                              dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                              (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                              num_heads=hq, kv_num_heads=hkv, max_chunk=50, cache_quant_type=quant,
                              cu_seqlens_q=dev["cu_seqlens_q"], prefill_rows=1, sqattn_top_k=top_k, decode_tokens=T)
    torch.cuda.synchronize()
    kc, vc = np_of(c["key_cache"]).copy(), np_of(c["value_cache"]).copy()
    ks, vs = np_of(c["cache_k_scale"]).copy(), np_of(c["cache_v_scale"]).copy()
    bt, cu, decs = np_of(c["block_tables"]), np_of(c["cu_seqlens_q"]), np_of(c["seq_lens_decoder"])
    q, k_new, v_new = oracle.write_cache_kv(bits(c["qkv"]), kc, vc, ks, vs, np_of(c["rope_cos"]), np_of(c["rope_sin"]),
                                            bt, decs, cu, hq, hkv, 128, 1, quant, want_kv_out=True)
    assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc)
    got = bits(out)
    for b in range(len(enc)):
        rows = list(range(cu[b], cu[b + 1]))
        if enc[b] > 0:
            want = oracle.append_attention_prefill(q, k_new, v_new, kc, vc, ks, vs, bt, decs, cu, hq, hkv, 128, quant,
                                                   token_ids=np.array(rows, np.int32))[rows]
        else:
            n = len(rows)
            qd = np.ascontiguousarray(q[rows])
            btd = np.ascontiguousarray(np.repeat(bt[b:b + 1], n, 0))
            kvl = np.array([decs[b] + t + 1 for t in range(n)], np.int32)
            per_token = oracle.sqattn_block_scores(qd, kc, ks, btd, kvl, hq, hkv, 128, quant)   # [n, hkv, max_blocks]
            for t in range(n):   # blocks past a token's length are not scored by it
                per_token[t, :, (kvl[t] + 63) // 64:] = -np.inf
            shared = per_token.max(axis=0, keepdims=True)
            kept, cnt = oracle.topk_select(shared, kvl[-1:], 64, top_k)
            want = oracle.decode_attention(qd, kc, vc, ks, vs, btd, kvl, hq, hkv, 128, quant,
                                           kept_blocks=np.ascontiguousarray(np.repeat(kept, n, 0)),
                                           kept_counts=np.ascontiguousarray(np.repeat(cnt, n, 0)))
        ok, mx, bad = bf16_close(got[rows], want)
        assert ok, "sequence %d: %d out of tolerance, max %.4g" % (b, bad, mx)


@pytest.mark.parametrize("quant,hq,hkv,tokens,d,bs", [
    (CACHE_FP8, 32, 8, 4, 128, 64),            # the int8 / fp8-MFMA selector and sparse decode kernel
    (CACHE_INT8_DYNAMIC, 16, 8, 3, 128, 64),
    (CACHE_INT8, 32, 8, 6, 128, 64),           # 24 (token, head) pairs per KV head: more than one list per row allows
    (CACHE_FP8_BLOCK, 8, 2, 3, 64, 16),        # the fp16-MFMA scoring pass and decode kernel
    (CACHE_INT8, 16, 4, 2, 256, 32),
    (CACHE_FP8, 6, 2, 3, 96, 32),              # the exact selector and the vector-ALU decode kernel
])
def test_mixed_step_with_a_block_list_per_token(oracle, quant, hq, hkv, tokens, d, bs):
    """sqattn_top_k, decode_tokens and sqattn_per_token together: every token of a decode row of several tokens keeps
    its OWN list - scored with its own query over the keys it attends to - and attends to it.  Against the oracle's
    pieces per token: block scores at that token's length, top-k (indices must agree exactly, or the outputs would
    not), one sparse decode.  Rows whose new tokens straddle a block boundary, a row on an empty cache, rows of fewer
    tokens, rows with no more blocks than are kept, an idle slot, a prefill row; and the lists of a row's tokens do
    differ, so the result is not the one-list step's."""
    T, top_k = tokens, 5
    enc = [0, 50, 0, 0, 0, 0, 0, 0, 0]
    dec = [bs * 20 + 7, 300, bs * 9 - 1, 0, bs * 31 - T + 1, bs * 3, bs * 12 + 30 % bs, bs * 15, 77]
    this = [T, 50, T, T, T, T, max(T - 1, 1), 1, 0]
    c = mixed_case(enc, dec, quant, seed=170 + T, hq=hq, hkv=hkv, d=d, bs=bs, max_pos=4096, this=this)
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    kw = dict(num_heads=hq, kv_num_heads=hkv, max_chunk=50, cache_quant_type=quant, cu_seqlens_q=dev["cu_seqlens_q"],
              prefill_rows=1, sqattn_top_k=top_k, decode_tokens=T)
    args = lambda: (dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"], dev["seq_lens_decoder"],
                    dev["seq_lens_this_time"], dev["block_tables"], (dev["rope_cos"], dev["rope_sin"]),
                    dev["cache_k_scale"], dev["cache_v_scale"])
    out = fd.append_attention(*args(), sqattn_per_token=True, **kw)
    torch.cuda.synchronize()
    kc, vc = np_of(c["key_cache"]).copy(), np_of(c["value_cache"]).copy()
    ks, vs = np_of(c["cache_k_scale"]).copy(), np_of(c["cache_v_scale"]).copy()
    bt, cu, decs = np_of(c["block_tables"]), np_of(c["cu_seqlens_q"]), np_of(c["seq_lens_decoder"])
    q, k_new, v_new = oracle.write_cache_kv(bits(c["qkv"]), kc, vc, ks, vs, np_of(c["rope_cos"]), np_of(c["rope_sin"]),
                                            bt, decs, cu, hq, hkv, d, 1, quant, want_kv_out=True)
    assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc)
    got = bits(out)
    lists_differ = False
    for b in range(len(enc)):
        rows = list(range(cu[b], cu[b + 1]))
        if not rows:
            continue
        if enc[b] > 0:
            want = oracle.append_attention_prefill(q, k_new, v_new, kc, vc, ks, vs, bt, decs, cu, hq, hkv, d, quant,
                                                   token_ids=np.array(rows, np.int32))[rows]
        else:
            n = len(rows)
            qd = np.ascontiguousarray(q[rows])
            btd = np.ascontiguousarray(np.repeat(bt[b:b + 1], n, 0))
            kvl = np.array([decs[b] + t + 1 for t in range(n)], np.int32)
            sc = oracle.sqattn_block_scores(qd, kc, ks, btd, kvl, hq, hkv, d, quant)   # [n, hkv, max_blocks]
            kept, cnt = oracle.topk_select(sc, kvl, bs, top_k)
            lists_differ |= any(not np.array_equal(kept[t], kept[t + 1]) for t in range(n - 1))
            want = oracle.decode_attention(qd, kc, vc, ks, vs, btd, kvl, hq, hkv, d, quant, kept_blocks=kept, kept_counts=cnt)
        ok, mx, bad = bf16_close(got[rows], want)
        assert ok, "sequence %d: %d out of tolerance, max %.4g" % (b, bad, mx)
    assert lists_differ
    # a workspace of the caller's, sized for batch x decode_tokens sequences, full of garbage, used twice
    ws = torch.full((append_attention_workspace_bytes(c["T"], len(enc) * T, hq, hkv, d, bt.shape[1], 1),), 0xAB,
                    dtype=torch.uint8, device="cuda")
    for _ in range(2):
        dev2 = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
        again = fd.append_attention(dev2["qkv"], dev2["key_cache"], dev2["value_cache"], dev2["seq_lens_encoder"],
                                    dev2["seq_lens_decoder"], dev2["seq_lens_this_time"], dev2["block_tables"],
                                    (dev2["rope_cos"], dev2["rope_sin"]), dev2["cache_k_scale"], dev2["cache_v_scale"],
                                    sqattn_per_token=True, workspace=ws, **kw)
        live = [t for b in range(len(enc)) for t in range(cu[b], cu[b + 1])]
        assert torch.equal(again[live], out[live])
    # one sized for the batch alone is refused before anything is written
    small = torch.empty(append_attention_workspace_bytes(c["T"], len(enc), hq, hkv, d, bt.shape[1], 1), dtype=torch.uint8,
                        device="cuda")
    with pytest.raises(ValueError, match="sqattn_per_token"):
        fd.append_attention(*args(), sqattn_per_token=True, workspace=small, **kw)


@pytest.mark.parametrize("quant,hq,hkv,tokens", [(CACHE_INT8, 32, 8, 2), (CACHE_FP8, 32, 8, 2), (CACHE_INT8_DYNAMIC, 32, 8, 2),
                                                 (CACHE_FP8_DYNAMIC, 16, 8, 4), (CACHE_INT8, 8, 8, 8), (CACHE_INT8_BLOCK, 32, 8, 2),
                                                 (CACHE_INT8, 24, 8, 2),
                                                 # more than 8 (token, head) pairs per KV head: the fp16-MFMA decode kernel's 16 columns
                                                 (CACHE_INT8, 32, 8, 4), (CACHE_FP8, 32, 8, 3), (CACHE_INT8_DYNAMIC, 32, 8, 4),
                                                 (CACHE_FP8_BLOCK, 24, 8, 5), (CACHE_FP8_DYNAMIC, 8, 8, 16), (CACHE_INT8, 40, 8, 3)])
def test_mixed_step_with_decode_rows_of_several_tokens(oracle, quant, hq, hkv, tokens):
    """decode_tokens in the one-call step: a row with seq_lens_encoder 0 and 2 .. decode_tokens tokens (speculative
    drafts) is served by the decode kernel in one pass - token t attends to cached + t + 1 tokens, all read back from
    the quantised cache.  Against the oracle: its writer, then one decode per token with that token's length (block
    boundaries inside the new tokens, a first step on an empty cache, rows of fewer tokens, a long row in several
    chunks); the prefill row and the one-token rows as ever; rows with more tokens than decode_tokens get none."""
    T = tokens
    enc = [0, 40, 0, 0, 0, 0, 0, 0]
    dec = [63, 100, 0, 64 * 3 - 1, 500, 64 * 70 + 3, 64 * 2 - T + 1, 77]
    this = [T, 40, T, T, 1, T, T - 1 if T > 2 else 1, T + 1]
    c = mixed_case(enc, dec, quant, seed=50 + T, hq=hq, hkv=hkv, max_pos=8192, this=this)
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    out = torch.full((c["T"], hq * 128), float("nan"), dtype=torch.bfloat16, device="cuda")
    fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                        dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                        (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                        num_heads=hq, kv_num_heads=hkv, max_chunk=40, cache_quant_type=quant,
                        cu_seqlens_q=dev["cu_seqlens_q"], prefill_rows=1, decode_tokens=T, out=out)
    torch.cuda.synchronize()
    kc, vc = np_of(c["key_cache"]).copy(), np_of(c["value_cache"]).copy()
    ks, vs = np_of(c["cache_k_scale"]).copy(), np_of(c["cache_v_scale"]).copy()
    bt, cu, decs = np_of(c["block_tables"]), np_of(c["cu_seqlens_q"]), np_of(c["seq_lens_decoder"])
    q, k_new, v_new = oracle.write_cache_kv(bits(c["qkv"]), kc, vc, ks, vs, np_of(c["rope_cos"]), np_of(c["rope_sin"]),
                                            bt, decs, cu, hq, hkv, 128, 1, quant, want_kv_out=True)
    assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc)
    got = bits(out)
    for b in range(len(enc)):
        rows = list(range(cu[b], cu[b + 1]))
        if enc[b] > 0:
            want = oracle.append_attention_prefill(q, k_new, v_new, kc, vc, ks, vs, bt, decs, cu, hq, hkv, 128, quant,
                                                   token_ids=np.array(rows, np.int32))[rows]
        elif this[b] <= T:   # every token of the row: one decode over its own length
            want = oracle.decode_attention(np.ascontiguousarray(q[rows]), kc, vc, ks, vs,
                                           np.ascontiguousarray(np.repeat(bt[b:b + 1], len(rows), 0)),
                                           np.array([decs[b] + t + 1 for t in range(len(rows))], np.int32),
                                           hq, hkv, 128, quant)
        else:                # too many tokens for a decode row: written to the cache, no attention output
            assert torch.isnan(out[rows].float()).all()
            continue
        ok, mx, bad = bf16_close(got[rows], want)
        assert ok, "sequence %d: %d out of tolerance, max %.4g" % (b, bad, mx)


@pytest.mark.parametrize("quant,hq,hkv,tokens,d,bs", [
    (CACHE_INT8, 8, 4, 8, 64, 16),             # 2 heads per KV head x 8 tokens: all 16 columns; tiles of two blocks
    (CACHE_FP8, 16, 4, 4, 256, 64),            # 4 x 4
    (CACHE_INT8_DYNAMIC, 8, 1, 2, 128, 32),    # 8 x 2; a tile is a block
    (CACHE_FP8_BLOCK, 12, 4, 5, 64, 48),       # 3 x 5 = 15 columns; a block size that is no power of two
    (CACHE_INT8, 4, 4, 16, 256, 128),          # 1 x 16
    (CACHE_FP8_DYNAMIC, 6, 2, 3, 128, 16),     # 3 x 3
])
def test_mixed_step_with_decode_rows_of_several_tokens_other_shapes(oracle, quant, hq, hkv, tokens, d, bs):
    """decode_tokens at the shapes of the fp16-MFMA decode kernel (head_dim 64 / 128 / 256, any block size): the
    columns of its MFMAs are (token, query head) pairs, masked by column where the row's own tokens begin.  Same
    check as at the int8-MFMA kernel's shape: the oracle's writer, then one decode per token with that token's length."""
    T = tokens
    enc = [0, 40, 0, 0, 0, 0, 0, 0]
    dec = [bs - 1, 100, 0, bs * 3 - 1, 500, bs * 20 + 3, bs * 2 - T + 1, 77]
    this = [T, 40, T, T, 1, T, T - 1 if T > 2 else 1, T + 1]
    c = mixed_case(enc, dec, quant, seed=60 + T, hq=hq, hkv=hkv, d=d, bs=bs, max_pos=4096, this=this)
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    out = torch.full((c["T"], hq * d), float("nan"), dtype=torch.bfloat16, device="cuda")
    fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                        dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                        (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                        num_heads=hq, kv_num_heads=hkv, max_chunk=40, cache_quant_type=quant,
                        cu_seqlens_q=dev["cu_seqlens_q"], prefill_rows=1, decode_tokens=T, out=out)
    torch.cuda.synchronize()
    kc, vc = np_of(c["key_cache"]).copy(), np_of(c["value_cache"]).copy()
    ks, vs = np_of(c["cache_k_scale"]).copy(), np_of(c["cache_v_scale"]).copy()
    bt, cu, decs = np_of(c["block_tables"]), np_of(c["cu_seqlens_q"]), np_of(c["seq_lens_decoder"])
    q, k_new, v_new = oracle.write_cache_kv(bits(c["qkv"]), kc, vc, ks, vs, np_of(c["rope_cos"]), np_of(c["rope_sin"]),
                                            bt, decs, cu, hq, hkv, d, 1, quant, want_kv_out=True)
    assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc)
    got = bits(out)
    for b in range(len(enc)):
        rows = list(range(cu[b], cu[b + 1]))
        if enc[b] > 0:
            want = oracle.append_attention_prefill(q, k_new, v_new, kc, vc, ks, vs, bt, decs, cu, hq, hkv, d, quant,
                                                   token_ids=np.array(rows, np.int32))[rows]
        elif this[b] <= T:   # every token of the row: one decode over its own length
            want = oracle.decode_attention(np.ascontiguousarray(q[rows]), kc, vc, ks, vs,
                                           np.ascontiguousarray(np.repeat(bt[b:b + 1], len(rows), 0)),
                                           np.array([decs[b] + t + 1 for t in range(len(rows))], np.int32),
                                           hq, hkv, d, quant)
        else:                # too many tokens for a decode row: written to the cache, no attention output
            assert torch.isnan(out[rows].float()).all()
            continue
        ok, mx, bad = bf16_close(got[rows], want)
        assert ok, "sequence %d: %d out of tolerance, max %.4g" % (b, bad, mx)


def test_decode_tokens_argument_checks():
    c = mixed_case([0, 0], [10, 20], CACHE_INT8, seed=1, this=[2, 2])
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    for kw in (dict(decode_tokens=5), dict(decode_tokens=5, sqattn_top_k=4)):   # 5 x 4 rows > 16, with or without the selector
        with pytest.raises(ValueError):
            fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                                dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                                (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                                num_heads=32, kv_num_heads=8, max_chunk=0, cu_seqlens_q=dev["cu_seqlens_q"], **kw)
    assert torch.equal(dev["key_cache"].cpu(), c["key_cache"])   # refused before anything was written


def test_step_output_is_the_out_projection_input_as_it_stands():
    """out is bf16 [num_tokens, num_heads * head_dim], row-major with the heads of a token side by side - the A operand
    of the out-projection GEMM.  The step writes it where the caller says (here: rows inside a larger activation
    buffer), the rows are dense (stride num_heads * head_dim, 16-byte aligned), and a GEMM reads them in place: its
    result equals that of a GEMM over a separately allocated copy, and nothing outside the rows is touched."""
    hq, hkv, d = 32, 8, 128
    c = mixed_case([0, 90, 0], [300, 0, 63], CACHE_INT8, seed=77)
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    T = c["T"]
    act = torch.full((T + 16, hq * d), 3.0, dtype=torch.bfloat16, device="cuda")
    view = act[7:7 + T]
    args = (dev["qkv"], dev["key_cache"].clone(), dev["value_cache"].clone(), dev["seq_lens_encoder"], dev["seq_lens_decoder"],
            dev["seq_lens_this_time"], dev["block_tables"], (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"],
            dev["cache_v_scale"])
    kw = dict(num_heads=hq, kv_num_heads=hkv, max_chunk=90, cu_seqlens_q=dev["cu_seqlens_q"])
    out = fd.append_attention(*args, out=view, **kw)
    fresh = fd.append_attention(args[0], dev["key_cache"].clone(), dev["value_cache"].clone(), *args[3:], **kw)
    torch.cuda.synchronize()
    assert out.data_ptr() == view.data_ptr() == act.data_ptr() + 7 * hq * d * 2
    assert out.shape == (T, hq * d) and out.stride() == (hq * d, 1) and out.is_contiguous() and out.data_ptr() % 16 == 0
    assert torch.equal(out, fresh)
    assert (act[:7] == 3.0).all() and (act[7 + T:] == 3.0).all()
    w_o = (torch.randn((hq * d, 512), generator=torch.Generator().manual_seed(1)) * 0.02).to(torch.bfloat16).cuda()
    assert torch.equal(out @ w_o, fresh.clone() @ w_o)                       # [T, hq*d] x [hq*d, hidden]
    assert torch.equal(out.view(T, hq, d)[:, 5], fresh[:, 5 * d:6 * d])      # head h of token t = columns h*d .. h*d+d-1
    with pytest.raises(ValueError):
        fd.append_attention(*args, out=act[:T - 1], **kw)


@pytest.mark.parametrize("enc,dec,hq,hkv,quant", [
    ([0, 200, 300, 0, 50], [700, 4500, 2100, 64, 3000], 32, 8, CACHE_INT8),      # three prefill rows: two splits each
    ([0, 40, 0, 64], [100, 5000, 30, 2500], 32, 8, CACHE_FP8),                   # short chunks, all heads of a KV head in a workgroup
    ([260, 0, 0], [6000, 900, 2000], 8, 2, CACHE_INT8_DYNAMIC),                  # two query tiles, few heads: eight splits
    ([0, 0, 0, 0], [500, 3000, 1, 64], 32, 8, CACHE_INT8),                       # no prefill row at all behind max_chunk > 0
    ([100] * 9 + [0], [3000] * 9 + [70], 32, 8, CACHE_FP8_BLOCK),                # enough prefill rows to fill the GPU: no splits
    # more sequences than a wavefront has lanes (the count and the merge's search for a token's sequence take several passes)
    ([0] * 70 + [300] + [0] * 60 + [40] + [0] * 5, [90 + 3 * i for i in range(70)] + [4000] + [0] * 30 + [64] * 30 + [2500] + [7] * 5, 8, 2, CACHE_INT8),
])
def test_mixed_step_counts_its_prefill_rows(oracle, enc, dec, hq, hkv, quant):
    """A step without the host's count of prefill rows: the prefill kernel counts them, splits the keys of their query
    tiles as the host would have for that count, and covers the further splits with a CU's worth of workgroups behind
    the grid over the batch.  Against the oracle, and bit for bit what the step with the count gives."""
    c = mixed_case(enc, dec, quant, seed=len(enc) + hq, hq=hq, hkv=hkv, max_pos=8192)
    rows, chunk = sum(1 for e in enc if e > 0), max(max(enc), 1)
    outs = []
    for hint in (None, rows):
        dev = {k: (v.clone().cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
        out = fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                                  dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                                  (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                                  num_heads=hq, kv_num_heads=hkv, max_chunk=chunk, cache_quant_type=quant,
                                  cu_seqlens_q=dev["cu_seqlens_q"], prefill_rows=hint or None)
        torch.cuda.synchronize()
        outs.append(bits(out))
        if hint is None:
            want, kc, vc = oracle_step(oracle, c, quant, hq, hkv, 128)
            assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc)
            ok, mx, bad = bf16_close(outs[0], want)
            assert ok, "%d out of tolerance, max %.4g" % (bad, mx)
    assert np.array_equal(outs[0], outs[1])


def random_steps(oracle, seed, iters):
    """Seeded random steps: 1 .. 8 slots that are prefill rows (1 .. 140 new tokens, with or without cached tokens),
    decode rows - of several draft tokens in some steps, block-sparse (top 1 .. 6 blocks) in some, with one block list
    per row or per token where both meet - or idle; 1 .. 8
    query heads per KV head; any cache format; with and without the prefill-row count.  Cache bytes (and scale
    caches) exact, outputs within tolerance."""
    rng = np.random.default_rng(seed)
    formats = [CACHE_INT8, CACHE_FP8, CACHE_INT8_DYNAMIC, CACHE_FP8_DYNAMIC, CACHE_INT8_BLOCK, CACHE_FP8_BLOCK]
    for it in range(iters):
        slots, group, hkv = int(rng.integers(1, 9)), int(rng.integers(1, 9)), int(rng.integers(1, 4))
        quant = formats[int(rng.integers(0, len(formats)))]
        tokens = int(rng.integers(1, 16 // group + 1)) if it % 3 == 2 else 1   # draft tokens a decode row may bring
        top_k = int(rng.integers(1, 7)) if it % 4 == 1 else 0                   # block-sparse decode rows
        per_token = it % 24 == 5   # (of the steps with both, every other one keeps a block list per token)
        enc, dec, this = [], [], []
        for _ in range(slots):
            kind = int(rng.integers(0, 4))   # prefill on nothing, prefill on a prefix, decode, idle
            enc.append(int(rng.integers(1, 141)) if kind < 2 else 0)
            dec.append(0 if kind in (0, 3) else int(rng.integers(1, 600)))
            this.append(enc[-1] if kind < 2 else (int(rng.integers(1, tokens + 1)) if kind == 2 else 0))
        if not any(this):
            dec[0], this[0] = 77, 1
        hq = group * hkv
        c = mixed_case(enc, dec, quant, seed=seed * 1000 + it, hq=hq, hkv=hkv, max_pos=1024, this=this)
        dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
        rows = sum(1 for e in enc if e > 0)
        out = fd.append_attention(dev["qkv"], dev["key_cache"], dev["value_cache"], dev["seq_lens_encoder"],
                                  dev["seq_lens_decoder"], dev["seq_lens_this_time"], dev["block_tables"],
                                  (dev["rope_cos"], dev["rope_sin"]), dev["cache_k_scale"], dev["cache_v_scale"],
                                  num_heads=hq, kv_num_heads=hkv, max_chunk=max(enc), cache_quant_type=quant,
                                  cu_seqlens_q=dev["cu_seqlens_q"], prefill_rows=rows if it % 2 else None,
                                  decode_tokens=tokens, sqattn_top_k=top_k, sqattn_per_token=per_token)
        torch.cuda.synchronize()
        what = "seed %d step %d: enc %r dec %r this %r group %d hkv %d quant %d tokens %d top_k %d per token %d" % (
            seed, it, enc, dec, this, group, hkv, quant, tokens, top_k, per_token)
        want, kc, vc = oracle_step(oracle, c, quant, hq, hkv, 128, decode_tokens=tokens, top_k=top_k,
                                   per_token=per_token and tokens > 1 and top_k > 0)
        assert np.array_equal(np_of(dev["key_cache"]), kc) and np.array_equal(np_of(dev["value_cache"]), vc), what
        if is_dynamic(quant):
            assert np.array_equal(np_of(dev["cache_k_scale"]), c["scales_after"][0]), what
            assert np.array_equal(np_of(dev["cache_v_scale"]), c["scales_after"][1]), what
        ok, mx, bad = bf16_close(bits(out), want)
        assert ok, "%s: %d out of tolerance, max %.4g" % (what, bad, mx)


def test_mixed_step_random_batches_against_the_oracle(oracle):
    random_steps(oracle, 7, 30)


def test_steps_over_block_pool_tables_with_a_shared_prefix(oracle):
    """Two steps driven by the block pool's tables: a prompt is prefilled, a second sequence forks its
    whole blocks and prefills only its own tail while the first decodes and a third arrives.  Every step is
    checked against the oracle on the same tables; the fork's outputs must also be bit-identical to those
    of a run whose prefix blocks are private copies."""
    from fastdeploy_amd.block_pool import BlockPool
    hq, hkv, d, bs, quant = 32, 8, 128, 64, CACHE_INT8
    g = torch.Generator().manual_seed(21)
    pool = BlockPool(num_blocks=24, block_size=bs, max_seqs=4, max_blocks_per_seq=6)
    ks = ((torch.rand((hkv, d), generator=g) * 2 + 2.0) / 127.0).contiguous()
    vs = ((torch.rand((hkv, d), generator=g) * 2 + 2.0) / 127.0).contiguous()
    cos, sin = rope_table(1024, d, 500000.0, "cpu")
    kc = torch.zeros((24, hkv, bs, d), dtype=torch.uint8)
    vc = torch.zeros_like(kc)
    kc_d, vc_d = kc.cuda(), vc.cuda()

    def step(enc, dec, tables, kc_dev, vc_dev, qkv):
        enc_t, dec_t = torch.tensor(enc, dtype=torch.int32), torch.tensor(dec, dtype=torch.int32)
        this = seq_lens_this_time_of(enc_t, dec_t)
        cu = cu_seqlens_of(this)
        c = dict(qkv=qkv, key_cache=kc_dev.cpu(), value_cache=vc_dev.cpu(), cache_k_scale=ks, cache_v_scale=vs,
                 block_tables=torch.from_numpy(np.array(tables)), seq_lens_encoder=enc_t, seq_lens_decoder=dec_t,
                 seq_lens_this_time=this, cu_seqlens_q=cu, rope_cos=cos, rope_sin=sin, T=int(cu[-1]))
        out = fd.append_attention(qkv.cuda(), kc_dev, vc_dev, enc_t.cuda(), dec_t.cuda(), this.cuda(),
                                  c["block_tables"].cuda(), (cos.cuda(), sin.cuda()), ks.cuda(), vs.cuda(),
                                  num_heads=hq, kv_num_heads=hkv, max_chunk=max(enc), cache_quant_type=quant,
                                  cu_seqlens_q=cu.cuda())
        torch.cuda.synchronize()
        want, kc_w, vc_w = oracle_step(oracle, c, quant)
        assert np.array_equal(np_of(kc_dev), kc_w) and np.array_equal(np_of(vc_dev), vc_w)
        ok, mx, bad = bf16_close(bits(out), want)
        assert ok, "%d out of tolerance, max %.4g" % (bad, mx)
        return out, cu

    width = (hq + 2 * hkv) * d
    # step 1: sequence 0 prefills a 200-token prompt
    pool.reserve(0, 200)
    step([200, 0, 0, 0], [0, 0, 0, 0], pool.block_tables, kc_d, vc_d,
         torch.randn((200, width), generator=g).to(torch.bfloat16))
    # step 2: slot 1 shares the prompt's three whole blocks and prefills 38 tokens of its own from position 192,
    # slot 0 decodes, slot 2 arrives with 70 tokens, slot 3 idles
    assert pool.fork(0, 1, 200) == 192
    pool.reserve(1, 192 + 38)
    pool.reserve(0, 201)
    pool.reserve(2, 70)
    assert pool.block_tables[1, :3].tolist() == pool.block_tables[0, :3].tolist()
    enc, dec = [0, 38, 70, 0], [200, 192, 0, 0]
    qkv2 = torch.randn((1 + 38 + 70, width), generator=g).to(torch.bfloat16)
    kc_p, vc_p = kc_d.clone(), vc_d.clone()                 # the state before step 2, for the private-copy run
    out_shared, cu = step(enc, dec, pool.block_tables, kc_d, vc_d, qkv2)
    # the same step with private copies of the prefix blocks (blocks 20..22 are unused by the pool so far)
    private = np.array(pool.block_tables)
    src = torch.from_numpy(private[0, :3].astype(np.int64)).cuda()
    dst = torch.tensor([20, 21, 22]).cuda()
    kc_p[dst], vc_p[dst] = kc_p[src], vc_p[src]
    private[1, :3] = [20, 21, 22]
    out_private, _ = step(enc, dec, private, kc_p, vc_p, qkv2)
    assert torch.equal(out_shared.view(torch.int16), out_private.view(torch.int16))
    pool.release(1)
    assert pool.refcount(int(private[0, 0])) == 1 and pool.free_blocks == 24 - 4 - 2
