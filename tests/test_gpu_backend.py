"""The attention backend over several steps and layers: prompts of different lengths arrive, are
prefilled in chunks, decode, fork and finish; every step of every layer is checked against the oracle
run on the same cache state (cache bytes exact, outputs within the path's tolerance)."""
import numpy as np
import pytest
import torch

import fastdeploy_amd as fd
from conftest import bf16_close, bits, np_of
from fastdeploy_amd.ops import CACHE_FP8_BLOCK, CACHE_INT8, CACHE_INT8_DYNAMIC, is_dynamic
from test_gpu_mixed_step import oracle_step

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("quant", [CACHE_INT8, CACHE_INT8_DYNAMIC, CACHE_FP8_BLOCK])
def test_generation_over_steps_and_layers(oracle, quant):
    hq, hkv, d, bs, layers = 32, 8, 128, 64, 2
    g = torch.Generator().manual_seed(31)
    be = fd.AppendAttentionBackend(hq, hkv, d, block_size=bs, max_position=1024, rope_theta=500000.0,
                                   cache_quant_type=quant)
    pool = fd.BlockPool(num_blocks=40, block_size=bs, max_seqs=5, max_blocks_per_seq=8)
    book = fd.SequenceBook(pool)
    lay = []
    for l in range(layers):
        ks = (torch.rand((hkv, d), generator=g) * 2 + 2.0) / 127.0
        vs = (torch.rand((hkv, d), generator=g) * 2 + 2.0) / 127.0
        extra = {}
        if l == 1:   # the second layer has the projection epilogue
            extra = dict(qkv_bias=(torch.randn((48 * d,), generator=g) * 0.25).to(torch.bfloat16).cuda(),
                         q_norm_weight=(torch.rand((d,), generator=g) + 0.5).cuda(),
                         k_norm_weight=(torch.rand((d,), generator=g) + 0.5).cuda(), rms_norm_eps=1e-6)
        lay.append(be.allocate_layer(40, **extra) if is_dynamic(quant) else be.allocate_layer(40, ks, vs, **extra))
    cos, sin = (t.cpu() for t in be.rotary_embs)

    def run_step(new_tokens, drafts=(), accepted=None):
        meta = be.init_attention_metadata(book.schedule(new_tokens, drafts))
        for l, layer in enumerate(lay):
            qkv = torch.randn((meta.num_tokens, 48 * d), generator=g).to(torch.bfloat16)
            before = dict(qkv=qkv, key_cache=layer.key_cache.cpu(), value_cache=layer.value_cache.cpu(),
                          cache_k_scale=layer.cache_k_scale.cpu(), cache_v_scale=layer.cache_v_scale.cpu(),
                          block_tables=meta.block_tables.cpu(), seq_lens_encoder=meta.seq_lens_encoder.cpu(),
                          seq_lens_decoder=meta.seq_lens_decoder.cpu(), seq_lens_this_time=meta.seq_lens_this_time.cpu(),
                          cu_seqlens_q=meta.cu_seqlens_q.cpu(), rope_cos=cos, rope_sin=sin, T=meta.num_tokens)
            out = be.forward_mixed(qkv.cuda(), layer, meta)
            torch.cuda.synchronize()
            ep = {}
            if layer.qkv_bias is not None:
                ep = dict(qkv_bias=bits(layer.qkv_bias), q_norm_weight=np_of(layer.q_norm_weight),
                          k_norm_weight=np_of(layer.k_norm_weight), rms_norm_eps=layer.rms_norm_eps)
            want, kc, vc = oracle_step(oracle, before, quant, decode_tokens=meta.decode_tokens, **ep)
            assert np.array_equal(np_of(layer.key_cache), kc) and np.array_equal(np_of(layer.value_cache), vc)
            if is_dynamic(quant):  # the scale caches follow the stored rows
                assert np.array_equal(np_of(layer.cache_k_scale), before["scales_after"][0])
                assert np.array_equal(np_of(layer.cache_v_scale), before["scales_after"][1])
            ok, mx, bad = bf16_close(bits(out), want)
            assert ok, "layer %d, step %r: %d out of tolerance, max %.4g" % (l, new_tokens, bad, mx)
        book.commit(accepted)

    run_step({0: 150, 1: 3})                 # two prompts
    run_step({0: 1, 1: 1, 2: 200})           # both decode while a third prompt's first chunk arrives
    run_step({0: 1, 1: 1, 2: 77})            # the third prompt's second chunk, on its cached first one
    assert book.fork(2, 3) == 256            # a fourth sequence continues from the third's four whole blocks
    run_step({0: 1, 2: 1, 3: 30})            # slot 1 idles; the fork prefills its own tail
    book.finish(1)
    run_step({0: 1, 2: 1, 3: 1, 4: 1})       # a one-token prompt in slot 4
    assert book.lengths == [154, 0, 279, 287, 1]
    # a speculative step: slots 0 and 2 bring two draft tokens each (decode rows of two tokens), slot 3 decodes;
    # slot 0's second draft is rejected, so its next token overwrites that position
    run_step({0: 2, 2: 2, 3: 1}, drafts={0, 2}, accepted={0: 1})
    assert book.lengths == [155, 0, 281, 288, 1]
    run_step({0: 2, 2: 1, 3: 1}, drafts={0})
    assert book.lengths == [157, 0, 282, 289, 1]
    assert pool.refcount(int(pool.block_tables[2, 0])) == 2


def test_backend_refuses_draft_rows_its_decode_kernel_cannot_take():
    """8 query heads per KV head leave no room for a third token in the decode kernel's 16 rows: the metadata step
    says so (the scheduler should send such rows as prefill rows) instead of the kernel call failing later."""
    be = fd.AppendAttentionBackend(64, 8, 128, block_size=64, max_position=256)
    pool = fd.BlockPool(num_blocks=8, block_size=64, max_seqs=2, max_blocks_per_seq=4)
    book = fd.SequenceBook(pool)
    be.init_attention_metadata(book.schedule({0: 5}))
    book.commit()
    with pytest.raises(ValueError, match="prefill rows"):
        be.init_attention_metadata(book.schedule({0: 3}, drafts={0}))
    meta = be.init_attention_metadata(book.schedule({0: 3}))     # the same tokens as a prefill row: fine
    assert meta.decode_tokens == 1 and meta.prefill_rows == 1


def test_backend_with_a_block_list_per_draft_token(oracle):
    """sqattn_per_token on the backend: the same 3 draft tokens at 8 query heads per KV head that the one-list step
    refuses are decode rows here, every token with its own top-k blocks (the decode side runs over tokens as rows, so
    the rows-per-KV-head limit of the kernels for rows of several tokens does not apply); each step against the oracle."""
    hq, hkv, d, bs, top_k = 64, 8, 128, 64, 3
    g = torch.Generator().manual_seed(77)
    be = fd.AppendAttentionBackend(hq, hkv, d, block_size=bs, max_position=1024, rope_theta=500000.0, sqattn_top_k=top_k,
                                   sqattn_per_token=True)
    pool = fd.BlockPool(num_blocks=24, block_size=bs, max_seqs=3, max_blocks_per_seq=8)
    book = fd.SequenceBook(pool)
    ks = (torch.rand((hkv, d), generator=g) * 2 + 2.0) / 127.0
    vs = (torch.rand((hkv, d), generator=g) * 2 + 2.0) / 127.0
    layer = be.allocate_layer(24, ks, vs)
    cos, sin = (t.cpu() for t in be.rotary_embs)
    for new_tokens, drafts in (({0: 380, 1: 200}, ()), ({0: 3, 1: 1}, {0}), ({0: 2, 1: 3, 2: 9}, {0, 1})):
        meta = be.init_attention_metadata(book.schedule(new_tokens, drafts))
        qkv = torch.randn((meta.num_tokens, (hq + 2 * hkv) * d), generator=g).to(torch.bfloat16)
        before = dict(qkv=qkv, key_cache=layer.key_cache.cpu(), value_cache=layer.value_cache.cpu(),
                      cache_k_scale=layer.cache_k_scale.cpu(), cache_v_scale=layer.cache_v_scale.cpu(),
                      block_tables=meta.block_tables.cpu(), seq_lens_encoder=meta.seq_lens_encoder.cpu(),
                      seq_lens_decoder=meta.seq_lens_decoder.cpu(), seq_lens_this_time=meta.seq_lens_this_time.cpu(),
                      cu_seqlens_q=meta.cu_seqlens_q.cpu(), rope_cos=cos, rope_sin=sin, T=meta.num_tokens)
        out = be.forward_mixed(qkv.cuda(), layer, meta)
        torch.cuda.synchronize()
        want, kc, vc = oracle_step(oracle, before, CACHE_INT8, hq=hq, hkv=hkv, decode_tokens=meta.decode_tokens,
                                   top_k=top_k, per_token=True)
        assert np.array_equal(np_of(layer.key_cache), kc) and np.array_equal(np_of(layer.value_cache), vc)
        ok, mx, bad = bf16_close(bits(out), want)
        assert ok, "step %r: %d out of tolerance, max %.4g" % (new_tokens, bad, mx)
        book.commit()
    assert book.lengths == [385, 204, 9]
