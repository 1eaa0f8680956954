"""The decode entry point that allocates nothing (fdattn_decode_attention_noalloc): its split-KV partials live in the
library's own device array instead of a caller's workspace.  Through the C ABI, its output must equal that of
fdattn_decode_attention bit for bit (the same kernels run), on two calls in a row, the second with a smaller input,
and shapes beyond the array's size must be refused before anything is enqueued."""
import ctypes

import numpy as np
import pytest
import torch

from conftest import bf16_close, bits, np_of
from fastdeploy_amd import _lib
from fastdeploy_amd import synthetic as syn

pytestmark = pytest.mark.gpu


def _call_pair(lib, case, partials=True):
    """(output of fdattn_decode_attention_noalloc, output of fdattn_decode_attention) on the same device tensors."""
    dev = syn.to_device(case, "cuda")
    batch, mb = dev["block_tables"].shape
    nb, hkv, bs, d = dev["key_cache"].shape
    hq, quant = case["hq"], case["quant"]
    if partials:
        assert lib.fdattn_decode_chunks_per_sequence(batch, hkv, mb) > 1, "the case must leave partials in the scratch"
    stream = torch.cuda.current_stream().cuda_stream
    ptrs = [dev[k].data_ptr() for k in ("q", "key_cache", "value_cache", "cache_k_scale", "cache_v_scale",
                                        "block_tables", "seq_lens_decoder")] + [None]
    dims = [batch, hq, hkv, d, bs, mb, nb, quant]
    scale = 1.0 / np.sqrt(d)
    got = torch.full((batch, hq * d), float("nan"), dtype=torch.bfloat16, device="cuda")
    want = torch.full_like(got, float("nan"))
    rc = lib.fdattn_decode_attention_noalloc(*ptrs, got.data_ptr(), *dims, scale, stream)
    assert rc == 0, lib.fdattn_last_error()
    n = lib.fdattn_decode_workspace_bytes(batch, hq, hkv, d, mb)
    ws = torch.empty(n, dtype=torch.uint8, device="cuda")
    rc = lib.fdattn_decode_attention(*ptrs, want.data_ptr(), ws.data_ptr(), n, *dims, scale, stream)
    assert rc == 0, lib.fdattn_last_error()
    torch.cuda.synchronize()
    return bits(got), bits(want)


@pytest.mark.parametrize("quant", [1, 2, 3, 4])
def test_noalloc_decode_equals_the_workspace_entry_point_twice_in_a_row(oracle, quant):
    lib = _lib.lib()
    assert lib.fdattn_decode_noalloc_scratch_bytes() == 16 << 20
    # two sequences of 128 / 100 blocks: 16 (sequence, KV head) lists cut into many chunks, partials + merge kernel
    first = syn.decode_case(batch=2, ctx=[8192, 6345], quant=quant, seed=11)
    # then a smaller input over the same scratch: stale partials of the first call lie beyond what this one writes
    second = syn.decode_case(batch=1, ctx=[2999], quant=quant, seed=12)
    for name, case in (("first", first), ("second, smaller", second)):
        got, want = _call_pair(lib, case)
        assert np.array_equal(got, want), "%s call: outputs of the two entry points differ" % name
        ref = oracle.decode_attention(bits(case["q"]), np_of(case["key_cache"]), np_of(case["value_cache"]),
                                      np_of(case["cache_k_scale"]), np_of(case["cache_v_scale"]),
                                      np_of(case["block_tables"]), np_of(case["seq_lens_decoder"]), case["hq"],
                                      case["hkv"], case["d"], case["quant"])
        ok, mx, bad = bf16_close(got, ref)
        assert ok, "%s call vs the oracle: %d out of tolerance, max abs %.4g" % (name, bad, mx)


def test_noalloc_decode_takes_the_headline_shape():
    """Batch 64 x 32 / 8 heads x head_dim 128 over 72-block tables: the int8-MFMA kernel needs 1 MiB of partials at most
    (none in fact: every list is one chunk), well inside the scratch, whatever the other kernels would need there."""
    lib = _lib.lib()
    g = torch.Generator().manual_seed(3)
    lens = torch.randint(3584, 4609, (64,), generator=g).tolist()
    case = syn.decode_case(batch=64, ctx=lens, pool_blocks=6000, seed=2, device="cuda", max_blocks=72)
    got, want = _call_pair(lib, case, partials=False)
    assert np.array_equal(got, want), "headline shape: outputs of the two entry points differ"
    # and a batch of the same sequences small enough to be cut into chunks (partials + merge), right after it
    small = {k: (v[:5].contiguous() if k in ("q", "block_tables", "seq_lens_decoder") else v) for k, v in case.items()}
    got, want = _call_pair(lib, small)
    assert np.array_equal(got, want), "5 of the 64 sequences: outputs of the two entry points differ"


def test_noalloc_decode_on_the_shape_agnostic_kernel_and_its_limit():
    lib = _lib.lib()
    # head_dim 64 runs on the shape-agnostic kernel, whose partials use the same scratch
    for case in (syn.decode_case(batch=3, ctx=[700, 64, 1500], d=64, seed=13), syn.decode_case(batch=1, ctx=[130], d=64, seed=14)):
        dev = syn.to_device(case, "cuda")
        batch, mb = dev["block_tables"].shape
        nb, hkv, bs, d = dev["key_cache"].shape
        stream = torch.cuda.current_stream().cuda_stream
        ptrs = [dev[k].data_ptr() for k in ("q", "key_cache", "value_cache", "cache_k_scale", "cache_v_scale",
                                            "block_tables", "seq_lens_decoder")] + [None]
        dims = [batch, case["hq"], hkv, d, bs, mb, nb, case["quant"]]
        got = torch.full((batch, case["hq"] * d), float("nan"), dtype=torch.bfloat16, device="cuda")
        want = torch.full_like(got, float("nan"))
        assert lib.fdattn_decode_attention_noalloc(*ptrs, got.data_ptr(), *dims, 0.125, stream) == 0, lib.fdattn_last_error()
        n = lib.fdattn_decode_workspace_bytes(batch, case["hq"], hkv, d, mb)
        ws = torch.empty(n, dtype=torch.uint8, device="cuda")
        assert lib.fdattn_decode_attention(*ptrs, want.data_ptr(), ws.data_ptr(), n, *dims, 0.125, stream) == 0
        torch.cuda.synchronize()
        assert np.array_equal(bits(got), bits(want))
    # beyond the scratch: refused with a message, nothing enqueued (the pointers are never touched)
    one = ctypes.c_void_p(256)
    big_batch = 9000
    assert lib.fdattn_decode_workspace_bytes(big_batch, 32, 8, 128, 72) > lib.fdattn_decode_noalloc_scratch_bytes()
    rc = lib.fdattn_decode_attention_noalloc(*([one] * 7), None, one, big_batch, 32, 8, 128, 64, 72, 6000, 1, 0.1, None)
    assert rc == -4 and b"static scratch" in lib.fdattn_last_error()
