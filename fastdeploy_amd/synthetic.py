"""Seeded synthetic workloads of the paged-KV attention path (inputs only: the caches
are filled with torch ops that restate the quantisation formulas, never with the
kernels under test).  Used by the tests, the smoke run and bench.py.

Shapes default to the Llama-3-8B attention layer: 32 query heads, 8 KV heads,
head_dim 128, block_size 64.
"""
import math

import torch

from .ops import CACHE_FP8, CACHE_INT8, byte_format, is_dynamic

HQ, HKV, D, BS = 32, 8, 128, 64


def quantize_ref(x, scale, quant):
    """fp32 x / scale -> cache bytes (uint8 view), the formulas of the cache format."""
    r = x.float() / scale
    if byte_format(quant) == CACHE_INT8:
        return torch.clamp(torch.round(r), -127, 127).to(torch.int8).view(torch.uint8)
    return torch.clamp(r, -448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)


def dequantize_ref(c, scale, quant):
    if byte_format(quant) == CACHE_INT8:
        return c.view(torch.int8).float() * scale
    return c.view(torch.float8_e4m3fn).float() * scale


def _gen(seed, device):
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def make_block_tables(ctx_lens, pool_blocks, bs, gen, device, max_blocks=None):
    """Random permutation of the pool handed out sequence by sequence; -1 padding."""
    need = [(int(c) + bs - 1) // bs for c in ctx_lens]
    mb = max_blocks or max(max(need), 1)
    assert sum(need) <= pool_blocks, "pool too small: need %d blocks, have %d" % (sum(need), pool_blocks)
    perm = torch.randperm(pool_blocks, generator=gen, device=device).to(torch.int32)
    bt = torch.full((len(ctx_lens), mb), -1, dtype=torch.int32, device=device)
    o = 0
    for b, n in enumerate(need):
        bt[b, :n] = perm[o:o + n]
        o += n
    return bt


def decode_case(batch=4, ctx=1024, pool_blocks=None, quant=CACHE_INT8, seed=0, device="cpu",
                hq=HQ, hkv=HKV, d=D, bs=BS, direct_bytes=False, extra_blocks=0, salient=0.0,
                max_blocks=None, row_log2=(-3, 3)):
    """A decode-attention case with a pre-filled cache.

    ctx: an int (every sequence), a (lo, hi) tuple (uniform, inclusive) or a list.
    direct_bytes: draw the cache bytes directly (values do not matter for bandwidth);
    otherwise K, V ~ N(0,1) bf16 quantised with per-channel scales = max-abs/127 (int8)
    or max-abs/448 (fp8).  salient: fraction of (sequence, block) pairs whose K is x4.
    The dynamic formats get scale caches [pool, hkv, bs]: every stored row's own max-abs/127 (/448)
    with the rows scaled by 2^U{row_log2} so that the scales differ widely, or (direct_bytes) random ones;
    the slots of no token hold NaN there, which nothing may read.
    """
    g = _gen(seed, device)
    if isinstance(ctx, tuple):
        lens = torch.randint(ctx[0], ctx[1] + 1, (batch,), generator=g, device=device).tolist()
    elif isinstance(ctx, int):
        lens = [ctx] * batch
    else:
        lens = list(ctx)
    need = sum((c + bs - 1) // bs for c in lens)
    pool = pool_blocks or (need + extra_blocks)
    bt = make_block_tables(lens, pool, bs, g, device, max_blocks)
    q = torch.randn((batch, hq * d), generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
    dyn, fmt = is_dynamic(quant), byte_format(quant)
    qmax = 127.0 if fmt == CACHE_INT8 else 448.0
    kc = torch.zeros((pool, hkv, bs, d), dtype=torch.uint8, device=device)
    vc = torch.zeros((pool, hkv, bs, d), dtype=torch.uint8, device=device)
    if direct_bytes:
        if fmt == CACHE_INT8:
            kc = torch.randint(-127, 128, kc.shape, generator=g, device=device, dtype=torch.int8).view(torch.uint8)
            vc = torch.randint(-127, 128, vc.shape, generator=g, device=device, dtype=torch.int8).view(torch.uint8)
        else:  # any finite e4m3 code: magnitude field 0..0x7e, random sign
            mk = torch.randint(0, 0x7F, kc.shape, generator=g, device=device, dtype=torch.uint8)
            mv = torch.randint(0, 0x7F, vc.shape, generator=g, device=device, dtype=torch.uint8)
            sk = torch.randint(0, 2, kc.shape, generator=g, device=device, dtype=torch.uint8) << 7
            sv = torch.randint(0, 2, vc.shape, generator=g, device=device, dtype=torch.uint8) << 7
            kc, vc = mk | sk, mv | sv
        ks = (torch.rand((hkv, d), generator=g, device=device) * 0.02 + 0.02) * (127.0 / qmax)
        vs = (torch.rand((hkv, d), generator=g, device=device) * 0.02 + 0.02) * (127.0 / qmax)
        if fmt == CACHE_FP8:
            ks, vs = ks * 0.05, vs * 0.05  # e4m3 codes reach 448: keep logits in a sane range
        if dyn:
            sc = 127.0 / qmax * (0.05 if fmt == CACHE_FP8 else 1.0)
            ks = (torch.rand((pool, hkv, bs), generator=g, device=device) * 0.03 + 0.01) * sc
            vs = (torch.rand((pool, hkv, bs), generator=g, device=device) * 0.03 + 0.01) * sc
    elif dyn:
        ks = torch.full((pool, hkv, bs), float("nan"), device=device)
        vs = torch.full((pool, hkv, bs), float("nan"), device=device)
        for b, n in enumerate(lens):
            if n == 0:
                continue
            k = torch.randn((n, hkv, d), generator=g, device=device).to(torch.bfloat16).float()
            v = torch.randn((n, hkv, d), generator=g, device=device).to(torch.bfloat16).float()
            k = k * torch.exp2(torch.randint(row_log2[0], row_log2[1] + 1, (n, hkv, 1), generator=g, device=device).float())
            v = v * torch.exp2(torch.randint(row_log2[0], row_log2[1] + 1, (n, hkv, 1), generator=g, device=device).float())
            if salient > 0:
                nb = (n + bs - 1) // bs
                pick = torch.rand((nb,), generator=g, device=device) < salient
                k = k * (1.0 + 3.0 * pick.repeat_interleave(bs)[:n].float())[:, None, None]
            sk, sv = k.abs().amax(-1) / qmax, v.abs().amax(-1) / qmax  # [n, hkv]
            sk, sv = torch.where(sk > 0, sk, torch.ones_like(sk)), torch.where(sv > 0, sv, torch.ones_like(sv))
            nb = (n + bs - 1) // bs
            pad = nb * bs - n
            kq, vq = quantize_ref(k, sk[..., None], quant), quantize_ref(v, sv[..., None], quant)
            if pad:
                z = torch.zeros((pad, hkv, d), dtype=torch.uint8, device=device)
                kq, vq = torch.cat([kq, z]), torch.cat([vq, z])
                nanpad = torch.full((pad, hkv), float("nan"), device=device)
                sk, sv = torch.cat([sk, nanpad]), torch.cat([sv, nanpad])
            idx = bt[b, :nb].long()
            kc[idx] = kq.view(nb, bs, hkv, d).permute(0, 2, 1, 3)
            vc[idx] = vq.view(nb, bs, hkv, d).permute(0, 2, 1, 3)
            ks[idx] = sk.view(nb, bs, hkv).permute(0, 2, 1)
            vs[idx] = sv.view(nb, bs, hkv).permute(0, 2, 1)
    else:
        ks_acc = torch.zeros((hkv, d), device=device)
        vs_acc = torch.zeros((hkv, d), device=device)
        ktoks, vtoks = [], []
        for b, n in enumerate(lens):
            k = torch.randn((n, hkv, d), generator=g, device=device).to(torch.bfloat16).float()
            v = torch.randn((n, hkv, d), generator=g, device=device).to(torch.bfloat16).float()
            if salient > 0:
                nb = (n + bs - 1) // bs
                pick = torch.rand((nb,), generator=g, device=device) < salient
                k = k * (1.0 + 3.0 * pick.repeat_interleave(bs)[:n].float())[:, None, None]
            ktoks.append(k)
            vtoks.append(v)
            if n:
                ks_acc = torch.maximum(ks_acc, k.abs().amax(0))
                vs_acc = torch.maximum(vs_acc, v.abs().amax(0))
        ks = torch.where(ks_acc > 0, ks_acc / qmax, torch.ones_like(ks_acc))
        vs = torch.where(vs_acc > 0, vs_acc / qmax, torch.ones_like(vs_acc))
        for b, n in enumerate(lens):
            if n == 0:
                continue
            nb = (n + bs - 1) // bs
            pad = nb * bs - n
            kq = quantize_ref(ktoks[b], ks, quant)
            vq = quantize_ref(vtoks[b], vs, quant)
            if pad:
                z = torch.zeros((pad, hkv, d), dtype=torch.uint8, device=device)
                kq, vq = torch.cat([kq, z]), torch.cat([vq, z])
            idx = bt[b, :nb].long()
            kc[idx] = kq.view(nb, bs, hkv, d).permute(0, 2, 1, 3)
            vc[idx] = vq.view(nb, bs, hkv, d).permute(0, 2, 1, 3)
    return dict(q=q, key_cache=kc, value_cache=vc, cache_k_scale=ks.contiguous(), cache_v_scale=vs.contiguous(),
                block_tables=bt, seq_lens_decoder=torch.tensor(lens, dtype=torch.int32, device=device),
                hq=hq, hkv=hkv, d=d, bs=bs, quant=quant, batch=batch)


def write_case(num_seqs=256, max_pos=8192, quant=CACHE_INT8, seed=0, device="cpu", hq=HQ, hkv=HKV, d=D,
               bs=BS, chunk=1, theta=500000.0, rope_style="neox", blocks_per_seq=None):
    """New-token qkv + caches with random prior contents; position of sequence b's first
    new token = seq_lens_decoder[b] ~ U{0..max_pos - chunk}."""
    from .rope import rope_table
    g = _gen(seed, device)
    T = num_seqs * chunk
    qkv = torch.randn((T, (hq + 2 * hkv) * d), generator=g, device=device).to(torch.bfloat16)
    dec = torch.randint(0, max_pos - chunk + 1, (num_seqs,), generator=g, device=device, dtype=torch.int32)
    mb = blocks_per_seq or (max_pos + bs - 1) // bs
    pool = num_seqs * mb
    perm = torch.randperm(pool, generator=g, device=device).to(torch.int32)
    bt = perm.view(num_seqs, mb).contiguous()
    kc = torch.randint(0, 256, (pool, hkv, bs, d), generator=g, device=device, dtype=torch.uint8)
    vc = torch.randint(0, 256, (pool, hkv, bs, d), generator=g, device=device, dtype=torch.uint8)
    if byte_format(quant) == CACHE_FP8:  # no NaN codes in the prior contents
        kc = torch.where((kc & 0x7F) == 0x7F, kc & 0xFE, kc)
        vc = torch.where((vc & 0x7F) == 0x7F, vc & 0xFE, vc)
    qmax = 127.0 if byte_format(quant) == CACHE_INT8 else 448.0
    if is_dynamic(quant):  # scale caches with prior contents: the rows already stored
        ks = (torch.rand((pool, hkv, bs), generator=g, device=device) * 2.0 + 3.0) / qmax
        vs = (torch.rand((pool, hkv, bs), generator=g, device=device) * 2.0 + 3.0) / qmax
    else:
        ks = (torch.rand((hkv, d), generator=g, device=device) * 2.0 + 3.0) / qmax
        vs = (torch.rand((hkv, d), generator=g, device=device) * 2.0 + 3.0) / qmax
    cos, sin = rope_table(max_pos, d, theta, device)
    this = torch.full((num_seqs,), chunk, dtype=torch.int32, device=device)
    cu = torch.arange(0, T + 1, chunk, dtype=torch.int32, device=device)
    return dict(qkv=qkv, key_cache=kc, value_cache=vc, cache_k_scale=ks.contiguous(), cache_v_scale=vs.contiguous(),
                block_tables=bt, seq_lens_decoder=dec, seq_lens_this_time=this,
                seq_lens_encoder=(this if chunk > 1 else torch.zeros_like(this)), cu_seqlens_q=cu,
                rope_cos=cos, rope_sin=sin, hq=hq, hkv=hkv, d=d, bs=bs, quant=quant, rope_style=rope_style,
                batch=num_seqs, chunk=chunk)


def to_device(case, device):
    return {k: (v.to(device) if isinstance(v, torch.Tensor) else v) for k, v in case.items()}


def decode_kv_bytes(seq_lens, hkv=HKV, d=D):
    """Algorithmic K+V bytes of one decode pass: sum_b ctx_b * hkv * d * 2."""
    return int(sum(int(c) for c in seq_lens)) * hkv * d * 2


def decode_algorithmic_bytes(seq_lens, batch, hq=HQ, hkv=HKV, d=D, bs=BS):
    """K+V bytes + Q + out (bf16) + both scale tables + the block-table entries read."""
    kv = decode_kv_bytes(seq_lens, hkv, d)
    tables = sum((int(c) + bs - 1) // bs for c in seq_lens) * 4
    return kv + 2 * batch * hq * d * 2 + 2 * hkv * d * 4 + tables


def prefill_flops(prefix, chunk, hq=HQ, d=D):
    """4 * d * hq * sum_i (prefix + i + 1) for one sequence."""
    pairs = chunk * prefix + chunk * (chunk + 1) // 2
    return 4 * d * hq * pairs


SM_SCALE = 1.0 / math.sqrt(D)
