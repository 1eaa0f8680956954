// Cache writer: rotary embedding on Q/K + int8 / fp8-e4m3 quantisation of K/V into
// block-tabled pages; optionally the QKV projection's epilogue in front of it (bias, per-head
// RMS norm of Q and K).  Memory-bound and tiny (launch-bound at decode sizes): one
// thread per 16 channels, 16-byte loads of qkv, 8/16-byte stores into the page.  The
// dynamic formats derive one scale per stored row from the row itself and store it beside it.
//
// Bit-exactness contract (shared with the CPU oracle): every fp32 product, sum and
// the one division are rounded on their own - this file is compiled with
// -ffp-contract=off and uses the *_rn intrinsics so nothing is fused - and cos/sin
// come from a host-built table, never from device libm.
#include "fdattn_common.h"

namespace fdattn {

struct WriterArgs {
  const uint16_t* qkv;
  uint16_t* q_out;
  uint16_t* k_out;
  uint16_t* v_out;
  uint8_t* key_cache;
  uint8_t* value_cache;
  const float* k_scale;  // per channel [hkv, d]; DYN: the scale cache [num_blocks, hkv, bs], written here
  const float* v_scale;
  const float* rope_cos;
  const float* rope_sin;
  const int32_t* block_tables;
  const int32_t* seq_lens_decoder;
  const int32_t* cu_seqlens_q;
  int num_tokens, batch, hq, hkv, d, bs, max_blocks, num_blocks, max_pos, rope_style;
  // the projection's epilogue, all optional
  const uint16_t* qkv_bias;     // bf16 [(hq + 2 hkv) * d]
  const float* q_norm_weight;   // [d]: RMS norm of every Q head before the rotation
  const float* k_norm_weight;   // [d]: the same for K
  float rms_norm_eps;
  int tok0;  // first token of this launch (the grid's y dimension holds 65,535)
};

template <int QUANT>
__device__ __forceinline__ u32 quant1(float x, float s) {
  float r = __fdiv_rn(x, s);
  if (QUANT == FDATTN_CACHE_INT8) {
    if (r != r) return 0u;  // NaN quantises to 0
    r = __builtin_rintf(r);
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    return (u32)(int)r & 0xffu;
  } else {
    return f32_to_e4m3(r);
  }
}

// One unit = 8 rotation pairs (16 channels) of one head of one token.
//   heads [0, hq)            Q   : rotate, round to bf16, store to q_out
//   heads [hq, hq+hkv)       K   : rotate, (bf16 -> k_out), quantise, store to key_cache
//   heads [hq+hkv, hq+2hkv)  V   : (copy -> v_out), quantise, store to value_cache
// DYN: one scale per stored row, (largest magnitude of the row) / 127 or / 448, stored beside the row.
template <int QUANT, bool DYN>
__global__ __launch_bounds__(256) void write_cache_kv_kernel(WriterArgs a) {
  // grid (units of a token / 256, tokens): the token - and with it the sequence, the position and the
  // cache slot - is uniform over the workgroup and is worked out in scalar registers
  const int units_per_head = a.d / 16;
  const int heads = a.hq + 2 * a.hkv;
  const int unit = blockIdx.x * blockDim.x + threadIdx.x;
  if (unit >= heads * units_per_head) return;
  const int head = unit / units_per_head, u = unit - head * units_per_head;
  const int tok = a.tok0 + blockIdx.y;

  // sequence of this token: last b with cu_seqlens_q[b] <= tok
  int lo = 0, hi = a.batch;
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (a.cu_seqlens_q[mid] <= tok) lo = mid; else hi = mid;
  }
  const int b = lo;
  if (tok >= a.cu_seqlens_q[b + 1]) return;  // token past the last sequence
  const int pos = a.seq_lens_decoder[b] + (tok - a.cu_seqlens_q[b]);
  // a position outside the rope table cannot be rotated: the token is skipped
  if (pos < 0 || (a.rope_cos != nullptr && pos >= a.max_pos)) return;

  const int half = a.d / 2;
  const uint16_t* row = a.qkv + (size_t)tok * heads * a.d + (size_t)head * a.d;
  const bool is_v = head >= a.hq + a.hkv;
  const bool is_k = !is_v && head >= a.hq;

  // channel indices of the 8 pairs: NeoX (j, j+half), interleaved (2j, 2j+1), j = 8u..8u+7.
  // V has no pairs: it takes channels 16u..16u+15 in the same two registers.
  int c1, c2;  // start channels of the two 8-element groups
  const bool neox = a.rope_style == FDATTN_ROPE_NEOX;
  if (is_v || !neox) { c1 = 16 * u; c2 = 16 * u + 8; } else { c1 = 8 * u; c2 = 8 * u + half; }

  uint4 w1 = *reinterpret_cast<const uint4*>(row + c1);
  uint4 w2 = *reinterpret_cast<const uint4*>(row + c2);
  u32 ws1[4] = {w1.x, w1.y, w1.z, w1.w}, ws2[4] = {w2.x, w2.y, w2.z, w2.w};
  float x1[8], x2[8];  // V / NeoX: x1 = group c1.., x2 = group c2..; interleaved: x1 = even, x2 = odd
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float a0 = bf16lo_to_f32(ws1[i]), a1 = bf16hi_to_f32(ws1[i]);
    float b0 = bf16lo_to_f32(ws2[i]), b1 = bf16hi_to_f32(ws2[i]);
    if (is_v || neox) {
      x1[2 * i] = a0; x1[2 * i + 1] = a1; x2[2 * i] = b0; x2[2 * i + 1] = b1;
    } else {  // 16 contiguous channels: pair i of w1 = (a0, a1), pair 4+i from w2
      x1[i] = a0; x2[i] = a1; x1[4 + i] = b0; x2[4 + i] = b1;
    }
  }

  bool changed = false;  // x no longer equals the loaded bf16 values
  if (a.qkv_bias != nullptr) {
    // x = bf16(x + bias): the sum an unfused bf16 add would have produced
    const uint16_t* brow = a.qkv_bias + (size_t)head * a.d;
    const uint4 b1 = *reinterpret_cast<const uint4*>(brow + c1);
    const uint4 b2 = *reinterpret_cast<const uint4*>(brow + c2);
    const u32 bs1[4] = {b1.x, b1.y, b1.z, b1.w}, bs2[4] = {b2.x, b2.y, b2.z, b2.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a0 = bf16lo_to_f32(bs1[i]), a1 = bf16hi_to_f32(bs1[i]);
      const float b0 = bf16lo_to_f32(bs2[i]), b1f = bf16hi_to_f32(bs2[i]);
      if (is_v || neox) {
        x1[2 * i] = __fadd_rn(x1[2 * i], a0); x1[2 * i + 1] = __fadd_rn(x1[2 * i + 1], a1);
        x2[2 * i] = __fadd_rn(x2[2 * i], b0); x2[2 * i + 1] = __fadd_rn(x2[2 * i + 1], b1f);
      } else {
        x1[i] = __fadd_rn(x1[i], a0); x2[i] = __fadd_rn(x2[i], a1);
        x1[4 + i] = __fadd_rn(x1[4 + i], b0); x2[4 + i] = __fadd_rn(x2[4 + i], b1f);
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      x1[i] = bf16_to_f32(f32_to_bf16(x1[i]));
      x2[i] = bf16_to_f32(f32_to_bf16(x2[i]));
    }
    changed = true;
  }
  const float* nw = is_v ? nullptr : (is_k ? a.k_norm_weight : a.q_norm_weight);
  if (nw != nullptr) {
    // RMS norm over the head.  The sum of squares has a fixed order (the oracle follows it): within
    // a thread first members of its 8 pairs, then second members, each sequentially; across the
    // d/16 threads of the head a butterfly (the host checked that d/16 is a power of two), whose
    // additions are commutative, so every thread ends with the same bits.
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      s1 = __fadd_rn(s1, __fmul_rn(x1[i], x1[i]));
      s2 = __fadd_rn(s2, __fmul_rn(x2[i], x2[i]));
    }
    float ss = __fadd_rn(s1, s2);
    for (int o = 1; o < units_per_head; o <<= 1) ss = __fadd_rn(ss, __shfl_xor(ss, o, 64));
    // sqrtf, not __fsqrt_rn: that intrinsic is the approximate square root here; sqrtf and the division
    // are correctly rounded (hipcc's default), which is what the oracle's libm gives
    const float r = __fdiv_rn(1.0f, sqrtf(__fadd_rn(__fdiv_rn(ss, (float)a.d), a.rms_norm_eps)));
    // weights of this thread's channels, in the order of x1 / x2
    const float4 wa = *reinterpret_cast<const float4*>(nw + c1), wb = *reinterpret_cast<const float4*>(nw + c1 + 4);
    const float4 wc = *reinterpret_cast<const float4*>(nw + c2), wd = *reinterpret_cast<const float4*>(nw + c2 + 4);
    const float g1w[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
    const float g2w[8] = {wc.x, wc.y, wc.z, wc.w, wd.x, wd.y, wd.z, wd.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float w1v, w2v;
      if (neox) { w1v = g1w[i]; w2v = g2w[i]; }
      else { w1v = i < 4 ? g1w[2 * i] : g2w[2 * (i - 4)]; w2v = i < 4 ? g1w[2 * i + 1] : g2w[2 * (i - 4) + 1]; }
      x1[i] = __fmul_rn(__fmul_rn(x1[i], r), w1v);
      x2[i] = __fmul_rn(__fmul_rn(x2[i], r), w2v);
    }
  }

  float y1[8], y2[8];
  if (!is_v && a.rope_cos != nullptr) {
    const float* cs = a.rope_cos + (size_t)pos * half + 8 * u;
    const float* sn = a.rope_sin + (size_t)pos * half + 8 * u;
    float4 ca = *reinterpret_cast<const float4*>(cs), cb = *reinterpret_cast<const float4*>(cs + 4);
    float4 sa = *reinterpret_cast<const float4*>(sn), sb = *reinterpret_cast<const float4*>(sn + 4);
    float c[8] = {ca.x, ca.y, ca.z, ca.w, cb.x, cb.y, cb.z, cb.w};
    float s[8] = {sa.x, sa.y, sa.z, sa.w, sb.x, sb.y, sb.z, sb.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      y1[i] = __fsub_rn(__fmul_rn(x1[i], c[i]), __fmul_rn(x2[i], s[i]));
      y2[i] = __fadd_rn(__fmul_rn(x2[i], c[i]), __fmul_rn(x1[i], s[i]));
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) { y1[i] = x1[i]; y2[i] = x2[i]; }
  }

  // back to channel order: g1 = channels c1..c1+7, g2 = channels c2..c2+7
  float g1[8], g2[8];
  if (is_v || neox) {
#pragma unroll
    for (int i = 0; i < 8; ++i) { g1[i] = y1[i]; g2[i] = y2[i]; }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      g1[2 * i] = y1[i]; g1[2 * i + 1] = y2[i]; g2[2 * i] = y1[4 + i]; g2[2 * i + 1] = y2[4 + i];
    }
  }

  if (!is_k && !is_v) {
    uint16_t* o = a.q_out + ((size_t)tok * a.hq + head) * a.d;
    u32 p1[4], p2[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p1[i] = (u32)f32_to_bf16(g1[2 * i]) | ((u32)f32_to_bf16(g1[2 * i + 1]) << 16);
      p2[i] = (u32)f32_to_bf16(g2[2 * i]) | ((u32)f32_to_bf16(g2[2 * i + 1]) << 16);
    }
    *reinterpret_cast<uint4*>(o + c1) = make_uint4(p1[0], p1[1], p1[2], p1[3]);
    *reinterpret_cast<uint4*>(o + c2) = make_uint4(p2[0], p2[1], p2[2], p2[3]);
    return;
  }

  const int h = is_k ? head - a.hq : head - a.hq - a.hkv;
  uint16_t* side = is_k ? a.k_out : a.v_out;
  if (side != nullptr) {
    uint16_t* o = side + ((size_t)tok * a.hkv + h) * a.d;
    if (is_v && !changed) {
      *reinterpret_cast<uint4*>(o + c1) = w1;
      *reinterpret_cast<uint4*>(o + c2) = w2;
    } else {
      u32 p1[4], p2[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        p1[i] = (u32)f32_to_bf16(g1[2 * i]) | ((u32)f32_to_bf16(g1[2 * i + 1]) << 16);
        p2[i] = (u32)f32_to_bf16(g2[2 * i]) | ((u32)f32_to_bf16(g2[2 * i + 1]) << 16);
      }
      *reinterpret_cast<uint4*>(o + c1) = make_uint4(p1[0], p1[1], p1[2], p1[3]);
      *reinterpret_cast<uint4*>(o + c2) = make_uint4(p2[0], p2[1], p2[2], p2[3]);
    }
  }

  const int lb = pos / a.bs, slot = pos - lb * a.bs;
  if (lb >= a.max_blocks) return;
  const int pb = a.block_tables[(size_t)b * a.max_blocks + lb];
  if (pb < 0 || pb >= a.num_blocks) return;
  uint8_t* dst = (is_k ? a.key_cache : a.value_cache) + (((size_t)pb * a.hkv + h) * a.bs + slot) * a.d;
  float s1[8], s2[8];
  if (DYN) {
    // the row's largest magnitude: over this thread's 16 channels, then over the d/16 threads of the head
    // (a butterfly; the host checked that d/16 is a power of two).  fmaxf drops NaNs, as the oracle's does.
    float m = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) m = fmaxf(m, fmaxf(fabsf(g1[i]), fabsf(g2[i])));
    for (int o = 1; o < units_per_head; o <<= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    const float sc = m > 0.f ? __fdiv_rn(m, QUANT == FDATTN_CACHE_INT8 ? 127.0f : 448.0f) : 1.0f;
    if (u == 0)
      const_cast<float*>(is_k ? a.k_scale : a.v_scale)[((size_t)pb * a.hkv + h) * a.bs + slot] = sc;
#pragma unroll
    for (int i = 0; i < 8; ++i) s1[i] = s2[i] = sc;
  } else {
    const float* sc = (is_k ? a.k_scale : a.v_scale) + (size_t)h * a.d;
    float4 s1a = *reinterpret_cast<const float4*>(sc + c1), s1b = *reinterpret_cast<const float4*>(sc + c1 + 4);
    float4 s2a = *reinterpret_cast<const float4*>(sc + c2), s2b = *reinterpret_cast<const float4*>(sc + c2 + 4);
    const float t1[8] = {s1a.x, s1a.y, s1a.z, s1a.w, s1b.x, s1b.y, s1b.z, s1b.w};
    const float t2[8] = {s2a.x, s2a.y, s2a.z, s2a.w, s2b.x, s2b.y, s2b.z, s2b.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) { s1[i] = t1[i]; s2[i] = t2[i]; }
  }
  u32 q1[2] = {0, 0}, q2[2] = {0, 0};
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    q1[i >> 2] |= quant1<QUANT>(g1[i], s1[i]) << (8 * (i & 3));
    q2[i >> 2] |= quant1<QUANT>(g2[i], s2[i]) << (8 * (i & 3));
  }
  *reinterpret_cast<uint2*>(dst + c1) = make_uint2(q1[0], q1[1]);
  *reinterpret_cast<uint2*>(dst + c2) = make_uint2(q2[0], q2[1]);
}

}  // namespace fdattn

using namespace fdattn;

extern "C" int fdattn_write_cache_kv(
    const void* qkv, void* q_out, void* k_out, void* v_out, void* key_cache, void* value_cache,
    const float* cache_k_scale, const float* cache_v_scale, const float* rope_cos,
    const float* rope_sin, const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* cu_seqlens_q, int num_tokens, int batch, int hq, int hkv, int head_dim,
    int block_size, int max_blocks_per_seq, int num_blocks, int max_pos, int rope_style,
    int cache_quant_type, void* stream) {
  return fdattn_write_cache_kv_ex(qkv, q_out, k_out, v_out, key_cache, value_cache, cache_k_scale, cache_v_scale,
                                  rope_cos, rope_sin, block_tables, seq_lens_decoder, cu_seqlens_q, num_tokens, batch,
                                  hq, hkv, head_dim, block_size, max_blocks_per_seq, num_blocks, max_pos, rope_style,
                                  cache_quant_type, nullptr, stream);
}

extern "C" int fdattn_write_cache_kv_ex(
    const void* qkv, void* q_out, void* k_out, void* v_out, void* key_cache, void* value_cache,
    const float* cache_k_scale, const float* cache_v_scale, const float* rope_cos,
    const float* rope_sin, const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* cu_seqlens_q, int num_tokens, int batch, int hq, int hkv, int head_dim,
    int block_size, int max_blocks_per_seq, int num_blocks, int max_pos, int rope_style,
    int cache_quant_type, const fdattn_step_extras* extras, void* stream) {
  const fdattn_step_extras none = {nullptr, nullptr, nullptr, 0.f, 0};
  const fdattn_step_extras& ep = extras ? *extras : none;
  if (quant_dynamic(cache_quant_type)) {
    const int u = head_dim / 16;
    if (head_dim % 16 != 0 || u <= 0 || (u & (u - 1)) != 0 || u > 64)
      return fail(FDATTN_ERR_SHAPE, "fdattn_write_cache_kv: the dynamic cache formats need head_dim = 16 * a power "
                  "of two up to 1024, got %d", head_dim);
  }
  if (ep.q_norm_weight || ep.k_norm_weight) {
    const int u = head_dim / 16;
    if (head_dim % 16 != 0 || u <= 0 || (u & (u - 1)) != 0 || u > 64)
      return fail(FDATTN_ERR_SHAPE, "fdattn_write_cache_kv: the RMS norm needs head_dim = 16 * a power of two "
                  "up to 1024, got %d", head_dim);
    if (!(ep.rms_norm_eps >= 0.f))
      return fail(FDATTN_ERR_SHAPE, "fdattn_write_cache_kv: rms_norm_eps must not be negative");
  }
  if (!qkv || !q_out || !key_cache || !value_cache || !cache_k_scale || !cache_v_scale ||
      !block_tables || !seq_lens_decoder || !cu_seqlens_q)
    return fail(FDATTN_ERR_NULL, "fdattn_write_cache_kv: a required pointer is NULL");
  if ((rope_cos == nullptr) != (rope_sin == nullptr))
    return fail(FDATTN_ERR_NULL, "fdattn_write_cache_kv: rope_cos and rope_sin must both be given or both NULL");
  if (num_tokens < 0 || batch <= 0 || hq <= 0 || hkv <= 0 || hq % hkv != 0 || head_dim <= 0 ||
      head_dim % 32 != 0 || block_size <= 0 || max_blocks_per_seq <= 0 || num_blocks <= 0)
    return fail(FDATTN_ERR_SHAPE,
                "fdattn_write_cache_kv: unsupported shape (tokens=%d batch=%d hq=%d hkv=%d head_dim=%d "
                "block_size=%d max_blocks=%d num_blocks=%d; head_dim must be a multiple of 32)",
                num_tokens, batch, hq, hkv, head_dim, block_size, max_blocks_per_seq, num_blocks);
  if (rope_cos && max_pos <= 0)
    return fail(FDATTN_ERR_SHAPE, "fdattn_write_cache_kv: max_pos must be positive with a rope table");
  if (rope_style != FDATTN_ROPE_INTERLEAVED && rope_style != FDATTN_ROPE_NEOX)
    return fail(FDATTN_ERR_QUANT, "fdattn_write_cache_kv: unknown rope_style %d", rope_style);
  if (!quant_known(cache_quant_type))
    return fail(FDATTN_ERR_QUANT, "fdattn_write_cache_kv: unknown cache_quant_type %d", cache_quant_type);
  if (num_tokens == 0) return 0;
  WriterArgs a{(const uint16_t*)qkv, (uint16_t*)q_out, (uint16_t*)k_out, (uint16_t*)v_out,
               (uint8_t*)key_cache, (uint8_t*)value_cache, cache_k_scale, cache_v_scale, rope_cos,
               rope_sin, block_tables, seq_lens_decoder, cu_seqlens_q, num_tokens, batch, hq, hkv,
               head_dim, block_size, max_blocks_per_seq, num_blocks, max_pos, rope_style,
               (const uint16_t*)ep.qkv_bias, ep.q_norm_weight, ep.k_norm_weight, ep.rms_norm_eps, 0};
  const int units = (hq + 2 * hkv) * (head_dim / 16);
  hipStream_t s = (hipStream_t)stream;
  // the y dimension of a grid holds 65,535 workgroups: more tokens go in slices
  for (int t0 = 0; t0 < num_tokens; t0 += 65535) {
    a.tok0 = t0;
    const dim3 grid((units + 255) / 256, num_tokens - t0 < 65535 ? num_tokens - t0 : 65535);
    if (cache_quant_type == FDATTN_CACHE_INT8)
      hipLaunchKernelGGL((write_cache_kv_kernel<FDATTN_CACHE_INT8, false>), grid, dim3(256), 0, s, a);
    else if (cache_quant_type == FDATTN_CACHE_FP8_E4M3)
      hipLaunchKernelGGL((write_cache_kv_kernel<FDATTN_CACHE_FP8_E4M3, false>), grid, dim3(256), 0, s, a);
    else if (cache_quant_type == FDATTN_CACHE_INT8_DYNAMIC)
      hipLaunchKernelGGL((write_cache_kv_kernel<FDATTN_CACHE_INT8, true>), grid, dim3(256), 0, s, a);
    else
      hipLaunchKernelGGL((write_cache_kv_kernel<FDATTN_CACHE_FP8_E4M3, true>), grid, dim3(256), 0, s, a);
  }
  return check_launch("fdattn_write_cache_kv");
}
