// Cache writer: rotary embedding on Q/K + int8 / fp8-e4m3 quantisation of K/V into
// block-tabled pages; optionally the QKV projection's epilogue in front of it (bias, per-head
// RMS norm of Q and K).  Memory-bound and tiny (launch-bound at decode sizes): one
// thread per 16 channels, 16-byte loads of qkv, 8/16-byte stores into the page.  The
// dynamic formats derive one scale per stored row from the row itself and store it beside it; the
// per-block formats keep one scale per (block, KV head) tile, which a second kernel maintains (one
// workgroup per tile that the call stores into).
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
  float* k_scale;  // per channel [hkv, d], read; DYN: the scale cache [num_blocks, hkv, bs], written here;
                   // per-block formats: the scale cache [num_blocks, hkv], read and written by the tile kernel
  float* v_scale;
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
  int tiles_write_rows;  // per-block formats, long chunks: k_out / v_out are the tile kernel's (the token kernel writes q_out only)
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

// The same byte as quant1(x, s) when many values share the scale: x * (1 / s) with the hardware's reciprocal (rs, taken
// once) is within a few units in the last place of the correctly rounded x / s, so the two can only round to different
// integers next to a tie - there, and for anything that is not a number, the division decides.  int8 only (the e4m3
// grid is not uniform: fp8 takes quant1).
template <int QUANT>
__device__ __forceinline__ u32 quant1_shared(float x, float s, float rs) {
  if (QUANT != FDATTN_CACHE_INT8) return quant1<QUANT>(x, s);
  float q = __fmul_rn(x, rs);
  float t = __builtin_rintf(q);
  if (!(fabsf(q - t) <= 0.499f)) {
    q = __fdiv_rn(x, s);
    if (q != q) return 0u;
    t = __builtin_rintf(q);
  }
  t = fminf(fmaxf(t, -127.0f), 127.0f);
  return (u32)(int)t & 0xffu;
}

// The values of one unit - 8 rotation pairs (16 channels) of one head of one token - after the projection's
// epilogue and the rotation, in channel order: g1 = channels c1 .. c1+7, g2 = channels c2 .. c2+7.
// The RMS norm's sum runs over the d/16 adjacent lanes that hold the head's units: every one of them must be here.
struct UnitValues {
  float g1[8], g2[8];
  int c1, c2;
  uint4 w1, w2;   // the 16 loaded bf16 values
  bool changed;   // the values no longer equal the loaded ones
};
__device__ __forceinline__ UnitValues unit_values(const WriterArgs& a, int tok, int head, int u, int pos) {
  UnitValues o;
  const int units_per_head = a.d / 16;
  const int heads = a.hq + 2 * a.hkv;
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
  // Two 8-element groups of bf16 -> first and second members of the 8 pairs.  V / NeoX (grouped): first = group c1..,
  // second = group c2..; interleaved: the 16 channels are contiguous, first = the even ones, second = the odd ones.
  // Every register index below is a compile-time constant and the style picks between VALUES: an index that depends
  // on the style would send the arrays to scratch memory.
  const bool grouped = is_v || neox;
  auto unpack = [&](const uint4& wa, const uint4& wb, float (&first)[8], float (&second)[8]) {
    const u32 s1[4] = {wa.x, wa.y, wa.z, wa.w}, s2[4] = {wb.x, wb.y, wb.z, wb.w};
    float lo1[4], hi1[4], lo2[4], hi2[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      lo1[i] = bf16lo_to_f32(s1[i]); hi1[i] = bf16hi_to_f32(s1[i]);
      lo2[i] = bf16lo_to_f32(s2[i]); hi2[i] = bf16hi_to_f32(s2[i]);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float f_grouped = (j & 1) ? hi1[j >> 1] : lo1[j >> 1], s_grouped = (j & 1) ? hi2[j >> 1] : lo2[j >> 1];
      const float f_inter = j < 4 ? lo1[j & 3] : lo2[j & 3], s_inter = j < 4 ? hi1[j & 3] : hi2[j & 3];
      first[j] = grouped ? f_grouped : f_inter;
      second[j] = grouped ? s_grouped : s_inter;
    }
  };
  float x1[8], x2[8];
  unpack(w1, w2, x1, x2);

  bool changed = false;  // x no longer equals the loaded bf16 values
  if (a.qkv_bias != nullptr) {
    // x = bf16(x + bias): the sum an unfused bf16 add would have produced
    const uint16_t* brow = a.qkv_bias + (size_t)head * a.d;
    const uint4 b1 = *reinterpret_cast<const uint4*>(brow + c1);
    const uint4 b2 = *reinterpret_cast<const uint4*>(brow + c2);
    float bx1[8], bx2[8];
    unpack(b1, b2, bx1, bx2);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      x1[i] = bf16_to_f32(f32_to_bf16(__fadd_rn(x1[i], bx1[i])));
      x2[i] = bf16_to_f32(f32_to_bf16(__fadd_rn(x2[i], bx2[i])));
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
      const float w1i = i < 4 ? g1w[(2 * i) & 7] : g2w[(2 * i) & 7], w2i = i < 4 ? g1w[(2 * i + 1) & 7] : g2w[(2 * i + 1) & 7];
      const float w1v = neox ? g1w[i] : w1i, w2v = neox ? g2w[i] : w2i;
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

  // back to channel order (interleaved: channel c1 + j is member j & 1 of pair j >> 1, channel c2 + j of pair 4 + (j >> 1))
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float g1_inter = (j & 1) ? y2[j >> 1] : y1[j >> 1], g2_inter = (j & 1) ? y2[4 + (j >> 1)] : y1[4 + (j >> 1)];
    o.g1[j] = grouped ? y1[j] : g1_inter;
    o.g2[j] = grouped ? y2[j] : g2_inter;
  }
  o.c1 = c1; o.c2 = c2; o.w1 = w1; o.w2 = w2; o.changed = changed;
  return o;
}


// The tile that token `tok` of sequence b starts in this call.
struct TileJob {
  int tok;         // the call's first token of the tile
  int r0, r1;      // positions [r0, r1) are stored into the tile by this call
  int lb, pb;      // logical and physical block
  int prior_rows;  // rows of earlier calls in the tile
};
__device__ __forceinline__ bool tile_job(const WriterArgs& a, const SeqRows& sr, int tok, TileJob& j);
template <int QUANT>
__device__ __forceinline__ void write_tile_rows(const WriterArgs& a, const TileJob& j, int h, bool is_k, int head, int u,
                                                const UnitValues& first);

// One thread per unit:
//   heads [0, hq)            Q   : rotate, round to bf16, store to q_out
//   heads [hq, hq+hkv)       K   : rotate, (bf16 -> k_out), quantise, store to key_cache
//   heads [hq+hkv, hq+2hkv)  V   : (copy -> v_out), quantise, store to value_cache
// A K or V row's unit into k_out / v_out (o: the row): V that the epilogue left unchanged goes as it was loaded.
__device__ __forceinline__ void store_side_unit(uint16_t* o, const UnitValues& uv, bool is_v) {
  if (is_v && !uv.changed) {
    *reinterpret_cast<uint4*>(o + uv.c1) = uv.w1;
    *reinterpret_cast<uint4*>(o + uv.c2) = uv.w2;
    return;
  }
  u32 p1[4], p2[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    p1[i] = pack2_bf16(uv.g1[2 * i], uv.g1[2 * i + 1]);
    p2[i] = pack2_bf16(uv.g2[2 * i], uv.g2[2 * i + 1]);
  }
  *reinterpret_cast<uint4*>(o + uv.c1) = make_uint4(p1[0], p1[1], p1[2], p1[3]);
  *reinterpret_cast<uint4*>(o + uv.c2) = make_uint4(p2[0], p2[1], p2[2], p2[3]);
}

// MODE 0: per-channel scales.  MODE 1: one scale per stored row, (largest magnitude of the row) / 127 or / 448, stored
// beside the row.  MODE 2: the cache is left to write_cache_tiles_kernel (one scale per tile needs all rows of the tile).
// MODE 3: one scale per tile, kept by this kernel itself - the threads that hold a K or V head of a token that stands
// for a tile do the tile's whole job (write_tile_rows): for steps of at most one token per sequence, where a job is one
// row and a second launch would cost more than the write.  MODE 4: q_out only - the cache, k_out and v_out are the tile
// kernel's (long chunks: it computes every K and V row anyway); the K and V rows of skipped tokens are zeroed here.
template <int QUANT, int MODE>
__device__ __forceinline__ void write_token_units(const WriterArgs& a, int unit_block, int tok_in_launch) {
  constexpr bool DYN = MODE == 1;
  // (block of 256 units of a token, token): the token - and with it the sequence, the position and the
  // cache slot - is uniform over the workgroup and is worked out in scalar registers
  const int units_per_head = a.d / 16;
  const int heads = a.hq + 2 * a.hkv;
  const int unit = unit_block * 256 + threadIdx.x;
  const int tok = a.tok0 + tok_in_launch;
  BatchRows rows;  // (before any thread leaves)
  rows.load(a.cu_seqlens_q, a.seq_lens_decoder, a.batch);
  const SeqRows sr = rows.at(rows.seq_of(tok));
  if (unit >= heads * units_per_head) return;
  const int head = unit / units_per_head, u = unit - head * units_per_head;
  if (tok >= sr.end) return;  // token past the last sequence
  const int pos = sr.cached + (tok - sr.first);
  // a position outside the rope table cannot be rotated: the token is skipped - nothing is written to the cache, and
  // its rows of q_out / k_out / v_out are zeros (not whatever the buffers held), so that an attention pass that still
  // counts the token reads defined values
  if (pos < 0 || (a.rope_cos != nullptr && pos >= a.max_pos)) {
    const bool v_head = head >= a.hq + a.hkv, k_head = !v_head && head >= a.hq;
    uint16_t* o = !k_head && !v_head ? a.q_out + ((size_t)tok * a.hq + head) * a.d
                                     : (k_head ? a.k_out : a.v_out);
    if (o != nullptr) {
      if (k_head || v_head) o += ((size_t)tok * a.hkv + (head - a.hq - (v_head ? a.hkv : 0))) * a.d;
      *reinterpret_cast<uint4*>(o + 16 * u) = make_uint4(0u, 0u, 0u, 0u);
      *reinterpret_cast<uint4*>(o + 16 * u + 8) = make_uint4(0u, 0u, 0u, 0u);
    }
    return;
  }

  if (MODE == 4 && head >= a.hq) return;
  const UnitValues uv = unit_values(a, tok, head, u, pos);
  const bool is_v = head >= a.hq + a.hkv;
  const bool is_k = !is_v && head >= a.hq;
  const int c1 = uv.c1, c2 = uv.c2;
  const float (&g1)[8] = uv.g1;
  const float (&g2)[8] = uv.g2;

  if (!is_k && !is_v) {
    uint16_t* o = a.q_out + ((size_t)tok * a.hq + head) * a.d;
    u32 p1[4], p2[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p1[i] = pack2_bf16(g1[2 * i], g1[2 * i + 1]);
      p2[i] = pack2_bf16(g2[2 * i], g2[2 * i + 1]);
    }
    *reinterpret_cast<uint4*>(o + c1) = make_uint4(p1[0], p1[1], p1[2], p1[3]);
    *reinterpret_cast<uint4*>(o + c2) = make_uint4(p2[0], p2[1], p2[2], p2[3]);
    return;
  }

  const int h = is_k ? head - a.hq : head - a.hq - a.hkv;
  uint16_t* side = is_k ? a.k_out : a.v_out;
  if (side != nullptr) store_side_unit(side + ((size_t)tok * a.hkv + h) * a.d, uv, is_v);

  if (MODE == 2 || MODE == 4) return;
  if constexpr (MODE == 3) {
    TileJob j;
    if (tile_job(a, sr, tok, j)) write_tile_rows<QUANT>(a, j, h, is_k, head, u, uv);  // (the same for every thread of the workgroup)
    return;
  }
  const int lb = pos / a.bs, slot = pos - lb * a.bs;
  if (lb >= a.max_blocks) return;
  const int pb = a.block_tables[(size_t)sr.b * a.max_blocks + lb];
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
      (is_k ? a.k_scale : a.v_scale)[((size_t)pb * a.hkv + h) * a.bs + slot] = sc;
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
  if (DYN) {  // one scale for the row
    const float rs = __builtin_amdgcn_rcpf(s1[0]);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      q1[i >> 2] |= quant1_shared<QUANT>(g1[i], s1[0], rs) << (8 * (i & 3));
      q2[i >> 2] |= quant1_shared<QUANT>(g2[i], s1[0], rs) << (8 * (i & 3));
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      q1[i >> 2] |= quant1<QUANT>(g1[i], s1[i]) << (8 * (i & 3));
      q2[i >> 2] |= quant1<QUANT>(g2[i], s2[i]) << (8 * (i & 3));
    }
  }
  *reinterpret_cast<uint2*>(dst + c1) = make_uint2(q1[0], q1[1]);
  *reinterpret_cast<uint2*>(dst + c2) = make_uint2(q2[0], q2[1]);
}

// grid (units of a token / 256, tokens)
template <int QUANT, int MODE>
__global__ __launch_bounds__(256) void write_cache_kv_kernel(WriterArgs a) {
  write_token_units<QUANT, MODE>(a, blockIdx.x, blockIdx.y);
}

// One stored byte under a tile scale that grew from s_old to s: (value of the byte * s_old) / s, quantised again.
template <int QUANT>
__device__ __forceinline__ u32 requant1(u32 byte, float s_old, float s) {
  if (QUANT == FDATTN_CACHE_INT8) return quant1<QUANT>(__fmul_rn((float)(int)(int8_t)byte, s_old), s);
  if ((byte & 0x7fu) == 0x7fu) return byte;  // a NaN code stays what it is
  return quant1<QUANT>(__fmul_rn(e4m3_to_f32(byte), s_old), s);
}

// ---- Per-block formats: one scale per (block, KV head) tile, kept at (largest magnitude stored in the tile) / 127 or / 448.
// The token kernel has computed every K and V row already (for k_out / v_out), but a tile's scale needs all the rows
// that the call stores into the tile, so the cache is written by kernels that own whole tiles: the token that is the
// first one this call stores into a tile - the first new token of its sequence, or one whose position is a multiple of
// the block size - stands for the tile.

__device__ __forceinline__ bool tile_job(const WriterArgs& a, const SeqRows& sr, int tok, TileJob& j) {
  const int b = sr.b, tok_first = sr.first;
  const int tok_end = min(sr.end, a.num_tokens);
  if (tok < tok_first || tok >= tok_end) return false;
  const int p0 = sr.cached;
  const int pos = p0 + (tok - tok_first);
  // tokens before position 0 or past the rope table are skipped, as by the token kernel
  const int p_first = max(p0, 0);
  int p_end = p0 + (tok_end - tok_first);
  if (a.rope_cos != nullptr) p_end = min(p_end, a.max_pos);
  if (pos < p_first || pos >= p_end) return false;
  const int lb = pos / a.bs;
  if (pos != p_first && pos != lb * a.bs) return false;  // another token stands for this tile
  int pb = lb < a.max_blocks ? a.block_tables[(size_t)b * a.max_blocks + lb] : -1;
  if (pb < 0 || pb >= a.num_blocks) {
    if (!a.tiles_write_rows) return false;
    pb = -1;  // no block to store into, but the rows are still owed to k_out / v_out
  }
  j.tok = tok;
  j.r0 = pos;
  j.r1 = min(p_end, (lb + 1) * a.bs);
  j.lb = lb;
  j.pb = pb;
  j.prior_rows = pos - lb * a.bs;
  return true;
}

// The K (or the V) half of one tile of KV head h by NT threads (64: a wavefront on its own; 256: a workgroup, red = its
// reduction buffer): (1) the rows that the call stores into the tile, recomputed, and their largest magnitude, (2) the tile's
// scale - if rows of earlier calls are in the tile the scale only grows, and when it grows those rows are
// requantised in place -, (3) the rows stored quantised (computed once more unless the threads hold them all: NT * 16 /
// head_dim rows per pass, two passes' worth in a workgroup's registers).
template <int QUANT, int NT>
__device__ __forceinline__ void write_tile(const WriterArgs& a, const TileJob& j, int h, bool is_k, float (*red)[4]) {
  const int tid = threadIdx.x;
  const bool cached = j.pb >= 0;  // (false: the table names no block for these rows - they only go to k_out / v_out)
  const size_t at = (size_t)(cached ? j.pb : 0) * a.hkv + h;
  float* const scale = is_k ? a.k_scale : a.v_scale;
  // the old scale is asked for now - before anything of this tile is stored - and needed after the rows' maximum
  float s_old = 0.f;
  if (cached && j.prior_rows > 0) s_old = scale[at];
  // the rows as the attention kernels take them (long chunks: the token kernel leaves them to this one)
  uint16_t* const side = is_k ? a.k_out : a.v_out;
  auto side_row = [&](int r, const UnitValues& x) {
    if (a.tiles_write_rows && side) store_side_unit(side + ((size_t)(j.tok + (r - j.r0)) * a.hkv + h) * a.d, x, !is_k);
  };

  const int uph = a.d / 16, rows_per_pass = NT / uph;
  const int u = tid % uph, row_in_pass = tid / uph;
  const int head = a.hq + (is_k ? 0 : a.hkv) + h;
  const int r0 = j.r0, r1 = j.r1;
  // a workgroup keeps two rows per thread in registers (a tile of 64 rows at head_dim 128: every row is computed once
  // and all loads of the tile are in flight together), a wavefront one
  constexpr int RPT = NT > 64 ? 2 : 1;
  const bool kept = r1 - r0 <= RPT * rows_per_pass;

  UnitValues x[RPT];
  float m = 0.f;  // fmaxf drops NaNs, as the oracle's does
  auto take = [&](const UnitValues& xx) {
#pragma unroll
    for (int i = 0; i < 8; ++i) m = fmaxf(m, fmaxf(fabsf(xx.g1[i]), fabsf(xx.g2[i])));
  };
  if (kept) {
#pragma unroll
    for (int e = 0; e < RPT; ++e) {
      const int rr = r0 + e * rows_per_pass + row_in_pass;
      const int r = rr < r1 ? rr : r1 - 1;  // (idle lanes repeat the last row: the norm's butterfly needs every lane)
      x[e] = unit_values(a, j.tok + (r - r0), head, u, r);
      if (rr < r1) take(x[e]), side_row(rr, x[e]);
    }
  } else {
    for (int rb = r0; rb < r1; rb += rows_per_pass) {
      const bool live = rb + row_in_pass < r1;
      const int r = live ? rb + row_in_pass : r1 - 1;
      const UnitValues xx = unit_values(a, j.tok + (r - r0), head, u, r);
      if (live) take(xx), side_row(r, xx);
    }
  }
  m = wave_max(m);
  if (NT > 64) {
    __syncthreads();  // (the buffer may still be read for the workgroup's previous tile)
    if ((tid & 63) == 0) red[0][tid >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
  }
  const float qmax = QUANT == FDATTN_CACHE_INT8 ? 127.0f : 448.0f;
  const float s_now = m > 0.f ? __fdiv_rn(m, qmax) : 0.f;
  const float sc = j.prior_rows > 0 ? (s_now > s_old ? s_now : s_old) : (s_now > 0.f ? s_now : 1.0f);
  if (!cached) return;  // (uniform over the workgroup; its barriers are behind it)
  if (tid == 0) scale[at] = sc;

  uint8_t* const tile = (is_k ? a.key_cache : a.value_cache) + at * a.bs * a.d;
  if (j.prior_rows > 0 && sc > s_old) {  // the scale grew: the rows of earlier calls move to the new grid
    const int pieces = j.prior_rows * a.d / 16;
    for (int i = tid; i < pieces; i += NT) {
      uint4 w = *reinterpret_cast<const uint4*>(tile + (size_t)i * 16);
      u32 ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        u32 o = 0;
#pragma unroll
        for (int by = 0; by < 4; ++by) o |= requant1<QUANT>((ws[e] >> (8 * by)) & 0xffu, s_old, sc) << (8 * by);
        ws[e] = o;
      }
      *reinterpret_cast<uint4*>(tile + (size_t)i * 16) = make_uint4(ws[0], ws[1], ws[2], ws[3]);
    }
  }
  const float rsc = __builtin_amdgcn_rcpf(sc);
  auto store_row = [&](int r, const UnitValues& xx) {
    u32 q1[2] = {0, 0}, q2[2] = {0, 0};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      q1[i >> 2] |= quant1_shared<QUANT>(xx.g1[i], sc, rsc) << (8 * (i & 3));
      q2[i >> 2] |= quant1_shared<QUANT>(xx.g2[i], sc, rsc) << (8 * (i & 3));
    }
    const size_t roff = (size_t)(r - j.lb * a.bs) * a.d;
    *reinterpret_cast<uint2*>(tile + roff + xx.c1) = make_uint2(q1[0], q1[1]);
    *reinterpret_cast<uint2*>(tile + roff + xx.c2) = make_uint2(q2[0], q2[1]);
  };
  if (kept) {
#pragma unroll
    for (int e = 0; e < RPT; ++e) {
      const int rr = r0 + e * rows_per_pass + row_in_pass;
      if (rr < r1) store_row(rr, x[e]);
    }
  } else {
    for (int rb = r0; rb < r1; rb += rows_per_pass) {
      const bool live = rb + row_in_pass < r1;
      const int r = live ? rb + row_in_pass : r1 - 1;
      const UnitValues xx = unit_values(a, j.tok + (r - r0), head, u, r);
      if (live) store_row(r, xx);
    }
  }
}

// The same job for ONE of the two tensors by the head_dim / 16 threads of the token kernel that hold the K (or V) head
// of the token that stands for the tile - adjacent lanes of one wavefront, unit u each; `first` = the values of the job's
// first row, which these threads have computed already.  A job of one row (every job of a decode step) costs no
// recomputation; longer ones walk their rows one at a time.
template <int QUANT>
__device__ __forceinline__ void write_tile_rows(const WriterArgs& a, const TileJob& j, int h, bool is_k, int head, int u,
                                                const UnitValues& first) {
  const int uph = a.d / 16;
  const size_t at = (size_t)j.pb * a.hkv + h;
  float* const scale = is_k ? a.k_scale : a.v_scale;
  float s_old = 0.f;  // asked for now - before anything of this tile is stored - and needed after the rows' maximum
  if (j.prior_rows > 0) s_old = scale[at];
  float m = 0.f;  // fmaxf drops NaNs, as the oracle's does
  for (int r = j.r0; r < j.r1; ++r) {
    const UnitValues x = r == j.r0 ? first : unit_values(a, j.tok + (r - j.r0), head, u, r);
#pragma unroll
    for (int i = 0; i < 8; ++i) m = fmaxf(m, fmaxf(fabsf(x.g1[i]), fabsf(x.g2[i])));
  }
  for (int o = 1; o < uph; o <<= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  const float qmax = QUANT == FDATTN_CACHE_INT8 ? 127.0f : 448.0f;
  const float s_now = m > 0.f ? __fdiv_rn(m, qmax) : 0.f;
  const float sc = j.prior_rows > 0 ? (s_now > s_old ? s_now : s_old) : (s_now > 0.f ? s_now : 1.0f);
  if (u == 0) scale[at] = sc;
  uint8_t* const tile = (is_k ? a.key_cache : a.value_cache) + at * a.bs * a.d;
  if (j.prior_rows > 0 && sc > s_old) {  // the scale grew: the rows of earlier calls move to the new grid
    const int pieces = j.prior_rows * a.d / 16;
    for (int i = u; i < pieces; i += uph) {
      const uint4 w = *reinterpret_cast<const uint4*>(tile + (size_t)i * 16);
      u32 ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        u32 o = 0;
#pragma unroll
        for (int by = 0; by < 4; ++by) o |= requant1<QUANT>((ws[e] >> (8 * by)) & 0xffu, s_old, sc) << (8 * by);
        ws[e] = o;
      }
      *reinterpret_cast<uint4*>(tile + (size_t)i * 16) = make_uint4(ws[0], ws[1], ws[2], ws[3]);
    }
  }
  const float rsc = __builtin_amdgcn_rcpf(sc);
  for (int r = j.r0; r < j.r1; ++r) {
    const UnitValues x = r == j.r0 ? first : unit_values(a, j.tok + (r - j.r0), head, u, r);
    u32 q1[2] = {0, 0}, q2[2] = {0, 0};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      q1[i >> 2] |= quant1_shared<QUANT>(x.g1[i], sc, rsc) << (8 * (i & 3));
      q2[i >> 2] |= quant1_shared<QUANT>(x.g2[i], sc, rsc) << (8 * (i & 3));
    }
    const size_t roff = (size_t)(r - j.lb * a.bs) * a.d;
    *reinterpret_cast<uint2*>(tile + roff + x.c1) = make_uint2(q1[0], q1[1]);
    *reinterpret_cast<uint2*>(tile + roff + x.c2) = make_uint2(q2[0], q2[1]);
  }
}

// Steps of few tokens per sequence (decode steps, speculative steps, mixed batches): grid (kv heads, tokens), one
// wavefront per token; the wavefront of a token that stands for a tile writes it, every other one leaves at once.
template <int QUANT>
__global__ __launch_bounds__(64) void write_cache_tiles_kernel(WriterArgs a) {
  const int h = blockIdx.x, tok = a.tok0 + blockIdx.y;
  BatchRows rows;
  rows.load(a.cu_seqlens_q, a.seq_lens_decoder, a.batch);
  TileJob j;
  if (tile_job(a, rows.at(rows.seq_of(tok)), tok, j)) write_tile<QUANT, 64>(a, j, h, blockIdx.z == 0, nullptr);
}

// Long chunks (most tokens stand for no tile; a tile has many rows): grid (kv heads, batch + groups of 64 tokens), one
// workgroup of 256 threads per candidate.  Candidates 0 .. batch-1: the tile that sequence c's first token starts.
// Candidate batch + g: the tiles started at a multiple of the block size by tokens 64 g .. 64 g + 63 of the call that
// are not the first of their sequence - walking the sequences that have tokens in that range.
template <int QUANT>
__device__ __forceinline__ void tile_candidate(const WriterArgs& a, int h, int c, bool is_k, float (*red)[4]) {
  BatchRows rows;
  rows.load(a.cu_seqlens_q, a.seq_lens_decoder, a.batch);
  TileJob j;
  // (every thread of the workgroup stays to the end: the cross-lane reads below see whole wavefronts)
  if (c < a.batch) {
    const SeqRows sr = rows.at(c);
    if (tile_job(a, sr, sr.first, j)) write_tile<QUANT, 256>(a, j, h, is_k, red);
    return;
  }
  const int t_lo = (c - a.batch) * 64, t_hi = min(t_lo + 64, a.num_tokens);
  if (t_lo >= t_hi) return;
  for (int b = rows.seq_of(t_lo); b < a.batch; ++b) {
    const SeqRows sr = rows.at(b);
    if (sr.first >= t_hi) break;
    const int tok_first = sr.first, p0 = sr.cached;
    // the first token of the sequence in the range whose position is a multiple of the block size, then every bs-th
    const int t_from = max(t_lo, tok_first + 1);
    const int pos_from = p0 + (t_from - tok_first);
    const int first_aligned = (pos_from + a.bs - 1) / a.bs * a.bs;
    for (int t = t_from + (first_aligned - pos_from); t < t_hi; t += a.bs)
      if (tile_job(a, sr, t, j)) write_tile<QUANT, 256>(a, j, h, is_k, red);
  }
}
template <int QUANT>
__global__ __launch_bounds__(256) void write_cache_tiles_chunk_kernel(WriterArgs a) {
  __shared__ float red[1][4];
  tile_candidate<QUANT>(a, blockIdx.x, blockIdx.y, blockIdx.z == 0, red);
}

// Long chunks in one launch: the first kv_heads x candidates x 2 workgroups are write_cache_tiles_chunk_kernel's (they
// run longest - a chain of loads, a reduction, stores - and start first), the others the token kernel's, which here
// writes q_out only; neither reads what the other writes.
template <int QUANT>
__global__ __launch_bounds__(256) void write_cache_chunk_kernel(WriterArgs a, int candidates, int unit_blocks) {
  __shared__ float red[1][4];
  const int tiles = 2 * a.hkv * candidates;
  if ((int)blockIdx.x < tiles) {
    const int i = blockIdx.x >> 1;
    tile_candidate<QUANT>(a, i % a.hkv, i / a.hkv, (blockIdx.x & 1) == 0, red);
  } else {
    write_token_units<QUANT, 4>(a, (blockIdx.x - tiles) % unit_blocks, (blockIdx.x - tiles) / unit_blocks);
  }
}

}  // namespace fdattn

using namespace fdattn;

extern "C" int fdattn_write_cache_kv(
    const void* qkv, void* q_out, void* k_out, void* v_out, void* key_cache, void* value_cache,
    float* cache_k_scale, float* cache_v_scale, const float* rope_cos,
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
    float* cache_k_scale, float* cache_v_scale, const float* rope_cos,
    const float* rope_sin, const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* cu_seqlens_q, int num_tokens, int batch, int hq, int hkv, int head_dim,
    int block_size, int max_blocks_per_seq, int num_blocks, int max_pos, int rope_style,
    int cache_quant_type, const fdattn_step_extras* extras, void* stream) {
  const fdattn_step_extras none = {nullptr, nullptr, nullptr, 0.f, 0};
  const fdattn_step_extras& ep = extras ? *extras : none;
  if (quant_dynamic(cache_quant_type)) {
    const int u = head_dim / 16;
    if (head_dim % 16 != 0 || u <= 0 || (u & (u - 1)) != 0 || u > 64)
      return fail(FDATTN_ERR_SHAPE, "fdattn_write_cache_kv: the dynamic and per-block cache formats need head_dim = "
                  "16 * a power of two up to 1024, got %d", head_dim);
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
               (const uint16_t*)ep.qkv_bias, ep.q_norm_weight, ep.k_norm_weight, ep.rms_norm_eps, 0, 0};
  const int units = (hq + 2 * hkv) * (head_dim / 16);
  hipStream_t s = (hipStream_t)stream;
  // the y dimension of a grid holds 65,535 workgroups: more tokens go in slices
  for (int t0 = 0; t0 < num_tokens; t0 += 65535) {
    a.tok0 = t0;
    const dim3 grid((units + 255) / 256, num_tokens - t0 < 65535 ? num_tokens - t0 : 65535);
    if (quant_blockwise(cache_quant_type) && num_tokens <= batch) {
      // no more tokens than sequences - a decode step: one launch, the token kernel keeps the tiles itself (a tile's job
      // is one row there; should a sequence bring several after all, its threads walk them)
      if (quant_bytes(cache_quant_type) == FDATTN_CACHE_INT8) hipLaunchKernelGGL((write_cache_kv_kernel<FDATTN_CACHE_INT8, 3>), grid, dim3(256), 0, s, a);
      else hipLaunchKernelGGL((write_cache_kv_kernel<FDATTN_CACHE_FP8_E4M3, 3>), grid, dim3(256), 0, s, a);
    } else if (quant_blockwise(cache_quant_type) && (long long)num_tokens >= 16LL * batch && num_tokens <= 65535 &&
               2LL * hkv * (batch + (num_tokens + 63) / 64) + (long long)grid.x * num_tokens <= 0x7fffffffLL) {
      // long chunks: a workgroup per candidate tile start computes the tile's K and V rows once and writes them to the
      // cache (with the tile's scales) and to k_out / v_out; the token kernel is left the Q heads
      a.tiles_write_rows = 1;
      const bool i8 = quant_bytes(cache_quant_type) == FDATTN_CACHE_INT8;
      const int candidates = batch + (num_tokens + 63) / 64;
      // (only the Q heads' unit blocks of a token do anything in the token part - plus the K and V rows of skipped
      // tokens, which is why all of them are launched)
      const dim3 mgrid((unsigned)(2 * hkv * candidates + (int)grid.x * num_tokens));
      if (i8) hipLaunchKernelGGL((write_cache_chunk_kernel<FDATTN_CACHE_INT8>), mgrid, dim3(256), 0, s, a, candidates, (int)grid.x);
      else hipLaunchKernelGGL((write_cache_chunk_kernel<FDATTN_CACHE_FP8_E4M3>), mgrid, dim3(256), 0, s, a, candidates, (int)grid.x);
    } else if (quant_blockwise(cache_quant_type)) {
      // Q, k_out, v_out from the token kernel; the cache and its tile scales from the tile kernel (independent of it)
      hipLaunchKernelGGL((write_cache_kv_kernel<FDATTN_CACHE_INT8, 2>), grid, dim3(256), 0, s, a);
      const bool i8 = quant_bytes(cache_quant_type) == FDATTN_CACHE_INT8;
      if ((long long)num_tokens >= 16LL * batch && batch + (num_tokens + 63) / 64 <= 65535) {
        // long chunks: a workgroup per candidate tile start (all in the first slice's launch: they cover every token)
        if (t0 == 0) {
          const dim3 cgrid(hkv, batch + (num_tokens + 63) / 64, 2);
          if (i8) hipLaunchKernelGGL((write_cache_tiles_chunk_kernel<FDATTN_CACHE_INT8>), cgrid, dim3(256), 0, s, a);
          else hipLaunchKernelGGL((write_cache_tiles_chunk_kernel<FDATTN_CACHE_FP8_E4M3>), cgrid, dim3(256), 0, s, a);
        }
      } else {
        const dim3 tgrid(hkv, grid.y, 2);
        if (i8) hipLaunchKernelGGL((write_cache_tiles_kernel<FDATTN_CACHE_INT8>), tgrid, dim3(64), 0, s, a);
        else hipLaunchKernelGGL((write_cache_tiles_kernel<FDATTN_CACHE_FP8_E4M3>), tgrid, dim3(64), 0, s, a);
      }
    } else if (cache_quant_type == FDATTN_CACHE_INT8)
      hipLaunchKernelGGL((write_cache_kv_kernel<FDATTN_CACHE_INT8, 0>), grid, dim3(256), 0, s, a);
    else if (cache_quant_type == FDATTN_CACHE_FP8_E4M3)
      hipLaunchKernelGGL((write_cache_kv_kernel<FDATTN_CACHE_FP8_E4M3, 0>), grid, dim3(256), 0, s, a);
    else if (cache_quant_type == FDATTN_CACHE_INT8_DYNAMIC)
      hipLaunchKernelGGL((write_cache_kv_kernel<FDATTN_CACHE_INT8, 1>), grid, dim3(256), 0, s, a);
    else
      hipLaunchKernelGGL((write_cache_kv_kernel<FDATTN_CACHE_FP8_E4M3, 1>), grid, dim3(256), 0, s, a);
  }
  return check_launch("fdattn_write_cache_kv");
}
