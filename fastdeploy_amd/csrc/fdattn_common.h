// Shared device/host helpers of libfdattn.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fdattn.h"

namespace fdattn {

// Records the message fdattn_last_error() returns for this thread; returns `code`.
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);

// Rows of a mixed batch (prefill rows, decode rows and idle slots in one step).  With both
// pointers NULL sequence b owns q / out row b and every sequence is a decode row.  Otherwise
// sequence b's tokens are rows cu_seqlens_q[b] .. cu_seqlens_q[b+1]-1; it is a decode row if
// it has exactly one token and seq_lens_encoder[b] == 0, a prefill row if seq_lens_encoder[b] > 0.
struct RowMap {
  const int32_t* cu_seqlens_q;
  const int32_t* seq_lens_encoder;
};
// false: sequence b is not a decode row (nothing to read, nothing to write); row = its q / out row
__device__ __forceinline__ bool decode_row(const RowMap& m, int b, int& row) {
  row = b;
  if (!m.cu_seqlens_q) return true;
  row = m.cu_seqlens_q[b];
  return m.cu_seqlens_q[b + 1] - row == 1 && (!m.seq_lens_encoder || m.seq_lens_encoder[b] == 0);
}
// The same for steps whose decode rows may bring up to max_tokens tokens (the draft tokens of a speculative step):
// toks = the sequence's tokens; row = the first of its q / out rows.
__device__ __forceinline__ bool decode_rows(const RowMap& m, int b, int max_tokens, int& row, int& toks) {
  row = b;
  toks = 1;
  if (!m.cu_seqlens_q) return true;
  row = m.cu_seqlens_q[b];
  toks = m.cu_seqlens_q[b + 1] - row;
  return toks >= 1 && toks <= max_tokens && (!m.seq_lens_encoder || m.seq_lens_encoder[b] == 0);
}
__device__ __forceinline__ bool prefill_row(const RowMap& m, int b) {
  return !m.seq_lens_encoder || m.seq_lens_encoder[b] > 0;
}

// The sequence of token tok: the last b with cu_seqlens_q[b] <= tok (sequences may be empty).  A binary search is a chain
// of log2(batch) dependent loads; a step of one token per sequence - the usual decode step - is answered by one probe
// of two independent loads, since then token t is sequence t.
__device__ __forceinline__ int seq_of_token(const int32_t* cu, int batch, int tok) {
  const int guess = min(max(tok, 0), batch - 1);
  const int c0 = cu[guess], c1 = cu[guess + 1];
  if (c0 <= tok && tok < c1) return guess;
  int lo = 0, hi = batch;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu[mid] <= tok) lo = mid; else hi = mid;
  }
  return lo;
}

// The batch's row bounds and cached lengths, held by a wavefront: lane l keeps sequence l's cu_seqlens_q[l],
// cu_seqlens_q[l + 1] and seq_lens_decoder[l] - three independent loads, one round trip to memory for everything a
// kernel needs to place a token, where a search through cu_seqlens_q followed by the sequence's entries is a chain of
// dependent ones (a microsecond each, and short-lived workgroups consist of little else).  Batches of more than 64
// sequences fall back to those loads.
// EVERY lane of the wavefront must be active in load(), seq_of() and at(): they read across lanes, and what a lane
// that has left a kernel early holds in its registers is undefined (the compiler moves and copies values under the
// mask of the lanes still active).  Take a sequence's SeqRows out first, branch afterwards.
struct SeqRows { int b, first, end, cached; };  // sequence b: its rows [first, end) of the call, its cached tokens
struct BatchRows {
  const int32_t* cu;
  const int32_t* dec;
  int batch;
  int c0, c1, d;  // lane l: sequence l
  __device__ __forceinline__ void load(const int32_t* cu_seqlens_q, const int32_t* seq_lens_decoder, int n) {
    cu = cu_seqlens_q, dec = seq_lens_decoder, batch = n;
    const int lane = threadIdx.x & 63;
    const bool in = n <= 64 && lane < n;
    c0 = in ? cu[lane] : 0x7fffffff;
    c1 = in ? cu[lane + 1] : 0x7fffffff;
    d = in ? dec[lane] : 0;
  }
  __device__ __forceinline__ SeqRows at(int b) const {
    if (batch <= 64) return SeqRows{b, __builtin_amdgcn_readlane(c0, b), __builtin_amdgcn_readlane(c1, b), __builtin_amdgcn_readlane(d, b)};
    return SeqRows{b, cu[b], cu[b + 1], dec[b]};
  }
  // the sequence of token tok, as seq_of_token gives it (tok: uniform over the wavefront)
  __device__ __forceinline__ int seq_of(int tok) const {
    if (batch > 64) return seq_of_token(cu, batch, tok);
    const unsigned long long holds = __ballot(c0 <= tok && tok < c1);
    if (holds) return __ffsll((long long)holds) - 1;
    const unsigned long long before = __ballot(c0 <= tok);  // no sequence holds it: the last one that starts at or before it
    return before ? 63 - __clzll((long long)before) : 0;
  }
};

// cache_quant_type -> how the bytes are encoded / where the scales live
__host__ __device__ constexpr int quant_bytes(int q) {
  return q == FDATTN_CACHE_INT8_DYNAMIC || q == FDATTN_CACHE_INT8_BLOCK
             ? FDATTN_CACHE_INT8
             : (q == FDATTN_CACHE_FP8_E4M3_DYNAMIC || q == FDATTN_CACHE_FP8_E4M3_BLOCK ? FDATTN_CACHE_FP8_E4M3 : q);
}
// one scale per (block, KV head) tile, in scale caches [num_blocks, hkv]
__host__ __device__ constexpr bool quant_blockwise(int q) {
  return q == FDATTN_CACHE_INT8_BLOCK || q == FDATTN_CACHE_FP8_E4M3_BLOCK;
}
// the scales travel with the stored rows (scale caches written by the cache writer) instead of per channel:
// one per stored row, [num_blocks, hkv, block_size], or one per tile.  The kernels treat a per-tile scale as
// a row of block_size equal scales: scale_rows() is the stride from tile to tile, and a row's scale sits
// scale_slot(slot) past the tile's first one.
__host__ __device__ constexpr bool quant_dynamic(int q) {
  return q == FDATTN_CACHE_INT8_DYNAMIC || q == FDATTN_CACHE_FP8_E4M3_DYNAMIC || quant_blockwise(q);
}
__host__ __device__ constexpr int scale_rows(int q, int block_size) { return quant_blockwise(q) ? 1 : block_size; }
__host__ __device__ constexpr bool quant_known(int q) { return q >= FDATTN_CACHE_INT8 && q <= FDATTN_CACHE_FP8_E4M3_BLOCK; }

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned int u32;

__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float((u32)h << 16); }
__device__ __forceinline__ float bf16lo_to_f32(u32 w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16hi_to_f32(u32 w) { return __uint_as_float(w & 0xffff0000u); }

// round to nearest even; NaN -> quiet NaN with the sign kept
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  u32 u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// two at once, by the hardware's conversion (v_cvt_pk_bf16_f32): the same bits as f32_to_bf16 for every one of the
// 2^32 inputs - NaNs and subnormals included (checked exhaustively on the GPU) - at a sixth of the instructions
__device__ __forceinline__ u32 pack2_bf16(float lo, float hi) {
  typedef float f2v __attribute__((ext_vector_type(2)));
  typedef __bf16 bf2v __attribute__((ext_vector_type(2)));
  const f2v x = {lo, hi};
  return __builtin_bit_cast(u32, __builtin_convertvector(x, bf2v));
}

// fp8 e4m3fn (OCP): 1-4-3, bias 7, max 448, no infinities.
__device__ __forceinline__ float e4m3_to_f32(u32 c) {
  // (c & 0x7f) << 20 is the value scaled by 2^-120 in fp32 terms (exponent field
  // shifted by 120); subnormal codes land on fp32 subnormal-free ground after the
  // multiply because 2^120 * 2^-126 * m/8 is exact.
  u32 mag = (c & 0x7fu) << 20;
  float v = __uint_as_float(mag) * 1.329227995784916e36f;  // 2^120
  return (c & 0x80u) ? -v : v;
}

// clamp to +-448, then round to nearest even onto the e4m3fn grid
__device__ __forceinline__ u32 f32_to_e4m3(float x) {
  u32 s = (__float_as_uint(x) >> 24) & 0x80u;
  float a = fabsf(x);
  if (a != a) return s | 0x7fu;
  if (a >= 448.0f) return s | 0x7eu;
  if (a < 0.015625f) return s | (u32)(int)__builtin_rintf(a * 512.0f);
  int e = (int)(__float_as_uint(a) >> 23) - 127;
  float scale = __uint_as_float((u32)(127 + 3 - e) << 23);
  int m = (int)__builtin_rintf(a * scale);  // [8, 16]
  if (m == 16) {
    m = 8;
    e += 1;
  }
  return s | ((u32)(e + 7) << 3) | (u32)(m - 8);
}

// 16-byte accesses with the non-temporal hint, for bytes that are read or written once per launch: without it a
// stream is allocated in the L2 and the memory-side cache on its way through and evicts itself
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 nt_load16(const void* p) {
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void nt_store16(void* p, uint4 v) {
  const u32x4 w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(p));
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

}  // namespace fdattn
