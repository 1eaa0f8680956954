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

// cache_quant_type -> how the bytes are encoded / whether the scales are per stored row
__host__ __device__ constexpr int quant_bytes(int q) {
  return q == FDATTN_CACHE_INT8_DYNAMIC ? FDATTN_CACHE_INT8 : (q == FDATTN_CACHE_FP8_E4M3_DYNAMIC ? FDATTN_CACHE_FP8_E4M3 : q);
}
__host__ __device__ constexpr bool quant_dynamic(int q) {
  return q == FDATTN_CACHE_INT8_DYNAMIC || q == FDATTN_CACHE_FP8_E4M3_DYNAMIC;
}
__host__ __device__ constexpr bool quant_known(int q) { return q >= FDATTN_CACHE_INT8 && q <= FDATTN_CACHE_FP8_E4M3_DYNAMIC; }

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
