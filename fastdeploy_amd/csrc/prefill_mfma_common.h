// Pieces shared by the MFMA append-attention kernels: vector types, conversions of cache bytes and of the chunk's own
// bf16 rows into the fp16 numbers the 16-bit MFMAs take, small LDS and cross-lane helpers.
#pragma once
#include "fdattn_common.h"

namespace fdattn {
namespace pf {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef u32 u4v __attribute__((ext_vector_type(4)));
typedef short v4s __attribute__((__vector_size__(4 * sizeof(short))));
typedef short v8s __attribute__((__vector_size__(8 * sizeof(short))));
typedef __attribute__((address_space(3))) uint16_t lds_u16;

__device__ __forceinline__ void lds_store16(lds_u16* p, uint4 v) {
  const u4v w = {v.x, v.y, v.z, v.w};
  *reinterpret_cast<__attribute__((address_space(3))) u4v*>(p) = w;
}

__device__ __forceinline__ u32 pack_bf16(float lo, float hi) { return (u32)f32_to_bf16(lo) | ((u32)f32_to_bf16(hi) << 16); }
__device__ __forceinline__ u32 pack_f16(float lo, float hi) {
  const v2h v = {(_Float16)lo, (_Float16)hi};
  return __builtin_bit_cast(u32, v);
}
__device__ __forceinline__ u32 pack_f16_rtz(float lo, float hi) { return __builtin_bit_cast(u32, __builtin_amdgcn_cvt_pkrtz(lo, hi)); }
__device__ __forceinline__ float sat_f16(float x) { return __builtin_amdgcn_fmed3f(x, -65504.0f, 65504.0f); }

// 8 bf16 values of the chunk's own V -> fp16, saturating (bf16 is exact in fp16 wherever fp16 is normal)
__device__ __forceinline__ uint4 chunk_v_f16(uint4 v) {
  const u32 vw[4] = {v.x, v.y, v.z, v.w};
  u32 hw[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) hw[e] = pack_f16(sat_f16(bf16lo_to_f32(vw[e])), sat_f16(bf16hi_to_f32(vw[e])));
  return make_uint4(hw[0], hw[1], hw[2], hw[3]);
}

// Running maximum and minimum over fp16 values, two lanes of a register and two registers per instruction
// (v_pk_maximum3_f16 / v_pk_minimum3_f16: 8 values cost 4 instructions), and the test of such a pair against a limit:
// does any value lie beyond +-limit?  (NaNs propagate through both and answer yes.)
struct F16Range { u32 mx, mn; };  // packed pairs; start from {0, 0}
__device__ __forceinline__ void f16x8_range(uint4 h, F16Range& r) {
  asm("v_pk_maximum3_f16 %0, %1, %2, %0" : "+v"(r.mx) : "v"(h.x), "v"(h.y));
  asm("v_pk_maximum3_f16 %0, %1, %2, %0" : "+v"(r.mx) : "v"(h.z), "v"(h.w));
  asm("v_pk_minimum3_f16 %0, %1, %2, %0" : "+v"(r.mn) : "v"(h.x), "v"(h.y));
  asm("v_pk_minimum3_f16 %0, %1, %2, %0" : "+v"(r.mn) : "v"(h.z), "v"(h.w));
}
__device__ __forceinline__ bool f16_range_beyond(const F16Range& r, float limit) {
  // on the bit patterns: a positive fp16 above the limit is a larger signed 16-bit integer than the limit's pattern,
  // a negative one below -limit a larger unsigned one than -limit's pattern (positive and negative NaNs included)
  const int pos = (int)__builtin_bit_cast(unsigned short, (_Float16)limit);
  const u32 neg = (u32)pos | 0x8000u;
  return (int)(short)(r.mx & 0xffffu) > pos || (int)(short)(r.mx >> 16) > pos || (r.mn & 0xffffu) > neg || (r.mn >> 16) > neg;
}

// Running sum of the magnitudes of fp16 values, as a packed pair (start from 0; 8 values cost 8 instructions; the
// caller keeps the pair's sums inside fp16) and the pair's total; further down, the sum of an integer over the
// wavefront (valid in lane 63: rotations within the rows of 16 lanes, then the rows' last lanes handed on).
__device__ __forceinline__ void f16x8_abs_sum(uint4 h, u32& acc) {
  const u32 w[4] = {h.x, h.y, h.z, h.w};
  v2h a = __builtin_bit_cast(v2h, acc);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const u32 m = w[e] & 0x7fff7fffu;
    a += __builtin_bit_cast(v2h, m);
  }
  acc = __builtin_bit_cast(u32, a);
}
// The same over cache bytes as they are: int8 codes by two instructions per four bytes (the sum of |b| is the sum of
// absolute differences of b ^ 0x80 from 0x80, byte by byte: v_sad_u8; exact, in an integer); e4m3 codes by way of their
// fp16 values.  acc: the integer sum (int8) or the packed pair (fp8).
template <int QUANT>
__device__ __forceinline__ void code_abs_sum(u32 w0, u32 w1, uint4 as_f16, u32& acc) {
  if (QUANT == FDATTN_CACHE_INT8) {
    acc = __builtin_amdgcn_sad_u8(w0 ^ 0x80808080u, 0x80808080u, acc);
    acc = __builtin_amdgcn_sad_u8(w1 ^ 0x80808080u, 0x80808080u, acc);
  } else {
    f16x8_abs_sum(as_f16, acc);
  }
}
__device__ __forceinline__ float f16_pair_total(u32 acc) {
  const v2h a = __builtin_bit_cast(v2h, acc);
  return (float)a[0] + (float)a[1];
}
// A thread's K sum and V sum of a tile (32 codes each) as one word, (K sum / unit) | (V sum / unit) << 16 with
// unit = 32 (int8) or 64 (e4m3), rounded: a field is at most 128 (224), the sum over four wavefronts at most 2^15
// (57344) - inside its 16 bits.  One integer reduction then serves both.
template <int QUANT>
__device__ __forceinline__ u32 magnitude_word(u32 k_acc, u32 v_acc) {
  if (QUANT == FDATTN_CACHE_INT8) return ((k_acc + 16u) >> 5) | (((v_acc + 16u) >> 5) << 16);
  const u32 k = (u32)(f16_pair_total(k_acc) * (1.0f / 64.0f) + 0.5f), v = (u32)(f16_pair_total(v_acc) * (1.0f / 64.0f) + 0.5f);
  return k | (v << 16);
}
template <int QUANT>
constexpr float magnitude_unit() { return QUANT == FDATTN_CACHE_INT8 ? 32.0f : 64.0f; }
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ u32 dpp_or_zero(u32 v) {
  return (u32)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xf, false);
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_or_zero(float v) {  // (the bits travel; a float must not be converted on its way into the integer version)
  return __uint_as_float(dpp_or_zero<CTRL, ROW_MASK>(__float_as_uint(v)));
}
__device__ __forceinline__ u32 wave_sum_lane63(u32 v) {
  v += dpp_or_zero<0x128, 0xf>(v);  // row_ror 8, 4, 2, 1: every lane holds its row's sum
  v += dpp_or_zero<0x124, 0xf>(v);
  v += dpp_or_zero<0x122, 0xf>(v);
  v += dpp_or_zero<0x121, 0xf>(v);
  v += dpp_or_zero<0x142, 0xa>(v);  // row_bcast 15 into rows 1 and 3: rows 0 + 1, rows 2 + 3
  v += dpp_or_zero<0x143, 0xc>(v);  // row_bcast 31 into rows 2 and 3: row 3 holds everything
  return v;
}

// 8 cache bytes -> 8 fp16 holding the bytes' exact values
template <int QUANT>
__device__ __forceinline__ uint4 cvt8(u32 w0, u32 w1) {
  if (QUANT == FDATTN_CACHE_INT8) {
    // one conversion per byte, each picking its (sign-extended) byte out of the word and writing its half of the
    // result register (v_cvt_f16_i16 with sub-dword addressing): every int8 value is an fp16 value
    u32 o[4];
    asm("v_cvt_f16_i16_sdwa %0, sext(%2) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_0\n\t"
        "v_cvt_f16_i16_sdwa %0, sext(%2) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_1\n\t"
        "v_cvt_f16_i16_sdwa %1, sext(%2) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_2\n\t"
        "v_cvt_f16_i16_sdwa %1, sext(%2) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_3"
        : "=&v"(o[0]), "=&v"(o[1])
        : "v"(w0));
    asm("v_cvt_f16_i16_sdwa %0, sext(%2) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_0\n\t"
        "v_cvt_f16_i16_sdwa %0, sext(%2) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_1\n\t"
        "v_cvt_f16_i16_sdwa %1, sext(%2) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_2\n\t"
        "v_cvt_f16_i16_sdwa %1, sext(%2) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_3"
        : "=&v"(o[2]), "=&v"(o[3])
        : "v"(w1));
    return make_uint4(o[0], o[1], o[2], o[3]);
  }
  // two e4m3 codes -> two fp16 numbers in one instruction (v_cvt_scalef32_pk_f16_fp8 with scale 1: every e4m3 value
  // is an fp16 value, so nothing is rounded)
  const v2h a = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((int)w0, 1.0f, false), b = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((int)w0, 1.0f, true);
  const v2h c = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((int)w1, 1.0f, false), d = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((int)w1, 1.0f, true);
  return make_uint4(__builtin_bit_cast(u32, a), __builtin_bit_cast(u32, b), __builtin_bit_cast(u32, c), __builtin_bit_cast(u32, d));
}

// The same conversion in instructions the compiler can see (five per four int8 bytes instead of four): for results
// that go straight into an MFMA.  The sub-dword writes above sit inside asm statements, which the compiler counts as one
// instruction each when it spaces a register's last write from the MFMA that reads it - and the register written
// by a statement's LAST instruction then reaches the MFMA one wait state too early (seen as one wrong element of
// eight in the scoring pass of the block selector).  b ^ 0x80 behind the exponent byte 0x64 is the fp16 number
// 1024 + 128 + b; a packed subtraction of 1152 leaves b.
template <int QUANT>
__device__ __forceinline__ uint4 cvt8_for_mfma(u32 w0, u32 w1) {
  if (QUANT != FDATTN_CACHE_INT8) return cvt8<QUANT>(w0, w1);
  const v2h off = {(_Float16)1152.0f, (_Float16)1152.0f};
  u32 o[4];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const u32 x = (i ? w1 : w0) ^ 0x80808080u;
    const u32 lo = __builtin_amdgcn_perm(0x64646464u, x, 0x04010400u), hi = __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u);
    o[2 * i] = __builtin_bit_cast(u32, __builtin_bit_cast(v2h, lo) - off);
    o[2 * i + 1] = __builtin_bit_cast(u32, __builtin_bit_cast(v2h, hi) - off);
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

// Workgroup barrier that orders LDS traffic only: __syncthreads() also waits for every global load in flight
// (vmcnt(0)), and the staging loads of a later tile are meant to stay in flight across it.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// the value held by lane ^ 32
__device__ __forceinline__ float swap32(float x) {
  typedef u32 u2v __attribute__((ext_vector_type(2)));
  const u2v r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(threadIdx.x & 32 ? r[0] : r[1]);
}

}  // namespace pf
}  // namespace fdattn
