// Device code shared by the kernels that stream (block, head) tiles of the int8 / fp8 cache
// through LDS and feed them to the MFMA units as they are: the decode-attention kernel and
// the SQAttn scoring kernel.  head_dim 128, 4 query heads per KV head, block_size 64.
#pragma once
#include "fdattn_common.h"

namespace fdattn {

constexpr int kWaves = 4;      // wavefronts per workgroup
constexpr int kTileB = 8192;   // bytes of one K or V tile (64 tokens x 128 channels)
constexpr int kD = 128, kG = 4, kBS = 64;  // kG: query heads per MFMA row set (16 rows = 4 heads x 4 limbs)
constexpr int kSlotFloats = kG * kD;       // partial o of one row set
constexpr int kMaxSets = 2;                // row sets a decode wavefront carries: up to 8 query heads per KV head
constexpr int kMaxSetsSpec = 4;            // decode rows of several tokens: up to 16 (token, head) rows
constexpr int kMaxChunk = 128;        // units per chunk: two unit-table entries per lane
constexpr int kMaxChunkDecode = 256;  // the decode kernel with one or two row sets: four entries per lane

__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
// all-reduce within each 16-lane row (row_ror 8, 4, 2, 1)
__device__ __forceinline__ float row_max16(float v) {
  v = fmaxf(v, dpp_f<0x128>(v));
  v = fmaxf(v, dpp_f<0x124>(v));
  v = fmaxf(v, dpp_f<0x122>(v));
  v = fmaxf(v, dpp_f<0x121>(v));
  return v;
}
__device__ __forceinline__ float row_sum16(float v) {
  v += dpp_f<0x128>(v);
  v += dpp_f<0x124>(v);
  v += dpp_f<0x122>(v);
  v += dpp_f<0x121>(v);
  return v;
}

// Direct global->LDS load of one 8 KiB tile: 8 instructions of 64 lanes x 16 B.  LDS
// receives lane l of instruction i at byte i*1024 + l*16 (row 8i + l/8, position l%8);
// the lane fetches the 16-byte chunk (l%8) ^ f(row) of that row, so that row r's chunk c
// sits at position c ^ f(r).  f = (r >> SHIFT) & 7 spreads the later LDS reads over banks.
// The eight per-lane byte offsets depend on the lane only and are computed once.
//
// Written as inline assembly on purpose: the wavefront tracks its own loads with
// explicit s_waitcnt vmcnt(N) (N = tile loads issued after the one waited for), which
// stays correct whatever other memory operations the compiler interleaves, because
// loads return in order and younger operations only make the wait stricter.
// The tile loads carry the non-temporal hint: every cache byte is read exactly once per launch, and without the hint
// the stream is allocated in (and evicts itself from) the L2 and the memory-side cache on its way through - measured on
// batch 64 x 4k context: 94.6 us per launch without it, 82.8 us with it (5.65 -> 6.45 TB/s).
#define FD_LDS_POLICY " nt"
struct DmaOffsets { u32 o[8]; };

template <int SHIFT>
__device__ __forceinline__ DmaOffsets dma_offsets(int lane) {
  DmaOffsets d;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = 8 * i + (lane >> 3);
    const int c = (lane & 7) ^ ((row >> SHIFT) & 7);
    d.o[i] = (u32)(row * 128 + c * 16);
  }
  return d;
}

__device__ __forceinline__ void dma_tile(const uint8_t* gtile_in, u32 lds_addr, const DmaOffsets& d) {
  // the tile address is wave-uniform by construction; make that explicit so it sits in SGPRs
  const unsigned long long gp = (unsigned long long)gtile_in;
  const u32 glo = __builtin_amdgcn_readfirstlane((u32)gp), ghi = __builtin_amdgcn_readfirstlane((u32)(gp >> 32));
  const uint8_t* gtile = (const uint8_t*)(((unsigned long long)ghi << 32) | glo);
  u32 saved_m0;  // m0 (the LDS base of these loads) is put back as it was found
  asm volatile(
      "s_mov_b32 %[sv], m0\n\t"
      "s_mov_b32 m0, %[l]\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %[o0], %[g]" FD_LDS_POLICY "\n\t"
      "s_add_u32 m0, m0, 0x400\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %[o1], %[g]" FD_LDS_POLICY "\n\t"
      "s_add_u32 m0, m0, 0x400\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %[o2], %[g]" FD_LDS_POLICY "\n\t"
      "s_add_u32 m0, m0, 0x400\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %[o3], %[g]" FD_LDS_POLICY "\n\t"
      "s_add_u32 m0, m0, 0x400\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %[o4], %[g]" FD_LDS_POLICY "\n\t"
      "s_add_u32 m0, m0, 0x400\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %[o5], %[g]" FD_LDS_POLICY "\n\t"
      "s_add_u32 m0, m0, 0x400\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %[o6], %[g]" FD_LDS_POLICY "\n\t"
      "s_add_u32 m0, m0, 0x400\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %[o7], %[g]" FD_LDS_POLICY "\n\t"
      "s_mov_b32 m0, %[sv]\n\t"
      : [sv] "=&s"(saved_m0)
      : [l] "s"(lds_addr), [g] "s"(gtile), [o0] "v"(d.o[0]), [o1] "v"(d.o[1]), [o2] "v"(d.o[2]),
        [o3] "v"(d.o[3]), [o4] "v"(d.o[4]), [o5] "v"(d.o[5]), [o6] "v"(d.o[6]), [o7] "v"(d.o[7])
      : "memory", "scc");
}

// Direct global->LDS load of 64 consecutive floats (one per lane, lane l lands at byte 4l): the scale row of one
// (block, head) tile of the formats that keep one scale per stored row.  One load for the vmcnt bookkeeping.
__device__ __forceinline__ void dma_row64(const float* grow_in, u32 lds_addr, u32 lane_x4) {
  const unsigned long long gp = (unsigned long long)grow_in;
  const u32 glo = __builtin_amdgcn_readfirstlane((u32)gp), ghi = __builtin_amdgcn_readfirstlane((u32)(gp >> 32));
  const float* grow = (const float*)(((unsigned long long)ghi << 32) | glo);
  u32 saved_m0;
  asm volatile(
      "s_mov_b32 %[sv], m0\n\t"
      "s_mov_b32 m0, %[l]\n\ts_nop 0\n\t"
      "global_load_lds_dword %[o], %[g]" FD_LDS_POLICY "\n\t"
      "s_mov_b32 m0, %[sv]\n\t"
      : [sv] "=&s"(saved_m0)
      : [l] "s"(lds_addr), [g] "s"(grow), [o] "v"(lane_x4)
      : "memory", "scc");
}

__device__ __forceinline__ u32 lds_addr_of(const void* p) {
  return (u32)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}

__device__ __forceinline__ void wait_vm8() { asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); }
__device__ __forceinline__ void wait_vm9() { asm volatile("s_waitcnt vmcnt(9)" ::: "memory"); }
__device__ __forceinline__ void wait_vm10() { asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); }
__device__ __forceinline__ void wait_vm0() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void wait_lgkm0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

constexpr int kShiftK = 2, kShiftV = 1;

// Per-pair state of a wavefront.
struct PairState {
  v4i aq[2];  // Q limbs as the MFMA A operand, two k-steps of 64 channels
  float rs;   // logit scale of this lane's head (S layout: head = lane / 16)
  float m, l;
  float o[8];  // channel 16*ct + lane%16 of head lane/16
};

// The q and k_scale values a lane needs for its A operand rows, as loaded: requested early (they depend
// on the pair alone), turned into limbs later, when the first tiles are already on their way.
struct PairRaw {
  uint4 w[2][2];    // k-step s: 16 bf16 channels 16*(g + 4s) .. +15 of head (lane%16)/4
  float4 ks[2][4];  // their K scales
};

// k_scale: the per-channel K scales [hkv, 128], or NULL (all ones: the scales are per stored row and are applied
// to the scores).  group: query heads per KV head; set: which four of them (heads 4 set .. 4 set + 3; heads
// past the group read as zeros).  toks > 0: the sequence owns q rows row .. row + toks - 1 and the MFMA rows are
// (token, head) in that order - row 4 set + i is token (4 set + i) / group, head (4 set + i) % group; rows of
// tokens past toks read as zeros.
__device__ __forceinline__ PairRaw load_pair_issue(const uint16_t* q, const float* k_scale, int hkv, int p, int row, int lane,
                                                   int group = kG, int set = 0, int toks = 0) {
  const int h = p % hkv;  // row: the sequence's (first) row of q
  const int m = lane & 15, g = lane >> 4;
  int head = 4 * set + (m >> 2), tok = 0;
  if (toks > 0) {
    tok = head / group;
    head -= tok * group;
  }
  const bool live = toks > 0 ? tok < toks : head < group;
  const uint16_t* qrow = q + ((size_t)(row + (live ? tok : 0)) * hkv * group + h * group + (live ? head : 0)) * kD;
  const float* ks = k_scale + (size_t)h * kD;
  PairRaw r;
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    const int c0 = 16 * (g + 4 * s);
    r.w[s][0] = live ? *reinterpret_cast<const uint4*>(qrow + c0) : make_uint4(0u, 0u, 0u, 0u);
    r.w[s][1] = live ? *reinterpret_cast<const uint4*>(qrow + c0 + 8) : make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      r.ks[s][i] = k_scale ? *reinterpret_cast<const float4*>(ks + c0 + 4 * i) : make_float4(1.f, 1.f, 1.f, 1.f);
  }
  return r;
}

// A operand rows: row = head*4 + limb; lane (m = lane%16, g = lane/16) holds channels
// 16*(g + 4s) .. +15 of k-step s.  qs_out (optional): the lane's 32 products q * k_scale.
template <int QUANT>
__device__ __forceinline__ void load_pair_finish(const PairRaw& r, float sm_scale_log2, int lane, PairState& st,
                                                 float (*qs_out)[16] = nullptr) {
  const int m = lane & 15, limb = m & 3;
  float qs[2][16];
  float amax = 0.f;
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    const u32 w[8] = {r.w[s][0].x, r.w[s][0].y, r.w[s][0].z, r.w[s][0].w, r.w[s][1].x, r.w[s][1].y, r.w[s][1].z, r.w[s][1].w};
    const float k[16] = {r.ks[s][0].x, r.ks[s][0].y, r.ks[s][0].z, r.ks[s][0].w, r.ks[s][1].x, r.ks[s][1].y,
                         r.ks[s][1].z, r.ks[s][1].w, r.ks[s][2].x, r.ks[s][2].y, r.ks[s][2].z, r.ks[s][2].w,
                         r.ks[s][3].x, r.ks[s][3].y, r.ks[s][3].z, r.ks[s][3].w};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      qs[s][2 * j] = bf16lo_to_f32(w[j]) * k[2 * j];
      qs[s][2 * j + 1] = bf16hi_to_f32(w[j]) * k[2 * j + 1];
      amax = fmaxf(amax, fmaxf(fabsf(qs[s][2 * j]), fabsf(qs[s][2 * j + 1])));
    }
    if (qs_out) {
#pragma unroll
      for (int j = 0; j < 16; ++j) qs_out[s][j] = qs[s][j];
    }
  }
  amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
  amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
  float rsval;
  if (QUANT == FDATTN_CACHE_INT8) {
    const float inv = amax > 0.f ? 1048575.0f / amax : 0.f;
    rsval = amax * (1.0f / 1048575.0f) * sm_scale_log2;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      u32 pk[4] = {0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int X = (int)__builtin_rintf(qs[s][j] * inv);
        const int x0 = ((X + 64) & 127) - 64;
        const int X1 = (X - x0) >> 7;
        const int x1 = ((X1 + 64) & 127) - 64;
        const int x2 = (X1 - x1) >> 7;
        const int d = limb == 0 ? x0 : (limb == 1 ? x1 : (limb == 2 ? x2 : 0));
        pk[j >> 2] |= ((u32)d & 0xffu) << (8 * (j & 3));
      }
      st.aq[s] = (v4i){(int)pk[0], (int)pk[1], (int)pk[2], (int)pk[3]};
    }
  } else {
    // residual e4m3 limbs of x = qs * 256 / amax: limb0 = fp8(x), limb1 = fp8(x - limb0), ...
    const float inv = amax > 0.f ? 256.0f / amax : 0.f;
    rsval = amax * (1.0f / 256.0f) * sm_scale_log2;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      u32 pk[4] = {0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        float x = qs[s][j] * inv;
        u32 code = 0;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const u32 c = (u32)__builtin_amdgcn_cvt_pk_fp8_f32(x, x, 0, false) & 0xffu;
          if (t == limb) code = c;
          x -= __builtin_amdgcn_cvt_f32_fp8((int)c, 0);
        }
        pk[j >> 2] |= code << (8 * (j & 3));
      }
      st.aq[s] = (v4i){(int)pk[0], (int)pk[1], (int)pk[2], (int)pk[3]};
    }
  }
  // lane 4*head' (g = 0, limb 0) knows head'’s scale; the S layout wants head = lane / 16
  st.rs = __shfl(rsval, 4 * (lane >> 4), 64);
  st.m = -INFINITY;
  st.l = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) st.o[i] = 0.f;
}

template <int QUANT>
__device__ __forceinline__ void load_pair(const uint16_t* q, const float* k_scale, int hkv, float sm_scale_log2, int p, int row,
                                          int lane, PairState& st) {
  load_pair_finish<QUANT>(load_pair_issue(q, k_scale, hkv, p, row, lane), sm_scale_log2, lane, st);
}

}  // namespace fdattn
