// Chunked-prefill ("append") attention on the bf16 MFMA units, head_dim 128, block_size 64.
//
// One workgroup = 128 new tokens of one query head (4 wavefronts x 32 tokens); it walks
// the keys in tiles of 64: first the cached prefix, one cache block per tile (int8 / fp8
// bytes converted to bf16 once per workgroup while they are staged into LDS - "dequantised
// in-tile"), then the chunk's own bf16 K/V up to the causal diagonal.
//
// Number formats: cache bytes (int8, e4m3) are exact in fp16, so the prefix tiles run on
// v_mfma_f32_32x32x16_f16 with Q*k_scale rounded to fp16 (11 significant bits); the chunk's
// own K stays bf16 and meets the bf16 Q on v_mfma_f32_32x32x16_bf16 (exact inputs).  The
// softmax weights and V always go through fp16 (V of the chunk is converted, saturating at
// +-65504): bf16 weights (8 bits) would not hold the 2e-3 / 1e-2 output tolerance on rows
// with few keys.
//
// The scores are computed transposed, S^T = K Q^T: in the
// result layout a lane owns one query and 16 of every 32 keys, so the softmax row
// reductions are in-lane plus one exchange with lane^32, and P^T is already laid out as
// the B operand of the second product O^T = V^T P^T - no trip through LDS.  V^T operands
// come transposed out of LDS by ds_read_b64_tr_b16.  The per-channel K scale is folded
// into Q for the prefix tiles; the V scale is applied to the accumulator once, when the
// walk passes from the prefix to the chunk.  K/V tiles are double-buffered in LDS with
// the next tile's global loads in flight during the current tile's MFMAs; one barrier
// per tile.
#include "prefill.h"

namespace fdattn {

namespace {

constexpr int BM = 128, BN = 64, HD = 128;
constexpr int LDK = 136;  // bf16 elements per LDS row (272 B: 16-byte aligned, off the 256 B bank period)
constexpr int TILE_ELEMS = BN * LDK;

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef short v8s __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

__device__ __forceinline__ u32 pack_bf16(float lo, float hi) {
  return (u32)f32_to_bf16(lo) | ((u32)f32_to_bf16(hi) << 16);
}
// two floats -> packed fp16, round to nearest even
__device__ __forceinline__ u32 pack_f16(float lo, float hi) {
  const v2h v = {(_Float16)lo, (_Float16)hi};
  return __builtin_bit_cast(u32, v);
}
// two floats -> packed fp16 in one instruction (round toward zero): exact for cache values
// (integers up to 127, e4m3 values), a 2^-11 downward nudge for softmax weights
__device__ __forceinline__ u32 pack_f16_fast(float lo, float hi) {
  return __builtin_bit_cast(u32, __builtin_amdgcn_cvt_pkrtz(lo, hi));
}
__device__ __forceinline__ float sat_f16(float x) { return fminf(fmaxf(x, -65504.0f), 65504.0f); }

template <int QUANT>
__device__ __forceinline__ float cvt8(u32 byte) {
  if (QUANT == FDATTN_CACHE_INT8) return (float)(int)(int8_t)byte;
  return __builtin_amdgcn_cvt_f32_fp8((int)byte, 0);
}

// 16 cache bytes -> 16 fp16 (two 16-byte LDS stores)
template <int QUANT>
__device__ __forceinline__ void cvt16_store(uint4 w, uint16_t* dst) {
  const u32 ws[4] = {w.x, w.y, w.z, w.w};
  u32 o[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    o[2 * i] = pack_f16_fast(cvt8<QUANT>(ws[i] & 0xff), cvt8<QUANT>((ws[i] >> 8) & 0xff));
    o[2 * i + 1] = pack_f16_fast(cvt8<QUANT>((ws[i] >> 16) & 0xff), cvt8<QUANT>(ws[i] >> 24));
  }
  *reinterpret_cast<uint4*>(dst) = make_uint4(o[0], o[1], o[2], o[3]);
  *reinterpret_cast<uint4*>(dst + 8) = make_uint4(o[4], o[5], o[6], o[7]);
}

struct Stage {  // one thread's share of a K tile and a V tile on its way to LDS
  uint4 k[4], v[4];
};

}  // namespace

template <int QUANT>
__global__ __launch_bounds__(256, 2) void prefill_mfma_kernel(PrefillArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];  // [2 buffers][K tile, V tile][64][LDK] 16-bit
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int b = blockIdx.z, qh = blockIdx.y, h = qh / (a.hq / a.hkv);
  const int tok0 = a.cu_seqlens_q[b], n_b = a.cu_seqlens_q[b + 1] - tok0, p = a.seq_lens_decoder[b];
  const int qt = (int)gridDim.x - 1 - (int)blockIdx.x;  // long rows (late tokens) first
  const int q0 = qt * BM;
  if (q0 >= n_b) return;

  const int j32 = lane & 31, hf = lane >> 5;
  // this lane's query; rows past the chunk behave like its last row and are not stored
  const int ci_raw = q0 + 32 * wv + j32;
  const int ci = min(ci_raw, n_b - 1);
  const bool wave_active = q0 + 32 * wv < n_b;
  const int ci_wave_max = min(q0 + 32 * wv + 31, n_b - 1);

  const int n_pre = (p + BN - 1) / BN;
  const int n_chk = (min(n_b, q0 + BM) + BN - 1) / BN;
  const int n_tiles = n_pre + n_chk;
  const int32_t* table = a.block_tables + (size_t)b * a.max_blocks;

  // ---- Q as the B operand: lane = query, 8 channels per k-step
  const uint16_t* qrow = a.q + ((size_t)(tok0 + ci) * a.hq + qh) * HD;
  uint4 qf[8];  // fp16 (q * k_scale) while the prefix is walked, bf16 q for the chunk
  auto load_q = [&](bool scaled) {
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int c0 = 16 * s + 8 * hf;
      uint4 w = *reinterpret_cast<const uint4*>(qrow + c0);
      if (scaled) {
        const float4 s0 = *reinterpret_cast<const float4*>(a.k_scale + h * HD + c0);
        const float4 s1 = *reinterpret_cast<const float4*>(a.k_scale + h * HD + c0 + 4);
        w.x = pack_f16(bf16lo_to_f32(w.x) * s0.x, bf16hi_to_f32(w.x) * s0.y);
        w.y = pack_f16(bf16lo_to_f32(w.y) * s0.z, bf16hi_to_f32(w.y) * s0.w);
        w.z = pack_f16(bf16lo_to_f32(w.z) * s1.x, bf16hi_to_f32(w.z) * s1.y);
        w.w = pack_f16(bf16lo_to_f32(w.w) * s1.z, bf16hi_to_f32(w.w) * s1.w);
      }
      qf[s] = w;
    }
  };

  // ---- staging: thread tid moves key tid/4, channels 32*(tid%4) .. +31 of a tile
  const int skey = tid >> 2, sc0 = (tid & 3) * 32;
  Stage stg;
  auto fetch = [&](int t) {
    if (t < n_pre) {
      int pb = table[t];
      pb = (pb >= 0 && pb < a.num_blocks) ? pb : 0;
      const size_t off = (((size_t)pb * a.hkv + h) * BN + skey) * HD + sc0;
      stg.k[0] = *reinterpret_cast<const uint4*>(a.key_cache + off);
      stg.k[1] = *reinterpret_cast<const uint4*>(a.key_cache + off + 16);
      stg.v[0] = *reinterpret_cast<const uint4*>(a.value_cache + off);
      stg.v[1] = *reinterpret_cast<const uint4*>(a.value_cache + off + 16);
    } else {
      const int j = min((t - n_pre) * BN + skey, n_b - 1);  // keys past the chunk are masked later
      const size_t off = ((size_t)(tok0 + j) * a.hkv + h) * HD + sc0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        stg.k[i] = *reinterpret_cast<const uint4*>(a.k_new + off + 8 * i);
        stg.v[i] = *reinterpret_cast<const uint4*>(a.v_new + off + 8 * i);
      }
    }
  };
  auto commit = [&](int t, int buf) {
    uint16_t* kd = lds + (size_t)buf * 2 * TILE_ELEMS + skey * LDK + sc0;
    uint16_t* vd = kd + TILE_ELEMS;
    if (t < n_pre) {
      if (t * BN + skey >= p) {
        // rows past the cached prefix hold stale bytes (fp8 has NaN codes, and 0 * NaN would
        // poison the second product): stage zeros for them
        stg.k[0] = stg.k[1] = stg.v[0] = stg.v[1] = make_uint4(0, 0, 0, 0);
      }
      cvt16_store<QUANT>(stg.k[0], kd);
      cvt16_store<QUANT>(stg.k[1], kd + 16);
      cvt16_store<QUANT>(stg.v[0], vd);
      cvt16_store<QUANT>(stg.v[1], vd + 16);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        *reinterpret_cast<uint4*>(kd + 8 * i) = stg.k[i];
        const u32 vw[4] = {stg.v[i].x, stg.v[i].y, stg.v[i].z, stg.v[i].w};
        u32 hw[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) hw[e] = pack_f16(sat_f16(bf16lo_to_f32(vw[e])), sat_f16(bf16hi_to_f32(vw[e])));
        *reinterpret_cast<uint4*>(vd + 8 * i) = make_uint4(hw[0], hw[1], hw[2], hw[3]);
      }
    }
  };

  v16f o[4];  // O^T: rows = channels 32*ct + (r%4) + 8*(r/4) + 4*hf, column = this lane's query
#pragma unroll
  for (int ct = 0; ct < 4; ++ct)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[ct][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const float sc = a.sm_scale * 1.4426950408889634f;  // logits go to the log2 domain

  load_q(n_pre > 0);
  fetch(0);
  for (int t = 0; t < n_tiles; ++t) {
    const int buf = t & 1;
    commit(t, buf);
    __syncthreads();
    if (t + 1 < n_tiles) fetch(t + 1);
    if (t == n_pre && n_pre > 0) {
      // leaving the quantised prefix: o holds sums over int8/fp8 values, give them their scale
      load_q(false);
#pragma unroll
      for (int ct = 0; ct < 4; ++ct)
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) {
          const float4 vs = *reinterpret_cast<const float4*>(a.v_scale + h * HD + 32 * ct + 8 * rb + 4 * hf);
          o[ct][4 * rb + 0] *= vs.x;
          o[ct][4 * rb + 1] *= vs.y;
          o[ct][4 * rb + 2] *= vs.z;
          o[ct][4 * rb + 3] *= vs.w;
        }
    }
    const bool is_pre = t < n_pre;
    const int key0 = is_pre ? t * BN : (t - n_pre) * BN;  // index of the tile's first key in its segment
    // a chunk tile wholly above this wavefront's diagonal contributes nothing
    const bool skip = !wave_active || (!is_pre && key0 > ci_wave_max);
    if (!skip) {
      const uint16_t* kt = lds + (size_t)buf * 2 * TILE_ELEMS;
      const uint16_t* vt = kt + TILE_ELEMS;
      // ---- S^T = K Q^T
      v16f st[2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        v16f acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
          const uint4 w = *reinterpret_cast<const uint4*>(kt + (32 * kb + j32) * LDK + 16 * s + 8 * hf);
          if (is_pre)
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, w), __builtin_bit_cast(v8h, qf[s]), acc, 0, 0, 0);
          else
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, w), __builtin_bit_cast(v8bf, qf[s]), acc, 0, 0, 0);
        }
        st[kb] = acc;
      }
      // ---- mask + online softmax; this lane: one query, keys 32kb + (r%4) + 8(r/4) + 4hf
      const int limit = is_pre ? p - key0 : ci - key0 + 1;  // keys [0, limit) of the tile are visible
      const bool need_mask = is_pre ? (key0 + BN > p) : (key0 + BN > q0 + 32 * wv + 1);
      float mx = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float s = st[kb][r] * sc;
          if (need_mask) {
            const int key = 32 * kb + (r & 3) + 8 * (r >> 2) + 4 * hf;
            s = key < limit ? s : -INFINITY;
          }
          st[kb][r] = s;
          mx = fmaxf(mx, s);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run, mx);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
      m_run = m_new;
      float psum = 0.f;
      v8h pf[2][2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int ss = 0; ss < 2; ++ss) {
          u32 w[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float p0 = __builtin_amdgcn_exp2f(st[kb][8 * ss + 2 * e] - m_use);
            const float p1 = __builtin_amdgcn_exp2f(st[kb][8 * ss + 2 * e + 1] - m_use);
            psum += p0 + p1;
            w[e] = pack_f16_fast(p0, p1);
          }
          pf[kb][ss] = __builtin_bit_cast(v8h, make_uint4(w[0], w[1], w[2], w[3]));
        }
      l_run = l_run * alpha + psum;
      // ---- O^T = O^T * alpha + V^T P^T
      const int q16 = lane >> 4, i16 = lane & 15;
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
#pragma unroll
        for (int r = 0; r < 16; ++r) o[ct][r] *= alpha;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int ss = 0; ss < 2; ++ss) {
            // k-slot e of lane group hf is key 32kb + 16ss + 8(e/4) + 4hf + e%4 (the P^T layout);
            // lane i16 supplies the row (key kbase + i16/4, channels cbase + 4(i16%4)..+3)
            const int kbase = 32 * kb + 16 * ss + 4 * hf + (i16 >> 2);
            const int cbase = 32 * ct + 16 * (q16 & 1) + 4 * (i16 & 3);
            const uint16_t* src = vt + kbase * LDK + cbase;
            const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)src);
            const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)(src + 8 * LDK));
            const v8s vv = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            o[ct] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, vv), pf[kb][ss], o[ct], 0, 0, 0);
          }
      }
    }
  }

  // ---- epilogue: normalise and store bf16 (every query saw at least its own chunk tile)
  if (!wave_active || ci_raw >= n_b) return;
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  uint16_t* orow = a.out + ((size_t)(tok0 + ci) * a.hq + qh) * HD;
#pragma unroll
  for (int ct = 0; ct < 4; ++ct)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      const int c = 32 * ct + 8 * rb + 4 * hf;
      const u32 w0 = pack_bf16(o[ct][4 * rb] * inv, o[ct][4 * rb + 1] * inv);
      const u32 w1 = pack_bf16(o[ct][4 * rb + 2] * inv, o[ct][4 * rb + 3] * inv);
      *reinterpret_cast<uint2*>(orow + c) = make_uint2(w0, w1);
    }
}

bool prefill_mfma_supported(int hq, int hkv, int d, int bs, int quant) {
  return d == HD && bs == BN && hq % hkv == 0 &&
         (quant == FDATTN_CACHE_INT8 || quant == FDATTN_CACHE_FP8_E4M3);
}

int prefill_mfma_launch(const PrefillArgs& a, int max_chunk, int quant, hipStream_t s) {
  const dim3 grid((max_chunk + BM - 1) / BM, a.hq, a.batch), block(256);
  const size_t shm = (size_t)2 * 2 * TILE_ELEMS * sizeof(uint16_t);  // 69,632 B
  if (a.batch > 65535 || a.hq > 65535)
    return fail(FDATTN_ERR_SHAPE, "fdattn_append_attention_prefill: batch or head count exceeds the grid limit");
  static bool attr_set[2] = {false, false};
  hipError_t e = hipSuccess;
  if (quant == FDATTN_CACHE_INT8) {
    if (!attr_set[0]) {
      e = hipFuncSetAttribute((const void*)prefill_mfma_kernel<FDATTN_CACHE_INT8>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm);
      attr_set[0] = e == hipSuccess;
    }
    if (e == hipSuccess) hipLaunchKernelGGL(prefill_mfma_kernel<FDATTN_CACHE_INT8>, grid, block, shm, s, a);
  } else {
    if (!attr_set[1]) {
      e = hipFuncSetAttribute((const void*)prefill_mfma_kernel<FDATTN_CACHE_FP8_E4M3>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm);
      attr_set[1] = e == hipSuccess;
    }
    if (e == hipSuccess) hipLaunchKernelGGL(prefill_mfma_kernel<FDATTN_CACHE_FP8_E4M3>, grid, block, shm, s, a);
  }
  if (e != hipSuccess) return fail((int)e, "fdattn_append_attention_prefill: %s", hipGetErrorString(e));
  return check_launch("fdattn_append_attention_prefill (mfma)");
}

}  // namespace fdattn
