// Chunked-prefill ("append") attention on the MFMA units, head_dim 128, block_size 64.
//
// One workgroup = NW wavefronts x 32 new tokens of one query head (NW = 8 -> 256 tokens, or
// 4 -> 128 for short chunks); it walks the keys in tiles of 64: first the cached prefix, one
// cache block per tile (int8 / fp8 bytes turned into fp16 once per workgroup while they are
// staged into LDS - "dequantised in-tile"), then the chunk's own bf16 K/V up to the causal
// diagonal.
//
// Number formats.  The prefix tiles run on v_mfma_f32_32x32x16_f16.  An int8 byte b becomes
// the fp16 SUBNORMAL with mantissa b ^ 0x80, i.e. the value 2^-24 (b + 128): one xor per four
// bytes and one byte permute per two, no int->float conversion.  The MFMA treats fp16
// subnormals exactly, so the products are exact; the factor 2^24 goes into the softmax scale
// and the offset 128 drops out algebraically:
//   scores:  sum_c q_c 2^-24 (k_c + 128)  =  2^-24 (q.k + 128 sum_c q_c)  - the second term is a
//            per-query constant, folded into the exponent's additive constant;
//   output:  sum_j p_j 2^-24 (v_j + 128)  =  2^-24 (sum_j p_j v_j + 128 l),  l = sum_j p_j -
//            removed once, when the walk leaves the prefix, with l summed from the same
//            fp16-rounded weights the MFMA multiplied (v_dot2_f32_f16).
// e4m3 bytes are converted by v_cvt_pk_f32_fp8 (exact in fp16).  Q * k_scale is rounded to
// fp16 (11 significant bits).  The chunk's own K stays bf16 and meets the bf16 Q on
// v_mfma_f32_32x32x16_bf16 (exact inputs).  The softmax weights and V always go through fp16
// (V of the chunk is converted, saturating at +-65504): bf16 weights (8 bits) would not hold
// the 2e-3 / 1e-2 output tolerance on rows with few keys.
//
// The scores are computed transposed, S^T = K Q^T: in the result layout a lane owns one query
// and 16 of every 32 keys, so the softmax row reductions are in-lane plus one exchange with
// lane^32, and P^T is already laid out as the B operand of the second product
// O^T = V^T P^T - no trip through LDS.  V^T operands come transposed out of LDS by
// ds_read_b64_tr_b16.  The exponent reference of a query is raised only when its weight sum
// over a tile exceeds 1024 (every weight then stays far inside fp16): the tile's maximum is
// not even computed on the other tiles, and the accumulator is rescaled on a handful of them.
// The per-channel K scale is folded into Q for the prefix tiles; the V scale is applied to the
// accumulator once, when the walk passes from the prefix to the chunk.  The formats with one
// scale per stored row (DYN) are dequantised while they are staged instead: the staged fp16
// number is byte x row scale, Q stays unscaled and nothing is left to apply at the end.
//
// Schedule.  The wavefronts form two groups that alternate between a matrix phase (the two
// MFMA streams of a tile, hand-scheduled: LDS operand reads six deep in flight, exact
// s_waitcnt counts) and a vector phase (staging of a later tile, then the softmax), half a
// tile out of step with each other, so that the MFMA units and the vector ALU of a SIMD are
// fed by different wavefronts at the same time.  Three K/V tiles are resident in LDS; the
// global loads of a tile are issued a whole tile before its bytes are converted.
//
// LDS rows: K 272 B apart (the 32 rows a ds_read_b128 touches fall on distinct banks), V
// 320 B apart (the 4 rows x 64 B a ds_read_b64_tr_b16 half-wave touches fall on distinct
// banks); both tiles are written as whole 256 B rows by 16 consecutive lanes.
#include <atomic>

#include "prefill.h"
#include "launch.h"

namespace fdattn {

namespace {

constexpr int BN = 64, HD = 128;
constexpr int LDK = 136;  // 16-bit elements per K row in LDS (272 B)
constexpr int LDV = 160;  // 16-bit elements per V row in LDS (320 B)
constexpr int K_ELEMS = BN * LDK, BUF_ELEMS = BN * (LDK + LDV);
constexpr int kSlots = 4;  // K/V tile slots in LDS (three are live at a time; four make the slot of a tile a mask)
constexpr int kMaxSplits = 8;  // workgroups that may share one query tile's keys
constexpr float kSumLimit = 1024.0f;  // a query's weight sum over one tile above which its exponent reference is raised

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef short v8s __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));

// how a cache byte sits in fp16: value = kMul^-1 (byte value + kOff).  DYN (one scale per stored row): the staged
// fp16 number is the dequantised value itself, byte x scale of its row.
template <int QUANT, bool DYN>
struct ByteFmt {
  static constexpr float kMul = (QUANT == FDATTN_CACHE_INT8 && !DYN) ? 16777216.0f : 1.0f;
  static constexpr float kOff = (QUANT == FDATTN_CACHE_INT8 && !DYN) ? 128.0f : 0.0f;
};

__device__ __forceinline__ u32 pack_bf16(float lo, float hi) {
  return (u32)f32_to_bf16(lo) | ((u32)f32_to_bf16(hi) << 16);
}
// two floats -> packed fp16, round to nearest even
__device__ __forceinline__ u32 pack_f16(float lo, float hi) {
  const v2h v = {(_Float16)lo, (_Float16)hi};
  return __builtin_bit_cast(u32, v);
}
// two floats -> packed fp16, round toward zero: exact for e4m3 values
__device__ __forceinline__ u32 pack_f16_fast(float lo, float hi) {
  return __builtin_bit_cast(u32, __builtin_amdgcn_cvt_pkrtz(lo, hi));
}
__device__ __forceinline__ float sat_f16(float x) { return __builtin_amdgcn_fmed3f(x, -65504.0f, 65504.0f); }

// 8 cache bytes -> 8 fp16
template <int QUANT>
__device__ __forceinline__ uint4 cvt8(u32 w0, u32 w1) {
  if (QUANT == FDATTN_CACHE_INT8) {
    const u32 x0 = w0 ^ 0x80808080u, x1 = w1 ^ 0x80808080u;
    return make_uint4(__builtin_amdgcn_perm(0u, x0, 0x0c010c00u), __builtin_amdgcn_perm(0u, x0, 0x0c030c02u),
                      __builtin_amdgcn_perm(0u, x1, 0x0c010c00u), __builtin_amdgcn_perm(0u, x1, 0x0c030c02u));
  }
  const v2f a = __builtin_amdgcn_cvt_pk_f32_fp8((int)w0, false), b = __builtin_amdgcn_cvt_pk_f32_fp8((int)w0, true);
  const v2f c = __builtin_amdgcn_cvt_pk_f32_fp8((int)w1, false), d = __builtin_amdgcn_cvt_pk_f32_fp8((int)w1, true);
  return make_uint4(pack_f16_fast(a[0], a[1]), pack_f16_fast(b[0], b[1]), pack_f16_fast(c[0], c[1]),
                    pack_f16_fast(d[0], d[1]));
}

// 8 cache bytes of one stored row -> 8 fp16 dequantised values, byte x s, each rounded to nearest once
template <int QUANT>
__device__ __forceinline__ uint4 cvt8_scaled(u32 w0, u32 w1, float s) {
  float f[8];
  if (QUANT == FDATTN_CACHE_INT8) {
    // byte b -> the fp16 number 1024 + (b + 128) (exponent byte 0x64 in front of the offset byte: one permute per two
    // bytes), then (1024 + b + 128) s - 1152 s = b s as one fused multiply-add in fp32, rounded to fp16 once
    // (the mixed-precision fma takes the fp16 operand and writes the fp16 result directly)
    const u32 x[2] = {w0 ^ 0x80808080u, w1 ^ 0x80808080u};
    const float c = -1152.0f * s;
    u32 out[4];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const v2h lo = __builtin_bit_cast(v2h, __builtin_amdgcn_perm(0x64646464u, x[i], 0x04010400u));
      const v2h hi = __builtin_bit_cast(v2h, __builtin_amdgcn_perm(0x64646464u, x[i], 0x04030402u));
      const v2h rl = {(_Float16)__builtin_fmaf((float)lo[0], s, c), (_Float16)__builtin_fmaf((float)lo[1], s, c)};
      const v2h rh = {(_Float16)__builtin_fmaf((float)hi[0], s, c), (_Float16)__builtin_fmaf((float)hi[1], s, c)};
      out[2 * i] = __builtin_bit_cast(u32, rl);
      out[2 * i + 1] = __builtin_bit_cast(u32, rh);
    }
    return make_uint4(out[0], out[1], out[2], out[3]);
  } else {
    const v2f a = __builtin_amdgcn_cvt_pk_f32_fp8((int)w0, false), b = __builtin_amdgcn_cvt_pk_f32_fp8((int)w0, true);
    const v2f c = __builtin_amdgcn_cvt_pk_f32_fp8((int)w1, false), d = __builtin_amdgcn_cvt_pk_f32_fp8((int)w1, true);
    f[0] = a[0] * s; f[1] = a[1] * s; f[2] = b[0] * s; f[3] = b[1] * s;
    f[4] = c[0] * s; f[5] = c[1] * s; f[6] = d[0] * s; f[7] = d[1] * s;
  }
  return make_uint4(pack_f16(f[0], f[1]), pack_f16(f[2], f[3]), pack_f16(f[4], f[5]), pack_f16(f[6], f[7]));
}

// ---- the matrix phase, hand-scheduled (generated by gen_prefill_sched.py).  Operands stream
// from LDS through six 4-register buffers: up to twelve reads are in flight while an MFMA
// runs, a buffer is refilled right after the MFMA that consumed it has issued, and every
// wait names exactly the reads that may still be outstanding.  The blocks open with
// lgkmcnt(0) so that nothing else (a scalar load returns out of order) disturbs the count.
typedef u32 u4v __attribute__((ext_vector_type(4)));
typedef u32 u2v __attribute__((ext_vector_type(2)));
#include "prefill_mfma_sched.inc"

// the value held by lane ^ 32
__device__ __forceinline__ float swap32(float x) {
  typedef u32 u2v __attribute__((ext_vector_type(2)));
  const u2v r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(threadIdx.x & 32 ? r[0] : r[1]);
}
__device__ __forceinline__ void lds_store16(u32 addr, uint4 v) {
  const u4v w = {v.x, v.y, v.z, v.w};
  *(__attribute__((address_space(3))) u4v*)(uintptr_t)addr = w;
}
__device__ __forceinline__ u32 lds_addr(const void* p) {
  return (u32)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}

}  // namespace

// The sequence a grid row stands for.  A grid over the whole batch: the row itself.  A grid over the prefill rows
// only (the host said how many there are): the r-th sequence with seq_lens_encoder > 0, found by every wavefront
// with ballots over the batch; -1 if there are fewer.
__device__ __forceinline__ int sequence_of_row(const PrefillArgs& a, int r) {
  if (a.rows >= a.batch || !a.seq_lens_encoder) return r;
  const int lane = threadIdx.x & 63;
  int seen = 0;
  for (int base = 0; base < a.batch; base += 64) {
    const int idx = base + lane;
    const unsigned long long m = __ballot(idx < a.batch && a.seq_lens_encoder[idx] > 0);
    const int c = __popcll(m);
    if (r < seen + c) {
      unsigned long long mm = m;
      for (int k = seen; k < r; ++k) mm &= mm - 1;  // drop the set bits before the wanted one
      return base + __ffsll((long long)mm) - 1;
    }
    seen += c;
  }
  return -1;
}

// how many of the launch's max_splits key splits a walk of n_tiles tiles uses
__device__ __forceinline__ int splits_of(int n_tiles, int max_splits) { return min(max(n_tiles / 16, 1), max_splits); }

template <int QUANT, int NW, bool DYN>
__global__ __launch_bounds__(64 * NW) void prefill_mfma_kernel(PrefillArgs a) {
  constexpr int BM = 32 * NW;       // queries per workgroup
  constexpr int PASSES = 16 / NW;   // 16-byte LDS chunks a thread stages per tile and tensor
  constexpr int ROWS = 2 * NW;      // tile rows covered by one staging pass of one wavefront group
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];  // [kSlots][K tile | V tile]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);  // in a scalar register: what depends on it stays uniform
  // Workgroup -> (sequence, query head, query tile).  The hardware deals workgroups to the 8 XCDs in
  // turn (workgroup i to XCD i % 8), each with its own L2.  So: the XCD index picks the (sequence, KV
  // head) pair - every workgroup that reads one pair's K and V shares one L2 - and inside an XCD the
  // query tiles come longest first (the causal rows of late tokens walk more keys), so every XCD gets
  // the same mix of long and short workgroups and the short ones fill the end of the launch.
  const int G = a.hq / a.hkv, pairs = a.rows * a.hkv, units = a.rows * a.hq;
  const bool pack = a.pack_slot > 0;  // short chunks: the workgroup holds every query head of its KV head
  // When a tile's global loads are issued: at the start of the matrix phase before the vector phase that stores them
  // (one phase in flight; the long walks of a large launch are bound by the vector phase's issue time and lose 3-6 %
  // to anything added to it), or a phase earlier, straight after the previous store (a whole tile period in flight:
  // 10 % faster where the walks are short and few, i.e. latency-bound - the packed short-chunk mode).
  const bool early = pack;
  int qt, b, qh;  // b: the grid row first, the sequence below; qh: the (first) query head
  if (pack) {
    qt = 0;
    b = blockIdx.x / a.hkv;
    qh = (blockIdx.x - b * a.hkv) * G;
  } else if ((pairs & 7) == 0) {
    const int ppx = pairs >> 3;  // pairs per XCD
    const int x = blockIdx.x & 7, jx = blockIdx.x >> 3;
    const int r = jx % (ppx * G), pk = (r / G) * 8 + x;
    qt = a.q_tiles - 1 - jx / (ppx * G);
    b = pk / a.hkv;
    qh = (pk - b * a.hkv) * G + r % G;
  } else {  // no whole number of pairs per XCD: query heads in turn, still longest tiles first
    const int u = blockIdx.x % units;
    qt = a.q_tiles - 1 - blockIdx.x / units;
    b = u / a.hq;
    qh = u - b * a.hq;
  }
  const int h = qh / G;
  b = sequence_of_row(a, b);
  if (b < 0) return;
  const int tok0 = a.cu_seqlens_q[b], n_b = a.cu_seqlens_q[b + 1] - tok0, p = a.seq_lens_decoder[b];
  const int q0 = qt * BM;
  if (q0 >= n_b) return;
  if (a.seq_lens_encoder && a.seq_lens_encoder[b] <= 0) return;  // a decode row or an idle slot of a mixed batch

  const int j32 = lane & 31, hf = lane >> 5;
  // this lane's query; rows past the chunk behave like its last row and are not stored
  int ci_raw = q0 + 32 * wv + j32;
  int qh_lane = qh;  // packed: query column x = 32 wv + j32 is head x / slot of the group, token x % slot
  if (pack) {
    const int x = 32 * wv + j32, hg = x / a.pack_slot;
    ci_raw = hg < G ? x - hg * a.pack_slot : n_b;
    qh_lane = qh + min(hg, G - 1);
  }
  const int ci = min(ci_raw, n_b - 1);
  const bool wave_active = pack ? __ballot(ci_raw < n_b) != 0ull : q0 + 32 * wv < n_b;
  const int ci_wave_max = pack ? n_b - 1 : min(q0 + 32 * wv + 31, n_b - 1);

  const int n_pre = (p + BN - 1) / BN;
  const int n_chk = (min(n_b, pack ? a.pack_slot : q0 + BM) + BN - 1) / BN;
  const int n_tiles = n_pre + n_chk;
  // this workgroup's share of the key tiles: [t0, t1).  A share is worth its fixed costs (prologue, partial,
  // merge) from about 16 tiles on: shorter walks are split less, or not at all - then split 0 walks everything
  // and writes the final rows itself.
  const int n_splits = splits_of(n_tiles, a.n_splits);
  if ((int)blockIdx.y >= n_splits) return;
  const int per = (n_tiles + n_splits - 1) / n_splits;
  const int t0 = (int)blockIdx.y * per, t1 = min(t0 + per, n_tiles);
  if (t0 >= t1) {  // nothing to walk (only with splits): an empty partial for each of the tile's queries
    for (int i = tid; i < BM; i += 64 * NW) {
      const int hg = pack ? i / a.pack_slot : 0, tk = pack ? i - hg * a.pack_slot : q0 + i;
      if (hg < G && tk < n_b) {
        float* ml = a.part_ml + (((size_t)blockIdx.y * a.num_tokens + tok0 + tk) * a.hq + qh + hg) * 2;
        ml[0] = -INFINITY;
        ml[1] = 0.f;
      }
    }
    return;
  }
  const int32_t* table = a.block_tables + (size_t)b * a.max_blocks;
  const float sc = a.sm_scale * 1.4426950408889634f;  // logits go to the log2 domain

  // ---- Q as the B operand: lane = query, 8 channels per k-step
  const uint16_t* qrow = a.q + ((size_t)(tok0 + ci) * a.hq + qh_lane) * HD;
  uint4 qf[8];       // fp16 (q * k_scale) while the prefix is walked, bf16 q for the chunk
  float qsum = 0.f;  // sum over this lane's 64 channels of the rounded q * k_scale
  auto load_q = [&](bool scaled) {
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int c0 = 16 * s + 8 * hf;
      uint4 w = *reinterpret_cast<const uint4*>(qrow + c0);
      if (scaled) {
        // DYN: the K scales sit in the staged tile, q goes to fp16 as it is
        const float4 one = make_float4(1.f, 1.f, 1.f, 1.f);
        const float4 s0 = DYN ? one : *reinterpret_cast<const float4*>(a.k_scale + h * HD + c0);
        const float4 s1 = DYN ? one : *reinterpret_cast<const float4*>(a.k_scale + h * HD + c0 + 4);
        const v2h h0 = {(_Float16)(bf16lo_to_f32(w.x) * s0.x), (_Float16)(bf16hi_to_f32(w.x) * s0.y)};
        const v2h h1 = {(_Float16)(bf16lo_to_f32(w.y) * s0.z), (_Float16)(bf16hi_to_f32(w.y) * s0.w)};
        const v2h h2 = {(_Float16)(bf16lo_to_f32(w.z) * s1.x), (_Float16)(bf16hi_to_f32(w.z) * s1.y)};
        const v2h h3 = {(_Float16)(bf16lo_to_f32(w.w) * s1.z), (_Float16)(bf16hi_to_f32(w.w) * s1.w)};
        qsum += ((float)h0[0] + (float)h0[1]) + ((float)h1[0] + (float)h1[1]) + ((float)h2[0] + (float)h2[1]) +
                ((float)h3[0] + (float)h3[1]);
        w = make_uint4(__builtin_bit_cast(u32, h0), __builtin_bit_cast(u32, h1), __builtin_bit_cast(u32, h2),
                       __builtin_bit_cast(u32, h3));
      }
      qf[s] = w;
    }
  };

  // ---- the two wavefront groups.  Group 0 (the first NW/2 wavefronts) and group 1 run the
  // same per-tile sequence  [matrix phase: O += V P of the previous tile, S = K Q of this
  // tile]  barrier  [vector phase: staging, softmax of this tile]  barrier,  but group 1
  // starts one barrier late: while one group keeps the MFMA units busy the other one keeps
  // the vector ALU busy (wavefronts w and w + NW/2 share a SIMD).  Tile u lives in LDS slot
  // u % 4: group 0 writes its rows in its vector phase of tile u-1 and group 1 in its vector
  // phase of tile u-2 (both end before group 0's matrix phase of tile u starts); K is read in
  // the matrix phases of tile u and V in those of tile u+1.
  const int grp = wv / (NW / 2);
  const int gtid = tid - grp * 32 * NW;
  const int lead = 1 + grp;  // in the vector phase of tile t a group stages its rows of tile t + lead
  // ---- staging: a group's 32*NW threads move rows 32*grp .. 32*grp+31 of a tile, one
  // 16-byte LDS chunk (8 channels) per thread and pass
  const int srow = 32 * grp + (gtid >> 4), scc = (gtid & 15) * 8;
  const u32 goff = (u32)(srow * HD + scc);  // this thread's byte offset inside a cache block
  // LDS byte addresses of its K and V chunk of pass 0 in slot 0
  const u32 kw0 = lds_addr(lds + srow * LDK + scc), vw0 = lds_addr(lds + K_ELEMS + srow * LDV + scc);
  uint4 stg_k[PASSES], stg_v[PASSES];
  float stg_ks[DYN ? PASSES : 1], stg_vs[DYN ? PASSES : 1];  // DYN: the scales of the fetched rows
  // The physical block of the next prefix tile to fetch is requested one fetch ahead and kept
  // in a vector register until it is needed (vzero hides from the compiler that the index is
  // uniform: it would otherwise move the value to a scalar register - and wait for the load -
  // straight away).
  int vzero;
  asm("v_mov_b32 %0, 0" : "=v"(vzero));
  int pb_next = t0 < n_pre ? table[t0 + vzero] : 0;
  auto fetch = [&](int t) {
    if (t >= t1) return;
    if (t < n_pre) {
      // the block id was requested one fetch earlier: its scalar load has long returned
      const int pb_u = __builtin_amdgcn_readfirstlane(pb_next);
      const int pb = (pb_u >= 0 && pb_u < a.num_blocks) ? pb_u : 0;
      pb_next = table[min(t + 1, n_pre - 1) + vzero];  // every group fetches its tiles in order 0, 1, 2, ...
      // a scalar block base plus this thread's fixed 32-bit offset: no per-tile vector arithmetic
      const size_t blk = ((size_t)pb * a.hkv + h) * (BN * HD);
      const uint8_t* kb = a.key_cache + blk;
      const uint8_t* vb = a.value_cache + blk;
#pragma unroll
      for (int i = 0; i < PASSES; ++i) {
        const uint2 kk = *reinterpret_cast<const uint2*>(kb + (goff + (u32)(i * ROWS * HD)));
        const uint2 vv = *reinterpret_cast<const uint2*>(vb + (goff + (u32)(i * ROWS * HD)));
        stg_k[i].x = kk.x, stg_k[i].y = kk.y, stg_v[i].x = vv.x, stg_v[i].y = vv.y;
      }
      if (DYN) {
        const size_t srow0 = ((size_t)pb * a.hkv + h) * BN + srow;
#pragma unroll
        for (int i = 0; i < PASSES; ++i) {
          stg_ks[i] = a.k_scale[srow0 + i * ROWS];
          stg_vs[i] = a.v_scale[srow0 + i * ROWS];
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < PASSES; ++i) {
        const int j = min((t - n_pre) * BN + srow + i * ROWS, n_b - 1);  // keys past the chunk are masked later
        const size_t off = ((size_t)(tok0 + j) * a.hkv + h) * HD + scc;
        stg_k[i] = *reinterpret_cast<const uint4*>(a.k_new + off);
        stg_v[i] = *reinterpret_cast<const uint4*>(a.v_new + off);
      }
    }
  };
  // this thread's fetched chunks of tile t into its LDS slot: fp16 for cache bytes and for the
  // chunk's V, the chunk's bf16 K as it is
  auto commit = [&](int t) {
    if (t >= t1) return;
    const u32 slot_off = (u32)(t & (kSlots - 1)) * (u32)(BUF_ELEMS * sizeof(uint16_t));
    const u32 kd = kw0 + slot_off, vd = vw0 + slot_off;
    if (t < n_pre) {
      // rows past the cached prefix hold stale bytes (fp8 has NaN codes, and 0 * NaN would
      // poison the second product): zero bytes are staged for them
      if ((t + 1) * BN > p) {
#pragma unroll
        for (int i = 0; i < PASSES; ++i)
          if (t * BN + srow + i * ROWS >= p) {
            stg_k[i].x = stg_k[i].y = stg_v[i].x = stg_v[i].y = 0u;
            if (DYN) stg_ks[i] = stg_vs[i] = 0.f;  // their scale slots may hold anything
          }
      }
#pragma unroll
      for (int i = 0; i < PASSES; ++i) {
        if (DYN) {
          lds_store16(kd + i * ROWS * LDK * 2, cvt8_scaled<QUANT>(stg_k[i].x, stg_k[i].y, stg_ks[i]));
          lds_store16(vd + i * ROWS * LDV * 2, cvt8_scaled<QUANT>(stg_v[i].x, stg_v[i].y, stg_vs[i]));
        } else {
          lds_store16(kd + i * ROWS * LDK * 2, cvt8<QUANT>(stg_k[i].x, stg_k[i].y));
          lds_store16(vd + i * ROWS * LDV * 2, cvt8<QUANT>(stg_v[i].x, stg_v[i].y));
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < PASSES; ++i) {
        lds_store16(kd + i * ROWS * LDK * 2, stg_k[i]);
        const u32 vw[4] = {stg_v[i].x, stg_v[i].y, stg_v[i].z, stg_v[i].w};
        u32 hw[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) hw[e] = pack_f16(sat_f16(bf16lo_to_f32(vw[e])), sat_f16(bf16hi_to_f32(vw[e])));
        lds_store16(vd + i * ROWS * LDV * 2, make_uint4(hw[0], hw[1], hw[2], hw[3]));
      }
    }
  };

  v16f o[4];  // O^T: rows = channels 32*ct + (r%4) + 8*(r/4) + 4*hf, column = this lane's query
#pragma unroll
  for (int ct = 0; ct < 4; ++ct)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[ct][r] = 0.f;
  float m_ref = -INFINITY;  // exponent reference of the weights: a maximum seen so far, at most ~10 (log2) below the largest score
  float l_run = 0.f;        // this lane's share (its 16 of every 32 keys) of the weight sum

  // tiles this wavefront computes on; chunk tiles wholly above its diagonal contribute
  // nothing and it only helps staging them
  const int my_tiles = wave_active ? min(n_pre + ci_wave_max / BN + 1, t1) : 0;
  const int q16 = lane >> 4, i16 = lane & 15;

  load_q(t0 < n_pre);
  // log2-domain constant that removes the byte offset from the prefix scores
  const float qbias = -ByteFmt<QUANT, DYN>::kOff * sc * (qsum + __shfl_xor(qsum, 32, 64));

  // prologue: the first tile (and group 1's rows of the second) into LDS
  fetch(t0);
  commit(t0);
  if (grp == 1) {
    fetch(t0 + 1);
    commit(t0 + 1);
  }
  if (early) fetch(t0 + lead);
  __syncthreads();
  if (grp == 1) __syncthreads();  // group 1 trails by one phase

  // leaving the quantised prefix: o holds sums over offset bytes; remove the offset and give the channels
  // their scale
  auto leave_prefix = [&]() {
    if (DYN) return;  // the staged values were the dequantised ones: nothing to remove, nothing to scale
    const float l_off = -ByteFmt<QUANT, DYN>::kOff * (l_run + __shfl_xor(l_run, 32, 64));
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
      for (int rb = 0; rb < 4; ++rb) {
        const float4 vs = *reinterpret_cast<const float4*>(a.v_scale + h * HD + 32 * ct + 8 * rb + 4 * hf);
        o[ct][4 * rb + 0] = (o[ct][4 * rb + 0] * ByteFmt<QUANT, DYN>::kMul + l_off) * vs.x;
        o[ct][4 * rb + 1] = (o[ct][4 * rb + 1] * ByteFmt<QUANT, DYN>::kMul + l_off) * vs.y;
        o[ct][4 * rb + 2] = (o[ct][4 * rb + 2] * ByteFmt<QUANT, DYN>::kMul + l_off) * vs.z;
        o[ct][4 * rb + 3] = (o[ct][4 * rb + 3] * ByteFmt<QUANT, DYN>::kMul + l_off) * vs.w;
      }
  };

  v16f st[2];
  v8h pf[2][2];
  for (int t = t0; t <= t1; ++t) {
    // ================= matrix phase =================
    if (t == n_pre && n_pre > 0 && t < my_tiles) load_q(false);  // the chunk's scores meet the bf16 q
    if (!early) fetch(t + lead);  // converted and written to LDS in the vector phase that follows
    // ---- O^T += V^T P^T, tile t-1, then S^T = K Q^T, tile t.  In the first product k-slot e of
    // lane group hf is key 32kb + 16ss + 8(e/4) + 4hf + e%4 (the P^T layout); lane i16 supplies
    // the row (key kbase + i16/4, channels cbase + 4(i16%4)..+3)
    const bool do_pv = t > t0 && t <= my_tiles, do_qk = t < my_tiles;
    const u32 va = lds_addr(lds + (size_t)((t + kSlots - 1) & (kSlots - 1)) * BUF_ELEMS + K_ELEMS + (4 * hf + (i16 >> 2)) * LDV +
                            16 * (q16 & 1) + 4 * (i16 & 3));
    const u32 ka = lds_addr(lds + (size_t)(t & (kSlots - 1)) * BUF_ELEMS + j32 * LDK + 8 * hf);
    if (do_pv) mm_pv(o, pf, va);
    if (do_qk) {
      if (t < n_pre)
        mm_qk<true>(st[0], st[1], qf, ka);
      else
        mm_qk<false>(st[0], st[1], qf, ka);
    }
    __syncthreads();
    // ================= vector phase =================
    // staging first: its LDS writes and global loads then run under the softmax arithmetic
    commit(t + lead);
    if (early) fetch(t + lead + 1);  // in flight for a whole tile period: this phase's arithmetic and the next matrix phase
    if (t < my_tiles) {
      if (t == n_pre && n_pre > 0) leave_prefix();
      // ---- mask + online softmax; this lane: one query, keys 32kb + (r%4) + 8(r/4) + 4hf
      const bool pre = t < n_pre;
      const int key0 = pre ? t * BN : (t - n_pre) * BN;  // index of the tile's first key in its segment
      const int limit = pre ? p - key0 : ci - key0 + 1;  // keys [0, limit) of the tile are visible
      const bool need_mask = pre ? (key0 + BN > p) : (pack || key0 + BN > q0 + 32 * wv + 1);
      if (need_mask) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = 32 * kb + (r & 3) + 8 * (r >> 2) + 4 * hf;
            st[kb][r] = key < limit ? st[kb][r] : -INFINITY;
          }
      }
      // logit (log2 domain) = accumulator * scl + add
      const float scl = pre ? sc * ByteFmt<QUANT, DYN>::kMul : sc;
      const float add = pre ? qbias : 0.f;
      // fp16 P^T operands and this lane's weight sum for the exponent reference m_ref
      float tsum;
      auto weights = [&]() {
        const float cst = add - (m_ref == -INFINITY ? 0.f : m_ref);
        const v2h ones = {(_Float16)1.0f, (_Float16)1.0f};
        float ls[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int ss = 0; ss < 2; ++ss) {
            // eight exponentials in flight at a time: the transcendental unit's latency is
            // paid once per batch, not once per pair
            float e8[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) e8[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(st[kb][8 * ss + e], scl, cst));
            u32 w[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              w[e] = pack_f16(e8[2 * e], e8[2 * e + 1]);  // round to nearest: truncation would bias every weight down
              // the sum is taken over the rounded weights, the ones the MFMA multiplies
              ls[e] = __builtin_amdgcn_fdot2(__builtin_bit_cast(v2h, w[e]), ones, ls[e], false);
            }
            pf[kb][ss] = __builtin_bit_cast(v8h, make_uint4(w[0], w[1], w[2], w[3]));
          }
        tsum = (ls[0] + ls[1]) + (ls[2] + ls[3]);
      };
      // Optimistic pass: weights against the reference as it stands.  Their sum over the
      // query's 64 keys bounds every one of them, so a sum within kSumLimit proves that the
      // reference was good enough (no weight beyond fp16, none worth rescaling for) without
      // ever looking for the tile's maximum.
      weights();
      const float qsum64 = tsum + swap32(tsum);
      const bool redo = !(qsum64 <= kSumLimit) || m_ref == -INFINITY;  // also true for inf / NaN sums
      if (__any(redo)) {
        // Rare (the first tile, and tiles whose scores outgrow the reference): take the exact
        // maximum, raise the reference of the queries that asked for it, rescale what they
        // have accumulated, and compute the weights again.
        float m4[4];  // four independent chains, not one of 32 dependent maxima
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          m4[c] = fmaxf(st[c >> 1][8 * (c & 1)], st[c >> 1][8 * (c & 1) + 1]);
#pragma unroll
          for (int r = 2; r < 8; ++r) m4[c] = fmaxf(m4[c], st[c >> 1][8 * (c & 1) + r]);
        }
        float mx = fmaxf(fmaxf(m4[0], m4[1]), fmaxf(m4[2], m4[3]));
        mx = fmaxf(mx, swap32(mx));
        mx = mx * scl + add;
        const bool raise = redo && mx > m_ref;
        const float alpha = raise ? __builtin_amdgcn_exp2f(m_ref - mx) : 1.0f;
        m_ref = raise ? mx : m_ref;
        l_run *= alpha;
#pragma unroll
        for (int ct = 0; ct < 4; ++ct)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[ct][r] *= alpha;
        weights();
      }
      l_run += tsum;
    }
    __syncthreads();
  }
  if (grp == 0) __syncthreads();  // the barrier group 1 took before its first phase

  if (!wave_active) return;
  if (t1 <= n_pre) leave_prefix();  // a share that ends inside the prefix (only with splits)
  if (ci_raw >= n_b) return;
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  if (n_splits > 1) {
    // ---- a partial for the merge: o unnormalised in fp32, the exponent reference and the weight sum
    const size_t row = ((size_t)blockIdx.y * a.num_tokens + tok0 + ci) * a.hq + qh_lane;
    float* po = a.part_o + row * HD;
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
      for (int rb = 0; rb < 4; ++rb)
        *reinterpret_cast<float4*>(po + 32 * ct + 8 * rb + 4 * hf) =
            make_float4(o[ct][4 * rb], o[ct][4 * rb + 1], o[ct][4 * rb + 2], o[ct][4 * rb + 3]);
    if (hf == 0) {
      a.part_ml[row * 2] = m_ref;
      a.part_ml[row * 2 + 1] = l_tot;
    }
    return;
  }
  // ---- epilogue: normalise and store bf16 (every query saw at least its own chunk tile)
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  uint16_t* orow = a.out + ((size_t)(tok0 + ci) * a.hq + qh_lane) * HD;
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

// Merge of the split partials: one wavefront per (new token of a prefill row, query head), lane = two channels.
// grid (ceil(max_chunk * hq / 4), rows), 256 threads.
__global__ __launch_bounds__(256) void prefill_merge_kernel(PrefillArgs a) {
  const int b = sequence_of_row(a, blockIdx.y), lane = threadIdx.x & 63;
  if (b < 0) return;
  if (a.seq_lens_encoder && a.seq_lens_encoder[b] <= 0) return;
  const int tok0 = a.cu_seqlens_q[b], n_b = a.cu_seqlens_q[b + 1] - tok0;
  const int unit = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int i = unit / a.hq, qh = unit - i * a.hq;
  if (i >= n_b) return;
  // the split count of this token's query tile, as the main kernel worked it out
  const int q0 = i / a.tile_tokens * a.tile_tokens;
  const int n_tiles = (a.seq_lens_decoder[b] + BN - 1) / BN + (min(n_b, q0 + a.tile_tokens) + BN - 1) / BN;
  const int n_splits = splits_of(n_tiles, a.n_splits);
  if (n_splits <= 1) return;  // the row is final already
  const size_t row0 = ((size_t)(tok0 + i)) * a.hq + qh, stride = (size_t)a.num_tokens * a.hq;
  // every partial is requested before any is used: one round trip to memory, not one per split
  float ms[kMaxSplits], ls[kMaxSplits];
  float2 v[kMaxSplits];
#pragma unroll
  for (int s = 0; s < kMaxSplits; ++s)
    if (s < n_splits) {
      ms[s] = a.part_ml[(row0 + s * stride) * 2];
      ls[s] = a.part_ml[(row0 + s * stride) * 2 + 1];
      // an empty share (m = -inf) has no o: the load is skipped by the weight 0 below, its address is still valid memory
      v[s] = *reinterpret_cast<const float2*>(a.part_o + (row0 + s * stride) * HD + 2 * lane);
    }
  float M = -INFINITY;
#pragma unroll
  for (int s = 0; s < kMaxSplits; ++s)
    if (s < n_splits) M = fmaxf(M, ms[s]);
  float L = 0.f, o0 = 0.f, o1 = 0.f;
  if (M > -INFINITY) {
#pragma unroll
    for (int s = 0; s < kMaxSplits; ++s)
      if (s < n_splits && ms[s] > -INFINITY) {
        const float f = __builtin_amdgcn_exp2f(ms[s] - M);
        L += ls[s] * f;
        o0 += v[s].x * f;
        o1 += v[s].y * f;
      }
  }
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  *reinterpret_cast<u32*>(a.out + row0 * HD + 2 * lane) = pack_bf16(o0 * inv, o1 * inv);
}

bool prefill_mfma_supported(int hq, int hkv, int d, int bs, int quant) {
  return d == HD && bs == BN && hq % hkv == 0 && quant_known(quant);
}

namespace {

template <int QUANT, int NW, bool DYN>
hipError_t launch_one(const PrefillArgs& a, int max_chunk, hipStream_t s) {
  constexpr int BM = 32 * NW;
  PrefillArgs args = a;
  args.q_tiles = a.pack_slot > 0 ? 1 : (max_chunk + BM - 1) / BM;
  const dim3 grid((unsigned)a.rows * (a.pack_slot > 0 ? a.hkv : a.hq) * args.q_tiles, a.n_splits), block(64 * NW);
  const size_t shm = (size_t)kSlots * BUF_ELEMS * sizeof(uint16_t);  // 151,552 B
  // the dynamic LDS limit is a per-device property of the kernel: raise it once on each device
  static std::atomic<unsigned long long> raised{0};  // bit d: done on device d (one word per instantiation)
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev >= 64 || !(raised.load(std::memory_order_relaxed) >> dev & 1ull)) {
    e = hipFuncSetAttribute((const void*)prefill_mfma_kernel<QUANT, NW, DYN>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)shm);
    if (e != hipSuccess) return e;
    if (dev < 64) raised.fetch_or(1ull << dev, std::memory_order_relaxed);
  }
  hipLaunchKernelGGL((prefill_mfma_kernel<QUANT, NW, DYN>), grid, block, shm, s, args);
  return hipSuccess;
}

}  // namespace

size_t prefill_split_workspace_bytes(int num_tokens, int hq, int n_splits) {
  if (n_splits <= 1 || num_tokens <= 0 || hq <= 0) return 0;
  if (n_splits > kMaxSplits) n_splits = kMaxSplits;
  return (size_t)n_splits * num_tokens * hq * (HD + 2) * sizeof(float);
}

// 256-token workgroups (8 wavefronts, the two groups overlapping MFMA and vector work) whenever they - times the
// key splits - cover the CUs (one workgroup fits a CU); 128-token ones otherwise
static bool wide_workgroups(int rows, int hq, int max_chunk, int n_splits) {
  return max_chunk > 128 && (long long)rows * hq * ((max_chunk + 255) / 256) * n_splits >= gpu_cu_count();
}

// Short chunks: when all query heads of a KV head, times the chunk's tokens, fit the query columns of one
// workgroup (128 or 256), the workgroup takes the whole group and its staged K / V tiles serve every head.
// Returns the tokens per head slot (0: not packed) and the workgroup's wavefront count.
static int pack_slot_for(int hq, int hkv, int max_chunk, int* nw) {
  const int g = hkv > 0 ? hq / hkv : 0;
  if (g < 2 || max_chunk <= 0 || (long long)g * max_chunk > 256) return 0;
  // always the 8-wavefront workgroup: its two wavefront groups overlap MFMA and vector work, and wavefronts whose
  // columns hold no token (slots are 256 / g tokens wide) only help with the staging
  *nw = 8;
  return 32 * *nw / g;
}

int prefill_auto_splits(int rows, int hq, int max_chunk, int hkv) {
  if (rows <= 0 || hq <= 0 || max_chunk <= 0) return 1;
  const int cus = gpu_cu_count();
  int nw = 0;
  if (pack_slot_for(hq, hkv, max_chunk, &nw) > 0) {  // one workgroup per (row, KV head)
    const long long wgs = (long long)rows * hkv, sp = (cus + wgs - 1) / wgs;
    return (int)(sp < 1 ? 1 : (sp > kMaxSplits ? kMaxSplits : sp));
  }
  auto splits_for = [&](int bm) {
    const long long wgs = (long long)rows * hq * ((max_chunk + bm - 1) / bm);
    const long long s = (cus + wgs - 1) / wgs;  // enough to give every CU a workgroup
    return (int)(s < 1 ? 1 : (s > kMaxSplits ? kMaxSplits : s));
  };
  if (max_chunk > 128) {
    const int s = splits_for(256);
    if (wide_workgroups(rows, hq, max_chunk, s)) return s;
  }
  return splits_for(128);
}

int prefill_mfma_launch(const PrefillArgs& a_in, int max_chunk, int quant, hipStream_t s, void* workspace,
                        size_t workspace_bytes, int n_splits, int rows_hint) {
  PrefillArgs a = a_in;
  if (n_splits > kMaxSplits) n_splits = kMaxSplits;
  while (n_splits > 1 && (!workspace || workspace_bytes < prefill_split_workspace_bytes(a.num_tokens, a.hq, n_splits))) --n_splits;
  a.n_splits = n_splits < 1 ? 1 : n_splits;
  a.rows = rows_hint > 0 && rows_hint < a.batch && a.seq_lens_encoder ? rows_hint : a.batch;
  a.part_o = (float*)workspace;
  a.part_ml = a.part_o + (size_t)a.n_splits * a.num_tokens * a.hq * HD;
  if ((long long)a_in.batch * a_in.hq * ((max_chunk + 127) / 128) > 0x7fffffffLL)
    return fail(FDATTN_ERR_SHAPE, "fdattn_append_attention_prefill: too many workgroups for one launch");
  // 256-token workgroups share each staged tile among 8 wavefronts (their two groups alternate between the MFMA
  // units and the vector ALU); short chunks keep 128
  // when they would still leave CUs without a workgroup (one fits a CU), 128-token workgroups cover twice as
  // many CUs: 10-14 % faster at e.g. 2 x 512 tokens, although a 4-wavefront workgroup overlaps nothing
  int pack_nw = 0;
  a.pack_slot = pack_slot_for(a.hq, a.hkv, max_chunk, &pack_nw);
  const bool wide = a.pack_slot > 0 ? pack_nw == 8 : wide_workgroups(a.rows, a.hq, max_chunk, a.n_splits);
  hipError_t e;
  if (quant == FDATTN_CACHE_INT8)
    e = wide ? launch_one<FDATTN_CACHE_INT8, 8, false>(a, max_chunk, s) : launch_one<FDATTN_CACHE_INT8, 4, false>(a, max_chunk, s);
  else if (quant == FDATTN_CACHE_FP8_E4M3)
    e = wide ? launch_one<FDATTN_CACHE_FP8_E4M3, 8, false>(a, max_chunk, s)
             : launch_one<FDATTN_CACHE_FP8_E4M3, 4, false>(a, max_chunk, s);
  else if (quant == FDATTN_CACHE_INT8_DYNAMIC)
    e = wide ? launch_one<FDATTN_CACHE_INT8, 8, true>(a, max_chunk, s) : launch_one<FDATTN_CACHE_INT8, 4, true>(a, max_chunk, s);
  else
    e = wide ? launch_one<FDATTN_CACHE_FP8_E4M3, 8, true>(a, max_chunk, s)
             : launch_one<FDATTN_CACHE_FP8_E4M3, 4, true>(a, max_chunk, s);
  if (e != hipSuccess) return fail((int)e, "fdattn_append_attention_prefill: %s", hipGetErrorString(e));
  int rc = check_launch("fdattn_append_attention_prefill (mfma)");
  if (rc || a.n_splits <= 1) return rc;
  a.tile_tokens = a.pack_slot > 0 ? a.pack_slot : (wide ? 256 : 128);
  hipLaunchKernelGGL(prefill_merge_kernel, dim3(((long long)max_chunk * a.hq + 3) / 4, a.rows), dim3(256), 0, s, a);
  return check_launch("fdattn_append_attention_prefill (merge)");
}

}  // namespace fdattn
