// Shape-agnostic decode attention over the quantised paged cache, and the split-KV
// combine.  One wavefront per (sequence, KV head, up to 8 of its query heads, KV split): lanes own
// tokens for q.K and channels for P.V.  This is the fall-back for shapes the MFMA kernel in
// decode_c8.hip does not cover (any head_dim <= 256, any group size, any block size);
// it makes no attempt to reach the HBM roofline.  The formats with one scale per stored
// row (DYN) multiply a token's score by its K scale and its weight by its V scale.
#include "launch.h"

namespace fdattn {

struct GenericDecodeArgs {
  const uint16_t* q;
  const uint8_t* key_cache;
  const uint8_t* value_cache;
  const float* k_scale;
  const float* v_scale;
  const int32_t* block_tables;
  const int32_t* seq_lens_decoder;
  const int32_t* seq_lens_this_time;
  const int32_t* kept_blocks;  // nullptr = dense
  const int32_t* kept_counts;
  int max_kept;
  float* part_o;  // [rows, max_splits, d]
  float* part_m;  // [rows, max_splits]
  float* part_l;
  RowMap rows;
  int batch, hq, hkv, d, bs, max_blocks, num_blocks, max_splits;
  float sm_scale;
};

template <int QUANT>
__device__ __forceinline__ float dq(u32 byte) {
  if (QUANT == FDATTN_CACHE_INT8) return (float)(int)(int8_t)byte;
  return e4m3_to_f32(byte);
}

constexpr int kMaxD = 256;

// One wavefront per (sequence, KV head, set of up to NH (4 or 8) of its query heads, KV split): the K and V bytes it reads
// serve all the heads of the set.  Scores: lane = token of a group of 64, its K row read in 16-byte words, one dot
// product per head against q * k_scale * softmax_scale in LDS.  P.V: lane = four channels of one of the 64 / (d/4)
// token rows read at a time; the rows' sums meet in LDS at the end.
// DYN: cache scales per stored row ([num_blocks, hkv, bs]) instead of per channel.
template <int QUANT, bool DYN, int NH>
__global__ __launch_bounds__(64) void decode_generic_kernel(GenericDecodeArgs a) {
  __shared__ __attribute__((aligned(16))) float qs[NH][kMaxD];  // q of the set's heads; at the end: their outputs
  __shared__ float pbuf[NH][64];
  const int lane = threadIdx.x;
  const int split = blockIdx.y, nsplit = gridDim.y;
  const int g = a.hq / a.hkv, sets = (g + NH - 1) / NH;
  const int set = blockIdx.x % sets, p = blockIdx.x / sets;
  const int b = p / a.hkv, h = p % a.hkv;
  const int g0 = set * NH, ng = min(NH, g - g0);  // heads h*g + g0 .. + ng - 1
  const int d = a.d, bs = a.bs;
  int qrow;  // the sequence's row of q
  if (!decode_row(a.rows, b, qrow)) return;
  const int kv_len = a.seq_lens_decoder[b] + (a.seq_lens_this_time ? a.seq_lens_this_time[b] : 0);

  for (int i = lane; i < NH * d; i += 64) {
    const int gg = i / d, c = i - gg * d;
    qs[gg][c] = gg < ng ? bf16_to_f32(a.q[((size_t)qrow * a.hq + h * g + g0 + gg) * d + c]) *
                              (DYN ? 1.0f : a.k_scale[h * d + c]) * a.sm_scale
                        : 0.f;  // heads past the set: zero rows, so that the loops below need no test
  }
  __syncthreads();

  int nblk = (kv_len + bs - 1) / bs;
  if (nblk > a.max_blocks) nblk = a.max_blocks;
  const int32_t* list = nullptr;
  if (a.kept_blocks) {
    list = a.kept_blocks + ((size_t)b * a.hkv + h) * a.max_kept;
    nblk = min(a.kept_counts[b * a.hkv + h], a.max_kept);
  }
  const int per = (nblk + nsplit - 1) / nsplit;
  const int i0 = split * per, i1 = min(nblk, i0 + per);

  // P.V layout: lanes_per_row lanes cover a row's d channels, 4 each; rows_per_pass rows at a time
  const int lanes_per_row = d / 4, rows_per_pass = 64 / lanes_per_row;
  const int vslot = lane / lanes_per_row, c4 = 4 * (lane - vslot * lanes_per_row);
  const bool vlane = vslot < rows_per_pass;

  float m[NH], l[NH], acc[NH][4];
#pragma unroll
  for (int gg = 0; gg < NH; ++gg) {
    m[gg] = -INFINITY, l[gg] = 0.f;
    acc[gg][0] = acc[gg][1] = acc[gg][2] = acc[gg][3] = 0.f;
  }
  const int32_t* table = a.block_tables + (size_t)b * a.max_blocks;

  for (int bi = i0; bi < i1; ++bi) {
    const int lb = list ? list[bi] : bi;
    if (lb < 0 || lb >= a.max_blocks) continue;
    const int pb = table[lb];
    if (pb < 0 || pb >= a.num_blocks) continue;
    const uint8_t* kp = a.key_cache + ((size_t)pb * a.hkv + h) * bs * d;
    const uint8_t* vp = a.value_cache + ((size_t)pb * a.hkv + h) * bs * d;
    const size_t srow = ((size_t)pb * a.hkv + h) * bs;  // DYN: this tile's rows in the scale caches
    for (int t0 = 0; t0 < bs; t0 += 64) {
      const int t = t0 + lane;
      const bool valid = t < bs && lb * bs + t < kv_len;
      if (!__any(valid)) continue;  // no valid token in this group
      float s[NH];
#pragma unroll
      for (int gg = 0; gg < NH; ++gg) s[gg] = 0.f;
      if (valid) {
        const uint8_t* kr = kp + (size_t)t * d;
        auto word = [&](u32 w, int c) {  // four channels of the row against every head's q
          const float k0 = dq<QUANT>(w & 0xff), k1 = dq<QUANT>((w >> 8) & 0xff), k2 = dq<QUANT>((w >> 16) & 0xff),
                      k3 = dq<QUANT>(w >> 24);
#pragma unroll
          for (int gg = 0; gg < NH; ++gg) {
            const float4 qv = *reinterpret_cast<const float4*>(&qs[gg][c]);
            s[gg] += qv.x * k0 + qv.y * k1 + qv.z * k2 + qv.w * k3;
          }
        };
        int c = 0;
        const int d16 = (d & 15) ? 0 : d;  // 16-byte words only where every row starts on one
        for (; c < d16; c += 16) {
          const uint4 w = *reinterpret_cast<const uint4*>(kr + c);
          word(w.x, c), word(w.y, c + 4), word(w.z, c + 8), word(w.w, c + 12);
        }
        for (; c < d; c += 4) word(*reinterpret_cast<const u32*>(kr + c), c);
      }
      const float ksc = (DYN && valid) ? a.k_scale[srow + t] : 1.0f;
      const float vsc = (DYN && valid) ? a.v_scale[srow + t] : 1.0f;  // the V row's scale rides on its weight
      // Softmax weights against a per-head reference that is raised only when a score outgrows it by more than
      // 2^10 (one ballot per head and group instead of a maximum over the wavefront; the weights stay below e^10);
      // the weight sums stay per lane until the end.
#pragma unroll
      for (int gg = 0; gg < NH; ++gg) {
        const float sv = valid ? s[gg] * ksc : -INFINITY;
        if (__any(valid && !(sv <= m[gg] + 10.0f))) {  // also the first group (m = -inf) and NaN scores
          const float m_new = fmaxf(m[gg], wave_max(sv));
          const float al = (m[gg] == -INFINITY) ? 0.f : __expf(m[gg] - m_new);
          l[gg] *= al;
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[gg][e] *= al;
          m[gg] = m_new;
        }
        const float pr = valid ? __expf(sv - m[gg]) : 0.f;
        l[gg] += pr;
        pbuf[gg][lane] = pr * vsc;
      }
      __syncthreads();
      const int nt = min(64, min(bs - t0, kv_len - lb * bs - t0));  // rows past the sequence weigh 0: not read
      if (vlane) {
        for (int tt = vslot; tt < nt; tt += rows_per_pass) {
          const u32 w = *reinterpret_cast<const u32*>(vp + (size_t)(t0 + tt) * d + c4);
          const float v0 = dq<QUANT>(w & 0xff), v1 = dq<QUANT>((w >> 8) & 0xff), v2 = dq<QUANT>((w >> 16) & 0xff),
                      v3 = dq<QUANT>(w >> 24);
#pragma unroll
          for (int gg = 0; gg < NH; ++gg) {
            const float pw = pbuf[gg][tt];
            acc[gg][0] += pw * v0, acc[gg][1] += pw * v1, acc[gg][2] += pw * v2, acc[gg][3] += pw * v3;
          }
        }
      }
      __syncthreads();
    }
  }
  // the row slots' sums meet in LDS (q is no longer needed), one slot after the other
  __syncthreads();
  for (int sl = 0; sl < rows_per_pass; ++sl) {
    if (vlane && vslot == sl) {
#pragma unroll
      for (int gg = 0; gg < NH; ++gg)
#pragma unroll
        for (int e = 0; e < 4; ++e) qs[gg][c4 + e] = (sl == 0 ? 0.f : qs[gg][c4 + e]) + acc[gg][e];
    }
    __syncthreads();
  }
  for (int gg = 0; gg < ng; ++gg) {
    const size_t slot = ((size_t)b * a.hq + h * g + g0 + gg) * a.max_splits + split;
    for (int c = lane; c < d; c += 64) a.part_o[slot * d + c] = DYN ? qs[gg][c] : qs[gg][c] * a.v_scale[h * d + c];
  }
#pragma unroll
  for (int gg = 0; gg < NH; ++gg) {
    const float lsum = wave_sum(l[gg]);
    if (lane == 0 && gg < ng) {
      const size_t slot = ((size_t)b * a.hq + h * g + g0 + gg) * a.max_splits + split;
      a.part_m[slot] = m[gg];
      a.part_l[slot] = lsum;
    }
  }
}

// out[r,:] = sum_s o_s e^(m_s - m) / sum_s l_s e^(m_s - m); one thread per channel.
// With a row map (hq > 0) partial row r = (sequence, head) goes to the sequence's out row, and
// sequences that are not decode rows are left alone.
__global__ void splitkv_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_m,
                                       const float* __restrict__ part_l, const int32_t* __restrict__ num_splits,
                                       uint16_t* __restrict__ out, int rows, int max_splits, int d, int hq,
                                       RowMap map) {
  const int r = blockIdx.x;
  size_t orow = (size_t)r;
  if (hq > 0) {
    int srow;
    if (!decode_row(map, r / hq, srow)) return;
    orow = (size_t)srow * hq + r % hq;
  }
  const int ns = num_splits ? min(num_splits[r], max_splits) : max_splits;
  float m = -INFINITY;
  for (int s = 0; s < ns; ++s) m = fmaxf(m, part_m[(size_t)r * max_splits + s]);
  float l = 0.f;
  for (int s = 0; s < ns; ++s) {
    const float ms = part_m[(size_t)r * max_splits + s];
    if (ms > -INFINITY) l += part_l[(size_t)r * max_splits + s] * __expf(ms - m);
  }
  for (int c = threadIdx.x; c < d; c += blockDim.x) {
    float o = 0.f;
    for (int s = 0; s < ns; ++s) {
      const float ms = part_m[(size_t)r * max_splits + s];
      if (ms > -INFINITY) o += part_o[((size_t)r * max_splits + s) * d + c] * __expf(ms - m);
    }
    out[orow * d + c] = f32_to_bf16(l > 0.f ? o / l : 0.f);
  }
}

constexpr int kGenericMaxSplits = 16;

size_t generic_workspace_bytes(int batch, int hq, int d) {
  return (size_t)batch * hq * kGenericMaxSplits * (d + 2) * sizeof(float);
}

int decode_generic_launch(const void* q, const void* key_cache, const void* value_cache,
                          const float* k_scale, const float* v_scale, const int32_t* block_tables,
                          const int32_t* seq_lens_decoder, const int32_t* seq_lens_this_time,
                          const int32_t* kept_blocks, const int32_t* kept_counts, int max_kept,
                          void* out, void* workspace, size_t workspace_bytes, int batch, int hq,
                          int hkv, int d, int bs, int max_blocks, int num_blocks, int quant,
                          float sm_scale, hipStream_t s, RowMap rmap) {
  if (d > kMaxD || d % 4 != 0)
    return fail(FDATTN_ERR_SHAPE, "fdattn_decode_attention: head_dim %d unsupported (multiple of 4, <= %d)", d, kMaxD);
  const size_t need = generic_workspace_bytes(batch, hq, d);
  if (workspace_bytes < need)
    return fail(FDATTN_ERR_WORKSPACE, "fdattn_decode_attention: workspace %zu B < required %zu B", workspace_bytes, need);
  const int rows = batch * hq;
  const int nh = hq / hkv <= 4 ? 4 : 8;  // query heads of one KV head a workgroup serves together
  const int sets = (hq / hkv + nh - 1) / nh, wgs = batch * hkv * sets;
  int nsplit = 4096 / wgs;
  nsplit = nsplit < 1 ? 1 : (nsplit > kGenericMaxSplits ? kGenericMaxSplits : nsplit);
  // partial layout [rows, nsplit, ...]: the combine then reads exactly the slots written
  float* part_o = (float*)workspace;
  float* part_m = part_o + (size_t)rows * nsplit * d;
  float* part_l = part_m + (size_t)rows * nsplit;
  GenericDecodeArgs a{(const uint16_t*)q, (const uint8_t*)key_cache, (const uint8_t*)value_cache,
                      k_scale, v_scale, block_tables, seq_lens_decoder, seq_lens_this_time,
                      kept_blocks, kept_counts, max_kept, part_o, part_m, part_l, rmap, batch, hq, hkv,
                      d, bs, max_blocks, num_blocks, nsplit, sm_scale};
  const dim3 grid(wgs, nsplit);
#define FDATTN_GEN_LAUNCH(Q, D)                                                                     \
  do {                                                                                              \
    if (nh == 4) hipLaunchKernelGGL((decode_generic_kernel<Q, D, 4>), grid, dim3(64), 0, s, a);     \
    else hipLaunchKernelGGL((decode_generic_kernel<Q, D, 8>), grid, dim3(64), 0, s, a);             \
  } while (0)
  if (quant == FDATTN_CACHE_INT8) FDATTN_GEN_LAUNCH(FDATTN_CACHE_INT8, false);
  else if (quant == FDATTN_CACHE_FP8_E4M3) FDATTN_GEN_LAUNCH(FDATTN_CACHE_FP8_E4M3, false);
  else if (quant == FDATTN_CACHE_INT8_DYNAMIC) FDATTN_GEN_LAUNCH(FDATTN_CACHE_INT8, true);
  else FDATTN_GEN_LAUNCH(FDATTN_CACHE_FP8_E4M3, true);
#undef FDATTN_GEN_LAUNCH
  int rc = check_launch("fdattn_decode_attention (generic)");
  if (rc) return rc;
  hipLaunchKernelGGL(splitkv_combine_kernel, dim3(rows), dim3(128), 0, s, part_o, part_m, part_l,
                     (const int32_t*)nullptr, (uint16_t*)out, rows, nsplit, d, hq, rmap);
  return check_launch("fdattn_splitkv_combine");
}

}  // namespace fdattn

using namespace fdattn;

extern "C" int fdattn_splitkv_combine(const float* part_o, const float* part_m, const float* part_l,
                                      const int32_t* num_splits, void* out, int rows, int max_splits,
                                      int head_dim, void* stream) {
  if (!part_o || !part_m || !part_l || !out)
    return fail(FDATTN_ERR_NULL, "fdattn_splitkv_combine: a required pointer is NULL");
  if (rows < 0 || max_splits <= 0 || head_dim <= 0)
    return fail(FDATTN_ERR_SHAPE, "fdattn_splitkv_combine: bad shape rows=%d max_splits=%d head_dim=%d", rows,
                max_splits, head_dim);
  if (rows == 0) return 0;
  hipLaunchKernelGGL(splitkv_combine_kernel, dim3(rows), dim3(128), 0, (hipStream_t)stream, part_o, part_m,
                     part_l, num_splits, (uint16_t*)out, rows, max_splits, head_dim, 0, RowMap{nullptr, nullptr});
  return check_launch("fdattn_splitkv_combine");
}
