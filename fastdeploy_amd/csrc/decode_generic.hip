// Shape-agnostic decode attention over the quantised paged cache, and the split-KV
// combine.  One wavefront per (sequence, query head, KV split): lanes own tokens for
// q.K and channels for P.V.  This is the fall-back for shapes the MFMA kernel in
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

// DYN: cache scales per stored row ([num_blocks, hkv, bs]) instead of per channel.
template <int QUANT, bool DYN>
__global__ __launch_bounds__(64) void decode_generic_kernel(GenericDecodeArgs a) {
  __shared__ float qs[kMaxD];
  __shared__ float pbuf[64];
  const int lane = threadIdx.x;
  const int row = blockIdx.x, split = blockIdx.y, nsplit = gridDim.y;
  const int b = row / a.hq, qh = row % a.hq, g = a.hq / a.hkv, h = qh / g;
  const int d = a.d, bs = a.bs;
  int qrow;  // the sequence's row of q
  if (!decode_row(a.rows, b, qrow)) return;
  const int kv_len = a.seq_lens_decoder[b] + (a.seq_lens_this_time ? a.seq_lens_this_time[b] : 0);

  for (int c = lane; c < d; c += 64)
    qs[c] = bf16_to_f32(a.q[((size_t)qrow * a.hq + qh) * d + c]) * (DYN ? 1.0f : a.k_scale[h * d + c]) * a.sm_scale;
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

  float m = -INFINITY, l = 0.f;
  float acc[kMaxD / 64] = {0.f, 0.f, 0.f, 0.f};
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
      float s = -INFINITY;
      if (valid) {
        s = 0.f;
        const uint8_t* kr = kp + (size_t)t * d;
        for (int c = 0; c < d; c += 4) {
          u32 w = *reinterpret_cast<const u32*>(kr + c);
          s += qs[c] * dq<QUANT>(w & 0xff) + qs[c + 1] * dq<QUANT>((w >> 8) & 0xff) +
               qs[c + 2] * dq<QUANT>((w >> 16) & 0xff) + qs[c + 3] * dq<QUANT>(w >> 24);
        }
        if (DYN) s *= a.k_scale[srow + t];
      }
      const float mb = wave_max(s);
      if (mb == -INFINITY) continue;  // uniform: no valid token in this group
      const float m_new = fmaxf(m, mb);
      const float alpha = (m == -INFINITY) ? 0.f : __expf(m - m_new);
      const float p = valid ? __expf(s - m_new) : 0.f;
      l = l * alpha + wave_sum(p);
      m = m_new;
      __syncthreads();
      pbuf[lane] = (DYN && valid) ? p * a.v_scale[srow + t] : p;  // the V row's scale rides on its weight
      __syncthreads();
      const int nt = min(64, bs - t0);
#pragma unroll
      for (int i = 0; i < kMaxD / 64; ++i) {
        const int c = lane + 64 * i;
        if (c < d) {
          float o = acc[i] * alpha;
          for (int tt = 0; tt < nt; ++tt) o += pbuf[tt] * dq<QUANT>(vp[(size_t)(t0 + tt) * d + c]);
          acc[i] = o;
        }
      }
    }
  }
  const size_t slot = (size_t)row * a.max_splits + split;
#pragma unroll
  for (int i = 0; i < kMaxD / 64; ++i) {
    const int c = lane + 64 * i;
    if (c < d) a.part_o[slot * d + c] = DYN ? acc[i] : acc[i] * a.v_scale[h * d + c];
  }
  if (lane == 0) {
    a.part_m[slot] = m;
    a.part_l[slot] = l;
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
  int nsplit = 2048 / rows;
  nsplit = nsplit < 1 ? 1 : (nsplit > kGenericMaxSplits ? kGenericMaxSplits : nsplit);
  // partial layout [rows, nsplit, ...]: the combine then reads exactly the slots written
  float* part_o = (float*)workspace;
  float* part_m = part_o + (size_t)rows * nsplit * d;
  float* part_l = part_m + (size_t)rows * nsplit;
  GenericDecodeArgs a{(const uint16_t*)q, (const uint8_t*)key_cache, (const uint8_t*)value_cache,
                      k_scale, v_scale, block_tables, seq_lens_decoder, seq_lens_this_time,
                      kept_blocks, kept_counts, max_kept, part_o, part_m, part_l, rmap, batch, hq, hkv,
                      d, bs, max_blocks, num_blocks, nsplit, sm_scale};
  const dim3 grid(rows, nsplit);
  if (quant == FDATTN_CACHE_INT8)
    hipLaunchKernelGGL((decode_generic_kernel<FDATTN_CACHE_INT8, false>), grid, dim3(64), 0, s, a);
  else if (quant == FDATTN_CACHE_FP8_E4M3)
    hipLaunchKernelGGL((decode_generic_kernel<FDATTN_CACHE_FP8_E4M3, false>), grid, dim3(64), 0, s, a);
  else if (quant == FDATTN_CACHE_INT8_DYNAMIC)
    hipLaunchKernelGGL((decode_generic_kernel<FDATTN_CACHE_INT8, true>), grid, dim3(64), 0, s, a);
  else
    hipLaunchKernelGGL((decode_generic_kernel<FDATTN_CACHE_FP8_E4M3, true>), grid, dim3(64), 0, s, a);
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
