// SQAttn block selector: per-block max q.k scores over the quantised K pages and a
// per-(sequence, KV head) top-k with ties to the lower block index.
//
// Scores are computed in fp64 with the channels summed in ascending order, one
// token per lane.  Every product (fp32 q*scale times an int8 / e4m3 value) is exact
// in fp64, so only the order of the additions matters for the bits of the result,
// and that order is fixed: the selection is reproducible bit for bit on a CPU.
#include "fdattn_common.h"

namespace fdattn {

struct ScoreArgs {
  const uint16_t* q;
  const uint8_t* key_cache;
  const float* k_scale;
  const int32_t* block_tables;
  const int32_t* seq_lens_decoder;
  const int32_t* seq_lens_this_time;
  double* scores;  // [batch, hkv, max_blocks]
  float* scores_f32;
  int batch, hq, hkv, d, bs, max_blocks, num_blocks;
};

constexpr int kSelMaxD = 256;
constexpr int kSelMaxG = 8;

template <int QUANT>
__device__ __forceinline__ double dq64(u32 byte) {
  if (QUANT == FDATTN_CACHE_INT8) return (double)(int)(int8_t)byte;
  return (double)e4m3_to_f32(byte);
}

// grid (max_blocks, hkv, batch), one wavefront: lane = token of the block
template <int QUANT>
__global__ __launch_bounds__(64) void sqattn_block_scores_kernel(ScoreArgs a) {
  __shared__ float qs[kSelMaxG][kSelMaxD];
  const int j = blockIdx.x, h = blockIdx.y, b = blockIdx.z, lane = threadIdx.x;
  const int g = a.hq / a.hkv, d = a.d, bs = a.bs;
  const int kv_len = a.seq_lens_decoder[b] + (a.seq_lens_this_time ? a.seq_lens_this_time[b] : 0);
  const size_t o = ((size_t)b * a.hkv + h) * a.max_blocks + j;
  const int t0 = j * bs;
  int pb = -1;
  if (t0 < kv_len) pb = a.block_tables[(size_t)b * a.max_blocks + j];
  if (pb < 0 || pb >= a.num_blocks) {
    if (lane == 0) {
      a.scores[o] = -INFINITY;
      if (a.scores_f32) a.scores_f32[o] = -INFINITY;
    }
    return;
  }
  for (int i = lane; i < g * d; i += 64) {
    const int gi = i / d, c = i % d;
    // one fp32 rounding, as the definition of the score says
    qs[gi][c] = __fmul_rn(bf16_to_f32(a.q[((size_t)b * a.hq + h * g + gi) * d + c]), a.k_scale[h * d + c]);
  }
  __syncthreads();
  double best = -INFINITY;
  const uint8_t* kp = a.key_cache + ((size_t)pb * a.hkv + h) * bs * d;
  for (int t = lane; t < bs; t += 64) {
    if (t0 + t >= kv_len) break;
    const uint8_t* kr = kp + (size_t)t * d;
    double s[kSelMaxG];
#pragma unroll
    for (int gi = 0; gi < kSelMaxG; ++gi) s[gi] = 0.0;
    for (int c = 0; c < d; c += 4) {
      const u32 w = *reinterpret_cast<const u32*>(kr + c);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const double kv = dq64<QUANT>((w >> (8 * e)) & 0xff);
#pragma unroll
        for (int gi = 0; gi < kSelMaxG; ++gi)
          if (gi < g) s[gi] = __dadd_rn(s[gi], __dmul_rn((double)qs[gi][c + e], kv));
      }
    }
#pragma unroll
    for (int gi = 0; gi < kSelMaxG; ++gi)
      if (gi < g) best = fmax(best, s[gi]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) best = fmax(best, __shfl_xor(best, off, 64));
  if (lane == 0) {
    a.scores[o] = best;
    if (a.scores_f32) a.scores_f32[o] = (float)best;
  }
}

// One workgroup per (sequence, KV head).  rank(j) = #{i : s_i > s_j or (s_i == s_j and i < j)};
// block j is kept iff rank(j) < k; kept indices are emitted in ascending order.
__global__ __launch_bounds__(256) void sqattn_topk_kernel(const double* __restrict__ scores,
                                                          const int32_t* __restrict__ seq_lens_decoder,
                                                          const int32_t* __restrict__ seq_lens_this_time,
                                                          int32_t* __restrict__ kept_blocks,
                                                          int32_t* __restrict__ kept_counts, int hkv, int bs,
                                                          int max_blocks, int top_k) {
  extern __shared__ double sm[];  // scores [max_blocks], then int flags/prefix
  int* keep = reinterpret_cast<int*>(sm + max_blocks);
  __shared__ int wave_tot[4];
  __shared__ int running;
  const int b = blockIdx.x / hkv, tid = threadIdx.x;
  const double* s = scores + (size_t)blockIdx.x * max_blocks;
  const int kv_len = seq_lens_decoder[b] + (seq_lens_this_time ? seq_lens_this_time[b] : 0);
  int nblk = (kv_len + bs - 1) / bs;
  if (nblk > max_blocks) nblk = max_blocks;
  const int k = top_k < nblk ? top_k : nblk;
  for (int j = tid; j < nblk; j += 256) sm[j] = s[j];
  if (tid == 0) running = 0;
  __syncthreads();
  for (int j = tid; j < nblk; j += 256) {
    const double sj = sm[j];
    int rank = 0;
    for (int i = 0; i < nblk; ++i) {
      const double si = sm[i];
      rank += (si > sj) || (si == sj && i < j);
    }
    keep[j] = rank < k;
  }
  __syncthreads();
  int32_t* o = kept_blocks + (size_t)blockIdx.x * top_k;
  // ordered compaction, 256 candidates at a time
  for (int base = 0; base < nblk; base += 256) {
    const int j = base + tid;
    const int f = j < nblk ? keep[j] : 0;
    const unsigned long long bal = __ballot(f);
    const int lane = tid & 63, w = tid >> 6;
    const int before = __popcll(bal & ((1ull << lane) - 1ull));
    if (lane == 0) wave_tot[w] = __popcll(bal);
    __syncthreads();
    int off = running;
    for (int ww = 0; ww < w; ++ww) off += wave_tot[ww];
    if (f) o[off + before] = j;
    __syncthreads();
    if (tid == 0) running += wave_tot[0] + wave_tot[1] + wave_tot[2] + wave_tot[3];
    __syncthreads();
  }
  for (int j = k + tid; j < top_k; j += 256) o[j] = -1;
  if (tid == 0) kept_counts[blockIdx.x] = k;
}

}  // namespace fdattn

using namespace fdattn;

extern "C" size_t fdattn_sqattn_workspace_bytes(int batch, int hkv, int max_blocks_per_seq) {
  if (batch <= 0 || hkv <= 0 || max_blocks_per_seq <= 0) return 256;
  size_t n = (size_t)batch * hkv * max_blocks_per_seq * sizeof(double);
  return (n + 255) & ~(size_t)255;
}

extern "C" int fdattn_sqattn_select(const void* q, const void* key_cache, const float* cache_k_scale,
                                    const int32_t* block_tables, const int32_t* seq_lens_decoder,
                                    const int32_t* seq_lens_this_time, float* scores, int32_t* kept_blocks,
                                    int32_t* kept_counts, void* workspace, size_t workspace_bytes, int batch,
                                    int hq, int hkv, int head_dim, int block_size, int max_blocks_per_seq,
                                    int num_blocks, int top_k, int cache_quant_type, void* stream) {
  if (!q || !key_cache || !cache_k_scale || !block_tables || !seq_lens_decoder || !kept_blocks ||
      !kept_counts || !workspace)
    return fail(FDATTN_ERR_NULL, "fdattn_sqattn_select: a required pointer is NULL");
  if (batch <= 0 || hq <= 0 || hkv <= 0 || hq % hkv != 0 || hq / hkv > kSelMaxG || head_dim <= 0 ||
      head_dim % 4 != 0 || head_dim > kSelMaxD || block_size <= 0 || max_blocks_per_seq <= 0 ||
      max_blocks_per_seq > 4096 || num_blocks <= 0 || top_k <= 0 || batch > 65535)
    return fail(FDATTN_ERR_SHAPE,
                "fdattn_sqattn_select: unsupported shape batch=%d hq=%d hkv=%d head_dim=%d block_size=%d "
                "max_blocks=%d top_k=%d (group <= %d, head_dim <= %d multiple of 4, max_blocks <= 4096)",
                batch, hq, hkv, head_dim, block_size, max_blocks_per_seq, top_k, kSelMaxG, kSelMaxD);
  if (cache_quant_type != FDATTN_CACHE_INT8 && cache_quant_type != FDATTN_CACHE_FP8_E4M3)
    return fail(FDATTN_ERR_QUANT, "fdattn_sqattn_select: unknown cache_quant_type %d", cache_quant_type);
  const size_t need = (size_t)batch * hkv * max_blocks_per_seq * sizeof(double);
  if (workspace_bytes < need)
    return fail(FDATTN_ERR_WORKSPACE, "fdattn_sqattn_select: workspace %zu B < required %zu B", workspace_bytes, need);
  hipStream_t s = (hipStream_t)stream;
  ScoreArgs a{(const uint16_t*)q, (const uint8_t*)key_cache, cache_k_scale, block_tables, seq_lens_decoder,
              seq_lens_this_time, (double*)workspace, scores, batch, hq, hkv, head_dim, block_size,
              max_blocks_per_seq, num_blocks};
  dim3 grid(max_blocks_per_seq, hkv, batch);
  if (cache_quant_type == FDATTN_CACHE_INT8)
    hipLaunchKernelGGL(sqattn_block_scores_kernel<FDATTN_CACHE_INT8>, grid, dim3(64), 0, s, a);
  else
    hipLaunchKernelGGL(sqattn_block_scores_kernel<FDATTN_CACHE_FP8_E4M3>, grid, dim3(64), 0, s, a);
  int rc = check_launch("fdattn_sqattn_select (scores)");
  if (rc) return rc;
  const size_t shm = (size_t)max_blocks_per_seq * (sizeof(double) + sizeof(int));
  hipLaunchKernelGGL(sqattn_topk_kernel, dim3(batch * hkv), dim3(256), shm, s, (const double*)workspace,
                     seq_lens_decoder, seq_lens_this_time, kept_blocks, kept_counts, hkv, block_size,
                     max_blocks_per_seq, top_k);
  return check_launch("fdattn_sqattn_select (top-k)");
}
