// Chunked-prefill ("append") attention.
#include "launch.h"
#include "prefill.h"

namespace fdattn {

constexpr int kPfMaxD = 256;

template <int QUANT>
__device__ __forceinline__ float pdq(u32 byte) {
  if (QUANT == FDATTN_CACHE_INT8) return (float)(int)(int8_t)byte;
  return e4m3_to_f32(byte);
}

// Shape-agnostic kernel: one wavefront per (new token, query head); lanes own keys for
// q.K and channels for P.V.  Keys [0, p) come from the quantised pages, keys [p, p+ci]
// from the chunk's bf16 K/V.
// DYN: cache scales per stored row ([num_blocks, hkv, bs]) instead of per channel.
template <int QUANT, bool DYN>
__global__ __launch_bounds__(64) void prefill_generic_kernel(PrefillArgs a) {
  __shared__ float qf[kPfMaxD];
  __shared__ float pbuf[64];
  const int lane = threadIdx.x, tok = blockIdx.x, qh = blockIdx.y;
  const int d = a.d, bs = a.bs, g = a.hq / a.hkv, h = qh / g;
  int lo = 0, hi = a.batch;
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (a.cu_seqlens_q[mid] <= tok) lo = mid; else hi = mid;
  }
  const int b = lo;
  if (tok >= a.cu_seqlens_q[b + 1]) return;
  if (a.seq_lens_encoder && a.seq_lens_encoder[b] <= 0) return;  // a decode row or an idle slot of a mixed batch
  const int ci = tok - a.cu_seqlens_q[b], p = a.seq_lens_decoder[b];
  const int nkeys = p + ci + 1;
  for (int c = lane; c < d; c += 64) qf[c] = bf16_to_f32(a.q[((size_t)tok * a.hq + qh) * d + c]) * a.sm_scale;
  __syncthreads();
  const float* ks = a.k_scale + h * d;
  const float* vs = a.v_scale + h * d;
  const int32_t* table = a.block_tables + (size_t)b * a.max_blocks;
  float m = -INFINITY, l = 0.f;
  float acc[kPfMaxD / 64] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < nkeys; k0 += 64) {
    const int kk = k0 + lane;
    const bool valid = kk < nkeys;
    float s = -INFINITY;
    if (valid) {
      s = 0.f;
      if (kk < p) {
        const int pb = table[kk / bs];
        const uint8_t* kr = a.key_cache + (((size_t)pb * a.hkv + h) * bs + kk % bs) * d;
        if (DYN) {
          for (int c = 0; c < d; c += 4) {
            const u32 w = *reinterpret_cast<const u32*>(kr + c);
            s += qf[c] * pdq<QUANT>(w & 0xff) + qf[c + 1] * pdq<QUANT>((w >> 8) & 0xff) +
                 qf[c + 2] * pdq<QUANT>((w >> 16) & 0xff) + qf[c + 3] * pdq<QUANT>(w >> 24);
          }
          s *= a.k_scale[((size_t)pb * a.hkv + h) * bs + kk % bs];
        } else {
          for (int c = 0; c < d; c += 4) {
            const u32 w = *reinterpret_cast<const u32*>(kr + c);
            s += qf[c] * (pdq<QUANT>(w & 0xff) * ks[c]) + qf[c + 1] * (pdq<QUANT>((w >> 8) & 0xff) * ks[c + 1]) +
                 qf[c + 2] * (pdq<QUANT>((w >> 16) & 0xff) * ks[c + 2]) + qf[c + 3] * (pdq<QUANT>(w >> 24) * ks[c + 3]);
          }
        }
      } else {
        const uint16_t* kr = a.k_new + ((size_t)(a.cu_seqlens_q[b] + kk - p) * a.hkv + h) * d;
        for (int c = 0; c < d; c += 2) {
          const u32 w = *reinterpret_cast<const u32*>(kr + c);
          s += qf[c] * bf16lo_to_f32(w) + qf[c + 1] * bf16hi_to_f32(w);
        }
      }
    }
    const float mb = wave_max(s);
    const float m_new = fmaxf(m, mb);
    const float alpha = (m == -INFINITY) ? 0.f : __expf(m - m_new);
    const float pr = valid ? __expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(pr);
    m = m_new;
    __syncthreads();
    pbuf[lane] = pr;
    __syncthreads();
    const int nt = min(64, nkeys - k0);
#pragma unroll
    for (int i = 0; i < kPfMaxD / 64; ++i) {
      const int c = lane + 64 * i;
      if (c < d) {
        float o = acc[i] * alpha;
        for (int tt = 0; tt < nt; ++tt) {
          const int kk2 = k0 + tt;
          float v;
          if (kk2 < p) {
            const int pb = table[kk2 / bs];
            v = pdq<QUANT>(a.value_cache[(((size_t)pb * a.hkv + h) * bs + kk2 % bs) * d + c]) *
                (DYN ? a.v_scale[((size_t)pb * a.hkv + h) * bs + kk2 % bs] : vs[c]);
          } else {
            v = bf16_to_f32(a.v_new[((size_t)(a.cu_seqlens_q[b] + kk2 - p) * a.hkv + h) * d + c]);
          }
          o += pbuf[tt] * v;
        }
        acc[i] = o;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < kPfMaxD / 64; ++i) {
    const int c = lane + 64 * i;
    if (c < d) a.out[((size_t)tok * a.hq + qh) * d + c] = f32_to_bf16(acc[i] / l);
  }
}

int prefill_launch(const void* q, const void* k_new, const void* v_new, const void* key_cache,
                   const void* value_cache, const float* cache_k_scale, const float* cache_v_scale,
                   const int32_t* block_tables, const int32_t* seq_lens_decoder, const int32_t* cu_seqlens_q,
                   const int32_t* seq_lens_encoder, void* out, int num_tokens, int batch, int max_chunk, int hq,
                   int hkv, int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
                   int cache_quant_type, float softmax_scale, hipStream_t s, bool force_generic, void* workspace,
                   size_t workspace_bytes, int n_splits, int rows_hint) {
  if (!q || !k_new || !v_new || !key_cache || !value_cache || !cache_k_scale || !cache_v_scale ||
      !block_tables || !seq_lens_decoder || !cu_seqlens_q || !out)
    return fail(FDATTN_ERR_NULL, "fdattn_append_attention_prefill: a required pointer is NULL");
  if (num_tokens < 0 || batch <= 0 || max_chunk <= 0 || hq <= 0 || hkv <= 0 || hq % hkv != 0 ||
      head_dim <= 0 || head_dim % 4 != 0 || head_dim > kPfMaxD || block_size <= 0 ||
      max_blocks_per_seq <= 0 || num_blocks <= 0 || hq > 65535)
    return fail(FDATTN_ERR_SHAPE,
                "fdattn_append_attention_prefill: unsupported shape tokens=%d batch=%d max_chunk=%d hq=%d hkv=%d "
                "head_dim=%d block_size=%d", num_tokens, batch, max_chunk, hq, hkv, head_dim, block_size);
  if (!quant_known(cache_quant_type))
    return fail(FDATTN_ERR_QUANT, "fdattn_append_attention_prefill: unknown cache_quant_type %d", cache_quant_type);
  if (num_tokens == 0) return 0;
  PrefillArgs a{(const uint16_t*)q, (const uint16_t*)k_new, (const uint16_t*)v_new, (const uint8_t*)key_cache,
                (const uint8_t*)value_cache, cache_k_scale, cache_v_scale, block_tables, seq_lens_decoder,
                cu_seqlens_q, seq_lens_encoder, (uint16_t*)out, num_tokens, batch, hq, hkv, head_dim, block_size,
                max_blocks_per_seq, num_blocks, softmax_scale};
  if (!force_generic && prefill_mfma_supported(hq, hkv, head_dim, block_size, cache_quant_type))
    return prefill_mfma_launch(a, max_chunk, cache_quant_type, s, workspace, workspace_bytes, n_splits, rows_hint);
  const dim3 grid(num_tokens, hq);
  if (cache_quant_type == FDATTN_CACHE_INT8)
    hipLaunchKernelGGL((prefill_generic_kernel<FDATTN_CACHE_INT8, false>), grid, dim3(64), 0, s, a);
  else if (cache_quant_type == FDATTN_CACHE_FP8_E4M3)
    hipLaunchKernelGGL((prefill_generic_kernel<FDATTN_CACHE_FP8_E4M3, false>), grid, dim3(64), 0, s, a);
  else if (cache_quant_type == FDATTN_CACHE_INT8_DYNAMIC)
    hipLaunchKernelGGL((prefill_generic_kernel<FDATTN_CACHE_INT8, true>), grid, dim3(64), 0, s, a);
  else
    hipLaunchKernelGGL((prefill_generic_kernel<FDATTN_CACHE_FP8_E4M3, true>), grid, dim3(64), 0, s, a);
  return check_launch("fdattn_append_attention_prefill");
}

}  // namespace fdattn

using namespace fdattn;

extern "C" int fdattn_append_attention_prefill(
    const void* q, const void* k_new, const void* v_new, const void* key_cache, const void* value_cache,
    const float* cache_k_scale, const float* cache_v_scale, const int32_t* block_tables,
    const int32_t* seq_lens_decoder, const int32_t* cu_seqlens_q, void* out, int num_tokens, int batch,
    int max_chunk, int hq, int hkv, int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
    int cache_quant_type, float softmax_scale, void* stream) {
  return prefill_launch(q, k_new, v_new, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                        seq_lens_decoder, cu_seqlens_q, nullptr, out, num_tokens, batch, max_chunk, hq, hkv,
                        head_dim, block_size, max_blocks_per_seq, num_blocks, cache_quant_type, softmax_scale,
                        (hipStream_t)stream, false, nullptr, 0, 1);
}

extern "C" int fdattn_prefill_auto_splits(int rows, int hq, int max_chunk) { return prefill_auto_splits(rows, hq, max_chunk); }
extern "C" int fdattn_prefill_auto_splits_for(int rows, int hq, int hkv, int max_chunk) {
  return prefill_auto_splits(rows, hq, max_chunk, hkv);
}

extern "C" size_t fdattn_append_attention_prefill_split_workspace_bytes(int num_tokens, int hq, int num_splits) {
  return prefill_split_workspace_bytes(num_tokens, hq, num_splits);
}

extern "C" int fdattn_append_attention_prefill_split(
    const void* q, const void* k_new, const void* v_new, const void* key_cache, const void* value_cache,
    const float* cache_k_scale, const float* cache_v_scale, const int32_t* block_tables,
    const int32_t* seq_lens_decoder, const int32_t* cu_seqlens_q, void* out, void* workspace, size_t workspace_bytes,
    int num_splits, int num_tokens, int batch, int max_chunk, int hq, int hkv, int head_dim, int block_size,
    int max_blocks_per_seq, int num_blocks, int cache_quant_type, float softmax_scale, void* stream) {
  if (num_splits < 1) return fail(FDATTN_ERR_SHAPE, "fdattn_append_attention_prefill_split: num_splits %d < 1", num_splits);
  if (num_splits > 1 && (!workspace || workspace_bytes < prefill_split_workspace_bytes(num_tokens, hq, num_splits)))
    return fail(FDATTN_ERR_WORKSPACE, "fdattn_append_attention_prefill_split: workspace %zu B < required %zu B",
                workspace_bytes, prefill_split_workspace_bytes(num_tokens, hq, num_splits));
  return prefill_launch(q, k_new, v_new, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                        seq_lens_decoder, cu_seqlens_q, nullptr, out, num_tokens, batch, max_chunk, hq, hkv,
                        head_dim, block_size, max_blocks_per_seq, num_blocks, cache_quant_type, softmax_scale,
                        (hipStream_t)stream, false, workspace, workspace_bytes, num_splits);
}

extern "C" int fdattn_append_attention_prefill_generic(
    const void* q, const void* k_new, const void* v_new, const void* key_cache, const void* value_cache,
    const float* cache_k_scale, const float* cache_v_scale, const int32_t* block_tables,
    const int32_t* seq_lens_decoder, const int32_t* cu_seqlens_q, void* out, int num_tokens, int batch,
    int max_chunk, int hq, int hkv, int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
    int cache_quant_type, float softmax_scale, void* stream) {
  return prefill_launch(q, k_new, v_new, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                        seq_lens_decoder, cu_seqlens_q, nullptr, out, num_tokens, batch, max_chunk, hq, hkv,
                        head_dim, block_size, max_blocks_per_seq, num_blocks, cache_quant_type, softmax_scale,
                        (hipStream_t)stream, true, nullptr, 0, 1);
}
