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

// Shape-agnostic kernel: one wavefront per (group of new tokens, KV head, set of its query heads): its 8 rows are
// (token, head) pairs - row v is token v / gs of the group, head v % gs of the set, gs = min(heads per KV head, 8) -
// so every K and V row it reads serves up to 8 query rows.  Scores: lane = key of a group of 64; P.V: lane = four
// channels of one of the 64 / (d/4) key rows read at a time.  Keys [0, p) come from the quantised pages, keys
// [p, p + ci] from the chunk's bf16 K/V.  The grid has one workgroup per token: those that do not lead a group leave.
// DYN: cache scales per stored row ([num_blocks, hkv, bs]) instead of per channel.
constexpr int kPfRows = 8;

template <int QUANT, bool DYN>
__global__ __launch_bounds__(64) void prefill_generic_kernel(PrefillArgs a) {
  __shared__ __attribute__((aligned(16))) float qc[kPfRows][kPfMaxD];  // q * softmax_scale * k_scale: against cache bytes
  __shared__ __attribute__((aligned(16))) float qn[kPfRows][kPfMaxD];  // q * softmax_scale: against the chunk's bf16 K
  __shared__ float pbuf[kPfRows][64];
  __shared__ int krow[64];  // where key k0 + i lives: a row of the caches (>= 0) or ~(a row of k_new / v_new)
  const int lane = threadIdx.x, tok = blockIdx.x;
  const int d = a.d, bs = a.bs, g = a.hq / a.hkv;
  const int gs = min(g, kPfRows), tw = kPfRows / gs, sets = (g + gs - 1) / gs;  // heads per set, tokens per group
  const int h = blockIdx.y / sets, g0 = (blockIdx.y - h * sets) * gs;
  int lo = 0, hi = a.batch;
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (a.cu_seqlens_q[mid] <= tok) lo = mid; else hi = mid;
  }
  const int b = lo;
  const int tok0 = a.cu_seqlens_q[b], tok1 = a.cu_seqlens_q[b + 1];
  if (tok >= tok1) return;
  if (a.seq_lens_encoder && a.seq_lens_encoder[b] <= 0) return;  // a decode row or an idle slot of a mixed batch
  const int ci = tok - tok0, p = a.seq_lens_decoder[b];
  if (ci % tw != 0) return;                 // not the first token of its group
  const int nt = min(tw, tok1 - tok);       // tokens of this group
  // row v: token ci + v / gs, head g0 + v % gs; live if both exist
  auto row_tok = [&](int v) { return v / gs; };
  auto row_live = [&](int v) { return v / gs < nt && g0 + v % gs < g; };
  for (int i = lane; i < kPfRows * d; i += 64) {
    const int v = i / d, c = i - v * d;
    float x = 0.f;  // rows that do not exist are zero, so that the loops below need no test
    if (row_live(v)) x = bf16_to_f32(a.q[((size_t)(tok + row_tok(v)) * a.hq + h * g + g0 + v % gs) * d + c]) * a.sm_scale;
    qn[v][c] = x;
    qc[v][c] = DYN ? x : x * a.k_scale[h * d + c];
  }
  __syncthreads();
  const int32_t* table = a.block_tables + (size_t)b * a.max_blocks;
  const int nkeys = p + ci + nt;            // keys the group's last token sees

  // P.V layout: lanes_per_row lanes cover a row's d channels, 4 each; rows_per_pass rows at a time
  const int lanes_per_row = d / 4, rows_per_pass = 64 / lanes_per_row;
  const int vslot = lane / lanes_per_row, c4 = 4 * (lane - vslot * lanes_per_row);
  const bool vlane = vslot < rows_per_pass;
  float vs4[4] = {1.f, 1.f, 1.f, 1.f};      // this lane's channels' V scales (per-channel formats)
  if (!DYN && vlane) {
#pragma unroll
    for (int e = 0; e < 4; ++e) vs4[e] = a.v_scale[h * d + c4 + e];
  }

  float m[kPfRows], l[kPfRows], acc[kPfRows][4];
  int fewer[kPfRows];  // row v sees this many keys fewer than the group's last token
#pragma unroll
  for (int v = 0; v < kPfRows; ++v) {
    m[v] = -INFINITY, l[v] = 0.f;
    acc[v][0] = acc[v][1] = acc[v][2] = acc[v][3] = 0.f;
    fewer[v] = max(nt - 1 - row_tok(v), 0);
  }

  // where key kk lives: a row of the caches (>= 0) or ~(a row of k_new / v_new)
  auto locate = [&](int kk) {
    if (kk >= nkeys) return 0;
    if (kk >= p) return ~(int)((size_t)(tok0 + kk - p) * a.hkv + h);
    const int lb = kk / bs;
    int pb = table[lb];
    pb = (pb >= 0 && pb < a.num_blocks) ? pb : 0;  // a table entry that names no block: read block 0, fault nothing
    return (int)(((size_t)pb * a.hkv + h) * bs + (kk - lb * bs));
  };
  int where_next = locate(lane);
  for (int k0 = 0; k0 < nkeys; k0 += 64) {
    const int kk = k0 + lane;
    const bool valid = kk < nkeys;
    const int where = where_next;
    where_next = locate(kk + 64);  // the table entry of the next group's key: a round trip hidden behind this group
    __syncthreads();  // the previous group's P.V has read krow and pbuf
    krow[lane] = where;
    float s[kPfRows];
#pragma unroll
    for (int v = 0; v < kPfRows; ++v) s[v] = 0.f;
    float ksc = 1.0f;
    if (valid && where >= 0) {
      const uint8_t* kr = a.key_cache + (size_t)where * d;
      auto word = [&](u32 w, int c) {  // four channels of the row against every query row
        const float k0f = pdq<QUANT>(w & 0xff), k1f = pdq<QUANT>((w >> 8) & 0xff), k2f = pdq<QUANT>((w >> 16) & 0xff),
                    k3f = pdq<QUANT>(w >> 24);
#pragma unroll
        for (int v = 0; v < kPfRows; ++v) {
          const float4 qv = *reinterpret_cast<const float4*>(&qc[v][c]);
          s[v] += qv.x * k0f + qv.y * k1f + qv.z * k2f + qv.w * k3f;
        }
      };
      int c = 0;
      const int d16 = (d & 15) ? 0 : d;  // 16-byte words only where every row starts on one
      for (; c < d16; c += 16) {
        const uint4 w = *reinterpret_cast<const uint4*>(kr + c);
        word(w.x, c), word(w.y, c + 4), word(w.z, c + 8), word(w.w, c + 12);
      }
      for (; c < d; c += 4) word(*reinterpret_cast<const u32*>(kr + c), c);
      if (DYN) ksc = a.k_scale[where];
    } else if (valid) {
      const uint16_t* kr = a.k_new + (size_t)(~where) * d;
      for (int c = 0; c < d; c += 4) {
        const uint2 w = *reinterpret_cast<const uint2*>(kr + c);
        const float k0f = bf16lo_to_f32(w.x), k1f = bf16hi_to_f32(w.x), k2f = bf16lo_to_f32(w.y), k3f = bf16hi_to_f32(w.y);
#pragma unroll
        for (int v = 0; v < kPfRows; ++v) {
          const float4 qv = *reinterpret_cast<const float4*>(&qn[v][c]);
          s[v] += qv.x * k0f + qv.y * k1f + qv.z * k2f + qv.w * k3f;
        }
      }
    }
    // Softmax weights against a per-row reference that is raised only when a score outgrows it by more than 2^10
    // (one ballot per row and group instead of a maximum over the wavefront; the weights stay below e^10); the
    // weight sums stay per lane until the end.
#pragma unroll
    for (int v = 0; v < kPfRows; ++v) {
      const bool sees = kk < nkeys - fewer[v];
      const float sv = sees ? s[v] * ksc : -INFINITY;
      if (__any(sees && !(sv <= m[v] + 10.0f))) {  // also the row's first keys (m = -inf) and NaN scores
        const float m_new = fmaxf(m[v], wave_max(sv));
        const float al = (m[v] == -INFINITY) ? 0.f : __expf(m[v] - m_new);
        l[v] *= al;
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[v][e] *= al;
        m[v] = m_new;
      }
      const float pr = sees ? __expf(sv - m[v]) : 0.f;
      l[v] += pr;
      pbuf[v][lane] = pr;
    }
    __syncthreads();
    const int ng = min(64, nkeys - k0);
    const int nc = min(max(p - k0, 0), ng);  // keys [0, nc) of the group are cache rows, [nc, ng) the chunk's
    if (vlane) {
      auto add = [&](int tt, float v0, float v1, float v2, float v3) {
#pragma unroll
        for (int v = 0; v < kPfRows; ++v) {
          const float pw = pbuf[v][tt];
          acc[v][0] += pw * v0, acc[v][1] += pw * v1, acc[v][2] += pw * v2, acc[v][3] += pw * v3;
        }
      };
      auto add_cache = [&](int tt, u32 w, float rs) {
        add(tt, pdq<QUANT>(w & 0xff) * (vs4[0] * rs), pdq<QUANT>((w >> 8) & 0xff) * (vs4[1] * rs),
            pdq<QUANT>((w >> 16) & 0xff) * (vs4[2] * rs), pdq<QUANT>(w >> 24) * (vs4[3] * rs));
      };
      auto add_chunk = [&](int tt, uint2 w) {
        add(tt, bf16lo_to_f32(w.x), bf16hi_to_f32(w.x), bf16lo_to_f32(w.y), bf16hi_to_f32(w.y));
      };
      const int rp = rows_per_pass;
      int tt = vslot;
      // four rows' loads in flight at a time (a load per iteration would pay a round trip to memory each)
      for (; tt + 3 * rp < nc; tt += 4 * rp) {
        u32 w[4];
        float rs[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int wh = krow[tt + e * rp];
          w[e] = *reinterpret_cast<const u32*>(a.value_cache + (size_t)wh * d + c4);
          rs[e] = DYN ? a.v_scale[wh] : 1.0f;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) add_cache(tt + e * rp, w[e], rs[e]);
      }
      for (; tt < nc; tt += rp) {
        const int wh = krow[tt];
        add_cache(tt, *reinterpret_cast<const u32*>(a.value_cache + (size_t)wh * d + c4), DYN ? a.v_scale[wh] : 1.0f);
      }
      for (; tt + 3 * rp < ng; tt += 4 * rp) {
        uint2 w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = *reinterpret_cast<const uint2*>(a.v_new + (size_t)(~krow[tt + e * rp]) * d + c4);
#pragma unroll
        for (int e = 0; e < 4; ++e) add_chunk(tt + e * rp, w[e]);
      }
      for (; tt < ng; tt += rp) add_chunk(tt, *reinterpret_cast<const uint2*>(a.v_new + (size_t)(~krow[tt]) * d + c4));
    }
  }
  // the row slots' sums meet in LDS (q is no longer needed), one slot after the other
  __syncthreads();
  for (int sl = 0; sl < rows_per_pass; ++sl) {
    if (vlane && vslot == sl) {
#pragma unroll
      for (int v = 0; v < kPfRows; ++v)
#pragma unroll
        for (int e = 0; e < 4; ++e) qc[v][c4 + e] = (sl == 0 ? 0.f : qc[v][c4 + e]) + acc[v][e];
    }
    __syncthreads();
  }
#pragma unroll
  for (int v = 0; v < kPfRows; ++v) {
    if (!row_live(v)) continue;
    uint16_t* o = a.out + ((size_t)(tok + row_tok(v)) * a.hq + h * g + g0 + v % gs) * d;
    const float inv = 1.0f / wave_sum(l[v]);
    for (int c = lane; c < d; c += 64) o[c] = f32_to_bf16(qc[v][c] * inv);
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
  if ((size_t)num_blocks * hkv * block_size > 0x7fffffffull || (size_t)num_tokens * hkv > 0x7fffffffull)
    return fail(FDATTN_ERR_SHAPE, "fdattn_append_attention_prefill: more than 2^31 cache rows (shape-agnostic kernel)");
  const int gs = hq / hkv < kPfRows ? hq / hkv : kPfRows;  // query heads of a KV head a workgroup serves
  const dim3 grid(num_tokens, hkv * ((hq / hkv + gs - 1) / gs));
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
