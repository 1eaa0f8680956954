// One attention step of a mixed batch - prefill rows, decode rows and idle slots together:
// cache write for every new token, decode attention for the decode rows, append attention
// for the prefill rows.  Nothing is gathered or synchronised: the kernels find their rows
// through cu_seqlens_q / seq_lens_encoder on the device.
#include "decode_generic.h"
#include "launch.h"

namespace fdattn {

static size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

struct StepWorkspace {
  size_t q_rot, k_new, v_new, decode, select, kept, split, view, total;  // byte offsets of the parts, and the sum
};

// The arrays of the token-as-row view of a step (fdattn_step_extras.sqattn_per_token): per view row a table row, then
// cu_seqlens_q (rows + 1), seq_lens_encoder, seq_lens_decoder and seq_lens_this_time of the view.
static size_t view_bytes(int rows, int max_blocks) { return ((size_t)rows * ((size_t)max_blocks + 4) + 1) * sizeof(int32_t); }

// Every token of a decode row as a row of its own: view row r = sequence r / T, token r % T.  Its table row repeats the
// sequence's, its cached length ends in front of that token and it brings one token, so the kernels behind see the
// step's decode tokens as so many decode rows of one token - which is what "every token selects its own blocks" means.
// Rows of tokens that a sequence does not have, and the rows of sequences that are no decode rows of this step, carry
// seq_lens_encoder 1: the decode-side kernels pass them over.
__global__ __launch_bounds__(256) void rows_per_token_kernel(const int32_t* cu, const int32_t* enc, const int32_t* dec,
                                                             const int32_t* tables, int batch, int T, int max_blocks,
                                                             int32_t* tables_v, int32_t* cu_v, int32_t* enc_v,
                                                             int32_t* dec_v, int32_t* this_v) {
  const int r = blockIdx.x, b = r / T, j = r - b * T;
  const int c0 = cu[b], n = cu[b + 1] - c0;
  const bool valid = enc[b] == 0 && j < n && n <= T;
  if (threadIdx.x == 0) {
    cu_v[r] = c0 + min(j, n);
    if (r == 0) cu_v[batch * T] = cu[batch];
    enc_v[r] = valid ? 0 : 1;
    dec_v[r] = dec[b] + j;
    this_v[r] = 1;
  }
  for (int i = threadIdx.x; i < max_blocks; i += 256)
    tables_v[(size_t)r * max_blocks + i] = valid ? tables[(size_t)b * max_blocks + i] : -1;
}

static StepWorkspace step_workspace(int num_tokens, int batch, int hq, int hkv, int d, int max_blocks, int prefill_splits) {
  StepWorkspace w;
  w.q_rot = 0;
  w.k_new = w.q_rot + align256((size_t)num_tokens * hq * d * 2);
  w.v_new = w.k_new + align256((size_t)num_tokens * hkv * d * 2);
  w.decode = w.v_new + align256((size_t)num_tokens * hkv * d * 2);
  // the block selector's scores and bounds, then its result (kept blocks - at most every block - and counts)
  // (decode partials: room for 16 rows per KV head, which decode rows of several tokens may use)
  size_t dec = fdattn_decode_workspace_bytes(batch, hq, hkv, d, max_blocks);
  if (hq % hkv == 0 && hq / hkv <= 8) {
    const size_t spec = c8_workspace_bytes(batch, hkv, max_blocks, 16);
    if (spec > dec) dec = spec;
  }
  w.select = w.decode + align256(dec);
  w.kept = w.select + align256(fdattn_sqattn_workspace_bytes(batch, hkv, max_blocks));
  w.split = w.kept + align256((size_t)batch * hkv * ((size_t)max_blocks + 1) * sizeof(int32_t));
  w.view = w.split + align256(prefill_split_workspace_bytes(num_tokens, hq, prefill_splits));
  w.total = w.view + align256(view_bytes(batch, max_blocks));
  return w;
}

}  // namespace fdattn

using namespace fdattn;

extern "C" size_t fdattn_append_attention_workspace_bytes(int num_tokens, int batch, int hq, int hkv, int head_dim,
                                                          int max_blocks_per_seq) {
  return fdattn_append_attention_workspace_bytes_ex(num_tokens, batch, hq, hkv, head_dim, max_blocks_per_seq, 1);
}

extern "C" size_t fdattn_append_attention_workspace_bytes_ex(int num_tokens, int batch, int hq, int hkv, int head_dim,
                                                             int max_blocks_per_seq, int prefill_splits) {
  if (num_tokens < 0 || batch <= 0 || hq <= 0 || hkv <= 0 || head_dim <= 0 || max_blocks_per_seq <= 0) return 256;
  return step_workspace(num_tokens, batch, hq, hkv, head_dim, max_blocks_per_seq, prefill_splits).total;
}

extern "C" int fdattn_append_attention(
    const void* qkv, void* key_cache, void* value_cache, float* cache_k_scale, float* cache_v_scale,
    const float* rope_cos, const float* rope_sin, const int32_t* block_tables, const int32_t* seq_lens_encoder,
    const int32_t* seq_lens_decoder, const int32_t* seq_lens_this_time, const int32_t* cu_seqlens_q, void* out,
    void* workspace, size_t workspace_bytes, int num_tokens, int batch, int max_chunk, int hq, int hkv,
    int head_dim, int block_size, int max_blocks_per_seq, int num_blocks, int max_pos, int rope_style,
    int cache_quant_type, float softmax_scale, void* stream) {
  return fdattn_append_attention_ex(qkv, key_cache, value_cache, cache_k_scale, cache_v_scale, rope_cos, rope_sin,
                                    block_tables, seq_lens_encoder, seq_lens_decoder, seq_lens_this_time, cu_seqlens_q,
                                    out, workspace, workspace_bytes, num_tokens, batch, max_chunk, hq, hkv, head_dim,
                                    block_size, max_blocks_per_seq, num_blocks, max_pos, rope_style, cache_quant_type,
                                    softmax_scale, nullptr, stream);
}

extern "C" int fdattn_append_attention_ex(
    const void* qkv, void* key_cache, void* value_cache, float* cache_k_scale, float* cache_v_scale,
    const float* rope_cos, const float* rope_sin, const int32_t* block_tables, const int32_t* seq_lens_encoder,
    const int32_t* seq_lens_decoder, const int32_t* seq_lens_this_time, const int32_t* cu_seqlens_q, void* out,
    void* workspace, size_t workspace_bytes, int num_tokens, int batch, int max_chunk, int hq, int hkv,
    int head_dim, int block_size, int max_blocks_per_seq, int num_blocks, int max_pos, int rope_style,
    int cache_quant_type, float softmax_scale,
    const fdattn_step_extras* extras, void* stream) {
  if (!seq_lens_encoder || !seq_lens_this_time || !cu_seqlens_q || !out || !workspace)
    return fail(FDATTN_ERR_NULL, "fdattn_append_attention: a required pointer is NULL");
  if (num_tokens < 0 || batch <= 0 || max_chunk < 0 || hq <= 0 || hkv <= 0 || head_dim <= 0 ||
      max_blocks_per_seq <= 0)
    return fail(FDATTN_ERR_SHAPE, "fdattn_append_attention: bad shape tokens=%d batch=%d max_chunk=%d hq=%d hkv=%d "
                "head_dim=%d max_blocks=%d", num_tokens, batch, max_chunk, hq, hkv, head_dim, max_blocks_per_seq);
  if (num_tokens == 0) return 0;
  // key splits for the prefill rows: from the host's count of them; without one, the most a single prefill row would
  // use - the prefill kernel then counts the rows itself and uses what that many need (the grid and the partials are
  // laid out for the most)
  const int prefill_rows = extras && extras->prefill_rows > 0 ? extras->prefill_rows : 0;
  int splits = max_chunk > 0 ? prefill_auto_splits(prefill_rows > 0 ? prefill_rows : 1, hq, max_chunk, hkv) : 1;
  const int top_k = extras && extras->sqattn_top_k > 0 ? (extras->sqattn_top_k < max_blocks_per_seq ? extras->sqattn_top_k : max_blocks_per_seq) : 0;
  const int decode_tokens = extras && extras->decode_tokens > 1 ? extras->decode_tokens : 1;
  // every token of a decode row with a block list of its own: the decode side of the step runs over the token-as-row
  // view, whose batch is what the workspace must be sized for
  const bool per_token = top_k > 0 && decode_tokens > 1 && extras->sqattn_per_token != 0;
  if (per_token && (long long)batch * decode_tokens * hkv > (1LL << 20))  // (the decode launchers' limit on (row, KV head) pairs)
    return fail(FDATTN_ERR_SHAPE, "fdattn_append_attention: sqattn_per_token: batch %d x decode_tokens %d x %d KV heads "
                "exceeds %d rows", batch, decode_tokens, hkv, 1 << 20);
  const int dbatch = per_token ? batch * decode_tokens : batch;
  StepWorkspace w = step_workspace(num_tokens, dbatch, hq, hkv, head_dim, max_blocks_per_seq, splits);
  while (splits > 1 && workspace_bytes < w.total)  // a workspace sized for fewer splits: use as many as it holds
    w = step_workspace(num_tokens, dbatch, hq, hkv, head_dim, max_blocks_per_seq, --splits);
  if (workspace_bytes < w.total)
    return fail(FDATTN_ERR_WORKSPACE, "fdattn_append_attention: workspace %zu B < required %zu B%s", workspace_bytes,
                w.total, per_token ? " (sqattn_per_token: size it for batch x decode_tokens sequences)" : "");
  // what the decode rows ask for, checked before anything is written
  const bool c8 = c8_supported(hq, hkv, head_dim, block_size, cache_quant_type);
  if (decode_tokens > 1 && !per_token && ((!c8 && !decode_tiles_supported(hq, hkv, head_dim)) || hq % hkv != 0 ||
                                          decode_tokens * (hq / hkv) > 16))
    return fail(FDATTN_ERR_SHAPE, "fdattn_append_attention: decode_tokens %d needs head_dim 64, 128 or 256 and "
                "decode_tokens x query heads per KV head <= 16", decode_tokens);
  // block-sparse decode rows: the MFMA selector and the int8-MFMA kernel at their shapes; elsewhere the exact (fp64)
  // selector and the kernels of the other shapes, for rows of one token
  const bool sel_fast = c8 && sqattn_fast_supported(hq, hkv, head_dim, block_size, max_blocks_per_seq);
  if (top_k > 0 && !sel_fast && ((decode_tokens > 1 && !per_token) || hq % hkv != 0 || hq / hkv > 8 || head_dim > 256 || head_dim % 4 != 0 ||
                                 max_blocks_per_seq > 4096))
    return fail(FDATTN_ERR_SHAPE, "fdattn_append_attention: sqattn_top_k needs at most 8 query heads per KV head, head_dim "
                "<= 256 and at most 4096 blocks per sequence (with decode_tokens and one list per row: head_dim 128, "
                "block_size 64, at most 2048 blocks)");
  char* ws = (char*)workspace;
  void* q_rot = ws + w.q_rot;
  const bool any_prefill = max_chunk > 0;  // the caller's word: 0 = no sequence has seq_lens_encoder > 0
  void* k_new = any_prefill ? ws + w.k_new : nullptr;
  void* v_new = any_prefill ? ws + w.v_new : nullptr;
  // 1. every new token: rotate, quantise, store (argument checks of the shared kind happen here)
  int rc = fdattn_write_cache_kv_ex(qkv, q_rot, k_new, v_new, key_cache, value_cache, cache_k_scale, cache_v_scale,
                                    rope_cos, rope_sin, block_tables, seq_lens_decoder, cu_seqlens_q, num_tokens,
                                    batch, hq, hkv, head_dim, block_size, max_blocks_per_seq, num_blocks, max_pos,
                                    rope_style, cache_quant_type, extras, stream);
  if (rc) return rc;
  // 2. decode rows: one token, seq_lens_encoder == 0; they read their own token back from the cache
  const RowMap rows{cu_seqlens_q, seq_lens_encoder};
  const size_t dws = w.select - w.decode;
  hipStream_t s = (hipStream_t)stream;
  if (prefill_rows >= batch) {
    // the caller's count says that every sequence is a prefill row: no decode pass
  } else if (per_token) {
    // block-sparse decode rows of several tokens, every token with its own list: selector and sparse decode over the
    // token-as-row view (rows of one token; the kernels and their shapes are those of the case below)
    int32_t* tables_v = (int32_t*)(ws + w.view);
    int32_t* cu_v = tables_v + (size_t)dbatch * max_blocks_per_seq;
    int32_t* enc_v = cu_v + dbatch + 1;
    int32_t* dec_v = enc_v + dbatch;
    int32_t* this_v = dec_v + dbatch;
    hipLaunchKernelGGL(rows_per_token_kernel, dim3((unsigned)dbatch), dim3(256), 0, s, cu_seqlens_q, seq_lens_encoder,
                       seq_lens_decoder, block_tables, batch, decode_tokens, max_blocks_per_seq, tables_v, cu_v, enc_v,
                       dec_v, this_v);
    rc = check_launch("fdattn_append_attention (token-as-row view)");
    if (rc) return rc;
    const RowMap vrows{cu_v, enc_v};
    int32_t* kept = (int32_t*)(ws + w.kept);
    int32_t* counts = kept + (size_t)dbatch * hkv * top_k;
    rc = sqattn_select_launch(q_rot, key_cache, cache_k_scale, tables_v, dec_v, this_v, kept, counts, ws + w.select,
                              w.kept - w.select, dbatch, hq, hkv, head_dim, block_size, max_blocks_per_seq, num_blocks,
                              top_k, cache_quant_type, s, vrows, 1);
    if (rc) return rc;
    if (sel_fast)
      rc = decode_c8_launch(q_rot, key_cache, value_cache, cache_k_scale, cache_v_scale, tables_v, dec_v, this_v, kept,
                            counts, top_k, out, ws + w.decode, dws, dbatch, hq, hkv, head_dim, block_size,
                            max_blocks_per_seq, num_blocks, cache_quant_type, softmax_scale, s, 3, vrows, 1);
    else
      rc = decode_generic_launch(q_rot, key_cache, value_cache, cache_k_scale, cache_v_scale, tables_v, dec_v, this_v,
                                 kept, counts, top_k, out, ws + w.decode, dws, dbatch, hq, hkv, head_dim, block_size,
                                 max_blocks_per_seq, num_blocks, cache_quant_type, softmax_scale, s, vrows);
  } else if (top_k > 0) {
    // block-sparse decode rows: select with the new query over the cache as the writer left it, then attend to
    // the kept blocks only (a row of several tokens: one list, scored by all of them)
    int32_t* kept = (int32_t*)(ws + w.kept);
    int32_t* counts = kept + (size_t)batch * hkv * top_k;
    rc = sqattn_select_launch(q_rot, key_cache, cache_k_scale, block_tables, seq_lens_decoder, seq_lens_this_time, kept,
                              counts, ws + w.select, w.kept - w.select, batch, hq, hkv, head_dim, block_size,
                              max_blocks_per_seq, num_blocks, top_k, cache_quant_type, s, rows, decode_tokens);
    if (rc) return rc;
    if (sel_fast)
      rc = decode_c8_launch(q_rot, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables, seq_lens_decoder,
                            seq_lens_this_time, kept, counts, top_k, out, ws + w.decode, dws, batch, hq, hkv, head_dim,
                            block_size, max_blocks_per_seq, num_blocks, cache_quant_type, softmax_scale, s, 3, rows,
                            decode_tokens);
    else
      rc = decode_generic_launch(q_rot, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                                 seq_lens_decoder, seq_lens_this_time, kept, counts, top_k, out, ws + w.decode, dws,
                                 batch, hq, hkv, head_dim, block_size, max_blocks_per_seq, num_blocks,
                                 cache_quant_type, softmax_scale, s, rows);
  } else if (c8 && decode_tokens * (hq / hkv) <= 8)
    // (rows of more than 8 (token, head) pairs per KV head cost the int8-MFMA kernel its second wavefront per SIMD:
    // the fp16-MFMA kernel, whose 16 columns they fill, serves them faster - 97 against 126 us for 64 rows x 4 tokens)
    rc = decode_c8_launch(q_rot, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                          seq_lens_decoder, seq_lens_this_time, nullptr, nullptr, 0, out, ws + w.decode, dws, batch,
                          hq, hkv, head_dim, block_size, max_blocks_per_seq, num_blocks, cache_quant_type,
                          softmax_scale, s, 3, rows, decode_tokens);
  else
    rc = decode_generic_launch(q_rot, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                               seq_lens_decoder, seq_lens_this_time, nullptr, nullptr, 0, out, ws + w.decode, dws,
                               batch, hq, hkv, head_dim, block_size, max_blocks_per_seq, num_blocks,
                               cache_quant_type, softmax_scale, s, rows, kDecodeAuto, decode_tokens);
  if (rc) return rc;
  // 3. prefill rows: seq_lens_encoder > 0; the chunk's own K/V come from this call, the prefix from the cache
  if (any_prefill)
    rc = prefill_launch(q_rot, k_new, v_new, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                        seq_lens_decoder, cu_seqlens_q, seq_lens_encoder, out, num_tokens, batch, max_chunk, hq, hkv,
                        head_dim, block_size, max_blocks_per_seq, num_blocks, cache_quant_type, softmax_scale, s,
                        false, ws + w.split, w.total - w.split, splits, prefill_rows > 0 ? prefill_rows : -1);
  return rc;
}
