// Launchers shared by the entry-point files of libfdattn.so.
#pragma once
#include "fdattn_common.h"
#include "prefill.h"

namespace fdattn {

size_t generic_workspace_bytes(int batch, int hq, int d, int hkv);
int decode_generic_launch(const void* q, const void* key_cache, const void* value_cache,
                          const float* k_scale, const float* v_scale, const int32_t* block_tables,
                          const int32_t* seq_lens_decoder, const int32_t* seq_lens_this_time,
                          const int32_t* kept_blocks, const int32_t* kept_counts, int max_kept,
                          void* out, void* workspace, size_t workspace_bytes, int batch, int hq,
                          int hkv, int d, int bs, int max_blocks, int num_blocks, int quant,
                          float sm_scale, hipStream_t s, RowMap rows = RowMap{nullptr, nullptr},
                          int impl = 0, int max_tokens = 1);
// impl: which kernel takes the launch - the fp16-MFMA one where it covers the shape and else the vector-ALU one,
// or one of them by name; max_tokens > 1 (fp16-MFMA kernel only): decode rows of up to that many tokens
constexpr int kDecodeAuto = 0, kDecodeVectorAlu = 1, kDecodeTiles = 2;
// compute units of the current device (256 on MI355X; that value if the query fails)
int gpu_cu_count();
// units (cache blocks) per workgroup for `pairs` block lists of at most max_units blocks: as few chunks per
// list as fill the GPU's workgroup slots once, at most `most` units each (the kernel's unit table: 128, or the 256 of
// the decode kernel with one or two row sets)
int c8_pick_chunk(int pairs, int max_units, int most = 128);
size_t c8_workspace_bytes(int batch, int hkv, int max_units, int group = 4);
bool c8_supported(int hq, int hkv, int d, int bs, int quant);
// stages: 1 = the split-KV kernel, 2 = the merge of its partials, 3 = both
int decode_c8_launch(const void* q, const void* key_cache, const void* value_cache,
                     const float* k_scale, const float* v_scale, const int32_t* block_tables,
                     const int32_t* seq_lens_decoder, const int32_t* seq_lens_this_time,
                     const int32_t* kept_blocks, const int32_t* kept_counts, int max_kept,
                     void* out, void* workspace, size_t workspace_bytes, int batch, int hq,
                     int hkv, int d, int bs, int max_blocks, int num_blocks, int quant,
                     float sm_scale, hipStream_t s, int stages, RowMap rows = RowMap{nullptr, nullptr},
                     int max_tokens = 1);
// the block selector on the decode rows of a mixed step (rows), MFMA shapes only
bool sqattn_fast_supported(int hq, int hkv, int d, int bs, int max_blocks);
int sqattn_select_launch(const void* q, const void* key_cache, const float* cache_k_scale, const int32_t* block_tables,
                         const int32_t* seq_lens_decoder, const int32_t* seq_lens_this_time, int32_t* kept_blocks,
                         int32_t* kept_counts, void* workspace, size_t workspace_bytes, int batch, int hq, int hkv,
                         int head_dim, int block_size, int max_blocks_per_seq, int num_blocks, int top_k,
                         int cache_quant_type, hipStream_t s, RowMap rows, int max_tokens = 1);
// append (prefill) attention; seq_lens_encoder may be NULL (every sequence is a prefill row)
// workspace / n_splits: the MFMA kernel may split every query tile's keys over n_splits workgroups (partials in
// workspace); rows_hint: how many of the batch's rows are prefill rows, if known (0: take n_splits as given; < 0: unknown,
// the MFMA kernel counts them and uses the splits, at most n_splits, that so many rows need)
int prefill_launch(const void* q, const void* k_new, const void* v_new, const void* key_cache,
                   const void* value_cache, const float* cache_k_scale, const float* cache_v_scale,
                   const int32_t* block_tables, const int32_t* seq_lens_decoder, const int32_t* cu_seqlens_q,
                   const int32_t* seq_lens_encoder, void* out, int num_tokens, int batch, int max_chunk, int hq,
                   int hkv, int head_dim, int block_size, int max_blocks, int num_blocks, int cache_quant_type,
                   float softmax_scale, hipStream_t s, bool force_generic, void* workspace = nullptr,
                   size_t workspace_bytes = 0, int n_splits = 1, int rows_hint = 0, bool force_tiles = false);

}  // namespace fdattn
