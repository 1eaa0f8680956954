// Arguments shared by the two append-attention kernels.
#pragma once
#include "fdattn_common.h"

namespace fdattn {

struct PrefillArgs {
  const uint16_t* q;
  const uint16_t* k_new;
  const uint16_t* v_new;
  const uint8_t* key_cache;
  const uint8_t* value_cache;
  const float* k_scale;
  const float* v_scale;
  const int32_t* block_tables;
  const int32_t* seq_lens_decoder;
  const int32_t* cu_seqlens_q;
  const int32_t* seq_lens_encoder;  // NULL, or > 0 for the sequences that are prefill rows of a mixed batch
  uint16_t* out;
  int num_tokens, batch, hq, hkv, d, bs, max_blocks, num_blocks;
  float sm_scale;
  int q_tiles;  // MFMA kernel: workgroups per (sequence, query head), set by its launcher
  // MFMA kernel, split along the keys: n_splits > 1 workgroups share a query tile, each walks 1/n_splits of its
  // key tiles and leaves a partial (unnormalised o in fp32, exponent reference m, weight sum l) for the merge
  int n_splits;
  int tile_tokens;  // queries per workgroup of this launch (128 or 256), for the merge kernel
  int rows;         // MFMA kernel: sequences the grid covers - the batch, or the number of prefill rows when the host gave it
  // MFMA kernel, short chunks: > 0 packs ALL query heads of a KV head into one workgroup - query column x of the
  // workgroup is head x / pack_slot of the group, token x % pack_slot - so that the staged K / V tiles serve the
  // whole group (the grid then runs over KV heads, not query heads); 0: one query head per workgroup
  int pack_slot;
  float* part_o;   // [n_splits][num_tokens][hq][128]
  float* part_ml;  // [n_splits][num_tokens][hq][2]
};

bool prefill_mfma_supported(int hq, int hkv, int d, int bs, int quant);
// workspace may be NULL (no split); n_splits is clamped to what the workspace holds
int prefill_mfma_launch(const PrefillArgs& a, int max_chunk, int quant, hipStream_t s, void* workspace = nullptr,
                        size_t workspace_bytes = 0, int n_splits = 1, int rows_hint = 0);
size_t prefill_split_workspace_bytes(int num_tokens, int hq, int n_splits);
// splits that fill the GPU when `rows` sequences bring at most max_chunk new tokens each (1 = none needed);
// hkv (optional): with it the count allows for short chunks running one workgroup per KV head
int prefill_auto_splits(int rows, int hq, int max_chunk, int hkv = 0);

}  // namespace fdattn
