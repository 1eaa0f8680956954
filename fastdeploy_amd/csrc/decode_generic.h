// Arguments and partial-result layout shared by the decode kernels of the shapes the int8-MFMA kernel
// (decode_c8.hip) does not take: the vector-ALU kernel (decode_generic.hip) and the fp16-MFMA kernel for
// head_dim 64 / 128 / 256 at any block size (decode_tiles.hip).  Both leave one partial per (sequence, query head,
// split) - o unnormalised in fp32, the exponent reference m (natural-log units) and the weight sum l - for
// splitkv_combine_kernel.
#pragma once
#include "fdattn_common.h"

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
  float* part_o;  // [rows, max_splits, d], rows = (sequence, query head)
  float* part_m;  // [rows, max_splits]
  float* part_l;
  uint16_t* out;  // bf16 [rows, hq, d]: written directly by a launch of one split of the fp16-MFMA kernel
  RowMap rows;
  int batch, hq, hkv, d, bs, max_blocks, num_blocks, max_splits;
  float sm_scale;
  int scale_rows;  // DYN: scales per tile in the scale caches: bs (one per stored row) or 1 (the tile shares one)
  int max_tokens;  // tokens a decode row may bring (fp16-MFMA kernel only; max_tokens x hq / hkv <= 16); the partials then
                   // are [batch, max_tokens, hq, max_splits, ..]
  // the fp16-MFMA kernel as the block selector's scoring pass (sqattn_scores_tiles_launch): per (sequence, KV head) pair
  // and block the largest score, a bound on its distance to the fp64 score, and per pair a bound that holds for all blocks
  float* sel_approx;      // [pairs][max_blocks]
  float* sel_ebound;      // [pairs][max_blocks], the formats with scale caches; else NULL
  float* sel_eps;         // [pairs]
  float* sel_scores_out;  // optional copy of sel_approx
  int sel_blocks_per_split;  // ceil(max_blocks / max_splits): the size of a scoring workgroup's per-block LDS arrays
};

// head_dim 64 / 128 / 256 with at most 64 query heads per KV head
bool decode_tiles_supported(int hq, int hkv, int d);
// key splits (grid.y, = a.max_splits) for batch x hkv (sequence, KV head) pairs of at most max_keys keys each
int decode_tiles_splits(int pairs, int d, int max_keys, int most);
// launches the split kernel only (a.max_splits splits); the caller runs the combine unless a.max_splits is 1 (the
// kernel then writes a.out itself)
hipError_t decode_tiles_launch(const GenericDecodeArgs& a, int quant, hipStream_t s);
// The same kernel's K half as the scoring pass of the block selector at head_dim 64 / 128 / 256 and any block size (up to
// 16 query heads per KV head, one token per row): fills a.sel_* for every pair; a.max_splits splits of whole blocks each.
hipError_t sqattn_scores_tiles_launch(const GenericDecodeArgs& a, int quant, hipStream_t s);
// LDS a scoring workgroup needs beyond the decode kernel's, and the largest number of blocks a split may hold
constexpr int kSelTilesMaxBlocksPerSplit = 2048;

}  // namespace fdattn
