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
};

bool prefill_mfma_supported(int hq, int hkv, int d, int bs, int quant);
int prefill_mfma_launch(const PrefillArgs& a, int max_chunk, int quant, hipStream_t s);

}  // namespace fdattn
