// Entry points of decode attention: argument checks and the choice between the
// MFMA kernel (head_dim 128, 4 query heads per KV head, block_size 64) and the
// shape-agnostic kernel.
#include <atomic>

#include "launch.h"

namespace fdattn {

// Scratch of fdattn_decode_attention_noalloc: the split-KV partials live here instead of in a caller's
// workspace.  Every GPU the library runs on holds its own copy of the array until the process ends.
constexpr size_t kStaticScratchBytes = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// In host code `scratch` is only a stand-in for the symbol: the memory of the current device's copy
// is what hipGetSymbolAddress returns, looked up once per device and kept.
constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

static int static_scratch(const char* fn, void** ptr) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail((int)e, "%s: hipGetDevice: %s", fn, hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(FDATTN_ERR_SHAPE, "%s: device ordinal %d not below %d", fn, dev, kMaxDevices);
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return fail(e != hipSuccess ? (int)e : FDATTN_ERR_NULL, "%s: hipGetSymbolAddress(scratch) on device %d: %s", fn, dev,
                  hipGetErrorString(e));
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // threads racing here store the same address
  }
  *ptr = p;
  return 0;
}

static int check_decode_args(const char* fn, const void* q, const void* kc, const void* vc, const float* ks,
                             const float* vs, const int32_t* bt, const int32_t* dec, const void* out,
                             const void* ws, int batch, int hq, int hkv, int d, int bs, int max_blocks,
                             int num_blocks, int quant) {
  if (!q || !kc || !vc || !ks || !vs || !bt || !dec || !out || !ws)
    return fail(FDATTN_ERR_NULL, "%s: a required pointer is NULL", fn);
  if (batch <= 0 || hq <= 0 || hkv <= 0 || hq % hkv != 0 || d <= 0 || bs <= 0 || max_blocks <= 0 ||
      num_blocks <= 0)
    return fail(FDATTN_ERR_SHAPE, "%s: bad shape batch=%d hq=%d hkv=%d head_dim=%d block_size=%d max_blocks=%d "
                "num_blocks=%d", fn, batch, hq, hkv, d, bs, max_blocks, num_blocks);
  if (!quant_known(quant))
    return fail(FDATTN_ERR_QUANT, "%s: unknown cache_quant_type %d", fn, quant);
  return 0;
}

}  // namespace fdattn

using namespace fdattn;

// widest: room for the splits a batch of very few sequences may use; else the least a launch accepts
static size_t decode_workspace_need(int batch, int hq, int hkv, int head_dim, int max_blocks_per_seq, bool widest) {
  if (batch <= 0 || hq <= 0 || hkv <= 0 || head_dim <= 0 || max_blocks_per_seq <= 0) return 256;
  size_t a = generic_workspace_bytes(batch, hq, head_dim, widest && hq % hkv == 0 ? hkv : 0);
  size_t b = hq % hkv == 0 ? c8_workspace_bytes(batch, hkv, max_blocks_per_seq, hq / hkv) : 0;
  size_t n = a > b ? a : b;
  return (n + 255) & ~(size_t)255;
}

extern "C" size_t fdattn_decode_workspace_bytes(int batch, int hq, int hkv, int head_dim, int max_blocks_per_seq) {
  return decode_workspace_need(batch, hq, hkv, head_dim, max_blocks_per_seq, true);
}

extern "C" int fdattn_decode_attention(
    const void* q, const void* key_cache, const void* value_cache, const float* cache_k_scale,
    const float* cache_v_scale, const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* seq_lens_this_time, void* out, void* workspace, size_t workspace_bytes, int batch,
    int hq, int hkv, int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
    int cache_quant_type, float softmax_scale, void* stream) {
  int rc = check_decode_args("fdattn_decode_attention", q, key_cache, value_cache, cache_k_scale,
                             cache_v_scale, block_tables, seq_lens_decoder, out, workspace, batch, hq, hkv,
                             head_dim, block_size, max_blocks_per_seq, num_blocks, cache_quant_type);
  if (rc) return rc;
  if (c8_supported(hq, hkv, head_dim, block_size, cache_quant_type))
    return decode_c8_launch(q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                            seq_lens_decoder, seq_lens_this_time, nullptr, nullptr, 0, out, workspace,
                            workspace_bytes, batch, hq, hkv, head_dim, block_size, max_blocks_per_seq,
                            num_blocks, cache_quant_type, softmax_scale, (hipStream_t)stream, 3);
  return decode_generic_launch(q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                               seq_lens_decoder, seq_lens_this_time, nullptr, nullptr, 0, out, workspace,
                               workspace_bytes, batch, hq, hkv, head_dim, block_size, max_blocks_per_seq,
                               num_blocks, cache_quant_type, softmax_scale, (hipStream_t)stream);
}

extern "C" size_t fdattn_decode_noalloc_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int fdattn_decode_attention_noalloc(
    const void* q, const void* key_cache, const void* value_cache, const float* cache_k_scale,
    const float* cache_v_scale, const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* seq_lens_this_time, void* out, int batch, int hq, int hkv, int head_dim, int block_size,
    int max_blocks_per_seq, int num_blocks, int cache_quant_type, float softmax_scale, void* stream) {
  const char* fn = "fdattn_decode_attention_noalloc";
  // `out` stands in for the workspace in the NULL check: the scratch pointer is resolved below
  int rc = check_decode_args(fn, q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                             seq_lens_decoder, out, out, batch, hq, hkv, head_dim, block_size,
                             max_blocks_per_seq, num_blocks, cache_quant_type);
  if (rc) return rc;
  // what the kernel that takes these shapes needs, and no more: the int8-MFMA kernel's partials (one per chunk of a
  // block list; none at all once every list is a single chunk) or, at the other shapes, the least the split-KV kernels
  // accept (a batch of very few sequences then uses the splits the scratch holds)
  const bool mfma_c8 = c8_supported(hq, hkv, head_dim, block_size, cache_quant_type);
  const size_t need = mfma_c8 ? c8_workspace_bytes(batch, hkv, max_blocks_per_seq, hq / hkv)
                              : generic_workspace_bytes(batch, hq, head_dim, 0);
  if (need > kStaticScratchBytes)
    return fail(FDATTN_ERR_WORKSPACE, "%s: these shapes need %zu B of split-KV scratch, the library's static scratch "
                "holds %zu B: call fdattn_decode_attention with a workspace of the caller's", fn, need, kStaticScratchBytes);
  void* ws = nullptr;
  rc = static_scratch(fn, &ws);
  if (rc) return rc;
  if (mfma_c8)
    return decode_c8_launch(q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                            seq_lens_decoder, seq_lens_this_time, nullptr, nullptr, 0, out, ws,
                            kStaticScratchBytes, batch, hq, hkv, head_dim, block_size, max_blocks_per_seq,
                            num_blocks, cache_quant_type, softmax_scale, (hipStream_t)stream, 3);
  return decode_generic_launch(q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                               seq_lens_decoder, seq_lens_this_time, nullptr, nullptr, 0, out, ws,
                               kStaticScratchBytes, batch, hq, hkv, head_dim, block_size, max_blocks_per_seq,
                               num_blocks, cache_quant_type, softmax_scale, (hipStream_t)stream);
}

extern "C" int fdattn_decode_uses_mfma(int hq, int hkv, int head_dim, int block_size, int cache_quant_type) {
  return c8_supported(hq, hkv, head_dim, block_size, cache_quant_type) ? 1 : 0;
}

extern "C" int fdattn_decode_chunks_per_sequence(int batch, int hkv, int max_blocks_per_seq) {
  if (batch <= 0 || hkv <= 0 || max_blocks_per_seq <= 0) return 0;
  const int chunk = c8_pick_chunk(batch * hkv, max_blocks_per_seq, 256);  // (rows of one token: the wide unit table)
  return (max_blocks_per_seq + chunk - 1) / chunk;
}

extern "C" int fdattn_decode_attention_stages(
    const void* q, const void* key_cache, const void* value_cache, const float* cache_k_scale,
    const float* cache_v_scale, const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* seq_lens_this_time, void* out, void* workspace, size_t workspace_bytes, int batch,
    int hq, int hkv, int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
    int cache_quant_type, float softmax_scale, int stages, void* stream) {
  int rc = check_decode_args("fdattn_decode_attention_stages", q, key_cache, value_cache, cache_k_scale,
                             cache_v_scale, block_tables, seq_lens_decoder, out, workspace, batch, hq, hkv,
                             head_dim, block_size, max_blocks_per_seq, num_blocks, cache_quant_type);
  if (rc) return rc;
  if (!c8_supported(hq, hkv, head_dim, block_size, cache_quant_type))
    return fail(FDATTN_ERR_SHAPE, "fdattn_decode_attention_stages: shape not covered by the MFMA kernel");
  if (stages < 1 || stages > 3)
    return fail(FDATTN_ERR_SHAPE, "fdattn_decode_attention_stages: stages must be 1, 2 or 3");
  return decode_c8_launch(q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                          seq_lens_decoder, seq_lens_this_time, nullptr, nullptr, 0, out, workspace,
                          workspace_bytes, batch, hq, hkv, head_dim, block_size, max_blocks_per_seq,
                          num_blocks, cache_quant_type, softmax_scale, (hipStream_t)stream, stages);
}

extern "C" int fdattn_decode_attention_generic(
    const void* q, const void* key_cache, const void* value_cache, const float* cache_k_scale,
    const float* cache_v_scale, const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* seq_lens_this_time, const int32_t* kept_blocks, const int32_t* kept_counts, int max_kept,
    void* out, void* workspace, size_t workspace_bytes, int batch,
    int hq, int hkv, int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
    int cache_quant_type, float softmax_scale, void* stream) {
  int rc = check_decode_args("fdattn_decode_attention_generic", q, key_cache, value_cache, cache_k_scale,
                             cache_v_scale, block_tables, seq_lens_decoder, out, workspace, batch, hq, hkv,
                             head_dim, block_size, max_blocks_per_seq, num_blocks, cache_quant_type);
  if (rc) return rc;
  if ((kept_blocks == nullptr) != (kept_counts == nullptr))
    return fail(FDATTN_ERR_NULL, "fdattn_decode_attention_generic: kept_blocks and kept_counts go together");
  return decode_generic_launch(q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                               seq_lens_decoder, seq_lens_this_time, kept_blocks, kept_counts, max_kept, out,
                               workspace, workspace_bytes, batch, hq, hkv, head_dim, block_size,
                               max_blocks_per_seq, num_blocks, cache_quant_type, softmax_scale,
                               (hipStream_t)stream, RowMap{nullptr, nullptr}, kDecodeVectorAlu);
}

extern "C" int fdattn_decode_attention_tiles(
    const void* q, const void* key_cache, const void* value_cache, const float* cache_k_scale,
    const float* cache_v_scale, const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* seq_lens_this_time, const int32_t* kept_blocks, const int32_t* kept_counts, int max_kept,
    void* out, void* workspace, size_t workspace_bytes, int batch,
    int hq, int hkv, int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
    int cache_quant_type, float softmax_scale, void* stream) {
  int rc = check_decode_args("fdattn_decode_attention_tiles", q, key_cache, value_cache, cache_k_scale,
                             cache_v_scale, block_tables, seq_lens_decoder, out, workspace, batch, hq, hkv,
                             head_dim, block_size, max_blocks_per_seq, num_blocks, cache_quant_type);
  if (rc) return rc;
  if ((kept_blocks == nullptr) != (kept_counts == nullptr))
    return fail(FDATTN_ERR_NULL, "fdattn_decode_attention_tiles: kept_blocks and kept_counts go together");
  return decode_generic_launch(q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                               seq_lens_decoder, seq_lens_this_time, kept_blocks, kept_counts, max_kept, out,
                               workspace, workspace_bytes, batch, hq, hkv, head_dim, block_size,
                               max_blocks_per_seq, num_blocks, cache_quant_type, softmax_scale,
                               (hipStream_t)stream, RowMap{nullptr, nullptr}, kDecodeTiles);
}

extern "C" int fdattn_decode_attention_sparse(
    const void* q, const void* key_cache, const void* value_cache, const float* cache_k_scale,
    const float* cache_v_scale, const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* seq_lens_this_time, const int32_t* kept_blocks, const int32_t* kept_counts, int max_kept,
    void* out, void* workspace, size_t workspace_bytes, int batch, int hq, int hkv, int head_dim,
    int block_size, int max_blocks_per_seq, int num_blocks, int cache_quant_type, float softmax_scale,
    void* stream) {
  int rc = check_decode_args("fdattn_decode_attention_sparse", q, key_cache, value_cache, cache_k_scale,
                             cache_v_scale, block_tables, seq_lens_decoder, out, workspace, batch, hq, hkv,
                             head_dim, block_size, max_blocks_per_seq, num_blocks, cache_quant_type);
  if (rc) return rc;
  if (!kept_blocks || !kept_counts || max_kept <= 0)
    return fail(FDATTN_ERR_NULL, "fdattn_decode_attention_sparse: kept_blocks / kept_counts / max_kept missing");
  if (c8_supported(hq, hkv, head_dim, block_size, cache_quant_type))
    return decode_c8_launch(q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                            seq_lens_decoder, seq_lens_this_time, kept_blocks, kept_counts, max_kept, out,
                            workspace, workspace_bytes, batch, hq, hkv, head_dim, block_size,
                            max_blocks_per_seq, num_blocks, cache_quant_type, softmax_scale,
                            (hipStream_t)stream, 3);
  return decode_generic_launch(q, key_cache, value_cache, cache_k_scale, cache_v_scale, block_tables,
                               seq_lens_decoder, seq_lens_this_time, kept_blocks, kept_counts, max_kept, out,
                               workspace, workspace_bytes, batch, hq, hkv, head_dim, block_size,
                               max_blocks_per_seq, num_blocks, cache_quant_type, softmax_scale,
                               (hipStream_t)stream);
}
