/*
 * fdattn.h - C ABI of libfdattn.so, the MI355X (gfx950) paged-KV attention path.
 *
 * Every entry point takes raw device pointers, explicit integer shapes and an
 * opaque stream handle (a hipStream_t passed as void*; NULL = the null stream).
 * Nothing here allocates, frees or synchronises: all buffers, the KV caches and
 * the workspace included, are owned by the caller ("__fd_keep" in the
 * reference's C API vocabulary, c_api/fastdeploy_capi/core/fd_common.h:30-56),
 * and work is only enqueued on the given stream, like the reference's custom
 * operators enqueue on their input's stream and return without a sync
 * (fastdeploy/runtime/backends/paddle/ops/voxelize_op.cu:287-351).
 *
 * The reference registers the operators it plugs into the engine through
 * PD_BUILD_OP(name).Inputs(...).Outputs(...).Attrs(...)
 * (fastdeploy/runtime/backends/paddle/ops/voxelize_op.cc:196-204) with kernel
 * functions of the form std::vector<paddle::Tensor> fn(const paddle::Tensor&...,
 * attrs...) (voxelize_op.cc:159-162).  Each function below is the body such a
 * kernel function would forward to: tensor inputs become pointers, attributes
 * become ints / floats.
 *
 * Errors: the reference's operators throw (PD_THROW, voxelize_op.cc:172) or
 * abort (FDASSERT, fastdeploy/utils/utils.h:104-111); its C API returns
 * FD_C_Bool (c_api/fastdeploy_capi/core/fd_common.h:58).  Nothing may unwind
 * through a C ABI, so every function returns an int:
 *    0  success (work enqueued)
 *   <0  argument error (FDATTN_ERR_*), nothing was enqueued
 *   >0  a hipError_t reported by the launch
 * and fdattn_last_error() returns the message for the calling thread.
 *
 * Data layouts (all row-major, innermost dimension last):
 *   qkv           bf16  [num_tokens, (hq + 2*hkv) * head_dim]   Q heads, K heads, V heads
 *   key_cache     u8    [num_blocks, hkv, block_size, head_dim] int8 (two's complement) or fp8 e4m3fn
 *   value_cache   u8    same
 *   cache_k_scale f32   [hkv, head_dim]  dequantisation multiplier (max-abs/127 or max-abs/448)
 *   cache_v_scale f32   [hkv, head_dim]
 *                       dynamic formats: [num_blocks, hkv, block_size], one scale per stored row (see below)
 *                       per-block formats: [num_blocks, hkv], one scale per (block, KV head) tile (see below)
 *   block_tables  i32   [batch, max_blocks_per_seq]  physical block per logical block, -1 = none
 *   seq_lens_*    i32   [batch]
 *   rope_cos/sin  f32   [max_pos, head_dim/2]  host-built table shared with the CPU oracle
 */
#ifndef FDATTN_H_
#define FDATTN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FDATTN_API __attribute__((visibility("default")))

/* cache_quant_type */
#define FDATTN_CACHE_INT8 1     /* q = clamp(rne(x / scale), -127, 127), stored as int8 */
#define FDATTN_CACHE_FP8_E4M3 2 /* q = e4m3fn(clamp(x / scale, -448, 448)), RNE        */
/*
 * The dynamic formats: the same bytes, but one scale per stored row - per (token, KV head) - that the
 * cache writer derives from the row itself: scale = max_c |x[c]| / 127 (/ 448 for fp8), one IEEE
 * division, NaNs ignored by the maximum, 1.0 for a row of zeros.  Wherever an entry point takes
 * cache_k_scale / cache_v_scale, they are then the scale CACHES, f32 [num_blocks, hkv, block_size],
 * indexed like the rows of key_cache / value_cache; the cache writer, the one-call step (which contains it)
 * and fdattn_kv_import STORE into them - those entry points take them as float*, mutated in place like the caches
 * (ownership stays with the caller: "__fd_keep", c_api/fastdeploy_capi/core/fd_common.h:30-56) -, every attention
 * entry point only reads them (const float*).  With the per-channel formats nothing ever writes a scale.
 * K scales are taken after the rotation.  Dequantised value = byte * scale of its row.
 * The block selector scores a token as (row scale) x sum_c q[c] * K8[t,c] for these formats: q unscaled, the
 * sum in fp64 in ascending channel order, one more fp64 rounding for the product with the scale.
 */
#define FDATTN_CACHE_INT8_DYNAMIC 3
#define FDATTN_CACHE_FP8_E4M3_DYNAMIC 4
/*
 * The per-block formats: the same bytes with ONE scale per (block, KV head) tile - the block_size rows of a
 * head in a block share it.  cache_k_scale / cache_v_scale are scale caches f32 [num_blocks, hkv]; who stores
 * into them and who only reads them is as for the dynamic formats, and so is every attention and selector
 * formula with "scale of the row" read as "scale of the row's tile".
 * The cache writer keeps a tile's scale at (largest magnitude stored in the tile so far) / 127 (/ 448):
 * per call, sequence, block and KV head, with m = the largest |x| over the rows this call stores into the tile
 * (NaNs ignored) and s_now = m / 127 (/ 448), one IEEE division, 0 for m = 0:
 *   - the call stores the tile's first row (the sequence's cached length is a multiple of block_size there):
 *     scale = s_now, or 1.0 when s_now is 0;
 *   - rows of earlier calls are in the tile: scale = max(old scale, s_now); if that is larger than the old
 *     scale, every earlier row of the tile is requantised in place, byte -> quantise((value of byte * old
 *     scale) / scale) with one fp32 product and one IEEE division (fp8 NaN codes stay as they are);
 *   then the call's rows are quantised with the tile's scale like any other.
 * A tile therefore changes only through calls that store into it, and a block shared between sequences (which
 * is always a full one) is never requantised.
 * A tile's scale only ever GROWS, and "earlier rows" are counted by position, not by what a scheduler keeps: after a
 * speculative step whose drafts are rejected, the rows written over them find the scale where the rejected rows put it
 * (and the accepted rows on that grid), so the cache is a function of the calls, not of the accepted tokens - it equals
 * what the same calls produce anywhere, not what a replay of the accepted tokens alone would.  Likewise a tile whose
 * first call brought only zeros stays at the placeholder scale 1.0 until a row with |x| > 127 (448) arrives; rows
 * appended to it with |x| < 0.5 quantise to 0.  A caller that needs tiles independent of rejected drafts or of leading
 * zeros rewrites the tile from its first row (one call that stores the tile's first row sets the scale afresh).
 */
#define FDATTN_CACHE_INT8_BLOCK 5
#define FDATTN_CACHE_FP8_E4M3_BLOCK 6

/* rope_style */
#define FDATTN_ROPE_INTERLEAVED 0 /* pairs (2j, 2j+1)          */
#define FDATTN_ROPE_NEOX 1        /* pairs (j, j + head_dim/2) */

/* argument errors */
#define FDATTN_ERR_NULL -1        /* a required pointer is NULL              */
#define FDATTN_ERR_SHAPE -2       /* a shape the kernels do not support      */
#define FDATTN_ERR_QUANT -3       /* unknown cache_quant_type / rope_style   */
#define FDATTN_ERR_WORKSPACE -4   /* workspace too small                     */
#define FDATTN_ERR_POOL -5        /* block pool exhausted / out of host memory */

/* Library identification, "fdattn <major>.<minor> gfx950". */
FDATTN_API const char* fdattn_version(void);

/* Message of the last failing call made by this thread ("" if none). */
FDATTN_API const char* fdattn_last_error(void);

/*
 * Cache writer: rotary embedding on Q and K, quantisation of K and V into their
 * block-tabled cache slots.  Stands where an engine-side custom operator body
 * would (plug-in pattern: fastdeploy/runtime/backends/paddle/ops/voxelize_op.cc:159-176);
 * saturation follows function::Clip (fastdeploy/function/clip.cc:20-30).
 *
 * Token i belongs to the sequence b with cu_seqlens_q[b] <= i < cu_seqlens_q[b+1]
 * and sits at position pos = seq_lens_decoder[b] + (i - cu_seqlens_q[b]).
 *   q_out  bf16 [num_tokens, hq*head_dim]   rotated Q (required)
 *   k_out  bf16 [num_tokens, hkv*head_dim]  rotated K, rounded to bf16 (optional, may be NULL)
 *   v_out  bf16 [num_tokens, hkv*head_dim]  V copied through (optional, may be NULL)
 * rope_cos / rope_sin may both be NULL: no rotation is applied then.
 * A token whose block-table entry is negative is skipped (no cache store).  A token whose position lies outside the
 * rope table (pos >= max_pos) is skipped as well and its rows of q_out / k_out / v_out are zero-filled: check lengths on
 * the host (the Python backend does).
 */
FDATTN_API int fdattn_write_cache_kv(
    const void* qkv, void* q_out, void* k_out, void* v_out,
    void* key_cache, void* value_cache,
    float* cache_k_scale, float* cache_v_scale,
    const float* rope_cos, const float* rope_sin,
    const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* cu_seqlens_q,
    int num_tokens, int batch, int hq, int hkv, int head_dim, int block_size,
    int max_blocks_per_seq, int num_blocks, int max_pos,
    int rope_style, int cache_quant_type, void* stream);

/*
 * Optional extras of a step (every member optional; engine-side operators take optional inputs
 * the same way, fastdeploy/runtime/backends/paddle/ops/voxelize_op.cc:194-204 lists inputs and
 * attributes).  The QKV projection's epilogue, fused in front of the cache writer:
 *   qkv_bias        bf16 [(hq + 2*hkv) * head_dim]: x = bf16(x + bias), the result of a bf16 add
 *   q_norm_weight   f32 [head_dim]: every Q head x -> x / sqrt(mean(x^2) + eps) * weight, before
 *   k_norm_weight   f32 [head_dim]  the rotation; the same for every K head (V is not normed)
 * All arithmetic is fp32 with every operation rounded on its own; nothing is rounded to bf16
 * between the norm and the rotation.  The norm needs head_dim = 16 * 2^n.
 *   prefill_rows    (fdattn_append_attention_ex only) the number of sequences with
 *                   seq_lens_encoder > 0 in this step, if the host knows it (0 = unknown: the prefill
 *                   pass covers the whole batch and, at head_dim 128 / block_size 64, counts the prefill
 *                   rows on the GPU: the query tiles are then shared as that count asks (about 10 % slower
 *                   than with the count for one prefill row among 63 decode rows), up to the
 *                   splits the workspace has room for - fdattn_append_attention_workspace_bytes_ex with
 *                   fdattn_prefill_auto_splits(1, hq, max_chunk) holds the most a step can use).
 *                   It is a promise, not a guess: the prefill pass
 *                   then covers the first prefill_rows such sequences only.  With it the pass launches
 *                   no workgroups for decode rows, and when the prefill rows alone would leave CUs
 *                   idle - one sequence's chunk of a few hundred tokens among decode rows - every
 *                   query tile is shared by fdattn_prefill_auto_splits(prefill_rows, hq, max_chunk)
 *                   workgroups, each walking a part of its keys, if the workspace has room for their
 *                   partials (fdattn_append_attention_workspace_bytes_ex with that number of splits).
 *                   A count equal to batch says that no sequence is a decode row: the decode pass is
 *                   not launched.
 *   sqattn_top_k    (fdattn_append_attention_ex only) > 0: the decode rows of the step run block-sparse - the
 *                   selector (fdattn_sqattn_select) keeps this many blocks per (row, KV head), scored with the
 *                   row's new query against the cache that already holds its new token, and the decode
 *                   attention reads only those (fdattn_decode_attention_sparse); rows with no more blocks
 *                   than that keep all.  At most 8 query heads per KV head, head_dim <= 256, at most 4096
 *                   blocks per sequence (outside the MFMA selector's shapes the exact fp64 selector scores,
 *                   for rows of one token).  The step's workspace always has
 *                   room for it.  0: dense.
 *   decode_tokens   (fdattn_append_attention_ex only) > 1: a row with seq_lens_encoder[b] == 0 and 2 ..
 *                   decode_tokens tokens - the draft tokens of a speculative step - is a decode row too: all
 *                   its tokens are written to the cache first, then token t (0-based) attends to the
 *                   seq_lens_decoder[b] + t + 1 first tokens of the sequence, read from the cache (so, unlike a
 *                   prefill row's, its own keys and values are the quantised ones).  One pass of the decode
 *                   kernel serves all the tokens of a row.  Needs head_dim 64, 128 or 256 and
 *                   decode_tokens x (query heads per KV head) <= 16 (any block size: the int8-MFMA kernel at
 *                   head_dim 128 / block_size 64, the fp16-MFMA kernel elsewhere).  Together with sqattn_top_k
 *                   (head_dim 128 / block_size 64 only) a row of several
 *                   tokens keeps ONE list of blocks per KV head: a block's score is the maximum over the row's
 *                   tokens (each over the keys it attends to) and query heads, min(top_k, blocks of the row) are
 *                   kept, and token t attends to the kept blocks' keys up to itself.  0 / 1: such
 *                   rows get no attention output (they are prefill rows if seq_lens_encoder says so).
 *   sqattn_per_token (fdattn_append_attention_ex only; with sqattn_top_k > 0 and decode_tokens > 1) != 0: every
 *                   token of a decode row keeps a list of its own - min(top_k, the blocks it sees) blocks per KV
 *                   head, scored with its own query over the seq_lens_decoder[b] + t + 1 keys it attends to - and
 *                   attends to those: the step treats the row's tokens as so many decode rows of one token (a
 *                   small kernel lays that view out in the workspace), so every shape of sqattn_top_k is served
 *                   and decode_tokens is bounded by the workspace alone.  The decode side then runs over batch x
 *                   decode_tokens rows: size the workspace with that number as `batch`
 *                   (fdattn_append_attention_workspace_bytes[_ex]); the selector streams the keys once per token.
 */
typedef struct fdattn_step_extras {
  const void* qkv_bias;
  const float* q_norm_weight;
  const float* k_norm_weight;
  float rms_norm_eps;
  int prefill_rows;
  int sqattn_top_k;
  int decode_tokens;
  int sqattn_per_token;
} fdattn_step_extras;

/* fdattn_write_cache_kv with the extras (host pointer, read during the call; NULL = none). */
FDATTN_API int fdattn_write_cache_kv_ex(
    const void* qkv, void* q_out, void* k_out, void* v_out,
    void* key_cache, void* value_cache,
    float* cache_k_scale, float* cache_v_scale,
    const float* rope_cos, const float* rope_sin,
    const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* cu_seqlens_q,
    int num_tokens, int batch, int hq, int hkv, int head_dim, int block_size,
    int max_blocks_per_seq, int num_blocks, int max_pos,
    int rope_style, int cache_quant_type, const fdattn_step_extras* extras, void* stream);

/*
 * Bytes of workspace fdattn_decode_attention / fdattn_decode_attention_sparse
 * need for these shapes (split-KV partial results).  Never 0.  The workspace needs
 * no initialisation; calls that overlap on the GPU must not share one.  At least 16 partial
 * results per output row; up to 64 for a batch of fewer (sequence, KV head) pairs than the GPU
 * has CUs, whose keys split over that many workgroups.  A call with a smaller workspace that
 * still holds 16 per row is accepted and uses the splits that fit.
 */
FDATTN_API size_t fdattn_decode_workspace_bytes(int batch, int hq, int hkv, int head_dim,
                                                int max_blocks_per_seq);

/*
 * Decode attention over the quantised paged cache: one query token per sequence,
 *   out[b, qh, :] = softmax_t(softmax_scale * q[b, qh] . K^[b, t]) . V^[b, t],
 *   t in [0, kv_len[b]),  kv_len[b] = seq_lens_decoder[b] + (seq_lens_this_time ? seq_lens_this_time[b] : 0),
 * with K^/V^ the dequantised cache rows of KV head qh / (hq/hkv), gathered through
 * block_tables.  Rows with kv_len 0 produce zeros.  Softmax follows the
 * max-shifted form of fastdeploy/function/softmax.cc:58-86 (without its -64 clip).
 *   q   bf16 [batch, hq*head_dim]     out bf16 [batch, hq*head_dim]
 * The split-KV partials live in `workspace` and are merged by a second, small kernel
 * enqueued behind the first.
 */
FDATTN_API int fdattn_decode_attention(
    const void* q, const void* key_cache, const void* value_cache,
    const float* cache_k_scale, const float* cache_v_scale,
    const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* seq_lens_this_time, void* out,
    void* workspace, size_t workspace_bytes,
    int batch, int hq, int hkv, int head_dim, int block_size,
    int max_blocks_per_seq, int num_blocks, int cache_quant_type,
    float softmax_scale, void* stream);

/*
 * fdattn_decode_attention without a workspace argument and without any allocation: the split-KV
 * partials go to a scratch array that the library itself holds in device memory (a file-scope
 * __device__ array of fdattn_decode_noalloc_scratch_bytes() = 16 MiB, one copy per GPU the library runs
 * on, held until the process ends).  It has no counterpart in the reference; it is for callers that
 * cannot allocate or size a workspace: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  Inputs, outputs and results are those of fdattn_decode_attention (the same
 * kernels run).  Shapes whose partials need more than the scratch holds are refused with
 * FDATTN_ERR_WORKSPACE and nothing is enqueued.  What a shape needs is what the kernel that takes it needs:
 *   - the int8-MFMA kernel (fdattn_decode_uses_mfma() = 1): one partial of ceil(hq/hkv / 4) x 2,080 B per chunk of
 *     a (sequence, KV head) pair's block list; lists are cut into ceil(2 x CUs / pairs) chunks (one, and then no
 *     partial is written at all, from 512 pairs on a 256-CU GPU), more only beyond 256 blocks per chunk.  Llama-3-8B
 *     decode at batch 64 (512 pairs, 72 blocks each) asks for 1 MiB; the limit is reached near 8,000 pairs of one
 *     chunk each, or e.g. 512 pairs of 2,048 blocks (128k tokens) each;
 *   - the other shapes: 16 partial rows of (head_dim + 2) floats per (sequence, query head), i.e.
 *     batch x hq <= 2,016 at head_dim 128 (4,032 at 64; 1,016 at 256).
 * The scratch needs no clearing between calls (every partial that is read has been written by the same
 * call).  All calls on one GPU share that GPU's array: calls that overlap there - on different streams,
 * or from different threads - race; serialise them or use fdattn_decode_attention with separate
 * workspaces.
 */
FDATTN_API size_t fdattn_decode_noalloc_scratch_bytes(void);
FDATTN_API int fdattn_decode_attention_noalloc(
    const void* q, const void* key_cache, const void* value_cache,
    const float* cache_k_scale, const float* cache_v_scale,
    const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* seq_lens_this_time, void* out,
    int batch, int hq, int hkv, int head_dim, int block_size,
    int max_blocks_per_seq, int num_blocks, int cache_quant_type,
    float softmax_scale, void* stream);

/*
 * 1 if fdattn_decode_attention(_sparse) runs these shapes on the int8-MFMA kernel (head_dim
 * 128, hq/hkv from 1 to 8, block_size 64, any cache format), 0 if on one of the others (the
 * fp16-MFMA kernel at head_dim 64 / 128 / 256 with hq/hkv <= 64, else the vector-ALU kernel).
 */
FDATTN_API int fdattn_decode_uses_mfma(int hq, int hkv, int head_dim, int block_size, int cache_quant_type);

/*
 * Into how many chunks the MFMA decode kernel cuts the block list of one (sequence, KV head)
 * for a launch of this size: as few as give every workgroup slot of the GPU one chunk.  1 means
 * that every list is finished by the main kernel and no merge kernel is launched.
 */
FDATTN_API int fdattn_decode_chunks_per_sequence(int batch, int hkv, int max_blocks_per_seq);

/*
 * fdattn_decode_attention split into its two kernels, for profiling and for callers
 * that overlap other work with the merge: stages = 1 runs only the split-KV kernel
 * (partials into `workspace`; sequences that fit one chunk are finished by it), 2 only
 * the merge (workspace -> out), 3 both.  MFMA shapes only (FDATTN_ERR_SHAPE otherwise).
 * Same plug-in position as fdattn_decode_attention.
 */
FDATTN_API int fdattn_decode_attention_stages(
    const void* q, const void* key_cache, const void* value_cache,
    const float* cache_k_scale, const float* cache_v_scale,
    const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* seq_lens_this_time, void* out,
    void* workspace, size_t workspace_bytes,
    int batch, int hq, int hkv, int head_dim, int block_size,
    int max_blocks_per_seq, int num_blocks, int cache_quant_type,
    float softmax_scale, int stages, void* stream);

/*
 * Same, restricted to a per-(sequence, KV head) list of logical blocks:
 *   kept_blocks i32 [batch, hkv, max_kept]  logical block indices, ascending, -1 padded
 *   kept_counts i32 [batch, hkv]
 * A kept block j covers tokens [j*block_size, min((j+1)*block_size, kv_len)).
 */
FDATTN_API int fdattn_decode_attention_sparse(
    const void* q, const void* key_cache, const void* value_cache,
    const float* cache_k_scale, const float* cache_v_scale,
    const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* seq_lens_this_time,
    const int32_t* kept_blocks, const int32_t* kept_counts, int max_kept,
    void* out, void* workspace, size_t workspace_bytes,
    int batch, int hq, int hkv, int head_dim, int block_size,
    int max_blocks_per_seq, int num_blocks, int cache_quant_type,
    float softmax_scale, void* stream);

/*
 * The shape-agnostic decode kernel on the vector ALUs (any head_dim <= 256 that is a
 * multiple of 4, any hq/hkv, any block_size), callable directly; the two functions
 * above fall back to it for shapes neither MFMA kernel covers (the int8-MFMA kernel:
 * head_dim 128, hq/hkv 1 .. 8, block_size 64; the fp16-MFMA kernel below: head_dim 64,
 * 128 or 256, hq/hkv <= 64, any block_size).  kept_blocks / kept_counts may both be
 * NULL (dense).  Same plug-in position as fdattn_decode_attention.
 */
FDATTN_API int fdattn_decode_attention_generic(
    const void* q, const void* key_cache, const void* value_cache,
    const float* cache_k_scale, const float* cache_v_scale,
    const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* seq_lens_this_time,
    const int32_t* kept_blocks, const int32_t* kept_counts, int max_kept,
    void* out, void* workspace, size_t workspace_bytes,
    int batch, int hq, int hkv, int head_dim, int block_size,
    int max_blocks_per_seq, int num_blocks, int cache_quant_type,
    float softmax_scale, void* stream);

/*
 * The fp16-MFMA decode kernel of the shapes the int8-MFMA kernel does not take
 * (head_dim 64, 128 or 256, hq/hkv <= 64, any block_size, every cache format, dense
 * or over kept blocks), callable directly at any shape it covers - head_dim 128 with
 * block_size 64 included, where the functions above pick the int8-MFMA kernel.
 * FDATTN_ERR_SHAPE for other shapes.  Same arguments, workspace and plug-in position
 * as fdattn_decode_attention_generic.
 */
FDATTN_API int fdattn_decode_attention_tiles(
    const void* q, const void* key_cache, const void* value_cache,
    const float* cache_k_scale, const float* cache_v_scale,
    const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* seq_lens_this_time,
    const int32_t* kept_blocks, const int32_t* kept_counts, int max_kept,
    void* out, void* workspace, size_t workspace_bytes,
    int batch, int hq, int hkv, int head_dim, int block_size,
    int max_blocks_per_seq, int num_blocks, int cache_quant_type,
    float softmax_scale, void* stream);

/*
 * Split-KV merge of partial attention results (log-sum-exp combine):
 *   m = max_s m_s,  l = sum_s l_s e^(m_s - m),  out = sum_s o_s e^(m_s - m) / l
 *   part_o f32 [rows, max_splits, head_dim]  unnormalised partial outputs
 *   part_m f32 [rows, max_splits]            partial maxima (natural-log domain)
 *   part_l f32 [rows, max_splits]            partial sums of exponentials
 *   num_splits i32 [rows] or NULL (= max_splits everywhere)
 *   out bf16 [rows, head_dim]
 * Max-shift as in fastdeploy/function/softmax.cc:58-66.
 */
FDATTN_API int fdattn_splitkv_combine(
    const float* part_o, const float* part_m, const float* part_l,
    const int32_t* num_splits, void* out,
    int rows, int max_splits, int head_dim, void* stream);

/*
 * Bytes of workspace fdattn_sqattn_select needs.
 */
FDATTN_API size_t fdattn_sqattn_workspace_bytes(int batch, int hkv, int max_blocks_per_seq);

/*
 * SQAttn block selector.  For every (sequence b, KV head h, logical block j):
 *   score[b,h,j] = max over the block's valid tokens t and the hq/hkv query heads g of head h
 *                  of  sum_c (q[b,g,c] * cache_k_scale[h,c]) * K8[t,c]
 * (reduction as function::Max, fastdeploy/function/reduce.cc:354-357), then the
 * top_k highest-scoring blocks per (b,h) are kept; equal scores resolve to the
 * lower block index as in TopKIndices (fastdeploy/vision/utils/utils.h:41-60).
 *   scores      f32 [batch, hkv, max_blocks_per_seq]  (optional output, may be NULL; -inf for absent blocks).
 *               For head_dim 64, 128 or 256, hq/hkv 1 .. 8, block sizes up to 256 and at most 4096 blocks per sequence
 *               these are the MFMA scores the selection starts from (within a small relative error of the fp64
 *               ones; blocks too close to the k-th score to call are re-scored in fp64 internally, so the kept
 *               indices are those of the fp64 scores): at head_dim 128 / block_size 64 with at most 2048 blocks per
 *               sequence computed on the int8 / fp8 MFMAs straight from the cache bytes, elsewhere on the fp16 MFMAs
 *               (fdattn_sqattn_path says which);
 *               otherwise the fp64 scores rounded to fp32.
 *   kept_blocks i32 [batch, hkv, top_k]  ascending logical block indices, -1 padded
 *   kept_counts i32 [batch, hkv]         min(top_k, ceil(kv_len / block_size))
 */
FDATTN_API int fdattn_sqattn_select(
    const void* q, const void* key_cache, const float* cache_k_scale,
    const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* seq_lens_this_time,
    float* scores, int32_t* kept_blocks, int32_t* kept_counts,
    void* workspace, size_t workspace_bytes,
    int batch, int hq, int hkv, int head_dim, int block_size,
    int max_blocks_per_seq, int num_blocks, int top_k,
    int cache_quant_type, void* stream);

/*
 * Which scoring pass fdattn_sqattn_select runs for a shape: 1 = the int8 / fp8 MFMAs on the cache bytes as they are
 * (head_dim 128, block_size 64, at most 2048 blocks per sequence), 2 = the fp16 MFMAs (head_dim 64 / 128 / 256, any
 * block size up to 256, at most 4096 blocks per sequence), 0 = every block in fp64 on the vector ALU (everything
 * else).  The kept indices are the same on all three.
 */
FDATTN_API int fdattn_sqattn_path(int hq, int hkv, int head_dim, int block_size, int max_blocks_per_seq);

/*
 * The selector with every block scored in fp64 (any head_dim <= 256, hq/hkv <= 8, any block_size):
 * what fdattn_sqattn_select falls back to for shapes its MFMA scoring does not cover; same kept
 * indices, `scores` = the fp64 scores rounded to fp32.  Same arguments and plug-in position.
 */
FDATTN_API int fdattn_sqattn_select_exact(
    const void* q, const void* key_cache, const float* cache_k_scale,
    const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* seq_lens_this_time,
    float* scores, int32_t* kept_blocks, int32_t* kept_counts,
    void* workspace, size_t workspace_bytes,
    int batch, int hq, int hkv, int head_dim, int block_size,
    int max_blocks_per_seq, int num_blocks, int top_k,
    int cache_quant_type, void* stream);

/*
 * Chunked-prefill ("append") attention.  Sequence b appends n_b =
 * cu_seqlens_q[b+1] - cu_seqlens_q[b] new tokens to p_b = seq_lens_decoder[b]
 * cached ones.  New token i (0-based in the chunk) attends to the p_b cached
 * tokens (quantised pages, dequantised in-tile) and to the chunk tokens j <= i
 * (bf16 K/V of this call).
 *   q     bf16 [num_tokens, hq*head_dim]    rotated Q   (q_out of the cache writer)
 *   k_new bf16 [num_tokens, hkv*head_dim]   rotated K   (k_out of the cache writer)
 *   v_new bf16 [num_tokens, hkv*head_dim]   V           (v_out of the cache writer)
 *   out   bf16 [num_tokens, hq*head_dim]
 * max_chunk bounds n_b (it sizes the launch grid).
 * block_tables: every entry that covers one of the p_b cached tokens must name a block of the pool.  An entry that
 * does not (-1, or >= num_blocks) is read as block 0, so that no access leaves the caches, and its keys take part
 * with block 0's contents - the prefill kernels mask by position only (the decode kernels skip such blocks).
 * Accuracy of the MFMA kernels (head_dim 64, 128, 256): scores are made of exact cache bytes and 22 significant
 * bits of q * k_scale (two fp16 terms).  The kernel for head_dim 128 / block_size 64 with per-channel scales spends the
 * second term per tile of 64 cached keys and per group of 64 queries, where it can matter: one term puts a random
 * error of standard deviation 2^-12 / sqrt(3) = 1.4e-4 times s_rms into a score (s_rms: the size the scores of the
 * tile have, softmax_scale * |q * k_scale|_2 * the root mean square of the K codes) and at most about half of that
 * times v_rms into an output (v_rms: that of the dequantised V values).  Both are measured as the tile is read - the
 * mean magnitudes of its K and V codes, taken as 0.8 of their root mean square, which flatter-than-Gaussian
 * distributions exceed (the safe side) - and the second term is taken whenever s_rms * v_rms > 3, i.e. wherever one
 * term could cost more than 2e-4: a tenth of the tolerance.  (Quantised unit-scale activations sit near 1.2; against
 * the CPU oracle, outputs computed with one term everywhere first leave the tolerance near 13.)
 * The softmax weights enter P.V in fp16: as ONE term (11 bits) for
 * tiles of 64 (32) keys whose dequantised values stay within +-6 - an output element is then within
 * 2^-11 * sum_j p_j |v_j| of the fp32 result (p: the normalised weights, v: the dequantised values) - and
 * as TWO terms (22 bits) for every tile that may hold a larger value: a cached tile by its scales (largest
 * code x the KV head's largest per-channel V scale; the row's or tile's own scale in the formats with scale
 * caches), a tile of the chunk's own V by its values.  So the one-term error is at most 2^-11 * 6 = 2.9e-3 in
 * the worst case (weights and signs aligned against the rounding), below 2e-3 whenever the weighted mean
 * magnitude of the values a query attends to is at most 4.1, and no magnitude beyond 6 meets one-term weights.
 * Values beyond +-65504 in the chunk's own V saturate (fp16).
 */
FDATTN_API int fdattn_append_attention_prefill(
    const void* q, const void* k_new, const void* v_new,
    const void* key_cache, const void* value_cache,
    const float* cache_k_scale, const float* cache_v_scale,
    const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* cu_seqlens_q, void* out,
    int num_tokens, int batch, int max_chunk, int hq, int hkv, int head_dim,
    int block_size, int max_blocks_per_seq, int num_blocks,
    int cache_quant_type, float softmax_scale, void* stream);

/*
 * fdattn_append_attention_prefill with the keys of every query tile split over num_splits
 * workgroups (MFMA shapes; elsewhere num_splits is ignored): each walks 1/num_splits of the key
 * tiles and leaves a partial (o in fp32, exponent reference, weight sum) in workspace, a second
 * kernel merges them.  For launches whose query tiles alone leave CUs idle - a single sequence's
 * chunk of a few hundred tokens: fdattn_prefill_auto_splits(rows, hq, max_chunk) says how many
 * splits fill the GPU (1..8) when `rows` sequences bring at most max_chunk new tokens each.
 * workspace: fdattn_append_attention_prefill_split_workspace_bytes(num_tokens, hq, num_splits),
 * no initialisation needed.  Same plug-in position as fdattn_append_attention_prefill.
 */
FDATTN_API int fdattn_prefill_auto_splits(int rows, int hq, int max_chunk);
/* The same when the number of KV heads is known: chunks short enough for one workgroup to hold every query
 * head of a KV head (hq / hkv x max_chunk <= 256) launch one workgroup per (row, KV head), and need more splits
 * to fill the GPU.  This is the count fdattn_append_attention_ex uses. */
FDATTN_API int fdattn_prefill_auto_splits_for(int rows, int hq, int hkv, int max_chunk);
FDATTN_API size_t fdattn_append_attention_prefill_split_workspace_bytes(int num_tokens, int hq, int num_splits);
FDATTN_API int fdattn_append_attention_prefill_split(
    const void* q, const void* k_new, const void* v_new,
    const void* key_cache, const void* value_cache,
    const float* cache_k_scale, const float* cache_v_scale,
    const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* cu_seqlens_q, void* out, void* workspace, size_t workspace_bytes, int num_splits,
    int num_tokens, int batch, int max_chunk, int hq, int hkv, int head_dim,
    int block_size, int max_blocks_per_seq, int num_blocks,
    int cache_quant_type, float softmax_scale, void* stream);

/*
 * The MFMA kernel fdattn_append_attention_prefill uses for head_dim 64, 128 (at block sizes other than 64) and
 * 256 with any block size - compiler-scheduled, the same arithmetic and accuracy as the kernel for head_dim
 * 128 / block_size 64 -, callable directly (at that shape too).  Same arguments and plug-in position.
 */
FDATTN_API int fdattn_append_attention_prefill_tiles(
    const void* q, const void* k_new, const void* v_new,
    const void* key_cache, const void* value_cache,
    const float* cache_k_scale, const float* cache_v_scale,
    const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* cu_seqlens_q, void* out,
    int num_tokens, int batch, int max_chunk, int hq, int hkv, int head_dim,
    int block_size, int max_blocks_per_seq, int num_blocks,
    int cache_quant_type, float softmax_scale, void* stream);

/*
 * The shape-agnostic kernel (vector ALU, fp32) fdattn_append_attention_prefill falls back to for every other
 * head_dim, callable directly.  Same arguments and plug-in position.
 */
FDATTN_API int fdattn_append_attention_prefill_generic(
    const void* q, const void* k_new, const void* v_new,
    const void* key_cache, const void* value_cache,
    const float* cache_k_scale, const float* cache_v_scale,
    const int32_t* block_tables, const int32_t* seq_lens_decoder,
    const int32_t* cu_seqlens_q, void* out,
    int num_tokens, int batch, int max_chunk, int hq, int hkv, int head_dim,
    int block_size, int max_blocks_per_seq, int num_blocks,
    int cache_quant_type, float softmax_scale, void* stream);

/*
 * Bytes of workspace fdattn_append_attention needs for these shapes (rotated Q, the
 * chunk's K and V, split-KV partial results).  Never 0; no initialisation needed.
 */
FDATTN_API size_t fdattn_append_attention_workspace_bytes(int num_tokens, int batch, int hq, int hkv,
                                                          int head_dim, int max_blocks_per_seq);
/* The same with room for the partials of prefill_splits key splits (fdattn_step_extras). */
FDATTN_API size_t fdattn_append_attention_workspace_bytes_ex(int num_tokens, int batch, int hq, int hkv,
                                                             int head_dim, int max_blocks_per_seq, int prefill_splits);

/*
 * One attention step of a layer over a mixed batch: the whole of what an engine-side
 * attention operator does between the QKV projection and the output projection
 * (plug-in position as for the pieces above,
 * fastdeploy/runtime/backends/paddle/ops/voxelize_op.cc:159-204).  Sequence b owns the
 * token rows cu_seqlens_q[b] .. cu_seqlens_q[b+1]-1 of qkv and out and is
 *   a prefill row  if seq_lens_encoder[b] > 0: its tokens are appended to the
 *                  seq_lens_decoder[b] cached ones (fdattn_append_attention_prefill),
 *   a decode row   if seq_lens_encoder[b] == 0 and it has one token: the token is written
 *                  to the cache and attends to seq_lens_decoder[b] + 1 cached tokens
 *                  (fdattn_decode_attention),
 *   idle           otherwise (no token: nothing is read or written for it).
 * A row that brings several tokens with causal attention among them - a prompt chunk, or the
 * draft tokens of a speculative step - is a prefill row: give it seq_lens_encoder[b] = its
 * number of tokens (a row with several tokens and seq_lens_encoder[b] == 0 gets its tokens
 * written to the cache but no attention output, unless fdattn_step_extras.decode_tokens makes
 * it a decode row of several tokens).
 * Every new token is first rotated and written to the cache (fdattn_write_cache_kv).
 * max_chunk bounds the tokens of a prefill row in this step; 0 says that the step has no
 * prefill row (the prefill pass is then not launched at all).
 * Nothing is gathered or synchronised on the host; out rows of idle slots do not exist.
 */
FDATTN_API int fdattn_append_attention(
    const void* qkv, void* key_cache, void* value_cache,
    float* cache_k_scale, float* cache_v_scale,
    const float* rope_cos, const float* rope_sin,
    const int32_t* block_tables, const int32_t* seq_lens_encoder,
    const int32_t* seq_lens_decoder, const int32_t* seq_lens_this_time,
    const int32_t* cu_seqlens_q, void* out, void* workspace, size_t workspace_bytes,
    int num_tokens, int batch, int max_chunk, int hq, int hkv, int head_dim,
    int block_size, int max_blocks_per_seq, int num_blocks, int max_pos,
    int rope_style, int cache_quant_type, float softmax_scale, void* stream);

/* fdattn_append_attention with the extras of a step (NULL = none). */
FDATTN_API int fdattn_append_attention_ex(
    const void* qkv, void* key_cache, void* value_cache,
    float* cache_k_scale, float* cache_v_scale,
    const float* rope_cos, const float* rope_sin,
    const int32_t* block_tables, const int32_t* seq_lens_encoder,
    const int32_t* seq_lens_decoder, const int32_t* seq_lens_this_time,
    const int32_t* cu_seqlens_q, void* out, void* workspace, size_t workspace_bytes,
    int num_tokens, int batch, int max_chunk, int hq, int hkv, int head_dim,
    int block_size, int max_blocks_per_seq, int num_blocks, int max_pos,
    int rope_style, int cache_quant_type, float softmax_scale, const fdattn_step_extras* extras, void* stream);

/*
 * Host-side block pool: the producer of block_tables (no counterpart in the reference,
 * whose engines own their memory, fastdeploy/runtime/backends/paddle/paddle_backend.cc:425-427;
 * handle-style C API after c_api/fastdeploy_capi/core/fd_type.h:104-155: create / destroy
 * pairs, the caller owns the handle).  num_blocks cache blocks of block_size tokens,
 * max_seqs sequence slots, each with a table row of max_blocks_per_seq entries (-1 = no
 * block).  Blocks are reference counted; fdattn_pool_fork shares the whole blocks of a
 * prefix between two slots.  Not thread-safe.  No GPU call is made: copy the table (int32
 * [max_seqs, max_blocks_per_seq]) to the device where block_tables is needed.
 */
typedef struct fdattn_block_pool fdattn_block_pool;
FDATTN_API fdattn_block_pool* fdattn_pool_create(int num_blocks, int block_size, int max_seqs,
                                                 int max_blocks_per_seq);            /* NULL on error */
FDATTN_API void fdattn_pool_destroy(fdattn_block_pool* pool);
/* Grow slot seq so that it covers num_tokens tokens (never shrinks).  All or nothing:
 * FDATTN_ERR_POOL if the free blocks do not suffice, and then nothing has changed. */
FDATTN_API int fdattn_pool_reserve(fdattn_block_pool* pool, int seq, int num_tokens);
/* Give every block of slot seq back (a shared block returns to the free list with its last owner). */
FDATTN_API int fdattn_pool_release(fdattn_block_pool* pool, int seq);
/* Let the empty slot dst_seq share the whole blocks that hold the first shared_tokens tokens of
 * src_seq.  Returns the number of tokens now shared (a multiple of block_size), or < 0. */
FDATTN_API int fdattn_pool_fork(fdattn_block_pool* pool, int src_seq, int dst_seq, int shared_tokens);
FDATTN_API int fdattn_pool_free_blocks(const fdattn_block_pool* pool);
FDATTN_API int fdattn_pool_seq_blocks(const fdattn_block_pool* pool, int seq);
FDATTN_API int fdattn_pool_refcount(const fdattn_block_pool* pool, int block);
/* The table, valid until the pool is destroyed; its contents change with reserve / release / fork. */
FDATTN_API const int32_t* fdattn_pool_block_tables(const fdattn_block_pool* pool);

/*
 * KV pages of whole sequences to and from a contiguous, self-describing buffer: what a prefill
 * instance hands to a decode instance, or a cache hands to host memory (no counterpart in the
 * reference; device buffers in and out like every tensor of its runtime,
 * fastdeploy/runtime/runtime.h:90-104 BindInputTensor / GetOutputTensor sharing memory with
 * the caller).  Layout of one sequence, little-endian, every section 256-byte aligned:
 *   header 256 B  u32 magic "FDKV" (0x564b4446), version 1, cache_quant_type, hkv, head_dim,
 *                 block_size, num_tokens, num_pages; u64 scales_off, sums_off, pages_off,
 *                 total_bytes; zero to the end
 *   scales        f32 K [hkv, head_dim], f32 V [hkv, head_dim]
 *   sums          u64 [num_pages][2][hkv]: sum of the 32-bit words of each (page, K|V, head) tile
 *   pages         u8 [num_pages][2][hkv][block_size][head_dim]; rows past num_tokens are zero, so
 *                 the bytes depend on the sequence's content only, not on stale cache rows
 * fdattn_kv_wire_bytes = total_bytes of a sequence of num_tokens tokens (0 for a bad shape).
 * Sequence b of a call lives at wire + wire_offsets[b] (device int64 [batch], multiples of 256);
 * num_tokens (device int32 [batch]) must hold the values the host sized the offsets with, each
 * <= max_tokens.  One launch per call, nothing synchronises.
 */
FDATTN_API size_t fdattn_kv_wire_bytes(int num_tokens, int hkv, int head_dim, int block_size);
/* The same for any cache format.  The dynamic formats carry their scales page by page: the scales section is
 * f32 [num_pages][2][hkv][block_size] (zero for rows past num_tokens), every tile's sum includes its scale row,
 * the import stores the rows into k_scale / v_scale (the scale caches, required then) and status bit 4 is
 * not used. */
FDATTN_API size_t fdattn_kv_wire_bytes_for(int num_tokens, int hkv, int head_dim, int block_size, int cache_quant_type);
/* cache -> wire.  A table entry outside [0, num_blocks) exports as a page of zeros. */
FDATTN_API int fdattn_kv_export(const void* key_cache, const void* value_cache, const float* k_scale,
                                const float* v_scale, const int32_t* block_tables, const int32_t* num_tokens,
                                const int64_t* wire_offsets, void* wire, int batch, int max_tokens, int hkv,
                                int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
                                int cache_quant_type, void* stream);
/* wire -> cache, into the blocks block_tables names.  status (device int32[2], zeroed by the caller):
 * [0] = OR of 1 (magic / version), 2 (header disagrees with the arguments), 4 (scales differ from
 * k_scale / v_scale; both NULL = not compared), 8 (a tile's sum disagrees), 16 (a table entry
 * outside the pool); [1] = number of tiles whose sum disagrees.  A sequence whose header fails
 * writes nothing; a tile whose sum fails has been written - discard the sequence.  No offset is
 * ever taken from the buffer: every access stays inside fdattn_kv_wire_bytes(num_tokens[b], ...). */
FDATTN_API int fdattn_kv_import(const void* wire, const int64_t* wire_offsets, void* key_cache, void* value_cache,
                                float* k_scale, float* v_scale, const int32_t* block_tables,
                                const int32_t* num_tokens, int32_t* status, int batch, int max_tokens, int hkv,
                                int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
                                int cache_quant_type, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FDATTN_H_ */