// SQAttn block selector: per-block max q.k scores over the quantised K pages and a
// per-(sequence, KV head) top-k with ties to the lower block index.
//
// The selection is DEFINED on scores computed in fp64 with the channels summed in
// ascending order.  Every product (fp32 q*scale times an int8 / e4m3 value) is exact in
// fp64, so only the order of the additions matters for the bits of a score, and that
// order is fixed: the kept indices are reproducible bit for bit on a CPU.
// The formats with one scale per stored row (DYN) take q unscaled and multiply a token's
// sum by its row's scale at the end (one more fp64 rounding); with one scale per (block,
// KV head) tile the tile's scale stands for each of its rows (scale_rows = 1).
//
// Two implementations give the same indices:
//  * exact: every block scored in fp64, one token per lane (any shape; fp64-VALU bound);
//  * fast (head_dim 128, up to 8 query heads per KV head, block_size 64): every block scored on
//    the MFMA units straight from the cache bytes (the streaming machinery of the decode
//    kernel, K tiles only - HBM bound), together with a bound eps on the error of those
//    scores.  The top-k kernel then classifies each block as surely kept (fewer than k
//    blocks could beat it even if every score were off by eps), surely dropped (k blocks
//    beat it whatever the errors are) or undecided; only the undecided blocks - those
//    within 2*eps of the k-th score, a handful - are re-scored in fp64 and ranked exactly.
#include "c8_common.h"
#include "decode_generic.h"
#include <mutex>
#include <set>
#include <utility>

#include "launch.h"

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
  int scale_rows;  // DYN: scales per tile in the scale cache: bs (one per stored row) or 1 (the tile shares one)
  RowMap rows;     // a mixed step: only its one-token decode rows are scored (q row through cu_seqlens_q)
};

constexpr int kSelMaxD = 256;
constexpr int kSelMaxG = 8;

template <int QUANT>
__device__ __forceinline__ double dq64(u32 byte) {
  if (QUANT == FDATTN_CACHE_INT8) return (double)(int)(int8_t)byte;
  return (double)e4m3_to_f32(byte);
}
// byte e (0 .. 3) of word w as a double.  e4m3: the code's exponent and mantissa bits land on the top of a double's
// (a double of exponent field E: (1 + m / 8) 2^(E - 1023), or m / 8 2^-1022 for E = 0) and one exact product with
// 2^1016 puts the value where it belongs, (1 + m / 8) 2^(E - 7) or m / 8 2^-6 - the same value as e4m3_to_f32's
template <int QUANT>
__device__ __forceinline__ double dq64_of_word(u32 w, int e) {
  if (QUANT == FDATTN_CACHE_INT8) return (double)((int)(w << (24 - 8 * e)) >> 24);
  const int sh = 17 - 8 * e;
  const u32 mag = (sh >= 0 ? w << sh : w >> -sh) & 0x00fe0000u;
  const u32 sgn = (w << (24 - 8 * e)) & 0x80000000u;
  return __dmul_rn(__hiloint2double((int)(mag | sgn), 0), 0x1p1016);
}

// grid (max_blocks, hkv, batch), one wavefront: lane = token of the block
template <int QUANT, bool DYN>
__global__ __launch_bounds__(64) void sqattn_block_scores_kernel(ScoreArgs a) {
  __shared__ float qs[kSelMaxG][kSelMaxD];
  const int j = blockIdx.x, h = blockIdx.y, b = blockIdx.z, lane = threadIdx.x;
  const int g = a.hq / a.hkv, d = a.d, bs = a.bs;
  const int kv_len = a.seq_lens_decoder[b] + (a.seq_lens_this_time ? a.seq_lens_this_time[b] : 0);
  const size_t o = ((size_t)b * a.hkv + h) * a.max_blocks + j;
  const int t0 = j * bs;
  int pb = -1, qrow;
  const bool scored = decode_row(a.rows, b, qrow);
  if (scored && t0 < kv_len) pb = a.block_tables[(size_t)b * a.max_blocks + j];
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
    const float qv = bf16_to_f32(a.q[((size_t)qrow * a.hq + h * g + gi) * d + c]);
    qs[gi][c] = DYN ? qv : __fmul_rn(qv, a.k_scale[h * d + c]);
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
    const double kt = DYN ? (double)a.k_scale[((size_t)pb * a.hkv + h) * a.scale_rows + (a.scale_rows == 1 ? 0 : t)] : 1.0;
#pragma unroll
    for (int gi = 0; gi < kSelMaxG; ++gi)
      if (gi < g) best = fmax(best, DYN ? __dmul_rn(s[gi], kt) : s[gi]);
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
                                                          int max_blocks, int top_k, RowMap rows) {
  extern __shared__ double sm[];  // scores [max_blocks], then int flags/prefix
  int* keep = reinterpret_cast<int*>(sm + max_blocks);
  __shared__ int wave_tot[4];
  __shared__ int running;
  const int b = blockIdx.x / hkv, tid = threadIdx.x;
  const double* s = scores + (size_t)blockIdx.x * max_blocks;
  const int kv_len = seq_lens_decoder[b] + (seq_lens_this_time ? seq_lens_this_time[b] : 0);
  int nblk = (kv_len + bs - 1) / bs;
  if (nblk > max_blocks) nblk = max_blocks;
  int qrow;
  if (!decode_row(rows, b, qrow)) nblk = 0;  // (a mixed step: no list for rows that are not decode rows)
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

// ---------------------------------------------------------------- fast path

struct SelArgs {
  const uint16_t* q;
  const uint8_t* key_cache;
  const float* k_scale;
  const int32_t* block_tables;
  const int32_t* seq_lens_decoder;
  const int32_t* seq_lens_this_time;
  float* approx;  // [pairs][max_blocks]
  float* eps;     // [pairs]: bound that holds for every block of the pair
  float* ebound;  // [pairs][max_blocks]: per-block bound (fp8 and the dynamic formats, else NULL)
  float* scores_out;  // optional copy of approx
  int32_t* kept_blocks;
  int32_t* kept_counts;
  int batch, hkv, max_blocks, num_blocks, chunk, chunks_per_pair, top_k;
  int group;  // query heads per KV head, 1 .. 8
  RowMap rows;  // inside a mixed step: which sequences are decode rows (the others keep no block) and their q rows
  int scale_rows;  // DYN: scales per tile in the scale cache: 64 (one per stored row) or 1 (the tile shares one)
  // inside a step whose decode rows may bring several tokens (> 1): a row's MFMA rows are (token, head) pairs -
  // row v is token v / group, head v % group - token t of T scores the keys it attends to (T - 1 - t fewer than the
  // last token) and a block's score is the maximum over all the row's tokens and heads: one list per (row, KV head)
  int max_tokens;
  int bs;  // block size (64 on the int8 / fp8-MFMA scoring kernel; any on the fp16-MFMA one)
};

// this step's q rows of sequence b: false if it is not a decode row; toks = its tokens (1 outside such steps)
__device__ __forceinline__ bool sel_rows(const SelArgs& a, int b, int& qrow, int& toks) {
  toks = 1;
  if (a.max_tokens > 1) return decode_rows(a.rows, b, a.max_tokens, qrow, toks);
  return decode_row(a.rows, b, qrow);
}

// One workgroup = `chunk` consecutive blocks of one (sequence, KV head); each wavefront
// streams blocks wave, wave+4, ... through two LDS slots (one tile computing, one or two
// in flight) and leaves one fp32 score per block.
// NSET: sets of 4 query heads (MFMA rows), as in the decode kernel: 1 for groups up to 4, 2 for 5 .. 8.
template <int QUANT, bool DYN, int NSET>
__global__ __launch_bounds__(kWaves * 64, NSET > 2 ? 1 : 2) void sqattn_scores_mfma_kernel(SelArgs a) {
  __shared__ __attribute__((aligned(16))) uint8_t ldsK[kWaves][2][kTileB];  // two K slots per wavefront
  __shared__ __attribute__((aligned(16))) float ldsS[DYN ? kWaves : 1][2][kBS];  // DYN: the slots' scale rows
  const int lane = threadIdx.x & 63;
  const int wv = uni(threadIdx.x >> 6);
  // chunk-major: every XCD (workgroups are dealt to them in turn) sees every chunk position
  const int pairs = a.batch * a.hkv;
  const int ck = blockIdx.x / pairs, p = blockIdx.x - ck * pairs;
  const int b = p / a.hkv, h = p - b * a.hkv;
  const int first = ck * a.chunk;
  // Everything that depends on the block index alone is requested first and together - the table
  // entries of this chunk (two per lane), q and the K scales - so that the start of a workgroup
  // costs two round trips to memory (these, then the first tiles), not one per step of a chain.
  int pb_raw[2] = {-1, -1};
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    const int u = lane + 64 * e;
    if (u < a.chunk && first + u < a.max_blocks) pb_raw[e] = a.block_tables[(size_t)b * a.max_blocks + first + u];
  }
  int qrow, toks;
  if (!sel_rows(a, b, qrow, toks)) return;  // not a decode row of this step: nothing to score
  const int vg = a.group * toks;  // MFMA rows in use
  PairRaw raw[NSET];
#pragma unroll
  for (int t = 0; t < NSET; ++t)
    raw[t] = load_pair_issue(a.q, DYN ? nullptr : a.k_scale, a.hkv, p, qrow, lane, a.group, t, a.max_tokens > 1 ? toks : 0);
  const int kv_len = a.seq_lens_decoder[b] + (a.seq_lens_this_time ? a.seq_lens_this_time[b] : 0);
  const int n_p = min((max(kv_len, 0) + kBS - 1) / kBS, a.max_blocks);
  const int cnt = min(a.chunk, n_p - first);
  float* const srow = a.approx + (size_t)p * a.max_blocks;
  // blocks of this chunk past the sequence: -inf
  for (int j = max(first, n_p) + (int)threadIdx.x; j < min(first + a.chunk, a.max_blocks); j += blockDim.x) {
    srow[j] = -INFINITY;
    if (a.scores_out) a.scores_out[(size_t)p * a.max_blocks + j] = -INFINITY;
  }
  if (cnt <= 0) return;

  const u32 saddr0 = (u32)uni((int)lds_addr_of(ldsK[wv][0]));
  const DmaOffsets offK = dma_offsets<kShiftK>(lane);
  const int n16 = lane & 15, g4 = lane >> 4;

  int my_pb[2] = {0, 0}, my_valid[2] = {0, 0};
  {
    asm volatile("" ::"v"(pb_raw[0]), "v"(pb_raw[1]));
#pragma unroll
    for (int e = 0; e < 2; ++e)
      if (lane + 64 * e < cnt && pb_raw[e] >= 0 && pb_raw[e] < a.num_blocks) {
        my_pb[e] = pb_raw[e];
        // (not cut at the block's size, so that an earlier token's smaller count can be taken from it)
        my_valid[e] = min(max(kv_len - (first + lane + 64 * e) * kBS, 0), kBS + 4 * kMaxSetsSpec);
      }
  }
  auto unit_pb = [&](int j) { return j < 64 ? __builtin_amdgcn_readlane(my_pb[0], j) : __builtin_amdgcn_readlane(my_pb[1], j - 64); };
  auto unit_valid = [&](int j) { return j < 64 ? __builtin_amdgcn_readlane(my_valid[0], j) : __builtin_amdgcn_readlane(my_valid[1], j - 64); };
  // this lane's score row of set t is MFMA row 4 t + g4 = token (4 t + g4) / group, which sees toks - 1 - token fewer
  // keys than the row's last token
  int fewer[NSET];
#pragma unroll
  for (int t = 0; t < NSET; ++t) fewer[t] = max(toks - 1 - (4 * t + (lane >> 4)) / a.group, 0);
  const size_t tile_stride = (size_t)kBS * kD;
  const uint8_t* const kbase = a.key_cache + (size_t)h * tile_stride;
  const size_t blk_stride = (size_t)a.hkv * tile_stride;

  // DYN: a tile's 64 row scales follow it into LDS (one more direct load, counted by the waits below)
  const u32 ssaddr0 = (u32)uni((int)lds_addr_of(ldsS[DYN ? wv : 0][0]));
  const u32 lane_x4 = a.scale_rows == 1 ? 0u : (u32)lane * 4u;  // one scale per tile: every lane loads that one
  auto fetch = [&](int blk, int slot) {
    dma_tile(kbase + (size_t)blk * blk_stride, saddr0 + (u32)slot * kTileB, offK);
    if (DYN) dma_row64(a.k_scale + ((size_t)blk * a.hkv + h) * a.scale_rows, ssaddr0 + (u32)slot * (kBS * 4), lane_x4);
  };
  if (wv < cnt) fetch(unit_pb(wv), 0);
  if (wv + kWaves < cnt) fetch(unit_pb(wv + kWaves), 1);

  if (ck == 0 && wv == 0) {
    // error bound of the MFMA scores of this pair (see the top of the file): q*scale is cut to
    // 21 bits (int8) or 16 significant bits in e4m3 limbs (fp8), and sums are kept in fp32
    float amax = 0.f, sabs = 0.f;
    for (int v = 0; v < vg; ++v) {  // every (token, head) row of the pair
      const int tk = v / a.group, g = v - tk * a.group;
      float sa = 0.f, am = 0.f;
      for (int c = lane; c < kD; c += 64) {
        const float qs = fabsf(bf16_to_f32(a.q[((size_t)(qrow + tk) * a.hkv * a.group + h * a.group + g) * kD + c]) * (DYN ? 1.0f : a.k_scale[h * kD + c]));
        sa += qs;
        am = fmaxf(am, qs);
      }
      sabs = fmaxf(sabs, wave_sum(sa));
      amax = fmaxf(amax, wave_max(am));
    }
    // int8: q*scale is rounded to a multiple of step = amax/1048575, at most step/2 off per channel, times
    //   |k| <= 127 over 128 channels; the integer dot products are exact and the fp32 recombination of the
    //   three limbs adds at most a few 2^-24 of the leading term (covered by the 2048).
    // fp8: four e4m3 residual limbs leave at most 2^-16 of |q*scale| per channel (or the subnormal floor,
    //   2^-10 in units of amax/256), and the fp32 accumulation of the products adds at most 2^-17 of
    //   sum |q*scale||k|; with |k| <= 448 that is below 2^-15 * 448 * sum |q*scale| + amax * 2^-18 * 128 * 448.
    float e;
    if (QUANT == FDATTN_CACHE_INT8) e = amax * ((128.0f * 127.0f * 0.5f + 2048.0f) / 1048575.0f);
    else e = sabs * 448.0f * 3.0517578125e-5f + amax * (128.0f * 448.0f * 3.814697265625e-6f);
    // DYN: this is the bound before the row scale; every block multiplies it by its largest scale (below)
    if (lane == 0) a.eps[p] = e * 1.0001f;
  }

  if (wv >= cnt) return;
  PairState st[NSET];
  // fp8: a second operand, |q*scale| in one e4m3 limb, gives sum_c |q*scale||k| per token next to the score;
  // the error of a block's score is a small multiple of that sum (see the bound below)
  v4i aabs[NSET][2];
  float amax_pair = 0.f;  // largest |q*scale| over the channels of the pair's heads
#pragma unroll
  for (int t = 0; t < NSET; ++t) {
    float qs[2][16];
    load_pair_finish<QUANT>(raw[t], 1.0f, lane, st[t], qs);  // scores in natural units
    aabs[t][0] = aabs[t][1] = (v4i){0, 0, 0, 0};
    if (QUANT != FDATTN_CACHE_INT8) {
      const int m = lane & 15, head = m >> 2, limb = m & 3;
      // st.rs = amax / 256 of this lane's S-layout head; the A layout wants the head of row m
      const float rs_row = __shfl(st[t].rs, 16 * head, 64);
      const float inv = rs_row > 0.f ? 1.0f / rs_row : 0.f;
#pragma unroll
      for (int k2 = 0; k2 < 2; ++k2) {
        u32 pk[4] = {0, 0, 0, 0};
#pragma unroll
        for (int jj = 0; jj < 16; ++jj) {
          const float x = fabsf(qs[k2][jj]) * inv;
          const u32 code = limb == 0 ? ((u32)__builtin_amdgcn_cvt_pk_fp8_f32(x, x, 0, false) & 0xffu) : 0u;
          pk[jj >> 2] |= code << (8 * (jj & 3));
        }
        aabs[t][k2] = (v4i){(int)pk[0], (int)pk[1], (int)pk[2], (int)pk[3]};
      }
    }
    const float rs_max = fmaxf(fmaxf(__shfl(st[t].rs, 0, 64), __shfl(st[t].rs, 16, 64)), fmaxf(__shfl(st[t].rs, 32, 64), __shfl(st[t].rs, 48, 64)));
    amax_pair = fmaxf(amax_pair, rs_max * (QUANT == FDATTN_CACHE_INT8 ? 1048575.0f : 256.0f));
  }

  int it = 0;
  for (int j = wv; j < cnt; j += kWaves, ++it) {
    const int valid = unit_valid(j);
    const uint8_t* kbuf = ldsK[wv][it & 1];  // indexed, not picked from a pointer array: stays an LDS address
    if (j + kWaves >= cnt) wait_vm0(); else if (DYN) wait_vm9(); else wait_vm8();
    float sv = -INFINITY, bv = 0.f;
    float kt[4] = {1.f, 1.f, 1.f, 1.f}, ktmax = 0.f;  // DYN: scales of this lane's tokens; the block's largest
    if (DYN) {
      const float4 k4 = *reinterpret_cast<const float4*>(&ldsS[wv][it & 1][4 * n16]);
      kt[0] = k4.x; kt[1] = k4.y; kt[2] = k4.z; kt[3] = k4.w;
#pragma unroll
      for (int stl = 0; stl < 4; ++stl) {
        kt[stl] = (4 * n16 + stl < valid) ? kt[stl] : 0.f;  // (a slot past the end may hold anything)
        ktmax = fmaxf(ktmax, fabsf(kt[stl]));
      }
      ktmax = row_max16(ktmax);
    }
#pragma unroll
    for (int stl = 0; stl < 4; ++stl) {
      const int tok = 4 * n16 + stl;
      v4i kb[2];
#pragma unroll
      for (int k2 = 0; k2 < 2; ++k2) {
        const int c = g4 + 4 * k2;
        kb[k2] = *reinterpret_cast<const v4i*>(kbuf + tok * 128 + ((c ^ ((tok >> kShiftK) & 7)) * 16));
      }
#pragma unroll
      for (int t = 0; t < NSET; ++t) {
        const bool live = tok < valid - fewer[t] && 4 * t + g4 < vg;  // (rows past the pair's are zero, not scores)
        float s;
        if (QUANT == FDATTN_CACHE_INT8) {
          v4i acc = {0, 0, 0, 0};
#pragma unroll
          for (int k2 = 0; k2 < 2; ++k2) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(st[t].aq[k2], kb[k2], acc, 0, 0, 0);
          s = st[t].rs * ((float)acc.x + 128.0f * (float)acc.y + 16384.0f * (float)acc.z);
          if (DYN) s *= kt[stl];
        } else {
          v4f acc = {0.f, 0.f, 0.f, 0.f}, ab = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int k2 = 0; k2 < 2; ++k2) {
            const long a0 = ((long)(u32)st[t].aq[k2].y << 32) | (u32)st[t].aq[k2].x;
            const long a1 = ((long)(u32)st[t].aq[k2].w << 32) | (u32)st[t].aq[k2].z;
            const long b0 = ((long)(u32)kb[k2].y << 32) | (u32)kb[k2].x;
            const long b1 = ((long)(u32)kb[k2].w << 32) | (u32)kb[k2].z;
            acc = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a0, b0, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a1, b1, acc, 0, 0, 0);
            const long m0 = ((long)(u32)aabs[t][k2].y << 32) | (u32)aabs[t][k2].x;
            const long m1 = ((long)(u32)aabs[t][k2].w << 32) | (u32)aabs[t][k2].z;
            ab = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(m0, b0 & 0x7f7f7f7f7f7f7f7fL, ab, 0, 0, 0);
            ab = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(m1, b1 & 0x7f7f7f7f7f7f7f7fL, ab, 0, 0, 0);
          }
          s = st[t].rs * ((acc.x + acc.y) + (acc.z + acc.w));
          if (DYN) s *= kt[stl];
          bv = fmaxf(bv, live ? st[t].rs * ab.x * (DYN ? fabsf(kt[stl]) : 1.0f) : 0.f);
        }
        sv = fmaxf(sv, live ? s : -INFINITY);
      }
    }
    wait_lgkm0();  // tile consumed: refill its slot with the block two steps ahead
    if (j + 2 * kWaves < cnt) fetch(unit_pb(j + 2 * kWaves), it & 1);
    sv = row_max16(sv);                          // over the tokens of this head
    sv = fmaxf(sv, __shfl_xor(sv, 16, 64));      // over the 4 heads of the group
    sv = fmaxf(sv, __shfl_xor(sv, 32, 64));
    if (QUANT != FDATTN_CACHE_INT8) {
      bv = row_max16(bv);
      bv = fmaxf(bv, __shfl_xor(bv, 16, 64));
      bv = fmaxf(bv, __shfl_xor(bv, 32, 64));
      // residual of the four limbs <= 2^-16 |q*scale| per channel (or the e4m3 subnormal floor, 2^-10 in units
      // of amax/256); fp32 accumulation <= 2^-17 of sum |q*scale||k|; the one-limb |q*scale| is itself up to
      // 2^-4 low: (2^-16 + 2^-17) * (1 + 2^-4) < 2^-15.3 -> 2.5e-5
      // DYN: the product with the row scale is one more fp32 rounding, at most 2^-24 of |score| <= the token's
      // sum |q||k| x scale, which bv holds (up to 2^-4 low): + 1.3e-7
      bv = bv * (DYN ? 2.513e-5f : 2.5e-5f) + amax_pair * (128.0f * 448.0f * 3.814697265625e-6f) * 1.0001f * (DYN ? ktmax : 1.0f);
    }
    if (DYN && QUANT == FDATTN_CACHE_INT8) {
      // the per-channel format's bound for this pair (from q alone) times the block's largest row scale, plus
      // the rounding of the product with the row scale: 2^-24 of |score| <= 128 * 127 * amax * scale
      bv = amax_pair * ktmax * (((128.0f * 127.0f * 0.5f + 2048.0f) / 1048575.0f) * 1.0001f + 128.0f * 127.0f * 1.2e-7f);
    }
    if (lane == 0) {
      srow[first + j] = sv;
      if (QUANT != FDATTN_CACHE_INT8 || DYN) a.ebound[(size_t)p * a.max_blocks + first + j] = bv;
      if (a.scores_out) a.scores_out[(size_t)p * a.max_blocks + first + j] = sv;
    }
  }
}

__device__ __forceinline__ unsigned order_key(float f) {
  const unsigned u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);  // unsigned order == float order
}
__device__ __forceinline__ float key_to_float(unsigned k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

constexpr int kResolveThreads = 1024;  // 16 wavefronts: the undecided blocks are re-scored one per wavefront

// Two order statistics in one sweep, by the whole workgroup (kResolveThreads threads): out[0] = the r0-th largest
// (r = 1 is the maximum) of v[j] - e[j] and out[1] = the r1-th largest of v[j] + e[j], j < n.  Radix
// selection over order-preserving integer keys, 4 passes of 8 bits.  Every pass has its own pair of
// histograms (hist: 4 x 2 x 256 ints, zeroed by the caller before its last barrier) and its own result
// slots (sel: 4 x 4 unsigneds), so a pass costs two barriers: count, then wavefront w < 2 scans histogram w
// - 4 bins per lane, one 64-lane prefix sum - for the bin where the count from the top reaches the rank.
__device__ void radix_select2_desc(const float* v, const float* e, int n, int r0, int r1, int* hist, unsigned* sel,
                                   float* out) {
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  unsigned prefix[2] = {0u, 0u}, mask = 0;
  int remaining[2] = {r0, r1};
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    int* hp = hist + 512 * pass;
    if (pass == 0) {
      // The first digit is the sign and the top of the exponent: scores of one pair share it, and 64 lanes adding to
      // one LDS word take their turns.  A wavefront adds once per distinct digit instead (one or two rounds).
      for (int j0 = 0; j0 < n; j0 += kResolveThreads) {  // (every lane of a wavefront stays in the loop: ballots)
        const int j = j0 + tid;
        const bool in = j < n;
        const unsigned k0 = in ? order_key(v[j] - e[j]) : 0u, k1 = in ? order_key(v[j] + e[j]) : 0u;
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          const unsigned bin = ((w ? k1 : k0) >> shift) & 255u;
          unsigned long long todo = __ballot(in);
          while (todo) {
            const int leader = __ffsll((long long)todo) - 1;
            const unsigned b = (unsigned)__shfl((int)bin, leader, 64);
            const unsigned long long same = __ballot(in && bin == b);
            if (lane == leader) atomicAdd(&hp[256 * w + b], (int)__popcll(same));
            todo &= ~same;
          }
        }
      }
    } else {
      for (int j = tid; j < n; j += kResolveThreads) {
        const unsigned k0 = order_key(v[j] - e[j]), k1 = order_key(v[j] + e[j]);
        if ((k0 & mask) == prefix[0]) atomicAdd(&hp[(k0 >> shift) & 255u], 1);
        if ((k1 & mask) == prefix[1]) atomicAdd(&hp[256 + ((k1 >> shift) & 255u)], 1);
      }
    }
    __syncthreads();
    if (wv < 2) {
      // lane l owns bins 255-4l .. 252-4l (descending); c[i] = their counts
      const int4 c4 = *reinterpret_cast<const int4*>(hp + 256 * wv + 252 - 4 * lane);  // bins 252-4l .. 255-4l
      const int c[4] = {c4.w, c4.z, c4.y, c4.x};
      const int mine = (c[0] + c[1]) + (c[2] + c[3]);
      int incl = mine;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int t = __shfl_up(incl, o, 64);
        if (lane >= o) incl += t;
      }
      const int rem = remaining[wv];
      const unsigned long long hit = __ballot(incl >= rem);  // never empty: the candidates number at least rem
      const int l = __ffsll((long long)hit) - 1;
      if (lane == l) {
        int before = incl - mine, i = 0;
        while (i < 3 && before + c[i] < rem) before += c[i++];
        sel[4 * pass + 2 * wv] = (unsigned)(255 - 4 * l - i);
        sel[4 * pass + 2 * wv + 1] = (unsigned)(rem - before);
      }
    }
    __syncthreads();
    prefix[0] |= sel[4 * pass] << shift;
    prefix[1] |= sel[4 * pass + 2] << shift;
    mask |= 255u << shift;
    remaining[0] = (int)sel[4 * pass + 1];
    remaining[1] = (int)sel[4 * pass + 3];
  }
  out[0] = key_to_float(prefix[0]);
  out[1] = key_to_float(prefix[1]);
}

// One workgroup per (sequence, KV head): classify, re-score the undecided blocks in fp64, emit.
// MT: rows of several tokens (SelArgs::max_tokens > 1): the rows of the re-scoring are (token, head) pairs with their
// own visible lengths, taken four at a time (sixteen fp64 accumulators would not fit beside the row).
// DD: head_dim (128 behind the int8 / fp8-MFMA scoring kernel; 64, 128 or 256 behind the fp16-MFMA one); the block size is
// a.bs.
template <int QUANT, bool DYN, int NSET, bool MT = false, int DD = kD>
__global__ __launch_bounds__(kResolveThreads) void sqattn_resolve_kernel(SelArgs a) {
  constexpr int GH = kG * NSET;  // query heads the re-scoring loop is unrolled for (those past the group are skipped)
  extern __shared__ double smd[];                  // exact scores of undecided blocks [max_blocks]
  float* sf = reinterpret_cast<float*>(smd + a.max_blocks);      // approx scores [max_blocks]
  float* se = sf + a.max_blocks;                                  // error bounds [max_blocks]
  int* state = reinterpret_cast<int*>(se + a.max_blocks);         // 0 dropped, 1 kept, 2 undecided
  int* ulist = state + a.max_blocks;                              // undecided block ids
  int* tbl = ulist + a.max_blocks;                                // this sequence's block table row
  __shared__ __attribute__((aligned(16))) double qs[DD][GH];  // q * k_scale as the re-scoring takes it: a channel's rows side by side
  __shared__ int few[GH];  // row g is token g / group, which sees toks - 1 - token fewer keys than the row's last token
  __shared__ int n_in, n_unc, wave_tot[kResolveThreads / 64], running;
  __shared__ __attribute__((aligned(16))) int hist[4 * 512];
  __shared__ unsigned sel[16];
  const int p = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int b = p / a.hkv, h = p - b * a.hkv;
  int qrow, toks;
  if (!sel_rows(a, b, qrow, toks)) {  // not a decode row of this step: it keeps no block
    if (tid == 0) a.kept_counts[p] = 0;
    return;
  }
  const int vg = a.group * toks;  // (token, head) rows of the pair
  if (MT && tid < GH) few[tid] = max(toks - 1 - tid / a.group, 0);
  // Everything the kernel will need from memory is requested here, in one round trip: the scores and
  // their bounds, the table row and q * k_scale of the re-scoring step (needed only if a block stays
  // undecided, but a second and third trip would cost more than these few KB).
  const float* s = a.approx + (size_t)p * a.max_blocks;
  const float* eb = a.ebound ? a.ebound + (size_t)p * a.max_blocks : nullptr;
  const float eps = a.eps[p];
  for (int j = tid; j < a.max_blocks; j += kResolveThreads) {
    sf[j] = s[j];
    se[j] = eb ? eb[j] : eps;
    tbl[j] = a.block_tables[(size_t)b * a.max_blocks + j];
  }
  for (int i = tid; i < GH * DD; i += kResolveThreads) {
    const int g = i / DD, c = i % DD;
    const int tk = g / a.group, hd = g - tk * a.group;
    // rows past the pair's are zero: the re-scoring loop runs over all GH rows without a test, the maximum skips them
    const float qv = g < vg ? bf16_to_f32(a.q[((size_t)(qrow + tk) * a.hkv * a.group + h * a.group + hd) * DD + c]) : 0.f;
    qs[c][g] = (double)(DYN ? qv : __fmul_rn(qv, a.k_scale[h * DD + c]));
  }
  const int kv_len = a.seq_lens_decoder[b] + (a.seq_lens_this_time ? a.seq_lens_this_time[b] : 0);
  const int nblk = min((max(kv_len, 0) + a.bs - 1) / a.bs, a.max_blocks);
  const int k = min(a.top_k, nblk);
  int32_t* out = a.kept_blocks + (size_t)p * a.top_k;
  if (tid == 0) { n_in = 0; n_unc = 0; running = 0; }
  for (int i = tid; i < 4 * 512; i += kResolveThreads) hist[i] = 0;
  __syncthreads();
  if (k < nblk) {
    // With score i known to within e_i (L_i = s_i - e_i, U_i = s_i + e_i): block j is surely kept if
    // L_j > the (k+1)-th largest U (then at most k blocks, itself included, can reach it) and surely
    // dropped if U_j < the k-th largest L (then k blocks beat it for certain); the rest is undecided.
    // k-th largest lower bound and (k+1)-th largest upper bound by radix selection, both in the same
    // four passes - not by ranking every block against every other
    float both[2];
    radix_select2_desc(sf, se, nblk, k, k + 1, hist, sel, both);
    const float lk = both[0], uk1 = both[1];
    for (int j = tid; j < nblk; j += kResolveThreads) {
      const float lj = sf[j] - se[j], uj = sf[j] + se[j];
      int stt = 2;
      if (lj > uk1) stt = 1;
      else if (uj < lk) stt = 0;
      state[j] = stt;
      if (stt == 1) atomicAdd(&n_in, 1);
      if (stt == 2) ulist[atomicAdd(&n_unc, 1)] = j;
    }
    __syncthreads();
    const int nu = n_unc, need = k - n_in;
    if (nu > 0) {

      // exact score of each undecided block: fp64, channels in ascending order, lane = token; blocks of 32 tokens or
      // fewer (a power of two) sit side by side in a wavefront, 64 / bs of them
      const bool side_by_side = a.bs <= 32 && (a.bs & (a.bs - 1)) == 0;
      const int span = side_by_side ? a.bs : 64, per_wave = 64 / span;
      const int sub = side_by_side ? lane >> (__ffs(a.bs) - 1) : 0, tok0 = lane - sub * span;
      for (int u0 = wv * per_wave; u0 < nu; u0 += (kResolveThreads / 64) * per_wave) {
        const int u = u0 + sub;
        const bool have = u < nu;
        const int j = have ? ulist[u] : 0;
        const int pb = have ? tbl[j] : -1;
        double best = -INFINITY;
        // (blocks of more than 64 tokens: 64 at a time)
        for (int tok = tok0; tok - tok0 < a.bs; tok += 64)
        if (pb >= 0 && pb < a.num_blocks && tok < a.bs && j * a.bs + tok < kv_len) {
          const uint8_t* kr = a.key_cache + (((size_t)pb * a.hkv + h) * a.bs + tok) * DD;
          // the whole row is requested before any of it is used (eight 16-byte loads in flight: one round trip to
          // memory instead of eight in a row - this loop is most of the kernel's time when a block is undecided); the
          // loop over the eight pieces stays rolled (unrolled it would not fit the registers) and picks its piece by
          // comparisons, every register index a constant
          // (head_dim 256: the row in two halves of eight pieces, requested per pass - sixteen would not fit beside the
          // accumulators at 16 wavefronts per workgroup)
          constexpr int RP = DD / 16 > 8 ? 8 : DD / 16, RG = DD / 16 / RP;  // pieces per group, groups per row
          uint4 row[RP];
          auto load_group = [&](int hg) {
#pragma unroll
            for (int i = 0; i < RP; ++i) row[i] = *reinterpret_cast<const uint4*>(kr + 16 * (RP * hg + i));
          };
          if (RG == 1) load_group(0);
          constexpr int GP = 4;  // rows per pass (eight accumulators would not fit beside the row at 16 wavefronts per workgroup)
          const int lim = kv_len - j * a.bs - tok;  // a row that sees `few` fewer keys sees this one if few < lim
#pragma unroll 1
          for (int g0 = 0; g0 < GH; g0 += GP) {
            double acc[GP];
#pragma unroll
            for (int g = 0; g < GP; ++g) acc[g] = 0.0;
            // the products are exact in fp64, so fma(q, k, acc) rounds exactly like add(acc, mul(q, k))
#pragma unroll 1
            for (int hg = 0; hg < RG; ++hg) {
              if (RG > 1) load_group(hg);
#pragma unroll 1
              for (int i = 0; i < RP; ++i) {
                const int c = 16 * (RP * hg + i);
                u32 ws[4] = {row[0].x, row[0].y, row[0].z, row[0].w};
#pragma unroll
                for (int j = 1; j < RP; ++j) {
                  const bool pick = i == j;
                  ws[0] = pick ? row[j].x : ws[0];
                  ws[1] = pick ? row[j].y : ws[1];
                  ws[2] = pick ? row[j].z : ws[2];
                  ws[3] = pick ? row[j].w : ws[3];
                }
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                  const double kv = dq64_of_word<QUANT>(ws[e >> 2], e & 3);
                  const double2* const qrow2 = reinterpret_cast<const double2*>(&qs[c + e][g0]);  // (the same address in every lane)
#pragma unroll
                  for (int g = 0; g < GP; g += 2) {
                    const double2 qq = qrow2[g >> 1];
                    acc[g] = __fma_rn(qq.x, kv, acc[g]);
                    acc[g + 1] = __fma_rn(qq.y, kv, acc[g + 1]);
                  }
                }
              }
            }
            if (DYN) {
              const double kt = (double)a.k_scale[((size_t)pb * a.hkv + h) * a.scale_rows + (a.scale_rows == 1 ? 0 : tok)];
#pragma unroll
              for (int g = 0; g < GP; ++g) acc[g] = __dmul_rn(acc[g], kt);
            }
#pragma unroll
            for (int g = 0; g < GP; ++g) {
              if (g0 + g < vg && (!MT || few[g0 + g] < lim)) best = fmax(best, acc[g]);
            }
          }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1)
          if (off < span) best = fmax(best, __shfl_xor(best, off, 64));
        if (tok0 == 0 && have) smd[u] = best;
      }
      __syncthreads();
      // the `need` best undecided blocks: exact score descending, block index ascending
      for (int u = tid; u < nu; u += kResolveThreads) {
        const double su = smd[u];
        const int ju = ulist[u];
        int rank = 0;
        for (int i = 0; i < nu; ++i) {
          const double si = smd[i];
          rank += (si > su) || (si == su && ulist[i] < ju);
        }
        state[ju] = rank < need ? 1 : 0;
      }
      __syncthreads();
    }
  } else {
    for (int j = tid; j < nblk; j += kResolveThreads) state[j] = 1;
    __syncthreads();
  }
  // ordered compaction of the kept blocks
  for (int base = 0; base < nblk; base += kResolveThreads) {
    const int j = base + tid;
    const int f = j < nblk ? (state[j] == 1) : 0;
    const unsigned long long bal = __ballot(f);
    const int before = __popcll(bal & ((1ull << lane) - 1ull));
    if (lane == 0) wave_tot[wv] = __popcll(bal);
    __syncthreads();
    int off = running;
    for (int ww = 0; ww < wv; ++ww) off += wave_tot[ww];
    if (f && off + before < a.top_k) out[off + before] = j;
    __syncthreads();
    if (tid == 0) {
      int tot = 0;
      for (int ww = 0; ww < kResolveThreads / 64; ++ww) tot += wave_tot[ww];
      running += tot;
    }
    __syncthreads();
  }
  for (int j = k + tid; j < a.top_k; j += kResolveThreads) out[j] = -1;
  if (tid == 0) a.kept_counts[p] = k;
}

// the shapes of the fp16-MFMA scoring pass (decode_tiles.hip): head_dim 64 / 128 / 256, any block size up to 256, up to 8
// query heads per KV head, rows of one token
constexpr size_t kResolveLdsPerBlock = sizeof(double) + 2 * sizeof(float) + 3 * sizeof(int);  // the resolve kernel's dynamic LDS
// A launch with more dynamic LDS than every kernel may have by default (64 KiB): the limit is a per-device property of
// the kernel, raised once per device to `most`.
static hipError_t allow_lds(const void* kernel, size_t bytes, size_t most) {
  if (bytes <= 64 * 1024) return hipSuccess;
  static std::mutex mu;
  static std::set<std::pair<const void*, int>> raised;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  std::lock_guard<std::mutex> lock(mu);
  if (raised.count({kernel, dev})) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)most);
  if (e == hipSuccess) raised.insert({kernel, dev});
  return e;
}
// (4096 blocks per sequence: 28 B of LDS per block in the resolve kernel, 112 KiB of the CU's 160)
constexpr int kSelTilesMaxBlocks = 4096;
static bool sel_tiles_supported(int hq, int hkv, int d, int bs, int max_blocks) {
  return (d == 64 || d == 128 || d == 256) && hkv > 0 && hq % hkv == 0 && hq / hkv <= kG * kMaxSets && bs >= 1 && bs <= 256 &&
         max_blocks <= kSelTilesMaxBlocks;
}
static bool sel_fast_supported(int hq, int hkv, int d, int bs, int max_blocks) {
  return d == kD && hkv > 0 && hq % hkv == 0 && hq / hkv <= kG * kMaxSets && bs == kBS &&
         max_blocks <= 2048;  // 28 B of LDS per block in the resolve kernel
}

}  // namespace fdattn

using namespace fdattn;

extern "C" size_t fdattn_sqattn_workspace_bytes(int batch, int hkv, int max_blocks_per_seq) {
  if (batch <= 0 || hkv <= 0 || max_blocks_per_seq <= 0) return 256;
  size_t n = (size_t)batch * hkv * ((size_t)max_blocks_per_seq * sizeof(double) + sizeof(float));
  return (n + 255) & ~(size_t)255;
}

namespace fdattn {
bool sqattn_fast_supported(int hq, int hkv, int d, int bs, int max_blocks) { return sel_fast_supported(hq, hkv, d, bs, max_blocks); }
}

static int sqattn_select_impl(bool allow_fast, const void* q, const void* key_cache, const float* cache_k_scale,
                                    const int32_t* block_tables, const int32_t* seq_lens_decoder,
                                    const int32_t* seq_lens_this_time, float* scores, int32_t* kept_blocks,
                                    int32_t* kept_counts, void* workspace, size_t workspace_bytes, int batch,
                                    int hq, int hkv, int head_dim, int block_size, int max_blocks_per_seq,
                                    int num_blocks, int top_k, int cache_quant_type, void* stream,
                                    RowMap rows = RowMap{nullptr, nullptr}, int max_tokens = 1) {
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
  if (!quant_known(cache_quant_type))
    return fail(FDATTN_ERR_QUANT, "fdattn_sqattn_select: unknown cache_quant_type %d", cache_quant_type);
  const size_t need = (size_t)batch * hkv * ((size_t)max_blocks_per_seq * sizeof(double) + sizeof(float));
  if (workspace_bytes < need)
    return fail(FDATTN_ERR_WORKSPACE, "fdattn_sqattn_select: workspace %zu B < required %zu B", workspace_bytes, need);
  hipStream_t s = (hipStream_t)stream;
  if (allow_fast && sel_fast_supported(hq, hkv, head_dim, block_size, max_blocks_per_seq)) {
    const int pairs = batch * hkv;
    const int chunk = c8_pick_chunk(pairs, max_blocks_per_seq);
    const int cpp = (max_blocks_per_seq + chunk - 1) / chunk;
    float* approx = (float*)workspace;
    float* ebound = approx + (size_t)pairs * max_blocks_per_seq;
    float* eps = ebound + (size_t)pairs * max_blocks_per_seq;
    SelArgs sa{(const uint16_t*)q, (const uint8_t*)key_cache, cache_k_scale, block_tables, seq_lens_decoder,
               seq_lens_this_time, approx, eps, cache_quant_type == FDATTN_CACHE_INT8 ? nullptr : ebound, scores,
               kept_blocks, kept_counts, batch, hkv,
               max_blocks_per_seq, num_blocks, chunk, cpp, top_k, hq / hkv, rows, scale_rows(cache_quant_type, kBS),
               max_tokens, kBS};
    const size_t shm2 = (size_t)max_blocks_per_seq * (sizeof(double) + 2 * sizeof(float) + 3 * sizeof(int));
    const dim3 g1(pairs * cpp), g2(pairs), b1(256), b2(kResolveThreads);
    const int sets = (hq / hkv * max_tokens + kG - 1) / kG;  // sets of four MFMA rows: (token, head) pairs
#define FDATTN_SEL_LAUNCH_N(Q, D, N)                                                                                \
  do {                                                                                                              \
    hipLaunchKernelGGL((sqattn_scores_mfma_kernel<Q, D, N>), g1, b1, 0, s, sa);                                     \
    if (max_tokens > 1) hipLaunchKernelGGL((sqattn_resolve_kernel<Q, D, N, true>), g2, b2, shm2, s, sa);            \
    else if constexpr (N <= kMaxSets) hipLaunchKernelGGL((sqattn_resolve_kernel<Q, D, N>), g2, b2, shm2, s, sa);    \
  } while (0)
#define FDATTN_SEL_LAUNCH(Q, D)                                                                                     \
  do {                                                                                                              \
    if (sets == 1) FDATTN_SEL_LAUNCH_N(Q, D, 1);                                                                    \
    else if (sets == 2) FDATTN_SEL_LAUNCH_N(Q, D, 2);                                                               \
    else if (sets == 3) FDATTN_SEL_LAUNCH_N(Q, D, 3);                                                               \
    else FDATTN_SEL_LAUNCH_N(Q, D, 4);                                                                              \
  } while (0)
    if (cache_quant_type == FDATTN_CACHE_INT8) FDATTN_SEL_LAUNCH(FDATTN_CACHE_INT8, false);
    else if (cache_quant_type == FDATTN_CACHE_FP8_E4M3) FDATTN_SEL_LAUNCH(FDATTN_CACHE_FP8_E4M3, false);
    else if (quant_bytes(cache_quant_type) == FDATTN_CACHE_INT8) FDATTN_SEL_LAUNCH(FDATTN_CACHE_INT8, true);
    else FDATTN_SEL_LAUNCH(FDATTN_CACHE_FP8_E4M3, true);
#undef FDATTN_SEL_LAUNCH
#undef FDATTN_SEL_LAUNCH_N
    return check_launch("fdattn_sqattn_select (mfma)");
  }
  if (max_tokens > 1)
    return fail(FDATTN_ERR_SHAPE, "fdattn_sqattn_select: rows of several tokens need the MFMA selector's shapes");
  if (allow_fast && sel_tiles_supported(hq, hkv, head_dim, block_size, max_blocks_per_seq)) {
    // head_dim 64 / 128 / 256 at any block size: scores and bounds from the fp16-MFMA decode kernel's K half, then the
    // same classification and fp64 re-scoring of the undecided blocks
    const int pairs = batch * hkv;
    float* approx = (float*)workspace;
    float* ebound = approx + (size_t)pairs * max_blocks_per_seq;
    float* eps = ebound + (size_t)pairs * max_blocks_per_seq;
    const bool dyn = quant_dynamic(cache_quant_type);
    long long max_keys = (long long)max_blocks_per_seq * block_size;
    if (max_keys > 0x7fffffffLL) max_keys = 0x7fffffffLL;
    int splits = decode_tiles_splits(pairs, head_dim, (int)max_keys, 64);
    // (a split's blocks have their maxima in the scoring workgroup's LDS: at most kSelTilesMaxBlocksPerSplit of them)
    const int least = (max_blocks_per_seq + kSelTilesMaxBlocksPerSplit - 1) / kSelTilesMaxBlocksPerSplit;
    if (splits < least) splits = least;
    if (splits > max_blocks_per_seq) splits = max_blocks_per_seq;
    const int per = (max_blocks_per_seq + splits - 1) / splits;
    GenericDecodeArgs ga{};
    ga.q = (const uint16_t*)q, ga.key_cache = (const uint8_t*)key_cache, ga.k_scale = cache_k_scale;
    ga.block_tables = block_tables, ga.seq_lens_decoder = seq_lens_decoder, ga.seq_lens_this_time = seq_lens_this_time;
    ga.rows = rows, ga.batch = batch, ga.hq = hq, ga.hkv = hkv, ga.d = head_dim, ga.bs = block_size;
    ga.max_blocks = max_blocks_per_seq, ga.num_blocks = num_blocks, ga.max_splits = splits, ga.sm_scale = 1.0f;
    ga.scale_rows = scale_rows(cache_quant_type, block_size), ga.max_tokens = 1;
    ga.sel_approx = approx, ga.sel_ebound = dyn ? ebound : nullptr, ga.sel_eps = eps, ga.sel_scores_out = scores;
    ga.sel_blocks_per_split = per;
    const hipError_t e = sqattn_scores_tiles_launch(ga, cache_quant_type, s);
    if (e != hipSuccess) return fail((int)e, "fdattn_sqattn_select (fp16-mfma scores): %s", hipGetErrorString(e));
    int rc = check_launch("fdattn_sqattn_select (fp16-mfma scores)");
    if (rc) return rc;
    SelArgs sa{(const uint16_t*)q, (const uint8_t*)key_cache, cache_k_scale, block_tables, seq_lens_decoder,
               seq_lens_this_time, approx, eps, dyn ? ebound : nullptr, nullptr, kept_blocks, kept_counts, batch, hkv,
               max_blocks_per_seq, num_blocks, 0, 0, top_k, hq / hkv, rows, scale_rows(cache_quant_type, block_size), 1,
               block_size};
    const size_t shm2 = (size_t)max_blocks_per_seq * kResolveLdsPerBlock;
    const dim3 g2(pairs), b2(kResolveThreads);
#define FDATTN_RES_LAUNCH_N(Q, DY, N, DD)                                                                 \
  do {                                                                                                   \
    const hipError_t er = allow_lds((const void*)sqattn_resolve_kernel<Q, DY, N, false, DD>, shm2,        \
                                    (size_t)kSelTilesMaxBlocks * kResolveLdsPerBlock);                    \
    if (er != hipSuccess) return fail((int)er, "fdattn_sqattn_select (resolve): %s", hipGetErrorString(er)); \
    hipLaunchKernelGGL((sqattn_resolve_kernel<Q, DY, N, false, DD>), g2, b2, shm2, s, sa);               \
  } while (0)
#define FDATTN_RES_LAUNCH(Q, DY, DD)                                                                      \
  do {                                                                                                   \
    if (hq / hkv <= kG) FDATTN_RES_LAUNCH_N(Q, DY, 1, DD);                                               \
    else FDATTN_RES_LAUNCH_N(Q, DY, 2, DD);                                                              \
  } while (0)
#define FDATTN_RES_LAUNCH_D(Q, DY)                                     \
  do {                                                                 \
    if (head_dim == 64) FDATTN_RES_LAUNCH(Q, DY, 64);                  \
    else if (head_dim == 128) FDATTN_RES_LAUNCH(Q, DY, 128);           \
    else FDATTN_RES_LAUNCH(Q, DY, 256);                                \
  } while (0)
    if (cache_quant_type == FDATTN_CACHE_INT8) FDATTN_RES_LAUNCH_D(FDATTN_CACHE_INT8, false);
    else if (cache_quant_type == FDATTN_CACHE_FP8_E4M3) FDATTN_RES_LAUNCH_D(FDATTN_CACHE_FP8_E4M3, false);
    else if (quant_bytes(cache_quant_type) == FDATTN_CACHE_INT8) FDATTN_RES_LAUNCH_D(FDATTN_CACHE_INT8, true);
    else FDATTN_RES_LAUNCH_D(FDATTN_CACHE_FP8_E4M3, true);
#undef FDATTN_RES_LAUNCH_D
#undef FDATTN_RES_LAUNCH
#undef FDATTN_RES_LAUNCH_N
    return check_launch("fdattn_sqattn_select (resolve)");
  }
  ScoreArgs a{(const uint16_t*)q, (const uint8_t*)key_cache, cache_k_scale, block_tables, seq_lens_decoder,
              seq_lens_this_time, (double*)workspace, scores, batch, hq, hkv, head_dim, block_size,
              max_blocks_per_seq, num_blocks, scale_rows(cache_quant_type, block_size), rows};
  dim3 grid(max_blocks_per_seq, hkv, batch);
  if (cache_quant_type == FDATTN_CACHE_INT8)
    hipLaunchKernelGGL((sqattn_block_scores_kernel<FDATTN_CACHE_INT8, false>), grid, dim3(64), 0, s, a);
  else if (cache_quant_type == FDATTN_CACHE_FP8_E4M3)
    hipLaunchKernelGGL((sqattn_block_scores_kernel<FDATTN_CACHE_FP8_E4M3, false>), grid, dim3(64), 0, s, a);
  else if (quant_bytes(cache_quant_type) == FDATTN_CACHE_INT8)
    hipLaunchKernelGGL((sqattn_block_scores_kernel<FDATTN_CACHE_INT8, true>), grid, dim3(64), 0, s, a);
  else
    hipLaunchKernelGGL((sqattn_block_scores_kernel<FDATTN_CACHE_FP8_E4M3, true>), grid, dim3(64), 0, s, a);
  int rc = check_launch("fdattn_sqattn_select (scores)");
  if (rc) return rc;
  const size_t shm = (size_t)max_blocks_per_seq * (sizeof(double) + sizeof(int));
  hipLaunchKernelGGL(sqattn_topk_kernel, dim3(batch * hkv), dim3(256), shm, s, (const double*)workspace,
                     seq_lens_decoder, seq_lens_this_time, kept_blocks, kept_counts, hkv, block_size,
                     max_blocks_per_seq, top_k, rows);
  return check_launch("fdattn_sqattn_select (top-k)");
}

extern "C" int fdattn_sqattn_select(const void* q, const void* key_cache, const float* cache_k_scale,
                                    const int32_t* block_tables, const int32_t* seq_lens_decoder,
                                    const int32_t* seq_lens_this_time, float* scores, int32_t* kept_blocks,
                                    int32_t* kept_counts, void* workspace, size_t workspace_bytes, int batch,
                                    int hq, int hkv, int head_dim, int block_size, int max_blocks_per_seq,
                                    int num_blocks, int top_k, int cache_quant_type, void* stream) {
  return sqattn_select_impl(true, q, key_cache, cache_k_scale, block_tables, seq_lens_decoder, seq_lens_this_time,
                            scores, kept_blocks, kept_counts, workspace, workspace_bytes, batch, hq, hkv, head_dim,
                            block_size, max_blocks_per_seq, num_blocks, top_k, cache_quant_type, stream);
}

extern "C" int fdattn_sqattn_path(int hq, int hkv, int head_dim, int block_size, int max_blocks_per_seq) {
  if (sel_fast_supported(hq, hkv, head_dim, block_size, max_blocks_per_seq)) return 1;
  return sel_tiles_supported(hq, hkv, head_dim, block_size, max_blocks_per_seq) ? 2 : 0;
}

extern "C" int fdattn_sqattn_select_exact(const void* q, const void* key_cache, const float* cache_k_scale,
                                          const int32_t* block_tables, const int32_t* seq_lens_decoder,
                                          const int32_t* seq_lens_this_time, float* scores, int32_t* kept_blocks,
                                          int32_t* kept_counts, void* workspace, size_t workspace_bytes, int batch,
                                          int hq, int hkv, int head_dim, int block_size, int max_blocks_per_seq,
                                          int num_blocks, int top_k, int cache_quant_type, void* stream) {
  return sqattn_select_impl(false, q, key_cache, cache_k_scale, block_tables, seq_lens_decoder, seq_lens_this_time,
                            scores, kept_blocks, kept_counts, workspace, workspace_bytes, batch, hq, hkv, head_dim,
                            block_size, max_blocks_per_seq, num_blocks, top_k, cache_quant_type, stream);
}

namespace fdattn {
int sqattn_select_launch(const void* q, const void* key_cache, const float* cache_k_scale, const int32_t* block_tables,
                         const int32_t* seq_lens_decoder, const int32_t* seq_lens_this_time, int32_t* kept_blocks,
                         int32_t* kept_counts, void* workspace, size_t workspace_bytes, int batch, int hq, int hkv,
                         int head_dim, int block_size, int max_blocks_per_seq, int num_blocks, int top_k,
                         int cache_quant_type, hipStream_t s, RowMap rows, int max_tokens) {
  if (max_tokens < 1) max_tokens = 1;
  if (max_tokens > 1 && (!rows.cu_seqlens_q || hq / hkv * max_tokens > kG * kMaxSetsSpec ||
                         !sel_fast_supported(hq, hkv, head_dim, block_size, max_blocks_per_seq)))
    return fail(FDATTN_ERR_SHAPE, "fdattn_sqattn_select: rows of up to %d tokens need the MFMA selector's shapes and "
                "tokens x query heads per KV head <= %d", max_tokens, kG * kMaxSetsSpec);
  return sqattn_select_impl(true, q, key_cache, cache_k_scale, block_tables, seq_lens_decoder, seq_lens_this_time,
                            nullptr, kept_blocks, kept_counts, workspace, workspace_bytes, batch, hq, hkv, head_dim,
                            block_size, max_blocks_per_seq, num_blocks, top_k, cache_quant_type, (void*)s, rows, max_tokens);
}
}  // namespace fdattn
