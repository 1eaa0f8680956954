// Decode attention on the MFMA units for the shapes the int8-MFMA kernel (decode_c8.hip: head_dim 128, block_size 64)
// does not take: head_dim 64, 128 or 256 with ANY block size, up to 64 query heads per KV head (16 per workgroup),
// dense or over a list of kept blocks, every cache format.
//
// A workgroup = 4 autonomous wavefronts on one (sequence, KV head, key split); a wavefront walks every fourth tile
// of 32 keys of the split.  A tile's K and V bytes are read in whole rows (a load instruction covers 1 KB of
// consecutive rows, every row through the block table - a tile may span blocks; where it cannot, one table entry
// and constant offsets serve the tile), pass through registers into the wavefront's own two LDS tiles as they are,
// and become fp16 numbers holding the bytes' exact values on the way out of LDS.  The MFMAs are the 16 x 16 x 32
// ones (v_mfma_f32_16x16x32_f16): the 16 columns are the KV head's query heads, so that few lanes work on columns
// nobody asked for and the accumulators are small:
//   * S^T = K Q^T, two tiles of 16 keys: a lane reads its two keys' K rows in 16-byte pieces as the A operand; the
//     contraction runs over the channels in the order the pieces hold them, and Q - the per-channel K scale folded
//     in as two fp16 terms - is laid out in that order once;
//   * O^T += V^T P^T, 16 channels at a time: V is read transposed (ds_read_b64_tr_b8: 8 keys of one channel per
//     lane) as the A operand; the weights P^T are the scores' registers as they are.
// No barrier inside the walk; a tile's registers are requested again, for the wavefront's next tile, as soon as they
// have been stored, and the table entries of the tile after that and the list entries of the one after are in
// flight as well.  At the end the four wavefronts meet in LDS; a launch of one split writes the output itself, else
// one partial per (query head, split) goes to splitkv_combine_kernel.
#include <atomic>

#include "decode_generic.h"
#include "launch.h"
#include "prefill_mfma_common.h"

namespace fdattn {

namespace {

using namespace pf;

constexpr int kWavesDt = 4;

template <int D>
struct DecLay {
  // a wavefront's K and V tiles, raw bytes: a row starts 4 banks after the one before, so that neither the 16-byte
  // reads of 16 rows' pieces nor the 8 rows of a transposed read meet in a bank
  static constexpr int RS = D + 16;
  static constexpr int T_BYTES = 32 * RS;
  static constexpr int kWaveBytes = 2 * T_BYTES + 4 * 32 * (int)sizeof(float);  // + per key: score scale, log2 V scale (or the mask), 1 / V scale, position
  static constexpr int LDR = D + 1;              // floats per query head in the merge area (which reuses the tiles)
  static constexpr int kMergeOff = kWavesDt * kWaveBytes;  // then m and l of every (wavefront, column)
  // then Q: [k-step][hi, lo][quarter][column] x 16 B - as many columns as a row has (token, query head) pairs - and one slot of zeros
  static constexpr int kQOff = kMergeOff + 2 * kWavesDt * 16 * (int)sizeof(float);
  static constexpr size_t bytes(int columns) { return kQOff + (size_t)(D / 32) * 2 * 4 * columns * 16 + 16; }
  static_assert(16 * LDR * (int)sizeof(float) <= kMergeOff, "the merge area must fit the tiles");
};

// wavefronts per SIMD the registers are budgeted for: o and a tile in flight are D / 4 of them each
template <int D>
constexpr int waves_per_simd() { return D <= 64 ? 4 : (D <= 128 ? 3 : 2); }

// TB: the cache blocks a tile of 32 keys is made of when the block size says so - 1: the block size is 32 or a
// power-of-two multiple, the tile lies inside one block; 2: the block size is 16, the tile is two whole blocks - each
// with one table entry, the same for every lane, and constant per-lane offsets (FAST); 0: any other block size, every
// row through its own table entry.  MT: decode rows may bring several tokens (the one-token launches carry
// none of that bookkeeping)
// a float as an int that orders the same way (for an integer atomic maximum); the smallest int stands for "nothing yet"
__device__ __forceinline__ int score_key(float f) {
  const int u = __float_as_int(f);
  return u >= 0 ? u : u ^ 0x7fffffff;
}
__device__ __forceinline__ float key_score(int k) {
  if (k == (int)0x80000000) return -INFINITY;
  return __int_as_float(k >= 0 ? k : k ^ 0x7fffffff);
}

// SCORES: the kernel as the block selector's scoring pass - K only: per block of the split the largest score over its
// keys and the KV head's query heads (plain q . k, no softmax scale), kept in LDS while the wavefronts walk and written
// to a.sel_approx at the end, with a bound on its distance to the score summed in fp64 (a.sel_eps per pair; a.sel_ebound
// per block for the formats with scale caches).
template <int QUANT, bool DYN, int D, int TB, bool MT, bool SCORES = false>
__global__ __launch_bounds__(64 * kWavesDt, waves_per_simd<D>()) void decode_tiles_kernel(GenericDecodeArgs a) {
  using L = DecLay<D>;
  static_assert(!(SCORES && MT), "the scoring pass takes rows of one token");
  constexpr bool FAST = TB > 0;
  constexpr bool TWO_AHEAD = SCORES && FAST;  // the scoring pass keeps two K tiles in flight per wavefront (see the walk)
  constexpr int RPB = FAST ? 32 / TB : 32;  // FAST: rows of a tile per block
  constexpr int KT = D / 32, DB = D / 16, NC = D / 32;  // k-steps of S = K Q (32 channels each); 16-channel blocks of O; 16-byte chunks per lane and tensor of a tile
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int j32 = lane & 31, hf = lane >> 5, g4 = lane >> 4, c16 = lane & 15;
  const int split = blockIdx.y, nsplit = gridDim.y;
  // more than 16 query heads per KV head: sets of 16 on workgroups of their own (GA = all of them, G = this set's,
  // hq0 = its first query head)
  const int GA = a.hq / a.hkv, sets = (GA + 15) >> 4;
  const int pair = blockIdx.x / sets, set = blockIdx.x - pair * sets;
  const int G = min(16, GA - 16 * set);
  const int b = pair / a.hkv, h = pair - b * a.hkv;
  const int hq0 = h * GA + 16 * set;
  // A decode row: one token, or (max_tokens > 1) the up to max_tokens draft tokens of a speculative step: the columns
  // are then (token, query head) pairs, and token t sees the keys before the row plus the row's tokens up to itself.
  int qrow, toks = 1;
  if (MT ? !decode_rows(a.rows, b, a.max_tokens, qrow, toks) : !decode_row(a.rows, b, qrow)) return;
  const int max_tokens = MT ? a.max_tokens : 1;
  const int kv_len = a.seq_lens_decoder[b] + (a.seq_lens_this_time ? a.seq_lens_this_time[b] : 0);
  const int QC = min(16, max_tokens * G);  // columns the launch provides for
  const int tok = MT ? c16 / G : 0, head = c16 - tok * G;
  const bool live = c16 < toks * G;
  const int p0 = kv_len - toks;     // keys before the row's first token
  const int lim = p0 + tok + 1;     // this column sees keys [0, lim)
  const float sc = SCORES ? 1.0f : a.sm_scale * 1.4426950408889634f;  // logits go to the log2 domain (the scoring pass: plain scores)
  typedef __attribute__((address_space(3))) uint8_t lds_u8;
  lds_u8* const kt = (lds_u8*)lds + (size_t)wv * L::kWaveBytes;  // this wavefront's K tile, then its V tile, then its scales
  lds_u8* const vt = kt + L::T_BYTES;
  float* const wsc = reinterpret_cast<float*>(lds + (size_t)wv * (L::kWaveBytes / 2) + L::T_BYTES);
  // the scoring pass: per block of the split its largest score (as an ordered int) and its largest K scale (bits of a
  // non-negative float), behind everything the decode pass keeps in LDS
  int* const sel_bmax = reinterpret_cast<int*>(reinterpret_cast<uint8_t*>(lds) + L::bytes(16));
  unsigned* const sel_smax = reinterpret_cast<unsigned*>(sel_bmax + a.sel_blocks_per_split);

  // ---- the split's keys: units [i0, i1) of the sequence's blocks (or of its list of kept blocks), bs keys each;
  // key x of the split sits in unit i0 + x / bs at slot x % bs, and tile t holds keys 32 t .. 32 t + 31
  int nblk = (kv_len + a.bs - 1) / a.bs;
  if (nblk > a.max_blocks) nblk = a.max_blocks;
  const int32_t* list = nullptr;
  if (a.kept_blocks) {
    list = a.kept_blocks + ((size_t)b * a.hkv + h) * a.max_kept;
    nblk = min(a.kept_counts[b * a.hkv + h], a.max_kept);
  }
  nblk = max(nblk, 0);
  const int per = (nblk + nsplit - 1) / nsplit;
  const int i0 = split * per, i1 = min(nblk, i0 + per);
  const int n_x = i1 > i0 ? (i1 - i0) * a.bs : 0;
  const int n_t = (n_x + 31) >> 5;
  const int32_t* const table = a.block_tables + (size_t)b * a.max_blocks;
  // (block sizes are powers of two almost always: a shift and a mask then, not a division per key and tile)
  const int bs_shift = (a.bs & (a.bs - 1)) == 0 ? __ffs(a.bs) - 1 : -1;
  auto block_of = [&](int x) { return bs_shift >= 0 ? x >> bs_shift : x / a.bs; };
  auto slot_of = [&](int x) { return bs_shift >= 0 ? x & (a.bs - 1) : x % a.bs; };

  // ---- loads: lane -> 16-byte chunk `cch` of rows crow + RPI n of the tile (a load instruction covers RPI whole
  // rows, 1 KB), every row through its own table entry.  One tile's bytes live in registers; they go to LDS as they
  // are, and a tensor's chunks are requested again - for the wavefront's next tile - as soon as they are stored.
  constexpr int CPR = D / 16, RPI = 64 / CPR;  // chunks per row; rows per load instruction (NC = 32 / RPI of them per tensor)
  const int crow = lane / CPR, cch = lane % CPR;
  uint4 kq[NC], vq[NC];
  float ssc = 1.f;  // DYN: lanes 0 .. 31 carry a key's K scale, 32 .. 63 its V scale
  u32 okq = 0u;     // bit n: row crow + RPI n of the tile in registers is a key; bit 31: the key whose scale the lane carries is one;
                    // bit 30: one of the lane's keys lies past the row's first token (rows of several tokens mask by column there)
  constexpr u32 kLate = 1u << 30;
  constexpr int NP = !MT ? 1 : (FAST ? TB : NC);
  int posq[NP];  // MT: the positions of the lane's rows of the tile in registers (FAST: of the first row of each of the tile's blocks)
#pragma unroll
  for (int n = 0; n < NP; ++n) posq[n] = 0;
  // the logical block of key r of tile t (-1: none), its physical block (-1: none)
  auto logical = [&](int t, int r) {
    const int x = 32 * t + r;
    if (x >= n_x) return -1;
    const int u = i0 + block_of(x);
    if constexpr (SCORES) return u;  // (the scoring pass walks the sequence's own blocks)
    return list ? list[u] : u;
  };
  auto physical = [&](int lb) { return lb >= 0 && lb < a.max_blocks ? table[lb] : -1; };
  // the entry of lb clamped into the table, without a branch around the load: the compiler then counts the loads in
  // flight across it instead of waiting for all of them (the scoring pass keeps another tile's bytes in flight over
  // this load)
  // and whether lb is a block at all is asked when the entry is used (request): a test here would wait for the load
  auto physical_always = [&](int lb) { return table[min(max(lb, 0), max(a.max_blocks, 1) - 1)]; };
  // cache row of key r of tile t given its blocks (false: none; row 0 of the cache is read instead, zeroed and masked later)
  auto cache_row = [&](int t, int r, int lb, int pb, u32& row, int& pos) {
    const int off = slot_of(32 * t + r);
    const bool ok = pb >= 0 && pb < a.num_blocks && (long long)lb * a.bs + off < kv_len;
    row = ok ? ((u32)pb * a.hkv + h) * a.bs + off : 0u;
    pos = ok ? lb * a.bs + off : 0x7fffffff;
    return ok;
  };
  constexpr int NB = FAST ? TB : NC;
  int lb1[NB], pb1[NB], lb2[NB];  // the blocks of this lane's rows of the next tile to request (FAST: of the tile); the logical ones of the tile after
  int lbs1 = -1, pbs1 = -1, lbs2 = -1;  // DYN, not FAST: the same for the key whose scale the lane carries
  const u32 lane_off = (u32)crow * D + 16 * cch;  // FAST: this lane's chunk of the first RPI rows of a tile
  // requests tile t's chunks into kd (and vq) given its rows' blocks lbr / pbr; returns the keys-that-are bits
  auto request = [&](int t, uint4 (&kd)[NC], float& sd, const int (&lbr)[NB], const int (&pbr)[NB]) {
    u32 ok = 0;
    if constexpr (FAST) {
      static_assert(RPI <= RPB, "a load instruction's rows must lie inside one block");
      const uint8_t* kp[TB];
      const uint8_t* vp[TB];
      long long left[TB];  // keys from the block's first row of the tile to the sequence's end
      bool blk[TB];
      size_t row0[TB], tile_id[TB];  // the tile's first row of block e in the caches; (block, KV head)
#pragma unroll
      for (int e = 0; e < TB; ++e) {
        const int lb = __builtin_amdgcn_readfirstlane(lbr[e]), pb = __builtin_amdgcn_readfirstlane(pbr[e]);
        const int off0 = TB == 1 ? (32 * t) & (a.bs - 1) : 0;
        blk[e] = pb >= 0 && pb < a.num_blocks && (!TWO_AHEAD || (lb >= 0 && lb < a.max_blocks));
        left[e] = (long long)kv_len - ((long long)lb * a.bs + off0);
        // (a block that is none reads block 0; rows past the sequence's end lie in the tile's block: zeroed and masked later)
        tile_id[e] = blk[e] ? (size_t)pb * a.hkv + h : 0;
        row0[e] = blk[e] ? tile_id[e] * a.bs + off0 : 0;
        kp[e] = a.key_cache + row0[e] * D + lane_off;
        vp[e] = a.value_cache + row0[e] * D + lane_off;
        if constexpr (MT) {
          posq[e] = blk[e] ? lb * a.bs + off0 : 0x7fffffff;
          if (blk[e] && left[e] > 0 && (long long)posq[e] + min(left[e], (long long)RPB) - 1 > p0) ok |= kLate;
        }
      }
#pragma unroll
      for (int n = 0; n < NC; ++n) {
        const int e = (RPI * n) / RPB, in_block = RPI * n - RPB * e;  // (constants once unrolled)
        kd[n] = nt_load16(kp[e] + in_block * D);
        if constexpr (!SCORES) vq[n] = nt_load16(vp[e] + in_block * D);
        ok |= blk[e] && crow + in_block < left[e] ? 1u << n : 0u;
      }
      if (DYN) {
        const int e = TB == 1 ? 0 : j32 / RPB, in_block = j32 - RPB * e;
        bool blk_e = blk[0];
        long long left_e = left[0];
        size_t row0_e = row0[0], tile_e = tile_id[0];
#pragma unroll
        for (int x = 1; x < TB; ++x)
          if (e == x) blk_e = blk[x], left_e = left[x], row0_e = row0[x], tile_e = tile_id[x];
        const bool oks = blk_e && in_block < left_e;
        ok |= oks ? 1u << 31 : 0u;
        const size_t srow = a.scale_rows == 1 ? tile_e : row0_e + in_block;
        sd = hf && !SCORES ? a.v_scale[srow] : a.k_scale[srow];
      }
      return ok;
    }
#pragma unroll
    for (int n = 0; n < NC; ++n) {
      u32 row;
      int pos;
      const bool okn = cache_row(t, crow + RPI * n, lbr[n], pbr[n], row, pos);
      ok |= okn ? 1u << n : 0u;
      if constexpr (MT) {
        ok |= okn && pos > p0 ? kLate : 0u;
        if constexpr (!FAST) posq[n] = pos;
      }
      kd[n] = nt_load16(a.key_cache + (size_t)row * D + 16 * cch);
      if constexpr (!SCORES) vq[n] = nt_load16(a.value_cache + (size_t)row * D + 16 * cch);
    }
    if (DYN) {
      u32 row;
      int pos;
      const bool oks = cache_row(t, j32, lbs1, pbs1, row, pos);
      ok |= oks ? 1u << 31 : 0u;
      const size_t srow = a.scale_rows == 1 ? (oks ? (size_t)pbs1 * a.hkv + h : 0) : row;  // one scale per (block, head) tile, or per stored row
      sd = hf && !SCORES ? a.v_scale[srow] : a.k_scale[srow];
    }
    return ok;
  };
  // moves the block pipeline on by one tile: t is the tile whose logical blocks are requested now
  auto advance = [&](int t) {
#pragma unroll
    for (int n = 0; n < NB; ++n) lb1[n] = lb2[n], pb1[n] = physical(lb1[n]), lb2[n] = logical(t, FAST ? RPB * n : crow + RPI * n);
    if (DYN && !FAST) lbs1 = lbs2, pbs1 = physical(lbs1), lbs2 = logical(t, j32);
  };

  // the wavefront's first tile is requested before anything else: its three dependent round trips (list entry, table
  // entry, bytes) pass while q is laid out
  int t = wv;
#pragma unroll
  for (int n = 0; n < NB; ++n) {
    lb1[n] = logical(t, FAST ? RPB * n : crow + RPI * n), lb2[n] = logical(t + kWavesDt, FAST ? RPB * n : crow + RPI * n);
    pb1[n] = physical(lb1[n]);
  }
  if (DYN && !FAST) lbs1 = logical(t, j32), lbs2 = logical(t + kWavesDt, j32), pbs1 = physical(lbs1);
  if (t < n_t) okq = request(t, kq, ssc, lb1, pb1);
  advance(t + 2 * kWavesDt);
  // The scoring pass has no V tile: the registers that would hold it take the wavefront's NEXT K tile, so that two
  // tiles' bytes are in flight per wavefront as in the decode pass (fewer bytes in flight do not fill the memory
  // pipeline).  Each of the two sets of registers has its own table entries (lb1 / pb1 and lbY / pbY), fetched a whole
  // tile period before the request that uses them: a wait for such an entry then never waits for the other set's bytes.
  int lbY[NB], pbY[NB];
  u32 okq2 = 0u;
  float ssc2 = 1.f;
  if constexpr (TWO_AHEAD) {
    okq2 = request(t + kWavesDt, vq, ssc2, lb1, pb1);
#pragma unroll
    for (int n = 0; n < NB; ++n) {
      lb1[n] = lb2[n], pb1[n] = physical_always(lb1[n]);
      lbY[n] = logical(t + 3 * kWavesDt, RPB * n), pbY[n] = physical_always(lbY[n]);
    }
  }

  // ---- Q as the B operand of S^T = K Q^T (v_mfma_f32_16x16x32_f16): lane = (column c16 = query head of the KV head,
  // quarter g4); k-step st holds, for quarter g4, channels 64 (st / 2) + 16 g4 + 8 (st % 2) .. + 7 - the order in
  // which a lane's 16-byte K pieces arrive.  The operands - the hi and lo fp16 terms of q x k_scale x c (the formats
  // with scale caches: q as it is, no lo term) - live in LDS, one 16-byte slot per (k-step, term, quarter, query
  // head), the same for the four wavefronts: each finds the row's scaling and stores every fourth k-step.  The
  // columns past the group read a slot of zeros.
  typedef __attribute__((address_space(3))) u4v lds_u4v;
  constexpr int QT = DYN ? 1 : 2;  // fp16 terms of q
  lds_u4v* const q_base = (lds_u4v*)((lds_u16*)lds + L::kQOff / 2);
  lds_u4v* const q_lane = q_base + (live ? g4 * QC + c16 : KT * QT * 4 * QC);
  const int q_step = live ? 4 * QC : 0;  // slots from one (k-step, term) to the next
  auto q_operand = [&](int st, int term) { return __builtin_bit_cast(v8h, q_lane[(QT * st + term) * q_step]); };
  float scl = sc;      // log2-logit per unit of the accumulator
  float sel_bound = 0.f;  // the scoring pass: how far a score of this pair may lie from the fp64 score (DYN: per unit of K scale)
  {
    const uint16_t* const qr = a.q + ((size_t)(qrow + (live ? tok : 0)) * a.hq + hq0 + (live ? head : 0)) * D;
    // the row times its K scales: once for its largest element, once more (every fourth k-step) for the operands
    auto scaled = [&](int st, float (&x)[8]) {
      const int c0 = 64 * (st >> 1) + 16 * g4 + 8 * (st & 1);
      const uint4 w = live ? *reinterpret_cast<const uint4*>(qr + c0) : make_uint4(0u, 0u, 0u, 0u);
      const float4 one = make_float4(1.f, 1.f, 1.f, 1.f);
      const float4 s0 = DYN ? one : *reinterpret_cast<const float4*>(a.k_scale + h * D + c0);
      const float4 s1 = DYN ? one : *reinterpret_cast<const float4*>(a.k_scale + h * D + c0 + 4);
      x[0] = bf16lo_to_f32(w.x) * s0.x, x[1] = bf16hi_to_f32(w.x) * s0.y;
      x[2] = bf16lo_to_f32(w.y) * s0.z, x[3] = bf16hi_to_f32(w.y) * s0.w;
      x[4] = bf16lo_to_f32(w.z) * s1.x, x[5] = bf16hi_to_f32(w.z) * s1.y;
      x[6] = bf16lo_to_f32(w.w) * s1.z, x[7] = bf16hi_to_f32(w.w) * s1.w;
    };
    float c = 1.0f, cinv = 1.0f;
    if (!DYN) {
      float amax = 0.f;
#pragma unroll
      for (int st = 0; st < KT; ++st) {
        float x[8];
        scaled(st, x);
#pragma unroll
        for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(x[e]));
      }
      // c = 2^(13 - floor(log2 amax)): the row's largest element lands in [2^13, 2^14)
      amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
      amax = fmaxf(amax, swap32(amax));
      int e = (int)((__float_as_uint(amax) >> 23) & 0xffu) - 127;
      e = amax > 0.f && amax < INFINITY ? min(max(13 - e, -100), 100) : 0;
      c = __uint_as_float((u32)(127 + e) << 23);
      cinv = __uint_as_float((u32)(127 - e) << 23);
    }
    scl = sc * cinv;
    if constexpr (SCORES) {
      // sum_c |q_c k_scale_c| of the lane's column: what every error term below is proportional to
      // (read through a pointer of its own that the compiler cannot see through: merged with the loads of the operand
      // loop below - which picks its k-step by the wavefront's number - this loop's values came out wrong in one
      // element of the upper k-steps, for the formats with scale caches)
      float asum = 0.f, amx = 0.f;
      const uint16_t* qr_own = qr;
      const float* ks_own = a.k_scale;
      asm volatile("" : "+v"(qr_own), "+v"(ks_own));
#pragma unroll
      for (int st = 0; st < KT; ++st) {
        const int c0 = 64 * (st >> 1) + 16 * g4 + 8 * (st & 1);
        const uint4 w = live ? *reinterpret_cast<const uint4*>(qr_own + c0) : make_uint4(0u, 0u, 0u, 0u);
        const u32 ws[4] = {w.x, w.y, w.z, w.w};
        float ksc[8] = {1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f};
        if (!DYN) {
          const float4 s0 = *reinterpret_cast<const float4*>(ks_own + h * D + c0), s1 = *reinterpret_cast<const float4*>(ks_own + h * D + c0 + 4);
          ksc[0] = s0.x, ksc[1] = s0.y, ksc[2] = s0.z, ksc[3] = s0.w, ksc[4] = s1.x, ksc[5] = s1.y, ksc[6] = s1.z, ksc[7] = s1.w;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float x0 = fabsf(bf16lo_to_f32(ws[e]) * ksc[2 * e]), x1 = fabsf(bf16hi_to_f32(ws[e]) * ksc[2 * e + 1]);
          asum += x0 + x1;
          amx = fmaxf(amx, fmaxf(x0, x1));
        }
      }
      asum += __shfl_xor(asum, 16, 64);
      asum += swap32(asum);
      amx = fmaxf(amx, __shfl_xor(amx, 16, 64));
      amx = fmaxf(amx, swap32(amx));
      constexpr float kCodeTop = QUANT == FDATTN_CACHE_INT8 ? 127.0f : 448.0f;
      constexpr float u22 = 2.384185791015625e-07f, u25 = 2.9802322387695312e-08f;  // 2^-22, 2^-25
      float bound;
      if (DYN) {
        // q as it is (bf16 in fp16: exact above fp16's subnormals, 2^-25 at most below; beyond fp16's range the
        // operand saturates: then nothing is known), D products accumulated in fp32 by the matrix unit (taken at four
        // times the textbook bound: its internal order and rounding are not documented), then one fp32 product with
        // the key's scale - everything per unit of that scale
        bound = kCodeTop * (asum * ((float)(D + 8) * u22 + 0.5f * u22) * 1.01f + (float)D * u25);
        if (!(amx <= 65000.0f)) bound = INFINITY;
      } else {
        // q * k_scale * c as hi + lo: off by 2^-22 of itself, or 2^-25 where lo is subnormal; 2 D products accumulated
        // in fp32 (four times the textbook bound again); the scaling by 1 / c is exact
        bound = kCodeTop * (asum * (float)(2 * D + 9) * u22 * 1.01f + (float)D * u25 * cinv);
      }
      bound = live ? bound : 0.f;
#pragma unroll
      for (int o = 1; o < 16; o <<= 1) bound = fmaxf(bound, __shfl_xor(bound, o, 64));
      sel_bound = bound;  // (the same in every lane of every wavefront; a NaN q leaves a NaN: every block then undecided)
      for (int j = tid; j < a.sel_blocks_per_split; j += 64 * kWavesDt) sel_bmax[j] = (int)0x80000000, sel_smax[j] = 0u;
    }
    for (int st = wv; st < KT; st += kWavesDt) {
      float x[8];
      scaled(st, x);
      u32 hw[4], lw[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float x0 = sat_f16(x[2 * e] * c), x1 = sat_f16(x[2 * e + 1] * c);
        const v2h hv = {(_Float16)x0, (_Float16)x1};
        hw[e] = __builtin_bit_cast(u32, hv);
        lw[e] = pack_f16(x0 - (float)hv[0], x1 - (float)hv[1]);
      }
      const u4v hv4 = {hw[0], hw[1], hw[2], hw[3]}, lv4 = {lw[0], lw[1], lw[2], lw[3]};
      if (live) {
        q_lane[(QT * st) * q_step] = hv4;
        if (!DYN) q_lane[(QT * st + 1) * q_step] = lv4;
      }
    }
    if (tid == 0) {
      const u4v z = {0u, 0u, 0u, 0u};
      q_base[KT * QT * 4 * QC] = z;
    }
  }
  __syncthreads();

  // O^T, 16 channels x 16 columns per MFMA: o[db][e] = channel 16 db + 4 g4 + e of this lane's column
  v4f o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) o[db] = v4f{0.f, 0.f, 0.f, 0.f};
  float m_ref = -INFINITY;  // exponent reference of the weights (log2 domain), the same in the four lanes of a column
  float l_run = 0.f;        // this lane's share (its 8 of every 32 keys) of the weight sum

  // operands out of the wavefront's tiles.  The tile's keys 0 .. 15 and 16 .. 31 make two score tiles; lane (c16, g4)
  // owns, as a row of K: key c16 of each; as scores and weights of column c16: keys 4 g4 + e and 16 + 4 g4 + e,
  // e = 0 .. 3 - eight k-slots of O^T += V^T P^T in that order.
  // K: 16 bytes of the lane's keys per pair of k-steps.  V^T: 16 lanes read 8 rows x 16 bytes transposed
  // (ds_read_b64_tr_b8): lane c16 of them ends up with column c16 of the 8 rows, which are the quarter's eight keys.
  const lds_u8* const k_lane = kt + c16 * L::RS + 16 * g4;
  const lds_u8* const v_lane = vt + (16 * (c16 >> 3) + 4 * g4 + ((c16 >> 1) & 3)) * L::RS + 8 * (c16 & 1);
  auto k_pieces = [&](int jp, uint4 (&w)[2]) {  // channels 64 jp + 16 g4 .. + 15 of key c16 and of key 16 + c16
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const u4v r = *reinterpret_cast<const __attribute__((address_space(3))) u4v*>(k_lane + 16 * half * L::RS + 64 * jp);
      w[half] = make_uint4(r.x, r.y, r.z, r.w);
    }
  };
  auto v_operand = [&](int db) {
    const v2i r = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i*)(v_lane + 16 * db));
    return __builtin_bit_cast(v8h, cvt8_for_mfma<QUANT>((u32)r.x, (u32)r.y));
  };

  // one tile: its bytes into LDS (and, `more`, tile tn's requested), S = K Q, softmax, O += V P
  auto compute = [&](int t, int tn, bool more, uint4 (&kq)[NC], u32& okq, float& ssc, const int (&lbr)[NB], const int (&pbr)[NB]) {
    const u32 want = (NC >= 32 ? 0xffffffffu : (1u << NC) - 1u) | (DYN ? 1u << 31 : 0u);
    const bool all_ok = __all((okq & ~kLate) == want) != 0;  // (uniform) most tiles: every key is one
    const bool by_column = MT && toks > 1 && __any((okq & kLate) != 0u);  // (uniform) keys that some of the row's tokens do not see
    if (!all_ok) {  // keys that are none count as rows of zeros: stale bytes may be fp8 NaN codes
#pragma unroll
      for (int n = 0; n < NC; ++n)
        if (!(okq >> n & 1u)) {
          kq[n] = make_uint4(0u, 0u, 0u, 0u);
          if constexpr (!SCORES) vq[n] = make_uint4(0u, 0u, 0u, 0u);
        }
    }
#pragma unroll
    for (int n = 0; n < NC; ++n) {
      const u4v kw = {kq[n].x, kq[n].y, kq[n].z, kq[n].w};
      *reinterpret_cast<__attribute__((address_space(3))) u4v*>(kt + (crow + RPI * n) * L::RS + 16 * cch) = kw;
      if constexpr (!SCORES) {
        const u4v vw = {vq[n].x, vq[n].y, vq[n].z, vq[n].w};
        *reinterpret_cast<__attribute__((address_space(3))) u4v*>(vt + (crow + RPI * n) * L::RS + 16 * cch) = vw;
      }
    }
    if (DYN) {  // what the softmax needs of a key's scales, worked out once per tile
      const bool oks = okq >> 31 != 0;
      if (hf == 0) {
        wsc[j32] = oks ? sc * ssc : 0.f;
        // the scoring pass: the block's largest K scale, for its error bound (a tile inside one or two blocks: the 16
        // lanes of a row agree on the block, so the row's maximum goes there once - 32 lanes on one LDS word take turns)
        if constexpr (SCORES) {
          u32 big = oks ? __float_as_uint(fabsf(ssc)) : 0u;
          if constexpr (TB >= 1) {
            big = max(big, dpp_or_zero<0x128, 0xf>(big));
            big = max(big, dpp_or_zero<0x124, 0xf>(big));
            big = max(big, dpp_or_zero<0x122, 0xf>(big));
            big = max(big, dpp_or_zero<0x121, 0xf>(big));
            if ((j32 & 15) == 0 && big != 0u) atomicMax(sel_smax + block_of(32 * t + j32), big);
          } else {
            if (oks) atomicMax(sel_smax + block_of(32 * t + j32), big);
          }
        }
      } else if constexpr (SCORES) {
        wsc[32 + j32] = oks ? 0.f : -INFINITY;  // (the mask only)
      } else {
        wsc[32 + j32] = oks ? __builtin_amdgcn_logf(ssc) : -INFINITY;  // log2
        wsc[64 + j32] = oks ? __builtin_amdgcn_rcpf(ssc) : 0.f;
      }
    } else if (!all_ok && cch == 0) {
#pragma unroll
      for (int n = 0; n < NC; ++n) wsc[32 + crow + RPI * n] = okq >> n & 1u ? 0.f : -INFINITY;
    }
    if (by_column && cch == 0) {  // the keys' positions, for the columns to compare with their own
      int* const wpos = reinterpret_cast<int*>(wsc + 96);
#pragma unroll
      for (int n = 0; n < NC; ++n) {
        const int e = FAST ? (RPI * n) / RPB : 0, in_block = crow + RPI * n - RPB * e;
        const int first = posq[MT && FAST ? e : 0];
        wpos[crow + RPI * n] = FAST ? (first == 0x7fffffff ? first : first + in_block) : posq[FAST || !MT ? 0 : n];
      }
    }
    if constexpr (TWO_AHEAD) {
      // The loop issues and takes the same loads in every iteration, whatever is left of the split: where two paths
      // with different loads in flight meet, the compiler's count of them keeps the smaller one, and every wait behind
      // the meeting point waits for too much - the other tile's bytes included.
      int lbu[NB], pbu[NB];
#pragma unroll
      for (int n = 0; n < NB; ++n) lbu[n] = __builtin_amdgcn_readfirstlane(lbr[n]), pbu[n] = __builtin_amdgcn_readfirstlane(pbr[n]);
      okq = request(tn, kq, ssc, lbu, pbu);  // (past the split's last tile: rows of block 0 that count as no keys)
    } else {
      if (more) okq = request(tn, kq, ssc, lbr, pbr);
    }
    // (the wavefront's LDS instructions execute in order: what its lanes stored above is there for the reads below)
    __builtin_amdgcn_wave_barrier();
    // S^T = K Q^T for the two score tiles: two accumulators, so that an MFMA does not wait for the one before it, and
    // the next pair of k-steps' operands requested from LDS before this pair's conversions and MFMAs
    v4f sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
    {
      uint4 kw[2][2];
      v8h qo[2][2 * QT];
      auto operands = [&](int jp, int slot) {
        k_pieces(jp, kw[slot]);
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int term = 0; term < QT; ++term) qo[slot][QT * u + term] = q_operand(2 * jp + u, term);
      };
      operands(0, 0);
#pragma unroll
      for (int jp = 0; jp < KT / 2; ++jp) {
        const int cur = jp & 1;
        if (jp + 1 < KT / 2) operands(jp + 1, cur ^ 1);
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const uint4 wa = kw[cur][0], wb = kw[cur][1];
          const v8h ka = __builtin_bit_cast(v8h, u ? cvt8_for_mfma<QUANT>(wa.z, wa.w) : cvt8_for_mfma<QUANT>(wa.x, wa.y));
          const v8h kb = __builtin_bit_cast(v8h, u ? cvt8_for_mfma<QUANT>(wb.z, wb.w) : cvt8_for_mfma<QUANT>(wb.x, wb.y));
#pragma unroll
          for (int term = 0; term < QT; ++term) {
            sa = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qo[cur][QT * u + term], sa, 0, 0, 0);
            sb = __builtin_amdgcn_mfma_f32_16x16x32_f16(kb, qo[cur][QT * u + term], sb, 0, 0, 0);
          }
        }
        __builtin_amdgcn_sched_barrier(0);  // one pair ahead, no more: operand reads hoisted over the whole row would cost its registers
      }
    }
    // log2-logits x[i] of the lane's keys: 4 g4 + i (i < 4), 16 + 4 g4 + i - 4
    float x[8], iv[8];
    if (DYN) {  // K scale on the score, V scale on the weight's exponent
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const float4 t4 = *reinterpret_cast<const float4*>(wsc + 16 * half + 4 * g4);
        const float4 l4 = *reinterpret_cast<const float4*>(wsc + 32 + 16 * half + 4 * g4);
        const float4 i4 = *reinterpret_cast<const float4*>(wsc + 64 + 16 * half + 4 * g4);
        const v4f sv = half ? sb : sa;
        x[4 * half] = __builtin_fmaf(sv[0], t4.x, l4.x), x[4 * half + 1] = __builtin_fmaf(sv[1], t4.y, l4.y);
        x[4 * half + 2] = __builtin_fmaf(sv[2], t4.z, l4.z), x[4 * half + 3] = __builtin_fmaf(sv[3], t4.w, l4.w);
        iv[4 * half] = i4.x, iv[4 * half + 1] = i4.y, iv[4 * half + 2] = i4.z, iv[4 * half + 3] = i4.w;
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] = sa[e] * scl, x[4 + e] = sb[e] * scl;
      if (!all_ok) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const float4 m4 = *reinterpret_cast<const float4*>(wsc + 32 + 16 * half + 4 * g4);
          x[4 * half] += m4.x, x[4 * half + 1] += m4.y, x[4 * half + 2] += m4.z, x[4 * half + 3] += m4.w;
        }
      }
    }
    if (by_column) {
      const int* const wpos = reinterpret_cast<const int*>(wsc + 96);
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int4 p4 = *reinterpret_cast<const int4*>(wpos + 16 * half + 4 * g4);
        x[4 * half] = p4.x < lim ? x[4 * half] : -INFINITY, x[4 * half + 1] = p4.y < lim ? x[4 * half + 1] : -INFINITY;
        x[4 * half + 2] = p4.z < lim ? x[4 * half + 2] : -INFINITY, x[4 * half + 3] = p4.w < lim ? x[4 * half + 3] : -INFINITY;
      }
    }
    if constexpr (SCORES) {
      // the largest score of every block the tile touches, over its keys and the live columns, into the split's LDS array
      if (!live) {
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = -INFINITY;
      }
      auto over_columns = [&](float v) {  // the 16 lanes of a quarter hold the 16 columns
        v = fmaxf(v, dpp_or_zero<0x128, 0xf>(v));
        v = fmaxf(v, dpp_or_zero<0x124, 0xf>(v));
        v = fmaxf(v, dpp_or_zero<0x122, 0xf>(v));
        return fmaxf(v, dpp_or_zero<0x121, 0xf>(v));
      };
      if constexpr (TB >= 1) {  // each half of the tile (16 keys) lies inside one block
        float ma = fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])), mb = fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7]));
        if (TB == 1) ma = fmaxf(ma, mb);
        ma = over_columns(ma);
        ma = fmaxf(ma, __shfl_xor(ma, 16, 64));
        ma = fmaxf(ma, swap32(ma));
        if (TB == 2) {
          mb = over_columns(mb);
          mb = fmaxf(mb, __shfl_xor(mb, 16, 64));
          mb = fmaxf(mb, swap32(mb));
        }
        if (lane == 0 && 32 * t < n_x) {  // (the walk may compute one tile past the split's end)
          atomicMax(sel_bmax + block_of(32 * t), score_key(ma));
          if (TB == 2 && 32 * t + 16 < n_x) atomicMax(sel_bmax + block_of(32 * t + 16), score_key(mb));  // (an odd number of blocks: the last tile holds one)
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float v = over_columns(x[i]);
          const int key = i < 4 ? 4 * g4 + i : 16 + 4 * g4 + (i - 4);
          if (c16 == 0 && 32 * t + key < n_x) atomicMax(sel_bmax + block_of(32 * t + key), score_key(v));
        }
      }
      __builtin_amdgcn_wave_barrier();
      return;
    }
    // the reference is raised when a score outgrows it by 2^13, which keeps every weight inside fp16
    float mt = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; ++i) mt = fmaxf(mt, x[i]);
    mt = fmaxf(mt, __shfl_xor(mt, 16, 64));
    mt = fmaxf(mt, swap32(mt));
    const bool had_ref = m_ref > -INFINITY;  // a column without one has accumulated nothing yet
    const bool raise = mt > m_ref + 13.0f || (!had_ref && mt > -INFINITY);
    const float alpha = raise ? (had_ref ? __builtin_amdgcn_exp2f(m_ref - mt) : 0.f) : 1.0f;
    l_run *= alpha;
    if (__any(raise && had_ref)) {
#pragma unroll
      for (int db = 0; db < DB; ++db) o[db] *= alpha;
    }
    m_ref = raise ? mt : m_ref;
    const float cst = m_ref == -INFINITY ? 0.f : -m_ref;
    u32 pw[4];
    float lsum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      const float e0 = __builtin_amdgcn_exp2f(x[i] + cst), e1 = __builtin_amdgcn_exp2f(x[i + 1] + cst);
      pw[i >> 1] = pack_f16(e0, e1);
      if (DYN) {  // the weight sum takes the weights without their V scale
        lsum = __builtin_fmaf(e0, iv[i], lsum);
        lsum = __builtin_fmaf(e1, iv[i + 1], lsum);
      } else {
        lsum += e0 + e1;
      }
    }
    l_run += lsum;
    const v8h pp = __builtin_bit_cast(v8h, make_uint4(pw[0], pw[1], pw[2], pw[3]));
#pragma unroll
    for (int db = 0; db < DB; ++db) o[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(v_operand(db), pp, o[db], 0, 0, 0);
    __builtin_amdgcn_wave_barrier();
  };

  // ---- the walk: tile t computed; the bytes of the wavefront's next tile in flight (requested as soon as the
  // registers that receive them have been stored), the table entries of the tile after it and the list entries of the
  // one after that as well
  if constexpr (TWO_AHEAD) {
    for (; t < n_t; t += 2 * kWavesDt) {
      compute(t, t + 2 * kWavesDt, true, kq, okq, ssc, lb1, pb1);
#pragma unroll
      for (int n = 0; n < NB; ++n) lb1[n] = logical(t + 4 * kWavesDt, RPB * n), pb1[n] = physical_always(lb1[n]);
      compute(t + kWavesDt, t + 3 * kWavesDt, true, vq, okq2, ssc2, lbY, pbY);  // (a tile past the end: no keys, no scores)
#pragma unroll
      for (int n = 0; n < NB; ++n) lbY[n] = logical(t + 5 * kWavesDt, RPB * n), pbY[n] = physical_always(lbY[n]);
    }
  } else {
    for (; t < n_t; t += kWavesDt) {
      compute(t, t + kWavesDt, t + kWavesDt < n_t, kq, okq, ssc, lb1, pb1);
      advance(t + 3 * kWavesDt);
    }
  }

  if constexpr (SCORES) {
    __syncthreads();
    const size_t row = (size_t)pair * a.max_blocks;
    for (int j = tid; j < i1 - i0; j += 64 * kWavesDt) {
      const float v = key_score(sel_bmax[j]);
      a.sel_approx[row + i0 + j] = v;
      if (a.sel_scores_out) a.sel_scores_out[row + i0 + j] = v;
      if (DYN) a.sel_ebound[row + i0 + j] = sel_bound * __uint_as_float(sel_smax[j]);
    }
    if (split == 0) {  // the blocks past the sequence's end score nothing
      for (int j = nblk + tid; j < a.max_blocks; j += 64 * kWavesDt) {
        a.sel_approx[row + j] = -INFINITY;
        if (a.sel_scores_out) a.sel_scores_out[row + j] = -INFINITY;
        if (DYN) a.sel_ebound[row + j] = 0.f;
      }
      if (tid == 0) a.sel_eps[pair] = DYN ? 0.f : sel_bound;
    }
    return;
  }
  // ---- the four wavefronts meet: a common reference per column, o and l summed in LDS (over the tiles)
  float l_tot = l_run + __shfl_xor(l_run, 16, 64);
  l_tot += swap32(l_tot);
  float* const ms = reinterpret_cast<float*>(lds + L::kMergeOff / 2);
  float* const ls = ms + kWavesDt * 16;
  float* const red = reinterpret_cast<float*>(lds);
  if (g4 == 0) ms[wv * 16 + c16] = m_ref;
  __syncthreads();  // (also: every wavefront has left its tiles)
  float M = ms[c16];
#pragma unroll
  for (int w = 1; w < kWavesDt; ++w) M = fmaxf(M, ms[w * 16 + c16]);
  const float alpha = m_ref > -INFINITY ? __builtin_amdgcn_exp2f(m_ref - M) : 0.f;
  if (g4 == 0) ls[wv * 16 + c16] = l_tot * alpha;
  for (int w = 0; w < kWavesDt; ++w) {
    if (wv == w && live) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float* const dst = red + c16 * L::LDR + 16 * db + 4 * g4 + e;
          *dst = (w ? *dst : 0.f) + o[db][e] * alpha;
        }
    }
    __syncthreads();
  }
  // column -> (token, query head) of the row; a partial's row is (sequence, token slot, query head)
  const int cols = toks * G;
  if (a.max_splits == 1) {  // the only split: the partial is the result
    for (int idx = tid; idx < cols * D; idx += 64 * kWavesDt) {
      const int col = idx / D, c = idx - col * D, tk = col / G, hd = col - tk * G;
      float lc = ls[col];
#pragma unroll
      for (int w = 1; w < kWavesDt; ++w) lc += ls[w * 16 + col];
      const float oc = DYN ? red[col * L::LDR + c] : red[col * L::LDR + c] * a.v_scale[h * D + c];
      a.out[((size_t)(qrow + tk) * a.hq + hq0 + hd) * D + c] = f32_to_bf16(lc > 0.f ? oc / lc : 0.f);
    }
    return;
  }
  for (int idx = tid; idx < cols * D; idx += 64 * kWavesDt) {
    const int col = idx / D, c = idx - col * D, tk = col / G, hd = col - tk * G;
    const size_t slot = (((size_t)b * max_tokens + tk) * a.hq + hq0 + hd) * a.max_splits + split;
    a.part_o[slot * D + c] = DYN ? red[col * L::LDR + c] : red[col * L::LDR + c] * a.v_scale[h * D + c];
  }
  if (tid < cols) {
    float Mc = ms[tid], lc = ls[tid];
#pragma unroll
    for (int w = 1; w < kWavesDt; ++w) Mc = fmaxf(Mc, ms[w * 16 + tid]), lc += ls[w * 16 + tid];
    const int tk = tid / G, hd = tid - tk * G;
    const size_t slot = (((size_t)b * max_tokens + tk) * a.hq + hq0 + hd) * a.max_splits + split;
    a.part_m[slot] = Mc * 0.6931471805599453f;  // the combine works in natural-log units
    a.part_l[slot] = lc;
  }
}

template <int QUANT, bool DYN, int D, int TB, bool MT>
hipError_t launch_dt_f(const GenericDecodeArgs& a, hipStream_t s) {
  using L = DecLay<D>;
  // the dynamic LDS limit is a per-device property of the kernel: raise it once on each device
  static std::atomic<unsigned long long> raised{0};  // bit d: done on device d (one word per instantiation)
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev >= 64 || !(raised.load(std::memory_order_relaxed) >> dev & 1ull)) {
    e = hipFuncSetAttribute((const void*)decode_tiles_kernel<QUANT, DYN, D, TB, MT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)L::bytes(16));
    if (e != hipSuccess) return e;
    if (dev < 64) raised.fetch_or(1ull << dev, std::memory_order_relaxed);
  }
  const int sets = (a.hq / a.hkv + 15) / 16;
  const dim3 grid((unsigned)a.batch * a.hkv * sets, a.max_splits), block(64 * kWavesDt);
  const int columns = a.max_tokens * (a.hq / a.hkv) < 16 ? a.max_tokens * (a.hq / a.hkv) : 16;
  hipLaunchKernelGGL((decode_tiles_kernel<QUANT, DYN, D, TB, MT>), grid, block, L::bytes(columns), s, a);
  return hipSuccess;
}

template <int QUANT, bool DYN, int D, int TB>
hipError_t launch_scores_f(const GenericDecodeArgs& a, hipStream_t s) {
  using L = DecLay<D>;
  const size_t shm = L::bytes(16) + (size_t)a.sel_blocks_per_split * 2 * sizeof(int);
  static std::atomic<unsigned long long> raised{0};  // (as in launch_dt_f)
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev >= 64 || !(raised.load(std::memory_order_relaxed) >> dev & 1ull)) {
    e = hipFuncSetAttribute((const void*)decode_tiles_kernel<QUANT, DYN, D, TB, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)(L::bytes(16) + (size_t)kSelTilesMaxBlocksPerSplit * 2 * sizeof(int)));
    if (e != hipSuccess) return e;
    if (dev < 64) raised.fetch_or(1ull << dev, std::memory_order_relaxed);
  }
  const dim3 grid((unsigned)a.batch * a.hkv, a.max_splits), block(64 * kWavesDt);
  hipLaunchKernelGGL((decode_tiles_kernel<QUANT, DYN, D, TB, false, true>), grid, block, shm, s, a);
  return hipSuccess;
}

template <int QUANT, bool DYN, int D>
hipError_t launch_scores(const GenericDecodeArgs& a, hipStream_t s) {
  const int tb = a.bs >= 32 && (a.bs & (a.bs - 1)) == 0 ? 1 : (a.bs == 16 ? 2 : 0);
  return tb == 1 ? launch_scores_f<QUANT, DYN, D, 1>(a, s) : (tb == 2 ? launch_scores_f<QUANT, DYN, D, 2>(a, s) : launch_scores_f<QUANT, DYN, D, 0>(a, s));
}

template <int D>
hipError_t launch_scores_d(const GenericDecodeArgs& a, int quant, hipStream_t s) {
  if (quant == FDATTN_CACHE_INT8) return launch_scores<FDATTN_CACHE_INT8, false, D>(a, s);
  if (quant == FDATTN_CACHE_FP8_E4M3) return launch_scores<FDATTN_CACHE_FP8_E4M3, false, D>(a, s);
  if (quant_bytes(quant) == FDATTN_CACHE_INT8) return launch_scores<FDATTN_CACHE_INT8, true, D>(a, s);
  return launch_scores<FDATTN_CACHE_FP8_E4M3, true, D>(a, s);
}

template <int QUANT, bool DYN, int D>
hipError_t launch_dt(const GenericDecodeArgs& a, hipStream_t s) {
  const int tb = a.bs >= 32 && (a.bs & (a.bs - 1)) == 0 ? 1 : (a.bs == 16 ? 2 : 0);
  if (a.max_tokens > 1)
    return tb == 1 ? launch_dt_f<QUANT, DYN, D, 1, true>(a, s) : (tb == 2 ? launch_dt_f<QUANT, DYN, D, 2, true>(a, s) : launch_dt_f<QUANT, DYN, D, 0, true>(a, s));
  return tb == 1 ? launch_dt_f<QUANT, DYN, D, 1, false>(a, s) : (tb == 2 ? launch_dt_f<QUANT, DYN, D, 2, false>(a, s) : launch_dt_f<QUANT, DYN, D, 0, false>(a, s));
}

template <int D>
hipError_t launch_dt_d(const GenericDecodeArgs& a, int quant, hipStream_t s) {
  if (quant == FDATTN_CACHE_INT8) return launch_dt<FDATTN_CACHE_INT8, false, D>(a, s);
  if (quant == FDATTN_CACHE_FP8_E4M3) return launch_dt<FDATTN_CACHE_FP8_E4M3, false, D>(a, s);
  if (quant_bytes(quant) == FDATTN_CACHE_INT8) return launch_dt<FDATTN_CACHE_INT8, true, D>(a, s);
  return launch_dt<FDATTN_CACHE_FP8_E4M3, true, D>(a, s);
}

}  // namespace

bool decode_tiles_supported(int hq, int hkv, int d) {
  return hkv > 0 && hq % hkv == 0 && hq / hkv <= 64 && (d == 64 || d == 128 || d == 256);
}

int decode_tiles_splits(int pairs, int d, int max_keys, int most) {
  // Measured on 8 .. 512 pairs with 1 k .. 32 k keys each: the launch is fastest with about 2 - 3 workgroups per CU
  // (more at the smaller head sizes, whose workgroups are shorter), as long as a split keeps a few tiles per
  // wavefront; one split - no partials, no merge launch - wins as soon as the pairs alone come near that; and a
  // launch of very few pairs (a batch of one or two sequences) splits down to 256 keys - two tiles per
  // wavefront - to put a workgroup on every CU.
  const int cus = gpu_cu_count();
  if (pairs < 1) pairs = 1;
  const int target = d <= 64 ? 3 * cus : (d <= 128 ? 5 * cus / 2 : 2 * cus);
  const int min_keys = d <= 64 ? 1024 : 2048;
  int n = target / pairs;
  if (n > max_keys / min_keys) n = max_keys / min_keys;
  int fill = (cus + pairs - 1) / pairs;
  if (fill > max_keys / 256) fill = max_keys / 256;
  if (n < fill) n = fill;
  return n < 1 ? 1 : (n > most ? most : n);
}

hipError_t sqattn_scores_tiles_launch(const GenericDecodeArgs& a, int quant, hipStream_t s) {
  if (a.d == 64) return launch_scores_d<64>(a, quant, s);
  if (a.d == 128) return launch_scores_d<128>(a, quant, s);
  return launch_scores_d<256>(a, quant, s);
}

hipError_t decode_tiles_launch(const GenericDecodeArgs& a, int quant, hipStream_t s) {
  if (a.d == 64) return launch_dt_d<64>(a, quant, s);
  if (a.d == 128) return launch_dt_d<128>(a, quant, s);
  return launch_dt_d<256>(a, quant, s);
}

}  // namespace fdattn
