// Decode attention over the int8 / fp8-e4m3 paged cache for head_dim 128, 1 .. 8 query
// heads per KV head, block_size 64 - the HBM-bound kernel of the path.
//
// Work unit: one (sequence, KV head, cache block) = an 8 KiB K tile + an 8 KiB V tile,
// each contiguous in HBM.  The block list of every (sequence, KV head) pair is cut into
// chunks of `chunk` units; one workgroup of 4 wavefronts takes one chunk (grid = chunks
// per pair x pairs, workgroups past the end of a list do nothing).  The chunk length is
// picked so that the launch fills the GPU's workgroup slots once (c8_pick_chunk): as
// few, as long workgroups as that allows, up to 256 units each (128 where rows of several
// tokens need three or four row sets).  Pair and chunk follow
// from the block index, the physical blocks from one coalesced read of the block table.
//
// Inside a workgroup every wavefront is autonomous: it takes units wave, wave+4, ... of
// the chunk, owns a K slot, a V slot and a P slot in LDS, fills them with direct
// global->LDS loads (16 B per lane, whole 128-byte rows) and meets no barrier until the
// chunk is done.  While it works on unit j, K(j+1) and V(j+1) are in flight.
//
// Arithmetic runs on the MFMA units without dequantising a single cache byte:
//   int8 cache: v_mfma_i32_16x16x64_i8.  The 4 query heads occupy the 16 MFMA rows as
//     4 heads x up to 4 byte "limbs": q*k_scale is split into 3 balanced base-128 digits
//     (21 bits), the softmax weights into 4 base-128 digits (28 bits).  Integer dot
//     products are exact; the limbs are recombined in fp32.
//   fp8 cache: v_mfma_f32_16x16x32_fp8_fp8 with q*k_scale and the weights split into 4
//     e4m3 residual limbs (16 significant bits).
//   Groups of up to 4 query heads use one such set of 16 rows (rows of absent heads are
//   zero); 5 .. 8 heads use two sets, and every K and V operand read from LDS feeds both.
// The per-channel K scale is folded into q, the V scale is applied once to the output.
// V tiles are transposed for free by ds_read_b64_tr_b8.
// The formats with one scale per stored row (DYN) bring a unit's 64 K scales and 64 V
// scales into LDS with two more direct loads; the K scale multiplies the token's score,
// the V scale - relative to the unit's largest - rides on the token's softmax weight
// before the weight is cut into limbs, and the unit's largest scales its P.V product.
// The formats with one scale per (block, KV head) tile run on the same instantiations:
// the two loads read the tile's one scale into all 64 LDS slots (C8Args::scale_rows = 1).
//
// At the end the 4 wavefronts merge their (m, l, o) through LDS.  A pair with a single
// chunk is finished on the spot (bf16 output written); otherwise the workgroup leaves one
// partial at workspace slot pair*chunks_per_pair + chunk and the merge kernel combines
// them.  Two variants were measured slower and dropped: merging inside the main kernel
// (the last workgroup to arrive at a pair combines it: the device-scope stores, the atomic
// and the barrier sit at the end of every workgroup, where nothing hides their latency),
// and handing chunks out through an atomic ticket counter instead of the block index.
#include <atomic>
#include <mutex>

#include "c8_common.h"


namespace fdattn {

struct C8Args {
  const uint16_t* q;
  const uint8_t* key_cache;
  const uint8_t* value_cache;
  const float* k_scale;  // [hkv, 128] per channel; DYN: [num_blocks, hkv, 64] per stored row, or [num_blocks, hkv] per tile
  const float* v_scale;
  const int32_t* block_tables;
  const int32_t* seq_lens_decoder;
  const int32_t* seq_lens_this_time;
  const int32_t* kept_blocks;
  const int32_t* kept_counts;
  int max_kept;
  float* part_o;   // [pairs * chunks_per_pair][sets * 4][128], sets = ceil(group / 4)
  float* part_ml;  // [pairs * chunks_per_pair][sets][8]: m[4] (log2 domain), l[4]
  uint16_t* out;
  RowMap rows;  // which sequences are decode rows and where their q / out rows are
  int batch, hkv, max_blocks, num_blocks;
  int chunk;            // units per workgroup
  int chunks_per_pair;  // grid.x
  float sm_scale_log2;  // softmax_scale * log2(e)
  int dyn;              // scales per stored row: the output takes no per-channel V scale
  int group;            // query heads per KV head, 1 .. 8
  int max_tokens;       // tokens a decode row may bring (1; speculative steps: up to 16 / group)
  int scale_rows;       // DYN: scales per (block, head) tile in the scale caches: 64, or 1 (every row of the tile shares it)
};

// Length of the pair's block list: every block of the sequence, or the kept ones.
template <bool SPARSE>
__device__ __forceinline__ int pair_units(const C8Args& a, int p, int kv_len) {
  if (SPARSE) return min(max(a.kept_counts[p], 0), a.max_kept);
  return min((max(kv_len, 0) + kBS - 1) / kBS, a.max_blocks);
}

// NSET: row sets of 4 query heads a wavefront carries (1: up to 4 query heads per KV head, 2: up to 8; 3 and 4:
// rows of several tokens only); every K
// and V operand read from LDS feeds the MFMAs of all sets.
// SPEC: a decode row may bring several tokens (a speculative step's drafts, all in the cache already): the MFMA
// rows are then (token, head) pairs - row v is token v / group, head v % group - and token t of T attends to the
// sequence's cached tokens and the new ones up to itself, i.e. to T - 1 - t fewer than the last one.
// (Three and four row sets - rows of several tokens only - need more than the 256 registers a wavefront has when two
// workgroups share a CU: those instantiations run one workgroup per CU.)
template <int QUANT, bool SPARSE, bool DYN, int NSET, bool SPEC = false>
__global__ __launch_bounds__(kWaves * 64, NSET > 2 ? 1 : 2) void decode_c8_kernel(C8Args a) {
  __shared__ __attribute__((aligned(16))) uint8_t ldsK[kWaves][kTileB];
  __shared__ __attribute__((aligned(16))) uint8_t ldsV[kWaves][kTileB];
  __shared__ __attribute__((aligned(16))) uint8_t ldsP[kWaves][NSET][1024];
  __shared__ __attribute__((aligned(16))) float ldsS[DYN ? kWaves : 1][2 * kBS];  // DYN: a unit's K scales, V scales
  const int lane = threadIdx.x & 63;
  const int wv = uni(threadIdx.x >> 6);
  const int ticket = blockIdx.x;
  // Chunk-major: workgroups are dealt to the 8 XCDs in turn, so with the pair running fastest every
  // XCD sees every chunk position (pair-major, a chunk count that shares a factor with 8 sends the
  // often-empty late chunks of short sequences to the same XCDs); and the launch ends with the
  // late chunks, the ones most often short or empty.
  const int pairs = a.batch * a.hkv;
  const int ck = ticket / pairs, p = ticket - ck * pairs;
  const int b = p / a.hkv, h = p - b * a.hkv;
  const int first = ck * a.chunk;
  // ---- unit table, requested before anything else: lane j asks for the physical block of unit
  // first + j.  The request depends on the block index alone, so it travels together with the
  // loads of the sequence's length below instead of behind them - under load every dependent
  // round trip to memory at the start of a workgroup costs microseconds in which its LDS slots
  // carry nothing.
  // (kEnt entries per lane: four hold chunks of up to 256 units; the kernels with three or four row sets, which have no
  // registers to spare, keep two)
  constexpr int kEnt = NSET <= 2 ? 4 : 2;
  int lb[kEnt], pb_raw[kEnt];
#pragma unroll
  for (int e = 0; e < kEnt; ++e) {
    lb[e] = -1, pb_raw[e] = -1;
    const int u = lane + 64 * e;
    if (u < a.chunk) {
      int l = first + u;
      if (SPARSE) l = l < a.max_kept ? a.kept_blocks[(size_t)p * a.max_kept + l] : -1;
      if (l >= 0 && l < a.max_blocks) pb_raw[e] = a.block_tables[(size_t)b * a.max_blocks + l];
      lb[e] = l;
    }
  }
  int row, toks = 1;
  if (SPEC ? !decode_rows(a.rows, b, a.max_tokens, row, toks) : !decode_row(a.rows, b, row)) return;
  PairRaw raw[NSET];  // in flight with the table entries
#pragma unroll
  for (int t = 0; t < NSET; ++t)
    raw[t] = load_pair_issue(a.q, DYN ? nullptr : a.k_scale, a.hkv, p, row, lane, a.group, t, SPEC ? toks : 0);
  const int kv_len = a.seq_lens_decoder[b] + (a.seq_lens_this_time ? a.seq_lens_this_time[b] : 0);
  const int n_p = pair_units<SPARSE>(a, p, kv_len);
  const int cnt = min(a.chunk, n_p - first);  // <= 0: past the end of this pair's list
  const bool single = n_p <= a.chunk;
  const int vg = a.group * toks;  // MFMA rows in use: (token, head) pairs
  // q / out row of MFMA row `head` of this pair (SPEC: token head / group, head head % group)
  auto out_row = [&](int head) {
    const int tok = SPEC ? head / a.group : 0;
    return a.out + ((size_t)(row + tok) * a.hkv * a.group + h * a.group + (head - tok * a.group)) * kD;
  };
  if (cnt <= 0) {
    if (n_p == 0 && ck == 0) {  // empty sequence: its output rows are zeros
      for (int head = threadIdx.x >> 6; head < vg; head += kWaves)
        *reinterpret_cast<u32*>(out_row(head) + (threadIdx.x & 63) * 2) = 0u;
    }
    return;
  }

  uint8_t* const kbuf = ldsK[wv];
  uint8_t* const vbuf = ldsV[wv];
  const u32 kaddr = uni((int)lds_addr_of(kbuf)), vaddr = uni((int)lds_addr_of(vbuf));
  const DmaOffsets offK = dma_offsets<kShiftK>(lane), offV = dma_offsets<kShiftV>(lane);
  const int n16 = lane & 15, g4 = lane >> 4;

  // lane j describes units first + j and first + j + 64 (physical block, valid tokens)
  int my_pb[kEnt], my_valid[kEnt];
  {
    // the table loads are consumed here on every path: nothing of the table build stays in
    // flight when the streaming loop starts
#pragma unroll
    for (int e = 0; e < kEnt; ++e) asm volatile("" ::"v"(lb[e]), "v"(pb_raw[e]));
#pragma unroll
    for (int e = 0; e < kEnt; ++e) {
      my_pb[e] = 0, my_valid[e] = 0;
      if (lane + 64 * e < cnt && pb_raw[e] >= 0 && pb_raw[e] < a.num_blocks) {
        my_pb[e] = pb_raw[e];
        // SPEC: not cut at the block's size, so that an earlier token's smaller count can be taken from it
        my_valid[e] = min(max(kv_len - lb[e] * kBS, 0), SPEC ? kBS + 4 * kMaxSetsSpec : kBS);
      }
    }
  }
  // entry of unit j (uniform)
  auto entry = [&](const int (&v)[kEnt], int j) {
    if (j < 64) return __builtin_amdgcn_readlane(v[0], j);
    if (kEnt == 2 || j < 128) return __builtin_amdgcn_readlane(v[1], j - 64);
    if (j < 192) return __builtin_amdgcn_readlane(v[kEnt > 2 ? 2 : 0], j - 128);
    return __builtin_amdgcn_readlane(v[kEnt > 2 ? 3 : 0], j - 192);
  };
  auto unit_pb = [&](int j) { return entry(my_pb, j); };
  auto unit_valid = [&](int j) { return entry(my_valid, j); };

  const size_t tile_stride = (size_t)kBS * kD;  // bytes of one (block, head) tile
  const uint8_t* const kbase = a.key_cache + (size_t)h * tile_stride;
  const uint8_t* const vbase = a.value_cache + (size_t)h * tile_stride;
  const size_t blk_stride = (size_t)a.hkv * tile_stride;
  // DYN: the scale rows of a unit travel with its K tile (the V row too: it is needed before the V tile is)
  const float* const sbuf = ldsS[DYN ? wv : 0];
  const u32 saddr = uni((int)lds_addr_of(sbuf));
  // one scale per tile: every lane loads that one scale, and LDS holds a row of 64 equal ones
  const u32 lane_x4 = a.scale_rows == 1 ? 0u : (u32)lane * 4u;
  auto fetch_k = [&](int blk) {
    dma_tile(kbase + (size_t)blk * blk_stride, kaddr, offK);
    if (DYN) {
      const size_t srow = ((size_t)blk * a.hkv + h) * a.scale_rows;
      dma_row64(a.k_scale + srow, saddr, lane_x4);
      dma_row64(a.v_scale + srow, saddr + 4 * kBS, lane_x4);
    }
  };

  // SPEC: this lane's score row of set t is MFMA row 4 t + g4 = token (4 t + g4) / group, which sees
  // toks - 1 - token fewer keys than the sequence's last token (rows of absent tokens: as the last one)
  int fewer[NSET];
#pragma unroll
  for (int t = 0; t < NSET; ++t) fewer[t] = SPEC ? max(toks - 1 - (4 * t + g4) / a.group, 0) : 0;

  PairState st[NSET];
#pragma unroll
  for (int t = 0; t < NSET; ++t) {
    st[t].m = -INFINITY;
    st[t].l = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) st[t].o[i] = 0.f;
  }

  if (wv < cnt) {  // this wavefront has units wv, wv + 4, ...
    int pb = unit_pb(wv);
    int valid = unit_valid(wv);
    fetch_k(pb);
    dma_tile(vbase + (size_t)pb * blk_stride, vaddr, offV);
#pragma unroll
    for (int t = 0; t < NSET; ++t) load_pair_finish<QUANT>(raw[t], a.sm_scale_log2, lane, st[t]);

    for (int j = wv; j < cnt; j += kWaves) {
      const bool has_next = j + kWaves < cnt;
      int pbn = 0, validn = 0;
      if (has_next) {
        pbn = unit_pb(j + kWaves);
        validn = unit_valid(j + kWaves);
      }

      // ---------------- S = Q K^T : rows = head*4 + limb, columns = token slots
      wait_vm8();  // K(j) landed (DYN: and the unit's scale rows); V(j) may still be in flight
      float kt[4] = {1.f, 1.f, 1.f, 1.f}, vt[4] = {1.f, 1.f, 1.f, 1.f};  // scales of this lane's tokens 4n .. 4n+3
      if (DYN) {
        const float4 k4 = *reinterpret_cast<const float4*>(sbuf + 4 * n16);
        const float4 v4 = *reinterpret_cast<const float4*>(sbuf + kBS + 4 * n16);
        kt[0] = k4.x; kt[1] = k4.y; kt[2] = k4.z; kt[3] = k4.w;
        vt[0] = v4.x; vt[1] = v4.y; vt[2] = v4.z; vt[3] = v4.w;
      }
      v4i S[NSET][4];
      v4f Sf[NSET][4];
#pragma unroll
      for (int stl = 0; stl < 4; ++stl) {
        const int tok = 4 * n16 + stl;  // this lane's column of tile stl is token 4n + stl
        v4i kb[2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const int c = g4 + 4 * s;
          kb[s] = *reinterpret_cast<const v4i*>(kbuf + tok * 128 + ((c ^ ((tok >> kShiftK) & 7)) * 16));
        }
#pragma unroll
        for (int t = 0; t < NSET; ++t) {
          if (QUANT == FDATTN_CACHE_INT8) {
            v4i acc = {0, 0, 0, 0};
#pragma unroll
            for (int s = 0; s < 2; ++s) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(st[t].aq[s], kb[s], acc, 0, 0, 0);
            S[t][stl] = acc;
          } else {
            v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 2; ++s) {
              const long a0 = ((long)(u32)st[t].aq[s].y << 32) | (u32)st[t].aq[s].x;
              const long a1 = ((long)(u32)st[t].aq[s].w << 32) | (u32)st[t].aq[s].z;
              const long b0 = ((long)(u32)kb[s].y << 32) | (u32)kb[s].x;
              const long b1 = ((long)(u32)kb[s].w << 32) | (u32)kb[s].z;
              acc = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a0, b0, acc, 0, 0, 0);
              acc = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a1, b1, acc, 0, 0, 0);
            }
            Sf[t][stl] = acc;
          }
        }
      }
      wait_lgkm0();  // K tile (and the scale rows) are in registers: their slots may be refilled
      if (has_next) fetch_k(pbn);

      // ---------------- online softmax in the S layout: lane = (token slot n, head g), one row set at a time
      float alpha[NSET], vmax[NSET];
#pragma unroll
      for (int t = 0; t < NSET; ++t) {
        float sv[4];
        float mb = -INFINITY;
#pragma unroll
        for (int stl = 0; stl < 4; ++stl) {
          float s;
          if (QUANT == FDATTN_CACHE_INT8)
            s = st[t].rs * ((float)S[t][stl].x + 128.0f * (float)S[t][stl].y + 16384.0f * (float)S[t][stl].z);
          else
            s = st[t].rs * ((Sf[t][stl].x + Sf[t][stl].y) + (Sf[t][stl].z + Sf[t][stl].w));
          if (DYN) s *= kt[stl];
          s = (4 * n16 + stl < valid - fewer[t]) ? s : -INFINITY;  // (a slot past the end may hold any scale, NaN included)
          sv[stl] = s;
          mb = fmaxf(mb, s);
        }
        mb = row_max16(mb);
        const float m_new = fmaxf(st[t].m, mb);
        // void unit (no valid token) and nothing seen yet: keep everything at zero
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        alpha[t] = __builtin_amdgcn_exp2f(st[t].m - m_use);
        st[t].m = m_new;
        u32 pw[4] = {0, 0, 0, 0};
        float lsum = 0.f;
        float prs[4];
#pragma unroll
        for (int stl = 0; stl < 4; ++stl) prs[stl] = __builtin_amdgcn_exp2f(sv[stl] - m_use);  // in [0, 1]
        // DYN: what is cut into limbs is weight x V scale of the token, relative to the largest such product of the
        // unit (so the unit's heaviest contribution always has full precision); that largest product scales the
        // unit's P.V.  The weight sum takes the plain weights.
        vmax[t] = 1.f;
        if (DYN) {
          float wm = 0.f;
#pragma unroll
          for (int stl = 0; stl < 4; ++stl) {
            lsum += prs[stl] * (QUANT == FDATTN_CACHE_INT8 ? 268435456.0f : 256.0f);
            prs[stl] *= (4 * n16 + stl < valid) ? vt[stl] : 0.f;  // (a slot past the end may hold any scale)
            wm = fmaxf(wm, prs[stl]);
          }
          float vm = row_max16(wm);
          // a unit whose heaviest product has all but vanished (its reciprocal would overflow, and 0 x inf is a
          // NaN) contributes nothing
          vm = vm > 7.9e-31f ? vm : 0.f;  // 2^-100
          const float inv = vm > 0.f ? 1.0f / vm : 0.f;
#pragma unroll
          for (int stl = 0; stl < 4; ++stl) prs[stl] *= inv;
          vmax[t] = vm;
        }
#pragma unroll
        for (int stl = 0; stl < 4; ++stl) {
          const float pr = prs[stl];
          if (QUANT == FDATTN_CACHE_INT8) {
            u32 x = (u32)__builtin_rintf(pr * 268435456.0f);  // 2^28
            x = min(x, 268435455u);
            if (!DYN) lsum += (float)x;
            pw[0] |= (x & 127u) << (8 * stl);
            pw[1] |= ((x >> 7) & 127u) << (8 * stl);
            pw[2] |= ((x >> 14) & 127u) << (8 * stl);
            pw[3] |= (x >> 21) << (8 * stl);
          } else {
            float x = pr * 256.0f, used = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const u32 c = (u32)__builtin_amdgcn_cvt_pk_fp8_f32(x, x, 0, false) & 0xffu;
              const float dv = __builtin_amdgcn_cvt_f32_fp8((int)c, 0);
              pw[e] |= c << (8 * stl);
              x -= dv;
              used += dv;
            }
            if (!DYN) lsum += used;
          }
        }
        st[t].l = st[t].l * alpha[t] + lsum;
        // P rows = head*4 + limb, 64 token bytes per row; this lane owns tokens 4n..4n+3
        uint8_t* const pbuf = ldsP[wv][t];
#pragma unroll
        for (int r = 0; r < 4; ++r) *reinterpret_cast<u32*>(pbuf + (4 * g4 + r) * 64 + 4 * n16) = pw[r];
      }
      wave_sync();

      // ---------------- O += P V : V^T operands come transposed out of LDS
      // V(j) landed; K(j+1) (DYN: with its two scale rows) may still be in flight
      if (!has_next) wait_vm0(); else if (DYN) wait_vm10(); else wait_vm8();
      if (QUANT != FDATTN_CACHE_INT8 && valid < kBS) {
        // e4m3 has NaN codes: a stale byte in a row past the sequence end would poison 0 * NaN
        for (int r = valid + (lane >> 3); r < kBS; r += 8)
          *reinterpret_cast<uint4*>(vbuf + r * 128 + (lane & 7) * 16) = make_uint4(0, 0, 0, 0);
        wave_sync();
      }
      v4i pa[NSET];
#pragma unroll
      for (int t = 0; t < NSET; ++t) pa[t] = *reinterpret_cast<const v4i*>(ldsP[wv][t] + n16 * 64 + 16 * g4);
#pragma unroll
      for (int ct = 0; ct < 8; ++ct) {
        v2i vr[2];
#pragma unroll
        for (int r = 0; r < 2; ++r) {
          const int tok = 16 * g4 + 8 * r + (n16 >> 1);
          const uint8_t* src = vbuf + tok * 128 + ((ct ^ ((tok >> kShiftV) & 7)) * 16) + 8 * (n16 & 1);
          vr[r] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i*)src);
        }
#pragma unroll
        for (int t = 0; t < NSET; ++t) {
          float ob;
          if (QUANT == FDATTN_CACHE_INT8) {
            const v4i vb = {vr[0].x, vr[0].y, vr[1].x, vr[1].y};
            const v4i z = {0, 0, 0, 0};
            const v4i d = __builtin_amdgcn_mfma_i32_16x16x64_i8(pa[t], vb, z, 0, 0, 0);
            ob = (float)d.x + 128.0f * (float)d.y + 16384.0f * (float)d.z + 2097152.0f * (float)d.w;
          } else {
            v4f d = {0.f, 0.f, 0.f, 0.f};
            const long a0 = ((long)(u32)pa[t].y << 32) | (u32)pa[t].x, a1 = ((long)(u32)pa[t].w << 32) | (u32)pa[t].z;
            const long b0 = ((long)(u32)vr[0].y << 32) | (u32)vr[0].x, b1 = ((long)(u32)vr[1].y << 32) | (u32)vr[1].x;
            d = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a0, b0, d, 0, 0, 0);
            d = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a1, b1, d, 0, 0, 0);
            ob = (d.x + d.y) + (d.z + d.w);
          }
          st[t].o[ct] = st[t].o[ct] * alpha[t] + (DYN ? ob * vmax[t] : ob);
        }
      }
      wait_lgkm0();  // V tile consumed
      if (has_next) dma_tile(vbase + (size_t)pbn * blk_stride, vaddr, offV);

      pb = pbn;
      valid = validn;
    }
  }

  // ---- merge the 4 wavefronts through LDS (their K slots are free now): [set][4 heads][128] floats of this
  // wavefront in its K slot, m[4], l[4] per set in its P slots
  {
    float* const mo = reinterpret_cast<float*>(kbuf);
#pragma unroll
    for (int t = 0; t < NSET; ++t) {
      float* const mml = reinterpret_cast<float*>(ldsP[wv][t]);
      const float l = row_sum16(st[t].l);
#pragma unroll
      for (int ct = 0; ct < 8; ++ct) mo[t * kSlotFloats + g4 * kD + 16 * ct + n16] = st[t].o[ct];
      if (n16 == 0) {
        mml[g4] = st[t].m;
        mml[4 + g4] = l;
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int t = 0; t < NSET; ++t) {
    const int tid = threadIdx.x, hs = tid >> 6, head = 4 * t + hs, c2 = (tid & 63) * 2;
    if (head >= vg) continue;
    float M = -INFINITY;
#pragma unroll
    for (int w2 = 0; w2 < kWaves; ++w2) M = fmaxf(M, reinterpret_cast<const float*>(ldsP[w2][t])[hs]);
    float L = 0.f, o0 = 0.f, o1 = 0.f;
    if (M > -INFINITY) {
#pragma unroll
      for (int w2 = 0; w2 < kWaves; ++w2) {
        const float* ml = reinterpret_cast<const float*>(ldsP[w2][t]);
        const float ms = ml[hs];
        const float f = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - M);
        L += ml[4 + hs] * f;
        const float2 v = *reinterpret_cast<const float2*>(reinterpret_cast<const float*>(ldsK[w2]) + t * kSlotFloats + hs * kD + c2);
        o0 += v.x * f;
        o1 += v.y * f;
      }
    }
    if (single) {
      // the only chunk of this pair: finish here
      const float inv = L > 0.f ? 1.0f / L : 0.f;
      const float r0 = o0 * inv * (DYN ? 1.f : a.v_scale[h * kD + c2]), r1 = o1 * inv * (DYN ? 1.f : a.v_scale[h * kD + c2 + 1]);
      *reinterpret_cast<u32*>(out_row(head) + c2) = (u32)f32_to_bf16(r0) | ((u32)f32_to_bf16(r1) << 16);
    } else {
      // partial of (pair, chunk): o [sets * 4 heads][128], then m[4], l[4] per set
      const size_t slot = (size_t)p * a.chunks_per_pair + ck;
      *reinterpret_cast<float2*>(a.part_o + slot * (NSET * kSlotFloats) + head * kD + c2) = make_float2(o0, o1);
      if ((tid & 63) == 0) {
        a.part_ml[slot * (NSET * 8) + t * 8 + hs] = M;
        a.part_ml[slot * (NSET * 8) + t * 8 + 4 + hs] = L;
      }
    }
  }
}

// One workgroup per (sequence, KV head, query head) whose list spans several chunks: merges their partials,
// applies the V scale and writes bf16.  Single-chunk pairs were finished by the main kernel.  The four
// wavefronts take the chunks in turn (wavefront w: chunks w, w + 4, ...), four chunks' loads in flight at a
// time - a list of 64 chunks costs 4 round trips to memory, not 64 - and meet in LDS.  Lane = two channels.
template <bool SPARSE>
__global__ __launch_bounds__(256) void decode_c8_combine_kernel(C8Args a) {
  __shared__ float red[kWaves][2 + 2 * 64];  // per wavefront: m, l, o[64][2]
  const int vgmax = a.group * a.max_tokens;  // MFMA rows of a pair: (token, head), token-major
  const int p = blockIdx.x / vgmax, head = blockIdx.x - p * vgmax, tid = threadIdx.x;
  const int b = p / a.hkv, h = p - b * a.hkv;
  const int sets = (vgmax + kG - 1) / kG, set = head >> 2, hs = head & 3;  // the partial's layout: see the main kernel
  int row, toks;
  if (!decode_rows(a.rows, b, a.max_tokens, row, toks)) return;
  const int tok = head / a.group;
  if (tok >= toks) return;
  const int kv_len = a.seq_lens_decoder[b] + (a.seq_lens_this_time ? a.seq_lens_this_time[b] : 0);
  const int n_p = pair_units<SPARSE>(a, p, kv_len);
  if (n_p <= a.chunk) return;
  const int wv = tid >> 6, lane = tid & 63, c2 = lane * 2;
  const int nch = (n_p + a.chunk - 1) / a.chunk;
  const size_t s0 = (size_t)p * a.chunks_per_pair;
  // this wavefront's chunks against its own running reference
  float M = -INFINITY, L = 0.f, o0 = 0.f, o1 = 0.f;
  for (int c0 = wv; c0 < nch; c0 += 4 * kWaves) {
    float ms[4], ls[4];
    float2 v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int c = c0 + k * kWaves;
      ms[k] = -INFINITY, ls[k] = 0.f, v[k] = make_float2(0.f, 0.f);
      if (c < nch) {
        ms[k] = a.part_ml[(s0 + c) * (sets * 8) + set * 8 + hs];
        ls[k] = a.part_ml[(s0 + c) * (sets * 8) + set * 8 + 4 + hs];
        v[k] = *reinterpret_cast<const float2*>(a.part_o + (s0 + c) * (sets * kSlotFloats) + head * kD + c2);
      }
    }
    float m_new = M;
#pragma unroll
    for (int k = 0; k < 4; ++k) m_new = fmaxf(m_new, ms[k]);
    if (m_new == -INFINITY) continue;
    const float alpha = __builtin_amdgcn_exp2f(M - m_new);  // M = -inf: 0
    L *= alpha, o0 *= alpha, o1 *= alpha;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float f = __builtin_amdgcn_exp2f(ms[k] - m_new);  // an empty chunk (m = -inf) weighs 0, its l and o are 0
      L += ls[k] * f;
      o0 += v[k].x * f;
      o1 += v[k].y * f;
    }
    M = m_new;
  }
  if (lane == 0) red[wv][0] = M, red[wv][1] = L;
  red[wv][2 + c2] = o0;
  red[wv][3 + c2] = o1;
  __syncthreads();
  if (wv != 0) return;
  float Mt = -INFINITY;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) Mt = fmaxf(Mt, red[w][0]);
  float Lt = 0.f, r0 = 0.f, r1 = 0.f;
  if (Mt > -INFINITY) {
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float f = __builtin_amdgcn_exp2f(red[w][0] - Mt);
      Lt += red[w][1] * f;
      r0 += red[w][2 + c2] * f;
      r1 += red[w][3 + c2] * f;
    }
  }
  const float inv = Lt > 0.f ? 1.0f / Lt : 0.f;
  r0 *= inv * (a.dyn ? 1.f : a.v_scale[h * kD + c2]);
  r1 *= inv * (a.dyn ? 1.f : a.v_scale[h * kD + c2 + 1]);
  uint16_t* o = a.out + ((size_t)(row + tok) * a.hkv * a.group + h * a.group + (head - tok * a.group)) * kD + c2;
  *reinterpret_cast<u32*>(o) = (u32)f32_to_bf16(r0) | ((u32)f32_to_bf16(r1) << 16);
}

// Units per workgroup.  The aim is one workgroup per LDS slot of the GPU (two per CU): every pair's
// block list is cut into as few chunks as fill the slots once, so that workgroups start once, stream
// for as long as possible and - when one chunk covers the pair - finish it without a partial or a
// merge.  Lists too long for the unit table (kMaxChunk entries) get more chunks; short lists keep at
// least one unit per wavefront.
int gpu_cu_count() {
  static std::atomic<int> cached{0};  // CUs of the current device (the devices of one machine are alike)
  int cus = cached.load(std::memory_order_relaxed);
  if (cus == 0) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    cached.store(cus, std::memory_order_relaxed);
  }
  return cus;
}

int c8_pick_chunk(int pairs, int max_units, int most) {
  const int cpp = (2 * gpu_cu_count() + pairs - 1) / pairs;  // two workgroups of this kernel fit a CU
  int chunk = (max_units + cpp - 1) / cpp;
  if (chunk < kWaves) chunk = kWaves;
  if (chunk > most) {
    // a list longer than the unit table: as few chunks as hold it, of equal size (273 units = 137 + 136, not 256 + 17:
    // the longest chunk sets the launch's duration)
    const int n = (max_units + most - 1) / most;
    chunk = (max_units + n - 1) / n;
  }
  return chunk;
}

// the decode kernel's unit table by its row sets (ceil(rows per KV head / 4))
static int decode_table_units(int sets) { return sets <= 2 ? kMaxChunkDecode : kMaxChunk; }

constexpr int kMaxPairs = 1 << 20;

// Enough for every launch over lists of AT MOST max_units units: the sparse entry point cuts the lists of
// min(max_kept, max_blocks) units, and the chunk count is not monotonic in the list length (213 units may be cut into
// more chunks than 257), so the largest count over all lengths up to max_units is taken.
size_t c8_workspace_bytes(int batch, int hkv, int max_units, int group) {
  const int pairs = batch * hkv;
  // The scan below sits on the per-step host path (every step sizes its workspace) and costs one division chain per
  // list length - tens of microseconds at 128k-token tables - so the last few answers are kept: a serving loop
  // asks for the same (pairs, max_units) step after step.
  struct Memo { int pairs, max_units, cus, most; };
  static std::mutex mu;
  static Memo memo[8];
  static int next = 0;
  const int cus = gpu_cu_count();
  int most = 0;
  {
    std::lock_guard<std::mutex> g(mu);
    for (const Memo& m : memo)
      if (m.most && m.pairs == pairs && m.max_units == max_units && m.cus == cus) most = m.most;
  }
  if (!most) {
    most = 1;
    for (int u = 1; u <= max_units; ++u) {
      const int chunk = c8_pick_chunk(pairs, u, kMaxChunk), n = (u + chunk - 1) / chunk;  // (the smaller table: never fewer chunks)
      if (n > most) most = n;
    }
    std::lock_guard<std::mutex> g(mu);
    memo[next] = Memo{pairs, max_units, cus, most};
    next = (next + 1) % 8;
  }
  const size_t slots = (size_t)pairs * most;
  const int sets = (group + kG - 1) / kG;
  return slots * sets * (kSlotFloats + 8) * sizeof(float);
}

bool c8_supported(int hq, int hkv, int d, int bs, int quant) {
  return d == kD && hkv > 0 && hq % hkv == 0 && hq / hkv >= 1 && hq / hkv <= kG * kMaxSets && bs == kBS && quant_known(quant);
}

namespace {

template <int QUANT, bool DYN, int NSET>
void launch_main(bool sparse, dim3 grid, dim3 block, hipStream_t s, const C8Args& a) {
  if (a.max_tokens > 1) {
    if (sparse) hipLaunchKernelGGL((decode_c8_kernel<QUANT, true, DYN, NSET, true>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((decode_c8_kernel<QUANT, false, DYN, NSET, true>), grid, block, 0, s, a);
  } else if constexpr (NSET <= kMaxSets) {  // (three and four row sets exist for rows of several tokens only)
    if (sparse) hipLaunchKernelGGL((decode_c8_kernel<QUANT, true, DYN, NSET>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((decode_c8_kernel<QUANT, false, DYN, NSET>), grid, block, 0, s, a);
  }
}

template <int NSET>
void launch_main_sets(int quant, bool sparse, dim3 grid, dim3 block, hipStream_t s, const C8Args& a) {
  if (quant == FDATTN_CACHE_INT8) launch_main<FDATTN_CACHE_INT8, false, NSET>(sparse, grid, block, s, a);
  else if (quant == FDATTN_CACHE_FP8_E4M3) launch_main<FDATTN_CACHE_FP8_E4M3, false, NSET>(sparse, grid, block, s, a);
  else if (quant_bytes(quant) == FDATTN_CACHE_INT8) launch_main<FDATTN_CACHE_INT8, true, NSET>(sparse, grid, block, s, a);
  else launch_main<FDATTN_CACHE_FP8_E4M3, true, NSET>(sparse, grid, block, s, a);
}

}  // namespace

int decode_c8_launch(const void* q, const void* key_cache, const void* value_cache, const float* k_scale,
                     const float* v_scale, const int32_t* block_tables, const int32_t* seq_lens_decoder,
                     const int32_t* seq_lens_this_time, const int32_t* kept_blocks, const int32_t* kept_counts,
                     int max_kept, void* out, void* workspace, size_t workspace_bytes, int batch, int hq,
                     int hkv, int d, int bs, int max_blocks, int num_blocks, int quant, float sm_scale,
                     hipStream_t s, int stages, RowMap rows, int max_tokens) {
  (void)d; (void)bs;
  const bool sparse = kept_blocks != nullptr;
  if (max_tokens < 1) max_tokens = 1;
  const int pairs = batch * hkv, group = hq / hkv, vgmax = group * max_tokens, sets = (vgmax + kG - 1) / kG;
  if (max_tokens > 1 && (!rows.cu_seqlens_q || vgmax > kG * kMaxSetsSpec))
    return fail(FDATTN_ERR_SHAPE, "fdattn_decode_attention: decode rows of up to %d tokens need a step's row map and "
                "tokens x query heads per KV head <= %d (here %d)", max_tokens, kG * kMaxSetsSpec, vgmax);
  const int max_units = sparse ? (max_kept < max_blocks ? max_kept : max_blocks) : max_blocks;
  const int chunk = c8_pick_chunk(pairs, max_units, decode_table_units(sets));
  const int cpp = ((max_units + chunk - 1) / chunk);
  if (pairs > kMaxPairs)
    return fail(FDATTN_ERR_SHAPE, "fdattn_decode_attention: batch*kv_heads = %d exceeds %d", pairs, kMaxPairs);
  if ((long long)pairs * (cpp > vgmax ? cpp : vgmax) > 0x7fffffffLL)
    return fail(FDATTN_ERR_SHAPE, "fdattn_decode_attention: %d pairs x %d chunks exceed the grid limit", pairs, cpp);
  const size_t slots = (size_t)pairs * cpp;
  const size_t need = slots * sets * (kSlotFloats + 8) * sizeof(float);
  if (workspace_bytes < need)
    return fail(FDATTN_ERR_WORKSPACE, "fdattn_decode_attention: workspace %zu B < required %zu B", workspace_bytes, need);
  float* part_o = (float*)workspace;
  float* part_ml = part_o + slots * sets * kSlotFloats;
  C8Args a{(const uint16_t*)q, (const uint8_t*)key_cache, (const uint8_t*)value_cache, k_scale, v_scale,
           block_tables, seq_lens_decoder, seq_lens_this_time, kept_blocks, kept_counts, max_kept, part_o,
           part_ml, (uint16_t*)out, rows, batch, hkv, max_blocks, num_blocks, chunk, cpp,
           sm_scale * 1.4426950408889634f, quant_dynamic(quant) ? 1 : 0, group, max_tokens, scale_rows(quant, kBS)};
  const dim3 grid(cpp * pairs), block(kWaves * 64);
  if (stages & 1) {
    if (sets == 1) launch_main_sets<1>(quant, sparse, grid, block, s, a);
    else if (sets == 2) launch_main_sets<2>(quant, sparse, grid, block, s, a);
    else if (sets == 3) launch_main_sets<3>(quant, sparse, grid, block, s, a);
    else launch_main_sets<4>(quant, sparse, grid, block, s, a);
  }
  int rc = check_launch("fdattn_decode_attention (mfma)");
  if (rc || !(stages & 2)) return rc;
  if (cpp == 1) return 0;  // every pair was one chunk and has been finished by the main kernel
  if (sparse) hipLaunchKernelGGL(decode_c8_combine_kernel<true>, dim3(pairs * vgmax), dim3(256), 0, s, a);
  else hipLaunchKernelGGL(decode_c8_combine_kernel<false>, dim3(pairs * vgmax), dim3(256), 0, s, a);
  return check_launch("fdattn_decode_attention (merge)");
}

}  // namespace fdattn
