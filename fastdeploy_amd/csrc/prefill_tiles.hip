// Chunked-prefill ("append") attention on the MFMA units for the shapes the hand-scheduled kernel
// (prefill_v2.hip: head_dim 128, block_size 64) does not take: head_dim 64, 128 or 256 with ANY block size.
//
// Same numbers as that kernel: cache bytes staged in LDS as fp16 holding the byte's exact value, the
// per-channel K scale folded into Q as two fp16 terms (22 significant bits), the formats with scale caches
// with Q as it is and the K scale on the fp32 score, the V scale on the weight's exponent; the chunk's own bf16
// K against the bf16 Q; fp16 softmax weights; scores transposed (S^T = K Q^T, v_mfma_f32_32x32x16) so that a
// lane owns one query and P^T is the B operand of O^T += V^T P^T, V^T read transposed out of LDS.
//
// Plain structure, scheduled by the compiler: a workgroup = 8 wavefronts (4 at head_dim 256) x 32 queries of one
// head - two wavefronts per SIMD, so that one's MFMAs fill the other's softmax - walks the keys
// in tiles of 32 - the cached prefix row by row through the block table (a tile may span blocks), then the
// chunk's own keys to the diagonal - with two tile buffers in LDS, the next tile's loads in registers and one
// barrier per tile; per tile a wavefront runs S = K Q, the softmax, O += V P one after the other.  The exponent
// reference of a query is raised only when its weight sum over a tile exceeds 2^14 (every weight stays inside fp16).
#include <atomic>

#include "launch.h"
#include "prefill.h"
#include "prefill_mfma_common.h"

namespace fdattn {

namespace {

using namespace pf;

constexpr int TK = 32;                          // keys per tile
// wavefronts per workgroup, 32 queries each: 8 (two per SIMD) where the registers allow it, so that a staged tile
// serves 256 queries; head_dim 256 has room for 4
template <int D>
constexpr int waves_t() { return D <= 128 ? 8 : 4; }

template <int D>
struct TileLay {
  // 16-bit elements per K / V row in LDS: 16 B of padding keep the 32 rows of a ds_read_b128 on distinct banks,
  // 64 B keep the rows a ds_read_b64_tr_b16 touches apart (the strides are 4 and 16 banks modulo 64 at every D)
  static constexpr int LDK = D + 8, LDV = D + 32;
  static constexpr int K_ELEMS = TK * LDK, BUF_ELEMS = TK * (LDK + LDV);
  static constexpr size_t kScales = 2 * (size_t)BUF_ELEMS * 2, kFlags = kScales + 2 * 3 * TK * sizeof(float);
  static constexpr size_t kBytes = kFlags + 16;  // four ints: which staged tiles hold large V values
};
// Dequantised V magnitudes (the chunk's own V included) beyond which a tile's P.V product takes the softmax weights as
// two fp16 terms (one term leaves an output element off by up to 2^-11 * sum_j p_j |v_j|): as in prefill_v2.hip.
constexpr float kExactAbove = 6.0f;

// (head_dim 64 with per-channel scales fits 128 registers - two workgroups per CU, four wavefronts per SIMD - when asked
// to: left to itself the compiler stops a few registers above, at one workgroup per CU and 1.4 times the time)
template <int QUANT, bool DYN, int D>
__global__ __launch_bounds__(64 * waves_t<D>(), (D == 64 && !DYN) ? 4 : 1) void prefill_tiles_kernel(PrefillArgs a) {
  using L = TileLay<D>;
  constexpr int KT = D / 16, CT = D / 32;  // k-steps of S = K Q; 32-channel blocks of O
  constexpr int CPR = D / 16;              // 16-byte chunks per cache row
  constexpr int NCH = TK * CPR;            // chunks per cache tile and tensor (a bf16 tile of the chunk has 2 NCH)
  constexpr int NT = 64 * waves_t<D>(), BMT = 32 * waves_t<D>();  // threads, queries per workgroup
  constexpr int NC = (NCH + NT - 1) / NT;  // of them per thread
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];  // [2][K tile | V tile], then [2][3][32] scales
  float* const lds_sc = reinterpret_cast<float*>(lds + 2 * L::BUF_ELEMS);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int G = a.hq / a.hkv, units = a.batch * a.hq;
  const int u = blockIdx.x % units, qt = a.q_tiles - 1 - blockIdx.x / units;  // long query tiles first
  const int b = u / a.hq, qh = u - b * a.hq, h = qh / G;
  if (a.seq_lens_encoder && a.seq_lens_encoder[b] <= 0) return;
  const int tok0 = a.cu_seqlens_q[b], n_b = a.cu_seqlens_q[b + 1] - tok0;
  const int q0 = qt * BMT;
  if (q0 >= n_b) return;
  // (a prefix longer than the table can describe is cut there: no entry past the row is read)
  const long long cap = (long long)a.max_blocks * a.bs;
  const int p = (int)min((long long)max(a.seq_lens_decoder[b], 0), cap);
  const int j32 = lane & 31, hf = lane >> 5, q16 = lane >> 4, i16 = lane & 15;
  const int ci_raw = q0 + 32 * wv + j32, ci = min(ci_raw, n_b - 1);  // this lane's query (rows past the chunk: as its last)
  const bool wave_active = q0 + 32 * wv < n_b;
  const int n_pre = (p + TK - 1) / TK, pre_full = p / TK;
  const int n_chk = (min(n_b, q0 + BMT) + TK - 1) / TK;
  const int n_tiles = n_pre + n_chk;
  const int g_end = wave_active ? n_pre + min(q0 + 32 * wv + 31, n_b - 1) / TK + 1 : 0;  // tiles of this wavefront
  const int32_t* const table = a.block_tables + (size_t)b * a.max_blocks;
  const float sc = a.sm_scale * 1.4426950408889634f;  // logits go to the log2 domain
  // ---- which tiles need two-term weights.  Per-channel formats: the whole prefix of this KV head, if the largest code
  // times its largest V scale may exceed the limit.  Formats with scale caches and the chunk's own tiles: per tile,
  // found while the tile is staged - the threads that see a large value leave the tile's number in tile_flag[tile % 4];
  // whatever else the word holds says no, and a stale match could only send a tile down the slower, exact path.
  __attribute__((address_space(3))) int* const tile_flag = (__attribute__((address_space(3))) int*)((__attribute__((address_space(3))) uint8_t*)lds + L::kFlags);
  constexpr float kCodeMax = QUANT == FDATTN_CACHE_INT8 ? 127.0f : 448.0f;
  bool pre_exact = false;
  if (!DYN) {
    float m = 0.f;
    for (int c = lane; c < D; c += 64) m = fmaxf(m, fabsf(a.v_scale[h * D + c]));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    pre_exact = !(m * kCodeMax <= kExactAbove);  // (NaN scales: the exact path)
  }
  auto flag_tile = [&](int t, bool large) {
    if (__any(large) && lane == 0) tile_flag[t & 3] = t + 1;
  };
  auto tile_exact = [&](int t) -> bool {
    if (t < n_pre && !DYN) return pre_exact;
    return __builtin_amdgcn_readfirstlane(tile_flag[t & 3]) == t + 1;
  };

  // ---- Q as the B operand: lane = query, channels 16 st + 8 hf .. + 7 of k-step st
  v8h qa[KT], ql[KT];  // prefix: the hi and lo fp16 terms of q x k_scale x c; chunk: qa = the bf16 q as it is
  float scl = sc;      // log2-logit per unit of the prefix accumulator
  const uint16_t* const qrow = a.q + ((size_t)(tok0 + ci) * a.hq + qh) * D;
  auto load_q_prefix = [&]() {
    float x[KT][8];
    float amax = 0.f;
#pragma unroll
    for (int st = 0; st < KT; ++st) {
      const int c0 = 16 * st + 8 * hf;
      const uint4 w = *reinterpret_cast<const uint4*>(qrow + c0);
      const float4 one = make_float4(1.f, 1.f, 1.f, 1.f);
      const float4 s0 = DYN ? one : *reinterpret_cast<const float4*>(a.k_scale + h * D + c0);
      const float4 s1 = DYN ? one : *reinterpret_cast<const float4*>(a.k_scale + h * D + c0 + 4);
      x[st][0] = bf16lo_to_f32(w.x) * s0.x, x[st][1] = bf16hi_to_f32(w.x) * s0.y;
      x[st][2] = bf16lo_to_f32(w.y) * s0.z, x[st][3] = bf16hi_to_f32(w.y) * s0.w;
      x[st][4] = bf16lo_to_f32(w.z) * s1.x, x[st][5] = bf16hi_to_f32(w.z) * s1.y;
      x[st][6] = bf16lo_to_f32(w.w) * s1.z, x[st][7] = bf16hi_to_f32(w.w) * s1.w;
#pragma unroll
      for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(x[st][e]));
    }
    float c = 1.0f, cinv = 1.0f;
    if (!DYN) {
      // c = 2^(13 - floor(log2 amax)): the row's largest element lands in [2^13, 2^14)
      amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
      int e = (int)((__float_as_uint(amax) >> 23) & 0xffu) - 127;
      e = amax > 0.f && amax < INFINITY ? min(max(13 - e, -100), 100) : 0;
      c = __uint_as_float((u32)(127 + e) << 23);
      cinv = __uint_as_float((u32)(127 - e) << 23);
    }
    scl = sc * cinv;
#pragma unroll
    for (int st = 0; st < KT; ++st) {
      u32 hw[4], lw[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float x0 = sat_f16(x[st][2 * e] * c), x1 = sat_f16(x[st][2 * e + 1] * c);
        const v2h hv = {(_Float16)x0, (_Float16)x1};
        hw[e] = __builtin_bit_cast(u32, hv);
        lw[e] = pack_f16(x0 - (float)hv[0], x1 - (float)hv[1]);
      }
      qa[st] = __builtin_bit_cast(v8h, make_uint4(hw[0], hw[1], hw[2], hw[3]));
      ql[st] = __builtin_bit_cast(v8h, make_uint4(lw[0], lw[1], lw[2], lw[3]));
    }
  };
  auto load_q_chunk = [&]() {  // the chunk's scores meet the bf16 q as it is
#pragma unroll
    for (int st = 0; st < KT; ++st) qa[st] = __builtin_bit_cast(v8h, *reinterpret_cast<const uint4*>(qrow + 16 * st + 8 * hf));
  };

  // ---- staging.  Cache tile: thread -> 16-byte chunks tid + NT i of the tile's 32 rows x D bytes (row = chunk / CPR);
  // chunk tile: twice as many chunks of 8 bf16.  Every row finds its block through the table.
  const uint16_t* const k_new_seq = a.k_new + ((size_t)tok0 * a.hkv + h) * D;
  const uint16_t* const v_new_seq = a.v_new + ((size_t)tok0 * a.hkv + h) * D;
  const u32 new_stride = (u32)a.hkv * D;
  uint4 sk[2 * NC], sv[2 * NC];
  float s_scale = 1.f;  // DYN: threads 0..31 carry a key's K scale, 32..63 its V scale
  // Table entries are requested one tile ahead of the loads that need them (a dependent round trip inside fetch would
  // hold up the wavefront's whole instruction stream): ent[i] = the entry of this thread's row of chunk i of the
  // tile that the next fetch takes, ent_s the same for the key whose scales the thread carries.
  // (tiles inside one block, below: ent[i] holds the thread's constant byte offset instead, ent_s the tile's one entry)
  int ent[NC], ent_s = -1;
  // (block sizes are powers of two almost always: a shift and a mask then, not a division per row and tile)
  const int bs_shift = (a.bs & (a.bs - 1)) == 0 ? __ffs(a.bs) - 1 : -1;
  auto block_of = [&](int key) {
    if (bs_shift >= 0) return key >> bs_shift;
    return key / a.bs;
  };
  auto slot_of = [&](int key) {
    if (bs_shift >= 0) return key & (a.bs - 1);
    return key % a.bs;
  };
  auto entry_of = [&](int key) { return key < p ? table[block_of(key)] : -1; };
  // Blocks of 32 keys or a power-of-two multiple: a tile lies inside one block, so one entry (the same for every
  // thread) serves the whole tile and a thread's address is the tile's base plus an offset that never changes.
  const bool tile_in_block = bs_shift >= 5;
  if (tile_in_block) {
#pragma unroll
    for (int i = 0; i < NC; ++i) ent[i] = ((tid + NT * i) / CPR) * D + ((tid + NT * i) % CPR) * 16;
  }
  auto request_entries = [&](int t) {
    if (tile_in_block) {
      ent_s = table[(t * TK) >> bs_shift];  // (t < n_pre: the tile's first key is cached)
      return;
    }
#pragma unroll
    for (int i = 0; i < NC; ++i) ent[i] = tid + NT * i < NCH ? entry_of(t * TK + (tid + NT * i) / CPR) : -1;
    if (DYN && tid < 2 * TK) ent_s = entry_of(t * TK + (tid & (TK - 1)));
  };
  // cache row (block, slot) of key `key` of the sequence, given its table entry.  An entry inside the cached prefix must
  // name a block; one that does not (-1, or past the pool) is read as block 0 so that no access leaves the caches - its
  // keys then take part with block 0's contents: the prefill kernels mask by position only.
  auto cache_row = [&](int key, int pb) {
    return ((size_t)(pb >= 0 && pb < a.num_blocks ? pb : 0) * a.hkv + h) * a.bs + slot_of(key);
  };
  auto fetch = [&](int t) {
    if (t >= n_tiles) return;
    if (t < n_pre && tile_in_block) {
      const int pb_u = __builtin_amdgcn_readfirstlane(ent_s);
      const size_t row0 = ((size_t)(pb_u >= 0 && pb_u < a.num_blocks ? pb_u : 0) * a.hkv + h) * a.bs + ((t * TK) & (a.bs - 1));
      const uint8_t* const kb = a.key_cache + row0 * D;
      const uint8_t* const vb = a.value_cache + row0 * D;
#pragma unroll
      for (int i = 0; i < NC; ++i)
        if (tid + NT * i < NCH) {
          sk[i] = *reinterpret_cast<const uint4*>(kb + (u32)ent[i]);
          sv[i] = *reinterpret_cast<const uint4*>(vb + (u32)ent[i]);
        }
      if (DYN && tid < 2 * TK) {
        const size_t row = row0 + (tid & (TK - 1));
        const size_t srow = a.scale_rows == 1 ? row >> bs_shift : row;  // one scale per (block, head) tile, or per stored row
        s_scale = tid < TK ? a.k_scale[srow] : a.v_scale[srow];
      }
      if (t + 1 < n_pre) request_entries(t + 1);
    } else if (t < n_pre) {
#pragma unroll
      for (int i = 0; i < NC; ++i) {
        const int idx = tid + NT * i;
        if (idx < NCH) {
          const size_t off = cache_row(t * TK + idx / CPR, ent[i]) * D + (idx % CPR) * 16;
          sk[i] = *reinterpret_cast<const uint4*>(a.key_cache + off);
          sv[i] = *reinterpret_cast<const uint4*>(a.value_cache + off);
        }
      }
      if (DYN && tid < 2 * TK) {
        const size_t row = cache_row(t * TK + (tid & (TK - 1)), ent_s);
        const size_t srow = a.scale_rows == 1 ? (bs_shift >= 0 ? row >> bs_shift : row / a.bs) : row;  // one scale per (block, head) tile, or per stored row
        s_scale = tid < TK ? a.k_scale[srow] : a.v_scale[srow];
      }
      if (t + 1 < n_pre) request_entries(t + 1);
    } else {
#pragma unroll
      for (int i = 0; i < 2 * NC; ++i) {
        const int idx = tid + NT * i;
        if (idx < 2 * NCH) {
          const int j = min((t - n_pre) * TK + idx / (2 * CPR), n_b - 1);  // keys past the chunk are masked later
          const size_t off = (size_t)j * new_stride + (idx % (2 * CPR)) * 8;
          sk[i] = *reinterpret_cast<const uint4*>(k_new_seq + off);
          sv[i] = *reinterpret_cast<const uint4*>(v_new_seq + off);
        }
      }
    }
  };
  auto commit = [&](int t) {
    if (t >= n_tiles) return;
    lds_u16* const kd = (lds_u16*)lds + (size_t)(t & 1) * L::BUF_ELEMS;
    lds_u16* const vd = kd + L::K_ELEMS;
    if (t < n_pre) {
#pragma unroll
      for (int i = 0; i < NC; ++i) {
        const int idx = tid + NT * i;
        if (idx < NCH) {
          const int row = idx / CPR, ch = idx % CPR;
          // rows past the cached prefix (in its last tile) hold stale bytes (fp8 has NaN codes): zeros are staged for them
          uint4 kw = sk[i], vw = sv[i];
          if ((t + 1) * TK > p && t * TK + row >= p) kw = make_uint4(0u, 0u, 0u, 0u), vw = make_uint4(0u, 0u, 0u, 0u);
          lds_store16(kd + row * L::LDK + ch * 16, cvt8<QUANT>(kw.x, kw.y));
          lds_store16(kd + row * L::LDK + ch * 16 + 8, cvt8<QUANT>(kw.z, kw.w));
          lds_store16(vd + row * L::LDV + ch * 16, cvt8<QUANT>(vw.x, vw.y));
          lds_store16(vd + row * L::LDV + ch * 16 + 8, cvt8<QUANT>(vw.z, vw.w));
        }
      }
      if (DYN) flag_tile(t, tid >= TK && tid < 2 * TK && t * TK + (tid - TK) < p && !(fabsf(s_scale) * kCodeMax <= kExactAbove));
      if (DYN && tid < 2 * TK) {  // what the softmax needs of a key's scales, worked out once per tile
        const float sv1 = t * TK + (tid & (TK - 1)) < p ? s_scale : 1.f;  // (slots past the prefix may hold anything)
        float* const dst = lds_sc + (t & 1) * 3 * TK;
        if (tid < TK) {
          dst[tid] = sc * sv1;
        } else {
          dst[tid] = __builtin_amdgcn_logf(sv1);  // log2
          dst[TK + tid] = __builtin_amdgcn_rcpf(sv1);
        }
      }
    } else {
      F16Range vr = {0u, 0u};
#pragma unroll
      for (int i = 0; i < 2 * NC; ++i) {
        const int idx = tid + NT * i;
        if (idx < 2 * NCH) {
          const int row = idx / (2 * CPR), ch = idx % (2 * CPR);
          lds_store16(kd + row * L::LDK + ch * 8, sk[i]);
          const uint4 vh = chunk_v_f16(sv[i]);
          lds_store16(vd + row * L::LDV + ch * 8, vh);
          f16x8_range(vh, vr);
        }
      }
      flag_tile(t, f16_range_beyond(vr, kExactAbove));
    }
  };

  // ---- operands: K rows as the A operand of S^T = K Q^T; V^T, transposed on the way out of LDS, as the A operand of
  // O^T += V^T P^T.  k-slot e of lane group hf is key 16 ss + 8 (e / 4) + 4 hf + e % 4, the layout the scores come in.
  const lds_u16* const k_lane = (const lds_u16*)lds + j32 * L::LDK + 8 * hf;
  const lds_u16* const v_lane = (const lds_u16*)lds + L::K_ELEMS + (4 * hf + (i16 >> 2)) * L::LDV + 16 * (q16 & 1) + 4 * (i16 & 3);
  auto k_operand = [&](int buf, int st) {
    return *reinterpret_cast<const __attribute__((address_space(3))) v8h*>(k_lane + (size_t)buf * L::BUF_ELEMS + 16 * st);
  };
  auto v_operand = [&](int buf, int ss, int ct) {
    const lds_u16* src = v_lane + (size_t)buf * L::BUF_ELEMS + (16 * ss) * L::LDV + 32 * ct;
    const v4s r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)src);
    const v4s r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)(src + 8 * L::LDV));
    const v8s av = {r0[0], r0[1], r0[2], r0[3], r1[0], r1[1], r1[2], r1[3]};
    return __builtin_bit_cast(v8h, av);
  };

  // O^T: o[ct][r] = channel 32 ct + (r % 4) + 8 (r / 4) + 4 hf of this lane's query
  v16f o[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[ct][r] = 0.f;
  float m_ref = -INFINITY;  // exponent reference of the weights (log2 domain)
  float l_run = 0.f;        // this lane's share (its 16 of every 32 keys) of the weight sum

  // one tile of this wavefront: S = K Q, softmax, O += V P
  auto tile = [&](int g) {
    const bool pre = g < n_pre;
    const int buf = g & 1;
    v16f s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.f;
    if (pre) {
#pragma unroll
      for (int st = 0; st < KT; ++st) {
        const v8h ka = k_operand(buf, st);
        s = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka, qa[st], s, 0, 0, 0);
        if (!DYN) s = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka, ql[st], s, 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int st = 0; st < KT; ++st)
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, k_operand(buf, st)), __builtin_bit_cast(v8bf, qa[st]), s, 0, 0, 0);
    }
    // log2-logits x[r] of keys (r % 4) + 8 (r / 4) + 4 hf of the tile; keys [0, last] are visible
    const int key0 = (pre ? g : g - n_pre) * TK;
    const int last = (pre ? p - 1 - key0 : ci - key0) - 4 * hf;
    // DYN: the scales of this lane's keys, four neighbours at a time: sc x K scale, log2 V scale, 1 / V scale
    float tk[16], lv[16], iv[16];
    if (DYN && pre) {
      const float* const scales = lds_sc + buf * 3 * TK + 4 * hf;
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const float4 t4 = *reinterpret_cast<const float4*>(scales + 8 * q4);
        const float4 l4 = *reinterpret_cast<const float4*>(scales + TK + 8 * q4);
        const float4 i4 = *reinterpret_cast<const float4*>(scales + 2 * TK + 8 * q4);
        tk[4 * q4] = t4.x, tk[4 * q4 + 1] = t4.y, tk[4 * q4 + 2] = t4.z, tk[4 * q4 + 3] = t4.w;
        lv[4 * q4] = l4.x, lv[4 * q4 + 1] = l4.y, lv[4 * q4 + 2] = l4.z, lv[4 * q4 + 3] = l4.w;
        iv[4 * q4] = i4.x, iv[4 * q4 + 1] = i4.y, iv[4 * q4 + 2] = i4.z, iv[4 * q4 + 3] = i4.w;
      }
    }
    float x[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      x[r] = s[r] * (pre ? scl : sc);
      if (DYN && pre) x[r] = __builtin_fmaf(s[r], tk[r], lv[r]);  // K scale on the score, V scale on the weight
    }
    // the mask, where the tile has keys some query of the wavefront does not see (the prefix's last tile; the chunk's
    // tiles from the wavefront's first query on)
    if (pre ? g >= pre_full : key0 + TK - 1 > q0 + 32 * wv) {
#pragma unroll
      for (int r = 0; r < 16; ++r) x[r] = (r & 3) + 8 * (r >> 2) <= last ? x[r] : -INFINITY;
    }
    // Optimistic weights against the reference as it stands: a query's weight sum over the tile bounds every one of
    // them, so a sum <= 2^14 proves that all fit fp16 and the tile's maximum is never taken.  Otherwise (the first
    // tile, scores outgrowing the reference): the exact maximum, the reference raised, what the query has accumulated
    // rescaled, the weights computed again.
    u32 pw[8];
    // a tile with large V values: its weights enter O += V P as TWO fp16 terms, p = fp16(p) + fp16(p - fp16(p))
    const bool exact = tile_exact(g);
    float esum, lsum;  // the plain sum of the lane's weights; the sum that goes to the query's weight sum
    auto weights = [&]() {
      const float cst = m_ref == -INFINITY ? 0.f : -m_ref;
      esum = 0.f, lsum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        const float e0 = __builtin_amdgcn_exp2f(x[r] + cst), e1 = __builtin_amdgcn_exp2f(x[r + 1] + cst);
        pw[r >> 1] = pack_f16(e0, e1);  // round to nearest
        esum += e0 + e1;
        if (DYN && pre) {  // the weight sum takes the weights without their V scale
          lsum = __builtin_fmaf(e0, iv[r], lsum);
          lsum = __builtin_fmaf(e1, iv[r + 1], lsum);
        }
      }
      if (!(DYN && pre)) lsum = esum;
    };
    // (head_dim 64 takes the tile's maximum every time instead: eight registers fewer, which there decide whether a CU
    // holds one workgroup or two)
    constexpr bool kOptimistic = D > 64;
    bool redo = true;
    if (kOptimistic) {
      weights();
      const float qsum = esum + swap32(esum);
      redo = !(qsum <= 16384.0f) || m_ref == -INFINITY;  // also true for inf / NaN sums
    }
    if (!kOptimistic || __any(redo)) {
      float mt = -INFINITY;
#pragma unroll
      for (int r = 0; r < 16; ++r) mt = fmaxf(mt, x[r]);
      mt = fmaxf(mt, swap32(mt));
      // (every tile: raised when a score outgrows the reference by 2^13, which keeps every weight inside fp16 as well)
      const bool raise = kOptimistic ? redo && mt > m_ref : mt > m_ref + 13.0f || (m_ref == -INFINITY && mt > -INFINITY);
      const bool had_ref = m_ref > -INFINITY;  // a query without one has accumulated nothing yet
      const float alpha = raise ? (had_ref ? __builtin_amdgcn_exp2f(m_ref - mt) : 0.f) : 1.0f;
      l_run *= alpha;
      if (__any(raise && had_ref)) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[ct][r] *= alpha;
      }
      m_ref = raise ? mt : m_ref;
      weights();
    }
    l_run += lsum;
    // O += V P.  An exact tile runs the product twice: with the weights as rounded to fp16, then with what the rounding
    // left - p - fp16(p), from the logits again (exact in fp32 next to the first term, itself rounded to fp16: 22 bits in
    // all), written over the first terms.  One copy of the product's code in a loop, and no register beyond what the
    // softmax's own peak needs: head_dim 64 has two to spare before a CU holds one workgroup instead of two.
#pragma unroll 1
    for (int term = 0; term < (exact ? 2 : 1); ++term) {
      if (term == 1) {
        const float cst = m_ref == -INFINITY ? 0.f : -m_ref;
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const float e0 = __builtin_amdgcn_exp2f(x[r] + cst), e1 = __builtin_amdgcn_exp2f(x[r + 1] + cst);
          const v2h hv = __builtin_bit_cast(v2h, pw[r >> 1]);
          pw[r >> 1] = pack_f16(e0 - (float)hv[0], e1 - (float)hv[1]);
        }
      }
      const v8h pp[2] = {__builtin_bit_cast(v8h, make_uint4(pw[0], pw[1], pw[2], pw[3])),
                         __builtin_bit_cast(v8h, make_uint4(pw[4], pw[5], pw[6], pw[7]))};
#pragma unroll
      for (int ss = 0; ss < 2; ++ss)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) o[ct] = __builtin_amdgcn_mfma_f32_32x32x16_f16(v_operand(buf, ss, ct), pp[ss], o[ct], 0, 0, 0);
    }
  };


  // (the flags start empty: whatever an earlier workgroup left in these words must not name one of this walk's tiles)
  if (tid < 4) tile_flag[tid] = 0;
  __syncthreads();
  // ---- the walk: tile g in buffer g & 1, tile g + 1 staged into the other at the start of step g, tile g + 2 in flight
  bool q_is_chunk = n_pre == 0;
  if (n_pre > 0) request_entries(0);
  fetch(0);
  if (wave_active) {
    if (q_is_chunk) load_q_chunk(); else load_q_prefix();
  }
  commit(0);
  fetch(1);
  __syncthreads();
  for (int g = 0; g < n_tiles; ++g) {
    commit(g + 1);
    fetch(g + 2);
    if (g < g_end) {
      if (g == n_pre && !q_is_chunk) {
        // leaving the quantised prefix: the channels of o take their V scale (per-channel formats), q becomes the bf16 one
        if (!DYN) {
#pragma unroll
          for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) {
              const float4 vs = *reinterpret_cast<const float4*>(a.v_scale + h * D + 32 * ct + 8 * rb + 4 * hf);
              o[ct][4 * rb] *= vs.x, o[ct][4 * rb + 1] *= vs.y, o[ct][4 * rb + 2] *= vs.z, o[ct][4 * rb + 3] *= vs.w;
            }
        }
        load_q_chunk();
        q_is_chunk = true;
      }
      tile(g);
    }
    __syncthreads();  // tile g + 1 is in LDS; nobody reads tile g any more
  }

  if (!wave_active || ci_raw >= n_b) return;
  // (every wavefront's walk ends in the chunk - its own diagonal tile - so o has left the prefix's units by now)
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  uint16_t* const orow = a.out + ((size_t)(tok0 + ci) * a.hq + qh) * D;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
      *reinterpret_cast<uint2*>(orow + 32 * ct + 8 * rb + 4 * hf) =
          make_uint2(pack_bf16(o[ct][4 * rb] * inv, o[ct][4 * rb + 1] * inv), pack_bf16(o[ct][4 * rb + 2] * inv, o[ct][4 * rb + 3] * inv));
}

template <int QUANT, bool DYN, int D>
hipError_t launch_tiles(const PrefillArgs& a, int max_chunk, hipStream_t s) {
  PrefillArgs args = a;
  constexpr int BMT = 32 * waves_t<D>();
  args.q_tiles = (max_chunk + BMT - 1) / BMT;
  const dim3 grid((unsigned)a.batch * a.hq * args.q_tiles), block(64 * waves_t<D>());
  // the dynamic LDS limit is a per-device property of the kernel: raise it once on each device
  static std::atomic<unsigned long long> raised{0};  // bit d: done on device d (one word per instantiation)
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev >= 64 || !(raised.load(std::memory_order_relaxed) >> dev & 1ull)) {
    e = hipFuncSetAttribute((const void*)prefill_tiles_kernel<QUANT, DYN, D>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)TileLay<D>::kBytes);
    if (e != hipSuccess) return e;
    if (dev < 64) raised.fetch_or(1ull << dev, std::memory_order_relaxed);
  }
  hipLaunchKernelGGL((prefill_tiles_kernel<QUANT, DYN, D>), grid, block, TileLay<D>::kBytes, s, args);
  return hipSuccess;
}

template <int D>
hipError_t launch_tiles_d(const PrefillArgs& a, int max_chunk, int quant, hipStream_t s) {
  if (quant == FDATTN_CACHE_INT8) return launch_tiles<FDATTN_CACHE_INT8, false, D>(a, max_chunk, s);
  if (quant == FDATTN_CACHE_FP8_E4M3) return launch_tiles<FDATTN_CACHE_FP8_E4M3, false, D>(a, max_chunk, s);
  if (quant_bytes(quant) == FDATTN_CACHE_INT8) return launch_tiles<FDATTN_CACHE_INT8, true, D>(a, max_chunk, s);
  return launch_tiles<FDATTN_CACHE_FP8_E4M3, true, D>(a, max_chunk, s);
}

}  // namespace

bool prefill_tiles_supported(int hq, int hkv, int d, int bs, int quant) {
  return (d == 64 || d == 128 || d == 256) && bs > 0 && hkv > 0 && hq % hkv == 0 && quant_known(quant);
}

int prefill_tiles_launch(const PrefillArgs& a, int max_chunk, int quant, hipStream_t s) {
  if ((long long)a.batch * a.hq * ((max_chunk + 127) / 128) > 0x7fffffffLL)
    return fail(FDATTN_ERR_SHAPE, "fdattn_append_attention_prefill: too many workgroups for one launch");
  hipError_t e;
  if (a.d == 64) e = launch_tiles_d<64>(a, max_chunk, quant, s);
  else if (a.d == 128) e = launch_tiles_d<128>(a, max_chunk, quant, s);
  else e = launch_tiles_d<256>(a, max_chunk, quant, s);
  if (e != hipSuccess) return fail((int)e, "fdattn_append_attention_prefill: %s", hipGetErrorString(e));
  return check_launch("fdattn_append_attention_prefill (mfma, any block size)");
}

}  // namespace fdattn
