// Chunked-prefill ("append") attention on the MFMA units, head_dim 128, block_size 64.
//
// One workgroup = 4 wavefronts, one per SIMD with the whole register file (512 registers), each carrying
// 64 new tokens of one query head as two blocks of 32 queries; the workgroup walks the keys in tiles of
// 64 - first the cached prefix, one cache block per tile, then the chunk's own bf16 K / V up to the
// causal diagonal.  Every K or V operand a wavefront reads from LDS feeds the MFMAs of both query
// blocks (the LDS delivers one 1 KiB operand per 8 cycles to the whole CU; with one operand per MFMA
// the four SIMDs would ask for exactly that, so a 32-query wavefront is bound by LDS, not by MFMA).
//
// Numbers.  Cache bytes are staged in LDS as fp16 holding the byte's exact value (int8: the
// integer; e4m3: the code's value); the per-channel K scale is folded into Q, which enters the
// prefix scores as up to TWO fp16 terms, Q c = hi + lo (c: a power of two per query that puts
// the row's largest element at 2^13 .. 2^14), both accumulated by the MFMA into the same fp32
// accumulator - 22 significant bits of q * k_scale.  One fp16 term (11 bits) leaves a relative
// error of 2^-12 per channel in every score, which is beyond the output tolerance for caches
// whose dequantised magnitudes reach 5 .. 8 and far inside it for quantised unit-scale
// activations: the steady state computes the hi term and adds the lo term for the tiles whose
// measured magnitudes, with the wavefront's queries, call for it (kLoAbove); the first tiles of a
// walk and the tiles around the end of the prefix always take both.  The formats with one scale per stored row keep
// Q unscaled - bf16 is exact in fp16, one term - and apply the row's K scale to the score and
// its V scale to the softmax weight, both in fp32.  The chunk's own K stays bf16 and meets the
// bf16 Q (exact inputs).  Softmax weights are fp16, round to nearest, summed as rounded; V is
// exact (cache bytes, or bf16 -> fp16 saturating).  The per-channel V scale multiplies the
// accumulator once, when the walk leaves the prefix.
//
// Scores are computed transposed, S^T = K Q^T (v_mfma_f32_32x32x16): a lane owns one query of
// each block and 16 of every 32 keys, so row reductions are in-lane plus one exchange with
// lane ^ 32, and P^T is already the B operand of O^T += V^T P^T; V^T operands come transposed
// out of LDS (ds_read_b64_tr_b16).  The exponent reference of a query is raised only when its
// weight sum over 32 keys exceeds 2^14 (or nothing has been seen yet).
//
// The first tiles of a walk, the three tiles around the switch from the prefix to the chunk and a wavefront's
// last tile take a plain path (one product after the other); everything else runs the schedule below.  The
// output rows leave through the wavefront's private LDS as whole 256-byte rows.
//
// Schedule.  The walk advances in half tiles (32 keys).  Step g issues, in one basic block and
// with no dependence between them,  O += V P of half tile g,  S = K Q of half tile g + 2  and
// the softmax of half tile g + 1: the matrix pipe always has an MFMA stream to run while the
// vector ALU works on the softmax.  A wavefront issues in program order and an MFMA leaves it
// about half of its 32 cycles, so the softmax, the operand reads and the staging are written
// BETWEEN the MFMAs in small portions (fast_step).  Staging (global -> registers -> fp16 -> LDS)
// runs two tiles ahead with one barrier per tile; three tile slots in LDS.
#include <atomic>
#include <utility>

#include "launch.h"
#include "prefill.h"
#include "prefill_mfma_common.h"

namespace fdattn {

namespace {

using namespace pf;

constexpr int BN = 64, HD = 128, HB = 32;  // HB: keys per half tile
constexpr int LDK = 136;                   // 16-bit elements per K row in LDS (272 B: ds_read_b128 of 32 rows is conflict-free)
constexpr int LDV = 160;                   // per V row (320 B: the rows a ds_read_b64_tr_b16 touches fall on distinct banks)
constexpr int K_ELEMS = BN * LDK, BUF_ELEMS = BN * (LDK + LDV);
constexpr int kSlots = 3;
constexpr int kWavesPf = 4, BM = 64 * kWavesPf;  // queries per workgroup
constexpr int kMaxSplitsV2 = 8;
constexpr float kSumLimit = 16384.0f;  // a query's weight sum over 32 keys above which its exponent reference is raised (every weight stays inside fp16)
constexpr size_t kLdsScales = (size_t)kSlots * BUF_ELEMS * 2, kLdsQlo = kLdsScales + (size_t)kSlots * 3 * BN * sizeof(float);
constexpr size_t kLdsFlags = kLdsQlo + (size_t)kWavesPf * 8 * 64 * 16;  // four ints: which staged tiles hold large V values
constexpr size_t kLdsStats = kLdsFlags + 16;  // [4 tiles][4 wavefronts] words: what each wavefront saw of a staged prefix tile's magnitudes
constexpr size_t kLdsSink = kLdsStats + 4 * kWavesPf * sizeof(u32);  // a word per thread: where the stores of the lanes that hold no total go
constexpr size_t kLdsBytes = kLdsSink + BM * sizeof(float);
// Dequantised V magnitudes (the chunk's own V included) beyond which a tile's P.V product takes the softmax weights as
// TWO fp16 terms: one term leaves an output element off by up to 2^-11 * sum_j p_j |v_j| <= 2^-11 * max|v|, which
// passes 2e-3 only while the values a query attends to stay moderate.
constexpr float kExactAbove = 6.0f;
// The second fp16 term of q * k_scale (see the head of the file) is spent per prefix tile and wavefront, where it can
// matter.  One term rounds every q_c k_scale_c by up to 2^-12 of itself, independently per channel: the score of a key
// is then off by a random amount of standard deviation 2^-12 / sqrt(3) * (softmax_scale * sqrt(sum_c (q_c k_scale_c
// K_c)^2)) = 1.4e-4 * s_rms, s_rms being the size the scores themselves have, and an output element by at most about
// half of that times the spread v_rms of the values the query mixes (two keys of weight 1/2 each: the worst shape).
// The tile is measured while it is staged - the mean magnitude of its K codes and of its V codes, which for values
// spread like a Gaussian is 0.8 of their root mean square (flatter distributions give more: the safe side) - and a
// wavefront takes the second term for a tile when  s_rms * v_rms > kLoAbove  with
//   s_rms = softmax_scale * max over its queries |q * k_scale|_2 * 1.25 * mean |K code|,
//   v_rms = max_c v_scale_c * 1.25 * mean |V code|:
// one term then costs an output at most 7e-5 * kLoAbove = 2.1e-4 standard deviations, a tenth of the tolerance.
// (Quantised N(0,1) activations: s_rms * v_rms is about 1.2; measured against the oracle, single terms first fail at 13.)
constexpr float kLoAbove = 3.0f;

// Register plan.  A wavefront owns the SIMD's whole register file.  The upper AGPRs hold what only MFMAs touch and are
// addressed BY NAME in single-instruction asm statements; the compiler is left the 256 VGPRs and a[0:31] (it parks
// long-lived, rarely used values in the lowest AGPRs when the VGPRs run short; the build checks that it stays
// below a32 and spills nothing):
//   (per-channel formats; the formats with one scale per stored row: everything 32 higher, no lo terms, a[0:63] left)
//   a[32:159]   O^T accumulators, o[qb][ct] at 32 + 64 qb + 16 ct
//   a[160:223]  Q hi terms (fp16; bf16 q while the chunk's own keys are walked), q[qb][st] at 160 + 32 qb + 4 st
//   a[224:255]  Q lo terms of query block 0, at 224 + 4 st; those of block 1 live in LDS (a private 8 KiB per
//               wavefront, [st][lane] 16 B each) and pass through VGPRs on their way to the MFMA
// The score accumulators and the P operands are ordinary values in VGPRs.  The compiler does not know what the
// statements are, so the wait states between an MFMA's write and a vector-ALU read of the same register (11 for an
// 8-pass MFMA; nothing interlocks this in hardware) are put in by hand: mfma_settle().

template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

#define FD_A16(b) "a" #b
// names the AGPRs as clobbered once, so that the register accounting of the kernel includes all 256
__device__ __forceinline__ void claim_agprs() {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("; the AGPRs are addressed by name from here on" ::: "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", "a10", "a11", "a12", "a13", "a14", "a15", "a16", "a17", "a18", "a19", "a20", "a21", "a22", "a23", "a24", "a25", "a26", "a27", "a28", "a29", "a30", "a31", "a32", "a33", "a34", "a35", "a36", "a37", "a38", "a39", "a40", "a41", "a42", "a43", "a44", "a45", "a46", "a47", "a48", "a49", "a50", "a51", "a52", "a53", "a54", "a55", "a56", "a57", "a58", "a59", "a60", "a61", "a62", "a63", "a64", "a65", "a66", "a67", "a68", "a69", "a70", "a71", "a72", "a73", "a74", "a75", "a76", "a77", "a78", "a79", "a80", "a81", "a82", "a83", "a84", "a85", "a86", "a87", "a88", "a89", "a90", "a91", "a92", "a93", "a94", "a95", "a96", "a97", "a98", "a99", "a100", "a101", "a102", "a103", "a104", "a105", "a106", "a107", "a108", "a109", "a110", "a111", "a112", "a113", "a114", "a115", "a116", "a117", "a118", "a119", "a120", "a121", "a122", "a123", "a124", "a125", "a126", "a127", "a128", "a129", "a130", "a131", "a132", "a133", "a134", "a135", "a136", "a137", "a138", "a139", "a140", "a141", "a142", "a143", "a144", "a145", "a146", "a147", "a148", "a149", "a150", "a151", "a152", "a153", "a154", "a155", "a156", "a157", "a158", "a159", "a160", "a161", "a162", "a163", "a164", "a165", "a166", "a167", "a168", "a169", "a170", "a171", "a172", "a173", "a174", "a175", "a176", "a177", "a178", "a179", "a180", "a181", "a182", "a183", "a184", "a185", "a186", "a187", "a188", "a189", "a190", "a191", "a192", "a193", "a194", "a195", "a196", "a197", "a198", "a199", "a200", "a201", "a202", "a203", "a204", "a205", "a206", "a207", "a208", "a209", "a210", "a211", "a212", "a213", "a214", "a215", "a216", "a217", "a218", "a219", "a220", "a221", "a222", "a223", "a224", "a225", "a226", "a227", "a228", "a229", "a230", "a231", "a232", "a233", "a234", "a235", "a236", "a237", "a238", "a239", "a240", "a241", "a242", "a243", "a244", "a245", "a246", "a247", "a248", "a249", "a250", "a251", "a252", "a253", "a254", "a255");
#endif
}
#undef FD_A16

// acc = K q (first k-step) / acc += K q, the Q operand in a[QREG : QREG + 3]
template <bool F16, int QREG>
__device__ __forceinline__ void mfma_s_first(v16f& acc, v8h ka) {
  if (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, a[%2:%3], 0" : "=&v"(acc) : "v"(ka), "n"(QREG), "n"(QREG + 3));
  else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, a[%2:%3], 0" : "=&v"(acc) : "v"(ka), "n"(QREG), "n"(QREG + 3));
}
template <bool F16, int QREG>
__device__ __forceinline__ void mfma_s(v16f& acc, v8h ka) {
  if (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, a[%2:%3], %0" : "+v"(acc) : "v"(ka), "n"(QREG), "n"(QREG + 3));
  else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, a[%2:%3], %0" : "+v"(acc) : "v"(ka), "n"(QREG), "n"(QREG + 3));
}
// acc += K q with the Q operand in VGPRs
__device__ __forceinline__ void mfma_s_vq(v16f& acc, v8h ka, const u4v qq) {
  asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(ka), "v"(qq));
}
// a[OREG : OREG + 15] += V p
template <int OREG>
__device__ __forceinline__ void mfma_o(v8h va, v8h p) {
  asm volatile("v_mfma_f32_32x32x16_f16 a[%0:%1], %2, %3, a[%0:%1]" : : "n"(OREG), "n"(OREG + 15), "v"(va), "v"(p));
}
template <int REG>
__device__ __forceinline__ void acc_write(u32 x) { asm volatile("v_accvgpr_write_b32 a[%0], %1" : : "n"(REG), "v"(x)); }
template <int REG>
__device__ __forceinline__ float acc_read() {
  float x;
  asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(x) : "n"(REG));
  return x;
}
// a[REG] *= f
template <int REG>
__device__ __forceinline__ void acc_scale(float f) {
  float t;
  asm volatile("v_accvgpr_read_b32 %0, a[%2]\n\tv_mul_f32 %0, %0, %1\n\tv_accvgpr_write_b32 a[%2], %0" : "=&v"(t) : "v"(f), "n"(REG));
}
// four query-side operand registers into a[REG : REG + 3]
template <int REG>
__device__ __forceinline__ void acc_write4(u32 x0, u32 x1, u32 x2, u32 x3) {
  acc_write<REG>(x0), acc_write<REG + 1>(x1), acc_write<REG + 2>(x2), acc_write<REG + 3>(x3);
}
__device__ __forceinline__ void mfma_settle(v16f (&s)[2]) { asm volatile("s_nop 7\n\ts_nop 4" : "+v"(s[0]), "+v"(s[1])); }
__device__ __forceinline__ void mfma_settle() { asm volatile("s_nop 7\n\ts_nop 4"); }

// the sequence of launch row r: r itself, or - nth - the r-th prefill row of the batch (-1: there is none)
__device__ __forceinline__ int sequence_of_row_v2(const PrefillArgs& a, int r, bool nth) {
  if (!nth || !a.seq_lens_encoder) return r < a.batch ? r : -1;
  const int lane = threadIdx.x & 63;
  int seen = 0;
  for (int base = 0; base < a.batch; base += 64) {
    const int idx = base + lane;
    const unsigned long long m = __ballot(idx < a.batch && a.seq_lens_encoder[idx] > 0);
    const int c = __popcll(m);
    if (r < seen + c) {
      unsigned long long mm = m;
      for (int k = seen; k < r; ++k) mm &= mm - 1;
      return base + __ffsll((long long)mm) - 1;
    }
    seen += c;
  }
  return -1;
}

// how many of the launch's max_splits key splits a walk of n_tiles tiles uses
__device__ __forceinline__ int splits_of_v2(int n_tiles, int max_splits) { return min(max(n_tiles / 16, 1), max_splits); }

// The most key splits a query tile of this launch may use: n_splits, or - when the host left the number of prefill
// rows open - as many as give every CU a workgroup for the prefill rows the wavefront counts here (the host's
// prefill_auto_splits over the counted rows).  Every lane of the wavefront must be active.
// counted: the prefill rows found (at least 1), when they were counted.
__device__ __forceinline__ int launch_splits_v2(const PrefillArgs& a, int& counted) {
  counted = 1;
  if (a.split_cus <= 0 || a.n_splits <= 1) return a.n_splits;
  const int lane = threadIdx.x & 63, per_row = a.pack_slot > 0 ? a.hkv : a.hq * a.q_tiles;
  int n = 0;
  // (a count whose workgroups fill the CUs means one split whatever follows: a large batch is not read to its end)
  for (int base = 0; base < a.batch && (long long)n * per_row < a.split_cus; base += 64) {
    const int idx = base + lane;
    n += __popcll(__ballot(idx < a.batch && (!a.seq_lens_encoder || a.seq_lens_encoder[idx] > 0)));
  }
  counted = max(n, 1);
  const long long wgs = (long long)counted * per_row;
  const long long sp = (a.split_cus + wgs - 1) / wgs;
  return (int)min((long long)a.n_splits, max(sp, 1ll));
}

}  // namespace

// BLKF (with DYN): the scale caches hold one scale per (block, KV head) tile (PrefillArgs::scale_rows == 1)
template <int QUANT, bool DYN, bool BLKF>
__global__ __launch_bounds__(64 * kWavesPf) __attribute__((amdgpu_waves_per_eu(1, 1))) void prefill_v2_kernel(PrefillArgs a) {
  static_assert(DYN || !BLKF, "per-tile scales are scale caches");
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];  // [kSlots][K tile | V tile], then (DYN) [kSlots][3][64]: per key sc * K scale, log2(V scale), 1 / V scale
  float* const lds_sc = reinterpret_cast<float*>(lds + (size_t)kSlots * BUF_ELEMS);
  // this lane's Q lo operands of query block 1: k-step st at + 64 st
  __attribute__((address_space(3))) u4v* const qlo1 = (__attribute__((address_space(3))) u4v*)((__attribute__((address_space(3))) uint8_t*)lds + kLdsQlo) + (threadIdx.x >> 6) * 512 + (threadIdx.x & 63);
  claim_agprs();
  // the formats with one scale per stored row have no lo terms: their map sits 32 registers higher and the compiler may park values in a[0:63]
  constexpr int kAccO = DYN ? 64 : 32, kAccQhi = kAccO + 128, kAccQlo = 224;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Workgroup -> (sequence, query head, query tile): the XCD index (workgroup i runs on XCD i % 8) picks the
  // (sequence, KV head) pair, so that every workgroup reading one pair's K and V shares one L2, and inside an
  // XCD the query tiles come longest first.
  const bool pack = a.pack_slot > 0;
  // Launch row -> sequence, and the key split.  The host's count of prefill rows: the grid covers those rows (the
  // r-th prefill row is looked up) x the splits.  No count: the grid covers the batch once - split 0 - and, behind
  // that, one workgroup per CU for the further splits of the prefill rows counted here ((splits - 1) x their
  // workgroups < CUs, by the choice of the splits), so that the decode rows of a mixed batch cost one workgroup
  // per tile and head, not one per split as well.
  // (The count is a pass over seq_lens_encoder: the workgroups behind the batch take it first, those over the batch
  // only once they know that their row is a prefill row.)
  int bx = blockIdx.x, split = blockIdx.y, rows = a.rows, max_splits = a.n_splits;
  bool nth = a.rows < a.batch, count_later = false;
  if (a.split_cus > 0) {
    const int per_row = pack ? a.hkv : a.hq * a.q_tiles, first = a.batch * per_row;
    count_later = bx < first;
    if (!count_later) {
      int counted;
      max_splits = launch_splits_v2(a, counted);
      const int e = bx - first, wgs = counted * per_row;
      if (e >= (max_splits - 1) * wgs) return;
      split = 1 + e / wgs;
      bx = e - (split - 1) * wgs;
      rows = counted;
      nth = true;
    }
  }
  const int G = a.hq / a.hkv, pairs = rows * a.hkv, units = rows * a.hq;
  int qt, b, qh;
  if (pack) {
    qt = 0;
    b = bx / a.hkv;
    qh = (bx - b * a.hkv) * G;
  } else if ((pairs & 7) == 0) {
    const int ppx = pairs >> 3;
    const int x = bx & 7, jx = bx >> 3;
    const int r = jx % (ppx * G), pk = (r / G) * 8 + x;
    qt = a.q_tiles - 1 - jx / (ppx * G);
    b = pk / a.hkv;
    qh = (pk - b * a.hkv) * G + r % G;
  } else {
    const int u = bx % units;
    qt = a.q_tiles - 1 - bx / units;
    b = u / a.hq;
    qh = u - b * a.hq;
  }
  const int h = qh / G;
  b = sequence_of_row_v2(a, b, nth);
  if (b < 0) return;
  const int tok0 = a.cu_seqlens_q[b], n_b = a.cu_seqlens_q[b + 1] - tok0, p = a.seq_lens_decoder[b];
  const int q0 = qt * BM;
  if (q0 >= n_b) return;
  if (a.seq_lens_encoder && a.seq_lens_encoder[b] <= 0) return;
  if (count_later) {
    int counted;
    max_splits = launch_splits_v2(a, counted);
  }

  const int j32 = lane & 31, hf = lane >> 5, q16 = lane >> 4, i16 = lane & 15;
  // this lane's two queries (blocks qb = 0, 1): rows past the chunk behave like its last row and are not stored
  int ci_raw[2], ci[2], qh_lane[2];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int x = 64 * wv + 32 * qb + j32;
    ci_raw[qb] = q0 + x;
    qh_lane[qb] = qh;
    if (pack) {  // query column x is head x / slot of the group, token x % slot
      const int hg = x / a.pack_slot;
      ci_raw[qb] = hg < G ? x - hg * a.pack_slot : n_b;
      qh_lane[qb] = qh + min(hg, G - 1);
    }
    ci[qb] = min(ci_raw[qb], n_b - 1);
  }
  const bool wave_active = pack ? __ballot(ci_raw[0] < n_b || ci_raw[1] < n_b) != 0ull : q0 + 64 * wv < n_b;
  const int ci_wave_max = pack ? n_b - 1 : min(q0 + 64 * wv + 63, n_b - 1);
  const int ci_wave_min = pack ? 0 : q0 + 64 * wv;

  const int n_pre = (p + BN - 1) / BN, pre_full = p / BN;
  const int n_chk = (min(n_b, pack ? a.pack_slot : q0 + BM) + BN - 1) / BN;
  const int n_tiles = n_pre + n_chk;
  const int n_splits = splits_of_v2(n_tiles, max_splits);
  if (split >= n_splits) return;
  const int per = (n_tiles + n_splits - 1) / n_splits;
  const int t0 = split * per, t1 = min(t0 + per, n_tiles);
  if (t0 >= t1) {  // nothing to walk (only with splits): an empty partial for each of the tile's queries
    for (int i = tid; i < BM; i += 64 * kWavesPf) {
      const int hg = pack ? i / a.pack_slot : 0, tk = pack ? i - hg * a.pack_slot : q0 + i;
      if (hg < G && tk < n_b) {
        float* ml = a.part_ml + (((size_t)split * a.num_tokens + tok0 + tk) * a.hq + qh + hg) * 2;
        ml[0] = -INFINITY;
        ml[1] = 0.f;
      }
    }
    return;
  }
  const int32_t* table = a.block_tables + (size_t)b * a.max_blocks;
  const float sc = a.sm_scale * 1.4426950408889634f;  // logits go to the log2 domain
  // ---- which tiles need two-term weights (see kExactAbove).  Per-channel formats: the whole prefix of this KV head, if
  // the largest code times its largest V scale may exceed the limit (no byte is looked at).  Formats with scale caches
  // and the chunk's own tiles: per tile, found while the tile is staged - the staging threads that see a large value
  // leave the tile's number in tile_flag[tile % 4]; whatever else the word holds (an older tile, nothing yet) says no,
  // and a stale match could only send a tile down the slower, exact path.
  __attribute__((address_space(3))) int* const tile_flag = (__attribute__((address_space(3))) int*)((__attribute__((address_space(3))) uint8_t*)lds + kLdsFlags);
  constexpr float kCodeMax = QUANT == FDATTN_CACHE_INT8 ? 127.0f : 448.0f;
  bool pre_exact = false;
  float v_scale_max = 0.f;  // per-channel formats: the largest |v_scale| of this KV head
  if (!DYN) {
    const float2 vs2 = *reinterpret_cast<const float2*>(a.v_scale + h * HD + 2 * lane);
    float m = fmaxf(fabsf(vs2.x), fabsf(vs2.y));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    pre_exact = !(m * kCodeMax <= kExactAbove);  // (NaN scales: the exact path)
    v_scale_max = __any(vs2.x != vs2.x || vs2.y != vs2.y) ? NAN : m;
  }
  auto flag_tile = [&](int t, bool large) {
    if (__any(large) && lane == 0) tile_flag[t & 3] = t + 1;
  };
  auto tile_exact = [&](int t) -> bool {
    if (t >= t1) return false;
    if (t < n_pre && !DYN) return pre_exact;
    return __builtin_amdgcn_readfirstlane(tile_flag[t & 3]) == t + 1;
  };

  // ---- which prefix tiles take the second term of q * k_scale (see kLoAbove; per-channel formats): every wavefront leaves
  // what it staged of a tile - the sum of the K codes' magnitudes and of the V codes', as one word (magnitude_word) - in
  // its own word of tile_stat[tile % 4]; a reader adds the four.  lo_gain: everything else of the test, per wavefront
  // (set by q_prefix).
  __attribute__((address_space(3))) u32* const tile_stat = (__attribute__((address_space(3))) u32*)((__attribute__((address_space(3))) uint8_t*)lds + kLdsStats);
  const int wv_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  // (every lane stores - lane 63 the total, the others their partial sums into a word of their own that nobody reads:
  // a branch around the store would cut the steady state's one basic block in two)
  const int stat_sink = (int)((kLdsSink - kLdsStats) / sizeof(u32)) + tid;
  auto stat_put = [&](int t, u32 k_acc, u32 v_acc) {
    const u32 total = wave_sum_lane63(magnitude_word<QUANT>(k_acc, v_acc));
    tile_stat[lane == 63 ? (t & 3) * kWavesPf + wv_u : stat_sink] = total;
  };
  float lo_gain = INFINITY;  // times (sum |K code|) (sum |V code|) of a tile > 1: the tile takes the second term

  // half-tile steps of this wavefront: [g_begin, g_end); chunk halves wholly above its diagonal are not computed
  const int g_begin = 2 * t0;
  const int g_end = wave_active ? min(2 * t1, 2 * n_pre + ci_wave_max / HB + 1) : g_begin;

  // ---- Q as the B operand: lane = query, channels 16 s + 8 hf .. + 7 of k-step s
  float scl_pre[2] = {sc, sc};  // log2-logit per unit of the prefix accumulator
  bool q_is_chunk = false;
  // the two query rows of this lane as they are in memory: requested in one go, used by q_prefix / q_chunk below
  uint4 qraw[2][8];
  auto q_request = [&]() {
    static_for<16>([&](auto I) {
      constexpr int qb = decltype(I)::value >> 3, s = decltype(I)::value & 7;
      const uint16_t* qrow = a.q + ((size_t)(tok0 + ci[qb]) * a.hq + qh_lane[qb]) * HD;
      qraw[qb][s] = *reinterpret_cast<const uint4*>(qrow + 16 * s + 8 * hf);
    });
  };
  auto q_prefix = [&]() {
    static_for<2>([&](auto QB) {
      constexpr int qb = decltype(QB)::value;
      float x[8][8];
      float amax = 0.f, q2 = 0.f;
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        const int c0 = 16 * s + 8 * hf;
        const uint4 w = qraw[qb][s];
        const float4 one = make_float4(1.f, 1.f, 1.f, 1.f);
        const float4 s0 = DYN ? one : *reinterpret_cast<const float4*>(a.k_scale + h * HD + c0);
        const float4 s1 = DYN ? one : *reinterpret_cast<const float4*>(a.k_scale + h * HD + c0 + 4);
        x[s][0] = bf16lo_to_f32(w.x) * s0.x, x[s][1] = bf16hi_to_f32(w.x) * s0.y;
        x[s][2] = bf16lo_to_f32(w.y) * s0.z, x[s][3] = bf16hi_to_f32(w.y) * s0.w;
        x[s][4] = bf16lo_to_f32(w.z) * s1.x, x[s][5] = bf16hi_to_f32(w.z) * s1.y;
        x[s][6] = bf16lo_to_f32(w.w) * s1.z, x[s][7] = bf16hi_to_f32(w.w) * s1.w;
#pragma unroll
        for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(x[s][e])), q2 = __builtin_fmaf(x[s][e], x[s][e], q2);
      }
      float c = 1.0f, cinv = 1.0f;
      if (!DYN) {
        // the largest |q * k_scale|_2 among the wavefront's queries (a NaN or an infinity: the second term everywhere)
        q2 += swap32(q2);
        float qn = q2;
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) qn = fmaxf(qn, __shfl_xor(qn, o, 64));
        const float per_tile = 1.25f * magnitude_unit<QUANT>() / (float)(BN * HD);
        const float gain = a.sm_scale * __builtin_sqrtf(qn) * v_scale_max * per_tile * per_tile * (1.0f / kLoAbove);
        lo_gain = (qb == 0 || !(gain <= lo_gain)) && lo_gain == lo_gain ? gain : lo_gain;  // the larger one; a NaN stays

        // c = 2^(13 - floor(log2 amax)): the row's largest element lands in [2^13, 2^14)
        amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
        int e = (int)((__float_as_uint(amax) >> 23) & 0xffu) - 127;
        e = amax > 0.f && amax < INFINITY ? min(max(13 - e, -100), 100) : 0;
        c = __uint_as_float((u32)(127 + e) << 23);
        cinv = __uint_as_float((u32)(127 - e) << 23);
      }
      scl_pre[qb] = sc * cinv;
      static_for<8>([&](auto ST) {
        constexpr int st = decltype(ST)::value;
        u32 hw[4], lw[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float x0 = sat_f16(x[st][2 * e] * c), x1 = sat_f16(x[st][2 * e + 1] * c);
          const v2h hv = {(_Float16)x0, (_Float16)x1};
          hw[e] = __builtin_bit_cast(u32, hv);
          lw[e] = pack_f16(x0 - (float)hv[0], x1 - (float)hv[1]);
        }
        acc_write4<kAccQhi + 32 * qb + 4 * st>(hw[0], hw[1], hw[2], hw[3]);
        if (!DYN) {
          if (qb == 0) acc_write4<kAccQlo + 4 * st>(lw[0], lw[1], lw[2], lw[3]);
          else qlo1[64 * st] = (u4v){lw[0], lw[1], lw[2], lw[3]};
        }
      });
    });
    q_is_chunk = false;
  };
  auto q_chunk = [&]() {  // the chunk's scores meet the bf16 q as it is
    static_for<2>([&](auto QB) {
      constexpr int qb = decltype(QB)::value;
      static_for<8>([&](auto ST) {
        constexpr int st = decltype(ST)::value;
        const uint4 w = qraw[qb][st];
        acc_write4<kAccQhi + 32 * qb + 4 * st>(w.x, w.y, w.z, w.w);
      });
    });
    q_is_chunk = true;
  };
  auto load_q_chunk = [&]() {
    q_request();
    q_chunk();
  };

  // ---- staging: thread = rows (tid >> 4) + 16 i, i < 4, 8 channels each (one 16-byte LDS chunk per row and tensor)
  const int srow = tid >> 4, scc = (tid & 15) * 8;
  // cache bytes: rows (tid >> 3) + 32 i, i < 2, 16 channels each (one 16-byte load, two 16-byte LDS chunks)
  const int prow = tid >> 3, pcc = (tid & 7) * 16;
  const u32 goff = (u32)(prow * HD + pcc);
  // the chunk's own rows of this sequence and KV head (uniform bases; a thread adds row * new_stride + scc)
  const uint16_t* const k_new_seq = a.k_new + ((size_t)tok0 * a.hkv + h) * HD;
  const uint16_t* const v_new_seq = a.v_new + ((size_t)tok0 * a.hkv + h) * HD;
  const u32 new_stride = (u32)a.hkv * HD;
  uint4 stg_k[4], stg_v[4];
  float stg_s = 1.f;  // DYN: threads 0..63 carry a row's K scale, 64..127 its V scale
  int vzero;
  asm("v_mov_b32 %0, 0" : "=v"(vzero));  // hides from the compiler that the table index is uniform (no early scalar wait)
  int pb_next = 0;
  // the loads of tile t into a set of staging registers; entry: the tile's block-table entry (prefix tiles)
  auto fetch_to = [&](int t, int entry, uint4 (&stg_k)[4], uint4 (&stg_v)[4], float& stg_s) {
    if (t >= t1) return;
    if (t < n_pre) {
      const int pb_u = __builtin_amdgcn_readfirstlane(entry);
      const int pb = (pb_u >= 0 && pb_u < a.num_blocks) ? pb_u : 0;
      const size_t blk = ((size_t)pb * a.hkv + h) * (BN * HD);
      const uint8_t* kb = a.key_cache + blk;
      const uint8_t* vb = a.value_cache + blk;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        stg_k[i] = *reinterpret_cast<const uint4*>(kb + (goff + (u32)(i * 32 * HD)));
        stg_v[i] = *reinterpret_cast<const uint4*>(vb + (goff + (u32)(i * 32 * HD)));
      }
      if (DYN && tid < 2 * BN) {
        const size_t srow0 = ((size_t)pb * a.hkv + h) * a.scale_rows + (a.scale_rows == 1 ? 0 : (tid & (BN - 1)));
        stg_s = tid < BN ? a.k_scale[srow0] : a.v_scale[srow0];
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = min((t - n_pre) * BN + srow + i * 16, n_b - 1);  // keys past the chunk are masked later
        const size_t off = (size_t)j * new_stride + scc;
        stg_k[i] = *reinterpret_cast<const uint4*>(k_new_seq + off);
        stg_v[i] = *reinterpret_cast<const uint4*>(v_new_seq + off);
      }
    }
  };
  // the walk's own staging registers; the table entry of the tile after the one fetched is requested on the way
  auto fetch = [&](int t) {
    const int entry = pb_next;
    if (t < n_pre && t < t1) pb_next = table[min(t + 1, n_pre - 1) + vzero];
    fetch_to(t, entry, stg_k, stg_v, stg_s);
  };
  auto commit_from = [&](int t, uint4 (&stg_k)[4], uint4 (&stg_v)[4], float& stg_s) {
    if (t >= t1) return;
    const int slot = t % kSlots;
    lds_u16* const kd = (lds_u16*)lds + (size_t)slot * BUF_ELEMS + srow * LDK + scc;
    lds_u16* const vd = (lds_u16*)lds + (size_t)slot * BUF_ELEMS + K_ELEMS + srow * LDV + scc;
    if (t < n_pre) {
      if (DYN) flag_tile(t, tid >= BN && tid < 2 * BN && t * BN + (tid - BN) < p && !(fabsf(stg_s) * kCodeMax <= kExactAbove));
      // rows past the cached prefix hold stale bytes (fp8 has NaN codes): zeros are staged for them
      if ((t + 1) * BN > p) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
          if (t * BN + prow + i * 32 >= p) stg_k[i] = make_uint4(0u, 0u, 0u, 0u), stg_v[i] = make_uint4(0u, 0u, 0u, 0u);
        if (DYN && t * BN + (tid & (BN - 1)) >= p) stg_s = 1.f;  // their scale slots may hold anything (the rows are masked)
      }
      lds_u16* const pkd = (lds_u16*)lds + (size_t)slot * BUF_ELEMS + prow * LDK + pcc;
      lds_u16* const pvd = (lds_u16*)lds + (size_t)slot * BUF_ELEMS + K_ELEMS + prow * LDV + pcc;
      u32 k_abs = 0u, v_abs = 0u;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const uint4 k0 = cvt8<QUANT>(stg_k[i].x, stg_k[i].y), k1 = cvt8<QUANT>(stg_k[i].z, stg_k[i].w);
        const uint4 v0 = cvt8<QUANT>(stg_v[i].x, stg_v[i].y), v1 = cvt8<QUANT>(stg_v[i].z, stg_v[i].w);
        lds_store16(pkd + i * 32 * LDK, k0);
        lds_store16(pkd + i * 32 * LDK + 8, k1);
        lds_store16(pvd + i * 32 * LDV, v0);
        lds_store16(pvd + i * 32 * LDV + 8, v1);
        if (!DYN) {
          code_abs_sum<QUANT>(stg_k[i].x, stg_k[i].y, k0, k_abs), code_abs_sum<QUANT>(stg_k[i].z, stg_k[i].w, k1, k_abs);
          code_abs_sum<QUANT>(stg_v[i].x, stg_v[i].y, v0, v_abs), code_abs_sum<QUANT>(stg_v[i].z, stg_v[i].w, v1, v_abs);
        }
      }
      if (!DYN) stat_put(t, k_abs, v_abs);
      if (DYN && tid < 2 * BN) {  // what the softmax needs of a row's scales, worked out once per tile
        if (tid < BN) {
          lds_sc[slot * 3 * BN + tid] = sc * stg_s;
        } else {
          lds_sc[slot * 3 * BN + tid] = __builtin_amdgcn_logf(stg_s);  // log2
          lds_sc[slot * 3 * BN + BN + tid] = __builtin_amdgcn_rcpf(stg_s);
        }
      }
    } else {
      F16Range vr = {0u, 0u};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        lds_store16(kd + i * 16 * LDK, stg_k[i]);
        const uint4 vh = chunk_v_f16(stg_v[i]);
        lds_store16(vd + i * 16 * LDV, vh);
        f16x8_range(vh, vr);
      }
      flag_tile(t, f16_range_beyond(vr, kExactAbove));
    }
  };
  auto commit = [&](int t) { commit_from(t, stg_k, stg_v, stg_s); };

  // O^T per query block in a[64 qb + 16 ct ..]: rows = channels 32 ct + (r % 4) + 8 (r / 4) + 4 hf, column = this lane's query
  static_for<128>([&](auto R) { acc_write<kAccO + decltype(R)::value>(0u); });
  float m_ref[2] = {-INFINITY, -INFINITY};  // exponent reference of the weights (log2 domain)
  float l_run[2] = {0.f, 0.f};              // this lane's share (its 16 of every 32 keys) of the weight sum
  v16f S[2][2];                             // [half-tile parity][query block]
  v8h P[2][2];                              // [query block][k-step of 16 keys]: one buffer - a step issues the MFMAs that read it before its softmax writes it

  // LDS addresses of this lane's operands in slot 0, half tile 0
  const lds_u16* const k_lane = (const lds_u16*)lds + j32 * LDK + 8 * hf;
  const lds_u16* const v_lane = (const lds_u16*)lds + K_ELEMS + (4 * hf + (i16 >> 2)) * LDV + 16 * (q16 & 1) + 4 * (i16 & 3);
  auto k_operand = [&](int slot, int kb, int st) {
    return *reinterpret_cast<const __attribute__((address_space(3))) v8h*>(k_lane + (size_t)slot * BUF_ELEMS + HB * kb * LDK + 16 * st);
  };
  // k-slot e of lane group hf is key 32 kb + 16 ss + 8 (e / 4) + 4 hf + e % 4 (the layout the scores come in); lane i16
  // supplies the row (key base + i16 / 4, channels 32 ct + 4 (i16 % 4) .. + 3)
  auto v_operand = [&](int slot, int kb, int ss, int ct) {
    const lds_u16* src = v_lane + (size_t)slot * BUF_ELEMS + (HB * kb + 16 * ss) * LDV + 32 * ct;
    const v4s r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)src);
    const v4s r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)(src + 8 * LDV));
    const v8s av = {r0[0], r0[1], r0[2], r0[3], r1[0], r1[1], r1[2], r1[3]};
    return __builtin_bit_cast(v8h, av);
  };

  // ---- S = K Q^T of half tile g (keys 32 (g & 1) .. + 31 of tile g / 2): rows = keys, columns = queries
  auto qk = [&](int g, v16f (&s)[2]) {
    const int t = g >> 1, kb = g & 1, slot = t % kSlots;
    if (t < n_pre) {
      static_for<8>([&](auto ST) {
        constexpr int st = decltype(ST)::value;
        const v8h ka = k_operand(slot, kb, st);
        if (st == 0) {
          mfma_s_first<true, kAccQhi>(s[0], ka);
          mfma_s_first<true, kAccQhi + 32>(s[1], ka);
        } else {
          mfma_s<true, kAccQhi + 4 * st>(s[0], ka);
          mfma_s<true, kAccQhi + 32 + 4 * st>(s[1], ka);
        }
        if (!DYN) {
          mfma_s<true, kAccQlo + 4 * st>(s[0], ka);
          {
            const u4v ql = qlo1[64 * st];
            mfma_s_vq(s[1], ka, ql);
          }
        }
      });
    } else {
      static_for<8>([&](auto ST) {
        constexpr int st = decltype(ST)::value;
        const v8h ka = k_operand(slot, kb, st);
        if (st == 0) {
          mfma_s_first<false, kAccQhi>(s[0], ka);
          mfma_s_first<false, kAccQhi + 32>(s[1], ka);
        } else {
          mfma_s<false, kAccQhi + 4 * st>(s[0], ka);
          mfma_s<false, kAccQhi + 32 + 4 * st>(s[1], ka);
        }
      });
    }
  };

  // the second term of q * k_scale into the scores of prefix half tile g, behind their first term (per-channel formats;
  // the steady state's steps make the first term only and call this for the tiles that need it: see kLoAbove)
  auto qk_second_term = [&](int g, v16f (&s)[2]) {
    const int t = g >> 1, kb = g & 1, slot = t % kSlots;
    static_for<8>([&](auto ST) {
      constexpr int st = decltype(ST)::value;
      const v8h ka = k_operand(slot, kb, st);
      const u4v ql = qlo1[64 * st];
      mfma_s<true, kAccQlo + 4 * st>(s[0], ka);
      mfma_s_vq(s[1], ka, ql);
    });
  };

  // ---- O^T += V^T P^T of half tile g
  auto pv = [&](int g, const v8h (&pp)[2][2]) {
    const int t = g >> 1, kb = g & 1, slot = t % kSlots;
    static_for<8>([&](auto I) {
      constexpr int ss = decltype(I)::value >> 2, ct = decltype(I)::value & 3;
      const v8h va = v_operand(slot, kb, ss, ct);
      mfma_o<kAccO + 16 * ct>(va, pp[0][ss]);
      mfma_o<kAccO + 64 + 16 * ct>(va, pp[1][ss]);
    });
  };

  // ---- softmax of half tile g, in pieces so that a caller can place them between its MFMAs.
  // DYN prefix tiles: where the scales of half tile g's keys are (this lane's keys of piece i at + 8 i)
  auto sm_scales = [&](int g) -> const float* { return lds_sc + ((g >> 1) % kSlots) * 3 * BN + HB * (g & 1) + 4 * hf; };
  auto sm_mask = [&](int g, v16f (&s)[2]) {
    const int t = g >> 1, kb = g & 1;
    const bool pre = t < n_pre;
    const int key0 = (pre ? t : t - n_pre) * BN + HB * kb;  // index of the half tile's first key in its segment
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      // keys [0, last] of the half tile are visible; this lane's keys are (r & 3) + 8 (r >> 2) + 4 hf: the lane's part
      // goes to the limit, so that the comparison is against a literal
      const int last = (pre ? p - 1 - key0 : ci[qb] - key0) - 4 * hf;
#pragma unroll
      for (int r = 0; r < 16; ++r) s[qb][r] = (r & 3) + 8 * (r >> 2) <= last ? s[qb][r] : -INFINITY;
    }
  };
  // weights of 4 scores (elements 4 piece .. + 3 of query block qb): half of one P operand, partial sums into ls / lt
  struct SmAcc { float ls[4], lt[4]; u32 w[4]; };
  struct SmScales { float4 tk, lv, iv; };
  auto sm_piece = [&](bool pre, int qb, int piece, const v16f& s, float scl, float cst, const float* scales, SmAcc& acc,
                      v8h (&pp)[2], SmScales* kept = nullptr) {
    float e4[4];
    if (DYN && pre) {
      // (the two query blocks have the same keys: where a caller deals with a piece of block 0 and then the same piece
      // of block 1, the second call takes the scales the first one read - `kept` - instead of reading them again)
      float4 tk, lv, iv;
      if (kept && qb == 1) {
        tk = kept->tk, lv = kept->lv, iv = kept->iv;
      } else {
        tk = *reinterpret_cast<const float4*>(scales + 8 * piece);
        lv = *reinterpret_cast<const float4*>(scales + BN + 8 * piece);
        iv = *reinterpret_cast<const float4*>(scales + 2 * BN + 8 * piece);
        if (kept) kept->tk = tk, kept->lv = lv, kept->iv = iv;
      }
      const float tks[4] = {tk.x, tk.y, tk.z, tk.w}, lvs[4] = {lv.x, lv.y, lv.z, lv.w}, ivs[4] = {iv.x, iv.y, iv.z, iv.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        e4[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[4 * piece + e], tks[e], cst) + lvs[e]);
        acc.lt[e] = __builtin_fmaf(e4[e], ivs[e], acc.lt[e]);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) e4[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[4 * piece + e], scl, cst));
    }
    const int wi = 2 * (piece & 1);
    acc.w[wi] = pack_f16(e4[0], e4[1]);  // round to nearest
    acc.w[wi + 1] = pack_f16(e4[2], e4[3]);
    // the weight sum takes the weights before their rounding to fp16 (relative difference < 2^-12 per weight, random in
    // sign): plain adds - a dot-product instruction between MFMAs of the same wavefront stalls it for ~10 cycles
    if (piece == 0) acc.ls[0] = e4[0], acc.ls[1] = e4[1], acc.ls[2] = e4[2], acc.ls[3] = e4[3];  // (a constant where it is called: no add to a zero)
    else acc.ls[0] += e4[0], acc.ls[1] += e4[1], acc.ls[2] += e4[2], acc.ls[3] += e4[3];
    if (piece & 1) pp[piece >> 1] = __builtin_bit_cast(v8h, make_uint4(acc.w[0], acc.w[1], acc.w[2], acc.w[3]));
  };
  // The same in units of two scores, split in two halves that fit behind one MFMA each (per-channel formats, whole
  // prefix tiles): elements 2 j and 2 j + 1 of a query block become word j % 4 of its P operand j / 4.
  struct SmCarry { float w0, t1; };
  auto sm_pair_a = [&](auto J, const v16f& s, float scl, float cst, SmCarry& c) {
    constexpr int j = decltype(J)::value;
    const float t0 = __builtin_fmaf(s[2 * j], scl, cst);
    c.t1 = __builtin_fmaf(s[2 * j + 1], scl, cst);
    c.w0 = __builtin_amdgcn_exp2f(t0);
  };
  auto sm_pair_b = [&](auto J, SmAcc& acc, const SmCarry& c, v8h (&pp)[2]) {
    constexpr int j = decltype(J)::value;
    const float w1 = __builtin_amdgcn_exp2f(c.t1);
    if constexpr (j < 2) {  // (the four partial sums start with their first weights, not with a zero and an add)
      acc.ls[(2 * j) & 3] = c.w0;
      acc.ls[(2 * j + 1) & 3] = w1;
    } else {
      acc.ls[(2 * j) & 3] += c.w0;
      acc.ls[(2 * j + 1) & 3] += w1;
    }
    u4v words = __builtin_bit_cast(u4v, pp[j >> 2]);
    words[j & 3] = pack_f16(c.w0, w1);
    pp[j >> 2] = __builtin_bit_cast(v8h, words);
  };
  auto sm_begin = [&](int qb, SmAcc& acc, float& cst) {
#pragma unroll
    for (int e = 0; e < 4; ++e) acc.ls[e] = 0.f, acc.lt[e] = 0.f;
    cst = -(m_ref[qb] == -INFINITY ? 0.f : m_ref[qb]);
  };
  // the optimistic weights are in pp; if some query's sum over the 32 keys says that its reference was too low (or it had
  // none yet): exact maximum, raise the reference of the queries that asked for it, rescale what they have
  // accumulated, compute the weights again.  Rare: the first half tile, and scores outgrowing the reference.
  // PER_TILE (per-block formats on the schedule in pairs): tile_iv = 1 / the tile's V scale - the pairs summed the
  // weights as they are stored, V scale included, and the weight sum takes them without it
  auto sm_finish = [&](bool pre, int qb, const v16f& s, float scl, const float* scales, SmAcc& acc, v8h (&pp)[2], auto PER_TILE, float tile_iv) {
    float tsum = (acc.ls[0] + acc.ls[1]) + (acc.ls[2] + acc.ls[3]);
    const float qsum = tsum + swap32(tsum);
    const bool redo = !(qsum <= kSumLimit) || m_ref[qb] == -INFINITY;  // also true for inf / NaN sums
    if (__any(redo)) {
      float mx = -INFINITY;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float x = s[r] * scl;
        if (DYN && pre) x = s[r] == -INFINITY ? -INFINITY : __builtin_fmaf(s[r], scales[8 * (r >> 2) + (r & 3)], scales[BN + 8 * (r >> 2) + (r & 3)]);
        mx = fmaxf(mx, x);
      }
      mx = fmaxf(mx, swap32(mx));
      const bool raise = redo && mx > m_ref[qb];
      const bool had_ref = m_ref[qb] > -INFINITY;  // a query without one has accumulated nothing yet: zeros need no rescaling
      const float alpha = raise ? __builtin_amdgcn_exp2f(m_ref[qb] - mx) : 1.0f;
      m_ref[qb] = raise ? mx : m_ref[qb];
      l_run[qb] *= alpha;
      if (__any(raise && had_ref)) {
        mfma_settle();
        if (qb == 0) static_for<64>([&](auto R) { acc_scale<kAccO + decltype(R)::value>(alpha); });
        else static_for<64>([&](auto R) { acc_scale<kAccO + 64 + decltype(R)::value>(alpha); });
      }
      float cst;
      sm_begin(qb, acc, cst);
#pragma unroll
      for (int piece = 0; piece < 4; ++piece) sm_piece(pre, qb, piece, s, scl, cst, scales, acc, pp);
      tsum = (acc.ls[0] + acc.ls[1]) + (acc.ls[2] + acc.ls[3]);
      // (this pass summed the weights without their V scales itself: in the form the statement below takes)
      if constexpr (decltype(PER_TILE)::value) tsum = ((acc.lt[0] + acc.lt[1]) + (acc.lt[2] + acc.lt[3])) / tile_iv;
    }
    if constexpr (decltype(PER_TILE)::value) l_run[qb] = __builtin_fmaf(tsum, tile_iv, l_run[qb]);
    else l_run[qb] += (DYN && pre) ? (acc.lt[0] + acc.lt[1]) + (acc.lt[2] + acc.lt[3]) : tsum;
  };
  // the whole softmax of half tile g, one query block after the other
  // The second fp16 term of the weights of half tile g, p - fp16(p), into O += V P: for half tiles of tiles that hold
  // large V values (tile_exact), right behind their softmax - the tile is in LDS, the scores s and the first terms pp
  // are at hand, the query's reference is final - while the first terms follow with the next step as always.  One
  // 16-key step of one query block at a time, from the scores again (one more exponential per weight: cheaper in
  // registers than carrying the fp32 weights, and this is the rare case); a weight is exact in fp32 next to its first
  // term, and the remainder is rounded to fp16: 22 bits in all.
  auto sm_second_term = [&](int g, const v16f (&s)[2], const v8h (&pp)[2][2]) {
    const int t = g >> 1, kb = g & 1, slot = t % kSlots;
    const bool pre = t < n_pre;
    const float* scales = sm_scales(g);
    static_for<2>([&](auto QB) {
      constexpr int qb = decltype(QB)::value;
      const float scl = pre ? scl_pre[qb] : sc;
      const float cst = -(m_ref[qb] == -INFINITY ? 0.f : m_ref[qb]);  // the reference the first terms were made against
      static_for<2>([&](auto SS) {
        constexpr int ss = decltype(SS)::value;
        u32 w[4];
        const u4v first = __builtin_bit_cast(u4v, pp[qb][ss]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int r = 8 * ss + 2 * j;
          float x0 = __builtin_fmaf(s[qb][r], scl, cst), x1 = __builtin_fmaf(s[qb][r + 1], scl, cst);
          if (DYN && pre) {
            x0 = __builtin_fmaf(s[qb][r], scales[8 * (r >> 2) + (r & 3)], cst) + scales[BN + 8 * (r >> 2) + (r & 3)];
            x1 = __builtin_fmaf(s[qb][r + 1], scales[8 * ((r + 1) >> 2) + ((r + 1) & 3)], cst) + scales[BN + 8 * ((r + 1) >> 2) + ((r + 1) & 3)];
          }
          const float e0 = __builtin_amdgcn_exp2f(x0), e1 = __builtin_amdgcn_exp2f(x1);
          const u32 first_j = first[j];  // (a scalar copy: this compiler's bit cast of a vector ELEMENT reads element 0 whatever the index)
          const v2h hv = __builtin_bit_cast(v2h, first_j);
          w[j] = pack_f16(e0 - (float)hv[0], e1 - (float)hv[1]);
        }
        const v8h pl = __builtin_bit_cast(v8h, make_uint4(w[0], w[1], w[2], w[3]));
        static_for<4>([&](auto CT) {
          constexpr int ct = decltype(CT)::value;
          mfma_o<kAccO + 64 * qb + 16 * ct>(v_operand(slot, kb, ss, ct), pl);
        });
      });
    });
  };
  // the whole softmax of half tile g, one query block after the other
  auto softmax = [&](int g, bool masked, v16f (&s)[2], v8h (&pp)[2][2]) {
    const bool pre = (g >> 1) < n_pre;
    mfma_settle(s);
    const float* scales = sm_scales(g);
    if (masked) sm_mask(g, s);
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const float scl = pre ? scl_pre[qb] : sc;
      SmAcc acc;
      float cst;
      sm_begin(qb, acc, cst);
#pragma unroll
      for (int piece = 0; piece < 4; ++piece) sm_piece(pre, qb, piece, s[qb], scl, cst, scales, acc, pp[qb]);
      sm_finish(pre, qb, s[qb], scl, scales, acc, pp[qb], std::false_type{}, 0.f);
    }
    if (tile_exact(g >> 1)) sm_second_term(g, s, pp);
  };

  // leaving the quantised prefix: the channels of o take their V scale (per-channel formats)
  auto leave_prefix = [&]() {
    if (DYN) return;
    mfma_settle();
    static_for<16>([&](auto I) {
      constexpr int ct = decltype(I)::value >> 2, rb = decltype(I)::value & 3;
      const float4 vs = *reinterpret_cast<const float4*>(a.v_scale + h * HD + 32 * ct + 8 * rb + 4 * hf);
      acc_scale<kAccO + 16 * ct + 4 * rb>(vs.x), acc_scale<kAccO + 64 + 16 * ct + 4 * rb>(vs.x);
      acc_scale<kAccO + 16 * ct + 4 * rb + 1>(vs.y), acc_scale<kAccO + 64 + 16 * ct + 4 * rb + 1>(vs.y);
      acc_scale<kAccO + 16 * ct + 4 * rb + 2>(vs.z), acc_scale<kAccO + 64 + 16 * ct + 4 * rb + 2>(vs.z);
      acc_scale<kAccO + 16 * ct + 4 * rb + 3>(vs.w), acc_scale<kAccO + 64 + 16 * ct + 4 * rb + 3>(vs.w);
    });
  };

  // is every key of half tile g visible to every query of this wavefront?
  auto unmasked = [&](int g) {
    const int t = g >> 1;
    if (t < n_pre) return t < pre_full;
    return !pack && (t - n_pre) * BN + HB * (g & 1) + HB - 1 <= ci_wave_min && q0 + 64 * wv + 63 < n_b;
  };

  // ---- the steady state of the walk: step g = O += V P of half tile g, then S = K Q of half tile g + 2 with the
  // softmax of half tile g + 1 dealt out between its MFMAs; the staging of tile t + 2 (registers -> LDS) and the
  // loads of tile t + 3 (global -> registers) ride between the MFMAs.  All tiles involved are whole prefix tiles
  // (CHK false) or all are tiles of the chunk's own keys (CHK true).  One basic block up to the (rare) raise of a
  // reference; the vector work is pinned where the source puts it.
  v8h va_carry[2];
  bool va_valid = false;
  const uint8_t* st_kbp = nullptr;  // block of tile t + 3 in the caches (set by the kb 0 step, used by both)
  const uint8_t* st_vbp = nullptr;
  int st_row3 = 0;  // chunk steps: this thread's first row of tile t + 3 in the chunk
  F16Range st_vr = {0u, 0u};  // chunk steps: the range of the V values this thread has staged of tile t + 2
  u32 st_abs = 0u, st_abs_k = 0u;  // prefix steps (per-channel formats): the magnitudes of what it has staged of tile t + 2's K, then V
  bool take_lo = false;            // prefix steps (per-channel formats): does tile t + 1 take the second term of q * k_scale?
  // the LDS slots of tiles t, t + 1, t + 2 of the walk's loop, rotated as it goes (a division per step otherwise)
  int slot_now = t0 % kSlots, slot_1 = (t0 + 1) % kSlots, slot_2 = (t0 + 2) % kSlots;
  auto fast_step = [&](int t, auto KB, auto CHK, auto BLKC) {
    constexpr int kb = decltype(KB)::value;
    constexpr bool CH = decltype(CHK)::value;  // the tiles are the chunk's own keys: bf16 K against the bf16 q, one term, no scales; the softmax is masked where the wavefront's diagonal crosses the half tile
    // prefix tiles of a per-block format: one K scale and one V scale per tile, so the softmax needs no per-key scales -
    // the K scale is the step's score scale, the V scale's logarithm joins the exponent reference, and the weight sum
    // takes the tile's sum times 1 / V scale: the schedule in pairs of the per-channel formats, with no second terms
    constexpr bool BLK = DYN && !CH && decltype(BLKC)::value;
    constexpr bool PAIRS = !DYN || CH || BLK;
    const int g = 2 * t + kb;
    const int slot_pv = slot_now, slot_qk = slot_1, slot_st = slot_2;  // t % kSlots, (t + 1) % kSlots, (t + 2) % kSlots: kept by the walk
    v16f (&s_new)[2] = S[kb];
    v16f (&s_sm)[2] = S[kb ^ 1];
    lds_u16* const kd = (lds_u16*)lds + (size_t)slot_st * BUF_ELEMS + prow * LDK + pcc;
    lds_u16* const vd = (lds_u16*)lds + (size_t)slot_st * BUF_ELEMS + K_ELEMS + prow * LDV + pcc;
    if (kb == 0 && CH) st_row3 = (t + 3 - n_pre) * BN + srow;
    if (kb == 0 && !CH) {
      const int pb_u = __builtin_amdgcn_readfirstlane(pb_next);
      const int pb = (pb_u >= 0 && pb_u < a.num_blocks) ? pb_u : 0;
      pb_next = table[min(t + 4, n_pre - 1) + vzero];
      const size_t blk = ((size_t)pb * a.hkv + h) * (BN * HD);
      st_kbp = a.key_cache + blk;
      st_vbp = a.value_cache + blk;
      if (DYN && tid < 2 * BN) {
        const size_t srow0 = ((size_t)pb * a.hkv + h) * a.scale_rows + (a.scale_rows == 1 ? 0 : (tid & (BN - 1)));
        const float next = tid < BN ? a.k_scale[srow0] : a.v_scale[srow0];
        flag_tile(t + 2, tid >= BN && !(fabsf(stg_s) * kCodeMax <= kExactAbove));  // (threads BN .. 2 BN - 1 hold the V scales of tile t + 2)
        if (tid < BN) {
          lds_sc[slot_st * 3 * BN + tid] = sc * stg_s;
        } else {
          lds_sc[slot_st * 3 * BN + tid] = __builtin_amdgcn_logf(stg_s);
          lds_sc[slot_st * 3 * BN + BN + tid] = __builtin_amdgcn_rcpf(stg_s);
        }
        stg_s = next;
      }
    }
    // Staging of tile t + 2, one 16-byte LDS chunk at a time, spread over the step's MFMA groups (four per half step:
    // LDS stores of all four wavefronts at once would hold up the operand reads queued behind them); a register whose
    // two chunks are out is refilled at once from tile t + 3, a whole tile period before it is needed.
    auto stage_chunk = [&](auto C) {
      constexpr int c = decltype(C)::value, pass = (c >> 1) & 1, half = c & 1;
      if constexpr (CH) {  // rows srow + 16 i of the chunk tile: K as it is (chunks 0 .. 3), V to fp16 (4 .. 7)
        constexpr int i = c & 3;
        const int j = min(st_row3 + 16 * i, n_b - 1);
        const size_t off = (size_t)j * new_stride + scc;
        // (in the walk's last tiles there is nothing left to stage or to fetch: the stores then fill a slot that nobody
        // reads any more and the loads re-read the chunk's last row - cheaper than a branch around each of them)
        if constexpr (c < 4) {
          lds_store16((lds_u16*)lds + (size_t)slot_st * BUF_ELEMS + (srow + 16 * i) * LDK + scc, stg_k[i]);
          stg_k[i] = *reinterpret_cast<const uint4*>(k_new_seq + off);
        } else {
          const uint4 vh = chunk_v_f16(stg_v[i]);
          lds_store16((lds_u16*)lds + (size_t)slot_st * BUF_ELEMS + K_ELEMS + (srow + 16 * i) * LDV + scc, vh);
          if constexpr (c == 4) st_vr = F16Range{0u, 0u};
          f16x8_range(vh, st_vr);
          if constexpr (c == 7) flag_tile(t + 2, f16_range_beyond(st_vr, kExactAbove));
          stg_v[i] = *reinterpret_cast<const uint4*>(v_new_seq + off);
        }
      } else if constexpr (c < 4) {
        const uint4 kh = half ? cvt8<QUANT>(stg_k[pass].z, stg_k[pass].w) : cvt8<QUANT>(stg_k[pass].x, stg_k[pass].y);
        lds_store16(kd + pass * 32 * LDK + 8 * half, kh);
        if constexpr (!DYN) {  // what this thread stages of tile t + 2's K, for the test of kLoAbove
          if constexpr (c == 0) st_abs = 0u;
          code_abs_sum<QUANT>(half ? stg_k[pass].z : stg_k[pass].x, half ? stg_k[pass].w : stg_k[pass].y, kh, st_abs);
        }
        if constexpr (half == 1) stg_k[pass] = *reinterpret_cast<const uint4*>(st_kbp + (goff + (u32)(pass * 32 * HD)));
      } else {
        const uint4 vh = half ? cvt8<QUANT>(stg_v[pass].z, stg_v[pass].w) : cvt8<QUANT>(stg_v[pass].x, stg_v[pass].y);
        lds_store16(vd + pass * 32 * LDV + 8 * half, vh);
        if constexpr (!DYN) {
          if constexpr (c == 4) st_abs_k = st_abs, st_abs = 0u;
          code_abs_sum<QUANT>(half ? stg_v[pass].z : stg_v[pass].x, half ? stg_v[pass].w : stg_v[pass].y, vh, st_abs);
        }
        if constexpr (half == 1) stg_v[pass] = *reinterpret_cast<const uint4*>(st_vbp + (goff + (u32)(pass * 32 * HD)));
        if constexpr (!DYN && c == 7) stat_put(t + 2, st_abs_k, st_abs);
      }
    };
    // does half tile g + 1 (whose weights this step makes) belong to a tile with large V values?  Asked now, used at the end
    const int flag_sm = (CH || DYN) ? tile_flag[((g + 1) >> 1) & 3] : 0;
    // and does half tile g + 2 (whose scores this step makes: tile t + 1) take the second term of q * k_scale?
    // (both half tiles of tile t + 1 get the same answer: worked out in the step of the first, kept for the second)
    u4v stat_w = {0u, 0u, 0u, 0u};
    if constexpr (!CH && !DYN && kb == 0) stat_w = *(const __attribute__((address_space(3))) u4v*)(tile_stat + ((t + 1) & 3) * kWavesPf);
    mfma_settle(s_sm);
    if constexpr (CH) {
      if (!unmasked(g + 1)) sm_mask(g + 1, s_sm);  // the wavefront's diagonal
    }
    // (sm_scales(g + 1), from the slots the walk keeps: half tile g + 1 is the second half of tile t or the first of t + 1)
    const float* scales = lds_sc + (kb == 0 ? slot_pv : slot_qk) * 3 * BN + HB * (kb ^ 1) + 4 * hf;
    float scl[2] = {CH ? sc : scl_pre[0], CH ? sc : scl_pre[1]};
    SmAcc acc[2];
    float cst[2];
    sm_begin(0, acc[0], cst[0]);
    sm_begin(1, acc[1], cst[1]);
    float tile_iv = 0.f;
    if constexpr (BLK) {  // the scales of half tile g + 1's tile, as its keys' entries hold them (all 64 the same)
      const float* const sct = lds_sc + (kb == 0 ? slot_pv : slot_qk) * 3 * BN;
      scl[0] = scl[1] = sct[0];
      const float lv = sct[BN];
      cst[0] += lv, cst[1] += lv;
      tile_iv = sct[2 * BN];
    }
    // ---- O += V P (g): 8 groups of two MFMAs.  The first two V operands were requested at the end of the previous
    // fast step (va_carry); the first K operands of the second product are requested under the last
    // groups.  Groups 4 .. 7 read P[.][1] only, so the first half of softmax(g + 1), which writes P[.][0], runs there.
    constexpr int VD = 4;  // V operands in flight ahead of the MFMA that uses them (the groups of this product are short: two MFMAs)
    v8h va[VD + 1], ka[3];
    u4v ql[3];
    if (va_valid) {
      va[0] = va_carry[0], va[1] = va_carry[1];
    } else {
      va[0] = v_operand(slot_pv, kb, 0, 0);
      va[1] = v_operand(slot_pv, kb, 0, 1);
    }
    static_for<VD - 2>([&](auto J) { constexpr int j = decltype(J)::value + 2; va[j] = v_operand(slot_pv, kb, j >> 2, j & 3); });
    if constexpr (PAIRS) {
      // One MFMA, then at most a few vector instructions, then the next MFMA: an 8-pass MFMA keeps its wavefront from
      // issuing for half of its 32 cycles and leaves the other half to whatever follows it in program order.  So the
      // softmax of half tile g + 1 is cut into 16 pairs of scores x two halves and dealt out one half per MFMA: the
      // pairs of P[.][0] from group 4 of O += V P on (its MFMAs no longer read that operand), those of P[.][1] under
      // S = K Q, three halves per k-step of two MFMAs (the hi terms of q * k_scale; a tile that needs the lo terms
      // gets them behind the step: qk_second_term); the staging chunks go where no softmax half is (groups 1 and 3
      // of the first product, k-steps 3 and 7 of the second).  (The formats with
      // scale caches keep the coarser schedule below: their softmax reads three scales per score from LDS, which
      // comes cheaper four scores at a time.)
      SmCarry c1, c2;
      static_for<8>([&](auto I) {
        constexpr int i = decltype(I)::value;
        if constexpr (i + VD < 8) va[(i + VD) % (VD + 1)] = v_operand(slot_pv, kb, (i + VD) >> 2, (i + VD) & 3);
        if constexpr (i >= 6) {
          ka[i - 6] = k_operand(slot_qk, kb, i - 6);
        }
        mfma_o<kAccO + 16 * (i & 3)>(va[i % (VD + 1)], P[0][i >> 2]);
        if constexpr (i >= 4) sm_pair_a(std::integral_constant<int, i - 4>{}, s_sm[0], scl[0], cst[0], c1);  // block 0, pairs 0 .. 3
        __builtin_amdgcn_sched_barrier(0);
        mfma_o<kAccO + 64 + 16 * (i & 3)>(va[i % (VD + 1)], P[1][i >> 2]);
        if constexpr (i >= 4) sm_pair_b(std::integral_constant<int, i - 4>{}, acc[0], c1, P[0]);
        if constexpr (i == 1) stage_chunk(std::integral_constant<int, 4 * kb>{});
        if constexpr (i == 3) stage_chunk(std::integral_constant<int, 4 * kb + 1>{});
        __builtin_amdgcn_sched_barrier(0);
      });
      if constexpr (!CH && !DYN && kb == 0) {  // (worked out here, long before the branch at the step's end asks for it)
        const u32 both = (stat_w[0] + stat_w[1]) + (stat_w[2] + stat_w[3]);
        const float risk = (float)(both & 0xffffu) * (float)(both >> 16) * lo_gain;
        take_lo = !(__uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(risk))) <= 1.0f);
      }
      static_for<8>([&](auto ST) {
        constexpr int st = decltype(ST)::value;
        // first pair of the k-step: block 1's pairs 0 .. 3, then block 0's pairs 4 .. 7; second pair (over two k-steps):
        // block 1's pairs 4 .. 7
        constexpr int qb1 = st < 4 ? 1 : 0, j1 = st, j2 = 4 + (st >> 1);
        const v8h kc = ka[st % 3];
        if (st == 0) mfma_s_first<!CH, kAccQhi>(s_new[0], kc); else mfma_s<!CH, kAccQhi + 4 * st>(s_new[0], kc);
        if constexpr (st + 2 < 8) {
          ka[(st + 2) % 3] = k_operand(slot_qk, kb, st + 2);
        } else {  // the next half step's first V operands: half tile g + 1
          va_carry[st - 6] = v_operand(kb == 0 ? slot_pv : slot_qk, kb ^ 1, 0, st - 6);
        }
        sm_pair_a(std::integral_constant<int, j1>{}, s_sm[qb1], scl[qb1], cst[qb1], c1);
        __builtin_amdgcn_sched_barrier(0);
        if (st == 0) mfma_s_first<!CH, kAccQhi + 32>(s_new[1], kc); else mfma_s<!CH, kAccQhi + 32 + 4 * st>(s_new[1], kc);
        sm_pair_b(std::integral_constant<int, j1>{}, acc[qb1], c1, P[qb1]);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr ((st & 1) == 0) sm_pair_a(std::integral_constant<int, j2>{}, s_sm[1], scl[1], cst[1], c2);
        else sm_pair_b(std::integral_constant<int, j2>{}, acc[1], c2, P[1]);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (st == 3) stage_chunk(std::integral_constant<int, 4 * kb + 2>{});
        if constexpr (st == 7) stage_chunk(std::integral_constant<int, 4 * kb + 3>{});
        __builtin_amdgcn_sched_barrier(0);
      });
    } else {
      SmScales piece_scales;  // a piece's scales, read for query block 0 and kept for block 1
    static_for<8>([&](auto I) {
        constexpr int i = decltype(I)::value;
        if constexpr (i + VD < 8) va[(i + VD) % (VD + 1)] = v_operand(slot_pv, kb, (i + VD) >> 2, (i + VD) & 3);
        if constexpr (i >= 6) {
          ka[i - 6] = k_operand(slot_qk, kb, i - 6);
          if (!DYN) ql[i - 6] = qlo1[64 * (i - 6)];
        }
        mfma_o<kAccO + 16 * (i & 3)>(va[i % (VD + 1)], P[0][i >> 2]);
        mfma_o<kAccO + 64 + 16 * (i & 3)>(va[i % (VD + 1)], P[1][i >> 2]);
        if constexpr (i == 1) stage_chunk(std::integral_constant<int, 4 * kb>{});
        if constexpr (i == 3) stage_chunk(std::integral_constant<int, 4 * kb + 1>{});
        if constexpr (i >= 4) {
          constexpr int qb = i & 1, piece = (i - 4) >> 1;
          sm_piece(true, qb, piece, s_sm[qb], scl_pre[qb], cst[qb], scales, acc[qb], P[qb], &piece_scales);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
      // ---- S(g + 2): 8 k-steps of four MFMAs; the second half of softmax(g + 1) in the first four
      static_for<8>([&](auto ST) {
        constexpr int st = decltype(ST)::value;
        if constexpr (st + 2 < 8) {
          ka[(st + 2) % 3] = k_operand(slot_qk, kb, st + 2);
          if (!DYN) ql[(st + 2) % 3] = qlo1[64 * (st + 2)];
        } else {  // the next half step's first V operands: half tile g + 1
          va_carry[st - 6] = v_operand(kb == 0 ? slot_pv : slot_qk, kb ^ 1, 0, st - 6);
        }
        const v8h kc = ka[st % 3];
        if (st == 0) {
          mfma_s_first<true, kAccQhi>(s_new[0], kc);
          mfma_s_first<true, kAccQhi + 32>(s_new[1], kc);
        } else {
          mfma_s<true, kAccQhi + 4 * st>(s_new[0], kc);
          mfma_s<true, kAccQhi + 32 + 4 * st>(s_new[1], kc);
        }
        if (!DYN) {
          mfma_s<true, kAccQlo + 4 * st>(s_new[0], kc);
          mfma_s_vq(s_new[1], kc, ql[st % 3]);
        }
        if constexpr (st < 4) {
          constexpr int qb = st & 1, piece = 2 + (st >> 1);
          sm_piece(true, qb, piece, s_sm[qb], scl_pre[qb], cst[qb], scales, acc[qb], P[qb], &piece_scales);
        }
        if constexpr (st == 4) stage_chunk(std::integral_constant<int, 4 * kb + 2>{});
        if constexpr (st == 6) stage_chunk(std::integral_constant<int, 4 * kb + 3>{});
        __builtin_amdgcn_sched_barrier(0);
      });
    }
    va_valid = true;
    sm_finish(!CH, 0, s_sm[0], scl[0], scales, acc[0], P[0], std::bool_constant<BLK>{}, tile_iv);
    sm_finish(!CH, 1, s_sm[1], scl[1], scales, acc[1], P[1], std::bool_constant<BLK>{}, tile_iv);
    if ((CH || DYN) ? __builtin_amdgcn_readfirstlane(flag_sm) == ((g + 1) >> 1) + 1 : pre_exact) sm_second_term(g + 1, s_sm, P);
    if constexpr (!CH && !DYN) {
      if (take_lo) qk_second_term(g + 2, s_new);
    }
  };

  // (the flags start empty: whatever an earlier workgroup left in these words must not name one of this walk's tiles)
  if (tid < 4) tile_flag[tid] = 0;
  __syncthreads();
  // ---- prologue: two tiles into LDS, the third on its way; the first two half tiles' scores, the first softmax
  // Everything that depends on the sequence's lengths alone is requested before anything is waited for: the block-table
  // entries of the first three tiles, the query rows, the first tile; the conversion of q runs while they are on their
  // way, and the second tile is requested (into registers of its own) before the first is waited for.
  {
    const int e0 = t0 < n_pre ? table[t0 + vzero] : 0;
    const int e1 = t0 + 1 < n_pre ? table[t0 + 1 + vzero] : 0;
    pb_next = t0 < n_pre ? table[min(t0 + 2, n_pre - 1) + vzero] : 0;
    q_request();
    uint4 xk[4], xv[4];
    float xs = 1.f;
    fetch_to(t0, e0, stg_k, stg_v, stg_s);
    if (t0 < n_pre) q_prefix(); else q_chunk();
    fetch_to(t0 + 1, e1, xk, xv, xs);
    commit(t0);
    commit_from(t0 + 1, xk, xv, xs);
    fetch(t0 + 2);
  }
  __syncthreads();
  if (g_begin < g_end) qk(g_begin, S[0]);
  if (g_begin + 1 < g_end) qk(g_begin + 1, S[1]);
  if (g_begin < g_end) softmax(g_begin, !unmasked(g_begin), S[0], P);

  for (int t = t0; t < t1; ++t, slot_now = slot_1, slot_1 = slot_2, slot_2 = slot_2 == kSlots - 1 ? 0 : slot_2 + 1) {
    lds_barrier();  // tile t + 1 is in LDS; nobody reads tile t - 1 any more
    if (t + 3 < n_pre && t + 3 < t1 && 2 * t + 3 < g_end) {  // tiles t .. t + 3 are whole prefix tiles of this walk
      fast_step(t, std::integral_constant<int, 0>{}, std::false_type{}, std::bool_constant<BLKF>{});
      fast_step(t, std::integral_constant<int, 1>{}, std::false_type{}, std::bool_constant<BLKF>{});
      continue;
    }
    // the same schedule over the chunk's own keys, for as long as this wavefront has scores to compute two half
    // tiles ahead (up to 2 t + 3; its last tile takes the plain path below)
    if (t >= n_pre && q_is_chunk && 2 * t + 3 < g_end) {
      fast_step(t, std::integral_constant<int, 0>{}, std::true_type{}, std::false_type{});
      fast_step(t, std::integral_constant<int, 1>{}, std::true_type{}, std::false_type{});
      continue;
    }
    va_valid = false;
    commit(t + 2);
    fetch(t + 3);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const int g = 2 * t + kb;
      if (g >= g_end) break;
      if (g + 2 < g_end && (g + 2) == 2 * n_pre && !q_is_chunk) load_q_chunk();
      pv(g, P);
      // the prefix's last half tile is in: o leaves the quantised units here - before the softmax below, whose half
      // tile is the chunk's first and may add its weights' second terms to o at once
      // (a share that ends with the prefix leaves it behind the loop, like every share that ends inside it)
      if (g + 1 == 2 * n_pre && t0 < n_pre && t1 > n_pre) leave_prefix();
      if (g + 2 < g_end) qk(g + 2, S[kb]);
      if (g + 1 < g_end) softmax(g + 1, !unmasked(g + 1), S[kb ^ 1], P);
    }
  }
  mfma_settle();

  if (!wave_active) return;
  if (t1 <= n_pre) leave_prefix();  // a share that ends inside the prefix (only with splits)
  const bool partial = n_splits > 1;  // partials for the merge: o unnormalised in fp32, the exponent reference and the weight sum
  // the wavefront's private LDS (its lo terms are no longer needed): one query block's bf16 rows, 256 B each, the
  // 16-byte pieces of row r at piece ^ (r & 15) so that neither the column-wise writes nor the row-wise reads
  // pile up on a bank
  __attribute__((address_space(3))) uint8_t* const obuf = (__attribute__((address_space(3))) uint8_t*)lds + kLdsQlo + (size_t)wv * 8192;
  // (the lane index passes through an opaque statement: otherwise the addresses below are worked out before the walk
  // and held in registers all the way through it)
  int lane_e = lane;
  asm volatile("" : "+v"(lane_e));
  const int e_j32 = lane_e & 31, e_hf = lane_e >> 5, e_q16 = lane_e >> 4, e_i16 = lane_e & 15;
  // query column x of the workgroup -> its token of the chunk and its query head; false: the column holds no row
  auto column = [&](int x, int& tok, int& head) {
    if (pack) {
      const int hg = x / a.pack_slot;
      tok = x - hg * a.pack_slot;
      head = qh + hg;
      return hg < G && tok < n_b;
    }
    tok = q0 + x;
    head = qh;
    return tok < n_b;
  };
  static_for<2>([&](auto QB) {
    constexpr int qb = decltype(QB)::value;
    const float l_tot = l_run[qb] + __shfl_xor(l_run[qb], 32, 64);
    if (partial) {
      int tok, head;
      if (!column(64 * wv + 32 * qb + e_j32, tok, head)) return;
      const size_t prow = ((size_t)split * a.num_tokens + tok0 + tok) * a.hq + head;
      float* po = a.part_o + prow * HD;
      static_for<16>([&](auto I) {
        constexpr int ct = decltype(I)::value >> 2, rb = decltype(I)::value & 3, r0 = kAccO + 64 * qb + 16 * ct + 4 * rb;
        *reinterpret_cast<float4*>(po + 32 * ct + 8 * rb + 4 * e_hf) = make_float4(acc_read<r0>(), acc_read<r0 + 1>(), acc_read<r0 + 2>(), acc_read<r0 + 3>());
      });
      if (e_hf == 0) {
        a.part_ml[prow * 2] = m_ref[qb];
        a.part_ml[prow * 2 + 1] = l_tot;
      }
      return;
    }
    // Final rows.  A lane holds one query's channels in pieces of four: stored from here, every instruction would
    // touch 64 rows with 8 bytes each.  The block goes through LDS instead and leaves as whole 256-byte rows, 16
    // lanes x 16 bytes per row.
    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    static_for<16>([&](auto I) {
      constexpr int ct = decltype(I)::value >> 2, rb = decltype(I)::value & 3, r0 = kAccO + 64 * qb + 16 * ct + 4 * rb;
      const v2f lo = {acc_read<r0>() * inv, acc_read<r0 + 1>() * inv}, hi = {acc_read<r0 + 2>() * inv, acc_read<r0 + 3>() * inv};
      typedef u32 u2v __attribute__((ext_vector_type(2)));
      const u2v w = {__builtin_bit_cast(u32, __builtin_convertvector(lo, v2bf)), __builtin_bit_cast(u32, __builtin_convertvector(hi, v2bf))};
      *reinterpret_cast<__attribute__((address_space(3))) u2v*>(obuf + e_j32 * 256 + (((4 * ct + rb) ^ (e_j32 & 15)) << 4) + 8 * e_hf) = w;
    });
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = 4 * i + e_q16, x = 64 * wv + 32 * qb + r;  // row r of the block = query column x of the workgroup
      const u4v w = *reinterpret_cast<const __attribute__((address_space(3))) u4v*>(obuf + r * 256 + ((e_i16 ^ (r & 15)) << 4));
      int tok, head;
      if (column(x, tok, head)) *reinterpret_cast<u4v*>(a.out + ((size_t)(tok0 + tok) * a.hq + head) * HD + 8 * e_i16) = w;
    }
    __builtin_amdgcn_wave_barrier();
  });
}

// Merge of the split partials: one wavefront per (new token of the batch, query head), lane = two channels.  The
// grid runs over the batch's tokens - not over rows x the longest chunk, most of which a mixed batch leaves empty -
// and a token's sequence is the one whose row starts at or before it and ends beyond it.
__global__ __launch_bounds__(256) void prefill_v2_merge_kernel(PrefillArgs a) {
  const int lane = threadIdx.x & 63;
  const long long unit = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int t = (int)(unit / a.hq), qh = (int)(unit - (long long)t * a.hq);
  if (t >= a.num_tokens) return;
  // 64-ary search over the row starts: cu_seqlens_q[lo] <= t throughout; sequences without tokens are stepped over
  int lo = 0, n = a.batch;
  while (n > 64) {
    const int step = (n + 63) / 64, idx = lo + lane * step;
    const int k = __popcll(__ballot(idx < lo + n && a.cu_seqlens_q[idx] <= t));  // >= 1: lane 0 looks at lo
    const int nlo = lo + (k - 1) * step;
    n = min(step, lo + n - nlo);
    lo = nlo;
  }
  const unsigned long long m = __ballot(lane < n && a.cu_seqlens_q[lo + lane] <= t && a.cu_seqlens_q[lo + lane + 1] > t);
  if (!m) return;
  const int b = lo + __ffsll((long long)m) - 1;
  if (a.seq_lens_encoder && a.seq_lens_encoder[b] <= 0) return;
  if (a.rows < a.batch && a.seq_lens_encoder) {  // the main kernel covered the first a.rows prefill rows only
    int before = 0;
    for (int base = 0; base < b; base += 64) before += __popcll(__ballot(base + lane < b && a.seq_lens_encoder[base + lane] > 0));
    if (before >= a.rows) return;
  }
  const int tok0 = a.cu_seqlens_q[b], n_b = a.cu_seqlens_q[b + 1] - tok0, i = t - tok0;
  const int q0 = i / a.tile_tokens * a.tile_tokens;
  const int n_tiles = (a.seq_lens_decoder[b] + BN - 1) / BN + (min(n_b, q0 + a.tile_tokens) + BN - 1) / BN;
  int counted;
  const int n_splits = splits_of_v2(n_tiles, launch_splits_v2(a, counted));
  if (n_splits <= 1) return;  // the row is final already
  const size_t row0 = ((size_t)(tok0 + i)) * a.hq + qh, stride = (size_t)a.num_tokens * a.hq;
  float ms[kMaxSplitsV2], ls[kMaxSplitsV2];
  float2 v[kMaxSplitsV2];
#pragma unroll
  for (int s = 0; s < kMaxSplitsV2; ++s)
    if (s < n_splits) {
      ms[s] = a.part_ml[(row0 + s * stride) * 2];
      ls[s] = a.part_ml[(row0 + s * stride) * 2 + 1];
      v[s] = *reinterpret_cast<const float2*>(a.part_o + (row0 + s * stride) * HD + 2 * lane);
    }
  float M = -INFINITY;
#pragma unroll
  for (int s = 0; s < kMaxSplitsV2; ++s)
    if (s < n_splits) M = fmaxf(M, ms[s]);
  float L = 0.f, o0 = 0.f, o1 = 0.f;
  if (M > -INFINITY) {
#pragma unroll
    for (int s = 0; s < kMaxSplitsV2; ++s)
      if (s < n_splits && ms[s] > -INFINITY) {
        const float f = __builtin_amdgcn_exp2f(ms[s] - M);
        L += ls[s] * f;
        o0 += v[s].x * f;
        o1 += v[s].y * f;
      }
  }
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  *reinterpret_cast<u32*>(a.out + row0 * HD + 2 * lane) = pack_bf16(o0 * inv, o1 * inv);
}

bool prefill_mfma_supported(int hq, int hkv, int d, int bs, int quant) {
  return d == HD && bs == BN && hq % hkv == 0 && quant_known(quant);
}

namespace {

template <int QUANT, bool DYN, bool BLKF = false>
hipError_t launch_v2(const PrefillArgs& a, int max_chunk, hipStream_t s) {
  PrefillArgs args = a;
  args.q_tiles = a.pack_slot > 0 ? 1 : (max_chunk + BM - 1) / BM;
  dim3 grid((unsigned)a.rows * (a.pack_slot > 0 ? a.hkv : a.hq) * args.q_tiles, a.n_splits), block(64 * kWavesPf);
  if (a.split_cus > 0) grid = dim3(grid.x + (unsigned)a.split_cus, 1);  // the batch once, and a CU's worth of workgroups for the further splits
  // the dynamic LDS limit is a per-device property of the kernel: raise it once on each device
  static std::atomic<unsigned long long> raised{0};  // bit d: done on device d (one word per instantiation)
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev >= 64 || !(raised.load(std::memory_order_relaxed) >> dev & 1ull)) {
    e = hipFuncSetAttribute((const void*)prefill_v2_kernel<QUANT, DYN, BLKF>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
    if (e != hipSuccess) return e;
    if (dev < 64) raised.fetch_or(1ull << dev, std::memory_order_relaxed);
  }
  hipLaunchKernelGGL((prefill_v2_kernel<QUANT, DYN, BLKF>), grid, block, kLdsBytes, s, args);
  return hipSuccess;
}

}  // namespace

size_t prefill_split_workspace_bytes(int num_tokens, int hq, int n_splits) {
  if (n_splits <= 1 || num_tokens <= 0 || hq <= 0) return 0;
  if (n_splits > kMaxSplitsV2) n_splits = kMaxSplitsV2;
  return (size_t)n_splits * num_tokens * hq * (HD + 2) * sizeof(float);
}

// Short chunks: when all query heads of a KV head, times the chunk's tokens, fit the 256 query columns of one
// workgroup, the workgroup takes the whole group and its staged K / V tiles serve every head.
// Returns the tokens per head slot (0: not packed).
static int pack_slot_for(int hq, int hkv, int max_chunk) {
  const int g = hkv > 0 ? hq / hkv : 0;
  if (g < 2 || max_chunk <= 0 || (long long)g * max_chunk > BM) return 0;
  return BM / g;
}

int prefill_auto_splits(int rows, int hq, int max_chunk, int hkv) {
  if (rows <= 0 || hq <= 0 || max_chunk <= 0) return 1;
  const int cus = gpu_cu_count();
  long long wgs = (long long)rows * hq * ((max_chunk + BM - 1) / BM);
  if (pack_slot_for(hq, hkv, max_chunk) > 0) wgs = (long long)rows * hkv;  // one workgroup per (row, KV head)
  const long long sp = (cus + wgs - 1) / wgs;  // enough to give every CU a workgroup
  return (int)(sp < 1 ? 1 : (sp > kMaxSplitsV2 ? kMaxSplitsV2 : sp));
}

int prefill_mfma_launch(const PrefillArgs& a_in, int max_chunk, int quant, hipStream_t s, void* workspace,
                        size_t workspace_bytes, int n_splits, int rows_hint) {
  PrefillArgs a = a_in;
  if (n_splits > kMaxSplitsV2) n_splits = kMaxSplitsV2;
  while (n_splits > 1 && (!workspace || workspace_bytes < prefill_split_workspace_bytes(a.num_tokens, a.hq, n_splits))) --n_splits;
  a.n_splits = n_splits < 1 ? 1 : n_splits;
  a.rows = rows_hint > 0 && rows_hint < a.batch && a.seq_lens_encoder ? rows_hint : a.batch;
  a.split_cus = rows_hint < 0 && a.n_splits > 1 ? gpu_cu_count() : 0;  // rows_hint < 0: the kernels count the prefill rows
  a.part_o = (float*)workspace;
  a.part_ml = a.part_o + (size_t)a.n_splits * a.num_tokens * a.hq * HD;
  if ((long long)a_in.batch * a_in.hq * ((max_chunk + BM - 1) / BM) + a.split_cus > 0x7fffffffLL)  // (the workgroups behind the batch included)
    return fail(FDATTN_ERR_SHAPE, "fdattn_append_attention_prefill: too many workgroups for one launch");
  a.pack_slot = pack_slot_for(a.hq, a.hkv, max_chunk);
  a.q_tiles = a.pack_slot > 0 ? 1 : (max_chunk + BM - 1) / BM;
  hipError_t e;
  if (quant == FDATTN_CACHE_INT8) e = launch_v2<FDATTN_CACHE_INT8, false>(a, max_chunk, s);
  else if (quant == FDATTN_CACHE_FP8_E4M3) e = launch_v2<FDATTN_CACHE_FP8_E4M3, false>(a, max_chunk, s);
  else if (quant_bytes(quant) == FDATTN_CACHE_INT8)
    e = a.scale_rows == 1 ? launch_v2<FDATTN_CACHE_INT8, true, true>(a, max_chunk, s) : launch_v2<FDATTN_CACHE_INT8, true>(a, max_chunk, s);
  else
    e = a.scale_rows == 1 ? launch_v2<FDATTN_CACHE_FP8_E4M3, true, true>(a, max_chunk, s) : launch_v2<FDATTN_CACHE_FP8_E4M3, true>(a, max_chunk, s);
  if (e != hipSuccess) return fail((int)e, "fdattn_append_attention_prefill: %s", hipGetErrorString(e));
  int rc = check_launch("fdattn_append_attention_prefill (mfma)");
  if (rc || a.n_splits <= 1) return rc;
  a.tile_tokens = a.pack_slot > 0 ? a.pack_slot : BM;
  hipLaunchKernelGGL(prefill_v2_merge_kernel, dim3((unsigned)(((long long)a.num_tokens * a.hq + 3) / 4)), dim3(256), 0, s, a);
  return check_launch("fdattn_append_attention_prefill (merge)");
}

}  // namespace fdattn
