// KV pages of whole sequences to and from a contiguous, self-describing buffer ("wire" form): what
// a prefill instance hands to a decode instance, or a cache hands to host memory.  HBM-bound copies:
// a unit is one (page, K|V, head) tile of block_size * head_dim bytes, contiguous in the cache and in
// the wire buffer; one workgroup moves one unit with 16-byte accesses and sums its 32-bit words.
//
// Wire layout of one sequence (little-endian, every section 256-byte aligned):
//   header   256 B   u32 magic 'FDKV', version, cache_quant_type, hkv, head_dim, block_size,
//                    num_tokens, num_pages; u64 scales_off, sums_off, pages_off, total_bytes
//   scales           f32 K [hkv, head_dim], f32 V [hkv, head_dim];
//                    dynamic formats: f32 [num_pages][2][hkv][block_size], the stored rows' scales (0 past num_tokens)
//   sums             u64 [num_pages][2][hkv]: sum of the unit's 32-bit words (dynamic: its scale row included)
//   pages            [num_pages][2][hkv][block_size][head_dim] bytes; rows past num_tokens are zero
#include "fdattn_common.h"

namespace fdattn {
namespace {

constexpr u32 kMagic = 0x564b4446u;  // "FDKV"
constexpr u32 kVersion = 1;
constexpr int kHeaderBytes = 256;

__host__ __device__ inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

struct WireLayout {
  size_t scales_off, sums_off, pages_off, total;
  int pages;
};
__host__ __device__ inline size_t scale_bytes(int pages, int hkv, int d, int bs, bool dyn) {
  return (dyn ? (size_t)pages * 2 * hkv * bs : (size_t)2 * hkv * d) * sizeof(float);
}
__host__ __device__ inline WireLayout wire_layout(int num_tokens, int hkv, int d, int bs, bool dyn) {
  WireLayout w;
  w.pages = (num_tokens + bs - 1) / bs;
  w.scales_off = kHeaderBytes;
  w.sums_off = align256(w.scales_off + scale_bytes(w.pages, hkv, d, bs, dyn));
  w.pages_off = align256(w.sums_off + (size_t)w.pages * 2 * hkv * sizeof(unsigned long long));
  w.total = align256(w.pages_off + (size_t)w.pages * 2 * hkv * bs * d);
  return w;
}

struct WireArgs {
  uint8_t* key_cache;
  uint8_t* value_cache;
  const float* k_scale;  // dynamic formats: the scale caches [num_blocks, hkv, bs], written by the import
  const float* v_scale;
  const int32_t* block_tables;  // [batch, max_blocks]
  const int32_t* num_tokens;    // [batch]
  const int64_t* wire_offsets;  // [batch] byte offset of each sequence's buffer inside wire
  uint8_t* wire;
  int32_t* status;  // import: [0] error bits, [1] units whose sum disagrees
  int hkv, d, bs, max_blocks, num_blocks, quant, max_tokens;
};

// sum over the workgroup (256 threads); the result is valid in thread 0
__device__ __forceinline__ unsigned long long block_sum(unsigned long long v, unsigned long long* sh) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_down(v, o, 64);
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
  __syncthreads();
  return sh[0] + sh[1] + sh[2] + sh[3];
}

__device__ __forceinline__ unsigned long long words_of(const uint4& w) {
  return (unsigned long long)w.x + w.y + w.z + w.w;
}

// header word i (0..63) of a sequence with this layout
__device__ __forceinline__ u32 header_word(int i, const WireArgs& a, int tokens, const WireLayout& w) {
  const unsigned long long off[4] = {w.scales_off, w.sums_off, w.pages_off, w.total};
  switch (i) {
    case 0: return kMagic;
    case 1: return kVersion;
    case 2: return (u32)a.quant;
    case 3: return (u32)a.hkv;
    case 4: return (u32)a.d;
    case 5: return (u32)a.bs;
    case 6: return (u32)tokens;
    case 7: return (u32)w.pages;
    default: break;
  }
  if (i < 16) return (u32)(off[(i - 8) >> 1] >> (32 * (i & 1)));
  return 0u;
}

// grid (pages * 2 * hkv, batch); IMPORT = false: cache -> wire, true: wire -> cache
template <bool IMPORT>
__global__ __launch_bounds__(256) void kv_wire_kernel(WireArgs a) {
  __shared__ unsigned long long sh[4];
  const int b = blockIdx.y;
  const int tokens = min(max(a.num_tokens[b], 0), a.max_tokens);
  const bool dyn = quant_dynamic(a.quant);
  const WireLayout w = wire_layout(tokens, a.hkv, a.d, a.bs, dyn);
  const int unit = blockIdx.x;
  uint8_t* wire = a.wire + a.wire_offsets[b];
  u32* hdr = reinterpret_cast<u32*>(wire);
  bool hdr_ok = true;
  if (IMPORT) {
    // Every workgroup checks the header against the layout the arguments imply before it writes into
    // the cache (16 words, the same for all threads); nothing read from the buffer is used as an offset.
    u32 magic_bad = 0, shape_bad = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const u32 diff = hdr[i] ^ header_word(i, a, tokens, w);
      if (i < 2) magic_bad |= diff; else shape_bad |= diff;
    }
    hdr_ok = (magic_bad | shape_bad) == 0;
    if (unit == 0 && threadIdx.x == 0 && !hdr_ok) atomicOr(a.status, (magic_bad ? 1 : 0) | (shape_bad ? 2 : 0));
  }
  if (unit == 0) {
    // header and scales travel with unit 0 (a sequence of zero tokens still has both)
    const int ns = a.hkv * a.d;
    if (!IMPORT) {
      if (threadIdx.x < 64) hdr[threadIdx.x] = header_word(threadIdx.x, a, tokens, w);
      float* sc = reinterpret_cast<float*>(wire + w.scales_off);
      if (!dyn)  // (the dynamic formats' scale rows travel with their units)
        for (int i = threadIdx.x; i < ns; i += 256) sc[i] = a.k_scale[i], sc[ns + i] = a.v_scale[i];
      // the alignment gaps behind the three sections (each under 256 bytes) are zero: the buffer's
      // bytes are a function of the sequence alone
      const size_t gap[3][2] = {{w.scales_off + scale_bytes(w.pages, a.hkv, a.d, a.bs, dyn), w.sums_off},
                                {w.sums_off + (size_t)w.pages * 2 * a.hkv * sizeof(unsigned long long), w.pages_off},
                                {w.pages_off + (size_t)w.pages * 2 * a.hkv * a.bs * a.d, w.total}};
#pragma unroll
      for (int g = 0; g < 3; ++g)
        if (gap[g][0] + threadIdx.x < gap[g][1]) wire[gap[g][0] + threadIdx.x] = 0;
    } else if (a.k_scale && hdr_ok && !dyn) {
      const float* sc = reinterpret_cast<const float*>(wire + w.scales_off);
      bool bad = false;
      for (int i = threadIdx.x; i < ns; i += 256)
        bad |= __float_as_uint(sc[i]) != __float_as_uint(a.k_scale[i]) ||
               __float_as_uint(sc[ns + i]) != __float_as_uint(a.v_scale[i]);
      if (bad) atomicOr(a.status, 4);
    }
  }
  if (!hdr_ok) return;  // uniform over the workgroup
  if (unit >= w.pages * 2 * a.hkv) return;  // uniform over the workgroup
  const int page = unit / (2 * a.hkv), kv = (unit / a.hkv) & 1, h = unit % a.hkv;
  const int valid = min(a.bs, tokens - page * a.bs);  // rows of this page that hold tokens
  const size_t unit_bytes = (size_t)a.bs * a.d;
  int pb = a.block_tables[(size_t)b * a.max_blocks + page];
  const bool pb_ok = pb >= 0 && pb < a.num_blocks;
  pb = pb_ok ? pb : 0;
  uint8_t* cache = (kv ? a.value_cache : a.key_cache) + ((size_t)pb * a.hkv + h) * unit_bytes;
  uint8_t* wu = wire + w.pages_off + (size_t)unit * unit_bytes;
  unsigned long long* sums = reinterpret_cast<unsigned long long*>(wire + w.sums_off);
  unsigned long long s = 0;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
  for (size_t off = (size_t)threadIdx.x * 16; off < unit_bytes; off += 256 * 16) {
    const bool live = (int)(off / a.d) < valid;
    if (!IMPORT) {
      const uint4 v = (live && pb_ok) ? *reinterpret_cast<const uint4*>(cache + off) : zero;
      *reinterpret_cast<uint4*>(wu + off) = v;
      s += words_of(v);
    } else {
      const uint4 v = *reinterpret_cast<const uint4*>(wu + off);
      s += words_of(v);
      if (pb_ok) *reinterpret_cast<uint4*>(cache + off) = v;
    }
  }
  if (dyn && (int)threadIdx.x < a.bs) {
    // the unit's scale row: bs floats beside the tile, zero for the rows past the sequence's end
    float* crow = const_cast<float*>(kv ? a.v_scale : a.k_scale) + ((size_t)pb * a.hkv + h) * a.bs;
    u32* wrow = reinterpret_cast<u32*>(wire + w.scales_off) + (size_t)unit * a.bs;
    const int t = threadIdx.x;
    if (!IMPORT) {
      const u32 v = (t < valid && pb_ok) ? __float_as_uint(crow[t]) : 0u;
      wrow[t] = v;
      s += v;
    } else {
      const u32 v = wrow[t];
      s += v;
      if (pb_ok) crow[t] = __uint_as_float(v);
    }
  }
  s = block_sum(s, sh);
  if (threadIdx.x == 0) {
    if (!IMPORT) {
      sums[unit] = s;
    } else {
      if (sums[unit] != s) {
        atomicOr(a.status, 8);
        atomicAdd(a.status + 1, 1);
      }
      if (!pb_ok) atomicOr(a.status, 16);
    }
  }
}

int check_shape(const char* what, int batch, int max_tokens, int hkv, int d, int bs, int max_blocks, int num_blocks,
                int quant) {
  if (!quant_known(quant)) return fail(FDATTN_ERR_QUANT, "%s: unknown cache_quant_type %d", what, quant);
  if (quant_dynamic(quant) && bs > 256)
    return fail(FDATTN_ERR_SHAPE, "%s: the dynamic formats' scale rows need block_size <= 256, got %d", what, bs);
  if (batch < 0 || max_tokens < 0 || hkv <= 0 || d <= 0 || bs <= 0 || max_blocks <= 0 || num_blocks <= 0 || d % 16 != 0 ||
      batch > 65535)
    return fail(FDATTN_ERR_SHAPE, "%s: bad shape batch=%d max_tokens=%d hkv=%d head_dim=%d block_size=%d "
                "max_blocks_per_seq=%d num_blocks=%d (head_dim must be a multiple of 16)",
                what, batch, max_tokens, hkv, d, bs, max_blocks, num_blocks);
  if (((long long)max_tokens + bs - 1) / bs > max_blocks)
    return fail(FDATTN_ERR_SHAPE, "%s: %d tokens need more than the %d blocks of a table row", what, max_tokens,
                max_blocks);
  return 0;
}

}  // namespace
}  // namespace fdattn

using namespace fdattn;

extern "C" size_t fdattn_kv_wire_bytes_for(int num_tokens, int hkv, int head_dim, int block_size, int cache_quant_type) {
  if (num_tokens < 0 || hkv <= 0 || head_dim <= 0 || block_size <= 0 || !quant_known(cache_quant_type)) return 0;
  return wire_layout(num_tokens, hkv, head_dim, block_size, quant_dynamic(cache_quant_type)).total;
}

extern "C" size_t fdattn_kv_wire_bytes(int num_tokens, int hkv, int head_dim, int block_size) {
  return fdattn_kv_wire_bytes_for(num_tokens, hkv, head_dim, block_size, FDATTN_CACHE_INT8);
}

extern "C" int fdattn_kv_export(const void* key_cache, const void* value_cache, const float* k_scale,
                                const float* v_scale, const int32_t* block_tables, const int32_t* num_tokens,
                                const int64_t* wire_offsets, void* wire, int batch, int max_tokens, int hkv,
                                int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
                                int cache_quant_type, void* stream) {
  if (!key_cache || !value_cache || !k_scale || !v_scale || !block_tables || !num_tokens || !wire_offsets || !wire)
    return fail(FDATTN_ERR_NULL, "fdattn_kv_export: NULL pointer argument");
  if (int rc = check_shape("fdattn_kv_export", batch, max_tokens, hkv, head_dim, block_size, max_blocks_per_seq,
                           num_blocks, cache_quant_type))
    return rc;
  if (batch == 0) return 0;
  WireArgs a{(uint8_t*)key_cache, (uint8_t*)value_cache, k_scale, v_scale, block_tables, num_tokens, wire_offsets,
             (uint8_t*)wire, nullptr, hkv, head_dim, block_size, max_blocks_per_seq, num_blocks, cache_quant_type, max_tokens};
  const int pages = (max_tokens + block_size - 1) / block_size;
  const dim3 grid(pages * 2 * hkv > 0 ? pages * 2 * hkv : 1, batch);
  hipLaunchKernelGGL(kv_wire_kernel<false>, grid, dim3(256), 0, (hipStream_t)stream, a);
  return check_launch("fdattn_kv_export");
}

extern "C" int fdattn_kv_import(const void* wire, const int64_t* wire_offsets, void* key_cache, void* value_cache,
                                const float* k_scale, const float* v_scale, const int32_t* block_tables,
                                const int32_t* num_tokens, int32_t* status, int batch, int max_tokens, int hkv,
                                int head_dim, int block_size, int max_blocks_per_seq, int num_blocks,
                                int cache_quant_type, void* stream) {
  if (!key_cache || !value_cache || !block_tables || !num_tokens || !wire_offsets || !wire || !status)
    return fail(FDATTN_ERR_NULL, "fdattn_kv_import: NULL pointer argument");
  if ((k_scale == nullptr) != (v_scale == nullptr))
    return fail(FDATTN_ERR_NULL, "fdattn_kv_import: pass both scale tables or neither");
  if (quant_dynamic(cache_quant_type) && !k_scale)
    return fail(FDATTN_ERR_NULL, "fdattn_kv_import: the dynamic formats need the scale caches to import into");
  if (int rc = check_shape("fdattn_kv_import", batch, max_tokens, hkv, head_dim, block_size, max_blocks_per_seq,
                           num_blocks, cache_quant_type))
    return rc;
  if (batch == 0) return 0;
  WireArgs a{(uint8_t*)key_cache, (uint8_t*)value_cache, k_scale, v_scale, block_tables, num_tokens, wire_offsets,
             (uint8_t*)wire, status, hkv, head_dim, block_size, max_blocks_per_seq, num_blocks, cache_quant_type, max_tokens};
  const int pages = (max_tokens + block_size - 1) / block_size;
  const dim3 grid(pages * 2 * hkv > 0 ? pages * 2 * hkv : 1, batch);
  hipLaunchKernelGGL(kv_wire_kernel<true>, grid, dim3(256), 0, (hipStream_t)stream, a);
  return check_launch("fdattn_kv_import");
}
