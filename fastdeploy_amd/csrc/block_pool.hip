// Host-side page pool: the component that produces block_tables.  A fixed pool of cache blocks
// with a free list and per-block reference counts; every sequence slot owns a row of the block
// table (logical block -> physical block, -1 padded) - the layout the kernels read.  Prefix
// sharing is by whole blocks: a forked sequence references the full blocks of its parent and
// appends into blocks of its own, so no copy-on-write is ever needed.  No device code here;
// the caller copies the table (or the rows that changed) to the GPU.  Not thread-safe: one
// scheduler thread owns a pool.
#include <stdlib.h>
#include <string.h>

#include <new>
#include <vector>

#include "fdattn_common.h"

struct fdattn_block_pool {
  int num_blocks, block_size, max_seqs, max_blocks_per_seq;
  std::vector<int32_t> table;     // [max_seqs][max_blocks_per_seq]
  std::vector<int32_t> seq_len;   // blocks held by each sequence slot
  std::vector<int32_t> refcount;  // per physical block
  std::vector<int32_t> free_list; // stack; the lowest block ids are handed out first
};

using fdattn::fail;

static bool bad_seq(const fdattn_block_pool* p, int seq) { return seq < 0 || seq >= p->max_seqs; }

extern "C" fdattn_block_pool* fdattn_pool_create(int num_blocks, int block_size, int max_seqs, int max_blocks_per_seq) {
  if (num_blocks <= 0 || block_size <= 0 || max_seqs <= 0 || max_blocks_per_seq <= 0) {
    fail(FDATTN_ERR_SHAPE, "fdattn_pool_create: bad shape num_blocks=%d block_size=%d max_seqs=%d max_blocks_per_seq=%d",
         num_blocks, block_size, max_seqs, max_blocks_per_seq);
    return nullptr;
  }
  fdattn_block_pool* p = new (std::nothrow) fdattn_block_pool;
  if (!p) {
    fail(FDATTN_ERR_POOL, "fdattn_pool_create: out of host memory");
    return nullptr;
  }
  p->num_blocks = num_blocks, p->block_size = block_size, p->max_seqs = max_seqs, p->max_blocks_per_seq = max_blocks_per_seq;
  p->table.assign((size_t)max_seqs * max_blocks_per_seq, -1);
  p->seq_len.assign(max_seqs, 0);
  p->refcount.assign(num_blocks, 0);
  p->free_list.resize(num_blocks);
  for (int i = 0; i < num_blocks; ++i) p->free_list[i] = num_blocks - 1 - i;  // pop_back() yields 0, 1, 2, ...
  return p;
}

extern "C" void fdattn_pool_destroy(fdattn_block_pool* p) { delete p; }

extern "C" int fdattn_pool_free_blocks(const fdattn_block_pool* p) { return p ? (int)p->free_list.size() : 0; }

extern "C" int fdattn_pool_seq_blocks(const fdattn_block_pool* p, int seq) {
  return (!p || bad_seq(p, seq)) ? 0 : p->seq_len[seq];
}

extern "C" int fdattn_pool_refcount(const fdattn_block_pool* p, int block) {
  return (!p || block < 0 || block >= p->num_blocks) ? 0 : p->refcount[block];
}

extern "C" const int32_t* fdattn_pool_block_tables(const fdattn_block_pool* p) { return p ? p->table.data() : nullptr; }

extern "C" int fdattn_pool_reserve(fdattn_block_pool* p, int seq, int num_tokens) {
  if (!p) return fail(FDATTN_ERR_NULL, "fdattn_pool_reserve: pool is NULL");
  if (bad_seq(p, seq) || num_tokens < 0)
    return fail(FDATTN_ERR_SHAPE, "fdattn_pool_reserve: bad sequence slot %d or token count %d", seq, num_tokens);
  const long long need = ((long long)num_tokens + p->block_size - 1) / p->block_size;
  if (need > p->max_blocks_per_seq)
    return fail(FDATTN_ERR_SHAPE, "fdattn_pool_reserve: %d tokens need %lld blocks, a table row holds %d", num_tokens,
                need, p->max_blocks_per_seq);
  const int have = p->seq_len[seq];
  const int grow = (int)need - have;
  if (grow <= 0) return 0;  // reservations only grow; fdattn_pool_release gives blocks back
  if ((size_t)grow > p->free_list.size())  // all or nothing: a failed call changes no state
    return fail(FDATTN_ERR_POOL, "fdattn_pool_reserve: %d blocks wanted, %zu free", grow, p->free_list.size());
  int32_t* row = p->table.data() + (size_t)seq * p->max_blocks_per_seq;
  for (int i = 0; i < grow; ++i) {
    const int32_t b = p->free_list.back();
    p->free_list.pop_back();
    p->refcount[b] = 1;
    row[have + i] = b;
  }
  p->seq_len[seq] = (int)need;
  return 0;
}

extern "C" int fdattn_pool_release(fdattn_block_pool* p, int seq) {
  if (!p) return fail(FDATTN_ERR_NULL, "fdattn_pool_release: pool is NULL");
  if (bad_seq(p, seq)) return fail(FDATTN_ERR_SHAPE, "fdattn_pool_release: bad sequence slot %d", seq);
  int32_t* row = p->table.data() + (size_t)seq * p->max_blocks_per_seq;
  for (int i = p->seq_len[seq] - 1; i >= 0; --i) {  // last block first: a released sequence's blocks come back in order
    const int32_t b = row[i];
    if (--p->refcount[b] == 0) p->free_list.push_back(b);
    row[i] = -1;
  }
  p->seq_len[seq] = 0;
  return 0;
}

extern "C" int fdattn_pool_fork(fdattn_block_pool* p, int src_seq, int dst_seq, int shared_tokens) {
  if (!p) return fail(FDATTN_ERR_NULL, "fdattn_pool_fork: pool is NULL");
  if (bad_seq(p, src_seq) || bad_seq(p, dst_seq) || src_seq == dst_seq || shared_tokens < 0)
    return fail(FDATTN_ERR_SHAPE, "fdattn_pool_fork: bad arguments src=%d dst=%d shared_tokens=%d", src_seq, dst_seq,
                shared_tokens);
  if (p->seq_len[dst_seq] != 0)
    return fail(FDATTN_ERR_SHAPE, "fdattn_pool_fork: destination slot %d is not empty", dst_seq);
  int full = shared_tokens / p->block_size;  // only whole blocks are shared
  if (full > p->seq_len[src_seq]) full = p->seq_len[src_seq];
  const int32_t* src = p->table.data() + (size_t)src_seq * p->max_blocks_per_seq;
  int32_t* dst = p->table.data() + (size_t)dst_seq * p->max_blocks_per_seq;
  for (int i = 0; i < full; ++i) {
    dst[i] = src[i];
    ++p->refcount[src[i]];
  }
  p->seq_len[dst_seq] = full;
  return full * p->block_size;  // tokens the destination now shares
}
