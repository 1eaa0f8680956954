"""Block pool: the producer of ``block_tables`` (host side, C++ inside libfdattn.so).

A fixed number of cache blocks, a free list, per-block reference counts and one table row per
sequence slot.  The table is the int32 ``[max_seqs, max_blocks_per_seq]`` array (-1 = no block)
that every kernel of this package takes as ``block_tables``.  Handle ownership follows the
reference's C API (c_api/fastdeploy_capi/core/fd_type.h:104-155: create / destroy pairs).
"""
import ctypes

import numpy as np

from . import _lib


class BlockPool:
    def __init__(self, num_blocks, block_size=64, max_seqs=64, max_blocks_per_seq=64):
        self._h = _lib.lib().fdattn_pool_create(num_blocks, block_size, max_seqs, max_blocks_per_seq)
        if not self._h:
            raise ValueError("fdattn_pool_create failed: " + _lib.lib().fdattn_last_error().decode())
        self.num_blocks, self.block_size = num_blocks, block_size
        self.max_seqs, self.max_blocks_per_seq = max_seqs, max_blocks_per_seq
        ptr = _lib.lib().fdattn_pool_block_tables(self._h)
        # a live, read-only view of the pool's own table
        self._table = np.ctypeslib.as_array(ptr, shape=(max_seqs, max_blocks_per_seq))
        self._table.flags.writeable = False

    def close(self):
        if self._h:
            self._table = None
            _lib.lib().fdattn_pool_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _handle(self):
        if not self._h:
            raise ValueError("the pool is closed")
        return self._h

    def reserve(self, seq, num_tokens):
        """Slot ``seq`` covers ``num_tokens`` tokens afterwards; all or nothing (ValueError)."""
        _lib.check(_lib.lib().fdattn_pool_reserve(self._handle(), seq, num_tokens), "fdattn_pool_reserve")

    def release(self, seq):
        _lib.check(_lib.lib().fdattn_pool_release(self._handle(), seq), "fdattn_pool_release")

    def fork(self, src_seq, dst_seq, shared_tokens):
        """Empty slot ``dst_seq`` shares the whole blocks of the first ``shared_tokens`` tokens of
        ``src_seq``; returns how many tokens are shared (a multiple of the block size)."""
        rc = _lib.lib().fdattn_pool_fork(self._handle(), src_seq, dst_seq, shared_tokens)
        if rc < 0:
            _lib.check(rc, "fdattn_pool_fork")
        return rc

    @property
    def free_blocks(self):
        return _lib.lib().fdattn_pool_free_blocks(self._handle())

    def seq_blocks(self, seq):
        return _lib.lib().fdattn_pool_seq_blocks(self._handle(), seq)

    def refcount(self, block):
        return _lib.lib().fdattn_pool_refcount(self._handle(), block)

    @property
    def block_tables(self):
        """A copy of the table as it is now (numpy int32 [max_seqs, max_blocks_per_seq], -1 = no block)."""
        self._handle()
        return np.array(self._table)

    def block_tables_view(self):
        """The pool's own table, read-only and live: it changes with reserve / release / fork and must not
        be touched after close()."""
        self._handle()
        return self._table

    def block_tables_tensor(self, device="cuda", rows=None):
        """A device copy of the table (or of its first ``rows`` slots) for the kernels."""
        import torch
        t = np.array(self._table if rows is None else self._table[:rows])
        return torch.from_numpy(t).to(device)
