"""Host-side block pool (no GPU): free list, reference counts, table rows, error behaviour.
Checked against a dictionary model written here and against the invariants any allocator
has to keep: a block has exactly as many owners as its reference count says, a block with
no owner is free, free + owned = all, and a failed call changes nothing."""
import numpy as np
import pytest

from fastdeploy_amd.block_pool import BlockPool


def owners(pool):
    """block -> number of table rows that name it"""
    t = pool.block_tables
    ids, counts = np.unique(t[t >= 0], return_counts=True)
    return dict(zip(ids.tolist(), counts.tolist()))


def check_invariants(pool):
    own = owners(pool)
    for b in range(pool.num_blocks):
        assert pool.refcount(b) == own.get(b, 0)
    assert pool.free_blocks == pool.num_blocks - len(own)
    t = pool.block_tables
    for s in range(pool.max_seqs):
        n = pool.seq_blocks(s)
        assert (t[s, :n] >= 0).all() and (t[s, n:] == -1).all()
        assert len(set(t[s, :n].tolist())) == n          # no block twice in one sequence


def test_reserve_hands_out_blocks_in_order_and_pads_with_minus_one():
    p = BlockPool(num_blocks=10, block_size=64, max_seqs=3, max_blocks_per_seq=4)
    assert p.free_blocks == 10 and (p.block_tables == -1).all()
    p.reserve(0, 1)
    p.reserve(1, 64)
    p.reserve(2, 65)
    assert p.block_tables.tolist() == [[0, -1, -1, -1], [1, -1, -1, -1], [2, 3, -1, -1]]
    p.reserve(0, 129)                                      # grows by two blocks, keeps the first
    assert p.block_tables[0].tolist() == [0, 4, 5, -1]
    p.reserve(0, 10)                                       # never shrinks
    assert p.seq_blocks(0) == 3 and p.free_blocks == 4
    p.reserve(1, 0)
    assert p.seq_blocks(1) == 1
    check_invariants(p)


def test_exhaustion_is_all_or_nothing():
    p = BlockPool(num_blocks=5, block_size=16, max_seqs=2, max_blocks_per_seq=8)
    p.reserve(0, 48)                                       # 3 blocks
    before = p.block_tables.copy()
    with pytest.raises(ValueError, match="free"):
        p.reserve(1, 16 * 3)                               # wants 3, 2 free
    assert (p.block_tables == before).all() and p.free_blocks == 2 and p.seq_blocks(1) == 0
    with pytest.raises(ValueError, match="table row"):
        p.reserve(0, 16 * 8 + 1)                           # more than a row holds
    assert (p.block_tables == before).all()
    p.reserve(1, 32)                                       # exactly the rest
    assert p.free_blocks == 0
    check_invariants(p)


def test_release_returns_blocks_and_they_are_reused():
    p = BlockPool(num_blocks=6, block_size=64, max_seqs=3, max_blocks_per_seq=4)
    p.reserve(0, 128)
    p.reserve(1, 128)
    p.release(0)
    assert p.free_blocks == 4 and (p.block_tables[0] == -1).all() and p.seq_blocks(0) == 0
    p.reserve(2, 192)
    assert p.block_tables[2].tolist() == [0, 1, 4, -1]     # the released blocks first, lowest id first
    p.release(0)                                           # releasing an empty slot is a no-op
    check_invariants(p)


def test_fork_shares_whole_blocks_only():
    p = BlockPool(num_blocks=8, block_size=64, max_seqs=3, max_blocks_per_seq=4)
    p.reserve(0, 150)                                      # blocks 0 1 2, the last one partly filled
    assert p.fork(0, 1, 150) == 128                        # two whole blocks
    assert p.block_tables[1].tolist() == [0, 1, -1, -1]
    assert [p.refcount(b) for b in range(4)] == [2, 2, 1, 0]
    p.reserve(1, 150)                                      # the fork's own tail block
    assert p.block_tables[1].tolist() == [0, 1, 3, -1]
    assert p.fork(0, 2, 10_000) == 192                     # clipped to what the source holds
    assert [p.refcount(b) for b in range(4)] == [3, 3, 2, 1]
    check_invariants(p)
    p.release(0)
    assert p.free_blocks == 4                              # nothing came back: every block still has an owner
    p.release(2)
    assert p.free_blocks == 5 and p.refcount(2) == 0       # block 2 lost its last owner
    p.release(1)
    assert p.free_blocks == 8
    check_invariants(p)
    with pytest.raises(ValueError, match="not empty"):
        p.reserve(1, 1)
        p.fork(0, 1, 64)


def test_bad_arguments():
    with pytest.raises(ValueError):
        BlockPool(num_blocks=0)
    p = BlockPool(num_blocks=4, block_size=64, max_seqs=2, max_blocks_per_seq=2)
    for call in (lambda: p.reserve(2, 1), lambda: p.reserve(-1, 1), lambda: p.reserve(0, -1),
                 lambda: p.release(5), lambda: p.fork(0, 0, 64), lambda: p.fork(0, 9, 64)):
        with pytest.raises(ValueError):
            call()
    assert p.refcount(-1) == 0 and p.refcount(99) == 0 and p.seq_blocks(7) == 0
    p.close()
    with pytest.raises(ValueError, match="closed"):
        p.reserve(0, 1)


def test_random_workload_against_a_dictionary_model():
    rng = np.random.default_rng(5)
    N, BS, S, W = 96, 16, 12, 20
    p = BlockPool(num_blocks=N, block_size=BS, max_seqs=S, max_blocks_per_seq=W)
    model = {s: [] for s in range(S)}                      # slot -> block ids
    rc = [0] * N
    free = list(range(N - 1, -1, -1))
    for step in range(4000):
        op = rng.integers(0, 10)
        s = int(rng.integers(0, S))
        if op < 6:
            tokens = int(rng.integers(0, BS * W + 1))
            need = -(-tokens // BS) - len(model[s])
            if need > len(free):
                with pytest.raises(ValueError):
                    p.reserve(s, tokens)
            else:
                p.reserve(s, tokens)
                for _ in range(max(need, 0)):
                    b = free.pop()
                    rc[b] = 1
                    model[s].append(b)
        elif op < 8:
            p.release(s)
            for b in reversed(model[s]):
                rc[b] -= 1
                if rc[b] == 0:
                    free.append(b)
            model[s] = []
        else:
            d = int(rng.integers(0, S))
            tokens = int(rng.integers(0, BS * W + 1))
            if d == s or model[d]:
                with pytest.raises(ValueError):
                    p.fork(s, d, tokens)
            else:
                full = min(tokens // BS, len(model[s]))
                assert p.fork(s, d, tokens) == full * BS
                model[d] = model[s][:full]
                for b in model[d]:
                    rc[b] += 1
        if step % 97 == 0:
            check_invariants(p)
    t = p.block_tables
    for s in range(S):
        assert t[s, :len(model[s])].tolist() == model[s]
    assert p.free_blocks == len(free) and [p.refcount(b) for b in range(N)] == rc
    check_invariants(p)


def test_sequence_book_builds_the_step_description():
    """Host bookkeeping between steps: which slots are prefill rows, decode rows or idle, the lengths the
    kernels are given, blocks reserved before the step and lengths advanced after it."""
    from fastdeploy_amd.backend import SequenceBook
    pool = BlockPool(num_blocks=8, block_size=16, max_seqs=4, max_blocks_per_seq=4)
    book = SequenceBook(pool, device="cpu")
    m = book.schedule({0: 20, 2: 1})                       # a prompt, and a one-token prompt: both prefill rows
    assert m.seq_lens_encoder.tolist() == [20, 0, 1, 0] and m.seq_lens_decoder.tolist() == [0, 0, 0, 0]
    assert m.seq_lens_this_time.tolist() == [20, 0, 1, 0] and (m.num_tokens, m.max_enc_len_this_time) == (21, 20)
    assert m.block_tables.tolist() == [[0, 1, -1, -1], [-1] * 4, [2, -1, -1, -1], [-1] * 4]
    assert book.lengths == [0, 0, 0, 0]                    # nothing advances before commit
    book.commit()
    assert book.lengths == [20, 0, 1, 0]
    m = book.schedule({0: 1, 2: 1, 3: 0})                  # two decode rows; a zero count is an idle slot
    assert m.seq_lens_encoder.tolist() == [0, 0, 0, 0] and m.seq_lens_decoder.tolist() == [20, 0, 1, 0]
    assert m.seq_lens_this_time.tolist() == [1, 0, 1, 0] and m.max_enc_len_this_time == 0
    book.commit()
    m = book.schedule({0: 12})                             # a later chunk of several tokens: prefill row on a prefix
    assert m.seq_lens_encoder.tolist() == [12, 0, 0, 0] and m.seq_lens_decoder.tolist() == [21, 0, 2, 0]
    assert pool.seq_blocks(0) == 3                         # 33 tokens
    book.commit()
    assert book.fork(0, 1) == 32 and book.lengths[1] == 32 and pool.refcount(0) == 2
    with pytest.raises(ValueError):
        book.schedule({3: 16 * 4 + 1})                     # more than a table row holds
    with pytest.raises(ValueError):
        book.schedule({3: 16 * 4, 2: 60})                  # slot 3 takes the last four blocks, slot 2 finds none
    book.finish(3)
    book.finish(0)
    assert book.lengths[0] == 0 and pool.refcount(0) == 1 and pool.refcount(3) == 0 and pool.free_blocks == 5


def test_sequence_book_speculative_steps():
    """Draft slots: a slot named in `drafts` that already has tokens brings its tokens as a decode row of several
    tokens (seq_lens_encoder 0, decode_tokens = the largest such count); an empty slot named there is still a
    prompt.  commit(accepted) advances a slot by the tokens that were kept."""
    from fastdeploy_amd.backend import SequenceBook
    pool = BlockPool(num_blocks=8, block_size=16, max_seqs=4, max_blocks_per_seq=4)
    book = SequenceBook(pool, device="cpu")
    book.schedule({0: 20, 1: 3})
    book.commit()
    m = book.schedule({0: 3, 1: 2, 2: 2, 3: 1}, drafts={0, 1, 2})
    assert m.seq_lens_encoder.tolist() == [0, 0, 2, 1]      # slot 2 is empty: its two tokens are a prompt
    assert m.seq_lens_this_time.tolist() == [3, 2, 2, 1] and m.decode_tokens == 3
    assert (m.prefill_rows, m.max_enc_len_this_time, m.num_tokens) == (2, 2, 8)
    assert book.schedule({0: 1}).decode_tokens == 1         # (a schedule that is not committed changes no length)
    m = book.schedule({0: 3, 1: 2}, drafts={0, 1})
    book.commit(accepted={0: 1, 1: 2})
    assert book.lengths == [21, 5, 0, 0]
    book.schedule({0: 2}, drafts={0})
    with pytest.raises(ValueError):
        book.commit(accepted={0: 3})
