"""Host side of the paged cache: the C++ core (through the C ABI) against hand-computed
cases from blocks.rs / batch_info.rs and against the Python restatement, exactly."""
import numpy as np
import pytest

from aici_amd import paged
from aici_amd._lib import HipAttnError
from oracle import hostkv as ref


def test_allocation_order_and_slots_hand_case():
    a = paged.BlockAllocator(16, 8)
    assert a.get_num_free_blocks() == 8
    a.alloc_seq(1, 40)  # 3 blocks: 0, 1, 2 (free list (0..n).rev() popped from the back)
    a.alloc_seq(2, 16)  # 1 block: 3
    assert a.num_allocated_blocks(1) == 3 and a.num_allocated_blocks(2) == 1
    s1 = a.get_block_idxes(1, 40)
    assert s1[0] == 0 and s1[15] == 15 and s1[16] == 16 and s1[39] == 2 * 16 + 7
    assert list(a.get_block_idxes(2, 16)) == list(range(48, 64))
    a.delete(1)  # frees 0,1,2 in that order -> pushed back; next pop is 2
    assert a.get_num_free_blocks() == 7
    a.alloc_seq(3, 1)
    assert a.get_block_idxes(3, 1)[0] == 2 * 16


def test_fork_copy_on_write_and_trim_hand_case():
    a = paged.BlockAllocator(4, 10)
    a.alloc_seq(1, 6)       # blocks 0,1
    a.copy(1, 2, 6)         # fork: seq 2 shares blocks 0,1
    assert a.get_num_free_blocks() == 8
    # seq 2 appends token 7 (position 6 lives in shared block 1) -> COW copy of block 1
    pairs = a.append_slots(2, 6, 7)
    assert pairs == [(1, 2)]
    assert list(a.get_block_idxes(2, 7)) == [0, 1, 2, 3, 8, 9, 10]
    # seq 1 now owns block 1 alone -> no copy when it grows, new block when crossing a boundary
    assert a.append_slots(1, 6, 9) == []
    assert list(a.get_block_idxes(1, 9))[-1] == 3 * 4
    a.trim(1, 4)            # keep one block
    assert a.num_allocated_blocks(1) == 1
    a.delete(1)
    a.delete(2)
    assert a.get_num_free_blocks() == 10


def test_exhaustion_is_an_error_and_leaves_state_unchanged():
    a = paged.BlockAllocator(16, 2)
    with pytest.raises(HipAttnError, match="Out of memory! No free blocks"):
        a.alloc_seq(1, 33)
    assert a.get_num_free_blocks() == 2 and a.num_allocated_blocks(1) == 0
    a.alloc_seq(1, 32)
    with pytest.raises(HipAttnError, match="Out of memory"):
        a.append_slots(1, 32, 33)
    assert a.num_allocated_blocks(1) == 2
    with pytest.raises(HipAttnError, match="unknown sequence"):
        a.get_block_idxes(99, 1)


def test_admission_policy_hand_case():
    """blocks.rs:260-283, 321-343: 1 % of 250 blocks = 2.5 -> 2 blocks held back from new sequences."""
    for A in (paged.BlockAllocator, ref.BlockAllocator):
        a = A(16, 250)
        assert a.can_allocate(250 * 16) and not a.can_allocate(250 * 16 + 1)
        a.set_watermark(0.01)
        assert a.can_allocate(248 * 16) and not a.can_allocate(248 * 16 + 1)
        a.alloc_seq(1, 240 * 16)                      # 10 blocks left, 2 of them held back
        assert a.can_allocate(8 * 16) and not a.can_allocate(8 * 16 + 1)
        assert a.can_allocate(0)
        assert a.can_append_slot(10) and not a.can_append_slot(11)   # appends ignore the watermark
        a.set_watermark(0.0)
        assert a.can_allocate(10 * 16)


@pytest.mark.parametrize("seed", range(5))
def test_allocator_random_walk_matches_restatement(seed):
    rng = np.random.default_rng(seed)
    bs, nb = int(rng.choice([4, 16])), 64
    a, r = paged.BlockAllocator(bs, nb), ref.BlockAllocator(bs, nb)
    lens = {}
    next_id = 1
    for _ in range(200):
        op = rng.integers(0, 5)
        if op == 0 or not lens:
            n = int(rng.integers(1, 5 * bs))
            if r.get_num_free_blocks() < r.num_blocks(n):
                continue
            a.alloc_seq(next_id, n)
            r.alloc_seq(next_id, n)
            lens[next_id] = n
            next_id += 1
        elif op == 1:
            s = int(rng.choice(list(lens)))
            grow = int(rng.integers(1, 2 * bs))
            if r.get_num_free_blocks() < r.num_blocks(lens[s] + grow) + 2:
                continue
            computed = int(rng.integers(max(0, lens[s] - bs), lens[s] + 1))
            assert a.append_slots(s, computed, lens[s] + grow) == r.append_slots(s, computed, lens[s] + grow)
            lens[s] += grow
        elif op == 2:
            s = int(rng.choice(list(lens)))
            n = int(rng.integers(1, lens[s] + 1))
            a.copy(s, next_id, n)
            r.copy(s, next_id, n)
            lens[next_id] = min(n, lens[s])
            # a fork holds ceil(n/bs) blocks, so it can address up to that many tokens
            lens[next_id] = min(r.num_allocated_blocks(next_id) * bs, lens[s])
            next_id += 1
        elif op == 3:
            s = int(rng.choice(list(lens)))
            n = int(rng.integers(0, lens[s] + 1))
            a.trim(s, n)
            r.trim(s, n)
            if n == 0:
                del lens[s]
            else:
                lens[s] = min(lens[s], r.num_allocated_blocks(s) * bs)
        else:
            s = int(rng.choice(list(lens)))
            a.delete(s)
            r.delete(s)
            del lens[s]
        assert a.get_num_free_blocks() == r.get_num_free_blocks()
        for s, n in lens.items():
            assert a.num_allocated_blocks(s) == r.num_allocated_blocks(s)
            assert list(a.get_block_idxes(s, n)) == r.get_block_idxes(s, n)


def _as_dict(bi: paged.BatchInfo) -> dict:
    return dict(tokens=bi.tokens.tolist(), positions=bi.positions.tolist(), slot_mapping=bi.slot_mapping.tolist(),
                logit_idxs=bi.logit_idxs.tolist(), seq_ids=bi.seq_ids, seqlens_q=bi.seqlens_q.tolist(),
                seqlens_k=bi.seqlens_k.tolist(), max_seqlen_q=bi.max_seqlen_q, max_seqlen_k=bi.max_seqlen_k,
                gather_mapping=bi.gather_mapping.tolist(), seqlen_multi=bi.seqlen_multi, q_multi=bi.q_multi,
                paged_block_tables=bi.paged_block_tables.flatten().tolist(),
                paged_max_blocks=bi.paged_block_tables.shape[1], paged_context_lens=bi.paged_context_lens.tolist(),
                paged_block_size=bi.paged_block_size, paged_max_context_len=bi.paged_max_context_len)


def test_batch_builder_hand_case_multi_first_ordering():
    bs = 4
    a = paged.BlockAllocator(bs, 16)
    a.alloc_seq(10, 5)   # decode row: blocks 0,1 ; context 5
    a.alloc_seq(11, 6)   # prompt of 6: blocks 2,3
    a.alloc_seq(12, 9)   # decode row: blocks 4,5,6 ; context 9
    b = paged.BatchInfoBuilder(bs, 128, paged_attn_kernel_v=1)
    b.sched_out(a, 10, [100, 101, 102, 103, 104], 4)
    b.sched_out(a, 11, [200, 201, 202, 203, 204, 205], 0)
    b.sched_out(a, 12, list(range(300, 309)), 9)  # nothing new: recompute the last token
    bi = b.finish()
    assert bi.seq_ids == [11, 10, 12]                      # multi-token entry first, singles keep order
    assert bi.tokens.tolist() == [200, 201, 202, 203, 204, 205, 104, 308]
    assert bi.positions.tolist() == [0, 1, 2, 3, 4, 5, 4, 8]
    assert bi.slot_mapping.tolist() == [8, 9, 10, 11, 12, 13, 4, 24]
    assert bi.logit_idxs.tolist() == [5, 6, 7]
    assert bi.seqlens_q.tolist() == [0, 6] and bi.seqlens_k.tolist() == [0, 6]
    assert bi.gather_mapping.tolist() == [8, 9, 10, 11, 12, 13]
    assert bi.q_multi == 6 and bi.seqlen_multi == 1
    assert bi.paged_context_lens.tolist() == [5, 9] and bi.paged_max_context_len == 9
    assert bi.paged_block_tables.tolist() == [[0, 1, 0], [4, 5, 6]]   # zero padded
    # CPU-build behaviour: everything on the varlen path, original order
    b0 = paged.BatchInfoBuilder(bs, 128, paged_attn_kernel_v=0)
    b0.sched_out(a, 10, [100, 101, 102, 103, 104], 4)
    b0.sched_out(a, 11, [200, 201, 202, 203, 204, 205], 0)
    bi0 = b0.finish()
    assert bi0.seq_ids == [10, 11] and bi0.seqlen_multi == 2 and bi0.q_multi == 7
    assert bi0.seqlens_q.tolist() == [0, 1, 7] and bi0.seqlens_k.tolist() == [0, 5, 11]
    assert bi0.paged_block_tables.numel() == 0


@pytest.mark.parametrize("seed", range(4))
@pytest.mark.parametrize("paged_v", [0, 1])
def test_batch_builder_matches_restatement(seed, paged_v):
    rng = np.random.default_rng(100 + seed)
    bs = 16
    a, r = paged.BlockAllocator(bs, 256), ref.BlockAllocator(bs, 256)
    b = paged.BatchInfoBuilder(bs, 4096, paged_v)
    entries = []
    for sid in range(1, 12):
        n = int(rng.integers(1, 200))
        toks = rng.integers(0, 32000, size=n).tolist()
        a.alloc_seq(sid, n)
        r.alloc_seq(sid, n)
        computed = int(rng.choice([0, n, n - 1, max(0, n - 5)]))
        b.sched_out(a, sid, toks, computed)
        entries.append(ref.sched_entry(r, sid, toks, computed))
    got = _as_dict(b.finish())
    want = ref.build_batch(entries, bs, 4096, paged_v)
    assert got == want


def test_builder_errors():
    b = paged.BatchInfoBuilder(16, 8, 1)
    with pytest.raises(HipAttnError, match="no entries"):
        b.finish()
    b.add_entry(1, [9], [5], list(range(10)))
    with pytest.raises(HipAttnError, match="max_model_len"):
        b.finish()
    b2 = paged.BatchInfoBuilder(16, 100, 1)
    b2.add_entry(1, [2], [5], [3, 4, 5])  # first slot of the context is not block-aligned
    with pytest.raises(HipAttnError, match="not block-aligned"):
        b2.finish()


def test_cache_geometry():
    import torch
    assert paged.cache_x(torch.float16) == 8 and paged.cache_x(torch.bfloat16) == 8 and paged.cache_x(torch.float32) == 4
    assert paged.cache_block_bytes(16, 8, 128, 32, torch.bfloat16) == ref.cache_block_bytes(16, 8, 128, 32, 2) == 2 * 16 * 8 * 128 * 2 * 32


def test_multi_entry_block_tables_extension():
    """The builder also hands out block tables for multi-token entries when their slots walk the blocks in
    order (blocks.rs:122-127 slots always do); hand-made slots that do not are flagged."""
    a = paged.BlockAllocator(16, 32)
    b = paged.BatchInfoBuilder(16, 4096, 1)
    a.alloc_seq(1, 40)
    a.alloc_seq(2, 7)
    a.alloc_seq(3, 20)
    b.sched_out(a, 2, list(range(7)), 6)          # single token -> paged rows
    b.sched_out(a, 1, list(range(40)), 10)        # 30 new tokens
    b.sched_out(a, 3, list(range(20)), 0)         # prompt
    bi = b.finish()
    assert bi.seq_ids == [1, 3, 2] and bi.seqlen_multi == 2
    assert bi.multi_context_lens.tolist() == [40, 20]
    assert bi.multi_block_tables.tolist() == [[0, 1, 2], [4, 5, 0]]       # seq 2 took block 3
    # every gathered slot is reproduced by the table
    gm = bi.gather_mapping.tolist()
    want = [bi.multi_block_tables[0, p // 16].item() * 16 + p % 16 for p in range(40)] + \
           [bi.multi_block_tables[1, p // 16].item() * 16 + p % 16 for p in range(20)]
    assert gm == want
    b2 = paged.BatchInfoBuilder(16, 4096, 1)
    b2.add_entry(9, [0, 1, 2], [5, 6, 7], [32, 34, 33])                    # slots out of order
    assert b2.finish().multi_block_tables is None


def test_swap_out_and_in_hand_case_with_shared_blocks():
    """blocks.rs:176-210: swap_out hands over a sequence's blocks and releases them; swap_in on the
    other side allocates one block per distinct source block -- a block that two sequences of a group
    share (a fork) is allocated once and forked for the second."""
    for A in (paged.BlockAllocator, ref.BlockAllocator):
        gpu, cpu = A(16, 8), A(16, 6)
        gpu.alloc_seq(1, 40)                     # blocks 0, 1, 2
        gpu.copy(1, 2, 32)                       # seq 2 shares blocks 0, 1
        assert gpu.get_num_free_blocks() == 5
        mapping = {}
        b1 = gpu.swap_out(1)
        assert list(b1) == [0, 1, 2] and gpu.num_allocated_blocks(1) == 0
        assert gpu.get_num_free_blocks() == 6    # 0 and 1 are still held by seq 2
        cpu.swap_in(1, b1, mapping)
        assert mapping == {0: 0, 1: 1, 2: 2}
        b2 = gpu.swap_out(2)
        assert list(b2) == [0, 1] and gpu.get_num_free_blocks() == 8
        cpu.swap_in(2, b2, mapping)              # both blocks already mapped: forked, nothing allocated
        assert mapping == {0: 0, 1: 1, 2: 2} and cpu.get_num_free_blocks() == 3
        assert list(cpu.get_block_idxes(2, 32)) == list(range(32))
        cpu.delete(1)
        assert cpu.get_num_free_blocks() == 4    # block 2 came back; 0 and 1 are still seq 2's
        assert list(gpu.swap_out(7)) == []       # unknown sequence: nothing to hand over
        gpu.swap_in(7, [], {})
        assert gpu.num_allocated_blocks(7) == 0


def test_block_space_manager_admission_and_swaps():
    """blocks.rs:259-380 on 1 % of 300 = 3 watermark blocks."""
    m = paged.BlockSpaceManager(16, 300, 10, watermark=0.01)
    assert m.watermark_blocks == 3
    assert m.can_allocate(297 * 16) and not m.can_allocate(297 * 16 + 1)
    m.allocate(1, 5 * 16)
    m.allocate(2, 3 * 16 + 1)
    m.copy(2, 3, 3 * 16 + 1)                     # seq 3 forks seq 2's four blocks
    assert m.get_num_free_gpu_blocks() == 291 and m.num_phys_blocks([1, 2, 3]) == 13
    assert m.can_swap_out([2, 3]) and not m.can_swap_out([1, 2, 3])      # 8 <= 10 < 13
    to_host = m.swap_out([2, 3])
    assert to_host == {5: 0, 6: 1, 7: 2, 8: 3}                           # shared blocks travel once
    assert m.get_num_free_gpu_blocks() == 295 and m.get_num_free_cpu_blocks() == 6
    assert m.num_phys_blocks([2, 3]) == 8                                # now counted on the host side
    assert m.can_swap_in([2, 3])                                         # 8 + 2 + 3 <= 295
    to_dev = m.swap_in([2, 3])
    # the free list is a stack: the blocks that came back last go out first
    assert sorted(to_dev) == [0, 1, 2, 3] and len(set(to_dev.values())) == 4
    assert m.get_num_free_cpu_blocks() == 10 and m.get_num_free_gpu_blocks() == 291
    assert list(m.gpu_allocator.get_block_idxes(2, 49)) == list(m.gpu_allocator.get_block_idxes(3, 49))
    assert m.can_append_slot(291) and not m.can_append_slot(292)
    pairs = m.append_slots(3, 49, 50)            # seq 3 writes into the shared last block: copy-on-write
    assert len(pairs) == 1 and pairs[0][0] == to_dev[3]
    m.delete(2)
    m.delete(3)
    m.trim(1, 16)
    assert m.get_num_free_gpu_blocks() == 299


def test_swap_in_that_cannot_finish_changes_nothing():
    a = paged.BlockAllocator(16, 4)
    a.alloc_seq(1, 32)                      # two blocks taken, two free
    mapping = {7: 0}
    with pytest.raises(HipAttnError, match="needs 3 free blocks, 2 are available"):
        a.swap_in(2, [7, 8, 9, 10, 8], mapping)   # 7 is mapped, 8 / 9 / 10 need fresh blocks
    assert a.get_num_free_blocks() == 2 and a.num_allocated_blocks(2) == 0 and mapping == {7: 0}
    a.swap_in(2, [7, 8, 9, 8], mapping)     # fits: two fresh blocks, block 8 taken once
    assert a.get_num_free_blocks() == 0 and a.num_allocated_blocks(2) == 4
    assert mapping[8] != mapping[9] and set(mapping) == {7, 8, 9}


@pytest.mark.parametrize("seed", range(6))
def test_decode_batch_kept_across_steps_equals_the_rebuilt_one(seed):
    """Random life of a running batch -- sequences join with some context, decode token by token (new blocks,
    copy-on-write of a forked last block), leave, rejoin -- with the index vectors updated in place; after
    every step they equal what the step-by-step rebuild (BatchInfoBuilder, itself checked against the
    restatement of batch_info.rs above) gives for the same sequences."""
    rng = np.random.default_rng(300 + seed)
    bs = 16
    a = paged.BlockAllocator(bs, 4096)
    db = paged.DecodeBatch(bs, 1 << 16)
    toks, order, next_id = {}, [], 1

    def join(n):
        nonlocal next_id
        sid, next_id = next_id, next_id + 1
        toks[sid] = rng.integers(0, 32000, size=n).tolist()
        a.alloc_seq(sid, n)
        db.add(a, sid, toks[sid][-1], n)
        order.append(sid)
        return sid

    for _ in range(int(rng.integers(1, 6))):
        join(int(rng.integers(1, 300)))
    for step in range(60):
        ev = rng.random()
        if ev < 0.15 and len(order) < 12:
            join(int(rng.choice([1, 15, 16, 17, int(rng.integers(1, 2000))])))
        elif ev < 0.25 and len(order) > 1:
            sid = order.pop(int(rng.integers(len(order))))
            db.remove(sid)
            a.delete(sid)
        elif ev < 0.35 and order:
            # fork a sequence (blocks shared) and let the child join: its next token must copy the last block
            src = order[int(rng.integers(len(order)))]
            sid, next_id = next_id, next_id + 1
            toks[sid] = list(toks[src])
            a.copy(src, sid, len(toks[src]))
            db.add(a, sid, toks[sid][-1], len(toks[sid]))
            order.append(sid)
        # one generation step for everybody, row by row or all rows in one call
        new = rng.integers(0, 32000, size=len(order)).tolist()
        for sid, t in zip(order, new):
            n0 = len(toks[sid])
            toks[sid].append(t)
            a.append_slots(sid, n0, n0 + 1)
            if step % 2 == 0:
                db.advance(a, sid, t)
        if step % 2 == 1:
            db.advance_all(a, new)
        assert len(db) == len(order)
        b = paged.BatchInfoBuilder(bs, 1 << 16, 1)
        for sid in order:
            b.sched_out(a, sid, toks[sid], len(toks[sid]) - 1)
        assert _as_dict(db.info()) == _as_dict(b.finish())
    with pytest.raises(HipAttnError, match="not in the batch"):
        db.advance(a, 99999, 1)
    with pytest.raises(HipAttnError, match="in the batch already"):
        db.add(a, order[0], 1, len(toks[order[0]]))


def test_step_generation_hand_case():
    """8 blocks of 4 tokens.  Sequences 1, 2, 3 (arrival order) hold 3 + 3 + 2 = 8 blocks, all full: nothing is
    free.  Serving 1 needs a free block, so the latest arrival (3) is preempted and releases 2; 1 takes one
    (block 7, the one freed last... the free list is a stack), 2 takes the other; nobody is left for 3."""
    a = paged.BlockAllocator(4, 8)
    a.alloc_seq(1, 12)
    a.alloc_seq(2, 12)
    a.alloc_seq(3, 8)
    assert a.get_num_free_blocks() == 0
    scheduled, preempted, copies = a.step_generation([1, 2, 3], [13, 13, 9], [12, 12, 8])
    assert (scheduled, preempted, copies) == ([1, 2], [3], [])
    assert a.num_allocated_blocks(1) == 4 and a.num_allocated_blocks(2) == 4 and a.num_allocated_blocks(3) == 0
    assert a.get_num_free_blocks() == 0
    # trim(3, 0) released blocks 6 then 7; the stack hands 7 to sequence 1 and 6 to sequence 2
    assert a.get_block_idxes(1, 13)[-1] == 7 * 4 and a.get_block_idxes(2, 13)[-1] == 6 * 4
    # next step: again nothing free; 2 is preempted for 1, and 1 -- one free block is all the check asks for,
    # needed or not -- goes on
    scheduled, preempted, _ = a.step_generation([1, 2], [14, 14], [13, 13])
    assert (scheduled, preempted) == ([1], [2]) and a.get_num_free_blocks() == 4
    # a lone sequence that finds nothing free preempts itself
    b = paged.BlockAllocator(4, 2)
    b.alloc_seq(5, 8)
    assert b.step_generation([5], [9], [8]) == ([], [5], [])
    assert b.get_num_free_blocks() == 2


@pytest.mark.parametrize("seed", range(8))
def test_step_generation_matches_restatement(seed):
    rng = np.random.default_rng(400 + seed)
    bs, nb = 8, 40
    a, r = paged.BlockAllocator(bs, nb), ref.BlockAllocator(bs, nb)
    lens, running, next_id = {}, [], 1
    for step in range(80):
        # admit while the policy allows (by arrival: ids grow)
        while rng.random() < 0.5:
            n = int(rng.integers(1, 60))
            assert a.can_allocate(n) == r.can_allocate(n)
            if not a.can_allocate(n):
                break
            a.alloc_seq(next_id, n)
            r.alloc_seq(next_id, n)
            lens[next_id] = n
            running.append(next_id)
            next_id += 1
        if rng.random() < 0.1 and running:   # a fork: shared blocks, copy-on-write on the next append
            src = running[int(rng.integers(len(running)))]
            a.copy(src, next_id, lens[src])
            r.copy(src, next_id, lens[src])
            lens[next_id] = lens[src]
            running.append(next_id)
            next_id += 1
        if rng.random() < 0.1 and running:
            sid = running.pop(int(rng.integers(len(running))))
            a.delete(sid)
            r.delete(sid)
        grow = [1 for _ in running]   # a generation step: one token, hence at most one block, per sequence
        args = ([s for s in running], [lens[s] + g for s, g in zip(running, grow)], [lens[s] for s in running])
        got = a.step_generation(*args)
        want = ref.step_generation(r, list(zip(*args)))
        assert got == (want[0], want[1], want[2])
        for s, g in zip(running, grow):
            if s in got[0]:
                lens[s] += g
        running = [s for s in running if s in got[0]]
        assert a.get_num_free_blocks() == r.get_num_free_blocks()
        for s in running:
            assert a.get_block_idxes(s, lens[s]).tolist() == r.get_block_idxes(s, lens[s])


def _space(bs, n_gpu, n_cpu):
    m = paged.BlockSpaceManager(bs, n_gpu, n_cpu, watermark=0.0)
    return m, ref.BlockAllocator(bs, n_gpu), ref.BlockAllocator(bs, n_cpu)


def test_group_step_swaps_out_a_group_of_two_hand_case():
    """8 device blocks of 4 tokens, all taken: group A = sequence 1 (blocks 0-2), group B = sequence 2 (3-5),
    group C = sequences 3 and 4 which share blocks 6, 7 (a fork).  A needs one free block, so C, the latest
    arrival, is preempted; it runs two sequences, so it is swapped: blocks 6, 7 go to host blocks 0, 1 -- once,
    both sequences then hold host blocks [0, 1] -- and the device gets 6, 7 back (7 on top of the stack).  A takes
    7, B takes 6."""
    m, _, _ = _space(4, 8, 8)
    g = m.gpu_allocator
    g.alloc_seq(1, 12)
    g.alloc_seq(2, 12)
    g.alloc_seq(3, 8)
    g.copy(3, 4, 8)
    assert g.get_num_free_blocks() == 0
    R = paged.SEQ_RUNNING
    out = m.step_generation([(1, [(1, R, 13, 12)]), (1, [(2, R, 13, 12)]), (2, [(3, R, 9, 8), (4, R, 9, 8)])])
    assert out["fates"] == [paged.GROUP_SCHEDULED, paged.GROUP_SCHEDULED, paged.GROUP_SWAPPED_OUT]
    assert out["copies"] == [] and out["swap_out"] == [(6, 0), (7, 1)]
    assert g.num_allocated_blocks(3) == 0 and g.num_allocated_blocks(4) == 0
    c = m.cpu_allocator
    assert list(c.get_block_idxes(3, 8)) == list(c.get_block_idxes(4, 8)) == list(range(8))
    assert c.get_num_free_blocks() == 6 and g.get_num_free_blocks() == 0
    assert g.get_block_idxes(1, 13)[-1] == 7 * 4 and g.get_block_idxes(2, 13)[-1] == 6 * 4
    # the way back once there is room: the shared blocks stay shared
    g.delete(1)
    assert not m.can_swap_in([3, 4])   # the check counts a shared block once per holder, plus one per sequence
    g.delete(2)
    assert m.can_swap_in([3, 4])
    back = m.swap_in([3, 4])
    assert sorted(back) == [0, 1] and c.get_num_free_blocks() == 8
    assert list(g.get_block_idxes(3, 8)) == list(g.get_block_idxes(4, 8))
    assert g.get_num_free_blocks() == 6


def test_group_step_suspended_groups_hand_case():
    R, S, F = paged.SEQ_RUNNING, paged.SEQ_SUSPENDED, paged.SEQ_FINISHED
    # the suspended group arrived first: it is set aside, so the running group finds nobody to preempt but itself
    m, _, _ = _space(4, 4, 4)
    m.gpu_allocator.alloc_seq(1, 8)
    m.gpu_allocator.alloc_seq(2, 8)
    out = m.step_generation([(1, [(1, S, 8, 8)]), (1, [(2, R, 9, 8)])])
    assert out["fates"] == [paged.GROUP_SUSPENDED, paged.GROUP_RECOMPUTE]
    assert m.gpu_allocator.num_allocated_blocks(1) == 2 and m.gpu_allocator.num_allocated_blocks(2) == 0
    # the suspended group arrived last: it is still queued when a victim is needed.  With no running sequence it
    # is not a group of one, so it goes the swap way, where only running sequences move: nothing is freed and
    # the running group ends up preempting itself as well.
    m, _, _ = _space(4, 4, 4)
    m.gpu_allocator.alloc_seq(1, 8)
    m.gpu_allocator.alloc_seq(2, 8)
    out = m.step_generation([(1, [(1, R, 9, 8)]), (0, [(2, S, 8, 8)])])
    assert out["fates"] == [paged.GROUP_RECOMPUTE, paged.GROUP_SWAPPED_OUT] and out["swap_out"] == []
    assert m.gpu_allocator.num_allocated_blocks(2) == 2 and m.gpu_allocator.get_num_free_blocks() == 2
    # with room for everybody a suspended group just stays; a finished sequence beside a suspended one counts
    # as suspended, beside a running one it is skipped
    m, _, _ = _space(4, 16, 4)
    for s in (1, 2, 3, 4):
        m.gpu_allocator.alloc_seq(s, 8)
    out = m.step_generation([(2, [(1, S, 8, 8), (2, F, 8, 8)]), (2, [(3, R, 9, 8), (4, F, 8, 8)])])
    assert out["fates"] == [paged.GROUP_SUSPENDED, paged.GROUP_SCHEDULED]
    assert [m.gpu_allocator.num_allocated_blocks(s) for s in (1, 2, 3, 4)] == [2, 2, 3, 2]
    # one free block per running sequence is asked for: two free blocks do not serve a group of three
    m, _, _ = _space(4, 8, 8)
    for s in (1, 2, 3):
        m.gpu_allocator.alloc_seq(s, 8)
    out = m.step_generation([(3, [(1, R, 9, 8), (2, R, 9, 8), (3, R, 9, 8)])])
    assert out["fates"] == [paged.GROUP_SWAPPED_OUT] and len(out["swap_out"]) == 6
    assert m.gpu_allocator.get_num_free_blocks() == 8 and m.cpu_allocator.get_num_free_blocks() == 2


def test_group_step_errors():
    R, F = paged.SEQ_RUNNING, paged.SEQ_FINISHED
    m, _, _ = _space(4, 4, 1)
    m.gpu_allocator.alloc_seq(1, 8)
    m.gpu_allocator.alloc_seq(2, 4)
    m.gpu_allocator.alloc_seq(3, 4)
    with pytest.raises(HipAttnError, match="lack of CPU swap space"):
        m.step_generation([(1, [(1, R, 9, 8)]), (2, [(2, R, 5, 4), (3, R, 5, 4)])])
    # nothing moved: the check comes before the first block changes sides
    assert m.gpu_allocator.get_num_free_blocks() == 0 and m.cpu_allocator.get_num_free_blocks() == 1
    with pytest.raises(HipAttnError, match="has finished"):
        m.step_generation([(1, [(1, R, 9, 8)]), (1, [(2, R, 5, 4), (3, F, 4, 4)])])
    with pytest.raises(HipAttnError, match="phase"):
        m.step_generation([(1, [(1, 7, 9, 8)])])
    assert m.step_generation([]) == {"fates": [], "copies": [], "swap_out": []}


@pytest.mark.parametrize("seed", range(10))
def test_group_step_matches_restatement(seed):
    """A scheduler's life in little: groups are admitted, fork inside themselves, get suspended for a step,
    lose sequences, are swapped out and come back, or are dropped for recomputation and admitted again -- the
    C++ core and the restatement are given the same calls and must agree on every answer and every table."""
    rng = np.random.default_rng(900 + seed)
    bs, n_gpu, n_cpu = 4, 48, 40
    m, rg, rc = _space(bs, n_gpu, n_cpu)
    R, S, F = paged.SEQ_RUNNING, paged.SEQ_SUSPENDED, paged.SEQ_FINISHED
    on_gpu, swapped, waiting = [], [], []   # groups: {"best_of", "seqs": {id: len}, "finished": set}
    next_id = 1
    n_swaps = n_recomputes = 0

    def same_state():
        assert m.gpu_allocator.get_num_free_blocks() == rg.get_num_free_blocks()
        assert m.cpu_allocator.get_num_free_blocks() == rc.get_num_free_blocks()
        for grp in on_gpu + swapped:
            for s, n in grp["seqs"].items():
                for mine, theirs in ((m.gpu_allocator, rg), (m.cpu_allocator, rc)):
                    k = theirs.num_allocated_blocks(s)
                    assert mine.num_allocated_blocks(s) == k
                    if k:
                        assert list(mine.get_block_idxes(s, k * bs)) == theirs.get_block_idxes(s, k * bs)

    for step in range(120):
        # swapped groups come back first (step_swap_in), then prompts are admitted
        while swapped:
            grp = swapped[0]
            ids = list(grp["seqs"])
            want = sum(rc.num_allocated_blocks(s) for s in ids) + len(ids)
            assert m.can_swap_in(ids) == (rg.get_num_free_blocks() >= want)
            if not m.can_swap_in(ids):
                break
            got = m.swap_in(ids)
            mapping = {}
            for s in ids:
                rg.swap_in(s, rc.swap_out(s), mapping)
            assert got == mapping
            on_gpu.append(swapped.pop(0))
        while not swapped and rng.random() < 0.6:
            if waiting and rng.random() < 0.7:
                grp = waiting[0]
            else:
                grp = {"best_of": int(rng.choice([1, 1, 2, 3])), "seqs": {next_id: int(rng.integers(1, 30))},
                       "finished": set()}
                next_id += 1
            (sid, n), = grp["seqs"].items()
            assert m.can_allocate(n) == rg.can_allocate(n)
            if not rg.can_allocate(n):
                break
            m.allocate(sid, n)
            rg.alloc_seq(sid, n)
            if waiting and grp is waiting[0]:
                waiting.pop(0)
            on_gpu.append(grp)
        # after its prompt a group of best_of > 1 forks up to that many sequences
        for grp in on_gpu:
            live = [s for s in grp["seqs"] if s not in grp["finished"]]
            if live and len(grp["seqs"]) < grp["best_of"] and rng.random() < 0.5:
                src = live[int(rng.integers(len(live)))]
                m.gpu_allocator.copy(src, next_id, grp["seqs"][src])
                rg.copy(src, next_id, grp["seqs"][src])
                grp["seqs"][next_id] = grp["seqs"][src]
                next_id += 1
        # a sequence of a group finishes now and then; its blocks go
        for grp in list(on_gpu):
            live = [s for s in grp["seqs"] if s not in grp["finished"]]
            if live and rng.random() < 0.08:
                s = live[int(rng.integers(len(live)))]
                grp["finished"].add(s)
                m.gpu_allocator.delete(s)
                rg.delete(s)
                if len(grp["finished"]) == len(grp["seqs"]):
                    on_gpu.remove(grp)
        same_state()
        # the generation step
        on_gpu.sort(key=lambda grp: min(grp["seqs"]))     # arrival = first id handed out
        groups = []
        for grp in on_gpu:
            susp = rng.random() < 0.15
            seqs = []
            for s, n in grp["seqs"].items():
                ph = F if s in grp["finished"] else (S if susp else R)
                seqs.append((s, ph, n + 1, n))
            running = sum(ph == R for _, ph, _, _ in seqs)
            max_running = grp["best_of"] if grp["best_of"] > len(seqs) else running     # seq.rs:275-292
            groups.append((max_running, seqs))
        try:
            want = ref.step_generation_groups(rg, rc, groups)
        except (ref.OutOfBlocks, AssertionError):
            with pytest.raises(HipAttnError):
                m.step_generation(groups)
            break
        got = m.step_generation(groups)
        assert got["fates"] == want[0] and got["copies"] == want[1] and got["swap_out"] == want[2]
        keep = []
        for grp, (_, seqs), fate in zip(on_gpu, groups, got["fates"]):
            if fate == paged.GROUP_SCHEDULED:
                for s, ph, n1, _ in seqs:
                    if ph == R:
                        grp["seqs"][s] = n1
                keep.append(grp)
            elif fate == paged.GROUP_SUSPENDED:
                keep.append(grp)
            elif fate == paged.GROUP_SWAPPED_OUT:
                if any(ph == R for _, ph, _, _ in seqs):
                    n_swaps += 1
                    grp["seqs"] = {s: n for s, n in grp["seqs"].items() if s not in grp["finished"]}
                    grp["finished"] = set()
                    swapped.append(grp)
                else:
                    keep.append(grp)      # nothing moved: the group still sits on the device
            elif fate == paged.GROUP_RECOMPUTE:
                n_recomputes += 1
                first = min(grp["seqs"])
                grp["seqs"] = {first: grp["seqs"][first]}     # back to a prompt of one sequence
                waiting.append(grp)
            else:
                keep.append(grp)          # not reached: the walk ended before it
        on_gpu = keep
        same_state()
    assert n_swaps + n_recomputes > 0
