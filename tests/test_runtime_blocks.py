"""Page-ID allocator and token-window state machine: the library (C ABI) and the Python oracle run
the same scripts, whose expected values are the ones the reference's own tests assert:

  allocator bitmaps          crates/inference-runtime-core/src/memory/u32_id_allocator.rs:179-217
  range scan                 crates/inference-runtime-core/src/runtime/scheduler/executor_hibernate.rs:49-61
  vanilla (L=1)              .../trie_cache/blocks/trie/api_test_vanilla.rs:50-97,119-149,192-344,391-436,592-649,749-807
  stored drafts (L=1)        .../trie_cache/blocks/trie/api_test_w_dspark.rs:592-666
  MTP lanes (L=4)            .../trie_cache/blocks/trie/api_test_w_mtp.rs:759-861

Cases whose expected values depend on a prefix-cache hit (an immutable block found in the trie)
are replayed by prefilling that prefix first; the number of in-sync blocks then differs from the
reference's (no collision resets it) and is asserted with this build's own value.
The FIFO order in which freed IDs come back is stated by this build (the reference's tests assert
only counts and bitmaps).
"""
import pytest


def tv(*xs):
    return list(xs)


class OracleImpl:
    name = "oracle"

    def __init__(self, host_oracle):
        self.ho = host_oracle

    def allocator(self, capacity):
        return self.ho.U32IDAllocator(capacity)

    def exhausted(self):
        return self.ho.ResourceExhausted

    def bitmap(self, a):
        return list(a.bitmap)

    def ranges(self, words):
        out, start = [], None
        for i in range(len(words) * 64 + 1):
            bit = i < len(words) * 64 and (words[i >> 6] >> (i & 63)) & 1
            if bit and start is None:
                start = i
            elif not bit and start is not None:
                out.append((start, i))
                start = None
        return out

    def blocks(self, alloc, n, lanes, ppb, tokens):
        return _OracleBlocks(self.ho.DecoderBlocks(n, lanes, alloc, ppb, list(tokens)))


class _OracleBlocks:
    def __init__(self, b):
        self.b = b

    def init(self):
        return self.b.init_block_once()

    def uninit(self):
        return self.b.uninit_block_once()

    def set_spec(self, spec):
        self.b.spec_tokens = list(spec)

    def prepare(self, budget):
        q = self.b.prepare(budget)
        d = dict(kind=q[0], epoch=q[1], token_index=q[2], tokens=list(q[3]))
        if q[0] == "Prefill":
            d["window"] = q[4]
        else:
            d["spec_tokens"] = list(q[4])
        d["_raw"] = q
        return d

    def cancel(self, q):
        self.b.cancel(q["_raw"])

    def commit_prefill(self, q):
        self.b.commit(q["_raw"], None)

    def commit_decode(self, q, validated, sampled, spec):
        self.b.commit(q["_raw"], (list(validated), sampled, list(spec)))

    def prepare_blocks(self):
        return self.b.prepare_blocks()

    def cancel_blocks(self, sync):
        self.b.cancel_blocks(sync)

    def state(self):
        return self.b.state()

    def counts(self):
        return self.b.block_counts()

    def drop(self):
        self.b.drop()


class ProductImpl:
    name = "library"

    def __init__(self, psi):
        import importlib

        self.rt = importlib.import_module("psi-dec_amd.runtime")

    def allocator(self, capacity):
        return self.rt.U32IDAllocator(capacity)

    def exhausted(self):
        return self.rt.ResourceExhausted

    def bitmap(self, a):
        return a.allocated_ids_bitmap()

    def ranges(self, words):
        return self.rt.collect_allocated_id_ranges(words)

    def blocks(self, alloc, n, lanes, ppb, tokens):
        return _ProductBlocks(self.rt, self.rt.DecoderBlocks(alloc, n, lanes, ppb, tokens))


class _ProductBlocks:
    def __init__(self, rt, b):
        self.rt, self.b = rt, b

    def init(self):
        return self.b.init_block_once()

    def uninit(self):
        return self.b.uninit_block_once()

    def set_spec(self, spec):
        self.b.set_spec_tokens(spec)

    def prepare(self, budget):
        q = self.b.prepare(budget)
        d = dict(kind=q.kind, epoch=q.epoch, token_index=q.token_index, tokens=list(q.tokens))
        if q.kind == "Prefill":
            d["window"] = q.window
        else:
            d["spec_tokens"] = list(q.spec_tokens)
        d["_raw"] = q
        return d

    def cancel(self, q):
        self.b.cancel(q["_raw"])

    def commit_prefill(self, q):
        self.b.commit(q["_raw"], self.rt.SampledTokens.prefill(q["epoch"]))

    def commit_decode(self, q, validated, sampled, spec):
        self.b.commit(q["_raw"], self.rt.SampledTokens.decode(q["epoch"], validated, sampled, spec))

    def prepare_blocks(self):
        s = self.b.prepare_blocks()
        return (s.block_index, s.kv_page_ids)

    def cancel_blocks(self, sync):
        self.b.cancel_blocks(self.rt.DecoderSyncBlocks(sync[0], sync[1]))

    def state(self):
        return self.b.state()

    def counts(self):
        return self.b.block_counts()

    def drop(self):
        self.b.drop()


@pytest.fixture(params=["oracle", "library"])
def impl(request, host_oracle, psi):
    return OracleImpl(host_oracle) if request.param == "oracle" else ProductImpl(psi)


def public(q):
    return {k: v for k, v in q.items() if k != "_raw"}


# ------------------------------------------------------------------ allocator


def test_allocator_bitmap_capacity_65(impl):
    a = impl.allocator(65)
    assert impl.bitmap(a) == [0, 0]
    assert [a.alloc_one(), a.alloc_one()] == [0, 1]
    assert impl.bitmap(a) == [0b11, 0]
    assert (a.used(), a.free()) == (2, 63)


def test_allocator_bitmap_capacity_130(impl):
    a = impl.allocator(130)
    ids = a.alloc_many(66)
    assert ids == list(range(66))
    assert impl.bitmap(a) == [2**64 - 1, 0b11, 0]
    a.free_many([1, 63, 64, 65])
    assert impl.bitmap(a) == [(2**64 - 1) & ~(1 << 1) & ~(1 << 63), 0, 0]
    again = a.alloc_many(4)
    assert sorted(again) == [1, 63, 64, 65]
    assert impl.bitmap(a) == [2**64 - 1, 0b11, 0]


def test_allocator_reuses_freed_ids_first_in_first_out(impl):
    a = impl.allocator(16)
    assert a.alloc_many(10) == list(range(10))
    a.free_many([5, 2, 9])
    assert [a.alloc_one(), a.alloc_one(), a.alloc_one()] == [5, 2, 9]
    assert a.alloc_one() == 10  # only then a never-used ID
    a.free_one(3)
    a.free_one(0)
    assert a.alloc_many(4) == [3, 0, 11, 12]


def test_allocator_exhaustion_leaves_counts_unchanged(impl):
    a = impl.allocator(4)
    assert a.alloc_many(3) == [0, 1, 2]
    a.free_many([1])
    with pytest.raises(impl.exhausted()):
        a.alloc_many(3)  # one freed + one fresh available
    assert (a.used(), a.free(), a.capacity()) == (2, 2, 4)
    assert sorted(a.alloc_many(2)) == [1, 3]
    with pytest.raises(impl.exhausted()):
        a.alloc_one()


def test_allocator_zero_capacity(impl):
    a = impl.allocator(0)
    assert impl.bitmap(a) == []
    with pytest.raises(impl.exhausted()):
        a.alloc_one()
    assert a.alloc_many(0) == []


def test_allocated_id_ranges(impl):
    words = [0xB, 0x13, 0, 2**64 - 1]
    assert impl.ranges(words) == [(0, 2), (3, 4), (64, 66), (68, 69), (192, 256)]
    assert impl.ranges([]) == []
    assert impl.ranges([2**64 - 1, 1]) == [(0, 65)]


def test_library_rejects_double_free_and_out_of_range(psi):
    import importlib

    rt = importlib.import_module("psi-dec_amd.runtime")
    a = rt.U32IDAllocator(8)
    a.alloc_many(2)
    with pytest.raises(psi.PsiHipError, match="unallocated"):
        a.free_one(5)
    with pytest.raises(psi.PsiHipError, match="out of range"):
        a.free_one(8)
    with pytest.raises(psi.PsiHipError, match="unallocated"):
        a.free_many([1, 1])
    assert a.allocated_ids_bitmap() == [0b11]  # the failed call changed nothing


# ------------------------------------------------------------------ init / uninit (vanilla, N=4, L=1)

N = 4


def new_blocks(impl, tokens, capacity=1024, lanes=1, ppb=1):
    alloc = impl.allocator(capacity)
    return alloc, impl.blocks(alloc, N, lanes, ppb, tokens)


def test_init_half_block(impl):
    _, b = new_blocks(impl, tv(1, 2))
    assert b.init() == N
    assert b.counts() == (0, 0, 1)
    assert b.state() == (0, [], [], tv(1, 2), [], [])


def test_init_half_block_resource_limit(impl):
    _, b = new_blocks(impl, tv(1, 2), capacity=0)
    assert b.init() == "ResourceLimitExceeded"
    assert b.counts() == (0, 0, 0)
    assert b.state() == (0, [], [], [], tv(1, 2), [])


def test_init_full_block_stays_mutable(impl):
    _, b = new_blocks(impl, tv(1, 2, 3, 4))
    assert b.init() == N
    assert b.counts() == (0, 0, 1)
    assert b.state() == (0, [], [], tv(1, 2, 3, 4), [], [])


def test_init_full_and_half_block_becomes_semi_immutable(impl):
    _, b = new_blocks(impl, tv(1, 2, 3, 4, 5, 6))
    assert b.init() == N
    assert b.counts() == (0, 1, 0)
    assert b.state() == (0, [], [], tv(1, 2, 3, 4), tv(5, 6), [])


def test_init_full_and_half_block_resource_limit(impl):
    _, b = new_blocks(impl, tv(1, 2, 3, 4, 5, 6), capacity=0)
    assert b.init() == "ResourceLimitExceeded"
    assert b.state() == (0, [], [], [], tv(1, 2, 3, 4, 5, 6), [])


def test_init_second_block_after_semi_immutable(impl):
    _, b = new_blocks(impl, tv(1, 2, 3, 4, 5, 6, 7, 8, 9))
    assert b.init() == N
    assert b.init() == 2 * N
    assert b.counts() == (0, 1, 1)
    assert b.state() == (0, [], [], tv(1, 2, 3, 4, 5, 6, 7, 8), tv(9), [])


def test_init_second_block_resource_limit_keeps_first(impl):
    _, b = new_blocks(impl, tv(1, 2, 3, 4, 5, 6, 7, 8, 9), capacity=1)
    assert b.init() == N
    assert b.init() == "ResourceLimitExceeded"
    assert b.counts() == (0, 1, 0)
    assert b.state() == (0, [], [], tv(1, 2, 3, 4), tv(5, 6, 7, 8, 9), [])


def test_uninit_noop_mutable_and_semi_immutable(impl):
    _, b = new_blocks(impl, tv(1, 2))
    assert b.uninit() == 0
    assert b.state() == (0, [], [], [], tv(1, 2), [])
    b.init()
    assert b.state() == (0, [], [], tv(1, 2), [], [])
    assert b.uninit() == 0
    assert b.counts() == (0, 0, 0)
    assert b.state() == (0, [], [], [], tv(1, 2), [])

    alloc, b = new_blocks(impl, tv(1, 2, 3, 4, 5, 6))
    b.init()
    assert b.counts() == (0, 1, 0)
    assert b.uninit() == 0
    assert b.counts() == (0, 0, 0)
    assert b.state() == (0, [], [], [], tv(1, 2, 3, 4, 5, 6), [])
    assert alloc.used() == 0


# ------------------------------------------------------------------ prepare / cancel / commit


def test_prefill_zero_token_index(impl):
    _, b = new_blocks(impl, tv(1, 2, 3))
    assert b.init() == N
    q = b.prepare(2)
    sync = b.prepare_blocks()
    assert public(q) == dict(kind="Prefill", epoch=0, token_index=0, tokens=tv(1, 2), window=2)
    assert sync[0] == 0 and len(sync[1]) == 1 and len(sync[1][0]) == 1
    assert b.state() == (1, [], tv(1, 2), tv(3), [], [])
    b.cancel_blocks(sync)
    b.cancel(q)
    assert b.state() == (0, [], [], tv(1, 2, 3), [], [])
    q2 = b.prepare(2)
    sync2 = b.prepare_blocks()
    assert public(q2) == public(q) and sync2 == sync
    b.commit_prefill(q2)
    assert b.state() == (1, tv(1, 2), [], tv(3), [], [])


def test_prefill_then_decode_outstanding_together(impl):
    # api_test_vanilla.rs:520-590: two prepared queries, committed in order
    _, b = new_blocks(impl, tv(1, 2, 3))
    b.init()
    qp = b.prepare(2)
    qd = b.prepare(1)
    assert public(qp) == dict(kind="Prefill", epoch=0, token_index=0, tokens=tv(1, 2), window=2)
    assert public(qd) == dict(kind="Decode", epoch=0, token_index=2, tokens=tv(3), spec_tokens=[])
    b.cancel(qd)
    b.cancel(qp)
    assert b.state()[1:] == ([], [], tv(1, 2, 3), [], [])
    qp, qd = b.prepare(2), b.prepare(1)
    b.prepare_blocks()
    b.commit_prefill(qp)
    b.commit_decode(qd, [], 4, [])
    assert b.state() == (1, tv(1, 2, 3), [], tv(4), [], [])


def test_decode_zero_token_index(impl):
    _, b = new_blocks(impl, tv(1, 2, 3))
    b.init()
    q = b.prepare(3)
    sync = b.prepare_blocks()
    assert public(q) == dict(kind="Decode", epoch=0, token_index=0, tokens=tv(1, 2, 3), spec_tokens=[])
    assert b.state() == (1, [], tv(1, 2, 3), [], [], [])
    b.cancel_blocks(sync)
    b.cancel(q)
    assert b.state() == (0, [], [], tv(1, 2, 3), [], [])
    q = b.prepare(3)
    b.prepare_blocks()
    b.commit_decode(q, [], 4, [])
    assert b.state() == (1, tv(1, 2, 3), [], tv(4), [], [])


def prefill_prefix(b, count):
    """Runs `count` tokens (a multiple of N) through prefill so that they sit in immutable blocks."""
    done = 0
    while done < count:
        q = b.prepare(N)
        b.prepare_blocks()
        b.commit_prefill(q)
        done += N


def test_decode_nonzero_token_index(impl):
    _, b = new_blocks(impl, tv(1, 2, 3, 4, 5, 6, 7))
    assert b.init() == N  # semi-immutable [1,2,3,4]
    assert b.init() == 2 * N
    prefill_prefix(b, N)
    assert b.counts() == (1, 0, 1)
    assert b.state() == (2, tv(1, 2, 3, 4), [], tv(5, 6, 7), [], [])
    q = b.prepare(3)
    assert public(q) == dict(kind="Decode", epoch=0, token_index=N, tokens=tv(5, 6, 7), spec_tokens=[])
    assert b.state() == (2, tv(1, 2, 3, 4), tv(5, 6, 7), [], [], [])
    b.cancel(q)
    assert b.state() == (2, tv(1, 2, 3, 4), [], tv(5, 6, 7), [], [])
    q = b.prepare(3)
    b.commit_decode(q, [], 8, [])
    assert b.state() == (2, tv(1, 2, 3, 4, 5, 6, 7), [], tv(8), [], [])


def test_decode_full_block_sampled_token_stays_queued(impl):
    _, b = new_blocks(impl, tv(1, 2, 3, 4))
    assert b.init() == N
    q = b.prepare(N)
    b.prepare_blocks()
    assert public(q) == dict(kind="Decode", epoch=0, token_index=0, tokens=tv(1, 2, 3, 4), spec_tokens=[])
    b.commit_decode(q, [], 5, [])
    assert b.counts() == (1, 0, 0)
    # the reference reports 0 in-sync blocks here because its trie already held the block (collision)
    assert b.state() == (1, tv(1, 2, 3, 4), [], [], tv(5), [])
    assert b.init() == N
    assert b.state() == (1, tv(1, 2, 3, 4), [], tv(5), [], [])


def test_decode_with_stored_drafts_accept_one(impl):
    _, b = new_blocks(impl, tv(0))
    assert b.init() == N
    b.set_spec(tv(10, 11, 12))
    q = b.prepare(3)
    sync = b.prepare_blocks()
    assert public(q) == dict(kind="Decode", epoch=0, token_index=0, tokens=tv(0), spec_tokens=tv(10, 11))
    assert b.state() == (1, [], tv(0), [], [], tv(10, 11))
    b.cancel_blocks(sync)
    b.cancel(q)
    assert b.state() == (0, [], [], tv(0), [], tv(10, 11))
    q2 = b.prepare(3)
    b.prepare_blocks()
    assert public(q2) == public(q)
    b.commit_decode(q2, tv(10), 20, tv(30, 31))
    assert b.state() == (1, tv(0, 10), [], tv(20), [], tv(30, 31))
    assert b.counts() == (0, 0, 1)


def test_decode_with_stored_drafts_after_prefix(impl):
    _, b = new_blocks(impl, tv(0, 1, 2, 3, 4))
    b.init()
    b.init()
    prefill_prefix(b, N)
    b.set_spec(tv(10, 11, 12))
    q = b.prepare(3)
    assert public(q) == dict(kind="Decode", epoch=0, token_index=4, tokens=tv(4), spec_tokens=tv(10, 11))
    b.commit_decode(q, tv(10), 20, tv(30, 31))
    assert b.state()[1:] == (tv(0, 1, 2, 3, 4, 10), [], tv(20), [], tv(30, 31))


def test_rejected_drafts_roll_back_to_the_sampled_token(impl):
    _, b = new_blocks(impl, tv(7))
    b.init()
    b.set_spec(tv(10, 11, 12))
    q = b.prepare(4)
    assert q["spec_tokens"] == tv(10, 11, 12)
    b.commit_decode(q, [], 99, [])
    assert b.state()[1:] == (tv(7), [], tv(99), [], [])


def test_commit_rejects_validated_tokens_that_are_no_prefix(impl):
    _, b = new_blocks(impl, tv(0))
    b.init()
    b.set_spec(tv(10, 11))
    q = b.prepare(3)
    with pytest.raises(Exception, match="validated tokens must equal a prefix"):
        b.commit_decode(q, tv(11), 20, [])


def test_accepted_drafts_cross_a_block_boundary(impl):
    alloc, b = new_blocks(impl, tv(1, 2, 3))
    b.init()
    b.init()
    b.set_spec(tv(10, 11, 12))
    q = b.prepare(6)
    assert public(q) == dict(kind="Decode", epoch=0, token_index=0, tokens=tv(1, 2, 3), spec_tokens=tv(10, 11, 12))
    b.prepare_blocks()
    b.commit_decode(q, tv(10, 11, 12), 20, [])
    assert b.counts() == (1, 0, 1)
    assert b.state() == (2, tv(1, 2, 3, 10, 11, 12), [], tv(20), [], [])
    b.drop()
    assert alloc.used() == 0


# ------------------------------------------------------------------ MTP lanes (L=4)


def test_mtp_decode_zero_token_index(impl):
    alloc, b = new_blocks(impl, tv(0, 1, 2, 3), lanes=4)
    slots = 0
    while slots < 6:
        slots = b.init()
    assert slots == 2 * N and b.counts() == (0, 0, 2)
    assert alloc.used() == 8  # 2 blocks x 4 lanes x 1 page
    b.set_spec(tv(10, 11, 12))
    q = b.prepare(6)
    sync = b.prepare_blocks()
    assert public(q) == dict(kind="Decode", epoch=0, token_index=0, tokens=tv(0, 1, 2, 3), spec_tokens=tv(10, 11))
    assert sync[0] == 0 and [len(lane) for lane in sync[1]] == [2, 2, 2, 2]
    assert sync[1] == [[[0], [4]], [[1], [5]], [[2], [6]], [[3], [7]]]  # lanes draw in index order per block
    assert b.state() == (2, [], tv(0), [], tv(1, 2, 3), tv(10, 11))
    b.cancel_blocks(sync)
    b.cancel(q)
    assert b.state() == (0, [], [], tv(0), tv(1, 2, 3), tv(10, 11))
    q2 = b.prepare(6)
    sync2 = b.prepare_blocks()
    assert public(q2) == public(q) and sync2 == sync
    b.commit_decode(q2, tv(10), 20, tv(30, 31))
    assert b.state() == (2, tv(0, 1, 2), [], [], tv(3, 10, 20), tv(30, 31))


def test_mtp_decode_after_prefix(impl):
    _, b = new_blocks(impl, tv(0, 1, 2, 3, 4, 5, 6, 7), lanes=4)
    assert b.init() == N  # cachable 5 -> a full known block [0,1,2,3] with lookahead
    assert b.counts() == (0, 1, 0)
    q = b.prepare(N)
    assert public(q) == dict(kind="Prefill", epoch=0, token_index=0, tokens=tv(0, 1, 2, 3, 4, 5, 6), window=4)
    b.prepare_blocks()
    b.commit_prefill(q)
    assert b.counts() == (1, 0, 0)
    slots = 0
    while slots < 6:
        slots = b.init()
    b.set_spec(tv(10, 11, 12))
    q = b.prepare(6)
    assert public(q) == dict(kind="Decode", epoch=0, token_index=N, tokens=tv(4, 5, 6, 7), spec_tokens=tv(10, 11))
    assert b.state()[1:] == (tv(0, 1, 2, 3), tv(4), [], tv(5, 6, 7), tv(10, 11))
    b.cancel(q)
    assert b.state()[1:] == (tv(0, 1, 2, 3), [], tv(4), tv(5, 6, 7), tv(10, 11))
    q = b.prepare(6)
    b.commit_decode(q, tv(10), 20, tv(30, 31))
    assert b.state()[1:] == (tv(0, 1, 2, 3, 4, 5, 6), [], [], tv(7, 10, 20), tv(30, 31))


def test_prefill_chunk_must_end_where_the_lookahead_starts(impl):
    # With L > 1 the L-1 lookahead tokens are read from the queue, so a prefill chunk has to take
    # every ready token; the reference's scheduler only ever asks for such budgets.
    _, b = new_blocks(impl, tv(0, 1, 2, 3, 4, 5, 6, 7), lanes=4)
    b.init()
    with pytest.raises(Exception, match="prefill"):
        b.prepare(2)
    assert b.state() == (0, [], [], tv(0, 1, 2, 3), tv(4, 5, 6, 7), [])


def test_mtp_lane_allocation_rolls_back(impl):
    alloc, b = new_blocks(impl, tv(0, 1, 2, 3), capacity=3, lanes=4)
    assert b.init() == "ResourceLimitExceeded"
    assert (alloc.used(), alloc.free()) == (0, 3)
    assert b.state() == (0, [], [], [], tv(0, 1, 2, 3), [])
    # lanes 0..2 were released in lane order, so the IDs come back in that order
    assert alloc.alloc_many(3) == [0, 1, 2]


# ------------------------------------------------------------------ library vs oracle on random schedules


@pytest.mark.parametrize("lanes", [1, 2, 4])
@pytest.mark.parametrize("seed", range(6))
def test_random_schedules_agree(host_oracle, psi, lanes, seed):
    import random

    rng = random.Random(1000 * lanes + seed)
    o, p = OracleImpl(host_oracle), ProductImpl(psi)
    n_prompt = rng.randint(lanes, 23)
    prompt = [rng.randrange(1000) for _ in range(n_prompt)]
    ppb = rng.choice([1, 2, 3])
    cap = rng.choice([8, 64, 1024]) * lanes * ppb
    ao, ap = o.allocator(cap), p.allocator(cap)
    bo, bp = o.blocks(ao, N, lanes, ppb, prompt), p.blocks(ap, N, lanes, ppb, prompt)
    next_token = 5000
    for step in range(80):
        assert bo.state() == bp.state(), f"step {step}"
        assert bo.counts() == bp.counts()
        assert (ao.used(), ao.free()) == (ap.used(), ap.free())
        _, _, _, ready, queued, spec = bo.state()
        validated = len(ready) + len(queued)
        if len(queued) >= lanes and ready:
            # prefill chunk; with L > 1 it has to end where the queued lookahead starts
            budget = rng.randint(1, len(ready)) if lanes == 1 else len(ready)
        elif len(queued) >= lanes:
            budget = None  # nothing placed yet: add a block
        else:
            budget = validated + rng.randint(0, len(spec))
        # the reference's request loop: add blocks until the budget fits (req_resp.rs:77-98)
        exhausted = False
        while budget is None or bo.b.ready_token_slots() < budget:
            ro, rp = bo.init(), bp.init()
            assert ro == rp
            if ro == "ResourceLimitExceeded":
                exhausted = True
                break
            if budget is None:
                break
        if exhausted:
            assert bo.uninit() == bp.uninit()
            # The reference keeps a stale in-sync count when a synced block is released (its next
            # prepare_blocks then trips a debug assertion); the library clamps it to the blocks left.
            bo.b.num_in_sync_blocks = min(bo.b.num_in_sync_blocks, sum(bo.counts()))
            continue
        if budget is None:
            continue
        qo, qp = bo.prepare(budget), bp.prepare(budget)
        assert public(qo) == public(qp)
        so, sp = bo.prepare_blocks(), bp.prepare_blocks()
        assert so == sp
        if rng.random() < 0.25:
            bo.cancel_blocks(so), bp.cancel_blocks(sp)
            bo.cancel(qo), bp.cancel(qp)
            continue
        if qo["kind"] == "Prefill":
            bo.commit_prefill(qo), bp.commit_prefill(qp)
        else:
            accepted = rng.randint(0, len(qo["spec_tokens"]))
            new_spec = [next_token + 100 + i for i in range(rng.randint(0, 3))]
            bo.commit_decode(qo, qo["spec_tokens"][:accepted], next_token, new_spec)
            bp.commit_decode(qp, qp["spec_tokens"][:accepted], next_token, new_spec)
            next_token += 1
    assert next_token > 5000, "the schedule never reached a decode step"
    bo.drop(), bp.drop()
    assert (ao.used(), ap.used()) == (0, 0)
    assert o.bitmap(ao) == p.bitmap(ap)
