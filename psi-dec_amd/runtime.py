"""Host-side cache ownership over the C ABI: the page-ID allocator and the per-request token window.

Names follow the reference's runtime core so that its tests read the same here:
  U32IDAllocator     crates/inference-runtime-core/src/memory/u32_id_allocator.rs:18-37
  DecoderBlocks      crates/inference-runtime-core/src/runtime/decoder/trie_cache/blocks/mod.rs:12-41
                     (the `TrieDecoderBlocks` implementation, blocks/trie/api.rs:34-571, without a prefix trie)
  QueryTokens        crates/inference-runtime-core/src/compute/request/decoder/query_tokens.rs:4-17
  SampledTokens      crates/inference-runtime-core/src/compute/request/decoder/sample_tokens.rs:6-20
  DecoderSyncBlocks  crates/inference-runtime-core/src/compute/request/decoder/decoder_sync_blocks.rs:2-6
Everything here is a thin wrapper: the logic lives in csrc/runtime_blocks.cpp.
"""
import ctypes
from ctypes import byref, c_size_t, c_uint32, c_uint64, c_void_p
from dataclasses import dataclass, field
from typing import List, Tuple

from . import _lib
from ._lib import PsiHipError, check, u32_array


class ResourceExhausted(PsiHipError):
    """`Error::ResourceExhausted` (crates/inference-runtime-core/src/error.rs:2-23)."""


def _check(status):
    if status == _lib.ERR_RESOURCE_EXHAUSTED:
        raise ResourceExhausted(status, _lib.load().psi_hip_last_error().decode("utf-8", "replace"))
    check(status)


class U32IDAllocator:
    def __init__(self, capacity: int):
        self._lib = _lib.load()
        self._h = c_void_p()
        _check(self._lib.psi_hip_id_allocator_create(capacity, byref(self._h)))
        self._capacity = capacity

    def close(self):
        if self._h:
            self._lib.psi_hip_id_allocator_destroy(self._h)
            self._h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def handle(self):
        return self._h

    def alloc_one(self) -> int:
        out = c_uint32()
        _check(self._lib.psi_hip_id_allocator_alloc_one(self._h, byref(out)))
        return out.value

    def alloc_many(self, count: int) -> List[int]:
        out = (c_uint32 * max(count, 1))()
        _check(self._lib.psi_hip_id_allocator_alloc_many(self._h, count, out))
        return list(out[:count])

    def free_one(self, page_id: int):
        _check(self._lib.psi_hip_id_allocator_free_one(self._h, page_id))

    def free_many(self, page_ids):
        page_ids = list(page_ids)
        _check(self._lib.psi_hip_id_allocator_free_many(self._h, u32_array(page_ids), len(page_ids)))

    def _counts(self) -> Tuple[int, int, int]:
        used, free, cap = c_uint64(), c_uint64(), c_uint64()
        _check(self._lib.psi_hip_id_allocator_counts(self._h, byref(used), byref(free), byref(cap)))
        return used.value, free.value, cap.value

    def used(self) -> int:
        return self._counts()[0]

    def free(self) -> int:
        return self._counts()[1]

    def capacity(self) -> int:
        return self._counts()[2]

    def allocated_ids_bitmap(self) -> List[int]:
        n = (self._capacity + 63) // 64
        words = (c_uint64 * max(n, 1))()
        _check(self._lib.psi_hip_id_allocator_bitmap(self._h, words, n))
        return list(words[:n])


def collect_allocated_id_ranges(words) -> List[Tuple[int, int]]:
    """`collect_allocated_id_ranges` (crates/inference-runtime-core/src/runtime/scheduler/executor_hibernate.rs:10-47)."""
    lib = _lib.load()
    words = [int(w) for w in words]
    arr = (c_uint64 * max(len(words), 1))(*words)
    n = c_size_t()
    _check(lib.psi_hip_bitmap_allocated_ranges(arr, len(words), None, 0, byref(n)))
    out = (c_uint32 * max(2 * n.value, 1))()
    _check(lib.psi_hip_bitmap_allocated_ranges(arr, len(words), out, n.value, byref(n)))
    return [(out[2 * i], out[2 * i + 1]) for i in range(n.value)]


@dataclass
class QueryTokens:
    kind: str  # "Prefill" | "Decode"
    epoch: int
    token_index: int
    tokens: List[int]
    window: int = 0  # Prefill
    spec_tokens: List[int] = field(default_factory=list)  # Decode

    def _struct(self):
        tokens, spec = u32_array(self.tokens), u32_array(self.spec_tokens)
        s = _lib.QueryTokensStruct(
            kind=0 if self.kind == "Prefill" else 1, window=self.window, epoch=self.epoch, token_index=self.token_index,
            tokens=ctypes.cast(tokens, ctypes.POINTER(c_uint32)), num_tokens=len(self.tokens),
            tokens_capacity=len(self.tokens), spec_tokens=ctypes.cast(spec, ctypes.POINTER(c_uint32)),
            num_spec_tokens=len(self.spec_tokens), spec_tokens_capacity=len(self.spec_tokens))
        s._keep = (tokens, spec)
        return s


@dataclass
class SampledTokens:
    kind: str
    epoch: int = 0
    validated_tokens: List[int] = field(default_factory=list)
    sampled_token: int = 0
    spec_tokens: List[int] = field(default_factory=list)

    @staticmethod
    def prefill(epoch=0):
        return SampledTokens("Prefill", epoch)

    @staticmethod
    def decode(epoch, validated_tokens, sampled_token, spec_tokens=()):
        return SampledTokens("Decode", epoch, list(validated_tokens), sampled_token, list(spec_tokens))


@dataclass
class DecoderSyncBlocks:
    block_index: int
    kv_page_ids: List[List[List[int]]]  # [lane][block][pages_per_kv_block]


class DecoderBlocks:
    """One request's token window and block ownership (`N` tokens per block, `L` cache lanes)."""

    def __init__(self, allocator: U32IDAllocator, tokens_per_block: int, num_cache_lanes: int,
                 pages_per_kv_block: int, tokens):
        self._lib = _lib.load()
        self._alloc = allocator  # keeps the allocator alive
        self.n, self.lanes, self.ppb = tokens_per_block, num_cache_lanes, pages_per_kv_block
        tokens = list(tokens)
        cfg = _lib.DecoderBlocksConfigStruct(tokens_per_block, num_cache_lanes, pages_per_kv_block)
        self._h = c_void_p()
        _check(self._lib.psi_hip_decoder_blocks_create(allocator.handle, byref(cfg), u32_array(tokens), len(tokens),
                                                       byref(self._h)))

    def close(self):
        if self._h:
            self._lib.psi_hip_decoder_blocks_destroy(self._h)
            self._h = c_void_p()

    drop = close

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def ready_token_slots(self) -> int:
        out = c_size_t()
        _check(self._lib.psi_hip_decoder_blocks_ready_token_slots(self._h, byref(out)))
        return out.value

    def init_block_once(self):
        """Returns the ready token slots, or the string "ResourceLimitExceeded"
        (`InitBlockOnceResult`, .../trie_cache/blocks/mod.rs)."""
        out = c_size_t()
        status = self._lib.psi_hip_decoder_blocks_init_block_once(self._h, byref(out))
        if status == _lib.ERR_RESOURCE_EXHAUSTED:
            return "ResourceLimitExceeded"
        _check(status)
        return out.value

    def uninit_block_once(self) -> int:
        out = c_size_t()
        _check(self._lib.psi_hip_decoder_blocks_uninit_block_once(self._h, byref(out)))
        return out.value

    def set_spec_tokens(self, spec_tokens):
        spec_tokens = list(spec_tokens)
        _check(self._lib.psi_hip_decoder_blocks_set_spec_tokens(self._h, u32_array(spec_tokens), len(spec_tokens)))

    def prepare(self, token_budget: int) -> QueryTokens:
        cap_tokens = token_budget + self.lanes + self._count(_TOKENS["queued"])
        tokens, spec = (c_uint32 * cap_tokens)(), (c_uint32 * max(token_budget, 1))()
        q = _lib.QueryTokensStruct(tokens=ctypes.cast(tokens, ctypes.POINTER(c_uint32)), tokens_capacity=cap_tokens,
                                   spec_tokens=ctypes.cast(spec, ctypes.POINTER(c_uint32)),
                                   spec_tokens_capacity=max(token_budget, 1))
        _check(self._lib.psi_hip_decoder_blocks_prepare(self._h, token_budget, byref(q)))
        return QueryTokens("Prefill" if q.kind == 0 else "Decode", q.epoch, q.token_index,
                           list(tokens[:q.num_tokens]), q.window, list(spec[:q.num_spec_tokens]))

    def cancel(self, query: QueryTokens):
        s = query._struct()
        _check(self._lib.psi_hip_decoder_blocks_cancel(self._h, byref(s)))

    def commit(self, query: QueryTokens, sampled: SampledTokens):
        q = query._struct()
        validated, spec = u32_array(sampled.validated_tokens), u32_array(sampled.spec_tokens)
        s = _lib.SampledTokensStruct(
            kind=0 if sampled.kind == "Prefill" else 1, sampled_token=sampled.sampled_token, epoch=sampled.epoch,
            validated_tokens=ctypes.cast(validated, ctypes.POINTER(c_uint32)),
            num_validated_tokens=len(sampled.validated_tokens),
            spec_tokens=ctypes.cast(spec, ctypes.POINTER(c_uint32)), num_spec_tokens=len(sampled.spec_tokens))
        _check(self._lib.psi_hip_decoder_blocks_commit(self._h, byref(q), byref(s)))

    def prepare_blocks(self) -> DecoderSyncBlocks:
        start, count = c_size_t(), c_size_t()
        _check(self._lib.psi_hip_decoder_blocks_prepare_blocks(self._h, byref(start), byref(count), None, 0))
        total = self.lanes * count.value * self.ppb
        ids = (c_uint32 * max(total, 1))()
        _check(self._lib.psi_hip_decoder_blocks_prepare_blocks(self._h, byref(start), byref(count), ids, total))
        flat = list(ids[:total])
        per_lane = count.value * self.ppb
        return DecoderSyncBlocks(start.value, [
            [flat[lane * per_lane + blk * self.ppb: lane * per_lane + (blk + 1) * self.ppb]
             for blk in range(count.value)] for lane in range(self.lanes)])

    def cancel_blocks(self, sync_blocks: DecoderSyncBlocks):
        _check(self._lib.psi_hip_decoder_blocks_cancel_blocks(self._h, sync_blocks.block_index))

    def commit_blocks(self, sync_blocks: DecoderSyncBlocks):
        """No-op, as in the reference (blocks/trie/mod.rs:235-237)."""

    def block_counts(self) -> Tuple[int, int, int]:
        a, b, c, d = c_size_t(), c_size_t(), c_size_t(), c_size_t()
        _check(self._lib.psi_hip_decoder_blocks_counts(self._h, byref(a), byref(b), byref(c), byref(d)))
        return a.value, b.value, c.value

    @property
    def num_in_sync_blocks(self) -> int:
        d = c_size_t()
        _check(self._lib.psi_hip_decoder_blocks_counts(self._h, None, None, None, byref(d)))
        return d.value

    def _count(self, which):
        n = c_size_t()
        _check(self._lib.psi_hip_decoder_blocks_tokens(self._h, which, None, 0, byref(n)))
        return n.value

    def _tokens(self, which) -> List[int]:
        n = self._count(which)
        out = (c_uint32 * max(n, 1))()
        _check(self._lib.psi_hip_decoder_blocks_tokens(self._h, which, out, n, byref(c_size_t())))
        return list(out[:n])

    def cached_tokens(self):
        return self._tokens(_TOKENS["cached"])

    def scheduled_tokens(self):
        return self._tokens(_TOKENS["scheduled"])

    def ready_tokens(self):
        return self._tokens(_TOKENS["ready"])

    def queued_tokens(self):
        return self._tokens(_TOKENS["queued"])

    def spec_tokens(self):
        return self._tokens(_TOKENS["spec"])

    def state(self):
        """(in-sync blocks, cached, scheduled, ready, queued, spec): the tuple the reference's
        `assert_state` helper checks."""
        return (self.num_in_sync_blocks, self.cached_tokens(), self.scheduled_tokens(), self.ready_tokens(),
                self.queued_tokens(), self.spec_tokens())


_TOKENS = {"cached": 0, "scheduled": 1, "ready": 2, "queued": 3, "spec": 4}
