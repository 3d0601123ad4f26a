"""Thin Python facade over the native KVCacheManager (csrc/runtime/kv_manager.cpp)."""

from __future__ import annotations

import numpy as np

from .. import _native
from .sequence import Sequence


class StateSlots:
    """Fixed pool of per-sequence state slots (recurrent layers keep one state per live
    sequence).  A slot is taken at admission and given back with the sequence's blocks; lowest
    free slot first, so a freed slot is the next one handed out."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))     # pop() yields the lowest
        self._owner = {}                                     # seq_id -> slot

    def slot_of(self, seq_id: int) -> int:
        return self._owner.get(seq_id, -1)

    def acquire(self, seq_id: int) -> int:
        """The sequence's slot, newly taken if it had none; -1 when the pool is empty."""
        s = self._owner.get(seq_id)
        if s is not None:
            return s
        if not self._free:
            return -1
        s = self._free.pop()
        self._owner[seq_id] = s
        return s

    def release(self, seq_id: int) -> None:
        s = self._owner.pop(seq_id, None)
        if s is not None:
            self._free.append(s)
            self._free.sort(reverse=True)

    def num_free(self) -> int:
        return len(self._free)


class BlockManager:
    def __init__(self, num_blocks: int, block_size: int, prefix_caching: bool = True,
                 num_state_slots: int = 0):
        rt = _native.runtime()
        # a cached prefix skips its tokens, but a recurrent state cannot be skipped into
        prefix_caching = prefix_caching and num_state_slots == 0
        self.native = rt.KVCacheManager(num_blocks, block_size, prefix_caching)
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.prefix_caching = prefix_caching
        self._committed = {}   # seq_id -> full blocks already hashed
        self.slots = StateSlots(num_state_slots) if num_state_slots > 0 else None

    @staticmethod
    def _toks(seq: Sequence) -> np.ndarray:
        return np.asarray(seq.all_token_ids, dtype=np.int32)

    def has(self, seq: Sequence) -> bool:
        return self.native.has_seq(seq.seq_id)

    def allocate_prefix(self, seq: Sequence) -> int:
        return self.native.allocate_prefix(seq.seq_id, self._toks(seq),
                                           getattr(seq, "cache_salt", 0) or 0)

    def ensure(self, seq: Sequence, num_tokens: int) -> bool:
        """Blocks for the sequence's first ``num_tokens`` tokens and, for models with recurrent
        state, its state slot (kept until ``free``)."""
        if self.slots is not None and self.slots.acquire(seq.seq_id) < 0:
            return False
        return self.native.ensure(seq.seq_id, num_tokens)

    def state_slot(self, seq: Sequence) -> int:
        return self.slots.slot_of(seq.seq_id) if self.slots is not None else -1

    def commit(self, seq: Sequence) -> None:
        if not self.prefix_caching:
            return
        nfull = seq.num_computed_tokens // self.block_size
        if nfull > self._committed.get(seq.seq_id, 0):
            toks = np.asarray(seq.all_token_ids[: nfull * self.block_size], dtype=np.int32)
            self.native.commit(seq.seq_id, toks, nfull * self.block_size,
                               getattr(seq, "cache_salt", 0) or 0)
            self._committed[seq.seq_id] = nfull

    def free(self, seq: Sequence) -> None:
        self.native.free(seq.seq_id)
        if self.slots is not None:
            self.slots.release(seq.seq_id)
        self._committed.pop(seq.seq_id, None)

    def block_table(self, seq: Sequence):
        return self.native.block_table(seq.seq_id)

    def usage(self) -> float:
        return self.native.usage()

    def num_free_blocks(self) -> int:
        return self.native.num_free_blocks()

    def reset_prefix_cache(self) -> None:
        self.native.reset_prefix_cache()

    def check_invariants(self) -> str:
        return self.native.check_invariants()

    def stats(self) -> dict:
        return dict(self.native.stats())
