from collections import deque


class BlockManager:
    """Free-list allocator of fixed-size KV blocks.  The reference additionally de-duplicates full
    blocks by content hash (prefix cache, nanovllm/engine/block_manager.py:36-82); that is control-
    plane work outside the quantized-linear path and is not reproduced: every sequence owns its blocks."""

    def __init__(self, num_blocks: int, block_size: int):
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.free = deque(range(num_blocks))

    def _needed(self, seq):
        return (len(seq) + self.block_size - 1) // self.block_size

    def can_allocate(self, seq) -> bool:
        return len(self.free) >= self._needed(seq)

    def allocate(self, seq):
        assert not seq.block_table
        for _ in range(self._needed(seq)):
            seq.block_table.append(self.free.popleft())

    def deallocate(self, seq):
        self.free.extend(reversed(seq.block_table))
        seq.block_table.clear()

    def can_append(self, seq) -> bool:
        # a new block is needed when the token about to be written starts a block
        return len(self.free) >= (1 if len(seq) % self.block_size == 1 else 0)

    def may_append(self, seq):
        if len(seq) % self.block_size == 1 and len(seq.block_table) < self._needed(seq):
            seq.block_table.append(self.free.popleft())

    # ---- growth by portions (models whose prompts are cached piece by piece)
    def blocks_short(self, seq, num_tokens: int) -> int:
        """How many more blocks the sequence needs to hold ``num_tokens`` tokens."""
        return max(0, (num_tokens + self.block_size - 1) // self.block_size - len(seq.block_table))

    def reserve(self, seq, num_tokens: int) -> bool:
        """Grow the sequence's block table to hold ``num_tokens`` tokens; False (and nothing taken) if the pool cannot."""
        need = self.blocks_short(seq, num_tokens)
        if need > len(self.free):
            return False
        for _ in range(need):
            seq.block_table.append(self.free.popleft())
        return True


class SlotPool:
    """Fixed-size per-sequence state (the carried inputs of short convolutions, recurrent state) lives in numbered
    slots of one tensor; a sequence holds a slot from its first step until it ends or is preempted.  A slot is NOT
    cleared when it changes hands: the kernels never read state that lies before a sequence's first token."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self.free = deque(range(num_slots))

    def acquire(self, seq) -> bool:
        if seq.state_slot >= 0:
            return True
        if not self.free:
            return False
        seq.state_slot = self.free.popleft()
        return True

    def release(self, seq):
        if seq.state_slot >= 0:
            self.free.append(seq.state_slot)
            seq.state_slot = -1
