"""Minimal continuous-batching attention engine over the paged KV cache.

What a KV-cached replacement of TransformerLM.generate (llm-core/llm_core/model.py:187-236,
which re-runs the whole forward per token at :218) needs around the attention kernels: a block
allocator, per-sequence block tables, slot mapping for cache writes, a prefill call for newly
admitted sequences and a decode call that serves every running sequence with one kernel launch
per step.  One engine instance serves ONE attention layer (its own K/V pools); a model keeps one
per layer.  Projections, sampling and the scheduler policy stay with the caller.

All tensor work runs on the HIP kernels (rope_and_cache, flash_attn_varlen_prefill,
paged_attention_decode); the bookkeeping here is plain Python on host integers.
"""
from __future__ import annotations

import torch

from . import ops

BLOCK = 16


class OutOfBlocks(RuntimeError):
    pass


class BlockAllocator:
    """Free list of physical cache blocks."""

    def __init__(self, num_blocks: int):
        self.num_blocks = num_blocks
        self._free = list(range(num_blocks - 1, -1, -1))

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise OutOfBlocks("KV cache is out of blocks")
        return self._free.pop()

    def free(self, blocks) -> None:
        self._free.extend(blocks)


class PagedAttentionEngine:
    def __init__(self, num_blocks, n_q_heads, n_kv_heads, head_dim, context_length, *, rope_theta=10000.0,
                 max_batch=256, device="cuda:0"):
        self.device = torch.device(device)
        self.Hq, self.Hkv, self.D = n_q_heads, n_kv_heads, head_dim
        self.context_length = context_length
        self.k_cache = torch.zeros(num_blocks, n_kv_heads, BLOCK, head_dim, dtype=torch.bfloat16, device=self.device)
        self.v_cache = torch.zeros_like(self.k_cache)
        self.freq_cache = ops.build_rope_cache(context_length, head_dim, rope_theta, self.device)
        self.allocator = BlockAllocator(num_blocks)
        self.blocks: dict[int, list[int]] = {}      # sequence id -> physical blocks
        self.lengths: dict[int, int] = {}           # sequence id -> tokens in the cache
        self.max_blocks_per_seq = (context_length + BLOCK - 1) // BLOCK
        # persistent step buffers: no allocation on the decode path besides the kernel outputs
        self._tables = torch.zeros(max_batch, self.max_blocks_per_seq, dtype=torch.int32, device=self.device)
        self._workspace = ops.paged_decode_workspace(max_batch, n_q_heads, head_dim, context_length, self.device)
        self.max_batch = max_batch

    # ---- bookkeeping ---------------------------------------------------------
    def add_sequence(self, seq_id: int) -> None:
        if seq_id in self.blocks:
            raise ValueError(f"sequence {seq_id} already exists")
        self.blocks[seq_id] = []
        self.lengths[seq_id] = 0

    def remove_sequence(self, seq_id: int) -> None:
        self.allocator.free(self.blocks.pop(seq_id))
        del self.lengths[seq_id]

    def _reserve(self, seq_id: int, n_new: int) -> list[int]:
        """Slots for the next n_new tokens of a sequence (allocates blocks as needed)."""
        length = self.lengths[seq_id]
        if length + n_new > self.context_length:
            raise ValueError(f"sequence {seq_id} would exceed context_length {self.context_length}")
        blocks = self.blocks[seq_id]
        need = (length + n_new + BLOCK - 1) // BLOCK - len(blocks)
        if need > self.allocator.num_free:
            raise OutOfBlocks(f"sequence {seq_id} needs {need} blocks, {self.allocator.num_free} free")
        for _ in range(need):
            blocks.append(self.allocator.allocate())
        slots = [blocks[t // BLOCK] * BLOCK + t % BLOCK for t in range(length, length + n_new)]
        self.lengths[seq_id] = length + n_new
        return slots

    # ---- attention calls --------------------------------------------------------
    def prefill(self, seq_ids, lens, q, k, v):
        """Prompts of `seq_ids` (new, empty sequences) with `lens` tokens each, packed along dim 0.
        Writes rotated K and V into the cache and returns causal attention output (T,Hq,D)."""
        if sum(lens) != q.shape[0]:
            raise ValueError("sum(lens) must equal the number of packed tokens")
        slots, positions, cu = [], [], [0]
        for sid, n in zip(seq_ids, lens):
            if self.lengths[sid] != 0:
                raise ValueError(f"sequence {sid} already has tokens; chunked prefill is not supported")
            slots += self._reserve(sid, n)
            positions += list(range(n))
            cu.append(cu[-1] + n)
        dev = self.device
        pos = torch.tensor(positions, dtype=torch.int32, device=dev)
        slot_t = torch.tensor(slots, dtype=torch.int64, device=dev)
        cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
        q_rot = ops.rope_and_cache(q, k, v, pos, self.freq_cache, self.k_cache, self.v_cache, slot_t)
        k_rot = ops.rope_and_cache(k, k, v, pos, self.freq_cache)            # rotated keys, packed, for the prefill kernel
        return ops.flash_attn_varlen_prefill(q_rot, k_rot, v, cu_t, cu_t, max(lens), max(lens), causal=True)

    def decode_step(self, seq_ids, q, k, v):
        """One new token for each running sequence in `seq_ids`: q (B,Hq,D), k/v (B,Hkv,D) bf16.
        Appends the token's K/V to the cache and returns its attention output (B,Hq,D)."""
        B = len(seq_ids)
        if B > self.max_batch:
            raise ValueError(f"batch {B} exceeds max_batch {self.max_batch}")
        if q.shape[0] != B:
            raise ValueError("one query token per sequence expected")
        positions = [self.lengths[s] for s in seq_ids]
        slots = [self._reserve(s, 1)[0] for s in seq_ids]
        dev = self.device
        max_len = max(self.lengths[s] for s in seq_ids)
        max_blk = (max_len + BLOCK - 1) // BLOCK
        rows = torch.zeros(B, max_blk, dtype=torch.int32)
        for i, s in enumerate(seq_ids):
            b = self.blocks[s]
            rows[i, :len(b)] = torch.tensor(b, dtype=torch.int32)
        tables = self._tables[:B, :max_blk]
        tables.copy_(rows, non_blocking=False)
        ctx = torch.tensor([self.lengths[s] for s in seq_ids], dtype=torch.int32, device=dev)
        pos = torch.tensor(positions, dtype=torch.int32, device=dev)
        slot_t = torch.tensor(slots, dtype=torch.int64, device=dev)
        q_rot = ops.rope_and_cache(q, k, v, pos, self.freq_cache, self.k_cache, self.v_cache, slot_t)
        return ops.paged_attention_decode(q_rot, self.k_cache, self.v_cache, tables, ctx,
                                          max_context=max_blk * BLOCK, workspace=self._workspace)
