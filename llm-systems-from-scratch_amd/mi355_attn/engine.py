"""Minimal continuous-batching attention engine over the paged KV cache.

What a KV-cached replacement of TransformerLM.generate (llm-core/llm_core/model.py:187-236,
which re-runs the whole forward per token at :218) needs around the attention kernels: a block
allocator, per-sequence block tables, slot mapping for cache writes, a prefill call for newly
admitted sequences and a decode call that serves every running sequence with one kernel launch
per layer and step.  The bookkeeping (blocks, lengths, tables) is shared by all attention layers
of a model; every layer has its own K/V pools.  A step is planned once (`plan_prefill`,
`plan_decode`: host integers -> a few small device tensors) and then applied per layer
(`attend_prefill`, `attend_decode`).  Projections, sampling and the scheduler policy stay with
the caller.

All tensor work runs on the HIP kernels (rope_and_cache, flash_attn_varlen_prefill,
flash_attn_paged_prefill, paged_attention_decode); the bookkeeping here is plain Python on host integers.
"""
from __future__ import annotations

from dataclasses import dataclass

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


@dataclass
class PrefillPlan:
    positions: torch.Tensor      # (T,) int32
    slots: torch.Tensor          # (T,) int64
    cu_seqlens: torch.Tensor     # (B+1,) int32
    max_len: int
    last_rows: torch.Tensor      # (B,) int64: packed row of each sequence's last token
    # set when some sequence already had tokens in the cache (a further chunk of its prompt): the attention
    # then reads all keys and values through the block tables
    tables: torch.Tensor | None = None        # (B, max_blocks) int32
    context_lens: torch.Tensor | None = None  # (B,) int32: tokens in the cache, this chunk included
    total_context: int = 0                    # their sum (sizes the dequantised rows of an fp8 cache)
    cu_context: torch.Tensor | None = None    # (B+1,) int32: their running sum (fp8 cache: where each sequence's rows start)


@dataclass
class DecodePlan:
    positions: torch.Tensor      # (B,) int32
    slots: torch.Tensor          # (B,) int64
    tables: torch.Tensor         # (B, max_blocks) int32
    context_lens: torch.Tensor   # (B,) int32, the new token included
    max_context: int


class StaticDecodeStep:
    """Device tensors of one decode step at fixed addresses, refreshed from the host by one copy.

    Layout of the int32 buffer: token ids (int64), slots (int64), positions, context lengths,
    block tables (batch x max_blocks)."""

    def __init__(self, batch: int, max_blocks: int, device):
        B, M = batch, max_blocks
        self.batch, self.max_blocks = B, M
        n = 6 * B + B * M
        self._dev = torch.zeros(n, dtype=torch.int32, device=device)
        self._host = torch.zeros(n, dtype=torch.int32, pin_memory=True)
        self._copied = torch.cuda.Event()
        self._pending = False
        self.tokens = self._dev[0:2 * B].view(torch.int64)
        slots = self._dev[2 * B:4 * B].view(torch.int64)
        positions = self._dev[4 * B:5 * B]
        context_lens = self._dev[5 * B:6 * B]
        tables = self._dev[6 * B:].view(B, M)
        self.plan = DecodePlan(positions, slots, tables, context_lens, M * BLOCK)
        h = self._host
        self._h_tokens, self._h_slots = h[0:2 * B].view(torch.int64), h[2 * B:4 * B].view(torch.int64)
        self._h_positions, self._h_ctx, self._h_tables = h[4 * B:5 * B], h[5 * B:6 * B], h[6 * B:].view(B, M)

    def fill(self, tokens, slots, positions, context_lens, block_lists) -> None:
        if self._pending:
            self._copied.synchronize()              # the previous copy has left the staging buffer
        self._h_tokens.copy_(torch.tensor(tokens, dtype=torch.int64))
        self._h_slots.copy_(torch.tensor(slots, dtype=torch.int64))
        self._h_positions.copy_(torch.tensor(positions, dtype=torch.int32))
        self._h_ctx.copy_(torch.tensor(context_lens, dtype=torch.int32))
        for i, blocks in enumerate(block_lists):
            self._h_tables[i, :len(blocks)] = torch.tensor(blocks, dtype=torch.int32)
        self._dev.copy_(self._host, non_blocking=True)
        self._copied.record()
        self._pending = True


class PagedAttentionEngine:
    def __init__(self, num_blocks, n_q_heads, n_kv_heads, head_dim, context_length, *, rope_theta=10000.0,
                 max_batch=256, num_layers=1, kv_dtype="bf16", device="cuda:0"):
        self.device = torch.device(device)
        self.Hq, self.Hkv, self.D = n_q_heads, n_kv_heads, head_dim
        self.context_length = context_length
        self.num_layers = num_layers
        if kv_dtype not in ("bf16", "fp8"):
            raise ValueError("kv_dtype must be 'bf16' or 'fp8'")
        if kv_dtype == "fp8" and head_dim not in (64, 128):
            raise ValueError("an fp8 KV cache needs head_dim 64 or 128")
        self.kv_dtype = kv_dtype
        cache_dtype = torch.bfloat16 if kv_dtype == "bf16" else torch.uint8      # uint8 = e4m3 bit patterns
        self.k_caches = [torch.zeros(num_blocks, n_kv_heads, BLOCK, head_dim, dtype=cache_dtype, device=self.device)
                         for _ in range(num_layers)]
        self.v_caches = [torch.zeros_like(k) for k in self.k_caches]
        # per-(block, kv head) scales of an fp8 cache, maintained by the cache write
        self.k_scales = [torch.ones(num_blocks, n_kv_heads, dtype=torch.float32, device=self.device)
                         for _ in range(num_layers)] if kv_dtype == "fp8" else None
        self.v_scales = [torch.ones_like(s) for s in self.k_scales] if kv_dtype == "fp8" else None
        self.freq_cache = ops.build_rope_cache(context_length, head_dim, rope_theta, self.device)
        self.allocator = BlockAllocator(num_blocks)
        self.blocks: dict[int, list[int]] = {}      # sequence id -> physical blocks
        self.lengths: dict[int, int] = {}           # sequence id -> tokens in the cache
        self.max_blocks_per_seq = (context_length + BLOCK - 1) // BLOCK
        # persistent step buffers: no allocation on the decode path besides the kernel outputs
        self._tables = torch.zeros(max_batch, self.max_blocks_per_seq, dtype=torch.int32, device=self.device)
        self._workspace = ops.paged_decode_workspace(max_batch, n_q_heads, head_dim, context_length, self.device)
        self.max_batch = max_batch

    # the pools of layer 0 under their single-layer names
    @property
    def k_cache(self):
        return self.k_caches[0]

    @property
    def v_cache(self):
        return self.v_caches[0]

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

    # ---- planning (once per step) ---------------------------------------------
    def plan_prefill(self, seq_ids, lens) -> PrefillPlan:
        """Reserves cache slots for the next `lens[i]` prompt tokens of each sequence in `seq_ids`.  A sequence
        may be new (the usual case) or already hold tokens -- a further chunk of a long prompt, or a prompt on
        top of a cached prefix: the chunk's queries then attend to everything cached so far (with an fp8 cache: to
        the quantised keys and values, the chunk's own included, as every later decode step will)."""
        if len(seq_ids) != len(lens) or not seq_ids:
            raise ValueError("seq_ids and lens must be non-empty and of equal length")
        if len(set(seq_ids)) != len(seq_ids):
            raise ValueError("a sequence may appear only once per prefill")
        for sid, n in zip(seq_ids, lens):
            if n < 1 or self.lengths[sid] + n > self.context_length:
                raise ValueError(f"prompt lengths must be in 1..{self.context_length} (tokens already cached included)")
        chunked = any(self.lengths[sid] != 0 for sid in seq_ids)
        need = sum((self.lengths[sid] + n + BLOCK - 1) // BLOCK - len(self.blocks[sid]) for sid, n in zip(seq_ids, lens))
        if need > self.allocator.num_free:
            raise OutOfBlocks(f"prefill needs {need} blocks, {self.allocator.num_free} free")
        slots, positions, cu = [], [], [0]
        for sid, n in zip(seq_ids, lens):
            start = self.lengths[sid]
            slots += self._reserve(sid, n)
            positions += list(range(start, start + n))
            cu.append(cu[-1] + n)
        dev = self.device
        plan = PrefillPlan(torch.tensor(positions, dtype=torch.int32, device=dev),
                           torch.tensor(slots, dtype=torch.int64, device=dev),
                           torch.tensor(cu, dtype=torch.int32, device=dev), max(lens),
                           torch.tensor([c - 1 for c in cu[1:]], dtype=torch.int64, device=dev))
        if chunked:
            max_blk = max(len(self.blocks[sid]) for sid in seq_ids)
            rows = torch.zeros(len(seq_ids), max_blk, dtype=torch.int32)
            for i, sid in enumerate(seq_ids):
                b = self.blocks[sid]
                rows[i, :len(b)] = torch.tensor(b, dtype=torch.int32)
            plan.tables = rows.to(dev)
            plan.context_lens = torch.tensor([self.lengths[sid] for sid in seq_ids], dtype=torch.int32, device=dev)
            plan.total_context = sum(self.lengths[sid] for sid in seq_ids)
            if self.kv_dtype != "bf16":
                run = [0]
                for sid in seq_ids:
                    run.append(run[-1] + self.lengths[sid])
                plan.cu_context = torch.tensor(run, dtype=torch.int32, device=dev)
        return plan

    def _reserve_decode(self, seq_ids):
        """Host side of a decode step: checks, reserves one slot per sequence.  Returns (positions, slots)."""
        B = len(seq_ids)
        if B == 0 or B > self.max_batch:
            raise ValueError(f"batch {B} must be in 1..{self.max_batch}")
        if len(set(seq_ids)) != B:
            raise ValueError("a sequence may appear only once per decode step")
        for s in seq_ids:
            if self.lengths[s] == 0:
                raise ValueError(f"sequence {s} has no tokens; prefill it first")
            if self.lengths[s] + 1 > self.context_length:
                raise ValueError(f"sequence {s} would exceed context_length {self.context_length}")
        need = sum(1 for s in seq_ids if self.lengths[s] % BLOCK == 0)
        if need > self.allocator.num_free:
            raise OutOfBlocks(f"decode step needs {need} blocks, {self.allocator.num_free} free")
        positions = [self.lengths[s] for s in seq_ids]
        slots = [self._reserve(s, 1)[0] for s in seq_ids]
        return positions, slots

    def plan_decode(self, seq_ids) -> DecodePlan:
        """Reserves the slot of one new token for each running sequence in `seq_ids`."""
        B = len(seq_ids)
        positions, slots = self._reserve_decode(seq_ids)
        dev = self.device
        max_len = max(self.lengths[s] for s in seq_ids)
        max_blk = (max_len + BLOCK - 1) // BLOCK
        rows = torch.zeros(B, max_blk, dtype=torch.int32)
        for i, s in enumerate(seq_ids):
            b = self.blocks[s]
            rows[i, :len(b)] = torch.tensor(b, dtype=torch.int32)
        tables = self._tables[:B, :max_blk]
        tables.copy_(rows, non_blocking=False)
        return DecodePlan(torch.tensor(positions, dtype=torch.int32, device=dev),
                          torch.tensor(slots, dtype=torch.int64, device=dev), tables,
                          torch.tensor([p + 1 for p in positions], dtype=torch.int32, device=dev), max_blk * BLOCK)

    def make_static_decode(self, batch: int) -> "StaticDecodeStep":
        """Fixed device tensors for decode steps of `batch` sequences (what a captured HIP graph needs:
        the same addresses and shapes on every replay)."""
        if batch < 1 or batch > self.max_batch:
            raise ValueError(f"batch {batch} must be in 1..{self.max_batch}")
        return StaticDecodeStep(batch, self.max_blocks_per_seq, self.device)

    def plan_decode_into(self, seq_ids, tokens, static: "StaticDecodeStep") -> DecodePlan:
        """plan_decode whose tensors (and the new token ids) are written into `static`: one pinned staging
        buffer, one asynchronous copy on the current stream.  Tables have their full width and
        max_context is the context length, so nothing about the step's shapes depends on the data."""
        B = len(seq_ids)
        if B != static.batch or len(tokens) != B:
            raise ValueError("seq_ids, tokens and the static buffers disagree on the batch size")
        positions, slots = self._reserve_decode(seq_ids)
        static.fill([int(t) for t in tokens], slots, positions, [p + 1 for p in positions],
                    [self.blocks[s] for s in seq_ids])
        return static.plan

    # ---- attention calls (once per layer) -----------------------------------------
    def _write_cache(self, layer: int, plan, q, k, v, k_out=None):
        """RoPE on q and k, rotated k and v into layer `layer`'s cache (quantised when the cache is fp8);
        returns the rotated q -- with k_out=True the pair (rotated q, rotated k in packed form)."""
        kc, vc = self.k_caches[layer], self.v_caches[layer]
        if self.kv_dtype == "bf16":
            return ops.rope_and_cache(q, k, v, plan.positions, self.freq_cache, kc, vc, plan.slots, k_out=k_out)
        return ops.rope_and_cache_fp8(q, k, v, plan.positions, self.freq_cache, kc, vc, self.k_scales[layer],
                                      self.v_scales[layer], plan.slots, k_out=k_out)

    def attend_prefill(self, layer: int, plan: PrefillPlan, q, k, v):
        """q (T,Hq,D), k/v (T,Hkv,D) packed along dim 0 (token strides free, heads contiguous).  Writes
        rotated K and V of layer `layer` into its cache and returns causal attention output (T,Hq,D).
        New sequences attend to the packed tensors themselves (one launch rotates q and k and fills the
        cache); when a sequence already had cached tokens, keys and values are read back through the
        block tables, old and new alike."""
        if q.shape[0] != plan.positions.shape[0]:
            raise ValueError("the plan and the packed tensors disagree on the number of tokens")
        if plan.tables is not None:
            q_rot = self._write_cache(layer, plan, q, k, v)
            scales = {} if self.kv_dtype == "bf16" else {"k_scale": self.k_scales[layer], "v_scale": self.v_scales[layer],
                                                         "total_context": plan.total_context,
                                                         "cu_seqlens_k": plan.cu_context}
            return ops.flash_attn_paged_prefill(q_rot, self.k_caches[layer], self.v_caches[layer], plan.cu_seqlens,
                                                plan.tables, plan.context_lens, plan.max_len, **scales)
        q_rot, k_rot = self._write_cache(layer, plan, q, k, v, k_out=True)
        return ops.flash_attn_varlen_prefill(q_rot, k_rot, v, plan.cu_seqlens, plan.cu_seqlens, plan.max_len,
                                             plan.max_len, causal=True)

    def attend_decode(self, layer: int, plan: DecodePlan, q, k, v):
        """q (B,Hq,D), k/v (B,Hkv,D): appends the token's K/V to layer `layer`'s cache and returns its
        attention output (B,Hq,D)."""
        if q.shape[0] != plan.positions.shape[0]:
            raise ValueError("one query token per sequence expected")
        q_rot = self._write_cache(layer, plan, q, k, v)
        scales = {} if self.kv_dtype == "bf16" else {"k_scale": self.k_scales[layer], "v_scale": self.v_scales[layer]}
        return ops.paged_attention_decode(q_rot, self.k_caches[layer], self.v_caches[layer], plan.tables,
                                          plan.context_lens, max_context=plan.max_context, workspace=self._workspace,
                                          **scales)

    # ---- single-layer convenience ----------------------------------------------------
    def prefill(self, seq_ids, lens, q, k, v):
        """plan_prefill + attend_prefill on layer 0."""
        if sum(lens) != q.shape[0]:
            raise ValueError("sum(lens) must equal the number of packed tokens")
        return self.attend_prefill(0, self.plan_prefill(seq_ids, lens), q, k, v)

    def decode_step(self, seq_ids, q, k, v):
        """plan_decode + attend_decode on layer 0."""
        if q.shape[0] != len(seq_ids):
            raise ValueError("one query token per sequence expected")
        return self.attend_decode(0, self.plan_decode(seq_ids), q, k, v)
