"""Seeded synthetic inputs of the benchmark configurations (built on the GPU).

Config numbering follows the benchmark definition:
  1  prefill  bf16 dense   B4  H16/16 D64  S1024
  2  prefill  bf16 packed  B8  H32/8  D128 S4096 (cu_seqlens all 4096)
  3  decode   bf16 KV      B128 H32/8 D128 block 16, ctx ~ U[512, 16384]
  4  decode   fp8 KV       B256 H64/8 D128 block 16, ctx log-uniform [128, 32768]
  0  decode   bf16 KV      B4   H8/8  D64  block 16, ctx 256 (the small CPU-path shape)
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch

BLOCK = 16
FP8_MAX = 448.0


@dataclass
class DecodeCase:
    q: torch.Tensor
    k_cache: torch.Tensor
    v_cache: torch.Tensor
    block_tables: torch.Tensor
    context_lens: torch.Tensor
    k_scale: torch.Tensor | None
    v_scale: torch.Tensor | None
    max_context: int
    context_lens_host: torch.Tensor
    # fp8 cases only: the bf16 blocks (before quantisation) of the first `bf16_sample_seqs` sequences, in table
    # order, so that the quantisation error can be measured against a bf16-KV reference
    k_bf16_sample: torch.Tensor | None = None
    v_bf16_sample: torch.Tensor | None = None
    bf16_sample_seqs: int = 0

    @property
    def tokens(self) -> int:
        return int(self.context_lens_host.sum())

    def algorithmic_bytes(self) -> int:
        """KV bytes of the tokens actually attended + scales + q/out + the block-table entries used."""
        nb, hkv, bs, d = self.k_cache.shape
        kv_elem = self.k_cache.element_size()
        per_token = 2 * hkv * d * kv_elem
        blocks = int(((self.context_lens_host + bs - 1) // bs).sum())
        total = self.tokens * per_token + 2 * self.q.numel() * self.q.element_size() + 4 * blocks
        if self.k_scale is not None:
            total += blocks * 2 * hkv * 4
        return total

    def flops(self) -> int:
        return 4 * self.q.shape[1] * self.q.shape[2] * self.tokens


def draw_context_lens(kind: str, batch: int, lo: int, hi: int, seed: int) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed + 1000003)
    if kind == "fixed":
        return torch.full((batch,), hi, dtype=torch.int32)
    if kind == "uniform":
        return torch.randint(lo, hi + 1, (batch,), generator=g).to(torch.int32)
    if kind == "loguniform":
        u = torch.rand(batch, generator=g, dtype=torch.float64)
        x = torch.exp(math.log(lo) + u * (math.log(hi) - math.log(lo)))
        return torch.round(x).clamp(lo, hi).to(torch.int32)
    raise ValueError(kind)


def quantize_kv_fp8_(cache_bf16: torch.Tensor):
    """Per-(block, kv head) absmax quantisation to OCP e4m3 on the GPU; returns (uint8 cache, fp32 scales)."""
    nb = cache_bf16.shape[0]
    out = torch.empty(cache_bf16.shape, dtype=torch.uint8, device=cache_bf16.device)
    scale = torch.empty(cache_bf16.shape[:2], dtype=torch.float32, device=cache_bf16.device)
    step = max(1, (1 << 27) // (cache_bf16[0].numel()))
    for s in range(0, nb, step):
        x = cache_bf16[s:s + step].float()
        amax = x.abs().amax(dim=(2, 3))
        sc = torch.where(amax > 0, amax / FP8_MAX, torch.ones_like(amax))
        y = (x / sc[:, :, None, None]).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
        out[s:s + step] = y.view(torch.uint8)
        scale[s:s + step] = sc
    return out, scale


def make_decode_case(*, batch, n_q_heads, n_kv_heads, head_dim, ctx_kind, ctx_lo, ctx_hi, pool_factor, seed,
                     fp8=False, keep_bf16_seqs=0, device="cuda:0") -> DecodeCase:
    ctx = draw_context_lens(ctx_kind, batch, ctx_lo, ctx_hi, seed)
    nblk = (ctx + BLOCK - 1) // BLOCK
    total = int(nblk.sum())
    pool = max(int(math.ceil(total * pool_factor)), total)
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(pool, generator=g)
    max_blk = int(nblk.max())
    bt = torch.zeros(batch, max_blk, dtype=torch.int32)
    off = 0
    for b in range(batch):
        n = int(nblk[b])
        bt[b, :n] = perm[off:off + n].to(torch.int32)
        off += n
    gd = torch.Generator(device=device).manual_seed(seed)
    q = torch.randn(batch, n_q_heads, head_dim, generator=gd, device=device).to(torch.bfloat16)
    shape = (pool, n_kv_heads, BLOCK, head_dim)
    kc = torch.empty(shape, dtype=torch.bfloat16, device=device)
    vc = torch.empty(shape, dtype=torch.bfloat16, device=device)
    step = max(1, (1 << 27) // (n_kv_heads * BLOCK * head_dim))
    for s in range(0, pool, step):
        e = min(pool, s + step)
        kc[s:e] = torch.randn((e - s,) + shape[1:], generator=gd, device=device).to(torch.bfloat16)
        vc[s:e] = torch.randn((e - s,) + shape[1:], generator=gd, device=device).to(torch.bfloat16)
    ks = vs = k_keep = v_keep = None
    if fp8:
        keep_bf16_seqs = min(keep_bf16_seqs, batch)
        if keep_bf16_seqs:
            ids = torch.cat([bt[b, :int(nblk[b])] for b in range(keep_bf16_seqs)]).long().to(device)
            k_keep, v_keep = kc[ids], vc[ids]
        kc, ks = quantize_kv_fp8_(kc)
        vc, vs = quantize_kv_fp8_(vc)
    return DecodeCase(q, kc, vc, bt.to(device), ctx.to(device), ks, vs, max_blk * BLOCK, ctx, k_keep, v_keep,
                      keep_bf16_seqs if fp8 else 0)


def decode_config(cfg: int, seed: int = 0, device="cuda:0", keep_bf16_seqs: int = 0) -> DecodeCase:
    if cfg == 0:
        return make_decode_case(batch=4, n_q_heads=8, n_kv_heads=8, head_dim=64, ctx_kind="fixed", ctx_lo=256,
                                ctx_hi=256, pool_factor=1.0, seed=seed, device=device)
    if cfg == 3:
        return make_decode_case(batch=128, n_q_heads=32, n_kv_heads=8, head_dim=128, ctx_kind="uniform", ctx_lo=512,
                                ctx_hi=16384, pool_factor=1.1, seed=seed, device=device)
    if cfg == 4:
        return make_decode_case(batch=256, n_q_heads=64, n_kv_heads=8, head_dim=128, ctx_kind="loguniform",
                                ctx_lo=128, ctx_hi=32768, pool_factor=1.1, seed=seed, fp8=True,
                                keep_bf16_seqs=keep_bf16_seqs, device=device)
    raise ValueError(f"config {cfg} is not a decode configuration")


@dataclass
class PrefillCase:
    q: torch.Tensor
    k: torch.Tensor
    v: torch.Tensor
    cu_seqlens: torch.Tensor | None
    seqlen: int
    batch: int

    def flops(self) -> int:
        """FlashAttention convention for causal attention: half of 4*B*H*S^2*D."""
        hq, d = self.q.shape[-3] if self.cu_seqlens is None else self.q.shape[1], self.q.shape[-1]
        return 4 * self.batch * hq * d * self.seqlen * self.seqlen // 2

    def algorithmic_bytes(self) -> int:
        return (2 * self.q.numel() + self.k.numel() + self.v.numel()) * 2


def prefill_config(cfg: int, seed: int = 0, device="cuda:0") -> PrefillCase:
    gd = torch.Generator(device=device).manual_seed(seed)

    def rnd(*shape):
        return (torch.randn(*shape, generator=gd, device=device) * 0.5).to(torch.bfloat16)

    if cfg == 1:
        B, H, S, D = 4, 16, 1024, 64
        return PrefillCase(rnd(B, H, S, D), rnd(B, H, S, D), rnd(B, H, S, D), None, S, B)
    if cfg == 2:
        B, Hq, Hkv, S, D = 8, 32, 8, 4096, 128
        cu = (torch.arange(B + 1, dtype=torch.int32) * S).to(device)
        return PrefillCase(rnd(B * S, Hq, D), rnd(B * S, Hkv, D), rnd(B * S, Hkv, D), cu, S, B)
    raise ValueError(f"config {cfg} is not a prefill configuration")
