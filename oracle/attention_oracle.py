"""CPU oracle for the attention hot path.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it.  Nothing under the shipped package imports or calls it, and the
shipped ops raise when the HIP library is missing instead of falling back here.

What is restated from the reference (PyTorch, fp32 math):

* ``softmax``                      <- llm-core/llm_core/nn_functional.py:8-11
* ``scaled_dot_product_attention`` <- llm-core/llm_core/model.py:308-325
* ``causal_keep_mask``             <- llm-core/llm_core/model.py:384 (square tril, True = keep)

Everything else in this file (GQA expansion, varlen packing, paged KV gather,
fp8-e4m3 KV quantisation, split-K combine) has NO counterpart in the reference;
each helper reduces its case to the dense function above (gather -> dense ->
``scaled_dot_product_attention``), so the dense function is the single source
of arithmetic truth.

Parity pins (see tests/test_oracle.py): library equivalence with
``torch.nn.functional.scaled_dot_product_attention`` on CPU fp32 (the
equivalence the reference itself relies on at model.py:381-385), closed forms
(one key, identical keys, constant V, Q = 0 -> cumulative mean, dominant
score), invariants (softmax shift, key permutation, block-permutation of the
paged pool, split-count independence of the combine, GQA == MHA on repeated
heads, varlen == per-sequence dense) and an independent float64 triple loop on
tiny shapes.  The reference ships no tests, fixtures or golden vectors, so
there is nothing of its own to check against; no function here is left
"parity unpinned" by the checks above.

Paged KV layout used throughout this repository (defined here, consumed by the
HIP kernels):

    k_cache, v_cache : (num_blocks, num_kv_heads, block_size, head_dim)
    block_tables     : (batch, max_blocks_per_seq) int32, entry j is the physical
                       block holding tokens [j*block_size, (j+1)*block_size)
    context_lens     : (batch,) int32, >= 1
    k_scale, v_scale : (num_blocks, num_kv_heads) float32 (fp8 cache only);
                       real value = fp8 value * scale, scale = absmax / 448
    GQA              : query head h reads kv head h // (Hq // Hkv)
"""
from __future__ import annotations

import math

import numpy as np
import torch

FP8_E4M3_MAX = 448.0


# --------------------------------------------------------------------------
# Restated reference math
# --------------------------------------------------------------------------
def softmax(x: torch.Tensor, dim: int = -1) -> torch.Tensor:
    """Max-subtracted softmax; follows llm-core/llm_core/nn_functional.py:8-11.

    A row that is entirely -inf yields NaN, as in the reference.
    """
    x_max = torch.max(x, dim=dim, keepdim=True)[0]
    e = torch.exp(x - x_max)
    return e / torch.sum(e, dim=dim, keepdim=True)


def scaled_dot_product_attention(Q, K, V, mask=None):
    """softmax(Q K^T / sqrt(d_k) [masked]) V; follows llm-core/llm_core/model.py:308-325.

    Q (..., queries, d_k), K (..., keys, d_k), V (..., keys, d_v); ``mask`` is a
    boolean keep-mask (True = attend) broadcastable to (..., queries, keys).
    The scale is a division applied after the matmul and masked scores become
    -inf through ``where``, exactly as the reference does.  Math runs in the
    dtype of the inputs; callers wanting the fp32 oracle pass fp32 tensors.
    """
    d_k = K.shape[-1]
    scores = torch.matmul(Q, K.transpose(-1, -2)) / math.sqrt(d_k)
    if mask is not None:
        scores = torch.where(mask, scores, float("-inf"))
    weights = softmax(scores, dim=-1)
    return torch.matmul(weights, V)


def causal_keep_mask(n_queries: int, n_keys: int | None = None) -> torch.Tensor:
    """Boolean keep-mask.  Square case == torch.tril(ones) of model.py:384.

    For n_keys > n_queries the queries are the LAST n_queries positions of the
    key sequence (bottom-right alignment): query i keeps key j iff
    j <= i + (n_keys - n_queries).
    """
    n_keys = n_queries if n_keys is None else n_keys
    i = torch.arange(n_queries).unsqueeze(1)
    j = torch.arange(n_keys).unsqueeze(0)
    return j <= i + (n_keys - n_queries)


# --------------------------------------------------------------------------
# Helpers with no reference counterpart (each reduces to the dense function)
# --------------------------------------------------------------------------
def expand_kv_heads(x: torch.Tensor, n_rep: int, head_dim_index: int) -> torch.Tensor:
    """GQA -> MHA: kv head g serves query heads [g*n_rep, (g+1)*n_rep)."""
    return x if n_rep == 1 else torch.repeat_interleave(x, n_rep, dim=head_dim_index)


def _scaled_q(q32: torch.Tensor, softmax_scale: float | None) -> torch.Tensor:
    # The dense function always divides by sqrt(d).  A caller-chosen scale s is
    # expressed by pre-multiplying Q with s*sqrt(d) (scores are linear in Q).
    if softmax_scale is None:
        return q32
    return q32 * (softmax_scale * math.sqrt(q32.shape[-1]))


def prefill_reference(q, k, v, *, causal=True, softmax_scale=None, head_chunk=8):
    """Dense prefill oracle.  q (B,Hq,Sq,D); k,v (B,Hkv,Sk,D) -> (B,Hq,Sq,D) fp32.

    fp32 math on the given (possibly bf16-rounded) inputs.  Heads are processed
    ``head_chunk`` at a time so the score tensor stays small.
    """
    B, Hq, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    assert Hq % Hkv == 0
    n_rep = Hq // Hkv
    mask = causal_keep_mask(Sq, Sk) if causal else None
    out = torch.empty(B, Hq, Sq, v.shape[-1], dtype=torch.float32)
    for b in range(B):
        for h0 in range(0, Hq, head_chunk):
            h1 = min(Hq, h0 + head_chunk)
            kv_idx = torch.arange(h0, h1) // n_rep
            qq = _scaled_q(q[b, h0:h1].float(), softmax_scale)
            kk = k[b, kv_idx].float()
            vv = v[b, kv_idx].float()
            out[b, h0:h1] = scaled_dot_product_attention(qq, kk, vv, mask)
    return out


def varlen_prefill_reference(q, k, v, cu_seqlens_q, cu_seqlens_k, *, causal=True,
                             softmax_scale=None, head_chunk=8):
    """Packed prefill oracle.  q (Tq,Hq,D); k,v (Tk,Hkv,D); cu_seqlens int (B+1,).

    Sequence b owns rows [cu[b], cu[b+1]); result (Tq,Hq,D) fp32 equals the
    dense oracle run on each sequence separately.
    """
    out = torch.empty(q.shape[0], q.shape[1], v.shape[-1], dtype=torch.float32)
    cq = [int(x) for x in cu_seqlens_q]
    ck = [int(x) for x in cu_seqlens_k]
    for b in range(len(cq) - 1):
        if cq[b + 1] == cq[b]:
            continue
        qb = q[cq[b]:cq[b + 1]].transpose(0, 1).unsqueeze(0)
        kb = k[ck[b]:ck[b + 1]].transpose(0, 1).unsqueeze(0)
        vb = v[ck[b]:ck[b + 1]].transpose(0, 1).unsqueeze(0)
        ob = prefill_reference(qb, kb, vb, causal=causal, softmax_scale=softmax_scale,
                               head_chunk=head_chunk)
        out[cq[b]:cq[b + 1]] = ob[0].transpose(0, 1)
    return out


def prefill_backward_reference(q, k, v, dout, *, causal=True, softmax_scale=None):
    """Gradients of prefill_reference w.r.t. q, k, v for an upstream gradient dout, written out by hand
    (fp32): with P = softmax(scale * q k^T [masked]) and out = P v,

        dV = P^T dO,   dP = dO V^T,   dS = P * (dP - rowsum(dP * P)),   dQ = scale * dS K,   dK = scale * dS^T Q

    (rowsum(dP * P) = rowsum(dO * out)).  This is what autograd derives for the reference's
    scaled_dot_product_attention (llm-core/llm_core/model.py:308-325) -- tests/test_oracle.py checks it
    against torch.autograd on that function and against float64 finite differences.  GQA: the gradient of a
    kv head is the sum over its query heads.  q, dout (B,Hq,Sq,D); k, v (B,Hkv,Sk,D).  Also returns lse
    (B,Hq,Sq), the natural-log sum of exp of the scaled, masked scores."""
    B, Hq, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    n_rep = Hq // Hkv
    scale = 1.0 / math.sqrt(D) if softmax_scale is None else softmax_scale
    q32, do32 = q.float(), dout.float()
    k32 = expand_kv_heads(k.float(), n_rep, 1)
    v32 = expand_kv_heads(v.float(), n_rep, 1)
    s = torch.einsum("bhqd,bhkd->bhqk", q32, k32) * scale
    if causal:
        s = torch.where(causal_keep_mask(Sq, Sk), s, float("-inf"))
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse[..., None])
    dv = torch.einsum("bhqk,bhqd->bhkd", p, do32)
    dp = torch.einsum("bhqd,bhkd->bhqk", do32, v32)
    ds = p * (dp - (dp * p).sum(-1, keepdim=True))
    dq = torch.einsum("bhqk,bhkd->bhqd", ds, k32) * scale
    dk = torch.einsum("bhqk,bhqd->bhkd", ds, q32) * scale
    dk = dk.view(B, Hkv, n_rep, Sk, D).sum(2)
    dv = dv.view(B, Hkv, n_rep, Sk, D).sum(2)
    return dq, dk, dv, lse


def gather_paged_kv(cache, block_table_row, context_len, scale=None):
    """(num_blocks,Hkv,bs,D) cache + one block-table row -> (Hkv, context_len, D) fp32.

    With ``scale`` (num_blocks,Hkv) the cache holds fp8-e4m3 values (either
    torch.float8_e4m3fn or its uint8 bit pattern) and is dequantised.
    """
    bs = cache.shape[2]
    nblk = (int(context_len) + bs - 1) // bs
    ids = block_table_row[:nblk].long()
    blocks = cache[ids]
    if blocks.dtype == torch.uint8:
        blocks = blocks.view(torch.float8_e4m3fn)
    blocks = blocks.float()                                  # (nblk,Hkv,bs,D)
    if scale is not None:
        blocks = blocks * scale[ids].float()[:, :, None, None]
    Hkv, D = cache.shape[1], cache.shape[3]
    dense = blocks.permute(1, 0, 2, 3).reshape(Hkv, nblk * bs, D)
    return dense[:, :int(context_len)]


def paged_decode_reference(q, k_cache, v_cache, block_tables, context_lens, *,
                           softmax_scale=None, k_scale=None, v_scale=None):
    """Paged decode oracle: one query token per sequence.  q (B,Hq,D) -> (B,Hq,D) fp32."""
    B, Hq, D = q.shape
    Hkv = k_cache.shape[1]
    n_rep = Hq // Hkv
    out = torch.empty(B, Hq, v_cache.shape[3], dtype=torch.float32)
    for b in range(B):
        kk = gather_paged_kv(k_cache, block_tables[b], context_lens[b], k_scale)
        vv = gather_paged_kv(v_cache, block_tables[b], context_lens[b], v_scale)
        kk = expand_kv_heads(kk, n_rep, 0)
        vv = expand_kv_heads(vv, n_rep, 0)
        qq = _scaled_q(q[b].float(), softmax_scale).unsqueeze(1)          # (Hq,1,D)
        out[b] = scaled_dot_product_attention(qq, kk, vv, None).squeeze(1)
    return out


def paged_prefill_reference(q, k_cache, v_cache, cu_seqlens_q, block_tables, context_lens, *, softmax_scale=None):
    """Chunked-prefill oracle: q (T,Hq,D) packed; sequence b's chunk = rows [cu[b], cu[b+1]) attends to the
    context_lens[b] cached tokens of that sequence (its own included) under the bottom-right aligned causal
    mask -- prefill_reference on the gathered cache rows.  Returns (T,Hq,D) fp32."""
    out = torch.empty(q.shape[0], q.shape[1], v_cache.shape[3], dtype=torch.float32)
    cq = [int(x) for x in cu_seqlens_q]
    for b in range(len(cq) - 1):
        if cq[b + 1] == cq[b]:
            continue
        kk = gather_paged_kv(k_cache, block_tables[b], context_lens[b]).unsqueeze(0)        # (1,Hkv,ctx,D)
        vv = gather_paged_kv(v_cache, block_tables[b], context_lens[b]).unsqueeze(0)
        qb = q[cq[b]:cq[b + 1]].transpose(0, 1).unsqueeze(0)
        ob = prefill_reference(qb, kk, vv, causal=True, softmax_scale=softmax_scale)
        out[cq[b]:cq[b + 1]] = ob[0].transpose(0, 1)
    return out


def quantize_kv_fp8(cache):
    """Per-(block, kv-head) absmax quantisation to OCP fp8-e4m3 (max 448).

    cache (num_blocks,Hkv,bs,D) float -> (uint8 bit patterns, scale (num_blocks,Hkv) fp32)
    with scale = absmax/448 (1.0 for an all-zero block so no division by zero).
    """
    x = cache.float()
    absmax = x.abs().amax(dim=(2, 3))
    scale = torch.where(absmax > 0, absmax / FP8_E4M3_MAX, torch.ones_like(absmax))
    y = (x / scale[:, :, None, None]).clamp(-FP8_E4M3_MAX, FP8_E4M3_MAX)
    q8 = y.to(torch.float8_e4m3fn)
    return q8.view(torch.uint8), scale.contiguous()


def dequantize_kv_fp8(q8, scale):
    return q8.view(torch.float8_e4m3fn).float() * scale[:, :, None, None].float()


def split_partials_reference(q, k, v, bounds, softmax_scale=None):
    """Per-split partial attention of ONE head: q (D,), k,v (ctx,D) fp32.

    Returns a list of (m, l, o) with m = max score of the split, l = sum of
    exp(score - m), o = sum of exp(score - m) * v  (un-normalised).
    """
    d = k.shape[-1]
    s = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(d)
    parts = []
    for lo, hi in bounds:
        sc = (k[lo:hi] @ q) * s
        m = sc.max()
        p = torch.exp(sc - m)
        parts.append((m, p.sum(), p @ v[lo:hi]))
    return parts


def combine_splits_reference(parts):
    """o = sum_i e^{m_i-m} o_i / sum_i e^{m_i-m} l_i with m = max_i m_i."""
    m = torch.stack([p[0] for p in parts]).max()
    num = sum(torch.exp(p[0] - m) * p[2] for p in parts)
    den = sum(torch.exp(p[0] - m) * p[1] for p in parts)
    return num / den


# --------------------------------------------------------------------------
# RoPE + cache write (the step before the path)
# --------------------------------------------------------------------------
def build_rope_cache(context_length, d, theta=10000.0):
    """(2, context_length, d/2) cos/sin table; follows llm-core/llm_core/model.py:86-91."""
    inv_freq = theta ** -(torch.arange(0, d, 2) / d)
    angles = torch.arange(context_length)[:, None] * inv_freq[None, :]
    return torch.stack((torch.cos(angles), torch.sin(angles)))


def rope_reference(x, pos_ids, freq_cache):
    """Interleaved-pair rotation; follows llm-core/llm_core/model.py:93-104.  x (..., seq, d), pos_ids (..., seq)."""
    x1 = x[..., 0::2]
    x2 = x[..., 1::2]
    cos, sin = freq_cache[:, pos_ids, :]
    x1_rot = cos * x1 - sin * x2
    x2_rot = sin * x1 + cos * x2
    return torch.stack((x1_rot, x2_rot), dim=-1).flatten(-2)


def rope_and_cache_reference(q, k, v, positions, freq_cache, k_cache, v_cache, slot_mapping):
    """q (T,Hq,D), k/v (T,Hkv,D): returns rotated q (fp32) and updates fp32 copies of the caches."""
    pos = positions.long()
    q_rot = rope_reference(q.float().transpose(0, 1), pos, freq_cache).transpose(0, 1)
    k_rot = rope_reference(k.float().transpose(0, 1), pos, freq_cache).transpose(0, 1)
    kc, vc = k_cache.float().clone(), v_cache.float().clone()
    bs = kc.shape[2]
    for t in range(q.shape[0]):
        s = int(slot_mapping[t])
        if s < 0:
            continue
        kc[s // bs, :, s % bs] = k_rot[t]
        vc[s // bs, :, s % bs] = v[t].float()
    return q_rot, kc, vc


def _to_e4m3(x, scale):
    return (x / scale).clamp(-FP8_E4M3_MAX, FP8_E4M3_MAX).to(torch.float8_e4m3fn)


def append_rows_fp8(block8, scale, rows, offset):
    """Appends `rows` (n,D) fp32 at row `offset` of ONE (block, head) slab: block8 (16,D) uint8 e4m3, scale a float.

    The slab's scale stays absmax/448 of its valid rows: offset 0 starts afresh (1.0 for all-zero rows,
    as quantize_kv_fp8); otherwise scale' = max(scale, absmax(rows)/448) and, when that raised the scale,
    rows [0, offset) are re-expressed as e4m3((e4m3 value * scale) / scale').  Returns (block8, scale').
    """
    out = block8.clone()
    amax = rows.abs().amax()
    if offset == 0:
        new = amax / FP8_E4M3_MAX if amax > 0 else torch.tensor(1.0)
    else:
        old = torch.tensor(float(scale), dtype=torch.float32)
        new = torch.maximum(old, amax / FP8_E4M3_MAX)
        if float(new) != float(old):
            kept = out[:offset].view(torch.float8_e4m3fn).float() * old
            out[:offset] = _to_e4m3(kept, new).view(torch.uint8)
    out[offset:offset + rows.shape[0]] = _to_e4m3(rows.float(), new).view(torch.uint8)
    return out, float(new)


def rope_and_cache_fp8_reference(q, k, v, positions, freq_cache, k8, k_scale, v8, v_scale, slot_mapping):
    """rope_and_cache_reference with fp8 caches (uint8 e4m3 (nb,Hkv,16,D) + fp32 scales (nb,Hkv)).

    Rotated keys are rounded to bf16 (what a bf16 cache would hold) before quantisation.  Consecutive
    tokens with consecutive slots inside one block form a run and are appended together.
    Returns rotated q (fp32) and updated copies of (k8, k_scale, v8, v_scale).
    """
    pos = positions.long()
    q_rot = rope_reference(q.float().transpose(0, 1), pos, freq_cache).transpose(0, 1)
    k_rot = rope_reference(k.float().transpose(0, 1), pos, freq_cache).transpose(0, 1).to(torch.bfloat16).float()
    k8, v8, k_scale, v_scale = k8.clone(), v8.clone(), k_scale.clone(), v_scale.clone()
    T = q.shape[0]
    t = 0
    while t < T:
        s = int(slot_mapping[t])
        if s < 0 or s >= k8.shape[0] * 16:
            t += 1
            continue
        n = 1
        while t + n < T and (s + n) % 16 != 0 and int(slot_mapping[t + n]) == s + n:
            n += 1
        b, off = s // 16, s % 16
        for h in range(k8.shape[1]):
            k8[b, h], ks = append_rows_fp8(k8[b, h], k_scale[b, h], k_rot[t:t + n, h], off)
            v8[b, h], vs = append_rows_fp8(v8[b, h], v_scale[b, h], v[t:t + n, h].float(), off)
            k_scale[b, h], v_scale[b, h] = ks, vs
        t += n
    return q_rot, k8, k_scale, v8, v_scale


# --------------------------------------------------------------------------
# Independent brute force (float64 loops) used only to pin the functions above
# --------------------------------------------------------------------------
def bruteforce_attention_f64(Q, K, V, keep=None):
    """Triple-loop float64 attention on tiny inputs.  Q (q,d) K (k,d) V (k,dv) numpy."""
    Q = np.asarray(Q, dtype=np.float64)
    K = np.asarray(K, dtype=np.float64)
    V = np.asarray(V, dtype=np.float64)
    nq, d = Q.shape
    nk = K.shape[0]
    out = np.zeros((nq, V.shape[1]), dtype=np.float64)
    for i in range(nq):
        sc = []
        for j in range(nk):
            if keep is not None and not keep[i][j]:
                sc.append(None)
                continue
            acc = 0.0
            for t in range(d):
                acc += Q[i, t] * K[j, t]
            sc.append(acc / math.sqrt(d))
        live = [x for x in sc if x is not None]
        mx = max(live)
        den = sum(math.exp(x - mx) for x in live)
        for j in range(nk):
            if sc[j] is None:
                continue
            w = math.exp(sc[j] - mx) / den
            for t in range(V.shape[1]):
                out[i, t] += w * V[j, t]
    return out


# --------------------------------------------------------------------------
# Seeded synthetic workloads (the configurations the benchmark names)
# --------------------------------------------------------------------------
def make_paged_case(*, batch, n_q_heads, n_kv_heads, head_dim, block_size, context_lens,
                    pool_factor=1.0, seed=0, dtype=torch.float32, min_pool_blocks=0):
    """Build q, paged K/V pools and a block table from a seed (CPU tensors).

    Physical blocks are a seeded random permutation of the pool; the first
    sum(blocks_i) ids are dealt to the sequences in order.  Pool blocks outside
    every table are filled with random data too (they must not matter).
    """
    g = torch.Generator().manual_seed(seed)
    ctx = torch.as_tensor(context_lens, dtype=torch.int32)
    assert ctx.numel() == batch
    nblk = (ctx + block_size - 1) // block_size
    total = int(nblk.sum())
    pool = max(int(math.ceil(total * pool_factor)), min_pool_blocks, total)
    perm = torch.randperm(pool, generator=g)
    max_blk = int(nblk.max())
    bt = torch.zeros(batch, max_blk, dtype=torch.int32)
    off = 0
    for b in range(batch):
        n = int(nblk[b])
        bt[b, :n] = perm[off:off + n].to(torch.int32)
        off += n
    q = torch.randn(batch, n_q_heads, head_dim, generator=g).to(dtype)
    shape = (pool, n_kv_heads, block_size, head_dim)
    if dtype == torch.float32:
        k_cache = torch.randn(shape, generator=g)
        v_cache = torch.randn(shape, generator=g)
    else:
        # large pools: generate per slab to bound peak fp32 memory
        k_cache = torch.empty(shape, dtype=dtype)
        v_cache = torch.empty(shape, dtype=dtype)
        step = max(1, (1 << 26) // (n_kv_heads * block_size * head_dim))
        for s in range(0, pool, step):
            e = min(pool, s + step)
            k_cache[s:e] = torch.randn((e - s,) + shape[1:], generator=g).to(dtype)
            v_cache[s:e] = torch.randn((e - s,) + shape[1:], generator=g).to(dtype)
    return q, k_cache, v_cache, bt, ctx


def draw_context_lens(kind, batch, lo, hi, seed):
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
