"""Host-side operators: argument checking, output allocation, C-ABI calls.

Tensor conventions follow the reference attention module
(llm-core/llm_core/model.py:366-388): Q/K/V are (batch, heads, seq, d_head) with
arbitrary batch/head/seq strides (the reference's V is a strided view of the
(batch, seq, heads*d_head) projection) and a unit innermost stride.
"""
from __future__ import annotations

import math

import torch

from . import _lib

_BLOCK = 16


class _on:
    """`with _on(t0, t1, ...) as stream:` -- checks that every given tensor lives on one GPU, makes that GPU
    the current device for the launch and yields its current stream (as the integer the C ABI takes)."""

    def __init__(self, *tensors):
        ts = [t for t in tensors if t is not None]
        self.device = ts[0].device
        for t in ts:
            if t.device != self.device:
                raise ValueError(f"all tensors of one call must be on one device (got {self.device} and {t.device})")
        if self.device.type != "cuda":
            raise ValueError(f"tensors must live on the GPU (got {self.device}); this library has no CPU path")
        self._guard = torch.cuda.device(self.device)

    def __enter__(self):
        self._guard.__enter__()
        return torch.cuda.current_stream(self.device).cuda_stream

    def __exit__(self, *exc):
        return self._guard.__exit__(*exc)


def _require_gpu_bf16(name, t):
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got {t.device}); this library has no CPU path")
    if t.dtype != torch.bfloat16:
        raise TypeError(f"{name} must be bfloat16 (got {t.dtype})")


def _autocast_on() -> bool:
    try:
        return torch.is_autocast_enabled("cuda")
    except TypeError:                      # older signature without a device type
        return torch.is_autocast_enabled()


def _to_bf16(q, k, v):
    """The kernels compute on bf16 operands.  Inputs may be bfloat16 or float32 in any mix -- at
    llm-core/llm_core/model.py:382 the reference passes float32 Q and K (RoPE multiplies the bf16 projections by its
    float32 table, model.py:93-104) with a bfloat16 V under `--amp` (train.py:215), and three float32 tensors
    without it.  float32 inputs are rounded to bf16 (what autocast does to them in front of PyTorch's SDPA; the cast
    is differentiable).  Returns (q, k, v, out_dtype): float32 only when all three inputs are float32 and autocast
    is off -- the case in which the reference's next operator expects float32 -- bfloat16 otherwise."""
    for n, t in (("q", q), ("k", k), ("v", v)):
        if not t.is_cuda:
            raise ValueError(f"{n} must live on the GPU (got {t.device}); this library has no CPU path")
        if t.dtype not in (torch.bfloat16, torch.float32):
            raise TypeError(f"{n} must be bfloat16 or float32 (got {t.dtype})")
    all_f32 = all(t.dtype == torch.float32 for t in (q, k, v))
    out_dtype = torch.float32 if all_f32 and not _autocast_on() else torch.bfloat16
    q, k, v = (t if t.dtype == torch.bfloat16 else t.to(torch.bfloat16) for t in (q, k, v))
    return q, k, v, out_dtype


def _rows16(name, t):
    """Return `t` with unit innermost stride and 16-byte aligned rows (copy only if needed)."""
    ok = t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in t.stride()[:-1])
    return t if ok else t.contiguous()


def _packed_or_dense_strides(t, packed):
    """[batch, head, row] element strides of a (B,H,S,D) tensor, or of a packed (T,H,D) one (batch unused)."""
    return (0, t.stride(1), t.stride(0)) if packed else t.stride()[:3]


_N_CU = {}


def suggest_kv_splits(B, Hq, D, sq_max, sk_max, total_rows, causal, device):
    """The library's suggestion for this shape (mi355_prefill_suggest_kv_splits: a cost model of tile-loop time
    saved against the traffic of the partial rows); 1 = do not split."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if idx not in _N_CU:
        _N_CU[idx] = torch.cuda.get_device_properties(idx).multi_processor_count
    return _lib.load().mi355_prefill_suggest_kv_splits(int(B), int(Hq), int(D), int(sq_max), int(sk_max),
                                                       int(total_rows), 1 if causal else 0, _N_CU[idx])


def prefill_splitkv_workspace(total_q_rows, n_q_heads, head_dim, kv_splits, device):
    """Scratch tensor for a prefill call with kv_splits > 1 (fp32 partial rows and their log-sum-exps)."""
    n = _lib.load().mi355_prefill_splitkv_workspace_bytes(int(total_q_rows), n_q_heads, head_dim, int(kv_splits))
    return torch.empty(max(int(n), 16), dtype=torch.uint8, device=device)


def _split_args(kv_splits, workspace, B, Hq, D, sq_max, sk_max, total_rows, causal, device):
    """(n_split, workspace) for a forward-only prefill call; kv_splits None = choose."""
    n = suggest_kv_splits(B, Hq, D, sq_max, sk_max, total_rows, causal, device) if kv_splits is None else int(kv_splits)
    if n < 1 or n > 64:
        raise ValueError("kv_splits must be in 1..64")
    if n == 1:
        return 1, None
    if workspace is None:
        workspace = prefill_splitkv_workspace(total_rows, Hq, D, n, device)
    return n, workspace


def _prefill(q, k, v, out, cu_q, cu_k, mask, B, Hq, Hkv, Sq, Sk, D, scale, mode, lse=None, n_split=1, workspace=None,
             total_rows=0):
    lib = _lib.load()
    if n_split > 1:
        packed = cu_q is not None
        qs, ks, vs, os_ = (_packed_or_dense_strides(x, packed) for x in (q, k, v, out))
        with _on(q, k, v, out, cu_q, cu_k, workspace) as stream:
            rc = lib.mi355_prefill_fwd_splitkv(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                _lib.strides3(qs), _lib.strides3(ks), _lib.strides3(vs), _lib.strides3(os_),
                None if cu_q is None else cu_q.data_ptr(), None if cu_k is None else cu_k.data_ptr(),
                B, Hq, Hkv, Sq, Sk, D, float(scale), mode, _lib.MI355_BF16, int(n_split), int(total_rows),
                workspace.data_ptr(), workspace.numel() * workspace.element_size(), stream)
        _lib.check(rc, "mi355_prefill_fwd_splitkv")
        return
    if lse is not None and mask is not None:
        qs, ks, vs, os_ = (x.stride()[:3] for x in (q, k, v, out))
        with _on(q, k, v, out, lse, mask) as stream:
            rc = lib.mi355_prefill_fwd_mask_lse(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
                _lib.strides3(qs), _lib.strides3(ks), _lib.strides3(vs), _lib.strides3(os_), _lib.strides2(lse.stride()[:2]),
                mask.data_ptr(), _lib.strides3(mask.stride()[:3]), B, Hq, Hkv, Sq, Sk, D, float(scale), _lib.MI355_BF16, stream)
        _lib.check(rc, "mi355_prefill_fwd_mask_lse")
        return
    if lse is not None:
        packed = cu_q is not None
        qs, ks, vs, os_ = (_packed_or_dense_strides(x, packed) for x in (q, k, v, out))
        ls = (0, lse.stride(0)) if packed else lse.stride()[:2]
        with _on(q, k, v, out, lse, cu_q, cu_k) as stream:
            rc = lib.mi355_prefill_fwd_lse(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
                _lib.strides3(qs), _lib.strides3(ks), _lib.strides3(vs), _lib.strides3(os_), _lib.strides2(ls),
                None if cu_q is None else cu_q.data_ptr(), None if cu_k is None else cu_k.data_ptr(),
                B, Hq, Hkv, Sq, Sk, D, float(scale), mode, _lib.MI355_BF16, stream)
        _lib.check(rc, "mi355_prefill_fwd_lse")
        return
    if cu_q is None:
        qs, ks, vs, os_ = (x.stride()[:3] for x in (q, k, v, out))
    else:   # packed (T, H, D): [batch (unused), head, row]
        qs, ks, vs, os_ = ((0, x.stride(1), x.stride(0)) for x in (q, k, v, out))
    ms = (0, 0, 0) if mask is None else mask.stride()[:3]
    with _on(q, k, v, out, cu_q, cu_k, mask) as stream:
        rc = lib.mi355_prefill_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
            _lib.strides3(qs), _lib.strides3(ks), _lib.strides3(vs), _lib.strides3(os_),
            None if cu_q is None else cu_q.data_ptr(), None if cu_k is None else cu_k.data_ptr(),
            None if mask is None else mask.data_ptr(), _lib.strides3(ms),
            B, Hq, Hkv, Sq, Sk, D, float(scale), mode, _lib.MI355_BF16, stream)
    _lib.check(rc, "mi355_prefill_fwd")


def _dense(q, k, v, mask, mode, softmax_scale, want_lse=False, kv_splits=1, workspace=None):
    for n, t in (("q", q), ("k", k), ("v", v)):
        _require_gpu_bf16(n, t)
        if t.dim() != 4:
            raise ValueError(f"{n} must be (batch, heads, seq, d_head), got {tuple(t.shape)}")
    B, Hq, Sq, D = q.shape
    Bk, Hkv, Sk, Dk = k.shape
    if (Bk, Dk) != (B, D) or tuple(v.shape) != (B, Hkv, Sk, D):
        raise ValueError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)}")
    if Hq % Hkv:
        raise ValueError("query heads must be a multiple of kv heads")
    q, k, v = _rows16("q", q), _rows16("k", k), _rows16("v", v)
    scale = 1.0 / math.sqrt(D) if softmax_scale is None else softmax_scale
    # (B, S, H, D) memory returned as its (B, H, S, D) view: merging heads afterwards
    # (model.py:388) is then a free reshape instead of a copy.
    out = torch.empty(B, Sq, Hq, D, dtype=q.dtype, device=q.device).permute(0, 2, 1, 3)
    lse = torch.empty(B, Hq, Sq, dtype=torch.float32, device=q.device) if want_lse else None
    if B == 0 or Sq == 0:
        return (out, lse) if want_lse else out
    if Sk == 0:
        raise ValueError("attention over zero keys is undefined")
    n_split, workspace = (1, None) if (want_lse or mask is not None) else _split_args(
        kv_splits, workspace, B, Hq, D, Sq, Sk, B * Sq, mode == _lib.MASK_CAUSAL, q.device)
    _prefill(q, k, v, out, None, None, mask, B, Hq, Hkv, Sq, Sk, D, scale, mode, lse, n_split, workspace, B * Sq)
    return (out, lse) if want_lse else out


def _grad_like(t):
    """Gradient buffer with t's shape and, where t is dense, t's memory layout (so the gradient of the
    reference's strided V view lands in the layout of the projection it is a view of)."""
    g = torch.empty_like(t)
    ok = g.stride(-1) == 1 and all(s % 8 == 0 for s in g.stride()[:-1])
    return g if ok else torch.empty(t.shape, dtype=t.dtype, device=t.device)


def _prefill_backward(q, k, v, out, dout, lse, cu_q, cu_k, Sq, Sk, scale, mode, mask=None):
    """dq, dk, dv through mi355_prefill_bwd (mi355_prefill_bwd_mask with an explicit (B,H,Sq,Sk) uint8 mask);
    tensors dense (B,H,S,D) or packed (T,H,D)."""
    packed = cu_q is not None
    q, k, v, out, dout = (_rows16(n, t) for n, t in (("q", q), ("k", k), ("v", v), ("out", out), ("dout", dout)))
    dq, dk, dv = _grad_like(q), _grad_like(k), _grad_like(v)
    if q.numel() == 0 or k.numel() == 0:
        return dq.zero_(), dk.zero_(), dv.zero_()
    delta = torch.empty_like(lse)
    if packed:
        B, (_, Hq, D), Hkv = cu_q.numel() - 1, q.shape, k.shape[1]
        ls = (0, lse.stride(0))
    else:
        (B, Hq, _, D), Hkv = q.shape, k.shape[1]
        ls = lse.stride()[:2]
    st = [_lib.strides3(_packed_or_dense_strides(t, packed)) for t in (q, k, v, out, dout, dq, dk, dv)]
    if mask is not None:
        with _on(q, k, v, out, dout, lse, mask) as stream:
            rc = _lib.load().mi355_prefill_bwd_mask(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), dout.data_ptr(), lse.data_ptr(), delta.data_ptr(),
                dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), *st, _lib.strides2(ls), mask.data_ptr(),
                _lib.strides3(mask.stride()[:3]), B, Hq, Hkv, int(Sq), int(Sk), D, float(scale), _lib.MI355_BF16, stream)
        _lib.check(rc, "mi355_prefill_bwd_mask")
        return dq, dk, dv
    with _on(q, k, v, out, dout, lse, cu_q, cu_k) as stream:
        rc = _lib.load().mi355_prefill_bwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), dout.data_ptr(), lse.data_ptr(), delta.data_ptr(),
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), *st, _lib.strides2(ls),
            None if cu_q is None else cu_q.data_ptr(), None if cu_k is None else cu_k.data_ptr(),
            B, Hq, Hkv, int(Sq), int(Sk), D, float(scale), mode, _lib.MI355_BF16, stream)
    _lib.check(rc, "mi355_prefill_bwd")
    return dq, dk, dv


class _DensePrefillFn(torch.autograd.Function):
    """out = attention(q, k, v) on the HIP forward; backward on the HIP backward kernels."""

    @staticmethod
    def forward(ctx, q, k, v, causal, softmax_scale):
        mode = _lib.MASK_CAUSAL if causal else _lib.MASK_NONE
        out, lse = _dense(q, k, v, None, mode, softmax_scale, want_lse=True)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.mode = mode
        ctx.scale = 1.0 / math.sqrt(q.shape[-1]) if softmax_scale is None else softmax_scale
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse = ctx.saved_tensors
        dq, dk, dv = _prefill_backward(q, k, v, out, dout, lse, None, None, q.shape[2], k.shape[2], ctx.scale, ctx.mode)
        return dq, dk, dv, None, None


def _mask_words(m4):
    """A (B|1, H|1, Sq, Sk) uint8 keep-mask as the backward kernel reads it: four keys per 32-bit word, so rows,
    strides and the base address are multiples of 4 bytes and a row is readable up to the next multiple of 4 past Sk.
    Broadcast dimensions (stride 0) stay broadcast; anything else that does not fit is copied into padded rows."""
    nk = m4.shape[-1]
    st = m4.stride()
    if m4.data_ptr() % 4 == 0 and nk % 4 == 0 and st[3] == 1 and all(x % 4 == 0 for x in st[:3]):
        return m4
    lead = [1 if st[i] == 0 else m4.shape[i] for i in range(2)]
    buf = torch.zeros(*lead, m4.shape[2], (nk + 3) // 4 * 4, dtype=torch.uint8, device=m4.device)
    buf[..., :nk] = m4[:lead[0], :lead[1]]
    return buf[..., :nk].expand(m4.shape)


class _MaskedPrefillFn(torch.autograd.Function):
    """out = attention(q, k, v) under an explicit keep-mask (the call of model.py:384-385): the masked forward that
    also writes the log-sum-exp, and the backward kernels in their explicit-mask mode."""

    @staticmethod
    def forward(ctx, q, k, v, m4):
        out, lse = _dense(q, k, v, m4, _lib.MASK_BOOL, None, want_lse=True)
        ctx.save_for_backward(q, k, v, out, lse, m4)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse, m4 = ctx.saved_tensors
        dq, dk, dv = _prefill_backward(q, k, v, out, dout, lse, None, None, q.shape[2], k.shape[2],
                                       1.0 / math.sqrt(q.shape[-1]), _lib.MASK_BOOL, mask=m4)
        return dq, dk, dv, None


class _VarlenPrefillFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, cu_q, cu_k, max_q, max_k, causal, softmax_scale):
        out, lse = _varlen(q, k, v, cu_q, cu_k, max_q, max_k, causal, softmax_scale, want_lse=True)
        ctx.save_for_backward(q, k, v, out, lse, cu_q, cu_k)
        ctx.args = (int(max_q), int(max_k), _lib.MASK_CAUSAL if causal else _lib.MASK_NONE,
                    1.0 / math.sqrt(q.shape[-1]) if softmax_scale is None else softmax_scale)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse, cu_q, cu_k = ctx.saved_tensors
        max_q, max_k, mode, scale = ctx.args
        dq, dk, dv = _prefill_backward(q, k, v, out, dout, lse, cu_q, cu_k, max_q, max_k, scale, mode)
        return dq, dk, dv, None, None, None, None, None, None


def _needs_grad(*tensors):
    return torch.is_grad_enabled() and any(t.requires_grad for t in tensors)


def flash_attn_prefill(q, k, v, *, causal=True, softmax_scale=None, kv_splits=None, workspace=None):
    """Prefill forward.  q (B,Hq,Sq,D); k, v (B,Hkv,Sk,D) -> (B,Hq,Sq,D).

    Fills the slot of torch.nn.functional.scaled_dot_product_attention(Q, K, V,
    is_causal=True) at llm-core/llm_core/model.py:382.  With Sk > Sq the causal
    diagonal is bottom-right aligned (the queries are the last Sq positions).
    Inputs are bfloat16 or float32 in any mix (see _to_bf16: bf16 math either way; the result is
    float32 only for three float32 inputs outside autocast, bfloat16 otherwise).
    Differentiable: when an input requires grad, dq/dk/dv come from the HIP backward kernels
    (what autograd computes behind model.py:382 during train.py's loss.backward()).
    kv_splits (forward-only calls): split every sequence's keys over that many workgroups and merge the
    partial results (mi355_prefill_fwd_splitkv) -- for few query rows over many keys, where one workgroup
    per pair of 256-row query tiles would leave most of the GPU idle.  None chooses (1 whenever the plain
    launch already fills the GPU); `workspace` may carry a prefill_splitkv_workspace() tensor to reuse.
    """
    q, k, v, out_dtype = _to_bf16(q, k, v)
    if _needs_grad(q, k, v):
        out = _DensePrefillFn.apply(q, k, v, bool(causal), softmax_scale)
    else:
        out = _dense(q, k, v, None, _lib.MASK_CAUSAL if causal else _lib.MASK_NONE, softmax_scale,
                     kv_splits=kv_splits, workspace=workspace)
    return out if out.dtype == out_dtype else out.to(out_dtype)


def sdpa_slot(Q, K, V, is_causal=True):
    """Callable with the exact call shape used at llm-core/llm_core/model.py:382."""
    return flash_attn_prefill(Q, K, V, causal=is_causal)


def scaled_dot_product_attention(Q, K, V, mask=None):
    """Same signature and semantics as llm-core/llm_core/model.py:308-325.

    Q (..., queries, d_k), K (..., keys, d_k), V (..., keys, d_v); `mask` is a
    boolean keep-mask (True = attend) broadcastable to (..., queries, keys); the
    scale is 1/sqrt(d_k).  A query row whose keys are all masked yields NaN, as
    the reference softmax (llm-core/llm_core/nn_functional.py:8-11) does.
    Restrictions of the HIP path: d_v == d_k in {32, 64, 128}; bfloat16 or float32 tensors (bf16 math, see
    _to_bf16).  Differentiable with and without a mask (dq/dk/dv from the HIP backward kernels), so the reference's
    non-flash training branch (model.py:384-385: the tril mask rebuilt per call) runs through it unchanged; the
    explicit-mask kernels read the mask element by element, so flash_attn_prefill(causal=True) remains the fast way
    to train with a causal mask.  A fully masked query row gives NaN outputs like the reference but zero gradients
    (the reference propagates the NaN).
    """
    if Q.dim() < 2 or K.dim() != Q.dim() or V.dim() != Q.dim():
        raise ValueError("Q, K and V need the same number of dimensions (>= 2)")
    lead = torch.broadcast_shapes(Q.shape[:-2], K.shape[:-2], V.shape[:-2])
    nq, nk, d = Q.shape[-2], K.shape[-2], Q.shape[-1]
    if mask is not None:
        if mask.dtype != torch.bool:
            raise TypeError("mask must be a boolean keep-mask")
        lead = torch.broadcast_shapes(lead, mask.shape[:-2])

    def as4(t, rows):
        t = t.expand(*lead, rows, t.shape[-1])
        if t.dim() == 4:
            return t
        if t.dim() < 4:
            return t.reshape((1,) * (4 - t.dim()) + tuple(t.shape))
        return t.reshape(-1, *t.shape[-3:])

    Q, K, V, out_dtype = _to_bf16(Q, K, V)
    q4, k4, v4 = as4(Q, nq), as4(K, nk), as4(V, nk)
    m4 = None
    mode = _lib.MASK_NONE
    if mask is not None:
        m4 = as4(mask.expand(*mask.shape[:-2], nq, nk), nq).view(torch.uint8)
        if m4.stride(-1) != 1:
            m4 = m4.contiguous()
        mode = _lib.MASK_BOOL
    if _needs_grad(Q, K, V):
        if mask is not None:
            out = _MaskedPrefillFn.apply(q4, k4, v4, _mask_words(m4))
        else:
            out = _DensePrefillFn.apply(q4, k4, v4, False, None)
        return out.reshape(*lead, nq, d).to(out_dtype)
    out = _dense(q4, k4, v4, m4, mode, None, kv_splits=None)
    return out.reshape(*lead, nq, d).to(out_dtype)


def _varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, causal, softmax_scale, want_lse=False,
            kv_splits=1, workspace=None):
    for n, t in (("q", q), ("k", k), ("v", v)):
        _require_gpu_bf16(n, t)
        if t.dim() != 3:
            raise ValueError(f"{n} must be (tokens, heads, d_head), got {tuple(t.shape)}")
    for n, c in (("cu_seqlens_q", cu_seqlens_q), ("cu_seqlens_k", cu_seqlens_k)):
        if c.dtype != torch.int32 or not c.is_cuda or c.dim() != 1 or not c.is_contiguous():
            raise TypeError(f"{n} must be a contiguous 1-D int32 GPU tensor")
    if cu_seqlens_q.numel() != cu_seqlens_k.numel() or cu_seqlens_q.numel() < 2:
        raise ValueError("cu_seqlens_q and cu_seqlens_k must both have batch+1 entries")
    Tq, Hq, D = q.shape
    Tk, Hkv, Dk = k.shape
    if Dk != D or tuple(v.shape) != (Tk, Hkv, D) or Hq % Hkv:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)}")
    q, k, v = _rows16("q", q), _rows16("k", k), _rows16("v", v)
    B = cu_seqlens_q.numel() - 1
    # max_seqlen_* are the caller's promise about the longest sequence (they are on the host, the lengths are not).
    # What can be checked without reading device memory is checked here; a sequence longer than the promise is
    # still computed in full by the kernel (its workgroups walk on through the remaining query tiles).
    max_seqlen_q, max_seqlen_k = int(max_seqlen_q), int(max_seqlen_k)
    if (Tq and max_seqlen_q < 1) or (Tk and max_seqlen_k < 1):
        raise ValueError("max_seqlen_q and max_seqlen_k must be at least 1 when there are tokens")
    scale = 1.0 / math.sqrt(D) if softmax_scale is None else softmax_scale
    out = torch.empty(Tq, Hq, D, dtype=q.dtype, device=q.device)
    lse = torch.empty(Hq, Tq, dtype=torch.float32, device=q.device) if want_lse else None
    if Tq and max_seqlen_q:
        n_split, workspace = (1, None) if want_lse else _split_args(
            kv_splits, workspace, B, Hq, D, max_seqlen_q, max_seqlen_k, Tq, causal, q.device)
        _prefill(q, k, v, out, cu_seqlens_q, cu_seqlens_k, None, B, Hq, Hkv, int(max_seqlen_q), int(max_seqlen_k),
                 D, scale, _lib.MASK_CAUSAL if causal else _lib.MASK_NONE, lse, n_split, workspace, Tq)
    return (out, lse) if want_lse else out


def flash_attn_varlen_prefill(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, *,
                              causal=True, softmax_scale=None, kv_splits=None, workspace=None):
    """Packed ("varlen") prefill.  q (Tq,Hq,D); k, v (Tk,Hkv,D) bf16; cu_seqlens int32 (B+1,), cu[0]=0.

    Sequence b owns rows [cu[b], cu[b+1]).  Returns (Tq,Hq,D) bf16.  Differentiable like flash_attn_prefill;
    kv_splits / workspace as there.
    """
    q, k, v, out_dtype = _to_bf16(q, k, v)
    if _needs_grad(q, k, v):
        out = _VarlenPrefillFn.apply(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, bool(causal),
                                     softmax_scale)
    else:
        out = _varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, causal, softmax_scale,
                      kv_splits=kv_splits, workspace=workspace)
    return out if out.dtype == out_dtype else out.to(out_dtype)


def decode_chunk_tokens(batch, n_q_heads, n_kv_heads, max_context):
    """Tokens of one sequence that one workgroup of the split-K decode pass handles for these bounds."""
    return int(_lib.load().mi355_paged_decode_chunk_tokens(batch, n_q_heads, n_kv_heads, max_context))


def paged_decode_workspace(batch, n_q_heads, head_dim, max_context, device):
    """Scratch tensor for paged_attention_decode.  The requirement is monotonic in every argument, so a tensor
    sized for the largest batch and longest context serves every smaller call."""
    n = _lib.load().mi355_paged_decode_workspace_bytes(batch, n_q_heads, head_dim, max_context)
    return torch.empty(max(int(n), 16), dtype=torch.uint8, device=device)


def paged_attention_decode(q, k_cache, v_cache, block_tables, context_lens, *, softmax_scale=None,
                           k_scale=None, v_scale=None, max_context=None, workspace=None, out=None,
                           static_scratch=False):
    """Paged-KV decode attention, one query token per sequence.

    q (B,Hq,D) bf16; k_cache, v_cache (num_blocks,Hkv,16,D) bf16, or fp8-e4m3
    (torch.float8_e4m3fn / uint8 bit patterns) when k_scale and v_scale
    (num_blocks,Hkv) fp32 are given; block_tables (B,max_blocks) int32;
    context_lens (B,) int32 >= 1.  `max_context` bounds context_lens (default:
    block_tables.shape[1]*16) so no device->host sync is needed.  Returns (B,Hq,D) bf16.
    static_scratch=True (needs `out`) goes through mi355_paged_decode_fwd_static: nothing is allocated, the
    split-K partials live in the library's own device array (16 MiB per GPU; larger problems are rejected; calls
    that overlap in time on one GPU must be serialised by the caller).
    """
    _require_gpu_bf16("q", q)
    if q.dim() != 3:
        raise ValueError(f"q must be (batch, heads, d_head), got {tuple(q.shape)}")
    B, Hq, D = q.shape
    fp8 = k_scale is not None or v_scale is not None
    if fp8:
        if k_scale is None or v_scale is None:
            raise ValueError("k_scale and v_scale must be given together")
        for n, c in (("k_cache", k_cache), ("v_cache", v_cache)):
            if c.dtype not in (torch.uint8, torch.float8_e4m3fn):
                raise TypeError(f"{n} must be float8_e4m3fn or uint8 when scales are given (got {c.dtype})")
    else:
        for n, c in (("k_cache", k_cache), ("v_cache", v_cache)):
            if c.dtype != torch.bfloat16:
                raise TypeError(f"{n} must be bfloat16 (got {c.dtype}); pass k_scale/v_scale for an fp8 cache")
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape:
        raise ValueError("k_cache and v_cache must both be (num_blocks, kv_heads, 16, d_head)")
    nb, Hkv, bs, Dc = k_cache.shape
    if bs != _BLOCK or Dc != D:
        raise ValueError(f"cache must be (num_blocks, kv_heads, {_BLOCK}, {D}), got {tuple(k_cache.shape)}")
    for n, c in (("q", q), ("k_cache", k_cache), ("v_cache", v_cache)):
        if not c.is_contiguous() or not c.is_cuda:
            raise ValueError(f"{n} must be a contiguous GPU tensor")
    if block_tables.dtype != torch.int32 or context_lens.dtype != torch.int32:
        raise TypeError("block_tables and context_lens must be int32")
    if block_tables.dim() != 2 or block_tables.shape[0] != B or block_tables.stride(1) != 1:
        raise ValueError("block_tables must be (batch, max_blocks) with unit column stride")
    if context_lens.shape != (B,) or not context_lens.is_contiguous():
        raise ValueError("context_lens must be a contiguous (batch,) tensor")
    if fp8:
        for n, s in (("k_scale", k_scale), ("v_scale", v_scale)):
            if s.dtype != torch.float32 or tuple(s.shape) != (nb, Hkv) or not s.is_contiguous():
                raise ValueError(f"{n} must be a contiguous float32 (num_blocks, kv_heads) tensor")
    if max_context is None:
        max_context = block_tables.shape[1] * _BLOCK
    if max_context > block_tables.shape[1] * _BLOCK:
        raise ValueError("max_context exceeds what block_tables can address")
    scale = 1.0 / math.sqrt(D) if softmax_scale is None else softmax_scale
    if out is None:
        if static_scratch:
            raise ValueError("static_scratch=True allocates nothing: pass `out`")
        out = torch.empty_like(q)
    if B == 0:
        return out
    lib = _lib.load()
    if static_scratch:
        if workspace is not None:
            raise ValueError("static_scratch and workspace exclude each other")
        with _on(q, k_cache, v_cache, out, block_tables, context_lens, k_scale, v_scale) as stream:
            rc = lib.mi355_paged_decode_fwd_static(
                q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(),
                block_tables.data_ptr(), block_tables.stride(0), context_lens.data_ptr(),
                k_scale.data_ptr() if fp8 else None, v_scale.data_ptr() if fp8 else None,
                B, Hq, Hkv, D, bs, k_cache.shape[0], int(max_context), float(scale),
                _lib.MI355_FP8_E4M3 if fp8 else _lib.MI355_BF16, stream)
        _lib.check(rc, "mi355_paged_decode_fwd_static")
        return out
    if workspace is None:
        workspace = paged_decode_workspace(B, Hq, D, max_context, q.device)
    with _on(q, k_cache, v_cache, out, block_tables, context_lens, k_scale, v_scale, workspace) as stream:
        rc = lib.mi355_paged_decode_fwd(
            q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(),
            block_tables.data_ptr(), block_tables.stride(0), context_lens.data_ptr(),
            k_scale.data_ptr() if fp8 else None, v_scale.data_ptr() if fp8 else None,
            workspace.data_ptr(), workspace.numel() * workspace.element_size(),
            B, Hq, Hkv, D, bs, k_cache.shape[0], int(max_context), float(scale),
            _lib.MI355_FP8_E4M3 if fp8 else _lib.MI355_BF16, stream)
    _lib.check(rc, "mi355_paged_decode_fwd")
    return out


def flash_attn_paged_prefill(q, k_cache, v_cache, cu_seqlens_q, block_tables, context_lens, max_seqlen_q, *,
                             softmax_scale=None, out=None, max_context=None, kv_splits=None, workspace=None,
                             k_scale=None, v_scale=None, total_context=None, cu_seqlens_k=None):
    """Causal prefill of a chunk of new tokens over context that already sits in a paged cache.

    q (T,Hq,D) bf16, packed, contiguous heads (token stride free): sequence b owns rows
    [cu_seqlens_q[b], cu_seqlens_q[b+1]).  k_cache, v_cache (num_blocks,Hkv,16,D) bf16 hold ALL
    context_lens[b] tokens of sequence b -- the chunk's own too (write them first with rope_and_cache) --
    addressed through block_tables (B,max_blocks) int32.  Query i of the chunk keeps key j iff
    j <= i + (context_lens[b] - chunk length).  max_seqlen_q = longest chunk.  Returns (T,Hq,D) bf16.
    max_context bounds context_lens (default: what block_tables can address) and only guides the choice of
    kv_splits (see flash_attn_prefill): a short chunk over a long context is split over many workgroups.
    A context length beyond what a row of block_tables addresses is cut to it.
    With k_scale and v_scale (num_blocks,Hkv) fp32 the cache is fp8-e4m3 (uint8 / float8_e4m3fn, the layout
    of paged_attention_decode): the sequences' keys and values are first gathered and dequantised into packed
    bf16 rows (mi355_gather_kv_fp8; value = bf16(fp8 * scale)), then attended to by the packed prefill kernels.
    total_context (host int, optional): an upper bound on sum(context_lens) that sizes those rows (default
    batch * max_context); cu_seqlens_k (int32 (B+1,), optional): the running sum of the context lengths, if the
    caller has it on the device already (else it is computed here, a few small launches per call).
    The mathematics is that of llm-core/llm_core/model.py:308-325 with the mask of :384; the reference
    itself would re-run the whole prefix (model.py:218)."""
    _require_gpu_bf16("q", q)
    if k_scale is not None or v_scale is not None:
        return _paged_prefill_fp8(q, k_cache, v_cache, k_scale, v_scale, cu_seqlens_q, block_tables, context_lens,
                                  max_seqlen_q, softmax_scale, out, max_context, kv_splits, workspace, total_context,
                                  cu_seqlens_k)
    if q.dim() != 3 or q.stride(2) != 1 or q.stride(1) != q.shape[2]:
        raise ValueError("q must be (tokens, heads, d_head) with contiguous heads")
    T, Hq, D = q.shape
    for n, c in (("k_cache", k_cache), ("v_cache", v_cache)):
        if c.dtype != torch.bfloat16:
            raise TypeError(f"{n} must be bfloat16 (got {c.dtype}); chunked prefill reads a bf16 cache")
        if c.dim() != 4 or c.shape[2] != _BLOCK or c.shape[3] != D or not c.is_contiguous() or not c.is_cuda:
            raise ValueError(f"{n} must be a contiguous GPU tensor (num_blocks, kv_heads, {_BLOCK}, {D})")
    if k_cache.shape != v_cache.shape:
        raise ValueError("k_cache and v_cache must have the same shape")
    Hkv = k_cache.shape[1]
    if D not in (32, 64, 128):
        raise ValueError("d_head must be 32, 64 or 128")
    if Hq % Hkv != 0:
        raise ValueError("the number of query heads must be a multiple of the number of kv heads")
    for n, t in (("cu_seqlens_q", cu_seqlens_q), ("block_tables", block_tables), ("context_lens", context_lens)):
        if t.dtype != torch.int32:
            raise TypeError(f"{n} must be int32")
    B = cu_seqlens_q.numel() - 1
    if cu_seqlens_q.dim() != 1 or B < 0 or not cu_seqlens_q.is_contiguous():
        raise ValueError("cu_seqlens_q must be a contiguous (batch + 1,) tensor")
    if block_tables.dim() != 2 or block_tables.shape[0] != B or block_tables.stride(1) != 1:
        raise ValueError("block_tables must be (batch, max_blocks) with unit column stride")
    if context_lens.shape != (B,) or not context_lens.is_contiguous():
        raise ValueError("context_lens must be a contiguous (batch,) tensor")
    if int(max_seqlen_q) < 1 and T > 0:
        raise ValueError("max_seqlen_q must be at least 1")
    if q.stride(0) % 8 != 0 or q.data_ptr() % 16 != 0:
        raise ValueError("q must be 16-byte aligned with a token stride that is a multiple of 8 elements")
    if out is None:
        out = torch.empty(T, Hq, D, dtype=q.dtype, device=q.device)
    else:
        _require_gpu_bf16("out", out)
        if out.shape != q.shape or out.stride(2) != 1 or out.stride(1) != D or out.stride(0) % 8 != 0 \
                or out.data_ptr() % 16 != 0:
            raise ValueError("out must have q's shape with contiguous heads, 16-byte aligned")
    if T == 0 or B == 0:
        return out
    scale = 1.0 / math.sqrt(D) if softmax_scale is None else softmax_scale
    if max_context is None:
        max_context = block_tables.shape[1] * _BLOCK
    n_split, workspace = _split_args(kv_splits, workspace, B, Hq, D, int(max_seqlen_q), int(max_context), T, True,
                                     q.device)
    with _on(q, k_cache, v_cache, out, cu_seqlens_q, block_tables, context_lens, workspace) as stream:
        rc = _lib.load().mi355_prefill_paged_fwd(
            q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), q.stride(0), out.stride(0),
            cu_seqlens_q.data_ptr(), block_tables.data_ptr(), block_tables.stride(0), block_tables.shape[1],
            context_lens.data_ptr(),
            B, Hq, Hkv, int(max_seqlen_q), D, _BLOCK, k_cache.shape[0], float(scale), _lib.MI355_BF16,
            n_split, T, None if workspace is None else workspace.data_ptr(),
            0 if workspace is None else workspace.numel() * workspace.element_size(), stream)
    _lib.check(rc, "mi355_prefill_paged_fwd")
    return out


def gather_kv_fp8(k_cache, v_cache, k_scale, v_scale, block_tables, context_lens, *, max_context=None, total_context=None,
                  cu_seqlens_k=None, out=None):
    """The keys and values of a batch of sequences out of an fp8 paged cache, dequantised, as packed bf16 rows.
    Returns (k (rows,Hkv,D), v (rows,Hkv,D), cu_seqlens_k int32 (B+1,)): sequence b owns rows
    [cu_seqlens_k[b], cu_seqlens_k[b+1]), cu_seqlens_k the running sum of min(context_lens, max_context);
    rows = total_context when given (a host-side bound on that sum), else batch * max_context.  A caller that
    already holds that running sum on the device (a serving loop computes it once per step, not once per layer)
    passes it as cu_seqlens_k; out=(k, v) reuses two contiguous bf16 (rows, Hkv, D) tensors.  Nothing is read back
    from the device."""
    for n, c in (("k_cache", k_cache), ("v_cache", v_cache)):
        if c.dtype not in (torch.uint8, torch.float8_e4m3fn) or c.dim() != 4 or c.shape[2] != _BLOCK or not c.is_contiguous() \
                or not c.is_cuda:
            raise ValueError(f"{n} must be a contiguous uint8/float8_e4m3fn GPU tensor (num_blocks, kv_heads, {_BLOCK}, d_head)")
    if k_cache.shape != v_cache.shape:
        raise ValueError("k_cache and v_cache must have the same shape")
    nb, Hkv, _, D = k_cache.shape
    if D not in (32, 64, 128):
        raise ValueError("d_head must be 32, 64 or 128")
    if k_scale is None or v_scale is None:
        raise ValueError("k_scale and v_scale must be given together")
    for n, c in (("k_scale", k_scale), ("v_scale", v_scale)):
        if c.dtype != torch.float32 or tuple(c.shape) != (nb, Hkv) or not c.is_contiguous():
            raise ValueError(f"{n} must be a contiguous float32 (num_blocks, kv_heads) tensor")
    if block_tables.dtype != torch.int32 or context_lens.dtype != torch.int32:
        raise TypeError("block_tables and context_lens must be int32")
    B = context_lens.numel()
    if block_tables.dim() != 2 or block_tables.shape[0] != B or block_tables.stride(1) != 1 or block_tables.shape[1] < 1:
        raise ValueError("block_tables must be (batch, max_blocks) with unit column stride")
    if context_lens.shape != (B,) or not context_lens.is_contiguous():
        raise ValueError("context_lens must be a contiguous (batch,) tensor")
    width = block_tables.shape[1] * _BLOCK
    max_context = width if max_context is None else min(int(max_context), width)
    rows = B * max_context if total_context is None else min(int(total_context), B * max_context)
    dev = k_cache.device
    if cu_seqlens_k is not None:
        if cu_seqlens_k.dtype != torch.int32 or cu_seqlens_k.shape != (B + 1,) or not cu_seqlens_k.is_contiguous() \
                or cu_seqlens_k.device != dev:
            raise ValueError("cu_seqlens_k must be a contiguous int32 (batch + 1,) tensor on the caches' device")
        cu_k = cu_seqlens_k
    else:
        cu_k = torch.zeros(B + 1, dtype=torch.int32, device=dev)
        if B:
            cu_k[1:] = torch.cumsum(context_lens.clamp(max=max_context), 0)
    if out is not None:
        k_lin, v_lin = out
        for n, t in (("out[0]", k_lin), ("out[1]", v_lin)):
            if t.dtype != torch.bfloat16 or tuple(t.shape) != (max(rows, 1), Hkv, D) or not t.is_contiguous() or t.device != dev:
                raise ValueError(f"{n} must be a contiguous bfloat16 ({max(rows, 1)}, {Hkv}, {D}) tensor on the caches' device")
    else:
        k_lin = torch.empty(max(rows, 1), Hkv, D, dtype=torch.bfloat16, device=dev)
        v_lin = torch.empty(max(rows, 1), Hkv, D, dtype=torch.bfloat16, device=dev)
    if B and rows:
        with _on(k_cache, v_cache, k_scale, v_scale, block_tables, context_lens) as stream:
            rc = _lib.load().mi355_gather_kv_fp8(
                k_cache.data_ptr(), v_cache.data_ptr(), k_scale.data_ptr(), v_scale.data_ptr(), block_tables.data_ptr(),
                block_tables.stride(0), (max_context + _BLOCK - 1) // _BLOCK, context_lens.data_ptr(), cu_k.data_ptr(),
                k_lin.data_ptr(), v_lin.data_ptr(), Hkv * D, rows, B, Hkv, D, _BLOCK, nb, stream)
        _lib.check(rc, "mi355_gather_kv_fp8")
    return k_lin, v_lin, cu_k


def _paged_prefill_fp8(q, k_cache, v_cache, k_scale, v_scale, cu_seqlens_q, block_tables, context_lens, max_seqlen_q,
                       softmax_scale, out, max_context, kv_splits, workspace, total_context, cu_seqlens_k=None):
    """flash_attn_paged_prefill over an fp8 cache: gather + dequantise, then the packed prefill with more keys than
    queries per sequence (bottom-right aligned causal mask)."""
    if q.dim() != 3:
        raise ValueError("q must be (tokens, heads, d_head)")
    if block_tables.dim() != 2:
        raise ValueError("block_tables must be (batch, max_blocks)")
    width = block_tables.shape[1] * _BLOCK
    max_context = width if max_context is None else min(int(max_context), width)
    k_lin, v_lin, cu_k = gather_kv_fp8(k_cache, v_cache, k_scale, v_scale, block_tables, context_lens,
                                       max_context=max_context, total_context=total_context, cu_seqlens_k=cu_seqlens_k)
    res = flash_attn_varlen_prefill(q, k_lin, v_lin, cu_seqlens_q, cu_k, max_seqlen_q, max_context, causal=True,
                                    softmax_scale=softmax_scale, kv_splits=kv_splits, workspace=workspace)
    if out is not None:
        out.copy_(res)
        return out
    return res


def build_rope_cache(context_length, d, theta=10000.0, device="cuda"):
    """cos/sin table in the reference's layout (2, context_length, d/2) fp32, as
    RotaryEmbedding._build_cache builds it (llm-core/llm_core/model.py:86-91)."""
    inv_freq = theta ** -(torch.arange(0, d, 2, dtype=torch.float32) / d)
    angles = torch.arange(context_length, dtype=torch.float32)[:, None] * inv_freq[None, :]
    return torch.stack((torch.cos(angles), torch.sin(angles))).to(device)


def _packed_k_out(k_out, k):
    """k_out argument of the cache writes: None, True (allocate) or a tensor of k's shape to fill."""
    if k_out is None or k_out is False:
        return None
    if k_out is True:
        return torch.empty(k.shape, dtype=k.dtype, device=k.device)
    _require_gpu_bf16("k_out", k_out)
    if k_out.shape != k.shape or k_out.stride(2) != 1 or k_out.stride(1) != k.shape[2] or k_out.stride(0) % 8 != 0 \
            or k_out.data_ptr() % 16 != 0:
        raise ValueError("k_out must have k's shape with contiguous heads, 16-byte aligned, token stride a multiple of 8")
    return k_out


def _overlap(a, b):
    """Do the memory spans of two (tokens, heads, d_head) tensors with contiguous heads intersect?"""
    def span(t):
        lo = t.data_ptr()
        return lo, lo + ((t.shape[0] - 1) * t.stride(0) + t.shape[1] * t.shape[2]) * t.element_size()
    (a0, a1), (b0, b1) = span(a), span(b)
    return a0 < b1 and b0 < a1


def rope_and_cache(q, k, v, positions, freq_cache, k_cache=None, v_cache=None, slot_mapping=None, *, out=None,
                   k_out=None):
    """RoPE on q and k (interleaved pairs, llm-core/llm_core/model.py:93-104) and scatter of the
    rotated k and of v into the paged cache.

    q (T,Hq,D), k, v (T,Hkv,D) bf16 with contiguous heads; positions (T,) int32; freq_cache
    (2, context_length, D/2) fp32; slot_mapping (T,) int64 = block*16 + offset (negative: skip).
    Returns the rotated q (T,Hq,D) (written into `out` when given; `out` may be q itself); the
    caches are updated in place.  With `k_out` (True, or a (T,Hkv,D) tensor to fill) the same launch
    also writes the rotated keys in packed form -- the K operand of a prefill over the same tokens --
    and the return value is (rotated q, rotated k).
    """
    for n, t in (("q", q), ("k", k), ("v", v)):
        _require_gpu_bf16(n, t)
        if t.dim() != 3 or t.stride(2) != 1 or t.stride(1) != t.shape[2]:
            raise ValueError(f"{n} must be (tokens, heads, d_head) with contiguous heads")
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    if k.shape != v.shape or k.shape[0] != T or k.shape[2] != D:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)}")
    if freq_cache.dtype != torch.float32 or freq_cache.dim() != 3 or freq_cache.shape[0] != 2 \
            or freq_cache.shape[2] * 2 != D or not freq_cache.is_contiguous() or not freq_cache.is_cuda:
        raise ValueError("freq_cache must be a contiguous float32 GPU tensor (2, context_length, d_head/2)")
    if positions.dtype != torch.int32 or positions.shape != (T,) or not positions.is_contiguous():
        raise TypeError("positions must be a contiguous int32 (tokens,) tensor")
    if slot_mapping is not None:
        if slot_mapping.dtype != torch.int64 or slot_mapping.shape != (T,) or not slot_mapping.is_contiguous():
            raise TypeError("slot_mapping must be a contiguous int64 (tokens,) tensor")
        for n, c in (("k_cache", k_cache), ("v_cache", v_cache)):
            if c is None or c.dtype != torch.bfloat16 or c.dim() != 4 or c.shape[1:] != (Hkv, _BLOCK, D) \
                    or not c.is_contiguous():
                raise ValueError(f"{n} must be a contiguous bf16 (num_blocks, {Hkv}, {_BLOCK}, {D}) tensor")
    if out is None:
        q_out = torch.empty(T, Hq, D, dtype=q.dtype, device=q.device)
    else:
        q_out = out
        _require_gpu_bf16("out", q_out)
        if q_out.shape != q.shape or q_out.stride(2) != 1 or q_out.stride(1) != D:
            raise ValueError("out must have q's shape with contiguous heads")
    k_rot = _packed_k_out(k_out, k)
    if T == 0:
        return q_out if k_rot is None else (q_out, k_rot)
    with _on(q, k, v, q_out, freq_cache, positions, slot_mapping, k_cache, v_cache, k_rot) as stream:
        rc = _lib.load().mi355_rope_and_cache(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), q_out.data_ptr(),
            None if slot_mapping is None else k_cache.data_ptr(), None if slot_mapping is None else v_cache.data_ptr(),
            freq_cache.data_ptr(), positions.data_ptr(), None if slot_mapping is None else slot_mapping.data_ptr(),
            0 if slot_mapping is None else k_cache.shape[0], T, Hq, Hkv, D, freq_cache.shape[1], q.stride(0), k.stride(0),
            v.stride(0), q_out.stride(0), None if k_rot is None else k_rot.data_ptr(),
            0 if k_rot is None else k_rot.stride(0), stream)
    _lib.check(rc, "mi355_rope_and_cache")
    return q_out if k_rot is None else (q_out, k_rot)


def rope_and_cache_fp8(q, k, v, positions, freq_cache, k_cache, v_cache, k_scale, v_scale, slot_mapping, *, out=None,
                       k_out=None):
    """rope_and_cache into an fp8-e4m3 cache: k_cache, v_cache (num_blocks,Hkv,16,D) uint8 (or
    float8_e4m3fn), k_scale, v_scale (num_blocks,Hkv) fp32, all updated in place.  A block's scale is
    kept equal to absmax/448 of its valid rows; rows already in a block are re-expressed when new rows
    raise the scale.  Tokens that share a block must be adjacent with consecutive slots, one such run
    per block and call (what a prefill or a decode step produces).  Returns the rotated q, or, with
    `k_out` (True or a tensor to fill; not k itself or a view of it -- unlike in rope_and_cache the keys are read
    again, by other workgroups, after k_out is written), (rotated q, rotated keys in bf16, packed (T,Hkv,D))."""
    for n, t in (("q", q), ("k", k), ("v", v)):
        _require_gpu_bf16(n, t)
        if t.dim() != 3 or t.stride(2) != 1 or t.stride(1) != t.shape[2]:
            raise ValueError(f"{n} must be (tokens, heads, d_head) with contiguous heads")
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    if k.shape != v.shape or k.shape[0] != T or k.shape[2] != D:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)}")
    if D not in (32, 64, 128):
        raise ValueError("d_head must be 32, 64 or 128")
    if freq_cache.dtype != torch.float32 or freq_cache.dim() != 3 or freq_cache.shape[0] != 2 \
            or freq_cache.shape[2] * 2 != D or not freq_cache.is_contiguous() or not freq_cache.is_cuda:
        raise ValueError("freq_cache must be a contiguous float32 GPU tensor (2, context_length, d_head/2)")
    if positions.dtype != torch.int32 or positions.shape != (T,) or not positions.is_contiguous():
        raise TypeError("positions must be a contiguous int32 (tokens,) tensor")
    if slot_mapping.dtype != torch.int64 or slot_mapping.shape != (T,) or not slot_mapping.is_contiguous():
        raise TypeError("slot_mapping must be a contiguous int64 (tokens,) tensor")
    for n, c in (("k_cache", k_cache), ("v_cache", v_cache)):
        if c.dtype not in (torch.uint8, torch.float8_e4m3fn) or c.dim() != 4 or c.shape[1:] != (Hkv, _BLOCK, D) \
                or not c.is_contiguous() or c.shape[0] != k_cache.shape[0]:
            raise ValueError(f"{n} must be a contiguous uint8/float8_e4m3fn (num_blocks, {Hkv}, {_BLOCK}, {D}) tensor")
    nb = k_cache.shape[0]
    for n, c in (("k_scale", k_scale), ("v_scale", v_scale)):
        if c.dtype != torch.float32 or c.shape != (nb, Hkv) or not c.is_contiguous():
            raise ValueError(f"{n} must be a contiguous float32 ({nb}, {Hkv}) tensor")
    for n, t in (("q", q), ("k", k), ("v", v)):
        if t.stride(0) % 8 != 0 or t.data_ptr() % 16 != 0:
            raise ValueError(f"{n} must be 16-byte aligned with a token stride that is a multiple of 8 elements")
    if out is None:
        q_out = torch.empty(T, Hq, D, dtype=q.dtype, device=q.device)
    else:
        q_out = out
        _require_gpu_bf16("out", q_out)
        if q_out.shape != q.shape or q_out.stride(2) != 1 or q_out.stride(1) != D or q_out.stride(0) % 8 != 0 \
                or q_out.data_ptr() % 16 != 0:
            raise ValueError("out must have q's shape with contiguous heads, 16-byte aligned")
    k_rot = _packed_k_out(k_out, k)
    if k_rot is not None and T and _overlap(k_rot, k):
        raise ValueError("k_out must not share memory with k (the fp8 write reads the keys again after k_out is written)")
    if T == 0:
        return q_out if k_rot is None else (q_out, k_rot)
    with _on(q, k, v, q_out, freq_cache, positions, slot_mapping, k_cache, v_cache, k_scale, v_scale, k_rot) as stream:
        rc = _lib.load().mi355_rope_and_cache_fp8(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), q_out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
            k_scale.data_ptr(), v_scale.data_ptr(), freq_cache.data_ptr(), positions.data_ptr(), slot_mapping.data_ptr(),
            nb, T, Hq, Hkv, D, freq_cache.shape[1], q.stride(0), k.stride(0), v.stride(0), q_out.stride(0),
            None if k_rot is None else k_rot.data_ptr(), 0 if k_rot is None else k_rot.stride(0), stream)
    _lib.check(rc, "mi355_rope_and_cache_fp8")
    return q_out if k_rot is None else (q_out, k_rot)


def quantize_kv_cache_fp8(cache, *, out=None):
    """bf16 cache (num_blocks,Hkv,16,D) -> (uint8 e4m3 cache, fp32 scale (num_blocks,Hkv)), scale = absmax/448.
    `out` = (uint8 cache, fp32 scale) tensors to write into instead of new ones."""
    _require_gpu_bf16("cache", cache)
    if cache.dim() != 4 or cache.shape[2] != _BLOCK or not cache.is_contiguous():
        raise ValueError(f"cache must be a contiguous (num_blocks, kv_heads, {_BLOCK}, d_head) tensor")
    nb, Hkv, _, D = cache.shape
    if out is None:
        out = torch.empty(cache.shape, dtype=torch.uint8, device=cache.device)
        scale = torch.empty(nb, Hkv, dtype=torch.float32, device=cache.device)
    else:
        out, scale = out
        if out.dtype != torch.uint8 or out.shape != cache.shape or not out.is_contiguous() or out.device != cache.device:
            raise ValueError("out[0] must be a contiguous uint8 tensor of the cache's shape on its device")
        if scale.dtype != torch.float32 or scale.shape != (nb, Hkv) or not scale.is_contiguous() \
                or scale.device != cache.device:
            raise ValueError("out[1] must be a contiguous float32 (num_blocks, kv_heads) tensor on the cache's device")
    with _on(cache, out, scale) as stream:
        rc = _lib.load().mi355_quantize_kv_fp8(cache.data_ptr(), out.data_ptr(), scale.data_ptr(), nb, Hkv, D, _BLOCK,
                                               stream)
    _lib.check(rc, "mi355_quantize_kv_fp8")
    return out, scale


def _rows2d(name, t):
    """(…, n_cols) bf16 GPU tensor -> (n_rows, n_cols) view with a unit column stride (copy only if needed)."""
    _require_gpu_bf16(name, t)
    if t.dim() < 1:
        raise ValueError(f"{name} must have at least one dimension")
    t2 = t.reshape(-1, t.shape[-1])           # a view whenever the leading dims can be merged
    if t2.stride(1) != 1 and t2.shape[1] > 1:
        t2 = t2.contiguous()
    return t2


def rms_norm(x, weight, eps: float = 1e-5, *, residual=None, return_sum: bool = False, return_rstd: bool = False):
    """RMSNorm forward over the last dimension: weight * (h * rsqrt(mean(h^2) + eps)), fp32 math, bf16 in/out --
    RMSNorm.forward (llm-core/llm_core/model.py:60-67) and TritonRMSNorm's forward kernel
    (llm-systems/llm_systems/kernels/triton_rms_norm.py:30-74).

    x (..., d) bf16; weight (d,) bf16 or fp32.  With `residual` (same shape as x) the normalised
    tensor is h = bf16(x + residual), the add in front of each norm of TransformerBlock.forward
    (model.py:293-294); return_sum=True also returns h.  return_rstd=True also returns 1/rms
    (fp32, x.shape[:-1]) as the Triton kernel caches it.  Returns y, or (y, [h], [rstd]).
    """
    x2 = _rows2d("x", x)
    n_rows, d = x2.shape
    if weight.shape != (d,) or not weight.is_cuda or not weight.is_contiguous():
        raise ValueError(f"weight must be a contiguous GPU tensor of shape ({d},)")
    if weight.dtype == torch.bfloat16:
        wcode = _lib.MI355_BF16
    elif weight.dtype == torch.float32:
        wcode = _lib.MI355_FP32
    else:
        raise TypeError(f"weight must be bfloat16 or float32 (got {weight.dtype})")
    r2 = None
    if residual is not None:
        if residual.shape != x.shape:
            raise ValueError("residual must have x's shape")
        r2 = _rows2d("residual", residual)
    elif return_sum:
        raise ValueError("return_sum needs residual")
    y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    h = torch.empty(x.shape, dtype=x.dtype, device=x.device) if return_sum else None
    rstd = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device) if return_rstd else None
    if n_rows:
        with _on(x2, r2, weight) as stream:
            rc = _lib.load().mi355_rms_norm_fwd(
                x2.data_ptr(), None if r2 is None else r2.data_ptr(), weight.data_ptr(), y.data_ptr(),
                None if h is None else h.data_ptr(), None if rstd is None else rstd.data_ptr(),
                n_rows, d, x2.stride(0), 0 if r2 is None else r2.stride(0), d, d, float(eps), wcode, stream)
        _lib.check(rc, "mi355_rms_norm_fwd")
    extra = [t for t in (h, rstd) if t is not None]
    return (y, *extra) if extra else y


def silu_mul(gate, up):
    """bf16(silu(gate)) * up, silu in fp32 -- the fused kernel of FusedSwiGLU
    (llm-systems/llm_systems/kernels/triton_swiglu.py:27-47; SwiGLU.forward, model.py:304-305).
    gate and up (..., d_ff) bf16 may be strided row views, e.g. the two halves of a merged
    gate/up projection output (triton_swiglu.py:190-191): nothing is copied."""
    if gate.shape != up.shape:
        raise ValueError(f"shape mismatch: gate {tuple(gate.shape)} up {tuple(up.shape)}")
    g2, u2 = _rows2d("gate", gate), _rows2d("up", up)
    out = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
    n_rows, d = g2.shape
    if n_rows and d:
        with _on(g2, u2) as stream:
            rc = _lib.load().mi355_silu_mul_fwd(g2.data_ptr(), u2.data_ptr(), out.data_ptr(), n_rows, d,
                                                g2.stride(0), u2.stride(0), d, stream)
        _lib.check(rc, "mi355_silu_mul_fwd")
    return out
