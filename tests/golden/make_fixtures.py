#!/usr/bin/env python3
"""Writes tests/golden/attention_golden.npz: small seeded inputs and the oracle's outputs for them.

The reference ships no test vectors for this path, so these are produced by this build's own oracle
(oracle/attention_oracle.py, itself pinned by tests/test_oracle.py against library routines, closed forms and
float64 loops).  Their job is to catch DRIFT: a later edit of the oracle or of a kernel that changes results shows
up against numbers that were written down earlier.  bf16 inputs are stored as their 16-bit patterns (int16; numpy
has no bf16; load_golden() below turns them back into bfloat16 tensors), outputs as float32, fp8 bytes as uint8.

usage: python tests/golden/make_fixtures.py     (rewrites the .npz next to this file)
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import attention_oracle as orc  # noqa: E402


def bf16_values(*shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


def bits(t):
    return t.contiguous().view(torch.int16).numpy()


def load_golden(path=None):
    """The fixture file as a dict of torch tensors (int16 bit patterns viewed as bfloat16 again)."""
    path = path or os.path.join(HERE, "attention_golden.npz")
    raw = np.load(path)                      # allow_pickle stays False
    out = {}
    for name in raw.files:
        t = torch.from_numpy(raw[name])
        out[name] = t.view(torch.bfloat16) if t.dtype == torch.int16 else t
    return out


def build():
    out = {}
    # 1. dense attention, the reference signature (model.py:308-325): no mask, causal mask, rectangular
    q, k, v = bf16_values(1, 2, 33, 32, seed=1, scale=0.5), bf16_values(1, 2, 33, 32, seed=2, scale=0.5), bf16_values(1, 2, 33, 32, seed=3, scale=0.5)
    out["dense_q"], out["dense_k"], out["dense_v"] = (bits(t) for t in (q, k, v))
    out["dense_out_nomask"] = orc.scaled_dot_product_attention(q.float(), k.float(), v.float()).numpy()
    out["dense_out_causal"] = orc.prefill_reference(q, k, v, causal=True).numpy()
    # 2. GQA + packed varlen prefill
    lens = [5, 1, 20]
    cu = torch.tensor([0, 5, 6, 26], dtype=torch.int32)
    q, k, v = bf16_values(26, 4, 64, seed=4, scale=0.5), bf16_values(26, 2, 64, seed=5, scale=0.5), bf16_values(26, 2, 64, seed=6, scale=0.5)
    out["varlen_q"], out["varlen_k"], out["varlen_v"], out["varlen_cu"] = bits(q), bits(k), bits(v), cu.numpy()
    out["varlen_out"] = orc.varlen_prefill_reference(q, k, v, cu, cu, causal=True).numpy()
    dout = bf16_values(1, 4, 20, 64, seed=7, scale=0.5)
    qq, kk, vv = (t[6:26].transpose(0, 1)[None].contiguous() for t in (q, k, v))
    dq, dk, dv, lse = orc.prefill_backward_reference(qq, kk, vv, dout, causal=True)
    out["bwd_dout"] = bits(dout)
    out["bwd_dq"], out["bwd_dk"], out["bwd_dv"], out["bwd_lse"] = dq.numpy(), dk.numpy(), dv.numpy(), lse.numpy()
    # 3. paged decode, bf16 and fp8 KV
    ctx = [1, 17, 40]
    q, kc, vc, bt, cl = orc.make_paged_case(batch=3, n_q_heads=4, n_kv_heads=2, head_dim=64, block_size=16,
                                            context_lens=ctx, pool_factor=1.5, seed=8, dtype=torch.bfloat16)
    out["paged_q"], out["paged_k_cache"], out["paged_v_cache"] = bits(q), bits(kc), bits(vc)
    out["paged_block_tables"], out["paged_context_lens"] = bt.numpy(), cl.numpy()
    out["paged_out"] = orc.paged_decode_reference(q, kc, vc, bt, cl).numpy()
    k8, ks = orc.quantize_kv_fp8(kc)
    v8, vs = orc.quantize_kv_fp8(vc)
    out["paged_k_fp8"], out["paged_v_fp8"] = k8.view(torch.uint8).numpy(), v8.view(torch.uint8).numpy()
    out["paged_k_scale"], out["paged_v_scale"] = ks.numpy(), vs.numpy()
    out["paged_out_fp8"] = orc.paged_decode_reference(q, k8, v8, bt, cl, k_scale=ks, v_scale=vs).numpy()
    # 4. RoPE with the reference's table layout (model.py:86-104)
    fc = orc.build_rope_cache(64, 32)
    x = bf16_values(2, 7, 32, seed=9)
    pos = torch.tensor([0, 1, 2, 5, 17, 40, 63])
    out["rope_x"], out["rope_pos"] = bits(x), pos.numpy()
    out["rope_out"] = orc.rope_reference(x.float(), pos, fc).numpy()
    return out


if __name__ == "__main__":
    path = os.path.join(HERE, "attention_golden.npz")
    np.savez_compressed(path, **build())
    print("wrote", path, os.path.getsize(path), "bytes")
