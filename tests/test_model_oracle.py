"""Pins oracle/model_oracle.py (CPU): library equivalence, closed forms, invariants and an
independent float64 loop implementation, chosen so that a dropped term, a wrong sign, a
transposed weight or a wrong rounding order fails at least one check."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import attention_oracle as att
from oracle import model_oracle as mo

CFG = dict(vocab_size=97, context_length=48, d_model=32, num_layers=2, num_heads=4, d_ff=80, rope_theta=10000.0)


def test_rms_norm_matches_torch_library_and_closed_forms():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 7, 64, generator=g) * 3
    w = torch.randn(64, generator=g)
    torch.testing.assert_close(mo.rms_norm_reference(x, w, 1e-5), F.rms_norm(x, (64,), w, 1e-5), atol=1e-6, rtol=1e-6)
    # constant row c, weight 1: c / sqrt(c^2 + eps)
    c = torch.full((1, 16), 2.0)
    torch.testing.assert_close(mo.rms_norm_reference(c, torch.ones(16), 1e-5), c / math.sqrt(4.0 + 1e-5))
    # invariant to a positive scaling of the row (up to eps), linear in the weight
    y = mo.rms_norm_reference(x, w, 0.0)
    torch.testing.assert_close(mo.rms_norm_reference(7.5 * x, w, 0.0), y, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(mo.rms_norm_reference(x, 2 * w, 0.0), 2 * y)
    # eps sits inside the square root, added to the MEAN of squares: x = 0 -> 0, tiny x -> x / sqrt(eps)
    tiny = torch.full((1, 4), 1e-6)
    torch.testing.assert_close(mo.rms_norm_reference(tiny, torch.ones(4), 1e-2), tiny / math.sqrt(1e-12 + 1e-2))
    # bf16 input: fp32 math, one rounding back
    xb = x.to(torch.bfloat16)
    assert mo.rms_norm_reference(xb, w).dtype == torch.bfloat16
    torch.testing.assert_close(mo.rms_norm_reference(xb, w).float(), F.rms_norm(xb.float(), (64,), w, 1e-5),
                               atol=2 ** -6, rtol=2 ** -7)


def test_silu_mul_matches_torch_library_and_rounding_order():
    g = torch.Generator().manual_seed(1)
    a, b = torch.randn(9, 40, generator=g) * 4, torch.randn(9, 40, generator=g)
    torch.testing.assert_close(mo.silu_mul_reference(a, b), F.silu(a) * b, atol=1e-6, rtol=1e-6)
    assert mo.silu_reference(torch.tensor(0.0)) == 0 and abs(mo.silu_reference(torch.tensor(20.0)) - 20.0) < 1e-6
    # bf16: silu is rounded to bf16 BEFORE the product, and the product is a bf16 product
    ab, bb = a.to(torch.bfloat16), b.to(torch.bfloat16)
    want = (F.silu(ab.float()).to(torch.bfloat16).float() * bb.float()).to(torch.bfloat16)
    assert torch.equal(mo.silu_mul_reference(ab, bb), want)


def _library_forward(params, cfg, ids):
    """The same decoder written with torch library routines only (no oracle code)."""
    H, d = cfg["num_heads"], cfg["d_model"]
    dh = d // H
    B, S = ids.shape
    inv = cfg["rope_theta"] ** -(torch.arange(0, dh, 2, dtype=torch.float64) / dh)
    ang = torch.arange(S, dtype=torch.float64)[:, None] * inv[None]
    rot = torch.polar(torch.ones_like(ang), ang)                          # e^{i angle}: rotation as complex multiply

    def rope(t):                                                          # (B,H,S,dh)
        z = torch.view_as_complex(t.double().reshape(B, H, S, dh // 2, 2).contiguous()) * rot
        return torch.view_as_real(z).reshape(B, H, S, dh).float()

    x = F.embedding(ids, params["token_embeddings.weight"])
    for i in range(cfg["num_layers"]):
        pre = f"layers.{i}."
        h = F.rms_norm(x, (d,), params[pre + "attn_norm.weight"], 1e-5)
        q, k, v = (F.linear(h, params[pre + f"attn.{n}.weight"]).view(B, S, H, dh).permute(0, 2, 1, 3)
                   for n in ("q_proj", "k_proj", "v_proj"))
        a = F.scaled_dot_product_attention(rope(q), rope(k), v, is_causal=True)
        x = x + F.linear(a.permute(0, 2, 1, 3).reshape(B, S, d), params[pre + "attn.output_proj.weight"])
        h = F.rms_norm(x, (d,), params[pre + "ffn_norm.weight"], 1e-5)
        x = x + F.linear(F.silu(F.linear(h, params[pre + "ffn.gate_proj.weight"])) *
                         F.linear(h, params[pre + "ffn.up_proj.weight"]), params[pre + "ffn.down_proj.weight"])
    return F.linear(F.rms_norm(x, (d,), params["final_norm.weight"], 1e-5), params["lm_head.weight"])


def test_decoder_matches_torch_library_composition():
    params = mo.random_lm_params(CFG, seed=2)
    ids = torch.randint(0, CFG["vocab_size"], (3, 17), generator=torch.Generator().manual_seed(3))
    torch.testing.assert_close(mo.transformer_lm_reference(params, CFG, ids), _library_forward(params, CFG, ids),
                               atol=2e-4, rtol=2e-4)


def test_decoder_closed_forms_and_causality():
    params = mo.random_lm_params(CFG, seed=4)
    ids = torch.randint(0, CFG["vocab_size"], (2, 11), generator=torch.Generator().manual_seed(5))
    # zero output projections: every block is the identity, logits = lm_head(norm(embedding))
    z = dict(params)
    for i in range(CFG["num_layers"]):
        z[f"layers.{i}.attn.output_proj.weight"] = torch.zeros_like(params[f"layers.{i}.attn.output_proj.weight"])
        z[f"layers.{i}.ffn.down_proj.weight"] = torch.zeros_like(params[f"layers.{i}.ffn.down_proj.weight"])
    emb = params["token_embeddings.weight"][ids]
    want = mo.rms_norm_reference(emb, params["final_norm.weight"]) @ params["lm_head.weight"].T
    torch.testing.assert_close(mo.transformer_lm_reference(z, CFG, ids), want, atol=1e-5, rtol=1e-5)
    # causality: logits at position t do not change when later tokens change
    full = mo.transformer_lm_reference(params, CFG, ids)
    ids2 = ids.clone()
    ids2[:, 6:] = (ids2[:, 6:] + 1) % CFG["vocab_size"]
    torch.testing.assert_close(mo.transformer_lm_reference(params, CFG, ids2)[:, :6], full[:, :6], atol=1e-5, rtol=1e-5)
    assert not torch.allclose(mo.transformer_lm_reference(params, CFG, ids2)[:, 6:], full[:, 6:], atol=1e-3)
    # merged gate/up projection gives the same logits as the separate ones
    m = {k: v for k, v in params.items() if ".ffn." not in k}
    for i in range(CFG["num_layers"]):
        pre = f"layers.{i}.ffn."
        m[pre + "w_gate_up.weight"] = torch.cat((params[pre + "gate_proj.weight"], params[pre + "up_proj.weight"]))
        m[pre + "w_down.weight"] = params[pre + "down_proj.weight"]
    torch.testing.assert_close(mo.transformer_lm_reference(m, CFG, ids), full, atol=1e-5, rtol=1e-5)


def test_attention_block_against_float64_loops():
    """One attention block on a tiny shape, written as explicit loops in float64."""
    g = torch.Generator().manual_seed(6)
    B, S, H, dh = 1, 5, 2, 4
    d = H * dh
    x = torch.randn(B, S, d, generator=g)
    wq, wk, wv, wo = (torch.randn(d, d, generator=g) * 0.3 for _ in range(4))
    freq = att.build_rope_cache(16, dh, 100.0)
    got = mo.attention_block_reference(x, wq, wk, wv, wo, H, freq)
    xd = x.double()[0]
    q, k, v = xd @ wq.double().T, xd @ wk.double().T, xd @ wv.double().T

    def rot(vec, pos):                                                    # vec (dh,), pairs (2i, 2i+1)
        out = vec.clone()
        for i in range(dh // 2):
            ang = pos * 100.0 ** (-(2 * i) / dh)
            c, s = math.cos(ang), math.sin(ang)
            out[2 * i] = c * vec[2 * i] - s * vec[2 * i + 1]
            out[2 * i + 1] = s * vec[2 * i] + c * vec[2 * i + 1]
        return out

    merged = torch.zeros(S, d, dtype=torch.float64)
    for h in range(H):
        sl = slice(h * dh, (h + 1) * dh)
        for t in range(S):
            qt = rot(q[t, sl], t)
            scores = torch.tensor([float(qt @ rot(k[j, sl], j)) / math.sqrt(dh) for j in range(t + 1)], dtype=torch.float64)
            w = torch.exp(scores - scores.max())
            w = w / w.sum()
            merged[t, sl] = sum(w[j] * v[j, sl] for j in range(t + 1))
    want = merged @ wo.double().T
    torch.testing.assert_close(got[0].double(), want, atol=1e-5, rtol=1e-5)


def test_greedy_generate_recomputes_the_whole_context():
    params = mo.random_lm_params(CFG, seed=7)
    prompt = torch.tensor([3, 14, 15, 9, 2])
    toks, logits = mo.greedy_generate_reference(params, CFG, prompt, 6)
    assert toks.shape == (1, 6) and logits.shape == (6, CFG["vocab_size"])
    # step i's logits are the last-position logits of the model on prompt + first i tokens
    ids = torch.cat((prompt[None], toks[:, :3]), dim=-1)
    torch.testing.assert_close(logits[3], mo.transformer_lm_reference(params, CFG, ids)[0, -1])
    assert int(toks[0, 3]) == int(logits[3].argmax())
    # eos stops the loop before the eos token is appended (model.py:229-230)
    t2, _ = mo.greedy_generate_reference(params, CFG, prompt, 6, eos_token_id=int(toks[0, 2]))
    assert torch.equal(t2, toks[:, :2])
    # the context is truncated to context_length (model.py:215)
    long_prompt = torch.arange(60) % CFG["vocab_size"]
    t3, l3 = mo.greedy_generate_reference(params, CFG, long_prompt, 1)
    torch.testing.assert_close(l3[0], mo.transformer_lm_reference(params, CFG, long_prompt[None, -48:])[0, -1])
