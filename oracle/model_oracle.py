"""CPU oracle for the operators around attention and for the whole decoder.  TEST INFRASTRUCTURE ONLY.

Like oracle/attention_oracle.py this module is the checker, never the product: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import it.

Restated from the reference (PyTorch, fp32 math unless said otherwise):

* ``rms_norm_reference``       <- RMSNorm.forward, llm-core/llm_core/model.py:60-67
* ``silu_reference``           <- llm-core/llm_core/model.py:392-393
* ``silu_mul_reference``       <- _silu_mul_fwd_kernel, llm-systems/llm_systems/kernels/triton_swiglu.py:27-47
                                  (silu in fp32, cast to the dtype of ``up``, then the product)
* ``swiglu_reference``         <- SwiGLU.forward, model.py:296-305
* ``attention_block_reference``<- CausalMultiHeadSelfAttention.forward, model.py:352-390
* ``transformer_lm_reference`` <- TransformerLM.forward, model.py:180-185, with TransformerBlock.forward :292-295
* ``greedy_generate_reference``<- the loop of TransformerLM.generate, model.py:210-234, with argmax in place of
                                  the multinomial draw (the draw itself is torch's RNG and is not restated)

Parameters are passed as a dict with the reference's ``state_dict`` names
(``token_embeddings.weight``, ``layers.0.attn.q_proj.weight``, ``layers.0.ffn.gate_proj.weight``,
``layers.0.attn_norm.weight``, ``final_norm.weight``, ``lm_head.weight`` ...).  The merged
projection of FusedSwiGLU (``ffn.w_gate_up.weight`` / ``ffn.w_down.weight``, triton_swiglu.py:173-177)
is accepted too.

Parity pins (tests/test_model_oracle.py): ``rms_norm_reference`` against ``torch.nn.functional.rms_norm``
and the closed forms (constant row, scaling invariance); ``silu_mul_reference`` against
``torch.nn.functional.silu``; the decoder against an independent composition of torch library routines
(``F.embedding``, ``F.linear``, ``F.rms_norm``, ``F.silu``, ``F.scaled_dot_product_attention``), against
closed forms (zero output projections: logits = lm_head(norm(embedding)); one token: attention = V),
causality, and a float64 loop implementation of one block on a tiny shape.
"""
from __future__ import annotations

import math

import torch

from . import attention_oracle as att


def rms_norm_reference(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """model.py:60-67: upcast to fp32, x * rsqrt(mean(x^2) + eps), times weight, cast back."""
    in_dtype = x.dtype
    x32 = x.to(torch.float32)
    rms = torch.rsqrt(x32.pow(2).mean(-1, keepdim=True) + eps)
    return (weight.to(torch.float32) * (x32 * rms)).to(in_dtype)


def silu_reference(x: torch.Tensor) -> torch.Tensor:
    """model.py:392-393."""
    return x * torch.sigmoid(x)


def silu_mul_reference(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """triton_swiglu.py:27-47: silu(gate) in fp32, cast to up's dtype, times up (in up's dtype)."""
    return silu_reference(gate.to(torch.float32)).to(up.dtype) * up


def swiglu_reference(x, w_gate, w_up, w_down):
    """model.py:304-305: W2(silu(W1 x) * W3 x); weights are (d_out, d_in) as in Linear (model.py:26-31)."""
    return (silu_reference(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


def _ffn_weights(params, prefix):
    if prefix + "ffn.gate_proj.weight" in params:
        return (params[prefix + "ffn.gate_proj.weight"], params[prefix + "ffn.up_proj.weight"],
                params[prefix + "ffn.down_proj.weight"])
    merged = params[prefix + "ffn.w_gate_up.weight"]          # first d_ff rows = gate, last d_ff rows = up
    d_ff = merged.shape[0] // 2
    return merged[:d_ff], merged[d_ff:], params[prefix + "ffn.w_down.weight"]


def attention_core_reference(q_proj, k_proj, v_proj, num_heads, freq_cache, positions=None):
    """model.py:366-388 from the three projection outputs (batch, seq, heads*d_head) on: split heads, RoPE on Q
    and K, causal attention (model.py:384-385), merge heads -> (batch, seq, heads*d_head)."""
    B, S, d_model = q_proj.shape
    d_head = d_model // num_heads

    def split(t):                                             # (B,S,H*d) -> (B,H,S,d), model.py:366-370
        return t.view(B, S, num_heads, d_head).transpose(1, 2)

    Q, K, V = split(q_proj), split(k_proj), split(v_proj)
    if positions is None:
        positions = torch.arange(S).expand(B, S)              # model.py:373-374
    pos = positions[:, None, :].expand(B, num_heads, S)
    Q = att.rope_reference(Q, pos, freq_cache)
    K = att.rope_reference(K, pos, freq_cache)
    out = att.scaled_dot_product_attention(Q, K, V, att.causal_keep_mask(S))
    return out.transpose(1, 2).reshape(B, S, d_model)         # model.py:388


def attention_block_reference(x, wq, wk, wv, wo, num_heads, freq_cache, positions=None):
    """model.py:352-390 for x (batch, seq, d_model): project (model.py:362-364), attention_core_reference,
    output projection (model.py:390)."""
    merged = attention_core_reference(x @ wq.T, x @ wk.T, x @ wv.T, num_heads, freq_cache, positions)
    return merged @ wo.T


def transformer_lm_reference(params: dict, config: dict, token_ids: torch.Tensor) -> torch.Tensor:
    """TransformerLM.forward (model.py:180-185) in fp32: logits (batch, seq, vocab)."""
    p = {k: v.to(torch.float32) for k, v in params.items()}
    H = config["num_heads"]
    d_head = config["d_model"] // H
    freq = att.build_rope_cache(config["context_length"], d_head, config["rope_theta"])
    x = p["token_embeddings.weight"][token_ids]               # model.py:50
    for i in range(config["num_layers"]):
        pre = f"layers.{i}."
        h = rms_norm_reference(x, p[pre + "attn_norm.weight"])
        x = x + attention_block_reference(h, p[pre + "attn.q_proj.weight"], p[pre + "attn.k_proj.weight"],
                                          p[pre + "attn.v_proj.weight"], p[pre + "attn.output_proj.weight"], H, freq)
        h = rms_norm_reference(x, p[pre + "ffn_norm.weight"])
        x = x + swiglu_reference(h, *_ffn_weights(p, pre))
    x = rms_norm_reference(x, p["final_norm.weight"])
    return x @ p["lm_head.weight"].T


def greedy_generate_reference(params: dict, config: dict, prompt_ids: torch.Tensor, max_new_tokens: int,
                              eos_token_id: int | None = None):
    """The loop of TransformerLM.generate (model.py:210-234) with argmax instead of the multinomial draw:
    the whole context is run through the model for every new token (:218).  Returns (tokens (1, n), the
    next-token logits of every step (n, vocab))."""
    if prompt_ids.dim() == 1:
        prompt_ids = prompt_ids[None]
    ids = prompt_ids
    out, all_logits = [], []
    for _ in range(max_new_tokens):
        ctx = ids[:, -config["context_length"]:]
        logits = transformer_lm_reference(params, config, ctx)[:, -1]
        nxt = logits.argmax(-1, keepdim=True)
        all_logits.append(logits[0])
        if eos_token_id is not None and nxt.item() == eos_token_id:
            break
        ids = torch.cat((ids, nxt), dim=-1)
        out.append(nxt)
    toks = torch.cat(out, dim=-1) if out else ids[:, 0:0]
    return toks, (torch.stack(all_logits) if all_logits else torch.empty(0, config["vocab_size"]))


def random_lm_params(config: dict, seed: int = 0, fused_ffn: bool = False) -> dict:
    """Random parameters with the reference's names, shapes and initial scales (Linear: std sqrt(2/(in+out)),
    model.py:24-27; Embedding: std 1, model.py:41-45; norm weights near 1)."""
    g = torch.Generator().manual_seed(seed)
    d, ff, V, L = config["d_model"], config["d_ff"], config["vocab_size"], config["num_layers"]

    def lin(d_out, d_in):
        return torch.randn(d_out, d_in, generator=g) * math.sqrt(2.0 / (d_in + d_out))

    p = {"token_embeddings.weight": torch.randn(V, d, generator=g), "lm_head.weight": lin(V, d),
         "final_norm.weight": 1.0 + 0.1 * torch.randn(d, generator=g)}
    for i in range(L):
        pre = f"layers.{i}."
        for n in ("q_proj", "k_proj", "v_proj", "output_proj"):
            p[pre + f"attn.{n}.weight"] = lin(d, d)
        if fused_ffn:
            p[pre + "ffn.w_gate_up.weight"] = lin(2 * ff, d)
            p[pre + "ffn.w_down.weight"] = lin(d, ff)
        else:
            p[pre + "ffn.gate_proj.weight"] = lin(ff, d)
            p[pre + "ffn.up_proj.weight"] = lin(ff, d)
            p[pre + "ffn.down_proj.weight"] = lin(d, ff)
        p[pre + "attn_norm.weight"] = 1.0 + 0.1 * torch.randn(d, generator=g)
        p[pre + "ffn_norm.weight"] = 1.0 + 0.1 * torch.randn(d, generator=g)
    return p
