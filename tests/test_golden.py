"""Golden fixtures (tests/golden/attention_golden.npz, written by tests/golden/make_fixtures.py from the oracle):
the oracle must still reproduce them (CPU), and the HIP kernels must match them (GPU)."""
import os
import sys

import pytest
import torch

from oracle import attention_oracle as orc

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
from make_fixtures import build, load_golden  # noqa: E402


@pytest.fixture(scope="module")
def gold():
    return load_golden()


def test_fixture_file_is_what_the_generator_writes_today(gold):
    """Oracle drift: regenerating the vectors must give the committed ones (bit-identical inputs, outputs within
    float32 round-off of a differently ordered reduction)."""
    now = build()
    assert sorted(now) == sorted(gold)
    for name, arr in now.items():
        t = torch.from_numpy(arr)
        g = gold[name]
        if t.dtype == torch.int16:
            assert torch.equal(t.view(torch.bfloat16), g), name
        elif t.dtype.is_floating_point:
            assert torch.allclose(t, g, rtol=1e-5, atol=1e-6), name
        else:
            assert torch.equal(t, g), name


def test_oracle_reproduces_golden_outputs(gold):
    q, k, v = gold["dense_q"], gold["dense_k"], gold["dense_v"]
    assert torch.allclose(orc.prefill_reference(q, k, v, causal=True), gold["dense_out_causal"], rtol=1e-5, atol=1e-6)
    out = orc.paged_decode_reference(gold["paged_q"], gold["paged_k_cache"], gold["paged_v_cache"],
                                     gold["paged_block_tables"], gold["paged_context_lens"])
    assert torch.allclose(out, gold["paged_out"], rtol=1e-5, atol=1e-6)
    # the quantiser is bit-exact
    k8, ks = orc.quantize_kv_fp8(gold["paged_k_cache"])
    assert torch.equal(k8.view(torch.uint8), gold["paged_k_fp8"]) and torch.equal(ks, gold["paged_k_scale"])


def _close(got, ref, atol=2e-2, rtol=1e-2):
    err = (got.float().cpu() - ref).abs()
    assert bool((err <= atol + rtol * ref.abs()).all()), f"max err {float(err.max()):.4g}"


@pytest.mark.gpu
def test_kernels_match_golden_outputs(gold):
    import mi355_attn
    mi355_attn.load()
    print("case: golden fixtures", flush=True)
    dev = "cuda:0"
    q, k, v = (gold[n].to(dev) for n in ("dense_q", "dense_k", "dense_v"))
    _close(mi355_attn.scaled_dot_product_attention(q, k, v), gold["dense_out_nomask"])
    _close(mi355_attn.flash_attn_prefill(q, k, v, causal=True), gold["dense_out_causal"])
    q, k, v, cu = (gold[n].to(dev) for n in ("varlen_q", "varlen_k", "varlen_v", "varlen_cu"))
    _close(mi355_attn.flash_attn_varlen_prefill(q, k, v, cu, cu, 20, 20, causal=True), gold["varlen_out"])
    # backward of the last packed sequence (20 tokens) as a dense call
    qq, kk, vv = (t[6:26].transpose(0, 1)[None].contiguous().requires_grad_() for t in (q, k, v))
    mi355_attn.flash_attn_prefill(qq, kk, vv, causal=True).backward(gold["bwd_dout"].to(dev))
    for name, got in (("bwd_dq", qq.grad), ("bwd_dk", kk.grad), ("bwd_dv", vv.grad)):
        ref = gold[name]
        _close(got, ref, atol=2e-2 * float(ref.abs().max()), rtol=2e-2)
    args = [gold[n].to(dev) for n in ("paged_q", "paged_k_cache", "paged_v_cache", "paged_block_tables", "paged_context_lens")]
    _close(mi355_attn.paged_attention_decode(*args), gold["paged_out"])
    out8 = mi355_attn.paged_attention_decode(args[0], gold["paged_k_fp8"].to(dev), gold["paged_v_fp8"].to(dev), args[3], args[4],
                                             k_scale=gold["paged_k_scale"].to(dev), v_scale=gold["paged_v_scale"].to(dev))
    _close(out8, gold["paged_out_fp8"])
    # the HIP quantiser reproduces the stored fp8 bytes and scales exactly
    k8, ks = mi355_attn.quantize_kv_cache_fp8(args[1])
    assert torch.equal(k8.cpu(), gold["paged_k_fp8"]) and torch.equal(ks.cpu(), gold["paged_k_scale"])
    # RoPE through rope_and_cache (queries only): x (heads=2, tokens=7, d) -> (tokens, heads, d)
    x = gold["rope_x"].transpose(0, 1).contiguous().to(dev)
    fc = mi355_attn.build_rope_cache(64, 32, device=dev)
    got = mi355_attn.rope_and_cache(x, x[:, :1], x[:, :1], gold["rope_pos"].to(torch.int32).to(dev), fc)
    _close(got.transpose(0, 1), gold["rope_out"], atol=1e-2, rtol=1e-2)
    torch.cuda.synchronize()
