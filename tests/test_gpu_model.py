"""GPU parity of the operators around attention (RMSNorm, silu*up) and of the KV-cached decoder
(`CachedTransformerLM`) against the CPU oracle of the reference model.

Tolerances.  rms_norm / silu_mul: fp32 math with one rounding to bf16, so within one bf16 ulp of the
oracle's bf16 result: |got - ref| <= 2^-7 |ref| + 1e-3.  Decoder logits: the product path keeps weights,
activations and the residual stream in bf16 while the oracle computes in fp32 on the same bf16-rounded
weights; on the test models (2-3 layers, |logits| up to about 4) the observed error is below 0.03 and the
bound asserted is |got - ref| <= 8e-2 + 3e-2 |ref|.  Cached decode against a full forward of the same
path (same arithmetic, different kernels for attention): <= 3e-2 + 2e-2 |ref|.  Greedy tokens are checked
through the oracle's own logits: a generated token must be within 0.15 of the oracle's maximum at that step.
"""
import json

import pytest
import torch

from oracle import model_oracle as mo

pytestmark = pytest.mark.gpu

CFG = dict(vocab_size=211, context_length=64, d_model=128, num_layers=2, num_heads=4, d_ff=352, rope_theta=10000.0)


@pytest.fixture(scope="module")
def ops():
    import mi355_attn
    mi355_attn.load()
    return mi355_attn


def rnd(*shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


def close_bf16(got, ref):
    torch.testing.assert_close(got.float().cpu(), ref.float(), atol=1e-3, rtol=2 ** -7)


@pytest.mark.parametrize("n_cols", [64, 512, 1000, 1024, 2048, 4096, 8192, 8200, 33])
@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
def test_rms_norm_matches_oracle(ops, n_cols, wdtype):
    print(f"case: rms_norm n_cols={n_cols} weight={wdtype}", flush=True)
    x = rnd(3, 7, n_cols, seed=n_cols, scale=2.5)
    w = (1.0 + 0.2 * torch.randn(n_cols, generator=torch.Generator().manual_seed(1))).to(wdtype)
    ref = mo.rms_norm_reference(x, w, 1e-5)
    y, rstd = ops.rms_norm(x.cuda(), w.cuda(), 1e-5, return_rstd=True)
    torch.cuda.synchronize()
    assert y.shape == x.shape and y.dtype == torch.bfloat16
    close_bf16(y, ref)
    want_rstd = torch.rsqrt(x.float().pow(2).mean(-1) + 1e-5)
    torch.testing.assert_close(rstd.cpu(), want_rstd, atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("n_cols", [128, 1536, 40])
def test_rms_norm_with_fused_residual(ops, n_cols):
    print(f"case: rms_norm residual n_cols={n_cols}", flush=True)
    x, r = rnd(19, n_cols, seed=2), rnd(19, n_cols, seed=3, scale=3.0)
    w = 1.0 + 0.2 * torch.randn(n_cols, generator=torch.Generator().manual_seed(4))
    h_ref = (x.float() + r.float()).to(torch.bfloat16)               # the bf16 add in front of the norm
    y, h = ops.rms_norm(x.cuda(), w.cuda(), 1e-5, residual=r.cuda(), return_sum=True)
    torch.cuda.synchronize()
    assert torch.equal(h.cpu(), h_ref)
    close_bf16(y, mo.rms_norm_reference(h_ref, w, 1e-5))
    # fused == unfused, bit for bit
    assert torch.equal(y, ops.rms_norm(h, w.cuda(), 1e-5))


def test_rms_norm_strided_rows_and_errors(ops):
    print("case: rms_norm strided / errors", flush=True)
    wide = rnd(11, 3 * 256, seed=5).cuda()
    w = torch.ones(256, device="cuda")
    x = wide[:, 256:512]                                              # row stride 768
    assert torch.equal(ops.rms_norm(x, w), ops.rms_norm(x.contiguous(), w))
    assert ops.rms_norm(torch.empty(0, 256, dtype=torch.bfloat16, device="cuda"), w).shape == (0, 256)
    with pytest.raises(ValueError):
        ops.rms_norm(x, torch.ones(255, device="cuda"))
    with pytest.raises(TypeError):
        ops.rms_norm(x.float(), w)
    with pytest.raises(TypeError):
        ops.rms_norm(x, w.half())
    with pytest.raises(ValueError):
        ops.rms_norm(x.cpu(), w)
    with pytest.raises(ValueError):
        ops.rms_norm(x, w, return_sum=True)


@pytest.mark.parametrize("n_cols", [352, 1024, 37])
def test_silu_mul_matches_oracle(ops, n_cols):
    print(f"case: silu_mul n_cols={n_cols}", flush=True)
    g, u = rnd(4, 9, n_cols, seed=6, scale=3.0), rnd(4, 9, n_cols, seed=7)
    ref = mo.silu_mul_reference(g, u)
    out = ops.silu_mul(g.cuda(), u.cuda())
    torch.cuda.synchronize()
    close_bf16(out, ref)
    # exp/sigmoid differ from torch's by an fp32 ulp at most: almost every element is bit-identical
    assert (out.cpu() == ref).float().mean() > 0.99
    # the two halves of one merged projection output, read in place
    gu = torch.cat((g, u), dim=-1).cuda()
    assert torch.equal(ops.silu_mul(gu[..., :n_cols], gu[..., n_cols:]), out)
    with pytest.raises(ValueError):
        ops.silu_mul(g.cuda(), u.cuda()[..., :-1])


def _bf16_params(cfg, seed, fused=False):
    return {k: v.to(torch.bfloat16) for k, v in mo.random_lm_params(cfg, seed, fused_ffn=fused).items()}


def _logit_close(got, ref, atol=8e-2, rtol=3e-2):
    err = (got.float().cpu() - ref).abs()
    bound = atol + rtol * ref.abs()
    assert bool((err <= bound).all()), f"max err {float(err.max()):.4f}, worst excess {float((err - bound).max()):.4f}"


@pytest.mark.parametrize("fused", [False, True])
def test_decoder_forward_matches_oracle(ops, fused):
    print(f"case: decoder forward fused_ffn={fused}", flush=True)
    params = _bf16_params(CFG, seed=11, fused=fused)
    model = ops.CachedTransformerLM(CFG, params, max_batch=8)
    ids = torch.randint(0, CFG["vocab_size"], (3, 41), generator=torch.Generator().manual_seed(12))
    got = model.forward(ids)
    ref = mo.transformer_lm_reference(params, CFG, ids)
    assert got.shape == ref.shape
    _logit_close(got, ref)
    assert model.engine.allocator.num_free == model.engine.allocator.num_blocks


def test_cached_decode_equals_full_forward_and_oracle(ops):
    print("case: cached decode vs full forward", flush=True)
    cfg = dict(CFG, num_layers=3, num_heads=2, d_model=128)          # d_head 64
    params = _bf16_params(cfg, seed=13)
    model = ops.CachedTransformerLM(cfg, params, max_batch=4)
    g = torch.Generator().manual_seed(14)
    seqs = [torch.randint(0, cfg["vocab_size"], (n,), generator=g) for n in (50, 33)]
    n_prompt = [17, 30]
    sids = [model.new_sequence() for _ in seqs]
    logits = model.prefill(sids, [s[:n] for s, n in zip(seqs, n_prompt)])
    per_seq = [[logits[i]] for i in range(2)]
    live = [0, 1]
    pos = list(n_prompt)
    while live:
        lg = model.decode([sids[i] for i in live], [int(seqs[i][pos[i]]) for i in live])
        for j, i in enumerate(live):
            per_seq[i].append(lg[j])
            pos[i] += 1
        live = [i for i in live if pos[i] < len(seqs[i])]
    for i, s in enumerate(seqs):
        got = torch.stack(per_seq[i])                                  # logits after tokens n_prompt-1 .. len-1
        full = model.forward(s)[0, n_prompt[i] - 1:]
        err = (got - full).abs()
        assert bool((err <= 3e-2 + 2e-2 * full.abs()).all()), float(err.max())
        _logit_close(got, mo.transformer_lm_reference(params, cfg, s[None])[0, n_prompt[i] - 1:])
    for s in sids:
        model.free_sequence(s)
    assert model.engine.allocator.num_free == model.engine.allocator.num_blocks


def test_cached_decode_with_fp8_kv_cache_tracks_the_oracle(ops):
    """The same decode loop over an fp8 KV pool (fused quantising cache write + fp8 decode kernel).
    e4m3 keeps 4 significant bits, so the logits carry quantisation noise on top of the bf16 path's: the
    bound asserted is 0.15 + 5e-2 |ref| against the fp32 oracle (observed 0.07), and the mean absolute
    error must stay below 0.03."""
    print("case: cached decode, fp8 KV", flush=True)
    cfg = dict(CFG, num_layers=3, num_heads=2, d_model=128)          # d_head 64
    params = _bf16_params(cfg, seed=13)
    model = ops.CachedTransformerLM(cfg, params, max_batch=4, kv_dtype="fp8")
    assert model.engine.k_caches[0].dtype == torch.uint8
    g = torch.Generator().manual_seed(14)
    seqs = [torch.randint(0, cfg["vocab_size"], (n,), generator=g) for n in (50, 33)]
    n_prompt = [17, 30]
    sids = [model.new_sequence() for _ in seqs]
    logits = model.prefill(sids, [s[:n] for s, n in zip(seqs, n_prompt)])
    per_seq = [[logits[i]] for i in range(2)]
    live, pos = [0, 1], list(n_prompt)
    while live:
        lg = model.decode([sids[i] for i in live], [int(seqs[i][pos[i]]) for i in live])
        for j, i in enumerate(live):
            per_seq[i].append(lg[j])
            pos[i] += 1
        live = [i for i in live if pos[i] < len(seqs[i])]
    for i, s in enumerate(seqs):
        got = torch.stack(per_seq[i]).float().cpu()
        ref = mo.transformer_lm_reference(params, cfg, s[None])[0, n_prompt[i] - 1:]
        err = (got - ref).abs()
        print(f"fp8 KV logits: max err {float(err.max()):.4f} mean {float(err.mean()):.4f}", flush=True)
        assert bool((err <= 0.15 + 5e-2 * ref.abs()).all()), float(err.max())
        assert float(err.mean()) < 0.03
    for s in sids:
        model.free_sequence(s)
    assert model.engine.allocator.num_free == model.engine.allocator.num_blocks


@pytest.mark.parametrize("kv_dtype", ["bf16", "fp8"])
def test_decode_steps_replayed_from_a_hip_graph_equal_eager_steps(ops, kv_dtype):
    """decode_graphs=True: the first step of a batch size runs eagerly and is captured, later steps are
    replays.  Every step of a graphed model is compared with the same step of an eager twin (whose own
    launches and synchronisations sit between the replays); sequences cross block boundaries, one leaves
    (a second batch size, a second graph) and a new one joins."""
    print(f"case: decode graphs, {kv_dtype} KV", flush=True)
    cfg = dict(CFG, num_layers=3, num_heads=2, d_model=128)          # d_head 64
    params = _bf16_params(cfg, seed=21)
    eager = ops.CachedTransformerLM(cfg, params, max_batch=4, kv_dtype=kv_dtype)
    graphed = ops.CachedTransformerLM(cfg, params, max_batch=4, kv_dtype=kv_dtype, decode_graphs=True)
    g = torch.Generator().manual_seed(22)
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g) for n in (13, 30)]
    stream = torch.randint(0, cfg["vocab_size"], (40, 2), generator=g)
    se = [eager.new_sequence() for _ in prompts]
    sg = [graphed.new_sequence() for _ in prompts]
    torch.testing.assert_close(graphed.prefill(sg, prompts), eager.prefill(se, prompts))

    def step(ids_e, ids_g, toks):
        a = eager.decode(ids_e, toks)
        torch.cuda.synchronize()
        b = graphed.decode(ids_g, toks)
        torch.cuda.synchronize()
        err = (a - b).abs()
        assert bool((err <= 2e-2 + 2e-2 * a.abs()).all()), float(err.max())     # same kernels; the attention chunking differs
        return b

    for t in range(20):                                               # 13 -> 33 and 30 -> 50 tokens: new blocks on the way
        step(se, sg, stream[t].tolist())
    assert set(graphed._graphs) == {2} and graphed._graphs[2][1] is not None
    eager.free_sequence(se[0])
    graphed.free_sequence(sg[0])
    for t in range(20, 26):                                           # one sequence left: batch size 1
        step(se[1:], sg[1:], stream[t, 1:].tolist())
    ne, ng = eager.new_sequence(), graphed.new_sequence()             # a newcomer: back to batch size 2, its graph is reused
    p3 = torch.randint(0, cfg["vocab_size"], (5,), generator=g)
    torch.testing.assert_close(graphed.prefill([ng], [p3]), eager.prefill([ne], [p3]))
    for t in range(26, 34):
        last = step([se[1], ne], [sg[1], ng], stream[t].tolist())
    assert set(graphed._graphs) == {1, 2}
    # and against the oracle: the last step of the long sequence
    hist = torch.cat([prompts[1], stream[:26, 1], stream[26:34, 0]])    # what that sequence was fed
    ref = mo.transformer_lm_reference(params, cfg, hist[None])[0, -1]
    err = (last[0].float().cpu() - ref).abs()
    assert bool((err <= (0.15 if kv_dtype == "fp8" else 8e-2) + 5e-2 * ref.abs()).all()), float(err.max())


def _check_greedy(params, cfg, prompt, toks, margin=0.15):
    """Every generated token must be (nearly) the oracle's argmax given the tokens before it, with the
    reference's sliding window (model.py:215)."""
    ids = [int(t) for t in prompt]
    for t in toks:
        ctx = torch.tensor(ids[-cfg["context_length"]:])[None]
        lg = mo.transformer_lm_reference(params, cfg, ctx)[0, -1]
        assert float(lg.max() - lg[t]) <= margin, (len(ids), t, int(lg.argmax()))
        ids.append(int(t))


def test_generate_greedy_follows_oracle_including_window_slide(ops):
    print("case: generate greedy", flush=True)
    params = _bf16_params(CFG, seed=15)
    model = ops.CachedTransformerLM(CFG, params, max_batch=4)
    prompt = torch.randint(0, CFG["vocab_size"], (1, 9), generator=torch.Generator().manual_seed(16))
    out = model.generate(prompt, 12, temperature=0)
    assert out.shape == (1, 12) and out.dtype == torch.int64
    _check_greedy(params, CFG, prompt[0].tolist(), out[0].tolist())
    # eos: generation stops before the eos token (model.py:229-230)
    out2 = model.generate(prompt[0], 12, temperature=0, eos_token_id=int(out[0, 4]))
    first = out[0].tolist().index(int(out[0, 4]))
    assert out2[0].tolist() == out[0].tolist()[:first]
    # prompt close to the context length: the window slides and positions restart (model.py:215)
    long_prompt = torch.randint(0, CFG["vocab_size"], (60,), generator=torch.Generator().manual_seed(17))
    out3 = model.generate(long_prompt, 9, temperature=0)
    _check_greedy(params, CFG, long_prompt.tolist(), out3[0].tolist())
    # a prompt longer than the context is truncated to its last context_length tokens
    over = torch.randint(0, CFG["vocab_size"], (80,), generator=torch.Generator().manual_seed(18))
    out4 = model.generate(over, 3, temperature=0)
    _check_greedy(params, CFG, over.tolist(), out4[0].tolist())
    assert model.engine.allocator.num_free == model.engine.allocator.num_blocks


def test_generate_sampling_and_top_k(ops):
    print("case: generate sampling", flush=True)
    params = _bf16_params(CFG, seed=19)
    model = ops.CachedTransformerLM(CFG, params, max_batch=4)
    prompt = torch.tensor([5, 6, 7, 8])
    g = torch.Generator(device="cuda").manual_seed(1)
    a = model.generate(prompt, 8, temperature=0.8, top_k=5, generator=g)
    g.manual_seed(1)
    b = model.generate(prompt, 8, temperature=0.8, top_k=5, generator=g)
    assert torch.equal(a, b) and a.shape == (1, 8)
    # top_k=1 is greedy whatever the temperature
    assert torch.equal(model.generate(prompt, 6, temperature=1.3, top_k=1), model.generate(prompt, 6, temperature=0))
    # with top_k = 5 every sampled token is among the oracle's 5 best (up to near-ties)
    ids = prompt.tolist()
    for t in a[0].tolist():
        lg = mo.transformer_lm_reference(params, CFG, torch.tensor(ids)[None])[0, -1]
        assert float(torch.topk(lg, 5).values[-1] - lg[t]) <= 0.15
        ids.append(t)


def test_generate_batch_continuous_batching(ops):
    print("case: generate_batch", flush=True)
    params = _bf16_params(CFG, seed=20)
    model = ops.CachedTransformerLM(CFG, params, max_batch=8)
    g = torch.Generator().manual_seed(21)
    prompts = [torch.randint(0, CFG["vocab_size"], (n,), generator=g).tolist() for n in (3, 17, 58, 1, 33)]
    outs = model.generate_batch(prompts, 10, temperature=0)
    assert [len(o) for o in outs] == [10, 10, 64 - 58 + 1, 10, 10]     # the third one fills its context
    for p, o in zip(prompts, outs):
        _check_greedy(params, CFG, p, o)
    eos = outs[1][3]
    outs2 = model.generate_batch(prompts, 10, temperature=0, eos_token_id=eos)
    for o, o2 in zip(outs, outs2):
        want = o[:o.index(eos)] if eos in o else o
        assert o2 == want
    assert model.engine.allocator.num_free == model.engine.allocator.num_blocks
    with pytest.raises(ValueError):
        model.generate_batch([[1]] * 9, 1)


def test_from_pretrained_reads_reference_files(ops, tmp_path):
    print("case: from_pretrained", flush=True)
    params = mo.random_lm_params(CFG, seed=22)
    (tmp_path / "model_config.json").write_text(json.dumps(CFG))
    torch.save({"model": {"_orig_mod." + k: v for k, v in params.items()}}, tmp_path / "ckpt.pt")
    model = ops.CachedTransformerLM.from_pretrained(str(tmp_path / "model_config.json"), str(tmp_path / "ckpt.pt"), max_batch=2)
    ids = torch.arange(20)[None] % CFG["vocab_size"]
    bf = {k: v.to(torch.bfloat16) for k, v in params.items()}
    _logit_close(model.forward(ids), mo.transformer_lm_reference(bf, CFG, ids))
    with pytest.raises(ValueError):
        ops.CachedTransformerLM(dict(CFG, num_heads=8), bf)            # d_head 16 is not supported by the kernels
