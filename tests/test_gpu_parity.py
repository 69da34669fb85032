"""GPU parity: the HIP kernels (through the C ABI) against the CPU oracle.

Tolerance for bf16 paths (from the task statement): |out - ref| <= 2e-2 + 1e-2*|ref|
against the fp32 oracle evaluated on the same bf16-rounded inputs.
fp8-KV decode: the same tight bound against the oracle on the DEQUANTISED cache
(this is the parity gate of the kernel), and, against the oracle on the original
bf16 cache, the quantisation-noise bound |out - ref| <= 0.15 + 2^-4*|ref| per
element (e4m3 rounds with relative error <= 2^-4, so a one-key context is off by
at most 2^-4*|v|; short contexts add the softmax-weight perturbation, covered by
the absolute term) together with rms(out - ref) <= 0.06 * rms(ref).
"""
import math

import pytest
import torch

from oracle import attention_oracle as orc

pytestmark = pytest.mark.gpu

ATOL, RTOL = 2e-2, 1e-2
FP8_ATOL, FP8_RTOL, FP8_RMS = 0.15, 2.0 ** -4, 0.06


@pytest.fixture(scope="module")
def ops():
    import mi355_attn
    mi355_attn.load()            # raises if the HIP library is not built: no fallback
    return mi355_attn


def check(got, ref, atol=ATOL, rtol=RTOL, what=""):
    got = got.float().cpu()
    ref = ref.float()
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    err = (got - ref).abs()
    bound = atol + rtol * ref.abs()
    worst = (err - bound).max().item()
    assert worst <= 0, f"{what}: max err {err.max().item():.4g}, exceeds bound by {worst:.4g}"


def rnd(*shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


# --------------------------------------------------------------------------
# paged decode
# --------------------------------------------------------------------------
def run_decode(ops, q, kc, vc, bt, cl, **kw):
    dev = "cuda:0"
    args = [t.to(dev) for t in (q, kc, vc, bt, cl)]
    kw = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in kw.items()}
    out = ops.paged_attention_decode(*args, **kw)
    torch.cuda.synchronize()
    return out


def test_decode_config0_shape(ops):
    """B4, 8 q = 8 kv heads, D64, block 16, ctx 256, 64-block pool (the CPU-path configuration)."""
    print("case: decode config0", flush=True)
    q, kc, vc, bt, cl = orc.make_paged_case(batch=4, n_q_heads=8, n_kv_heads=8, head_dim=64, block_size=16,
                                            context_lens=[256] * 4, seed=0, dtype=torch.bfloat16)
    ref = orc.paged_decode_reference(q, kc, vc, bt, cl)
    check(run_decode(ops, q, kc, vc, bt, cl), ref, what="config0")


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("Hq,Hkv", [(4, 4), (8, 2), (16, 2), (16, 1)])
def test_decode_ragged_edges(ops, D, Hq, Hkv):
    ctx = [1, 15, 16, 17, 31, 32, 33, 255, 256, 257, 1023, 1024, 1025, 2049, 3000]
    print(f"case: decode ragged D={D} Hq={Hq} Hkv={Hkv}", flush=True)
    q, kc, vc, bt, cl = orc.make_paged_case(batch=len(ctx), n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D,
                                            block_size=16, context_lens=ctx, pool_factor=1.3, seed=D + Hq,
                                            dtype=torch.bfloat16)
    ref = orc.paged_decode_reference(q, kc, vc, bt, cl)
    check(run_decode(ops, q, kc, vc, bt, cl), ref, what=f"ragged D{D} {Hq}/{Hkv}")


@pytest.mark.parametrize("fp8", [False, True])
def test_decode_long_contexts_multi_chunk(ops, fp8):
    """Contexts around the 4096-token workgroup chunk used for long batches, several chunks per sequence."""
    ctx = [4095, 4096, 4097, 8191, 8193, 12000, 33, 1]
    print(f"case: decode long contexts fp8={fp8}", flush=True)
    q, kc, vc, bt, cl = orc.make_paged_case(batch=len(ctx), n_q_heads=8, n_kv_heads=2, head_dim=128, block_size=16,
                                            context_lens=ctx, pool_factor=1.1, seed=77, dtype=torch.bfloat16)
    if fp8:
        k8, ks = orc.quantize_kv_fp8(kc)
        v8, vs = orc.quantize_kv_fp8(vc)
        got = run_decode(ops, q, k8, v8, bt, cl, k_scale=ks, v_scale=vs)
        ref = orc.paged_decode_reference(q, k8, v8, bt, cl, k_scale=ks, v_scale=vs)
    else:
        got = run_decode(ops, q, kc, vc, bt, cl)
        ref = orc.paged_decode_reference(q, kc, vc, bt, cl)
    check(got, ref, what=f"long contexts fp8={fp8}")


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("ctx", [1025, 9000])
def test_decode_of_one_sequence_uses_the_shortest_chunks(ops, fp8, ctx):
    """One sequence on two kv heads: far fewer workgroups than compute units at any chunk size, so the split-K pass
    runs with its shortest chunks (4 wavefronts x 64 tokens; 5 and 36 chunks here, the last one partial) and the
    combine pass merges them."""
    print(f"case: decode one sequence ctx={ctx} fp8={fp8}", flush=True)
    q, kc, vc, bt, cl = orc.make_paged_case(batch=1, n_q_heads=8, n_kv_heads=2, head_dim=128, block_size=16,
                                            context_lens=[ctx], pool_factor=1.3, seed=91, dtype=torch.bfloat16)
    if fp8:
        k8, ks = orc.quantize_kv_fp8(kc)
        v8, vs = orc.quantize_kv_fp8(vc)
        got = run_decode(ops, q, k8, v8, bt, cl, k_scale=ks, v_scale=vs)
        ref = orc.paged_decode_reference(q, k8, v8, bt, cl, k_scale=ks, v_scale=vs)
    else:
        got = run_decode(ops, q, kc, vc, bt, cl)
        ref = orc.paged_decode_reference(q, kc, vc, bt, cl)
    check(got, ref, what=f"one sequence ctx={ctx} fp8={fp8}")


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("batch,ctx", [(1, 20000), (3, 5000), (9, 1500)])
def test_decode_of_few_sequences_combines_many_chunks(ops, D, batch, ctx):
    """Few sequences of long contexts run short chunks, up to hundreds per sequence, and their partial results are
    merged by the combine kernel that gives a workgroup to every row (more than four chunks per sequence, at most
    2048 rows): ragged lengths, so that rows of one launch have 1 to n chunks, every head size."""
    print(f"case: decode few sequences D={D} batch={batch} ctx={ctx}", flush=True)
    lens = [max(1, ctx - 977 * i) for i in range(batch)]
    q, kc, vc, bt, cl = orc.make_paged_case(batch=batch, n_q_heads=8, n_kv_heads=2, head_dim=D, block_size=16,
                                            context_lens=lens, pool_factor=1.2, seed=93, dtype=torch.bfloat16)
    got = run_decode(ops, q, kc, vc, bt, cl)
    ref = orc.paged_decode_reference(q, kc, vc, bt, cl)
    check(got, ref, what=f"few sequences D={D} batch={batch} ctx={ctx}")


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("slope", [0.4, 0.02, -0.02, -0.4])
def test_decode_scores_that_ramp_along_the_context(ops, fp8, slope):
    """Scores that rise (or fall) steadily with the token position, by much more or much less per 32-key step than
    the slack of the kernel's lazily moved exponent reference, plus one isolated spike in the middle: the output
    must follow the oracle whether the reference moves every step, every few steps or never."""
    ctx = [40, 700, 2500, 5000]
    D, Hq, Hkv = 128, 4, 2
    print(f"case: decode ramp slope={slope} fp8={fp8}", flush=True)
    q, kc, vc, bt, cl = orc.make_paged_case(batch=len(ctx), n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, block_size=16,
                                            context_lens=ctx, pool_factor=1.2, seed=31, dtype=torch.bfloat16)
    q = (q.float() * 0.05)
    q[:, :, 0] = math.sqrt(D)                     # score of token t = K[t, 0] + small noise (scale 1/sqrt(D))
    q[:, 1::2, 0] = -math.sqrt(D)                 # every other query head sees the ramp the other way round
    q = q.to(torch.bfloat16)
    for b, n in enumerate(ctx):
        t = torch.arange(n, dtype=torch.float32)
        col = slope * t
        col[n // 2] += 30.0 if slope > 0 else -30.0            # a spike (for the odd heads: a dip)
        for j in range((n + 15) // 16):
            rows = col[16 * j:16 * j + 16]
            kc[int(bt[b, j]), :, :rows.numel(), 0] = rows.to(torch.bfloat16)[None]
    if fp8:
        k8, ks = orc.quantize_kv_fp8(kc)
        v8, vs = orc.quantize_kv_fp8(vc)
        got = run_decode(ops, q, k8, v8, bt, cl, k_scale=ks, v_scale=vs)
        ref = orc.paged_decode_reference(q, k8, v8, bt, cl, k_scale=ks, v_scale=vs)
    else:
        got = run_decode(ops, q, kc, vc, bt, cl)
        ref = orc.paged_decode_reference(q, kc, vc, bt, cl)
    check(got, ref, what=f"ramp slope={slope} fp8={fp8}")


def test_decode_ignores_pool_garbage_and_table_tail(ops):
    """NaN/Inf bit patterns in unused blocks, in the tail of the last block and junk table entries are never used."""
    ctx = [5, 40, 100, 1030]
    print("case: decode garbage", flush=True)
    q, kc, vc, bt, cl = orc.make_paged_case(batch=4, n_q_heads=8, n_kv_heads=2, head_dim=128, block_size=16,
                                            context_lens=ctx, pool_factor=1.5, seed=7, dtype=torch.bfloat16)
    ref = orc.paged_decode_reference(q, kc, vc, bt, cl)
    used = torch.zeros(kc.shape[0], dtype=torch.bool)
    bt2 = bt.clone()
    for b, c in enumerate(ctx):
        n = (c + 15) // 16
        used[bt[b, :n].long()] = True
        bt2[b, n:] = 2 ** 30                    # junk ids past the sequence's blocks
    kc2, vc2 = kc.clone(), vc.clone()
    kc2[~used] = float("nan")
    vc2[~used] = float("inf")
    for b, c in enumerate(ctx):
        if c % 16:
            last = int(bt[b, (c - 1) // 16])
            kc2[last, :, c % 16:] = float("nan")
            vc2[last, :, c % 16:] = float("nan")
    check(run_decode(ops, q, kc2, vc2, bt2, cl), ref, what="garbage")


def test_decode_custom_scale_and_workspace_reuse(ops):
    ctx = [3000, 100]
    print("case: decode scale/workspace", flush=True)
    q, kc, vc, bt, cl = orc.make_paged_case(batch=2, n_q_heads=8, n_kv_heads=2, head_dim=128, block_size=16,
                                            context_lens=ctx, seed=11, dtype=torch.bfloat16)
    ref = orc.paged_decode_reference(q, kc, vc, bt, cl, softmax_scale=0.05)
    ws = ops.paged_decode_workspace(2, 8, 128, 3008, "cuda:0")
    ws.fill_(0xFF)                               # stale workspace contents must not matter
    got = run_decode(ops, q, kc, vc, bt, cl, softmax_scale=0.05, workspace=ws, max_context=3008)
    check(got, ref, what="scale")
    got2 = run_decode(ops, q, kc, vc, bt, cl, softmax_scale=0.05, workspace=ws, max_context=3008)
    assert torch.equal(got, got2)                # deterministic, no atomics


@pytest.mark.parametrize("D,Hq,Hkv", [(128, 16, 2), (64, 8, 8), (128, 8, 1)])
def test_decode_fp8_kv(ops, D, Hq, Hkv):
    ctx = [1, 16, 17, 100, 1024, 1025, 2500]
    print(f"case: decode fp8 D={D} Hq={Hq} Hkv={Hkv}", flush=True)
    q, kc, vc, bt, cl = orc.make_paged_case(batch=len(ctx), n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D,
                                            block_size=16, context_lens=ctx, pool_factor=1.2, seed=3 + D,
                                            dtype=torch.bfloat16)
    k8, ks = orc.quantize_kv_fp8(kc)
    v8, vs = orc.quantize_kv_fp8(vc)
    got = run_decode(ops, q, k8, v8, bt, cl, k_scale=ks, v_scale=vs)
    ref_dq = orc.paged_decode_reference(q, k8, v8, bt, cl, k_scale=ks, v_scale=vs)
    check(got, ref_dq, what="fp8 vs oracle on dequantised cache")
    ref_bf = orc.paged_decode_reference(q, kc, vc, bt, cl)
    check(got, ref_bf, FP8_ATOL, FP8_RTOL, what="fp8 vs oracle on bf16 cache")
    err = got.float().cpu() - ref_bf
    assert err.pow(2).mean().sqrt() <= FP8_RMS * ref_bf.pow(2).mean().sqrt()


def test_decode_equals_last_row_of_prefill(ops):
    """Round trip between the two kernels: decode over a cache == last query row of causal prefill."""
    S, Hq, Hkv, D = 700, 8, 2, 128
    print("case: decode vs prefill", flush=True)
    q, k, v = rnd(1, Hq, S, D, seed=21), rnd(1, Hkv, S, D, seed=22), rnd(1, Hkv, S, D, seed=23)
    nblk = (S + 15) // 16
    perm = torch.randperm(nblk + 5, generator=torch.Generator().manual_seed(1))[:nblk]
    kc = torch.zeros(nblk + 5, Hkv, 16, D, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    kp = torch.zeros(1, Hkv, nblk * 16, D, dtype=torch.bfloat16)
    vp = torch.zeros_like(kp)
    kp[:, :, :S], vp[:, :, :S] = k, v
    kc[perm] = kp[0].reshape(Hkv, nblk, 16, D).permute(1, 0, 2, 3)
    vc[perm] = vp[0].reshape(Hkv, nblk, 16, D).permute(1, 0, 2, 3)
    dec = run_decode(ops, q[0, :, -1].unsqueeze(0).contiguous(), kc, vc, perm.to(torch.int32)[None].contiguous(),
                     torch.tensor([S], dtype=torch.int32))
    pre = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=True)[0, :, -1]
    check(dec[0], pre.float().cpu(), what="decode vs prefill last row")


# --------------------------------------------------------------------------
# prefill
# --------------------------------------------------------------------------
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("S", [1, 17, 64, 128, 129, 333, 1024])
@pytest.mark.parametrize("causal", [True, False])
def test_prefill_dense_mha(ops, D, S, causal):
    print(f"case: prefill dense D={D} S={S} causal={causal}", flush=True)
    B, H = 2, 3
    q, k, v = rnd(B, H, S, D, seed=1, scale=0.5), rnd(B, H, S, D, seed=2, scale=0.5), rnd(B, H, S, D, seed=3, scale=0.5)
    ref = orc.prefill_reference(q, k, v, causal=causal)
    got = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=causal)
    torch.cuda.synchronize()
    check(got, ref, what=f"prefill D{D} S{S} causal={causal}")


def test_prefill_config1_shape_and_reference_layout(ops):
    """B4 H16 D64 S1024 causal, with V given as the strided view the reference builds (model.py:367-370)."""
    print("case: prefill config1", flush=True)
    B, H, S, D = 4, 16, 1024, 64
    q, k = rnd(B, H, S, D, seed=4, scale=0.5), rnd(B, H, S, D, seed=5, scale=0.5)
    v_proj = rnd(B, S, H * D, seed=6, scale=0.5)                       # (B, S, H*D) projection output
    v = v_proj.view(B, S, H, D).permute(0, 2, 1, 3)                    # (B, H, S, D) non-contiguous view
    ref = orc.prefill_reference(q, k, v, causal=True)
    vg = v_proj.cuda().view(B, S, H, D).permute(0, 2, 1, 3)
    assert not vg.is_contiguous()
    got = ops.sdpa_slot(q.cuda(), k.cuda(), vg, is_causal=True)
    torch.cuda.synchronize()
    check(got, ref, what="config1")
    # output memory is (B, S, H, D): merging heads like model.py:388 is a free view
    merged = got.permute(0, 2, 1, 3).reshape(B, S, H * D)
    assert merged.data_ptr() == got.data_ptr()


@pytest.mark.parametrize("Hq,Hkv,D", [(8, 2, 128), (6, 3, 64), (8, 1, 128)])
def test_prefill_gqa(ops, Hq, Hkv, D):
    print(f"case: prefill gqa {Hq}/{Hkv} D={D}", flush=True)
    B, S = 2, 300
    q, k, v = rnd(B, Hq, S, D, seed=7, scale=0.5), rnd(B, Hkv, S, D, seed=8, scale=0.5), rnd(B, Hkv, S, D, seed=9, scale=0.5)
    ref = orc.prefill_reference(q, k, v, causal=True)
    got = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=True)
    check(got, ref, what="gqa")


def test_prefill_rectangular_causal_and_scale(ops):
    """Sk > Sq: queries are the last Sq positions (bottom-right aligned diagonal); custom softmax scale."""
    print("case: prefill rect", flush=True)
    B, H, Sq, Sk, D = 1, 4, 100, 391, 128
    q, k, v = rnd(B, H, Sq, D, seed=10, scale=0.5), rnd(B, H, Sk, D, seed=11, scale=0.5), rnd(B, H, Sk, D, seed=12, scale=0.5)
    ref = orc.prefill_reference(q, k, v, causal=True, softmax_scale=0.2)
    got = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=True, softmax_scale=0.2)
    check(got, ref, what="rect causal")
    ref = orc.prefill_reference(q, k, v, causal=False)
    got = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=False)
    check(got, ref, what="rect full")


@pytest.mark.parametrize("lens", [[5, 1, 12, 130], [128, 256, 64], [1000, 3, 517]])
def test_prefill_varlen_ragged(ops, lens):
    print(f"case: prefill varlen {lens}", flush=True)
    Hq, Hkv, D = 8, 2, 128
    T = sum(lens)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    q, k, v = rnd(T, Hq, D, seed=13, scale=0.5), rnd(T, Hkv, D, seed=14, scale=0.5), rnd(T, Hkv, D, seed=15, scale=0.5)
    ref = orc.varlen_prefill_reference(q, k, v, cu, cu, causal=True)
    got = ops.flash_attn_varlen_prefill(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), cu.cuda(), max(lens), max(lens),
                                        causal=True)
    check(got, ref, what="varlen")


@pytest.mark.parametrize("Sq,Sk", [(256, 4096), (700, 1500), (64, 191), (513, 64), (300, 8192 + 37)])
def test_prefill_unmasked_head_dim_128_long_and_ragged(ops, Sq, Sk):
    """head_dim 128 without a mask runs on the kernel with 64 queries per wavefront, whose loop over whole K/V tiles
    is hand-scheduled assembly: many tiles, ragged query and key ends (the assembly stops three tiles before a
    partial last tile), GQA, fewer rows than a wavefront owns."""
    print(f"case: prefill unmasked D128 Sq={Sq} Sk={Sk}", flush=True)
    B, Hq, Hkv, D = 2, 4, 2, 128
    q, k, v = rnd(B, Hq, Sq, D, seed=81, scale=0.5), rnd(B, Hkv, Sk, D, seed=82, scale=0.5), rnd(B, Hkv, Sk, D, seed=83, scale=0.5)
    ref = orc.prefill_reference(q, k, v, causal=False)
    got = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=False, kv_splits=1)
    torch.cuda.synchronize()
    check(got, ref, what=f"unmasked D128 {Sq}x{Sk}")
    # the default may split the keys of so small a launch over several workgroups (another kernel and a merge)
    check(ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=False), ref, what=f"unmasked D128 {Sq}x{Sk}, default")
    # the reference's own signature (no GQA there: first kv head only)
    got2 = ops.scaled_dot_product_attention(q[:, :2].cuda(), k[:, :1].cuda(), v[:, :1].cuda())
    check(got2, ref[:, :2], what=f"unmasked D128 {Sq}x{Sk}, reference signature")


def test_prefill_unmasked_scores_that_outgrow_the_reference(ops):
    """Keys far along the sequence whose scores exceed everything before them by hundreds of binary orders: the
    assembly loop sees a weight reach 2, leaves (once with nothing of the tile accumulated, once with half of it),
    ordinary code moves the reference and the loop resumes.  Also a block of keys with hugely negative scores."""
    print("case: prefill unmasked D128, reference moves", flush=True)
    B, H, Sq, Sk, D = 1, 2, 128, 2048, 128
    q, k, v = rnd(B, H, Sq, D, seed=84, scale=1.0), rnd(B, H, Sk, D, seed=85, scale=1.0), rnd(B, H, Sk, D, seed=86, scale=1.0)
    k = k.float()
    k[:, :, 700] *= 9.0            # keys 0..31 of tile 10: first check of that tile
    k[:, :, 1000] *= 30.0          # key 40 of tile 15: second check (keys 32..63)
    k[:, :, 1300:1364] *= -25.0    # a whole tile of extreme scores of both signs
    k[:, :, 1999] *= 60.0
    k = k.to(torch.bfloat16)
    ref = orc.prefill_reference(q, k, v, causal=False)
    got = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=False)
    torch.cuda.synchronize()
    check(got, ref, what="reference moves")
    # the same through the 8-wavefront kernel (an all-true explicit mask takes that path): both must agree with the oracle
    keep = torch.ones(Sq, Sk, dtype=torch.bool, device="cuda")
    check(ops.scaled_dot_product_attention(q.cuda(), k.cuda(), v.cuda(), keep), ref, what="reference moves, masked path")


@pytest.mark.parametrize("D", [32, 64])
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_prefill_head_dim_64_32_preset_reference_against_tracked_maxima(ops, D, seed):
    """The 8-wavefront kernel first runs a query tile with a preset exponent reference, watching row sums, and runs it
    again with the reference tracked from the row maxima when a row's sum leaves the safe range.  An explicit
    all-visible mask takes the tracked path from the start, so the two paths can be compared with each other and with
    the oracle: drawn shapes (ragged, more keys than queries, GQA, causal or not), keys whose scores run away by
    tens to thousands of binary orders in both directions (rescaling in the loop, second attempts), keys split over
    workgroups, and rows whose scores are all hugely negative."""
    g = torch.Generator().manual_seed(3000 + 10 * D + seed)
    for case in range(5):
        B = int(torch.randint(1, 3, (1,), generator=g))
        Hkv = int(torch.randint(1, 3, (1,), generator=g))
        Hq = Hkv * int(torch.randint(1, 3, (1,), generator=g))
        Sq = int(torch.randint(1, 700, (1,), generator=g))
        Sk = Sq + int(torch.randint(0, 700, (1,), generator=g)) * int(torch.randint(0, 2, (1,), generator=g))
        causal = bool(torch.randint(0, 2, (1,), generator=g))
        print(f"case: preset/tracked D={D} seed={seed} #{case} B={B} Hq={Hq} Hkv={Hkv} Sq={Sq} Sk={Sk} causal={causal}", flush=True)
        q = torch.randn(B, Hq, Sq, D, generator=g).to(torch.bfloat16)
        k = torch.randn(B, Hkv, Sk, D, generator=g)
        v = torch.randn(B, Hkv, Sk, D, generator=g).to(torch.bfloat16)
        for _ in range(int(torch.randint(0, 6, (1,), generator=g))):          # runaway keys
            j = int(torch.randint(0, Sk, (1,), generator=g))
            n = int(torch.randint(1, 70, (1,), generator=g))
            k[:, :, j:j + n] *= float(torch.tensor([6.0, 20.0, -15.0, 45.0, 300.0])[int(torch.randint(0, 5, (1,), generator=g))])
        if case == 4:                                  # every score of the first head pair far below the preset reference
            k[:, 0] = k[:, 0].abs() * 12.0
            q[:, :Hq // Hkv] = -(q[:, :Hq // Hkv].float().abs() * 2.0).to(torch.bfloat16)
        k = k.to(torch.bfloat16)
        ref = orc.prefill_reference(q, k, v, causal=causal)
        fast = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=causal, kv_splits=1)
        keep = torch.ones(Sq, Sk, dtype=torch.bool)
        if causal:
            keep = torch.tril(keep, diagonal=Sk - Sq)
        slow = ops.scaled_dot_product_attention(q.cuda(), k.cuda().repeat_interleave(Hq // Hkv, 1),
                                                v.cuda().repeat_interleave(Hq // Hkv, 1), keep.cuda())
        shared = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=causal, kv_splits=2 + (seed + case) % 3)
        torch.cuda.synchronize()
        check(fast, ref, what=f"preset reference D={D} seed {seed} #{case}")
        check(slow, ref, what=f"tracked maxima D={D} seed {seed} #{case}")
        check(shared, ref, what=f"preset reference, keys split, D={D} seed {seed} #{case}")


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("splits", [2, 5, 64])
def test_prefill_split_keys_dense(ops, D, splits):
    """Every sequence's keys split over several workgroups whose fp32 partial rows a second kernel merges: causal
    (early rows see no key of the later shares: those partials are empty), rectangular, unmasked, GQA, more shares
    than K/V tiles, a ragged last query tile."""
    print(f"case: prefill split keys D={D} splits={splits}", flush=True)
    B, Hq, Hkv, Sq, Sk = 2, 4, 2, 333, 1500
    q, k, v = rnd(B, Hq, Sq, D, seed=91, scale=0.5), rnd(B, Hkv, Sk, D, seed=92, scale=0.5), rnd(B, Hkv, Sk, D, seed=93, scale=0.5)
    for causal in (True, False):
        ref = orc.prefill_reference(q, k, v, causal=causal)
        got = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=causal, kv_splits=splits)
        torch.cuda.synchronize()
        check(got, ref, what=f"split keys D{D} x{splits} causal={causal}")
    # square causal: the first query tile's later shares hold no tile at all
    ref = orc.prefill_reference(q, k[:, :, :Sq], v[:, :, :Sq], causal=True)
    ws = ops.prefill_splitkv_workspace(B * Sq, Hq, D, splits, "cuda:0")
    got = ops.flash_attn_prefill(q.cuda(), k[:, :, :Sq].cuda(), v[:, :, :Sq].cuda(), causal=True, kv_splits=splits, workspace=ws)
    check(got, ref, what=f"split keys square D{D} x{splits}")


def test_prefill_split_keys_is_chosen_for_few_long_sequences(ops):
    """A chunk of one prompt over a long context (one workgroup per pair of query tiles would occupy 8 of 256
    compute units): the default splits the keys; the result agrees with the unsplit kernel to rounding and with
    the oracle to tolerance."""
    print("case: prefill split keys, automatic", flush=True)
    B, Hq, Hkv, Sq, Sk, D = 1, 8, 2, 512, 4096, 128
    q, k, v = rnd(B, Hq, Sq, D, seed=94, scale=0.5), rnd(B, Hkv, Sk, D, seed=95, scale=0.5), rnd(B, Hkv, Sk, D, seed=96, scale=0.5)
    assert ops.suggest_kv_splits(B, Hq, D, Sq, Sk, B * Sq, True, torch.device("cuda:0")) > 1
    ref = orc.prefill_reference(q, k, v, causal=True)
    auto = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=True)
    one = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=True, kv_splits=1)
    torch.cuda.synchronize()
    check(auto, ref, what="auto split")
    check(one, ref, what="unsplit")
    assert not torch.equal(auto, one)            # (another kernel, another order of summation)
    assert (auto.float() - one.float()).abs().max().item() <= 2e-2
    with pytest.raises(ValueError):
        ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=True, kv_splits=65)


@pytest.mark.parametrize("splits", [3, 16])
def test_prefill_split_keys_varlen_and_paged(ops, splits):
    """Packed sequences of ragged lengths (one of them empty of keys for some shares, one a single token) and chunks
    over a paged cache, keys split."""
    print(f"case: prefill split keys varlen/paged splits={splits}", flush=True)
    Hq, Hkv, D = 8, 2, 128
    lens = [1000, 3, 517, 1]
    T = sum(lens)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    q, k, v = rnd(T, Hq, D, seed=97, scale=0.5), rnd(T, Hkv, D, seed=98, scale=0.5), rnd(T, Hkv, D, seed=99, scale=0.5)
    ref = orc.varlen_prefill_reference(q, k, v, cu, cu, causal=True)
    got = ops.flash_attn_varlen_prefill(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), cu.cuda(), max(lens), max(lens),
                                        causal=True, kv_splits=splits)
    check(got, ref, what="split keys varlen")

    ctx = [700, 391, 64, 1500, 17, 300]
    chunk = [203, 391, 1, 1, 17, 299]
    _, kc, vc, bt, cl = orc.make_paged_case(batch=len(ctx), n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, block_size=16,
                                            context_lens=ctx, pool_factor=1.3, seed=23, dtype=torch.bfloat16)
    cu = torch.tensor([0] + list(torch.tensor(chunk).cumsum(0)), dtype=torch.int32)
    q = rnd(int(cu[-1]), Hq, D, seed=24)
    ref = orc.paged_prefill_reference(q, kc, vc, cu, bt, cl)
    dev = "cuda:0"
    got = ops.flash_attn_paged_prefill(q.to(dev), kc.to(dev), vc.to(dev), cu.to(dev), bt.to(dev), cl.to(dev), max(chunk),
                                       kv_splits=splits)
    check(got, ref, what="split keys paged")
    unsplit = ops.flash_attn_paged_prefill(q.to(dev), kc.to(dev), vc.to(dev), cu.to(dev), bt.to(dev), cl.to(dev),
                                           max(chunk), kv_splits=1)
    assert (got.float() - unsplit.float()).abs().max().item() <= 2e-2


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_prefill_head_dim_128_two_kernels_agree_on_random_shapes(ops, seed):
    """The 64-query kernel (hand-scheduled, pipelined tile loop) against the 8-wavefront kernel (reached through an
    explicit boolean mask that says the same thing) and the oracle, on drawn shapes: ragged query and key counts,
    Sk >= Sq (bottom-right diagonal), GQA, several query tiles per workgroup, and keys whose scores run away in
    both directions at drawn places -- in unmasked tiles, on the diagonal, in the last partial tile -- so that the
    loop is left and re-entered at every kind of tile."""
    g = torch.Generator().manual_seed(1000 + seed)
    for case in range(5):
        B = int(torch.randint(1, 3, (1,), generator=g))
        Hkv = int(torch.randint(1, 3, (1,), generator=g))
        Hq = Hkv * int(torch.randint(1, 3, (1,), generator=g))
        Sq = int(torch.randint(1, 900, (1,), generator=g))
        Sk = Sq + int(torch.randint(0, 700, (1,), generator=g)) * int(torch.randint(0, 2, (1,), generator=g))
        causal = bool(torch.randint(0, 2, (1,), generator=g))
        print(f"case: two kernels seed={seed} #{case} B={B} Hq={Hq} Hkv={Hkv} Sq={Sq} Sk={Sk} causal={causal}", flush=True)
        q = (torch.randn(B, Hq, Sq, 128, generator=g)).to(torch.bfloat16)
        k = torch.randn(B, Hkv, Sk, 128, generator=g)
        v = (torch.randn(B, Hkv, Sk, 128, generator=g)).to(torch.bfloat16)
        for _ in range(int(torch.randint(0, 6, (1,), generator=g))):          # runaway keys
            j = int(torch.randint(0, Sk, (1,), generator=g))
            n = int(torch.randint(1, 70, (1,), generator=g))
            k[:, :, j:j + n] *= float(torch.tensor([6.0, 20.0, -15.0, 45.0])[int(torch.randint(0, 4, (1,), generator=g))])
        k = k.to(torch.bfloat16)
        ref = orc.prefill_reference(q, k, v, causal=causal)
        fast = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=causal, kv_splits=1)
        keep = torch.ones(Sq, Sk, dtype=torch.bool)
        if causal:
            keep = torch.tril(keep, diagonal=Sk - Sq)
        slow = ops.scaled_dot_product_attention(q.cuda(), k.cuda().repeat_interleave(Hq // Hkv, 1),
                                                v.cuda().repeat_interleave(Hq // Hkv, 1), keep.cuda())
        n_shares = 2 + (seed + case) % 3              # shares that start at odd and even tiles, some of them empty
        shared = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=causal, kv_splits=n_shares)
        torch.cuda.synchronize()
        check(fast, ref, what=f"64-query kernel seed {seed} #{case}")
        check(slow, ref, what=f"8-wavefront kernel seed {seed} #{case}")
        check(shared, ref, what=f"64-query kernel, keys split {n_shares} ways, seed {seed} #{case}")


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_prefill_head_dim_128_four_heads_per_workgroup_on_random_shapes(ops, seed):
    """Causal prefill with a multiple of four query heads per K/V head: the 64-query kernel then gives the four wavefronts
    of a workgroup the same 64 rows of four heads (one head each) instead of 4 x 64 rows of one head.  Drawn shapes --
    4, 8 or 12 query heads per K/V head, ragged query and key counts, more keys than queries, runaway keys -- against
    the oracle and against the other kernel; with the keys split (partial rows per head), with the log-sum-exp output,
    and the gradients that the training forward feeds."""
    g = torch.Generator().manual_seed(7000 + seed)
    for case in range(4):
        B = int(torch.randint(1, 3, (1,), generator=g))
        Hkv = int(torch.randint(1, 3, (1,), generator=g))
        Hq = Hkv * 4 * int(torch.randint(1, 4, (1,), generator=g))
        Sq = int(torch.randint(1, 700, (1,), generator=g))
        Sk = Sq + int(torch.randint(0, 500, (1,), generator=g)) * int(torch.randint(0, 2, (1,), generator=g))
        print(f"case: four heads per workgroup seed={seed} #{case} B={B} Hq={Hq} Hkv={Hkv} Sq={Sq} Sk={Sk}", flush=True)
        q = torch.randn(B, Hq, Sq, 128, generator=g).to(torch.bfloat16)
        k = torch.randn(B, Hkv, Sk, 128, generator=g)
        v = torch.randn(B, Hkv, Sk, 128, generator=g).to(torch.bfloat16)
        for _ in range(int(torch.randint(0, 4, (1,), generator=g))):          # runaway keys
            j = int(torch.randint(0, Sk, (1,), generator=g))
            k[:, :, j:j + int(torch.randint(1, 70, (1,), generator=g))] *= float(torch.tensor([6.0, 20.0, -15.0, 45.0])[int(torch.randint(0, 4, (1,), generator=g))])
        k = k.to(torch.bfloat16)
        ref = orc.prefill_reference(q, k, v, causal=True)
        fast = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=True, kv_splits=1)
        keep = torch.tril(torch.ones(Sq, Sk, dtype=torch.bool), diagonal=Sk - Sq)
        slow = ops.scaled_dot_product_attention(q.cuda(), k.cuda().repeat_interleave(Hq // Hkv, 1),
                                                v.cuda().repeat_interleave(Hq // Hkv, 1), keep.cuda())
        shared = ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=True, kv_splits=2 + (seed + case) % 3)
        from mi355_attn import ops as raw
        out2, lse = raw._dense(q.cuda(), k.cuda(), v.cuda(), None, 1, None, want_lse=True)
        torch.cuda.synchronize()
        check(fast, ref, what=f"four heads per workgroup seed {seed} #{case}")
        check(slow, ref, what=f"8-wavefront kernel seed {seed} #{case}")
        check(shared, ref, what=f"four heads per workgroup, keys split, seed {seed} #{case}")
        assert torch.equal(out2, fast)
        s_ = torch.einsum("bhqd,bhkd->bhqk", q.float(), k.float().repeat_interleave(Hq // Hkv, 1)) / math.sqrt(128)
        torch.testing.assert_close(lse.cpu(), torch.logsumexp(s_.masked_fill(~keep, float("-inf")), -1), atol=3e-3, rtol=1e-3)


def test_prefill_head_dim_128_four_heads_per_workgroup_packed_and_trained(ops):
    """The same job layout on a packed batch of drawn lengths (an empty sequence and a one-token one included), and
    through autograd: the forward with the log-sum-exp runs on this layout, the backward kernels read what it wrote."""
    print("case: four heads per workgroup, packed + backward", flush=True)
    Hq, Hkv, D = 8, 2, 128
    lens = [300, 0, 1, 129, 517, 64]
    T = sum(lens)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    q, k, v, dout = rnd(T, Hq, D, seed=7100), rnd(T, Hkv, D, seed=7101), rnd(T, Hkv, D, seed=7102), rnd(T, Hq, D, seed=7103)
    ref = orc.varlen_prefill_reference(q, k, v, cu, cu, causal=True)
    qg, kg, vg = (t.cuda().requires_grad_() for t in (q, k, v))
    out = ops.flash_attn_varlen_prefill(qg, kg, vg, cu.cuda(), cu.cuda(), max(lens), max(lens), causal=True)
    out.backward(dout.cuda())
    torch.cuda.synchronize()
    check(out.detach(), ref, what="packed, four heads per workgroup")
    for b, n in enumerate(lens):
        if n == 0:
            continue
        a, e = int(cu[b]), int(cu[b + 1])
        args = [t[a:e].transpose(0, 1)[None] for t in (q, k, v, dout)]
        dq, dk, dv, _ = orc.prefill_backward_reference(*args, causal=True)
        for name, got, want in (("dq", qg.grad[a:e], dq), ("dk", kg.grad[a:e], dk), ("dv", vg.grad[a:e], dv)):
            want = want[0].transpose(0, 1)
            check(got, want, atol=1e-4 + 2e-2 * float(want.abs().max()), rtol=2e-2, what=f"{name} of sequence {b}")


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_prefill_head_dim_128_packed_sequences_of_drawn_lengths(ops, seed):
    """Packed sequences of drawn lengths (empty ones included) through the persistent 64-query kernel: a workgroup
    walks from job to job across sequences of different lengths, prefetching the next job's rows and tiles; with
    a promised maximum that is too small for one sequence; forward-only and with the log-sum-exp output."""
    g = torch.Generator().manual_seed(2000 + seed)
    Hq, Hkv, D = 4, 2, 128
    n_seq = int(torch.randint(2, 9, (1,), generator=g))
    lens = [int(x) for x in torch.randint(0, 700, (n_seq,), generator=g)]
    lens[int(torch.randint(0, n_seq, (1,), generator=g))] = 1
    if sum(lens) == 0:
        lens[0] = 5
    print(f"case: packed drawn lengths seed={seed} lens={lens}", flush=True)
    T = sum(lens)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    q, k, v = rnd(T, Hq, D, seed=3000 + seed), rnd(T, Hkv, D, seed=3100 + seed), rnd(T, Hkv, D, seed=3200 + seed)
    ref = orc.varlen_prefill_reference(q, k, v, cu, cu, causal=True)
    got = ops.flash_attn_varlen_prefill(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), cu.cuda(), max(lens), max(lens),
                                        causal=True, kv_splits=1)
    check(got, ref, what="packed drawn lengths")
    short = ops.flash_attn_varlen_prefill(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), cu.cuda(), max(1, max(lens) // 3),
                                          max(1, max(lens) // 3), causal=True, kv_splits=1)
    check(short, ref, what="packed drawn lengths, promised maximum too small")
    from mi355_attn import ops as raw
    out2, lse = raw._varlen(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), cu.cuda(), max(lens), max(lens), True, None, want_lse=True)
    assert torch.equal(out2, got)
    scores = []
    for b, n in enumerate(lens):
        if n == 0:
            continue
        a, e = int(cu[b]), int(cu[b + 1])
        s_ = torch.einsum("qhd,khd->hqk", q[a:e].float(), k[a:e].float().repeat_interleave(Hq // Hkv, 1)) / math.sqrt(D)
        s_ = s_.masked_fill(~torch.tril(torch.ones(n, n, dtype=torch.bool)), float("-inf"))
        scores.append(torch.logsumexp(s_, -1))
    torch.testing.assert_close(lse.cpu(), torch.cat(scores, 1), atol=3e-3, rtol=1e-3)


@pytest.mark.parametrize("seed", [0, 1])
def test_prefill_head_dim_128_more_jobs_than_compute_units_on_ragged_sequences(ops, seed):
    """More (sequence, head, query tile) jobs than compute units, so that the persistent kernel deals several rounds
    of its job list, forwards and backwards (the small shapes of the other tests fit in one round; here the list is
    made of single tiles by tile index): ragged packed sequences, 32 query heads on 8 kv heads, causal and not, one
    promised maximum that is too small."""
    g = torch.Generator().manual_seed(4000 + seed)
    Hq, Hkv, D = 32, 8, 128
    lens = [int(x) for x in torch.randint(520, 1000, (3,), generator=g)]        # 3 or 4 query tiles each: > 256 triples
    lens[seed % 3] = 1 + int(torch.randint(0, 255, (1,), generator=g))
    print(f"case: several rounds of jobs seed={seed} lens={lens}", flush=True)
    T = sum(lens)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    q, k, v = rnd(T, Hq, D, seed=4100 + seed), rnd(T, Hkv, D, seed=4200 + seed), rnd(T, Hkv, D, seed=4300 + seed)
    for causal in (True, False):
        ref = orc.varlen_prefill_reference(q, k, v, cu, cu, causal=causal)
        got = ops.flash_attn_varlen_prefill(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), cu.cuda(), max(lens), max(lens),
                                            causal=causal, kv_splits=1)
        check(got, ref, what=f"several rounds of jobs, causal={causal}")
    ref = orc.varlen_prefill_reference(q, k, v, cu, cu, causal=True)
    short = ops.flash_attn_varlen_prefill(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), cu.cuda(), 600, 600, causal=True, kv_splits=1)
    check(short, ref, what="several rounds of jobs, promised maximum too small")
    shared = ops.flash_attn_varlen_prefill(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), cu.cuda(), max(lens), max(lens),
                                           causal=True, kv_splits=3)
    check(shared, ref, what="several rounds of jobs, keys split 3 ways")


@pytest.mark.parametrize("n_seq", [70, 150])
def test_prefill_head_dim_128_many_packed_sequences_of_very_different_lengths(ops, n_seq):
    """The persistent kernel orders its jobs by query tile index and finds the sequences that reach an index by
    counting over all sequences, 64 at a time: more than 64 sequences, most of them short or empty and a few long
    ones at drawn places, so that every class of the job list has its own set of sequences; causal and not, keys
    whole and split.  With 150 sequences the list is made of tile pairs (eight rounds and more on 256 compute units),
    with 70 of single tiles by tile index (four rounds, the last far from full)."""
    g = torch.Generator().manual_seed(5000 + n_seq)
    Hq, Hkv, D = 4, 2, 128
    lens = [int(x) for x in torch.randint(0, 40, (n_seq,), generator=g)]
    for _ in range(6):
        lens[int(torch.randint(0, n_seq, (1,), generator=g))] = int(torch.randint(200, 1300, (1,), generator=g))
    lens[n_seq - 1] = 700                     # the last sequence reaches the third level
    print(f"case: many packed sequences n_seq={n_seq} longest={max(lens)} total={sum(lens)}", flush=True)
    T = sum(lens)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    q, k, v = rnd(T, Hq, D, seed=5100 + n_seq), rnd(T, Hkv, D, seed=5200 + n_seq), rnd(T, Hkv, D, seed=5300 + n_seq)
    for causal in (True, False):
        ref = orc.varlen_prefill_reference(q, k, v, cu, cu, causal=causal)
        for splits in (1, 2):
            got = ops.flash_attn_varlen_prefill(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), cu.cuda(), max(lens), max(lens),
                                                causal=causal, kv_splits=splits)
            check(got, ref, what=f"{n_seq} packed sequences, causal={causal}, keys split {splits} ways")


def test_prefill_head_dim_128_more_packed_sequences_than_the_64_query_kernel_keeps_counts_for(ops):
    """The 64-query kernel keeps one number per sequence in LDS, 4096 at most; a packed batch of more sequences goes
    to the other kernel.  4100 sequences of one to three tokens."""
    n_seq, Hq, Hkv, D = 4100, 2, 1, 128
    g = torch.Generator().manual_seed(5500)
    lens = [int(x) for x in torch.randint(1, 4, (n_seq,), generator=g)]
    print(f"case: {n_seq} packed sequences total={sum(lens)}", flush=True)
    T = sum(lens)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    q, k, v = rnd(T, Hq, D, seed=5501), rnd(T, Hkv, D, seed=5502), rnd(T, Hkv, D, seed=5503)
    ref = orc.varlen_prefill_reference(q, k, v, cu, cu, causal=True)
    got = ops.flash_attn_varlen_prefill(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), cu.cuda(), 3, 3, causal=True, kv_splits=1)
    check(got, ref, what="4100 packed sequences")
    # the same tokens as 4096 sequences (the last one takes what is left): the 64-query kernel at its limit
    cu2 = torch.cat([cu[:4096], cu[-1:]])
    ref2 = orc.varlen_prefill_reference(q, k, v, cu2, cu2, causal=True)
    longest = int((cu2[1:] - cu2[:-1]).max())
    got2 = ops.flash_attn_varlen_prefill(q.cuda(), k.cuda(), v.cuda(), cu2.cuda(), cu2.cuda(), longest, longest, causal=True, kv_splits=1)
    check(got2, ref2, what="4096 packed sequences")


def test_prefill_head_dim_128_rows_too_far_apart_for_the_64_query_kernel(ops):
    """The 64-query kernel multiplies row strides as 32-bit byte offsets inside a tile; a query tensor whose rows lie
    2^23 elements apart (a view into a 1 GiB buffer) must be sent to the other kernel, not read from wrapped
    addresses.  Same inputs, contiguous, give the comparison."""
    Sq, D = 64, 128
    print("case: head_dim 128, query row stride 2^23 elements", flush=True)
    q, k, v = rnd(1, 1, Sq, D, seed=71), rnd(1, 1, 300, D, seed=72), rnd(1, 1, 300, D, seed=73)
    big = torch.zeros(Sq * (1 << 23), dtype=torch.bfloat16, device="cuda")
    q_far = big.as_strided((1, 1, Sq, D), (0, 0, 1 << 23, 1))
    q_far.copy_(q.cuda())
    ref = orc.prefill_reference(q, k, v, causal=True)
    got = ops.flash_attn_prefill(q_far, k.cuda(), v.cuda(), causal=True, kv_splits=1)
    check(got, ref, what="rows 2^23 elements apart")
    del big, q_far
    torch.cuda.empty_cache()


def _reference_module_tensors(x_proj, freq, num_heads, amp):
    """Q, K, V exactly as CausalMultiHeadSelfAttention.forward hands them to the attention call
    (llm-core/llm_core/model.py:362-378) from the three projection outputs (B, S, H*d): `rearrange` views, then
    RotaryEmbedding.forward (model.py:93-104) on Q and K with the float32 (2, ctx, d/2) table.  Under `--amp` the
    projections are bf16, so Q and K come out float32 and contiguous and V stays a strided bf16 view."""
    from einops import rearrange
    qp, kp, vp = x_proj
    Q, K, V = (rearrange(t, "... seq (heads d) -> ... heads seq d", heads=num_heads) for t in (qp, kp, vp))
    S = qp.shape[1]
    pos = torch.arange(S, device=qp.device).view(1, S)
    pos = rearrange(pos, "... seq -> ... 1 seq")

    def rope(x):
        x1, x2 = x[..., 0::2], x[..., 1::2]
        cos, sin = freq[:, pos, :]
        return rearrange([cos * x1 - sin * x2, sin * x1 + cos * x2], "xy ... half_d -> ... (half_d xy)", xy=2).contiguous()

    Q, K = rope(Q), rope(K)
    if amp:
        assert Q.dtype == torch.float32 and K.dtype == torch.float32 and V.dtype == torch.bfloat16
    assert Q.is_contiguous() and not V.is_contiguous()
    return Q, K, V


@pytest.mark.parametrize("D,Hq,Hkv", [(128, 8, 2), (64, 4, 4), (32, 4, 1)])
def test_paged_prefill_ragged_chunks_match_the_oracle(ops, D, Hq, Hkv):
    """Chunks of new tokens over cached context, read through the block table: ragged chunk lengths and
    contexts (a chunk that IS the whole context, one token over a long context, chunk ends inside a block,
    several query tiles), garbage in unused blocks, in the tail of the last block and in the table tail."""
    ctx = [700, 391, 64, 1500, 17, 300]
    chunk = [203, 391, 1, 1, 17, 299]
    print(f"case: paged prefill D={D} Hq={Hq} Hkv={Hkv}", flush=True)
    _, kc, vc, bt, cl = orc.make_paged_case(batch=len(ctx), n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, block_size=16,
                                            context_lens=ctx, pool_factor=1.3, seed=21, dtype=torch.bfloat16)
    cu = torch.tensor([0] + list(torch.tensor(chunk).cumsum(0)), dtype=torch.int32)
    q = rnd(int(cu[-1]), Hq, D, seed=22)
    ref = orc.paged_prefill_reference(q, kc, vc, cu, bt, cl)
    used = torch.zeros(kc.shape[0], dtype=torch.bool)
    bt2 = bt.clone()
    kc2, vc2 = kc.clone(), vc.clone()
    for b, c in enumerate(ctx):
        nb = (c + 15) // 16
        used[bt[b, :nb].long()] = True
        bt2[b, nb:] = 2 ** 30
        if c % 16:
            last = int(bt[b, (c - 1) // 16])
            kc2[last, :, c % 16:] = float("nan")
            vc2[last, :, c % 16:] = float("inf")
    kc2[~used] = float("nan")
    vc2[~used] = float("nan")
    dev = "cuda:0"
    got = ops.flash_attn_paged_prefill(q.to(dev), kc2.to(dev), vc2.to(dev), cu.to(dev), bt2.to(dev), cl.to(dev), max(chunk))
    torch.cuda.synchronize()
    check(got, ref, what="paged prefill")
    # a strided q (a slice of a fused projection) and a caller-provided output
    wide = torch.zeros(q.shape[0], Hq + 2, D, dtype=torch.bfloat16, device=dev)
    wide[:, :Hq] = q.to(dev)
    out = torch.empty_like(got)
    ret = ops.flash_attn_paged_prefill(wide[:, :Hq], kc2.to(dev), vc2.to(dev), cu.to(dev), bt2.to(dev), cl.to(dev),
                                       max(chunk), out=out)
    assert ret is out and torch.equal(out, got)


@pytest.mark.parametrize("Hq,Hkv,splits", [(8, 2, 1), (4, 4, 1), (6, 2, 1), (8, 2, 3)])
def test_paged_prefill_head_dim_128_long_contexts_through_the_block_table(ops, Hq, Hkv, splits):
    """head_dim 128 runs on the 64-query kernel, whose tile loop takes its block ids from a register that covers 63
    tiles at a time: contexts of more than 63, 126 and 189 tiles (so the loop is left and entered again with the next
    ids), chunk ends inside a block and inside a tile, one token over a long context, a chunk that is the whole
    context; four query heads per K/V head (the four wavefronts share the rows), one (they share the head) and three;
    keys split over workgroups; garbage in unused blocks, in the tail of the last block and in the table tail."""
    ctx = [9000, 2100, 12300, 64, 4033, 8129]
    chunk = [300, 2100, 1, 64, 257, 520]
    print(f"case: paged prefill D=128 long contexts Hq={Hq} Hkv={Hkv} splits={splits}", flush=True)
    D = 128
    _, kc, vc, bt, cl = orc.make_paged_case(batch=len(ctx), n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, block_size=16,
                                            context_lens=ctx, pool_factor=1.2, seed=31, dtype=torch.bfloat16)
    cu = torch.tensor([0] + list(torch.tensor(chunk).cumsum(0)), dtype=torch.int32)
    q = rnd(int(cu[-1]), Hq, D, seed=32)
    ref = orc.paged_prefill_reference(q, kc, vc, cu, bt, cl)
    used = torch.zeros(kc.shape[0], dtype=torch.bool)
    bt2, kc2, vc2 = bt.clone(), kc.clone(), vc.clone()
    for b, c in enumerate(ctx):
        nb = (c + 15) // 16
        used[bt[b, :nb].long()] = True
        bt2[b, nb:] = 2 ** 30
        if c % 16:
            last = int(bt[b, (c - 1) // 16])
            kc2[last, :, c % 16:] = float("nan")
            vc2[last, :, c % 16:] = float("inf")
    kc2[~used] = float("nan")
    vc2[~used] = float("nan")
    dev = "cuda:0"
    got = ops.flash_attn_paged_prefill(q.to(dev), kc2.to(dev), vc2.to(dev), cu.to(dev), bt2.to(dev), cl.to(dev), max(chunk),
                                       kv_splits=splits)
    torch.cuda.synchronize()
    check(got, ref, what="paged prefill, long contexts")


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_paged_prefill_head_dim_128_random_shapes_with_runaway_keys(ops, seed):
    """The block-table form of the 64-query kernel on drawn shapes: ragged contexts and chunks, one, two or four query
    heads per K/V head, and keys whose scores run away in both directions at drawn places, so that the tile loop is
    left (a row sum reached 2), entered again, and query tiles are computed a second time -- all of which fetch
    their block ids on the way.  Garbage past every context's end."""
    g = torch.Generator().manual_seed(2000 + seed)
    dev = "cuda:0"
    for case in range(4):
        B = int(torch.randint(1, 4, (1,), generator=g))
        Hkv = int(torch.randint(1, 3, (1,), generator=g))
        Hq = Hkv * int(torch.tensor([1, 2, 4])[int(torch.randint(0, 3, (1,), generator=g))])
        ctx = [int(torch.randint(1, 6000, (1,), generator=g)) for _ in range(B)]
        chunk = [int(torch.randint(1, min(c, 700) + 1, (1,), generator=g)) for c in ctx]
        print(f"case: paged runaway seed={seed} #{case} Hq={Hq} Hkv={Hkv} ctx={ctx} chunk={chunk}", flush=True)
        nblk = [(c + 15) // 16 for c in ctx]
        pool = sum(nblk) + 5
        perm = torch.randperm(pool, generator=g)
        kc = torch.full((pool, Hkv, 16, 128), float("nan"), dtype=torch.bfloat16)
        vc = torch.full((pool, Hkv, 16, 128), float("nan"), dtype=torch.bfloat16)
        bt = torch.full((B, max(nblk)), 2 ** 30, dtype=torch.int32)
        cu = torch.tensor([0] + list(torch.tensor(chunk).cumsum(0)), dtype=torch.int32)
        q = torch.randn(int(cu[-1]), Hq, 128, generator=g).to(torch.bfloat16)
        ref = torch.empty(int(cu[-1]), Hq, 128)
        off = 0
        for b in range(B):
            k = torch.randn(Hkv, ctx[b], 128, generator=g)
            v = torch.randn(Hkv, ctx[b], 128, generator=g).to(torch.bfloat16)
            for _ in range(int(torch.randint(0, 5, (1,), generator=g))):          # runaway keys
                j = int(torch.randint(0, ctx[b], (1,), generator=g))
                n = int(torch.randint(1, 70, (1,), generator=g))
                k[:, j:j + n] *= float(torch.tensor([6.0, 20.0, -15.0, 45.0])[int(torch.randint(0, 4, (1,), generator=g))])
            k = k.to(torch.bfloat16)
            ids = perm[off:off + nblk[b]]
            off += nblk[b]
            bt[b, :nblk[b]] = ids.to(torch.int32)
            pad = nblk[b] * 16 - ctx[b]
            kp = torch.cat([k, torch.full((Hkv, pad, 128), float("nan"), dtype=torch.bfloat16)], 1)
            vp = torch.cat([v, torch.full((Hkv, pad, 128), float("inf"), dtype=torch.bfloat16)], 1)
            kc[ids] = kp.view(Hkv, nblk[b], 16, 128).transpose(0, 1)
            vc[ids] = vp.view(Hkv, nblk[b], 16, 128).transpose(0, 1)
            qb = q[int(cu[b]):int(cu[b + 1])].transpose(0, 1)[None]
            ref[int(cu[b]):int(cu[b + 1])] = orc.prefill_reference(qb, k[None], v[None], causal=True)[0].transpose(0, 1)
        cl = torch.tensor(ctx, dtype=torch.int32)
        got = ops.flash_attn_paged_prefill(q.to(dev), kc.to(dev), vc.to(dev), cu.to(dev), bt.to(dev), cl.to(dev), max(chunk),
                                           kv_splits=1)
        n_shares = 2 + (seed + case) % 3
        shared = ops.flash_attn_paged_prefill(q.to(dev), kc.to(dev), vc.to(dev), cu.to(dev), bt.to(dev), cl.to(dev),
                                              max(chunk), kv_splits=n_shares)
        torch.cuda.synchronize()
        check(got, ref, what=f"paged 64-query kernel seed {seed} #{case}")
        check(shared, ref, what=f"paged 64-query kernel, keys split {n_shares} ways, seed {seed} #{case}")


@pytest.mark.parametrize("B", [4096, 4097])
def test_paged_prefill_head_dim_128_thousands_of_short_sequences(ops, B):
    """As many sequences as the 64-query kernel keeps counts for in LDS (4096: 64 groups of 64), and one more (the
    8-wavefront kernel then serves the launch): chunks of one to three tokens over contexts of a few blocks."""
    print(f"case: paged prefill D=128, {B} sequences", flush=True)
    g = torch.Generator().manual_seed(40)
    ctx = [int(x) for x in torch.randint(1, 40, (B,), generator=g)]
    chunk = [min(c, int(x)) for c, x in zip(ctx, torch.randint(1, 4, (B,), generator=g))]
    _, kc, vc, bt, cl = orc.make_paged_case(batch=B, n_q_heads=4, n_kv_heads=1, head_dim=128, block_size=16,
                                            context_lens=ctx, pool_factor=1.1, seed=41, dtype=torch.bfloat16)
    cu = torch.tensor([0] + list(torch.tensor(chunk).cumsum(0)), dtype=torch.int32)
    q = rnd(int(cu[-1]), 4, 128, seed=42)
    ref = orc.paged_prefill_reference(q, kc, vc, cu, bt, cl)
    dev = "cuda:0"
    got = ops.flash_attn_paged_prefill(q.to(dev), kc.to(dev), vc.to(dev), cu.to(dev), bt.to(dev), cl.to(dev), max(chunk),
                                       kv_splits=1)
    torch.cuda.synchronize()
    check(got, ref, what=f"paged prefill, {B} sequences")


@pytest.mark.parametrize("D,Hq,Hkv", [(128, 8, 2), (64, 4, 4), (128, 32, 8)])
def test_paged_prefill_over_an_fp8_cache_matches_the_oracle(ops, D, Hq, Hkv):
    """The same ragged chunks over an fp8-e4m3 cache with per-(block, kv head) scales: gathered and dequantised by
    mi355_gather_kv_fp8, attended to by the packed prefill kernels.  Kernel parity: within the bf16 tolerance of the
    oracle on the DEQUANTISED cache.  Quantisation noise: against the oracle on the bf16 cache the result stays within
    |err| <= 0.15 + 2^-4 |ref| with a relative rms error under 6 % (the bound of the fp8 decode)."""
    ctx = [700, 391, 64, 1500, 17, 300]
    chunk = [203, 391, 1, 1, 17, 299]
    print(f"case: paged prefill over fp8 D={D} Hq={Hq} Hkv={Hkv}", flush=True)
    _, kc, vc, bt, cl = orc.make_paged_case(batch=len(ctx), n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, block_size=16,
                                            context_lens=ctx, pool_factor=1.3, seed=31, dtype=torch.bfloat16)
    # the tail of a sequence's last block holds zeros (what a cache writer leaves there), so that a block's scale
    # comes from its valid rows
    for b, c in enumerate(ctx):
        if c % 16:
            last = int(bt[b, (c - 1) // 16])
            kc[last, :, c % 16:] = 0
            vc[last, :, c % 16:] = 0
    k8, ks = orc.quantize_kv_fp8(kc)
    v8, vs = orc.quantize_kv_fp8(vc)
    cu = torch.tensor([0] + list(torch.tensor(chunk).cumsum(0)), dtype=torch.int32)
    q = rnd(int(cu[-1]), Hq, D, seed=32)
    ref8 = orc.paged_prefill_reference(q, orc.dequantize_kv_fp8(k8, ks), orc.dequantize_kv_fp8(v8, vs), cu, bt, cl)
    ref16 = orc.paged_prefill_reference(q, kc, vc, cu, bt, cl)
    dev = "cuda:0"
    bt2 = bt.clone()
    for b, c in enumerate(ctx):
        bt2[b, (c + 15) // 16:] = 2 ** 30                      # the table tail is never read
    args = (q.to(dev), k8.to(dev), v8.to(dev), cu.to(dev), bt2.to(dev), cl.to(dev), max(chunk))
    got = ops.flash_attn_paged_prefill(*args, k_scale=ks.to(dev), v_scale=vs.to(dev))
    tight = ops.flash_attn_paged_prefill(*args, k_scale=ks.to(dev), v_scale=vs.to(dev), total_context=sum(ctx), kv_splits=1)
    torch.cuda.synchronize()
    check(got, ref8, what="paged prefill over fp8, oracle on the dequantised cache")
    check(tight, ref8, what="paged prefill over fp8, rows sized by total_context")
    # the caller's own running sum of the context lengths instead of one computed per call
    cu_ctx = torch.tensor([0] + list(torch.tensor(ctx).cumsum(0)), dtype=torch.int32, device=dev)
    given = ops.flash_attn_paged_prefill(*args, k_scale=ks.to(dev), v_scale=vs.to(dev), total_context=sum(ctx), kv_splits=1,
                                         cu_seqlens_k=cu_ctx)
    assert torch.equal(given, tight)
    e16 = (got.float().cpu() - ref16).abs()
    assert bool((e16 <= 0.15 + 2.0 ** -4 * ref16.abs()).all()), float(e16.max())
    assert float((got.float().cpu() - ref16).pow(2).mean().sqrt() / ref16.pow(2).mean().sqrt()) <= 0.06
    # the gathered rows themselves: bf16(fp8 * scale), row by row
    kl, vl, cu_k = ops.gather_kv_fp8(k8.to(dev), v8.to(dev), ks.to(dev), vs.to(dev), bt2.to(dev), cl.to(dev))
    assert cu_k.tolist() == [0] + list(torch.tensor(ctx).cumsum(0))
    for b in (0, 3, 4):
        want = orc.gather_paged_kv(orc.dequantize_kv_fp8(k8, ks), bt[b], ctx[b]).transpose(0, 1).to(torch.bfloat16)
        assert torch.equal(kl[int(cu_k[b]):int(cu_k[b + 1])].cpu(), want)


@pytest.mark.parametrize("fp8", [False, True])
def test_paged_prefill_cuts_a_context_length_beyond_the_table(ops, fp8):
    """A context_lens entry larger than what a row of the block table addresses (a corrupted length) must not walk
    past the row: the sequence is served as if its length were 16 * (table width), finite and equal to that call."""
    print(f"case: paged prefill, context length beyond the table, fp8={fp8}", flush=True)
    Hq, Hkv, D = 4, 2, 64
    ctx, chunk = [160, 96], [40, 96]
    _, kc, vc, bt, cl = orc.make_paged_case(batch=2, n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, block_size=16,
                                            context_lens=ctx, seed=9, dtype=torch.bfloat16)
    assert bt.shape[1] == 10
    cu = torch.tensor([0, 40, 136], dtype=torch.int32)
    q = rnd(136, Hq, D, seed=10)
    dev = "cuda:0"
    kw = {}
    kcd, vcd = kc.to(dev), vc.to(dev)
    if fp8:
        k8, ks = orc.quantize_kv_fp8(kc)
        v8, vs = orc.quantize_kv_fp8(vc)
        kcd, vcd, kw = k8.to(dev), v8.to(dev), {"k_scale": ks.to(dev), "v_scale": vs.to(dev)}
    good = ops.flash_attn_paged_prefill(q.to(dev), kcd, vcd, cu.to(dev), bt.to(dev), cl.to(dev), 96, **kw)
    wild = torch.tensor([160 + 5000, 96], dtype=torch.int32)
    # (the last sequence's row is the end of the table's memory: a walk past it would leave the allocation)
    wild2 = torch.tensor([160, 96 + 70000], dtype=torch.int32)
    got = ops.flash_attn_paged_prefill(q.to(dev), kcd, vcd, cu.to(dev), bt.to(dev), wild.to(dev), 96, **kw)
    got2 = ops.flash_attn_paged_prefill(q.to(dev), kcd, vcd, cu.to(dev), bt.to(dev), wild2.to(dev), 96, **kw)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(got.float()).all()) and bool(torch.isfinite(got2.float()).all())
    # sequence 0 with the wild length sees all 160 keys of its row as context: its 40 queries sit at the END of them
    assert torch.equal(got[:40], good[:40]) and torch.equal(got[40:], good[40:])
    # sequence 1 is cut to 160 keys = its 96 + 64 from blocks the row lists beyond its length (zeros in the table -> block 0)
    assert torch.equal(got2[:40], good[:40])


def test_paged_prefill_equals_dense_prefill_on_the_gathered_rows(ops):
    """The paged walk changes where keys come from, not the arithmetic: same bits as the packed kernel fed with
    the gathered rows (head_dim 64: both calls run the same kernel)."""
    print("case: paged prefill vs packed", flush=True)
    Hq, Hkv, D = 4, 2, 64
    ctx, chunk = [333, 130], [100, 130]
    _, kc, vc, bt, cl = orc.make_paged_case(batch=2, n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, block_size=16,
                                            context_lens=ctx, seed=5, dtype=torch.bfloat16)
    cu_q = torch.tensor([0, 100, 230], dtype=torch.int32)
    cu_k = torch.tensor([0, 333, 463], dtype=torch.int32)
    q = rnd(230, Hq, D, seed=6)
    kk = torch.cat([orc.gather_paged_kv(kc, bt[b], ctx[b]).transpose(0, 1) for b in range(2)]).to(torch.bfloat16)
    vv = torch.cat([orc.gather_paged_kv(vc, bt[b], ctx[b]).transpose(0, 1) for b in range(2)]).to(torch.bfloat16)
    dev = "cuda:0"
    a = ops.flash_attn_paged_prefill(q.to(dev), kc.to(dev), vc.to(dev), cu_q.to(dev), bt.to(dev), cl.to(dev), 130)
    b = ops.flash_attn_varlen_prefill(q.to(dev), kk.to(dev), vv.to(dev), cu_q.to(dev), cu_k.to(dev), 130, 333, causal=True)
    assert torch.equal(a, b)


@pytest.mark.parametrize("amp", [True, False])
def test_sdpa_slot_takes_the_reference_modules_tensors(ops, amp):
    """The swap at model.py:382 with the tensors the reference really passes there: float32 Q/K + strided bf16 V
    under autocast (train.py:215), three float32 tensors without it; the reference's sample shape (d_head 32,
    16 heads, configures/sample.yaml).  Checked through the head merge of model.py:388 against the oracle's
    attention block run on the same projection outputs.  float32 inputs are rounded to bf16 by the slot (bf16
    math, as autocast SDPA does), hence the bf16 tolerance for the float32 case too."""
    from einops import rearrange
    from oracle import model_oracle as morc
    print(f"case: sdpa_slot reference dtype flow amp={amp}", flush=True)
    B, S, H, d = 3, 256, 16, 32
    g = torch.Generator().manual_seed(31)
    proj = [torch.randn(B, S, H * d, generator=g) * 0.7 for _ in range(3)]
    if amp:
        proj = [t.to(torch.bfloat16) for t in proj]                   # what a Linear gives under autocast
    freq = orc.build_rope_cache(S, d)
    ref = morc.attention_core_reference(*(t.float() for t in proj), H, freq)

    Q, K, V = _reference_module_tensors([t.cuda() for t in proj], freq.cuda(), H, amp)
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=amp):
        out = ops.sdpa_slot(Q, K, V, is_causal=True)
    assert out.shape == (B, H, S, d)
    assert out.dtype == (torch.bfloat16 if amp else torch.float32)    # what F.scaled_dot_product_attention returns there
    merged = rearrange(out, "... heads seq d_head -> ... seq (heads d_head)").contiguous()
    torch.cuda.synchronize()
    check(merged, ref, what=f"model.py:382 slot, amp={amp}")


def test_sdpa_slot_trains_through_the_reference_dtype_flow(ops):
    """Gradients reach the float32 Q/K and the bf16 V of the autocast flow (the casts in front of the kernel are
    differentiable) and match the oracle's hand-derived backward."""
    print("case: sdpa_slot backward through mixed dtypes", flush=True)
    B, H, S, d = 2, 4, 96, 32
    q32, k32 = rnd(B, H, S, d, seed=41, scale=0.5).float(), rnd(B, H, S, d, seed=42, scale=0.5).float()
    v16, dout = rnd(B, H, S, d, seed=43, scale=0.5), rnd(B, H, S, d, seed=44, scale=0.5)
    Q, K, V = q32.cuda().requires_grad_(), k32.cuda().requires_grad_(), v16.cuda().requires_grad_()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = ops.sdpa_slot(Q, K, V, is_causal=True)
    assert out.dtype == torch.bfloat16 and out.requires_grad
    out.backward(dout.cuda())
    torch.cuda.synchronize()
    assert Q.grad.dtype == torch.float32 and V.grad.dtype == torch.bfloat16
    dq, dk, dv, _ = orc.prefill_backward_reference(q32.bfloat16(), k32.bfloat16(), v16, dout, causal=True)
    for name, got, ref in (("dq", Q.grad, dq), ("dk", K.grad, dk), ("dv", V.grad, dv)):
        check(got, ref, atol=2e-2 * float(ref.abs().max()), rtol=2e-2, what=name)


def test_sdpa_reference_signature_autograd(ops):
    """scaled_dot_product_attention (the model.py:384-385 branch, used in training without --flash-attn): with
    with or without a mask the result carries a grad_fn and the gradients match the oracle (the masked cases have their
    own tests in test_gpu_backward.py)."""
    print("case: sdpa signature autograd", flush=True)
    B, H, S, D = 1, 2, 80, 64
    q, k, v, dout = (rnd(B, H, S, D, seed=s, scale=0.5) for s in (51, 52, 53, 54))
    Q, K, V = (t.cuda().requires_grad_() for t in (q, k, v))
    out = ops.scaled_dot_product_attention(Q, K, V)
    assert out.requires_grad and out.grad_fn is not None
    out.backward(dout.cuda())
    torch.cuda.synchronize()
    dq, dk, dv, _ = orc.prefill_backward_reference(q, k, v, dout, causal=False)
    for name, got, ref in (("dq", Q.grad, dq), ("dk", K.grad, dk), ("dv", V.grad, dv)):
        check(got, ref, atol=2e-2 * float(ref.abs().max()), rtol=2e-2, what=name)
    tril = torch.tril(torch.ones(S, S, dtype=torch.bool, device="cuda"))
    for t in (Q, K, V):
        t.grad = None
    out = ops.scaled_dot_product_attention(Q, K, V, tril)
    assert out.requires_grad and out.grad_fn is not None
    out.backward(dout.cuda())
    torch.cuda.synchronize()
    dq, dk, dv, _ = orc.prefill_backward_reference(q, k, v, dout, causal=True)
    for name, got, ref in (("dq", Q.grad, dq), ("dk", K.grad, dk), ("dv", V.grad, dv)):
        check(got, ref, atol=2e-2 * float(ref.abs().max()), rtol=2e-2, what=name)
    with torch.no_grad():                                              # forward-only use is unaffected
        assert not ops.scaled_dot_product_attention(Q, K, V, tril).requires_grad


def test_prefill_varlen_sequence_longer_than_promised(ops):
    """max_seqlen_q smaller than the longest sequence: every row is still computed (the workgroups of a sequence
    walk on through its remaining query tiles), none is left unwritten."""
    print("case: prefill varlen with too small a max_seqlen", flush=True)
    lens = [40, 1500, 700]
    Hq, Hkv, D = 4, 2, 64
    T = sum(lens)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    q, k, v = rnd(T, Hq, D, seed=61, scale=0.5), rnd(T, Hkv, D, seed=62, scale=0.5), rnd(T, Hkv, D, seed=63, scale=0.5)
    ref = orc.varlen_prefill_reference(q, k, v, cu, cu, causal=True)
    got = ops.flash_attn_varlen_prefill(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), cu.cuda(), 300, 300, causal=True)
    check(got, ref, what="varlen, promise too small")
    with pytest.raises(ValueError, match="max_seqlen"):
        ops.flash_attn_varlen_prefill(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), cu.cuda(), 0, 0, causal=True)


def test_decode_more_than_16_query_heads_per_kv_head(ops):
    """Hq/Hkv = 32, 20 and 48 (multi-query style): the kv head is streamed once per 16 query heads, by workgroups
    that sit eight ids apart -- with whole blocks of eight (sequence, chunk) items, with fewer than eight items, and
    with eleven."""
    for Hq, Hkv, D, ctx in ((32, 1, 128, [1, 17, 300, 5000]), (40, 2, 64, [1, 17, 300, 5000]), (32, 1, 128, [5, 700, 1000]),
                            (48, 1, 64, [900, 3, 1024, 77, 512, 1, 640, 999, 16, 17, 1000])):
        print(f"case: decode Hq/Hkv > 16: {Hq}/{Hkv} ctx={ctx}", flush=True)
        q, kc, vc, bt, cl = orc.make_paged_case(batch=len(ctx), n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, block_size=16,
                                                context_lens=ctx, pool_factor=1.2, seed=Hq, dtype=torch.bfloat16)
        check(run_decode(ops, q, kc, vc, bt, cl), orc.paged_decode_reference(q, kc, vc, bt, cl), what=f"{Hq}/{Hkv}")


def test_sdpa_with_reference_signature(ops):
    """scaled_dot_product_attention(Q, K, V, mask): None, the reference's tril mask, and an arbitrary keep-mask."""
    print("case: sdpa signature", flush=True)
    B, H, S, D = 2, 4, 150, 64
    q, k, v = rnd(B, H, S, D, seed=16, scale=0.5), rnd(B, H, S, D, seed=17, scale=0.5), rnd(B, H, S, D, seed=18, scale=0.5)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    check(ops.scaled_dot_product_attention(qg, kg, vg), orc.scaled_dot_product_attention(q.float(), k.float(), v.float()),
          what="no mask")
    tril = torch.tril(torch.ones(S, S, dtype=torch.bool))                      # as built at model.py:384
    check(ops.scaled_dot_product_attention(qg, kg, vg, tril.cuda()),
          orc.scaled_dot_product_attention(q.float(), k.float(), v.float(), tril), what="tril mask")
    g = torch.Generator().manual_seed(5)
    keep = torch.rand(B, 1, S, S, generator=g) > 0.5
    keep[..., 0] = True
    check(ops.scaled_dot_product_attention(qg, kg, vg, keep.cuda()),
          orc.scaled_dot_product_attention(q.float(), k.float(), v.float(), keep), what="random mask")
    # 3-D inputs (no head axis), rectangular
    q3, k3, v3 = rnd(3, 40, 32, seed=19), rnd(3, 77, 32, seed=20), rnd(3, 77, 32, seed=21)
    check(ops.scaled_dot_product_attention(q3.cuda(), k3.cuda(), v3.cuda()),
          orc.scaled_dot_product_attention(q3.float(), k3.float(), v3.float()), what="3-D")


def test_sdpa_fully_masked_row_is_nan_like_reference(ops):
    q, k, v = rnd(1, 1, 8, 32, seed=22), rnd(1, 1, 8, 32, seed=23), rnd(1, 1, 8, 32, seed=24)
    keep = torch.ones(8, 8, dtype=torch.bool)
    keep[3] = False
    got = ops.scaled_dot_product_attention(q.cuda(), k.cuda(), v.cuda(), keep.cuda()).float().cpu()
    ref = orc.scaled_dot_product_attention(q.float(), k.float(), v.float(), keep)
    assert torch.isnan(ref[0, 0, 3]).all() and torch.isnan(got[0, 0, 3]).all()
    rows = [0, 1, 2, 4, 5, 6, 7]
    check(got[0, 0, rows], ref[0, 0, rows], what="other rows")


def test_errors_are_python_exceptions(ops):
    q = torch.zeros(1, 2, 8, 64, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(TypeError):
        ops.flash_attn_prefill(q.half(), q.half(), q.half())          # bfloat16 and float32 only
    with pytest.raises(TypeError):
        ops.sdpa_slot(q.double(), q.double(), q.double())
    with pytest.raises(ValueError):
        ops.flash_attn_prefill(q, q[:, :, :, :32], q)
    with pytest.raises(ValueError):
        ops.flash_attn_prefill(q.cpu(), q.cpu(), q.cpu())
    q96 = torch.zeros(1, 2, 8, 96, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="head_dim"):
        ops.flash_attn_prefill(q96, q96, q96)


def test_decode_clamps_block_ids_outside_the_pool(ops):
    """A corrupted block table must not make the kernel read outside the caches: entries outside
    [0, num_blocks) are clamped (the affected sequence's result is meaningless, the others' are exact)."""
    print("case: decode bad block ids", flush=True)
    ctx = [40, 300, 77]
    q, kc, vc, bt, cl = orc.make_paged_case(batch=3, n_q_heads=8, n_kv_heads=2, head_dim=128, block_size=16,
                                            context_lens=ctx, pool_factor=1.0, seed=5, dtype=torch.bfloat16)
    good = ops.paged_attention_decode(q.cuda(), kc.cuda(), vc.cuda(), bt.cuda(), cl.cuda())
    bad = bt.clone()
    bad[1, 3] = 2 ** 30
    bad[1, 5] = -7
    out = ops.paged_attention_decode(q.cuda(), kc.cuda(), vc.cuda(), bad.cuda(), cl.cuda())
    torch.cuda.synchronize()
    assert torch.equal(out[0], good[0]) and torch.equal(out[2], good[2])
    assert torch.isfinite(out[1].float()).all()
    # what the clamp means: ids above the pool read the last block, negative ids block 0
    fixed = bt.clone()
    fixed[1, 3] = kc.shape[0] - 1
    fixed[1, 5] = 0
    assert torch.equal(out, ops.paged_attention_decode(q.cuda(), kc.cuda(), vc.cuda(), fixed.cuda(), cl.cuda()))


def test_ops_reject_tensors_on_different_devices(ops):
    print("case: mixed devices", flush=True)
    q = rnd(1, 2, 16, 64, seed=1).cuda()
    with pytest.raises(ValueError):
        ops.flash_attn_prefill(q, q.cpu(), q)


def test_ops_run_on_the_current_stream(ops):
    """The wrappers hand torch's CURRENT stream to the library: inside `torch.cuda.stream(s)` the kernels are ordered
    after the work already queued on s (here a chain of matrix products that takes milliseconds and whose result the
    inputs depend on) and give exactly what the default stream gives."""
    print("case: non-default stream", flush=True)
    dev = "cuda:0"
    q, k, v = (rnd(2, 4, 300, 64, seed=s, scale=0.5).to(dev) for s in (1, 2, 3))
    dq, kc, vc, bt, cl = (t.to(dev) for t in orc.make_paged_case(batch=3, n_q_heads=8, n_kv_heads=2, head_dim=128, block_size=16,
                                                                 context_lens=[700, 5000, 33], seed=9, dtype=torch.bfloat16))
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        a = torch.randn(2048, 2048, device=dev)
        for _ in range(30):
            a = torch.tanh(a @ a)
        zero = (a[0, 0] * 0).to(torch.bfloat16)          # 0, available only when the chain has finished
        out_p = ops.flash_attn_prefill(q + zero, k, v, causal=True)
        out_d = ops.paged_attention_decode(dq + zero, kc, vc, bt, cl)
    side.synchronize()
    ref_p = ops.flash_attn_prefill(q, k, v, causal=True)
    ref_d = ops.paged_attention_decode(dq, kc, vc, bt, cl)
    torch.cuda.synchronize()
    assert torch.equal(out_p, ref_p) and torch.equal(out_d, ref_d)
