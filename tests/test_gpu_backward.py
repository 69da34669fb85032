"""GPU parity of the prefill backward (dq, dk, dv) and of the forward's log-sum-exp against the
CPU oracle, through the C ABI (ops -> ctypes -> mi355_prefill_fwd_lse / mi355_prefill_bwd).

Tolerance: the kernels recompute P from bf16 inputs, round P and dS to bf16 for the second MFMA and
round the results to bf16; against the fp32 oracle on the same bf16 inputs a gradient element is
accepted within 1e-4 + 2e-2 * max|grad of that tensor| + 2e-2 |ref| (gradients of long sequences sum many
terms, so the absolute part scales with the tensor), and the relative RMS error must stay below 1.5 %.
lse: |got - ref| <= 3e-3 + 1e-3 |ref| (the kernels sum the weights as rounded to bf16 -- exactly what multiplies V --
so a row whose weights all round the same way is off by up to 2^-9 = 0.002 in its log-sum-exp).
"""
import pytest
import torch

from oracle import attention_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import mi355_attn
    mi355_attn.load()
    return mi355_attn


def rnd(*shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


def check_grad(name, got, ref):
    got = got.float().cpu()
    err = (got - ref).abs()
    bound = 1e-4 + 2e-2 * float(ref.abs().max()) + 2e-2 * ref.abs()
    rms = float((got - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt().clamp_min(1e-3))
    assert bool((err <= bound).all()), f"{name}: max err {float(err.max()):.4g} (ref max {float(ref.abs().max()):.4g})"
    assert rms < 1.5e-2, f"{name}: relative rms error {rms:.4f}"


def run_dense(ops, B, Hq, Hkv, Sq, Sk, D, causal, seed, scale=None):
    q, k, v = rnd(B, Hq, Sq, D, seed=seed), rnd(B, Hkv, Sk, D, seed=seed + 1), rnd(B, Hkv, Sk, D, seed=seed + 2)
    dout = rnd(B, Hq, Sq, D, seed=seed + 3)
    qg, kg, vg = (t.cuda().requires_grad_() for t in (q, k, v))
    out = ops.flash_attn_prefill(qg, kg, vg, causal=causal, softmax_scale=scale)
    out.backward(dout.cuda())
    torch.cuda.synchronize()
    dq, dk, dv, _ = orc.prefill_backward_reference(q, k, v, dout, causal=causal, softmax_scale=scale)
    ref_out = orc.prefill_reference(q, k, v, causal=causal, softmax_scale=scale)
    torch.testing.assert_close(out.detach().float().cpu(), ref_out, atol=2e-2, rtol=1e-2)
    check_grad("dq", qg.grad, dq)
    check_grad("dk", kg.grad, dk)
    check_grad("dv", vg.grad, dv)


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("causal", [True, False])
def test_backward_square(ops, D, causal):
    print(f"case: backward square D={D} causal={causal}", flush=True)
    run_dense(ops, 2, 4, 4, 256, 256, D, causal, seed=10 + D)


@pytest.mark.parametrize("Sq,Sk", [(1, 1), (7, 7), (65, 65), (129, 129), (200, 333), (128, 64 + 128), (33, 500)])
def test_backward_ragged_and_rectangular(ops, Sq, Sk):
    print(f"case: backward ragged Sq={Sq} Sk={Sk}", flush=True)
    run_dense(ops, 1, 2, 2, Sq, Sk, 64, True, seed=Sq + Sk)
    run_dense(ops, 1, 2, 2, Sq, Sk, 128, False, seed=Sq + Sk + 1)


def test_backward_gqa_and_custom_scale(ops):
    print("case: backward GQA", flush=True)
    run_dense(ops, 2, 8, 2, 192, 192, 128, True, seed=40)
    run_dense(ops, 1, 6, 1, 100, 100, 64, True, seed=41, scale=0.2)


def test_backward_config1_shape_with_reference_layouts(ops):
    """configs[1] (B4, H16, S1024, D64, causal) with the reference's tensor layouts: contiguous Q/K, V as the
    strided view of the (B, S, H*D) projection (model.py:367-370); dV must come back in V's layout."""
    print("case: backward config1 layouts", flush=True)
    B, H, S, D = 4, 16, 1024, 64
    q, k = rnd(B, H, S, D, seed=50, scale=0.5), rnd(B, H, S, D, seed=51, scale=0.5)
    vproj = rnd(B, S, H * D, seed=52, scale=0.5)
    dout = rnd(B, H, S, D, seed=53)
    qg, kg = q.cuda().requires_grad_(), k.cuda().requires_grad_()
    vp = vproj.cuda().requires_grad_()
    vview = vp.view(B, S, H, D).permute(0, 2, 1, 3)
    out = ops.sdpa_slot(qg, kg, vview, is_causal=True)
    out.backward(dout.cuda())
    torch.cuda.synchronize()
    v = vproj.view(B, S, H, D).permute(0, 2, 1, 3)
    dq, dk, dv, _ = orc.prefill_backward_reference(q, k, v, dout, causal=True)
    check_grad("dq", qg.grad, dq)
    check_grad("dk", kg.grad, dk)
    check_grad("dv", vp.grad.view(B, S, H, D).permute(0, 2, 1, 3), dv)


def test_backward_varlen_equals_per_sequence(ops):
    print("case: backward varlen", flush=True)
    lens = [37, 128, 1, 200, 64]
    Hq, Hkv, D = 4, 2, 128
    T = sum(lens)
    cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
    q, k, v, dout = rnd(T, Hq, D, seed=60), rnd(T, Hkv, D, seed=61), rnd(T, Hkv, D, seed=62), rnd(T, Hq, D, seed=63)
    qg, kg, vg = (t.cuda().requires_grad_() for t in (q, k, v))
    out = ops.flash_attn_varlen_prefill(qg, kg, vg, cu.cuda(), cu.cuda(), max(lens), max(lens), causal=True)
    out.backward(dout.cuda())
    torch.cuda.synchronize()
    dq_ref, dk_ref, dv_ref = torch.zeros(T, Hq, D), torch.zeros(T, Hkv, D), torch.zeros(T, Hkv, D)
    for b, n in enumerate(lens):
        sl = slice(int(cu[b]), int(cu[b + 1]))
        args = [t[sl].transpose(0, 1)[None] for t in (q, k, v, dout)]
        a, bb, c, _ = orc.prefill_backward_reference(*args, causal=True)
        dq_ref[sl], dk_ref[sl], dv_ref[sl] = a[0].transpose(0, 1), bb[0].transpose(0, 1), c[0].transpose(0, 1)
    check_grad("dq", qg.grad, dq_ref)
    check_grad("dk", kg.grad, dk_ref)
    check_grad("dv", vg.grad, dv_ref)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("seed", [0, 1])
def test_backward_packed_sequences_of_very_different_lengths(ops, D, seed):
    """Packed sequences from one token to several query tiles, 8 query heads on 2 kv heads: the grids of the two
    backward kernels then hold several chunks of workgroup ids per XCD, whole rounds of eight chunks and a partial
    one, and many workgroups of short sequences that have nothing to do."""
    g = torch.Generator().manual_seed(7000 + seed)
    n_seq = int(torch.randint(6, 10, (1,), generator=g))
    lens = [int(x) for x in torch.randint(1, 900, (n_seq,), generator=g)]
    lens[int(torch.randint(0, n_seq, (1,), generator=g))] = 1
    print(f"case: backward packed D={D} seed={seed} lens={lens}", flush=True)
    Hq, Hkv = 8, 2
    T = sum(lens)
    cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
    q, k, v, dout = (rnd(T, Hq, D, seed=7100 + seed), rnd(T, Hkv, D, seed=7200 + seed), rnd(T, Hkv, D, seed=7300 + seed),
                     rnd(T, Hq, D, seed=7400 + seed))
    qg, kg, vg = (t.cuda().requires_grad_() for t in (q, k, v))
    out = ops.flash_attn_varlen_prefill(qg, kg, vg, cu.cuda(), cu.cuda(), max(lens), max(lens), causal=True)
    out.backward(dout.cuda())
    torch.cuda.synchronize()
    dq_ref, dk_ref, dv_ref = torch.zeros(T, Hq, D), torch.zeros(T, Hkv, D), torch.zeros(T, Hkv, D)
    for b in range(n_seq):
        sl = slice(int(cu[b]), int(cu[b + 1]))
        args = [t[sl].transpose(0, 1)[None] for t in (q, k, v, dout)]
        a, bb, c, _ = orc.prefill_backward_reference(*args, causal=True)
        dq_ref[sl], dk_ref[sl], dv_ref[sl] = a[0].transpose(0, 1), bb[0].transpose(0, 1), c[0].transpose(0, 1)
    check_grad("dq", qg.grad, dq_ref)
    check_grad("dk", kg.grad, dk_ref)
    check_grad("dv", vg.grad, dv_ref)


@pytest.mark.parametrize("D", [64, 128])
def test_forward_lse_matches_oracle(ops, D):
    """head_dim 64: the 8-wavefront kernel; 128: the 64-query kernel, whose log-sum-exp comes from its row sums and
    the exponent reference that went into them -- also after that reference has moved (keys with runaway scores),
    for ragged packed sequences, and for rows past the end of a partial query tile."""
    print(f"case: forward lse D={D}", flush=True)
    from mi355_attn import ops as raw
    B, Hq, Hkv, S = 2, 4, 2, 300
    q, k, v = rnd(B, Hq, S, D, seed=70, scale=2.0), rnd(B, Hkv, S, D, seed=71), rnd(B, Hkv, S, D, seed=72)
    out, lse = raw._dense(q.cuda(), k.cuda(), v.cuda(), None, 1, None, want_lse=True)
    torch.cuda.synchronize()
    _, _, _, lse_ref = orc.prefill_backward_reference(q, k, v, torch.zeros(B, Hq, S, D), causal=True)
    torch.testing.assert_close(lse.cpu(), lse_ref, atol=3e-3, rtol=1e-3)
    # the output is unchanged by asking for lse
    assert torch.equal(out, ops.flash_attn_prefill(q.cuda(), k.cuda(), v.cuda(), causal=True, kv_splits=1))
    # runaway keys, no mask, more keys than queries
    Sq, Sk = 200, 1100
    q, k, v = rnd(1, Hq, Sq, D, seed=73), rnd(1, Hkv, Sk, D, seed=74).float(), rnd(1, Hkv, Sk, D, seed=75)
    k[:, :, 500:520] *= 25.0
    k[:, :, 900] *= -40.0
    k = k.to(torch.bfloat16)
    out, lse = raw._dense(q.cuda(), k.cuda(), v.cuda(), None, 0, None, want_lse=True)
    _, _, _, lse_ref = orc.prefill_backward_reference(q, k, v, torch.zeros(1, Hq, Sq, D), causal=False)
    torch.testing.assert_close(lse.cpu(), lse_ref, atol=3e-3, rtol=1e-3)


def test_backward_is_deterministic_and_linear_in_dout(ops):
    print("case: backward determinism / linearity", flush=True)
    B, H, S, D = 1, 4, 384, 128
    q, k, v = rnd(B, H, S, D, seed=80).cuda(), rnd(B, H, S, D, seed=81).cuda(), rnd(B, H, S, D, seed=82).cuda()
    d1 = rnd(B, H, S, D, seed=83).cuda()

    def grads(dout):
        qg, kg, vg = (t.clone().requires_grad_() for t in (q, k, v))
        ops.flash_attn_prefill(qg, kg, vg, causal=True).backward(dout)
        return qg.grad, kg.grad, vg.grad

    a, b = grads(d1), grads(d1)
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    c = grads(2 * d1)                               # exact in bf16: every product and sum doubles
    for x, y in zip(a, c):
        assert torch.equal((2 * x.float()).to(torch.bfloat16), y)


def test_no_grad_path_and_errors(ops):
    print("case: backward misc", flush=True)
    q = rnd(1, 2, 64, 64, seed=90).cuda().requires_grad_()
    k, v = rnd(1, 2, 64, 64, seed=91).cuda(), rnd(1, 2, 64, 64, seed=92).cuda()
    with torch.no_grad():
        out = ops.flash_attn_prefill(q, k, v)
    assert not out.requires_grad
    out = ops.flash_attn_prefill(q, k, v)
    assert out.requires_grad
    out.sum().backward()
    assert q.grad is not None and k.grad is None


def test_backward_rows_without_keys_and_empty_sequences(ops):
    """Causal with more queries than keys: the first Sq - Sk rows see no key (forward: NaN rows, like the
    reference softmax of an all-masked row); they must get dq = 0 and leave dk, dv untouched, i.e. the
    gradients equal those of the problem restricted to the rows that do see keys.  Packed batch with a
    sequence that has keys but no queries, and one with queries but no keys: every gradient row is
    written (zeros where nothing contributes)."""
    print("case: backward rows without keys / empty sequences", flush=True)
    B, Hq, Hkv, Sq, Sk, D = 1, 4, 2, 200, 130, 64
    q, k, v, dout = rnd(B, Hq, Sq, D, seed=90), rnd(B, Hkv, Sk, D, seed=91), rnd(B, Hkv, Sk, D, seed=92), rnd(B, Hq, Sq, D, seed=93)
    qg, kg, vg = (t.cuda().requires_grad_() for t in (q, k, v))
    out = ops.flash_attn_prefill(qg, kg, vg, causal=True)
    out.backward(dout.cuda())
    torch.cuda.synchronize()
    dead = Sq - Sk
    assert bool(torch.isnan(out[:, :, :dead].float()).all()) and bool(torch.isfinite(out[:, :, dead:].float()).all())
    dq_ref, dk_ref, dv_ref, _ = orc.prefill_backward_reference(q[:, :, dead:], k, v, dout[:, :, dead:], causal=True)
    assert bool((qg.grad[:, :, :dead] == 0).all())
    check_grad("dq", qg.grad[:, :, dead:], dq_ref)
    check_grad("dk", kg.grad, dk_ref)
    check_grad("dv", vg.grad, dv_ref)

    lens_q, lens_k = [70, 0, 33, 40], [70, 50, 33, 0]
    Hq, Hkv, D = 4, 2, 128
    cu_q = torch.tensor([0] + torch.tensor(lens_q).cumsum(0).tolist(), dtype=torch.int32)
    cu_k = torch.tensor([0] + torch.tensor(lens_k).cumsum(0).tolist(), dtype=torch.int32)
    Tq, Tk = sum(lens_q), sum(lens_k)
    q, k, v, dout = rnd(Tq, Hq, D, seed=94), rnd(Tk, Hkv, D, seed=95), rnd(Tk, Hkv, D, seed=96), rnd(Tq, Hq, D, seed=97)
    qg, kg, vg = (t.cuda().requires_grad_() for t in (q, k, v))
    out = ops.flash_attn_varlen_prefill(qg, kg, vg, cu_q.cuda(), cu_k.cuda(), max(lens_q), max(lens_k), causal=False)
    out.backward(dout.cuda())
    torch.cuda.synchronize()
    dq_ref, dk_ref, dv_ref = torch.zeros(Tq, Hq, D), torch.zeros(Tk, Hkv, D), torch.zeros(Tk, Hkv, D)
    for b in range(len(lens_q)):
        sq, sk = slice(int(cu_q[b]), int(cu_q[b + 1])), slice(int(cu_k[b]), int(cu_k[b + 1]))
        if lens_q[b] == 0 or lens_k[b] == 0:
            continue                                                   # nothing attends / nothing to attend: zero gradients
        args = [q[sq].transpose(0, 1)[None], k[sk].transpose(0, 1)[None], v[sk].transpose(0, 1)[None], dout[sq].transpose(0, 1)[None]]
        a, bb, c, _ = orc.prefill_backward_reference(*args, causal=False)
        dq_ref[sq], dk_ref[sk], dv_ref[sk] = a[0].transpose(0, 1), bb[0].transpose(0, 1), c[0].transpose(0, 1)
    assert bool(torch.isnan(out[int(cu_q[3]):].float()).all())        # queries without keys: NaN rows, as for any row that keeps no key
    check_grad("dq", qg.grad, dq_ref)
    check_grad("dk", kg.grad, dk_ref)
    check_grad("dv", vg.grad, dv_ref)


def oracle_masked_grads(q, k, v, mask, dout):
    """autograd through the oracle's restatement of model.py:308-325 in fp32: what the reference's own training step
    derives behind its non-flash branch."""
    qq, kk, vv = (t.float().requires_grad_() for t in (q, k, v))
    out = orc.scaled_dot_product_attention(qq, kk, vv, mask)
    out.backward(dout.float())
    return out.detach(), qq.grad, kk.grad, vv.grad


@pytest.mark.parametrize("S,D", [(256, 32), (200, 64), (131, 128), (384, 128)])
def test_masked_sdpa_trains_like_the_reference_non_flash_branch(ops, S, D):
    """llm-core/llm_core/model.py:384-385 as the reference runs it under autograd: the tril keep-mask rebuilt per call,
    handed to scaled_dot_product_attention with inputs that require grad.  Outputs and gradients against the oracle's
    causal backward (S = 131: rows that are no multiple of 4 bytes go through the padded copy of the mask)."""
    print(f"case: sdpa(Q, K, V, tril mask) under autograd S={S} D={D}", flush=True)
    B, H = 2, 4
    q, k, v, dout = (rnd(B, H, S, D, seed=300 + i + S) for i in range(4))
    qg, kg, vg = (t.cuda().requires_grad_() for t in (q, k, v))
    causal_mask = torch.tril(torch.ones(S, S, dtype=torch.bool, device="cuda"))          # model.py:384
    out = ops.scaled_dot_product_attention(qg, kg, vg, causal_mask)                        # model.py:385
    out.backward(dout.cuda())
    torch.cuda.synchronize()
    dq, dk, dv, _ = orc.prefill_backward_reference(q, k, v, dout, causal=True)
    torch.testing.assert_close(out.detach().float().cpu(), orc.prefill_reference(q, k, v, causal=True), atol=2e-2, rtol=1e-2)
    check_grad("dq", qg.grad, dq)
    check_grad("dk", kg.grad, dk)
    check_grad("dv", vg.grad, dv)


@pytest.mark.parametrize("mask_lead", ["none", "batch", "full"])
def test_masked_sdpa_backward_with_an_arbitrary_mask(ops, mask_lead):
    """A random keep-mask (no row fully masked), more keys than queries, the mask broadcast over heads and/or batch:
    gradients against autograd through the oracle's scaled_dot_product_attention."""
    print(f"case: sdpa backward, random mask, lead={mask_lead}", flush=True)
    B, H, Sq, Sk, D = 2, 3, 150, 212, 64
    q, k, v, dout = rnd(B, H, Sq, D, seed=400), rnd(B, H, Sk, D, seed=401), rnd(B, H, Sk, D, seed=402), rnd(B, H, Sq, D, seed=403)
    g = torch.Generator().manual_seed(404)
    lead = {"none": (), "batch": (B, 1), "full": (B, H)}[mask_lead]
    mask = torch.rand(*lead, Sq, Sk, generator=g) < 0.6
    mask[..., torch.arange(Sq), torch.arange(Sq)] = True
    qg, kg, vg = (t.cuda().requires_grad_() for t in (q, k, v))
    out = ops.scaled_dot_product_attention(qg, kg, vg, mask.cuda())
    out.backward(dout.cuda())
    torch.cuda.synchronize()
    ref, dq, dk, dv = oracle_masked_grads(q, k, v, mask, dout)
    torch.testing.assert_close(out.detach().float().cpu(), ref, atol=2e-2, rtol=1e-2)
    check_grad("dq", qg.grad, dq)
    check_grad("dk", kg.grad, dk)
    check_grad("dv", vg.grad, dv)


def test_masked_sdpa_backward_of_a_fully_masked_row(ops):
    """A query row whose keys are all masked: NaN output row like the reference softmax; its gradients are zero here
    (the reference propagates the NaN) and every other row's gradients are those of the problem without that row."""
    print("case: sdpa backward, one fully masked row", flush=True)
    B, H, S, D = 1, 2, 96, 64
    q, k, v, dout = (rnd(B, H, S, D, seed=500 + i) for i in range(4))
    mask = torch.tril(torch.ones(S, S, dtype=torch.bool))
    mask[17] = False
    qg, kg, vg = (t.cuda().requires_grad_() for t in (q, k, v))
    out = ops.scaled_dot_product_attention(qg, kg, vg, mask.cuda())
    out.backward(dout.cuda())
    torch.cuda.synchronize()
    assert bool(torch.isnan(out[:, :, 17].float()).all())
    keep = [i for i in range(S) if i != 17]
    _, dq, dk, dv = oracle_masked_grads(q[:, :, keep], k, v, mask[keep], dout[:, :, keep])
    assert bool((qg.grad[:, :, 17] == 0).all())
    check_grad("dq", qg.grad[:, :, keep], dq)
    check_grad("dk", kg.grad, dk)
    check_grad("dv", vg.grad, dv)
