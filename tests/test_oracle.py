"""Pins the CPU oracle: library equivalence, closed forms, invariants, brute force.

The reference (llm-core/llm_core/model.py:308-325, nn_functional.py:8-11) ships
no tests or fixtures, so the oracle is pinned by what the mathematics fixes and
by the library routine the reference itself treats as interchangeable
(model.py:381-385).  Each check is chosen so a plausible slip (dropped scale,
wrong mask polarity, transposed operand, wrong head mapping) fails it.
"""
import math

import numpy as np
import pytest
import torch

from oracle import attention_oracle as orc


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


# ---- library equivalence ---------------------------------------------------
@pytest.mark.parametrize("S,D", [(1, 8), (17, 16), (64, 64), (130, 128)])
def test_dense_equals_torch_sdpa_causal(S, D):
    Q, K, V = rnd(2, 3, S, D, seed=1), rnd(2, 3, S, D, seed=2), rnd(2, 3, S, D, seed=3)
    got = orc.scaled_dot_product_attention(Q, K, V, orc.causal_keep_mask(S))
    want = torch.nn.functional.scaled_dot_product_attention(Q, K, V, is_causal=True)
    torch.testing.assert_close(got, want, atol=2e-5, rtol=1e-5)


def test_dense_equals_torch_sdpa_nomask_and_boolmask():
    Q, K, V = rnd(2, 2, 9, 16, seed=4), rnd(2, 2, 13, 16, seed=5), rnd(2, 2, 13, 24, seed=6)
    got = orc.scaled_dot_product_attention(Q, K, V)
    want = torch.nn.functional.scaled_dot_product_attention(Q, K, V)
    torch.testing.assert_close(got, want, atol=2e-5, rtol=1e-5)
    g = torch.Generator().manual_seed(7)
    keep = torch.rand(9, 13, generator=g) > 0.4
    keep[:, 0] = True
    got = orc.scaled_dot_product_attention(Q, K, V, keep)
    want = torch.nn.functional.scaled_dot_product_attention(Q, K, V, attn_mask=keep)
    torch.testing.assert_close(got, want, atol=2e-5, rtol=1e-5)


def test_softmax_equals_torch_and_shift_invariant():
    x = rnd(5, 7, seed=8, scale=4.0)
    torch.testing.assert_close(orc.softmax(x, -1), torch.softmax(x, -1))
    torch.testing.assert_close(orc.softmax(x, 0), torch.softmax(x, 0))
    torch.testing.assert_close(orc.softmax(x + 1000.0, -1), orc.softmax(x, -1), atol=1e-6, rtol=1e-4)
    assert torch.isnan(orc.softmax(torch.full((1, 4), float("-inf")), -1)).all()


# ---- closed forms ----------------------------------------------------------
def test_single_key_returns_its_value():
    Q, K, V = rnd(3, 5, 8, seed=9), rnd(3, 1, 8, seed=10), rnd(3, 1, 6, seed=11)
    out = orc.scaled_dot_product_attention(Q, K, V)
    torch.testing.assert_close(out, V.expand(3, 5, 6))


def test_identical_keys_give_mean_of_values():
    Q = rnd(4, 8, seed=12)
    K = rnd(1, 8, seed=13).expand(6, 8)
    V = rnd(6, 5, seed=14)
    out = orc.scaled_dot_product_attention(Q, K, V)
    torch.testing.assert_close(out, V.mean(0, keepdim=True).expand(4, 5), atol=1e-6, rtol=1e-5)


def test_constant_values_pass_through():
    Q, K = rnd(4, 8, seed=15), rnd(9, 8, seed=16)
    V = torch.full((9, 3), 2.5)
    torch.testing.assert_close(orc.scaled_dot_product_attention(Q, K, V), torch.full((4, 3), 2.5))


def test_zero_query_causal_is_cumulative_mean():
    S = 11
    K, V = rnd(S, 8, seed=17), rnd(S, 4, seed=18)
    out = orc.scaled_dot_product_attention(torch.zeros(S, 8), K, V, orc.causal_keep_mask(S))
    want = torch.cumsum(V, 0) / torch.arange(1, S + 1).unsqueeze(1)
    torch.testing.assert_close(out, want, atol=1e-6, rtol=1e-5)
    torch.testing.assert_close(out[0], V[0])                 # causal row 0 sees key 0 only


def test_dominant_score_selects_value_and_scale_is_one_over_sqrt_d():
    d = 16
    K = torch.eye(5, d)
    V = rnd(5, 3, seed=19)
    Q = torch.zeros(1, d)
    Q[0, 2] = 400.0                                          # score 100 for key 2, 0 for others
    torch.testing.assert_close(orc.scaled_dot_product_attention(Q, K, V)[0], V[2])
    # exact weights pin the 1/sqrt(d) scale: scores (ln 3)·e_0 -> weights 3/7, 1/7 ...
    Q = torch.zeros(1, d)
    Q[0, 0] = math.log(3.0) * math.sqrt(d)
    out = orc.scaled_dot_product_attention(Q, K, V)[0]
    w = torch.tensor([3.0, 1, 1, 1, 1]) / 7.0
    torch.testing.assert_close(out, w @ V, atol=1e-6, rtol=1e-5)


def test_mask_polarity_true_means_keep():
    Q, K, V = rnd(2, 4, seed=20), rnd(3, 4, seed=21), rnd(3, 2, seed=22)
    keep = torch.tensor([[True, False, False], [False, False, True]])
    out = orc.scaled_dot_product_attention(Q, K, V, keep)
    torch.testing.assert_close(out, torch.stack([V[0], V[2]]))


def test_causal_mask_square_is_tril_and_rect_is_bottom_right():
    assert torch.equal(orc.causal_keep_mask(6), torch.tril(torch.ones(6, 6, dtype=torch.bool)))
    m = orc.causal_keep_mask(2, 5)
    assert m.tolist() == [[True, True, True, True, False], [True] * 5]


# ---- invariants ------------------------------------------------------------
def test_key_permutation_invariance():
    Q, K, V = rnd(4, 8, seed=23), rnd(10, 8, seed=24), rnd(10, 8, seed=25)
    p = torch.randperm(10, generator=torch.Generator().manual_seed(1))
    torch.testing.assert_close(orc.scaled_dot_product_attention(Q, K[p], V[p]),
                               orc.scaled_dot_product_attention(Q, K, V), atol=1e-6, rtol=1e-5)


def test_output_in_convex_hull():
    Q, K, V = rnd(6, 8, seed=26), rnd(12, 8, seed=27), rnd(12, 4, seed=28)
    out = orc.scaled_dot_product_attention(Q, K, V)
    assert (out <= V.max(0)[0] + 1e-6).all() and (out >= V.min(0)[0] - 1e-6).all()


def test_custom_scale_equals_scaled_keys():
    q, k, v = rnd(1, 2, 7, 16, seed=29), rnd(1, 2, 7, 16, seed=30), rnd(1, 2, 7, 16, seed=31)
    a = orc.prefill_reference(q, k, v, causal=True, softmax_scale=0.7)
    b = orc.prefill_reference(q, k * (0.7 * 4.0), v, causal=True)      # default 1/sqrt(16)=1/4
    torch.testing.assert_close(a, b, atol=1e-5, rtol=1e-5)


def test_gqa_equals_mha_on_repeated_heads_and_head_mapping():
    q = rnd(2, 6, 9, 8, seed=32)
    k, v = rnd(2, 2, 9, 8, seed=33), rnd(2, 2, 9, 8, seed=34)
    a = orc.prefill_reference(q, k, v, causal=True, head_chunk=4)
    kk, vv = k.repeat_interleave(3, 1), v.repeat_interleave(3, 1)
    b = orc.scaled_dot_product_attention(q, kk, vv, orc.causal_keep_mask(9))
    torch.testing.assert_close(a, b, atol=1e-6, rtol=1e-5)
    # head 3 must read kv head 1 (3 // 3), not 3 % 2
    c = orc.scaled_dot_product_attention(q[:, 3], k[:, 1], v[:, 1], orc.causal_keep_mask(9))
    torch.testing.assert_close(a[:, 3], c, atol=1e-6, rtol=1e-5)


def test_varlen_equals_per_sequence_dense():
    lens = [5, 1, 12]
    cu = torch.tensor([0, 5, 6, 18], dtype=torch.int32)
    q, k, v = rnd(18, 4, 8, seed=35), rnd(18, 2, 8, seed=36), rnd(18, 2, 8, seed=37)
    out = orc.varlen_prefill_reference(q, k, v, cu, cu, causal=True)
    off = 0
    for L in lens:
        qb = q[off:off + L].transpose(0, 1)[None]
        kb = k[off:off + L].transpose(0, 1)[None]
        vb = v[off:off + L].transpose(0, 1)[None]
        want = orc.prefill_reference(qb, kb, vb, causal=True)[0].transpose(0, 1)
        torch.testing.assert_close(out[off:off + L], want)
        off += L


def test_batch_elements_independent():
    q, k, v = rnd(3, 2, 6, 8, seed=38), rnd(3, 2, 6, 8, seed=39), rnd(3, 2, 6, 8, seed=40)
    full = orc.prefill_reference(q, k, v)
    one = orc.prefill_reference(q[1:2], k[1:2], v[1:2])
    torch.testing.assert_close(full[1:2], one)


# ---- brute force -----------------------------------------------------------
@pytest.mark.parametrize("S", [1, 2, 15, 16, 17, 33])
def test_dense_vs_float64_loops(S):
    Q, K, V = rnd(S, 8, seed=41 + S), rnd(S, 8, seed=42 + S), rnd(S, 5, seed=43 + S)
    keep = orc.causal_keep_mask(S)
    want = orc.bruteforce_attention_f64(Q.numpy(), K.numpy(), V.numpy(), keep.tolist())
    got = orc.scaled_dot_product_attention(Q, K, V, keep).numpy()
    np.testing.assert_allclose(got, want, atol=2e-6, rtol=1e-5)


# ---- paged decode ----------------------------------------------------------
def _paged(ctx, seed=0, Hq=4, Hkv=2, D=8, bs=16, pool_factor=1.5):
    return orc.make_paged_case(batch=len(ctx), n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D,
                               block_size=bs, context_lens=ctx, pool_factor=pool_factor, seed=seed)


@pytest.mark.parametrize("ctx", [[1], [15, 16, 17], [255, 256, 257], [33, 1, 64]])
def test_paged_decode_vs_float64_loops(ctx):
    q, kc, vc, bt, cl = _paged(ctx, seed=3)
    got = orc.paged_decode_reference(q, kc, vc, bt, cl)
    Hq, Hkv, bs = q.shape[1], kc.shape[1], kc.shape[2]
    for b in range(len(ctx)):
        for h in range(Hq):
            g = h // (Hq // Hkv)
            rows_k = [kc[int(bt[b, t // bs]), g, t % bs] for t in range(ctx[b])]   # token-by-token walk
            rows_v = [vc[int(bt[b, t // bs]), g, t % bs] for t in range(ctx[b])]
            want = orc.bruteforce_attention_f64(q[b, h][None].numpy(), torch.stack(rows_k).numpy(),
                                                torch.stack(rows_v).numpy())
            np.testing.assert_allclose(got[b, h].numpy(), want[0], atol=2e-6, rtol=1e-5)


def test_paged_decode_invariant_to_physical_placement_and_pool_garbage():
    ctx = [40, 7, 100]
    q, kc, vc, bt, cl = _paged(ctx, seed=5, pool_factor=2.0)
    base = orc.paged_decode_reference(q, kc, vc, bt, cl)
    # move every used block to a new physical slot
    pool = kc.shape[0]
    perm = torch.randperm(pool, generator=torch.Generator().manual_seed(9))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(pool)
    kc2, vc2 = kc[perm], vc[perm]                 # new slot i holds old block perm[i]
    bt2 = inv[bt.long()].to(torch.int32)
    torch.testing.assert_close(orc.paged_decode_reference(q, kc2, vc2, bt2, cl), base)
    # garbage in unused blocks and in the tail of the last block must not matter
    used = torch.zeros(pool, dtype=torch.bool)
    for b, c in enumerate(ctx):
        used[bt[b, :(c + 15) // 16].long()] = True
    kc3, vc3 = kc.clone(), vc.clone()
    kc3[~used] = 1e4
    vc3[~used] = -1e4
    for b, c in enumerate(ctx):
        if c % 16:
            last = int(bt[b, (c - 1) // 16])
            kc3[last, :, c % 16:] = 1e4
            vc3[last, :, c % 16:] = 1e4
    torch.testing.assert_close(orc.paged_decode_reference(q, kc3, vc3, bt, cl), base)


def test_paged_decode_equals_dense_last_row_of_causal_prefill():
    S, Hq, Hkv, D = 37, 4, 2, 8
    q, k, v = rnd(1, Hq, S, D, seed=50), rnd(1, Hkv, S, D, seed=51), rnd(1, Hkv, S, D, seed=52)
    dense = orc.prefill_reference(q, k, v, causal=True)[0, :, -1]          # (Hq,D)
    nblk = (S + 15) // 16
    kc = torch.zeros(nblk + 2, Hkv, 16, D)
    vc = torch.zeros(nblk + 2, Hkv, 16, D)
    table = torch.tensor([[2, 0, 4]], dtype=torch.int32)
    for t in range(S):
        kc[int(table[0, t // 16]), :, t % 16] = k[0, :, t]
        vc[int(table[0, t // 16]), :, t % 16] = v[0, :, t]
    got = orc.paged_decode_reference(q[:, :, -1], kc, vc, table, torch.tensor([S], dtype=torch.int32))
    torch.testing.assert_close(got[0], dense, atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("bounds", [[(0, 50)], [(0, 16), (16, 50)], [(0, 1), (1, 2), (2, 49), (49, 50)]])
def test_split_combine_independent_of_splits(bounds):
    q, k, v = rnd(8, seed=60), rnd(50, 8, seed=61), rnd(50, 8, seed=62)
    want = orc.scaled_dot_product_attention(q[None], k, v)[0]
    got = orc.combine_splits_reference(orc.split_partials_reference(q, k, v, bounds))
    torch.testing.assert_close(got, want, atol=1e-6, rtol=1e-5)


# ---- fp8 KV ----------------------------------------------------------------
def test_fp8_quantiser_properties():
    x = rnd(6, 2, 16, 32, seed=70).to(torch.bfloat16)
    x[3] = 0                                                    # all-zero blocks
    q8, sc = orc.quantize_kv_fp8(x)
    assert q8.dtype == torch.uint8 and sc.shape == (6, 2) and sc.dtype == torch.float32
    assert (sc[3] == 1.0).all() and (q8[3] == 0).all()
    torch.testing.assert_close(sc[:3], x[:3].float().abs().amax((2, 3)) / 448.0)
    dq = orc.dequantize_kv_fp8(q8, sc)
    xf = x.float()
    # absmax element maps to +-448 exactly
    for b in (0, 1, 2, 4, 5):
        for h in range(2):
            i = xf[b, h].abs().argmax()
            assert abs(q8[b, h].view(torch.float8_e4m3fn).float().flatten()[i]) == 448.0
    # e4m3 keeps 3 mantissa bits: relative error <= 2^-4 for normals (|y| >= 2^-6 after scaling)
    y = xf / sc[:, :, None, None]
    normal = y.abs() >= 2.0 ** -6
    rel = ((dq - xf).abs() / xf.abs().clamp_min(1e-30))[normal]
    assert rel.max() <= 2.0 ** -4 + 1e-6
    # subnormals: absolute error <= half of the subnormal step 2^-9, times scale
    err_sub = ((dq - xf).abs() / sc[:, :, None, None])[~normal]
    assert err_sub.numel() == 0 or err_sub.max() <= 2.0 ** -10 + 1e-9


def test_fp8_e4m3_bit_patterns_are_ocp():
    # OCP e4m3fn: 0x7E = 448, 0x38 = 1.0, 0x01 = 2^-9, 0x7F = NaN (no infinities)
    b = torch.tensor([0x7E, 0x38, 0x01, 0xB8], dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    assert b.tolist() == [448.0, 1.0, 2.0 ** -9, -1.0]


def test_paged_decode_fp8_equals_oracle_on_dequantised_cache():
    ctx = [45, 16]
    q, kc, vc, bt, cl = _paged(ctx, seed=8, D=16)
    k8, ks = orc.quantize_kv_fp8(kc)
    v8, vs = orc.quantize_kv_fp8(vc)
    a = orc.paged_decode_reference(q, k8, v8, bt, cl, k_scale=ks, v_scale=vs)
    b = orc.paged_decode_reference(q, orc.dequantize_kv_fp8(k8, ks), orc.dequantize_kv_fp8(v8, vs), bt, cl)
    torch.testing.assert_close(a, b)
    full = orc.paged_decode_reference(q, kc, vc, bt, cl)
    assert (a - full).abs().max() < 0.15                       # quantisation noise only


# ---- workload generators ---------------------------------------------------
def test_workload_generators_are_seeded_and_well_formed():
    c1 = orc.draw_context_lens("uniform", 128, 512, 16384, 0)
    c2 = orc.draw_context_lens("uniform", 128, 512, 16384, 0)
    assert torch.equal(c1, c2) and c1.min() >= 512 and c1.max() <= 16384
    c3 = orc.draw_context_lens("loguniform", 256, 128, 32768, 0)
    assert c3.min() >= 128 and c3.max() <= 32768 and c3.float().median() < 5000
    q, kc, vc, bt, cl = orc.make_paged_case(batch=4, n_q_heads=8, n_kv_heads=8, head_dim=64, block_size=16,
                                            context_lens=[256] * 4, seed=0)
    assert kc.shape == (64, 8, 16, 64) and bt.shape == (4, 16)
    assert sorted(bt.flatten().tolist()) == list(range(64))     # a permutation of the 64 physical blocks


# ---- RoPE ------------------------------------------------------------------
def test_rope_equals_complex_rotation_and_cache_layout():
    d, ctx = 16, 50
    fc = orc.build_rope_cache(ctx, d)
    assert fc.shape == (2, ctx, d // 2)
    x = rnd(3, 7, d, seed=80)
    pos = torch.tensor([0, 1, 5, 17, 49, 3, 3])
    got = orc.rope_reference(x, pos, fc)
    # independent formulation: (x1 + i x2) * exp(i * pos * theta^(-2j/d)), in float64
    inv = 10000.0 ** (-np.arange(0, d, 2) / d)
    ang = pos.numpy()[:, None] * inv[None, :]
    z = (x[..., 0::2].numpy().astype(np.float64) + 1j * x[..., 1::2].numpy().astype(np.float64)) * np.exp(1j * ang)
    want = np.stack([z.real, z.imag], axis=-1).reshape(3, 7, d)
    np.testing.assert_allclose(got.numpy(), want, atol=2e-5, rtol=1e-5)
    torch.testing.assert_close(got[:, 0], x[:, 0])                       # position 0 is the identity
    # pair norms are preserved and scores depend on the position difference only
    torch.testing.assert_close(got.pow(2).unflatten(-1, (d // 2, 2)).sum(-1), x.pow(2).unflatten(-1, (d // 2, 2)).sum(-1),
                               atol=1e-5, rtol=1e-5)
    a, b = rnd(1, d, seed=81), rnd(1, d, seed=82)
    s1 = (orc.rope_reference(a, torch.tensor([9]), fc) * orc.rope_reference(b, torch.tensor([4]), fc)).sum()
    s2 = (orc.rope_reference(a, torch.tensor([25]), fc) * orc.rope_reference(b, torch.tensor([20]), fc)).sum()
    torch.testing.assert_close(s1, s2, atol=1e-4, rtol=1e-4)


def test_rope_and_cache_reference_scatters_to_slots():
    T, Hq, Hkv, D = 5, 4, 2, 8
    fc = orc.build_rope_cache(32, D)
    q, k, v = rnd(T, Hq, D, seed=83), rnd(T, Hkv, D, seed=84), rnd(T, Hkv, D, seed=85)
    pos = torch.tensor([3, 4, 5, 0, 9], dtype=torch.int32)
    slots = torch.tensor([16 * 2 + 3, 16 * 2 + 4, 16 * 0 + 15, -1, 16 * 1 + 0])
    kc, vc = torch.zeros(3, Hkv, 16, D), torch.zeros(3, Hkv, 16, D)
    q_rot, kc2, vc2 = orc.rope_and_cache_reference(q, k, v, pos, fc, kc, vc, slots)
    torch.testing.assert_close(q_rot[3], q[3])                                  # position 0
    torch.testing.assert_close(vc2[2, :, 3], v[0])
    torch.testing.assert_close(vc2[0, :, 15], v[2])
    torch.testing.assert_close(kc2[1, :, 0], orc.rope_reference(k[4][:, None], torch.tensor([9]), fc)[:, 0])
    assert kc2.abs().sum(dim=(1, 3)).count_nonzero() == 4                       # token 3 (slot -1) was not written


def test_fp8_append_whole_block_equals_block_quantiser():
    """One run that fills a block from offset 0 is exactly quantize_kv_fp8 of that block (scale and bytes)."""
    g = torch.Generator().manual_seed(31)
    rows = (torch.randn(16, 64, generator=g) * 3).to(torch.bfloat16).float()
    junk = torch.randint(0, 255, (16, 64), generator=g).to(torch.uint8)
    got8, got_scale = orc.append_rows_fp8(junk, 123.0, rows, 0)           # what the slab held before is dead
    ref8, ref_scale = orc.quantize_kv_fp8(rows.view(1, 1, 16, 64))
    assert torch.equal(got8, ref8[0, 0]) and got_scale == float(ref_scale[0, 0])
    z8, z_scale = orc.append_rows_fp8(junk, 5.0, torch.zeros(3, 64), 0)   # all-zero rows: guarded scale
    assert z_scale == 1.0 and torch.equal(z8[:3], torch.zeros(3, 64, dtype=torch.uint8)) and torch.equal(z8[3:], junk[3:])


def test_fp8_append_keeps_scale_equal_to_block_absmax_and_bounds_the_error():
    """Token-by-token appends: the scale is always absmax(valid rows)/448 (what the block quantiser
    gives); rows written under an unchanged scale keep their bytes; every re-expression costs at most
    one more e4m3 rounding (relative 2^-4 on normals, half a subnormal step below)."""
    g = torch.Generator().manual_seed(32)
    rows = (torch.randn(16, 128, generator=g) * torch.linspace(0.3, 2.0, 16)[:, None]).to(torch.bfloat16).float()
    block8 = torch.zeros(16, 128, dtype=torch.uint8)
    scale, raises = 0.0, 0
    for t in range(16):
        before, old = block8.clone(), scale
        block8, scale = orc.append_rows_fp8(block8, scale, rows[t:t + 1], t)
        assert scale == float(rows[:t + 1].abs().amax() / orc.FP8_E4M3_MAX)
        if t and scale == old:
            assert torch.equal(block8[:t], before[:t])
        elif t:
            raises += 1
        deq = block8[:t + 1].view(torch.float8_e4m3fn).float() * scale
        step = scale * 2.0 ** -9                                           # e4m3 subnormal spacing, in real units
        bound = (raises + 1) * (2.0 ** -4 * rows[:t + 1].abs() + step)
        assert bool(((deq - rows[:t + 1]).abs() <= bound).all())
    assert raises >= 2                                                     # the growing rows did raise the scale


def test_fp8_append_reexpression_is_exact_for_power_of_two_scale_changes():
    """When the scale doubles, bytes well inside the normal range just lose one exponent step: the
    re-expressed value equals the old one whenever it stays representable."""
    rows0 = torch.tensor([[448.0, 224.0, 112.0, 3.5, -28.0, 0.0, 1.75, 56.0]])        # scale 1.0
    b8, s = orc.append_rows_fp8(torch.zeros(16, 8, dtype=torch.uint8), 0.0, rows0, 0)
    assert s == 1.0
    b8, s = orc.append_rows_fp8(b8, s, torch.full((1, 8), 896.0), 1)                   # scale 2.0
    assert s == 2.0
    assert torch.equal(b8[0].view(torch.float8_e4m3fn).float() * s, rows0[0])
    assert torch.equal(b8[1].view(torch.float8_e4m3fn).float() * s, torch.full((8,), 896.0))


def test_rope_and_cache_fp8_reference_runs_and_layout():
    """With whole-block runs the fp8 cache equals quantize_kv_fp8 of the bf16 cache that
    rope_and_cache_reference builds; decode-style single-token appends keep scale = absmax/448."""
    g = torch.Generator().manual_seed(33)
    T, Hq, Hkv, D, ctx, nb = 48, 4, 2, 32, 64, 5
    q = torch.randn(T, Hq, D, generator=g).to(torch.bfloat16)
    k = torch.randn(T, Hkv, D, generator=g).to(torch.bfloat16)
    v = torch.randn(T, Hkv, D, generator=g).to(torch.bfloat16)
    fc = orc.build_rope_cache(ctx, D)
    pos = torch.arange(T, dtype=torch.int32) % ctx
    blocks = [3, 0, 4]                                                     # three full blocks of one sequence
    slots = torch.tensor([blocks[t // 16] * 16 + t % 16 for t in range(T)], dtype=torch.int64)
    k8 = torch.randint(0, 255, (nb, Hkv, 16, D), generator=g).to(torch.uint8)
    v8 = torch.randint(0, 255, (nb, Hkv, 16, D), generator=g).to(torch.uint8)
    ks, vs = torch.rand(nb, Hkv, generator=g), torch.rand(nb, Hkv, generator=g)
    q_rot, k8n, ksn, v8n, vsn = orc.rope_and_cache_fp8_reference(q, k, v, pos, fc, k8, ks, v8, vs, slots)
    q_ref, kc, vc = orc.rope_and_cache_reference(q, k, v, pos, fc, torch.zeros(nb, Hkv, 16, D), torch.zeros(nb, Hkv, 16, D), slots)
    assert torch.equal(q_rot, q_ref)
    rk8, rks = orc.quantize_kv_fp8(kc.to(torch.bfloat16))
    rv8, rvs = orc.quantize_kv_fp8(vc)
    for b in blocks:
        assert torch.equal(k8n[b], rk8[b]) and torch.equal(ksn[b], rks[b])
        assert torch.equal(v8n[b], rv8[b]) and torch.equal(vsn[b], rvs[b])
    for b in (1, 2):                                                       # untouched blocks keep bytes and scales
        assert torch.equal(k8n[b], k8[b]) and torch.equal(ksn[b], ks[b]) and torch.equal(v8n[b], v8[b])
    # the same tokens one call at a time (a decode loop): scales end up identical, bytes differ only by re-expression
    k8d, v8d, ksd, vsd = k8.clone(), v8.clone(), ks.clone(), vs.clone()
    for t in range(T):
        _, k8d, ksd, v8d, vsd = orc.rope_and_cache_fp8_reference(q[t:t + 1], k[t:t + 1], v[t:t + 1], pos[t:t + 1], fc,
                                                                 k8d, ksd, v8d, vsd, slots[t:t + 1])
    for b in blocks:
        assert torch.equal(ksd[b], rks[b]) and torch.equal(vsd[b], rvs[b])
        err = (orc.dequantize_kv_fp8(v8d, vsd)[b] - vc[b]).abs()
        assert bool((err <= 16 * (2.0 ** -4 * vc[b].abs() + vsd[b][:, None, None] * 2.0 ** -9)).all())
    # a slot outside the pool or negative is skipped
    bad = slots.clone()
    bad[0], bad[1] = -1, nb * 16
    _, k8b, _, _, _ = orc.rope_and_cache_fp8_reference(q[:2], k[:2], v[:2], pos[:2], fc, k8, ks, v8, vs, bad[:2])
    assert torch.equal(k8b, k8)


# ---------------------------------------------------------------------------------------------
# backward oracle
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("hq,hkv,sq,sk", [(4, 4, 9, 9), (6, 2, 7, 12), (2, 1, 5, 5)])
def test_backward_oracle_matches_autograd_of_the_dense_function(causal, hq, hkv, sq, sk):
    g = torch.Generator().manual_seed(hq * 100 + sq)
    q = torch.randn(2, hq, sq, 16, generator=g, requires_grad=True)
    k = torch.randn(2, hkv, sk, 16, generator=g, requires_grad=True)
    v = torch.randn(2, hkv, sk, 16, generator=g, requires_grad=True)
    dout = torch.randn(2, hq, sq, 16, generator=g)
    n_rep = hq // hkv
    mask = orc.causal_keep_mask(sq, sk) if causal else None
    out = orc.scaled_dot_product_attention(q, orc.expand_kv_heads(k, n_rep, 1), orc.expand_kv_heads(v, n_rep, 1), mask)
    want = torch.autograd.grad(out, (q, k, v), dout)
    dq, dk, dv, lse = orc.prefill_backward_reference(q.detach(), k.detach(), v.detach(), dout, causal=causal)
    for a, b in zip((dq, dk, dv), want):
        torch.testing.assert_close(a, b, atol=2e-5, rtol=2e-5)
    # lse is the log of the softmax denominator of the scaled scores
    s = torch.einsum("bhqd,bhkd->bhqk", q.detach(), orc.expand_kv_heads(k.detach(), n_rep, 1)) / 4.0
    if causal:
        s = torch.where(mask, s, float("-inf"))
    torch.testing.assert_close(lse, torch.log(torch.exp(s).sum(-1)), atol=1e-5, rtol=1e-5)


def test_backward_oracle_matches_float64_finite_differences_and_scale():
    g = torch.Generator().manual_seed(77)
    q, k, v = (torch.randn(1, 2, 4, 8, generator=g, dtype=torch.float64) for _ in range(3))
    dout = torch.randn(1, 2, 4, 8, generator=g, dtype=torch.float64)
    scale = 0.37

    def loss(q_, k_, v_):
        keep = orc.causal_keep_mask(4).tolist()
        tot = 0.0
        for h in range(2):                    # the 2-D float64 loop function, head by head
            o = orc.bruteforce_attention_f64((q_[0, h] * (scale * math.sqrt(8))).numpy(), k_[0, h].numpy(),
                                             v_[0, h].numpy(), keep)
            tot += float((o * dout[0, h].numpy()).sum())
        return tot

    dq, dk, dv, _ = orc.prefill_backward_reference(q.float(), k.float(), v.float(), dout.float(), causal=True,
                                                   softmax_scale=scale)
    eps = 1e-5
    for name, t, grad in (("q", q, dq), ("k", k, dk), ("v", v, dv)):
        for idx in [(0, 0, 0, 0), (0, 1, 2, 5), (0, 0, 3, 7), (0, 1, 1, 3)]:
            tp, tm = t.clone(), t.clone()
            tp[idx] += eps
            tm[idx] -= eps
            args_p = {"q": (tp, k, v), "k": (q, tp, v), "v": (q, k, tp)}[name]
            args_m = {"q": (tm, k, v), "k": (q, tm, v), "v": (q, k, tm)}[name]
            fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(fd - float(grad[idx])) < 2e-4, (name, idx, fd, float(grad[idx]))


def test_backward_oracle_closed_forms():
    # one key: out = v for every query, so dv = sum of dout rows, dq = dk = 0
    g = torch.Generator().manual_seed(5)
    q, dout = torch.randn(1, 1, 6, 8, generator=g), torch.randn(1, 1, 6, 8, generator=g)
    k, v = torch.randn(1, 1, 1, 8, generator=g), torch.randn(1, 1, 1, 8, generator=g)
    dq, dk, dv, _ = orc.prefill_backward_reference(q, k, v, dout, causal=False)
    torch.testing.assert_close(dv[0, 0, 0], dout[0, 0].sum(0))
    assert dq.abs().max() < 1e-6 and dk.abs().max() < 1e-6
    # gradients w.r.t. q and k vanish when dout is a multiple of ... a constant-V problem: out is constant
    v2 = torch.ones(1, 1, 5, 8)
    k2 = torch.randn(1, 1, 5, 8, generator=g)
    dq, dk, _, _ = orc.prefill_backward_reference(q, k2, v2, dout, causal=False)
    assert dq.abs().max() < 1e-5 and dk.abs().max() < 1e-5


def test_paged_prefill_reference_is_the_tail_of_a_whole_prefill():
    """A chunk attending to its cached context gives rows [c0, c1) of the causal prefill of the first c1 tokens."""
    Hq, Hkv, D = 4, 2, 16
    ctx = [45, 23]
    chunk = [13, 23]
    _, kc, vc, bt, cl = orc.make_paged_case(batch=2, n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, block_size=16,
                                            context_lens=ctx, pool_factor=1.5, seed=3)
    g = torch.Generator().manual_seed(4)
    q_full = [torch.randn(c, Hq, D, generator=g) for c in ctx]
    q = torch.cat([qf[c - n:] for qf, c, n in zip(q_full, ctx, chunk)])
    cu = torch.tensor([0, 13, 36])
    got = orc.paged_prefill_reference(q, kc, vc, cu, bt, cl)
    for b in range(2):
        kk = orc.gather_paged_kv(kc, bt[b], ctx[b])[None]
        vv = orc.gather_paged_kv(vc, bt[b], ctx[b])[None]
        whole = orc.prefill_reference(q_full[b].transpose(0, 1)[None], kk, vv, causal=True)[0].transpose(0, 1)
        torch.testing.assert_close(got[int(cu[b]):int(cu[b + 1])], whole[ctx[b] - chunk[b]:], rtol=1e-5, atol=1e-6)
