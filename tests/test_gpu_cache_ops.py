"""GPU parity of the cache producers (RoPE + cache write, fp8 quantisation) and an end-to-end
decode loop built from them: every decode step over the growing paged cache must equal the
matching row of one causal prefill over the whole sequence."""
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


@pytest.mark.parametrize("D", [32, 64, 128])
def test_rope_and_cache_matches_oracle(ops, D):
    print(f"case: rope_and_cache D={D}", flush=True)
    T, Hq, Hkv, ctx = 37, 8, 2, 256
    q, k, v = rnd(T, Hq, D, seed=1), rnd(T, Hkv, D, seed=2), rnd(T, Hkv, D, seed=3)
    g = torch.Generator().manual_seed(4)
    pos = torch.randint(0, ctx, (T,), generator=g).to(torch.int32)
    pos[0] = 0
    slots = torch.randperm(6 * 16, generator=g)[:T].to(torch.int64)
    slots[5] = -1
    kc0, vc0 = rnd(6, Hkv, 16, D, seed=5), rnd(6, Hkv, 16, D, seed=6)
    fc = orc.build_rope_cache(ctx, D)
    q_ref, kc_ref, vc_ref = orc.rope_and_cache_reference(q, k, v, pos, fc, kc0, vc0, slots)
    kc, vc = kc0.cuda(), vc0.cuda()
    fcg = ops.build_rope_cache(ctx, D)
    torch.testing.assert_close(fcg.cpu(), fc, atol=1e-6, rtol=1e-6)
    q_rot = ops.rope_and_cache(q.cuda(), k.cuda(), v.cuda(), pos.cuda(), fcg, kc, vc, slots.cuda())
    torch.cuda.synchronize()
    # fp32 math, one rounding to bf16: within one bf16 ulp of the fp32 oracle
    torch.testing.assert_close(q_rot.float().cpu(), q_ref, atol=2 ** -7, rtol=2 ** -7)
    torch.testing.assert_close(kc.float().cpu(), kc_ref, atol=2 ** -7, rtol=2 ** -7)
    assert torch.equal(vc.cpu().float(), vc_ref)                      # values are copied bit for bit
    assert torch.equal(q_rot[0].cpu(), q[0])                          # position 0: identity, exact


def test_rope_and_cache_pair_path_and_out_argument(ops):
    """Token strides that are not multiples of 8 elements take the 4-byte kernel; it and the
    16-byte kernel must give identical bits.  Also covers out= (in place on q)."""
    print("case: rope_and_cache pair path / out=", flush=True)
    T, Hq, Hkv, D, ctx = 53, 4, 2, 64, 128
    g = torch.Generator().manual_seed(11)
    pos = torch.randint(0, ctx, (T,), generator=g).to(torch.int32).cuda()
    slots = torch.randperm(4 * 16, generator=g)[:T].to(torch.int64).cuda()
    fcg = ops.build_rope_cache(ctx, D)
    q, k, v = rnd(T, Hq, D, seed=12).cuda(), rnd(T, Hkv, D, seed=13).cuda(), rnd(T, Hkv, D, seed=14).cuda()
    kc_a, vc_a = torch.zeros(4, Hkv, 16, D, dtype=torch.bfloat16, device="cuda"), torch.zeros(4, Hkv, 16, D, dtype=torch.bfloat16, device="cuda")
    kc_b, vc_b = torch.zeros_like(kc_a), torch.zeros_like(vc_a)
    q_a = ops.rope_and_cache(q, k, v, pos, fcg, kc_a, vc_a, slots)
    # the same rows inside a wider buffer: token stride Hq*D + 2 elements (even, not a multiple of 8)
    wide = torch.zeros(T, Hq * D + 2, dtype=torch.bfloat16, device="cuda")
    q_view = wide[:, :Hq * D].view(T, Hq, D)
    q_view.copy_(q)
    assert q_view.stride(0) % 8 != 0
    q_b = ops.rope_and_cache(q_view, k, v, pos, fcg, kc_b, vc_b, slots)
    torch.cuda.synchronize()
    assert torch.equal(q_a, q_b) and torch.equal(kc_a, kc_b) and torch.equal(vc_a, vc_b)
    q_inplace = q.clone()
    ret = ops.rope_and_cache(q_inplace, k, v, pos, fcg, kc_b, vc_b, slots, out=q_inplace)
    torch.cuda.synchronize()
    assert ret is q_inplace and torch.equal(q_inplace, q_a)
    with pytest.raises(ValueError):
        ops.rope_and_cache(q, k, v, pos, fcg, kc_b, vc_b, slots, out=torch.empty(T, Hq, D + 8, dtype=torch.bfloat16, device="cuda"))


def test_rope_and_cache_ignores_slots_outside_the_pool_and_clamps_positions(ops):
    print("case: rope_and_cache bad slots / positions", flush=True)
    T, Hq, Hkv, D, ctx, nb = 8, 2, 2, 64, 32, 3
    q, k, v = rnd(T, Hq, D, seed=21).cuda(), rnd(T, Hkv, D, seed=22).cuda(), rnd(T, Hkv, D, seed=23).cuda()
    fcg = ops.build_rope_cache(ctx, D)
    pos = torch.tensor([0, 1, 2, 3, 31, 32, 1000, -5], dtype=torch.int32).cuda()
    slots = torch.tensor([0, 1, nb * 16, 2 ** 40, 5, -1, 47, 46], dtype=torch.int64).cuda()
    guard = torch.full((nb + 2, Hkv, 16, D), 7.0, dtype=torch.bfloat16, device="cuda")      # pool = blocks 1..nb of this buffer
    kc, vc = guard[1:nb + 1], guard.clone()[1:nb + 1]
    q_rot = ops.rope_and_cache(q, k, v, pos, fcg, kc, vc, slots)
    torch.cuda.synchronize()
    assert bool((guard[0] == 7).all()) and bool((guard[nb + 1] == 7).all())                  # nothing outside the pool was written
    written = {0, 1, 5, 47, 46}
    flat = kc.permute(0, 2, 1, 3).reshape(nb * 16, Hkv, D)
    for s in range(nb * 16):
        assert bool((flat[s] == 7).all()) != (s in written)
    # positions outside the table behave like the nearest valid one
    pos_ok = torch.tensor([0, 1, 2, 3, 31, 31, 31, 0], dtype=torch.int32).cuda()
    assert torch.equal(q_rot, ops.rope_and_cache(q, k, v, pos_ok, fcg))


@pytest.mark.parametrize("D", [32, 64, 128])
def test_quantize_kv_fp8_is_bit_exact(ops, D):
    print(f"case: quantize D={D}", flush=True)
    cache = rnd(40, 3, 16, D, seed=7, scale=1.7)
    cache[11] = 0
    q8_ref, sc_ref = orc.quantize_kv_fp8(cache)
    q8, sc = ops.quantize_kv_cache_fp8(cache.cuda())
    torch.cuda.synchronize()
    assert torch.equal(sc.cpu(), sc_ref)
    assert torch.equal(q8.cpu(), q8_ref)
    out8, outs = torch.zeros_like(q8), torch.zeros_like(sc)
    ops.quantize_kv_cache_fp8(cache.cuda(), out=(out8, outs))
    torch.cuda.synchronize()
    assert torch.equal(out8, q8) and torch.equal(outs, sc)


def test_decode_loop_over_growing_cache_equals_causal_prefill(ops):
    """RoPE + cache write + paged decode, token by token, against one causal prefill of the same sequence."""
    print("case: decode loop", flush=True)
    S, Hq, Hkv, D, ctx = 70, 8, 2, 64, 128
    q, k, v = rnd(S, Hq, D, seed=8, scale=0.7), rnd(S, Hkv, D, seed=9, scale=0.7), rnd(S, Hkv, D, seed=10, scale=0.7)
    fc = orc.build_rope_cache(ctx, D)
    pos = torch.arange(S, dtype=torch.int32)
    # dense oracle on the rotated tensors
    q_rot = orc.rope_reference(q.float().transpose(0, 1), pos.long(), fc).to(torch.bfloat16)     # (Hq,S,D)
    k_rot = orc.rope_reference(k.float().transpose(0, 1), pos.long(), fc).to(torch.bfloat16)
    ref = orc.prefill_reference(q_rot[None], k_rot[None], v.transpose(0, 1)[None], causal=True)[0]   # (Hq,S,D)

    n_blocks = (S + 15) // 16
    table = torch.tensor([[3, 0, 6, 1, 5]], dtype=torch.int32)[:, :n_blocks]
    kc = torch.zeros(8, Hkv, 16, D, dtype=torch.bfloat16, device="cuda")
    vc = torch.zeros_like(kc)
    fcg = ops.build_rope_cache(ctx, D)
    outs = []
    for t in range(S):
        slot = torch.tensor([int(table[0, t // 16]) * 16 + t % 16], dtype=torch.int64, device="cuda")
        qt = ops.rope_and_cache(q[t:t + 1].cuda(), k[t:t + 1].cuda(), v[t:t + 1].cuda(), pos[t:t + 1].cuda(), fcg,
                                kc, vc, slot)
        o = ops.paged_attention_decode(qt, kc, vc, table.cuda(), torch.tensor([t + 1], dtype=torch.int32, device="cuda"))
        outs.append(o[0])
    got = torch.stack(outs, dim=1).float().cpu()                      # (Hq,S,D)
    err = (got - ref).abs()
    assert bool((err <= 2e-2 + 1e-2 * ref.abs()).all()), float(err.max())
    # and the fused prefill kernel on the same rotated tensors agrees as well
    pre = ops.flash_attn_prefill(q_rot[None].cuda(), k_rot[None].cuda(), v.transpose(0, 1)[None].cuda(), causal=True)[0]
    err = (pre.float().cpu() - ref).abs()
    assert bool((err <= 2e-2 + 1e-2 * ref.abs()).all()), float(err.max())
