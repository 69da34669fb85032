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


@pytest.mark.parametrize("D,fp8", [(128, False), (64, False), (6, False), (128, True)])
def test_rope_and_cache_also_returns_the_packed_rotated_keys(ops, D, fp8):
    """k_out: the same launch that fills the cache hands back the rotated keys in packed form; they equal the
    rows a separate rotation gives and (bf16 cache) the rows the cache received.  D = 6 takes the pair kernel."""
    print(f"case: rope_and_cache k_out D={D} fp8={fp8}", flush=True)
    T, Hq, Hkv, ctx = 50, 6, 2, 64
    q, k, v = rnd(T, Hq, D, seed=1).cuda(), rnd(T, Hkv, D, seed=2).cuda(), rnd(T, Hkv, D, seed=3).cuda()
    fcg = ops.build_rope_cache(ctx, D)
    pos = torch.arange(T, dtype=torch.int32).cuda()
    slots = (torch.arange(T, dtype=torch.int64) + 32).cuda()
    k_plain = ops.rope_and_cache(k, k, v, pos, fcg)                     # queries-only call: rotates its first argument
    q_plain = ops.rope_and_cache(q, k, v, pos, fcg)
    if fp8:
        k8 = torch.zeros(8, Hkv, 16, D, dtype=torch.uint8, device="cuda")
        v8 = torch.zeros_like(k8)
        ks, vs = torch.ones(8, Hkv, device="cuda"), torch.ones(8, Hkv, device="cuda")
        k8b, v8b, ksb, vsb = k8.clone(), v8.clone(), ks.clone(), vs.clone()
        q_rot, k_rot = ops.rope_and_cache_fp8(q, k, v, pos, fcg, k8, v8, ks, vs, slots, k_out=True)
        ops.rope_and_cache_fp8(q, k, v, pos, fcg, k8b, v8b, ksb, vsb, slots)
        assert torch.equal(k8, k8b) and torch.equal(v8, v8b) and torch.equal(ks, ksb) and torch.equal(vs, vsb)
    else:
        kc = torch.zeros(8, Hkv, 16, D, dtype=torch.bfloat16, device="cuda")
        vc = torch.zeros_like(kc)
        q_rot, k_rot = ops.rope_and_cache(q, k, v, pos, fcg, kc, vc, slots, k_out=True)
        rows = kc.permute(0, 2, 1, 3).reshape(-1, Hkv, D)[32:32 + T]
        assert torch.equal(rows, k_rot)
        # without a cache: rotated q and k from one launch
        q2, k2 = ops.rope_and_cache(q, k, v, pos, fcg, k_out=True)
        assert torch.equal(q2, q_plain) and torch.equal(k2, k_plain)
        # into a caller's tensor
        if D % 8 == 0:
            buf = torch.empty(T, Hkv, D, dtype=torch.bfloat16, device="cuda")
            _, k3 = ops.rope_and_cache(q, k, v, pos, fcg, k_out=buf)
            assert k3 is buf and torch.equal(buf, k_plain)
    assert torch.equal(q_rot, q_plain) and torch.equal(k_rot, k_plain)


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


def _ragged_prefill_case(lens, nb, seed):
    """Packed tokens of sequences with `lens` tokens, blocks dealt from a seeded permutation of the pool."""
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(nb, generator=g).tolist()
    slots, positions, tables = [], [], []
    for n in lens:
        blocks = [perm.pop() for _ in range((n + 15) // 16)]
        tables.append(blocks)
        slots += [blocks[t // 16] * 16 + t % 16 for t in range(n)]
        positions += list(range(n))
    return torch.tensor(slots, dtype=torch.int64), torch.tensor(positions, dtype=torch.int32), tables


@pytest.mark.parametrize("D", [32, 64, 128])
def test_rope_and_cache_fp8_prefill_then_decode_is_bit_exact_with_the_oracle(ops, D):
    """A packed prefill (ragged runs, random blocks) and then single-token appends.  Values are copied, and
    keys at position 0 rotate by the identity, so with all positions 0 both caches must equal the oracle's
    bit for bit (scales included)."""
    print(f"case: rope_and_cache_fp8 bit-exact D={D}", flush=True)
    Hq, Hkv, ctx, nb = 4, 2, 64, 12
    lens = [37, 1, 16, 5]
    slots, _, tables = _ragged_prefill_case(lens, nb, seed=40 + D)
    T = sum(lens)
    pos0 = torch.zeros(T, dtype=torch.int32)
    q, k, v = rnd(T, Hq, D, seed=41), rnd(T, Hkv, D, seed=42, scale=1.5), rnd(T, Hkv, D, seed=43, scale=0.8)
    g = torch.Generator().manual_seed(44)
    k8 = torch.randint(0, 255, (nb, Hkv, 16, D), generator=g).to(torch.uint8)       # a dirty pool: stale bytes and scales
    v8 = torch.randint(0, 255, (nb, Hkv, 16, D), generator=g).to(torch.uint8)
    ks, vs = torch.rand(nb, Hkv, generator=g) + 0.1, torch.rand(nb, Hkv, generator=g) + 0.1
    fc = orc.build_rope_cache(ctx, D)
    fcg = ops.build_rope_cache(ctx, D)
    q_ref, k8r, ksr, v8r, vsr = orc.rope_and_cache_fp8_reference(q, k, v, pos0, fc, k8, ks, v8, vs, slots)
    k8g, v8g, ksg, vsg = k8.cuda(), v8.cuda(), ks.cuda(), vs.cuda()
    q_rot = ops.rope_and_cache_fp8(q.cuda(), k.cuda(), v.cuda(), pos0.cuda(), fcg, k8g, v8g, ksg, vsg, slots.cuda())
    torch.cuda.synchronize()
    assert torch.equal(q_rot.cpu(), q)
    assert torch.equal(ksg.cpu(), ksr) and torch.equal(vsg.cpu(), vsr)
    assert torch.equal(k8g.cpu(), k8r) and torch.equal(v8g.cpu(), v8r)
    # decode steps: one token per sequence, growing amplitudes so that scales rise and rows are re-expressed
    cur = list(lens)
    for step in range(20):
        slots_d, live = [], []
        for i, blocks in enumerate(tables):
            if cur[i] % 16 == 0:
                if len(blocks) * 16 == cur[i]:
                    free = sorted(set(range(nb)) - {b for tb in tables for b in tb})
                    if not free:
                        continue
                    blocks.append(free[0])
            slots_d.append(blocks[cur[i] // 16] * 16 + cur[i] % 16)
            live.append(i)
            cur[i] += 1
        B = len(live)
        amp = 0.5 + 0.25 * step
        qd, kd, vd = rnd(B, Hq, D, seed=100 + step), rnd(B, Hkv, D, seed=200 + step, scale=amp), rnd(B, Hkv, D, seed=300 + step, scale=amp)
        sd = torch.tensor(slots_d, dtype=torch.int64)
        pd = torch.zeros(B, dtype=torch.int32)
        _, k8r, ksr, v8r, vsr = orc.rope_and_cache_fp8_reference(qd, kd, vd, pd, fc, k8r, ksr, v8r, vsr, sd)
        ops.rope_and_cache_fp8(qd.cuda(), kd.cuda(), vd.cuda(), pd.cuda(), fcg, k8g, v8g, ksg, vsg, sd.cuda())
        torch.cuda.synchronize()
        assert torch.equal(ksg.cpu(), ksr) and torch.equal(vsg.cpu(), vsr), step
        assert torch.equal(k8g.cpu(), k8r) and torch.equal(v8g.cpu(), v8r), step


def test_rope_and_cache_fp8_long_prefill_windows_are_bit_exact(ops):
    """4096 tokens and more take the 16-token-window path; ragged lengths put run starts anywhere inside
    the windows, and a second call appends mid-block chunks after them."""
    print("case: rope_and_cache_fp8 long packed prefill", flush=True)
    Hq, Hkv, D, ctx = 2, 2, 64, 4096
    lens = [3001, 1000, 137, 7]
    nb = sum((n + 15) // 16 for n in lens) + 300
    slots, _, tables = _ragged_prefill_case(lens, nb, seed=45)
    T = sum(lens)
    pos0 = torch.zeros(T, dtype=torch.int32)
    q, k, v = rnd(T, Hq, D, seed=46), rnd(T, Hkv, D, seed=47, scale=1.5), rnd(T, Hkv, D, seed=48, scale=0.8)
    g = torch.Generator().manual_seed(49)
    k8 = torch.randint(0, 255, (nb, Hkv, 16, D), generator=g).to(torch.uint8)
    v8 = torch.randint(0, 255, (nb, Hkv, 16, D), generator=g).to(torch.uint8)
    ks, vs = torch.rand(nb, Hkv, generator=g) + 0.1, torch.rand(nb, Hkv, generator=g) + 0.1
    fc, fcg = orc.build_rope_cache(ctx, D), ops.build_rope_cache(ctx, D)
    _, k8r, ksr, v8r, vsr = orc.rope_and_cache_fp8_reference(q, k, v, pos0, fc, k8, ks, v8, vs, slots)
    k8g, v8g, ksg, vsg = k8.cuda(), v8.cuda(), ks.cuda(), vs.cuda()
    ops.rope_and_cache_fp8(q.cuda(), k.cuda(), v.cuda(), pos0.cuda(), fcg, k8g, v8g, ksg, vsg, slots.cuda())
    torch.cuda.synchronize()
    assert torch.equal(ksg.cpu(), ksr) and torch.equal(vsg.cpu(), vsr)
    assert torch.equal(k8g.cpu(), k8r) and torch.equal(v8g.cpu(), v8r)
    # a chunk of 1100 more tokens per sequence, louder, starting mid-block: the old rows of the first block are re-expressed
    used = {b for tb in tables for b in tb}
    free = [b for b in range(nb) if b not in used]
    more, slots2 = 1100, []
    for i, n in enumerate(lens):
        for t in range(n, n + more):
            if t // 16 >= len(tables[i]):
                tables[i].append(free.pop())
            slots2.append(tables[i][t // 16] * 16 + t % 16)
    T2 = more * len(lens)
    q2, k2, v2 = rnd(T2, Hq, D, seed=56), rnd(T2, Hkv, D, seed=57, scale=3.0), rnd(T2, Hkv, D, seed=58, scale=2.0)
    s2, p2 = torch.tensor(slots2, dtype=torch.int64), torch.zeros(T2, dtype=torch.int32)
    _, k8r, ksr, v8r, vsr = orc.rope_and_cache_fp8_reference(q2, k2, v2, p2, fc, k8r, ksr, v8r, vsr, s2)
    ops.rope_and_cache_fp8(q2.cuda(), k2.cuda(), v2.cuda(), p2.cuda(), fcg, k8g, v8g, ksg, vsg, s2.cuda())
    torch.cuda.synchronize()
    assert torch.equal(ksg.cpu(), ksr) and torch.equal(vsg.cpu(), vsr)
    assert torch.equal(k8g.cpu(), k8r) and torch.equal(v8g.cpu(), v8r)


def test_rope_and_cache_fp8_with_rotation_matches_the_oracle_within_one_rounding(ops):
    """Real positions: the kernel's rotation may differ from the oracle's by one bf16 ulp before
    quantisation, so compare dequantised keys: equal scales up to that ulp, values within one e4m3 step."""
    print("case: rope_and_cache_fp8 rotation", flush=True)
    Hq, Hkv, D, ctx, nb = 8, 2, 128, 256, 16
    lens = [100, 33, 64]
    slots, pos, _ = _ragged_prefill_case(lens, nb, seed=50)
    T = sum(lens)
    q, k, v = rnd(T, Hq, D, seed=51), rnd(T, Hkv, D, seed=52), rnd(T, Hkv, D, seed=53)
    fc, fcg = orc.build_rope_cache(ctx, D), ops.build_rope_cache(ctx, D)
    z8, ones = torch.zeros(nb, Hkv, 16, D, dtype=torch.uint8), torch.ones(nb, Hkv)
    q_ref, k8r, ksr, v8r, vsr = orc.rope_and_cache_fp8_reference(q, k, v, pos, fc, z8, ones, z8, ones, slots)
    k8g, v8g, ksg, vsg = z8.cuda(), z8.cuda(), ones.cuda(), ones.cuda()
    q_rot = ops.rope_and_cache_fp8(q.cuda(), k.cuda(), v.cuda(), pos.cuda(), fcg, k8g, v8g, ksg, vsg, slots.cuda())
    torch.cuda.synchronize()
    torch.testing.assert_close(q_rot.float().cpu(), q_ref, atol=2 ** -7, rtol=2 ** -7)
    assert torch.equal(v8g.cpu(), v8r) and torch.equal(vsg.cpu(), vsr)              # values: no rotation, exact
    torch.testing.assert_close(ksg.cpu(), ksr, atol=0, rtol=2 ** -7)
    got, ref = orc.dequantize_kv_fp8(k8g.cpu(), ksg.cpu()), orc.dequantize_kv_fp8(k8r, ksr)
    assert bool(((got - ref).abs() <= 2 ** -3 * ref.abs() + ksr[:, :, None, None] * 2 ** -8).all())
    assert float((k8g.cpu() != k8r).float().mean()) < 0.02                            # and almost all bytes agree


def test_rope_and_cache_fp8_skips_bad_slots_and_rejects_bad_arguments(ops):
    print("case: rope_and_cache_fp8 bad slots / arguments", flush=True)
    T, Hq, Hkv, D, ctx, nb = 6, 2, 2, 64, 32, 3
    q, k, v = rnd(T, Hq, D, seed=61).cuda(), rnd(T, Hkv, D, seed=62).cuda(), rnd(T, Hkv, D, seed=63).cuda()
    fcg = ops.build_rope_cache(ctx, D)
    pos = torch.tensor([0, 1, 2, 3, 40, -2], dtype=torch.int32).cuda()
    slots = torch.tensor([16, 17, nb * 16, -1, 2 ** 40, 5], dtype=torch.int64).cuda()
    guard = torch.full((nb + 2, Hkv, 16, D), 9, dtype=torch.uint8, device="cuda")
    k8, v8 = guard[1:nb + 1], guard.clone()[1:nb + 1]
    sguard = torch.full((nb + 2, Hkv), 3.0, device="cuda")
    ks, vs = sguard[1:nb + 1], sguard.clone()[1:nb + 1]
    ops.rope_and_cache_fp8(q, k, v, pos, fcg, k8, v8, ks, vs, slots)
    torch.cuda.synchronize()
    assert bool((guard[0] == 9).all()) and bool((guard[nb + 1] == 9).all())
    assert bool((sguard[0] == 3).all()) and bool((sguard[nb + 1] == 3).all())
    flat = k8.permute(0, 2, 1, 3).reshape(nb * 16, Hkv, D)
    for s in range(nb * 16):
        assert bool((flat[s] == 9).all()) != (s in {16, 17, 5})
    assert bool((ks[2] == 3).all())                                                    # block 2 received nothing
    with pytest.raises(ValueError):
        ops.rope_and_cache_fp8(q, k, v, pos, fcg, k8, v8, ks[:2], vs, slots)           # scale shape
    with pytest.raises(ValueError):
        ops.rope_and_cache_fp8(q, k, v, pos, fcg, k8.to(torch.bfloat16), v8, ks, vs, slots)
    with pytest.raises(TypeError):
        ops.rope_and_cache_fp8(q, k, v, pos, fcg, k8, v8, ks, vs, slots.to(torch.int32))


def test_fp8_engine_decode_loop_tracks_the_bf16_oracle(ops):
    """PagedAttentionEngine with an fp8 cache: prefill + 40 decode steps of two sequences; every decode
    output within the fp8 bound of the fp32 oracle on the unquantised keys and values."""
    print("case: fp8 engine decode loop", flush=True)
    Hq, Hkv, D, ctx = 8, 2, 128, 256
    eng = ops.PagedAttentionEngine(24, Hq, Hkv, D, ctx, max_batch=4, kv_dtype="fp8")
    lens = [50, 23]
    steps = 40
    total = [n + steps for n in lens]
    qs = [rnd(n, Hq, D, seed=70 + i, scale=0.7) for i, n in enumerate(total)]
    ks = [rnd(n, Hkv, D, seed=80 + i, scale=0.7) for i, n in enumerate(total)]
    vs = [rnd(n, Hkv, D, seed=90 + i, scale=0.7) for i, n in enumerate(total)]
    fc = orc.build_rope_cache(ctx, D)
    refs = []
    for i, n in enumerate(total):
        p = torch.arange(n)
        qr = orc.rope_reference(qs[i].float().transpose(0, 1), p, fc).to(torch.bfloat16)
        kr = orc.rope_reference(ks[i].float().transpose(0, 1), p, fc).to(torch.bfloat16)
        refs.append(orc.prefill_reference(qr[None], kr[None], vs[i].transpose(0, 1)[None], causal=True)[0])   # (Hq,n,D)
    for i in range(2):
        eng.add_sequence(i)
    cat = lambda xs: torch.cat([x[:n] for x, n in zip(xs, lens)]).cuda()
    out = eng.prefill([0, 1], lens, cat(qs), cat(ks), cat(vs))
    torch.cuda.synchronize()
    ref = torch.cat([r[:, :n].transpose(0, 1) for r, n in zip(refs, lens)])
    err = (out.float().cpu() - ref).abs()
    assert bool((err <= 2e-2 + 1e-2 * ref.abs()).all())                                # prefill attends the bf16 tensors
    worst = 0.0
    for s in range(steps):
        row = lambda xs: torch.stack([x[n + s] for x, n in zip(xs, lens)]).cuda()
        o = eng.decode_step([0, 1], row(qs), row(ks), row(vs)).float().cpu()
        r = torch.stack([refs[i][:, lens[i] + s] for i in range(2)])
        err = (o - r).abs()
        worst = max(worst, float(err.max()))
        assert bool((err <= 0.15 + 2 ** -4 * r.abs()).all()), (s, float(err.max()))
    print(f"fp8 engine decode: worst abs err {worst:.4f}", flush=True)
