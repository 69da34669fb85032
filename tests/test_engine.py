"""Continuous-batching attention engine: block allocator on the CPU, and on the GPU a schedule in
which sequences join and leave between decode steps; every output row must equal dense causal
attention over that sequence's own (rotated) history."""
import pytest
import torch

from oracle import attention_oracle as orc


def test_block_allocator_reuses_freed_blocks():
    from mi355_attn.engine import BlockAllocator, OutOfBlocks
    a = BlockAllocator(3)
    got = [a.allocate() for _ in range(3)]
    assert sorted(got) == [0, 1, 2] and a.num_free == 0
    with pytest.raises(OutOfBlocks):
        a.allocate()
    a.free([got[1]])
    assert a.allocate() == got[1]


def rnd(*shape, seed, scale=0.7):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


@pytest.mark.gpu
def test_continuous_batching_matches_dense_causal_attention():
    import mi355_attn
    print("case: engine continuous batching", flush=True)
    Hq, Hkv, D, ctx = 8, 2, 128, 256
    eng = mi355_attn.PagedAttentionEngine(num_blocks=40, n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D,
                                          context_length=ctx, max_batch=8)
    fc = orc.build_rope_cache(ctx, D)
    # full token streams of 4 sequences (prompt + generated), seeded
    total = {0: 50, 1: 33, 2: 70, 3: 21}
    prompt = {0: 17, 1: 16, 2: 40, 3: 1}
    streams = {s: (rnd(n, Hq, D, seed=10 * s + 1), rnd(n, Hkv, D, seed=10 * s + 2), rnd(n, Hkv, D, seed=10 * s + 3))
               for s, n in total.items()}
    got = {s: torch.zeros(total[s], Hq, D) for s in total}

    def admit(sids):
        lens = [prompt[s] for s in sids]
        for s in sids:
            eng.add_sequence(s)
        q = torch.cat([streams[s][0][:prompt[s]] for s in sids]).cuda()
        k = torch.cat([streams[s][1][:prompt[s]] for s in sids]).cuda()
        v = torch.cat([streams[s][2][:prompt[s]] for s in sids]).cuda()
        out = eng.prefill(sids, lens, q, k, v).float().cpu()
        off = 0
        for s, n in zip(sids, lens):
            got[s][:n] = out[off:off + n]
            off += n

    admit([0, 1])
    running = [0, 1]
    step = 0
    while running:
        if step == 3:
            admit([2])
            running.append(2)
        if step == 10:
            admit([3])
            running.append(3)
        pos = {s: eng.lengths[s] for s in running}
        q = torch.stack([streams[s][0][pos[s]] for s in running]).cuda()
        k = torch.stack([streams[s][1][pos[s]] for s in running]).cuda()
        v = torch.stack([streams[s][2][pos[s]] for s in running]).cuda()
        out = eng.decode_step(running, q, k, v).float().cpu()
        for i, s in enumerate(running):
            got[s][pos[s]] = out[i]
        for s in list(running):
            if eng.lengths[s] == total[s]:
                eng.remove_sequence(s)                 # its blocks go back to the pool and are reused
                running.remove(s)
        step += 1
    assert eng.allocator.num_free == 40

    for s, n in total.items():
        q, k, v = streams[s]
        p = torch.arange(n)
        q_rot = orc.rope_reference(q.float().transpose(0, 1), p, fc).to(torch.bfloat16)
        k_rot = orc.rope_reference(k.float().transpose(0, 1), p, fc).to(torch.bfloat16)
        ref = orc.prefill_reference(q_rot[None], k_rot[None], v.transpose(0, 1)[None], causal=True)[0].transpose(0, 1)
        err = (got[s] - ref).abs()
        assert bool((err <= 2e-2 + 1e-2 * ref.abs()).all()), (s, float(err.max()))


@pytest.mark.gpu
@pytest.mark.parametrize("ctx_len", [2048, 4096])
def test_decode_with_full_batch_at_long_context_lengths(ctx_len):
    """The engine sizes its split-K workspace once, for (max_batch, context_length).  The kernel's chunk size
    changes with the longest context of a step (2048 and 4096 tokens are the thresholds), so steps at shorter
    lengths use MORE chunks per sequence than the sizing call: every such step must still fit the workspace."""
    import mi355_attn
    print(f"case: engine full batch at context_length {ctx_len}", flush=True)
    Hq, Hkv, D, B = 8, 2, 64, 6
    eng = mi355_attn.PagedAttentionEngine(num_blocks=B * ctx_len // 16, n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D,
                                          context_length=ctx_len, max_batch=B)
    fc = orc.build_rope_cache(ctx_len, D)
    lens = [ctx_len - 1 - 16 * i for i in range(B)]
    lens[-1] = 1500                                      # and one sequence between the thresholds' chunk sizes
    qs = [rnd(n + 1, Hq, D, seed=70 + i) for i, n in enumerate(lens)]
    ks = [rnd(n + 1, Hkv, D, seed=80 + i) for i, n in enumerate(lens)]
    vs = [rnd(n + 1, Hkv, D, seed=90 + i) for i, n in enumerate(lens)]
    sids = list(range(B))
    for s in sids:
        eng.add_sequence(s)
    eng.prefill(sids, lens, torch.cat([q[:-1] for q in qs]).cuda(), torch.cat([k[:-1] for k in ks]).cuda(),
                torch.cat([v[:-1] for v in vs]).cuda())
    out = eng.decode_step(sids, torch.stack([q[-1] for q in qs]).cuda(), torch.stack([k[-1] for k in ks]).cuda(),
                          torch.stack([v[-1] for v in vs]).cuda()).float().cpu()
    # a second step at a much shorter longest context (other chunk regime) reuses the same workspace
    for s in sids[:-1]:
        eng.remove_sequence(s)
    q2, k2, v2 = rnd(1, Hq, D, seed=101), rnd(1, Hkv, D, seed=102), rnd(1, Hkv, D, seed=103)
    out2 = eng.decode_step([sids[-1]], q2.cuda(), k2.cuda(), v2.cuda()).float().cpu()
    torch.cuda.synchronize()
    for i, n in enumerate(lens):
        p = torch.arange(n + 1)
        q_rot = orc.rope_reference(qs[i][-1:].float().transpose(0, 1), p[-1:], fc).to(torch.bfloat16)
        k_rot = orc.rope_reference(ks[i].float().transpose(0, 1), p, fc).to(torch.bfloat16)
        ref = orc.prefill_reference(q_rot[None], k_rot[None], vs[i].transpose(0, 1)[None], causal=True)[0, :, 0]
        err = (out[i] - ref).abs()
        assert bool((err <= 2e-2 + 1e-2 * ref.abs()).all()), (i, float(err.max()))
    i, n = B - 1, lens[-1] + 2
    p = torch.arange(n)
    k_all, v_all = torch.cat([ks[i], k2]), torch.cat([vs[i], v2])
    q_rot = orc.rope_reference(q2.float().transpose(0, 1), p[-1:], fc).to(torch.bfloat16)
    k_rot = orc.rope_reference(k_all.float().transpose(0, 1), p, fc).to(torch.bfloat16)
    ref = orc.prefill_reference(q_rot[None], k_rot[None], v_all.transpose(0, 1)[None], causal=True)[0, :, 0]
    err = (out2[0] - ref).abs()
    assert bool((err <= 2e-2 + 1e-2 * ref.abs()).all()), float(err.max())


@pytest.mark.gpu
@pytest.mark.parametrize("D", [128, 64])
def test_prompt_admitted_in_three_chunks_equals_one_shot_prefill(D):
    """A prompt fed through plan_prefill in three ragged chunks (the second and third on top of cached
    tokens, read back through the block tables) must give the attention rows of a one-shot prefill of
    the same prompt: both within the bf16 tolerance of the oracle, and close to each other."""
    import mi355_attn
    print(f"case: engine chunked prefill D={D}", flush=True)
    Hq, Hkv, ctx = 8, 2, 1024
    fc = orc.build_rope_cache(ctx, D)
    n = 700
    q, k, v = rnd(n, Hq, D, seed=31), rnd(n, Hkv, D, seed=32), rnd(n, Hkv, D, seed=33)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()

    one = mi355_attn.PagedAttentionEngine(num_blocks=64, n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D,
                                          context_length=ctx, max_batch=4)
    one.add_sequence(0)
    whole = one.prefill([0], [n], qg, kg, vg).float().cpu()

    eng = mi355_attn.PagedAttentionEngine(num_blocks=64, n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D,
                                          context_length=ctx, max_batch=4)
    eng.add_sequence(7)
    eng.add_sequence(8)                  # a second, new sequence rides along with the last chunk
    cuts = [0, 203, 460, n]              # ragged: none of the boundaries is a multiple of 16 or 64
    parts = []
    for c0, c1 in zip(cuts[:-1], cuts[1:]):
        if c1 == n:
            q2, k2, v2 = rnd(90, Hq, D, seed=41), rnd(90, Hkv, D, seed=42), rnd(90, Hkv, D, seed=43)
            out = eng.prefill([7, 8], [c1 - c0, 90], torch.cat([qg[c0:c1], q2.cuda()]),
                              torch.cat([kg[c0:c1], k2.cuda()]), torch.cat([vg[c0:c1], v2.cuda()])).float().cpu()
            parts.append(out[:c1 - c0])
            other = out[c1 - c0:]
        else:
            parts.append(eng.prefill([7], [c1 - c0], qg[c0:c1], kg[c0:c1], vg[c0:c1]).float().cpu())
    chunked = torch.cat(parts)
    assert eng.lengths[7] == n and eng.lengths[8] == 90
    # the caches hold the same rows either way
    blocks = one.blocks[0]
    assert torch.equal(one.k_cache[blocks], eng.k_cache[eng.blocks[7]])
    assert torch.equal(one.v_cache[blocks], eng.v_cache[eng.blocks[7]])

    def oracle(qq, kk, vv):
        p = torch.arange(qq.shape[0])
        q_rot = orc.rope_reference(qq.float().transpose(0, 1), p, fc).to(torch.bfloat16)
        k_rot = orc.rope_reference(kk.float().transpose(0, 1), p, fc).to(torch.bfloat16)
        return orc.prefill_reference(q_rot[None], k_rot[None], vv.transpose(0, 1)[None], causal=True)[0].transpose(0, 1)

    ref = oracle(q, k, v)
    for name, got in (("one-shot", whole), ("chunked", chunked)):
        err = (got - ref).abs()
        assert bool((err <= 2e-2 + 1e-2 * ref.abs()).all()), (name, float(err.max()))
    assert float((chunked - whole).abs().max()) <= 2e-2
    ref2 = oracle(q2, k2, v2)
    err = (other - ref2).abs()
    assert bool((err <= 2e-2 + 1e-2 * ref2.abs()).all()), float(err.max())
    # decoding continues from the chunked cache
    qd, kd, vd = rnd(1, Hq, D, seed=51), rnd(1, Hkv, D, seed=52), rnd(1, Hkv, D, seed=53)
    step = eng.decode_step([7], qd.cuda(), kd.cuda(), vd.cuda()).float().cpu()
    full = oracle(torch.cat([q, qd]), torch.cat([k, kd]), torch.cat([v, vd]))[-1:]
    err = (step - full).abs()
    assert bool((err <= 2e-2 + 1e-2 * full.abs()).all()), float(err.max())


@pytest.mark.gpu
def test_prompt_admitted_in_three_chunks_on_an_fp8_cache():
    """Chunked prefill over an fp8 cache: every chunk attends to the QUANTISED keys and values of everything cached so
    far, its own rows included (as the later decode steps will).  Each chunk's rows are checked against the oracle on
    the dequantised cache as it stands after that chunk (bf16 tolerance: kernel parity), and the whole prompt against
    a one-shot prefill on a bf16 cache within the fp8 bound |err| <= 0.15 + 2^-4 |ref|, relative rms <= 6 %."""
    import mi355_attn
    print("case: engine chunked prefill on an fp8 cache", flush=True)
    Hq, Hkv, D, ctx, n = 8, 2, 128, 1024, 700
    fc = orc.build_rope_cache(ctx, D)
    q, k, v = rnd(n, Hq, D, seed=31), rnd(n, Hkv, D, seed=32), rnd(n, Hkv, D, seed=33)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    one = mi355_attn.PagedAttentionEngine(num_blocks=64, n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, context_length=ctx, max_batch=4)
    one.add_sequence(0)
    whole = one.prefill([0], [n], qg, kg, vg).float().cpu()
    eng = mi355_attn.PagedAttentionEngine(num_blocks=64, n_q_heads=Hq, n_kv_heads=Hkv, head_dim=D, context_length=ctx, max_batch=4,
                                          kv_dtype="fp8")
    eng.add_sequence(7)
    cuts = [0, 203, 460, n]
    parts = []
    for c0, c1 in zip(cuts[:-1], cuts[1:]):
        got = eng.prefill([7], [c1 - c0], qg[c0:c1], kg[c0:c1], vg[c0:c1]).float().cpu()
        parts.append(got)
        if c0 == 0:
            continue                                  # the first chunk attends to its own unquantised keys (packed prefill)
        k8, v8 = eng.k_caches[0].cpu(), eng.v_caches[0].cpu()
        ks, vs = eng.k_scales[0].cpu(), eng.v_scales[0].cpu()
        table = torch.tensor([eng.blocks[7]], dtype=torch.int32)
        q_rot = orc.rope_reference(q[c0:c1].float().transpose(0, 1), torch.arange(c0, c1), fc).to(torch.bfloat16).transpose(0, 1)
        ref = orc.paged_prefill_reference(q_rot, orc.dequantize_kv_fp8(k8.view(torch.uint8), ks),
                                          orc.dequantize_kv_fp8(v8.view(torch.uint8), vs),
                                          torch.tensor([0, c1 - c0], dtype=torch.int32), table, torch.tensor([c1], dtype=torch.int32))
        err = (got - ref).abs()
        assert bool((err <= 2e-2 + 1e-2 * ref.abs()).all()), (c0, float(err.max()))
    chunked = torch.cat(parts)
    assert eng.lengths[7] == n
    e = (chunked - whole).abs()
    assert bool((e <= 0.15 + 2.0 ** -4 * whole.abs()).all()), float(e.max())
    assert float((chunked - whole).pow(2).mean().sqrt() / whole.pow(2).mean().sqrt()) <= 0.06
    # decoding continues from the chunked fp8 cache
    qd, kd, vd = rnd(1, Hq, D, seed=51), rnd(1, Hkv, D, seed=52), rnd(1, Hkv, D, seed=53)
    step = eng.decode_step([7], qd.cuda(), kd.cuda(), vd.cuda()).float().cpu()
    assert bool(torch.isfinite(step).all())
