"""The benchmark configurations at their full stated shapes (configs[2], [3], [4]).

The CPU oracle cannot cover these shapes whole in test time, so each case combines
  * the oracle on a sample that it finishes in seconds (whole sequences of the decode batches, whole
    heads of the prefill), and
  * properties that do not depend on size and involve every output element:
    decode   - the result does not depend on where the blocks live: after moving every block to a
               new physical position (and rewriting the tables) the output is identical bit for bit;
               a sequence served alone equals its row of the batch; outputs lie inside the range of
               the values attended;
    prefill  - causality: the rows of a prefix of every sequence are reproduced (bit for bit when the
               prefix is a whole number of query tiles) when the kernel is given only that prefix;
               constant values come back as that constant; a first token returns its own value row;
    backward - linearity in dO for a power-of-two factor (exact), plus the oracle's gradients on all
               query heads of one (sequence, kv head) group.
Tolerance where the oracle is involved: |got - ref| <= 2e-2 + 1e-2 |ref| (bf16 paths); fp8 KV is
checked against the oracle on the dequantised cache with the same bound (kernel parity) and, as configs[4]
defines its error, against fp32 math on the bf16 cache it was quantised from: |got - ref| <= 0.15 + 2^-4 |ref|
per element and rms(got - ref) <= 6 % of rms(ref) (e4m3 rounds with relative error <= 2^-4).
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


def _close(got, ref, atol=2e-2, rtol=1e-2):
    err = (got.float().cpu() - ref).abs()
    assert bool((err <= atol + rtol * ref.abs()).all()), f"max err {float(err.max()):.4f}"


def _oracle_rows(case, rows):
    """Oracle output for the sequences `rows` of a decode case: their blocks are gathered into a small pool."""
    ctx = case.context_lens_host[rows]
    nblk = (ctx + 15) // 16
    ids = torch.cat([case.block_tables[b, :int(n)] for b, n in zip(rows, nblk)]).long()
    kc, vc = case.k_cache[ids].cpu(), case.v_cache[ids].cpu()
    ks = case.k_scale[ids].cpu() if case.k_scale is not None else None
    vs = case.v_scale[ids].cpu() if case.v_scale is not None else None
    bt = torch.zeros(len(rows), int(nblk.max()), dtype=torch.int32)
    off = 0
    for i, n in enumerate(nblk):
        bt[i, :int(n)] = torch.arange(off, off + int(n), dtype=torch.int32)
        off += int(n)
    return orc.paged_decode_reference(case.q[rows].cpu(), kc, vc, bt, ctx, k_scale=ks, v_scale=vs)


def _oracle_rows_bf16(case, rows):
    """Oracle output for the sequences `rows` of an fp8 decode case on the bf16 blocks kept from before quantisation."""
    assert case.bf16_sample_seqs > max(rows)
    nblk_all = (case.context_lens_host + 15) // 16
    start = torch.cat([torch.zeros(1, dtype=torch.int64), nblk_all.long().cumsum(0)])
    ids = torch.cat([torch.arange(int(start[b]), int(start[b + 1])) for b in rows])
    kc, vc = case.k_bf16_sample[ids.cuda()].cpu(), case.v_bf16_sample[ids.cuda()].cpu()
    ctx = case.context_lens_host[rows]
    nblk = nblk_all[rows]
    bt = torch.zeros(len(rows), int(nblk.max()), dtype=torch.int32)
    off = 0
    for i, n in enumerate(nblk):
        bt[i, :int(n)] = torch.arange(off, off + int(n), dtype=torch.int32)
        off += int(n)
    return orc.paged_decode_reference(case.q[rows].cpu(), kc, vc, bt, ctx)


@pytest.mark.parametrize("cfg", [3, 4])
def test_decode_full_size(ops, cfg):
    from mi355_attn import workloads
    print(f"case: decode configs[{cfg}] full size", flush=True)
    case = workloads.decode_config(cfg, seed=0, keep_bf16_seqs=256)
    B = case.q.shape[0]
    scales = {} if case.k_scale is None else {"k_scale": case.k_scale, "v_scale": case.v_scale}
    out = ops.paged_attention_decode(case.q, case.k_cache, case.v_cache, case.block_tables, case.context_lens,
                                     max_context=case.max_context, **scales)
    torch.cuda.synchronize()
    assert out.shape == case.q.shape and bool(torch.isfinite(out.float()).all())

    # oracle on the shortest, the longest and six more sequences
    order = torch.argsort(case.context_lens_host)
    rows = sorted({int(order[0]), int(order[-1]), int(order[B // 2])} | {int(i) for i in order[torch.arange(5, B, B // 6)]})
    _close(out[rows], _oracle_rows(case, rows))
    if cfg == 4:
        # the configuration's own error metric: against a bf16-KV fp32-math reference, at the full shape
        ref16 = _oracle_rows_bf16(case, rows)
        got = out[rows].float().cpu()
        err = (got - ref16).abs()
        assert bool((err <= 0.15 + 2.0 ** -4 * ref16.abs()).all()), f"fp8 vs bf16 KV: max err {float(err.max()):.4f}"
        rms = float((got - ref16).pow(2).mean().sqrt() / ref16.pow(2).mean().sqrt())
        assert rms <= 0.06, f"fp8 vs bf16 KV: rms ratio {rms:.4f}"
        case.k_bf16_sample = case.v_bf16_sample = None

    # every output lies between the smallest and the largest value it can average (per sequence, kv head, dim)
    b = int(order[B // 3])
    n = int((case.context_lens_host[b] + 15) // 16)
    ids = case.block_tables[b, :n].long()
    vals = case.v_cache[ids]
    vals = (vals.view(torch.float8_e4m3fn).float() * case.v_scale[ids][:, :, None, None]) if case.k_scale is not None else vals.float()
    vals = vals.permute(1, 0, 2, 3).reshape(vals.shape[1], n * 16, -1)[:, :int(case.context_lens_host[b])]     # (Hkv, ctx, D)
    G = case.q.shape[1] // vals.shape[0]
    lo = vals.amin(1).repeat_interleave(G, 0)
    hi = vals.amax(1).repeat_interleave(G, 0)
    o = out[b].float()
    assert bool((o >= lo - 2e-2 - 1e-2 * lo.abs()).all()) and bool((o <= hi + 2e-2 + 1e-2 * hi.abs()).all())

    # a sequence alone equals its row in the batch (other chunking: within rounding, not bitwise)
    b = int(order[-1])
    alone = ops.paged_attention_decode(case.q[b:b + 1], case.k_cache, case.v_cache, case.block_tables[b:b + 1],
                                       case.context_lens[b:b + 1], **scales)
    _close(alone, out[b:b + 1].float().cpu(), atol=1e-2, rtol=1e-2)

    # move every block to a new physical position: the output must not change at all
    nb = case.k_cache.shape[0]
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(7)).cuda()        # new position of old block i
    for name in ("k_cache", "v_cache", "k_scale", "v_scale"):
        t = getattr(case, name)
        if t is not None:
            moved = torch.empty_like(t)
            moved[perm] = t
            setattr(case, name, moved)
            del t, moved
    tables = perm[case.block_tables.long()].to(torch.int32)
    scales = {} if case.k_scale is None else {"k_scale": case.k_scale, "v_scale": case.v_scale}
    out2 = ops.paged_attention_decode(case.q, case.k_cache, case.v_cache, tables, case.context_lens,
                                      max_context=case.max_context, **scales)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)


def test_prefill_full_size_is_the_same_on_every_launch(ops):
    """The persistent prefill kernel keeps its own books on what is in flight (query rows, K/V tiles and output rows
    pass through the same LDS, requests of the next query tile are issued while the current one is stored): a wait
    that is one request short shows up as a result that changes from launch to launch.  configs[2] at full size, and
    ragged packed sequences with the log-sum-exp output, twenty launches each, bit for bit."""
    from mi355_attn import workloads
    from mi355_attn import ops as raw
    print("case: prefill configs[2] full size, repeated launches", flush=True)
    case = workloads.prefill_config(2, seed=1)
    S = case.seqlen
    first = ops.flash_attn_varlen_prefill(case.q, case.k, case.v, case.cu_seqlens, case.cu_seqlens, S, S, causal=True)
    for i in range(20):
        again = ops.flash_attn_varlen_prefill(case.q, case.k, case.v, case.cu_seqlens, case.cu_seqlens, S, S, causal=True)
        assert torch.equal(first, again), f"launch {i + 1} differs from the first"
    del first, again
    print("case: ragged packed sequences with lse, repeated launches", flush=True)
    g = torch.Generator().manual_seed(77)
    lens = [int(x) for x in torch.randint(1, 3000, (24,), generator=g)]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32).cuda()
    T = sum(lens)
    gd = torch.Generator(device="cuda").manual_seed(78)
    q = (torch.randn(T, 32, 128, generator=gd, device="cuda") * 0.5).to(torch.bfloat16)
    k = (torch.randn(T, 8, 128, generator=gd, device="cuda") * 0.5).to(torch.bfloat16)
    v = (torch.randn(T, 8, 128, generator=gd, device="cuda") * 0.5).to(torch.bfloat16)
    out0, lse0 = raw._varlen(q, k, v, cu, cu, max(lens), max(lens), True, None, want_lse=True)
    for i in range(20):
        out1, lse1 = raw._varlen(q, k, v, cu, cu, max(lens), max(lens), True, None, want_lse=True)
        assert torch.equal(out0, out1) and torch.equal(lse0, lse1), f"launch {i + 1} differs from the first"
    for splits in (2, 5):
        sp0 = ops.flash_attn_varlen_prefill(q, k, v, cu, cu, max(lens), max(lens), causal=True, kv_splits=splits)
        for i in range(10):
            sp1 = ops.flash_attn_varlen_prefill(q, k, v, cu, cu, max(lens), max(lens), causal=True, kv_splits=splits)
            assert torch.equal(sp0, sp1), f"keys split {splits} ways: launch {i + 1} differs from the first"
        assert (sp0.float() - out0.float()).abs().max().item() <= 2e-2


def test_prefill_and_backward_full_size(ops):
    from mi355_attn import workloads
    print("case: prefill configs[2] full size", flush=True)
    case = workloads.prefill_config(2, seed=0)
    S, B = case.seqlen, case.batch
    Hq, Hkv, D = case.q.shape[1], case.k.shape[1], case.q.shape[2]
    out = ops.flash_attn_varlen_prefill(case.q, case.k, case.v, case.cu_seqlens, case.cu_seqlens, S, S, causal=True)
    torch.cuda.synchronize()
    assert out.shape == case.q.shape and bool(torch.isfinite(out.float()).all())

    # oracle on whole heads: (sequence, query head) samples
    for b, h in ((0, 0), (3, 13), (7, 31)):
        hk = h // (Hq // Hkv)
        rows = slice(b * S, (b + 1) * S)
        q = case.q[rows, h][None, None].cpu()
        k = case.k[rows, hk][None, None].cpu()
        v = case.v[rows, hk][None, None].cpu()
        _close(out[rows, h][None, None], orc.prefill_reference(q, k, v, causal=True))
    # the first token of every sequence attends only itself
    first = torch.arange(B, device="cuda") * S
    assert torch.equal(out[first], case.v[first].repeat_interleave(Hq // Hkv, 1))

    # causality: given only the first n tokens of every sequence, the kernel reproduces those rows - bit for bit
    # when n is a multiple of the 256-query tile (same tiles, same wavefronts), within rounding otherwise
    # (the rescaling decisions of a wavefront then see different neighbour rows)
    for n in (1536, 1500):
        idx = (torch.arange(B, device="cuda")[:, None] * S + torch.arange(n, device="cuda")[None]).reshape(-1)
        cu = (torch.arange(B + 1, dtype=torch.int32) * n).cuda()
        part = ops.flash_attn_varlen_prefill(case.q[idx], case.k[idx], case.v[idx], cu, cu, n, n, causal=True)
        torch.cuda.synchronize()
        if n % 256 == 0:
            assert torch.equal(part, out[idx])
        else:
            _close(part, out[idx].float().cpu(), atol=1e-2, rtol=1e-2)

    # constant values come back unchanged
    vconst = torch.full_like(case.v, 0.375)
    oc = ops.flash_attn_varlen_prefill(case.q, case.k, vconst, case.cu_seqlens, case.cu_seqlens, S, S, causal=True)
    torch.cuda.synchronize()
    assert float((oc.float() - 0.375).abs().max()) <= 2 ** -8
    del oc, vconst, part

    print("case: backward configs[2] full size", flush=True)
    g = torch.Generator(device="cuda").manual_seed(5)
    dout = (torch.randn(case.q.shape, generator=g, device="cuda") * 0.5).to(torch.bfloat16)

    def grads(do):
        q, k, v = (t.detach().clone().requires_grad_() for t in (case.q, case.k, case.v))
        ops.flash_attn_varlen_prefill(q, k, v, case.cu_seqlens, case.cu_seqlens, S, S, causal=True).backward(do)
        torch.cuda.synchronize()
        return q.grad, k.grad, v.grad

    dq, dk, dv = grads(dout)
    for t in (dq, dk, dv):
        assert bool(torch.isfinite(t.float()).all())
    # exactly linear in dO for a power-of-two factor
    dq4, dk4, dv4 = grads(dout * 4)
    assert torch.equal(dq4, dq * 4) and torch.equal(dk4, dk * 4) and torch.equal(dv4, dv * 4)
    del dq4, dk4, dv4
    # the oracle's gradients on one (sequence, kv head) group: all its query heads, full length
    b, hk = 5, 3
    G = Hq // Hkv
    rows = slice(b * S, (b + 1) * S)
    q = case.q[rows, hk * G:(hk + 1) * G].transpose(0, 1)[None].cpu()
    k = case.k[rows, hk:hk + 1].transpose(0, 1)[None].cpu()
    v = case.v[rows, hk:hk + 1].transpose(0, 1)[None].cpu()
    do = dout[rows, hk * G:(hk + 1) * G].transpose(0, 1)[None].cpu()
    rq, rk, rv, _ = orc.prefill_backward_reference(q, k, v, do, causal=True)
    for name, got, ref in (("dq", dq[rows, hk * G:(hk + 1) * G].transpose(0, 1)[None], rq),
                           ("dk", dk[rows, hk:hk + 1].transpose(0, 1)[None], rk),
                           ("dv", dv[rows, hk:hk + 1].transpose(0, 1)[None], rv)):
        err = (got.float().cpu() - ref).abs()
        bound = 2e-2 * float(ref.abs().max()) + 2e-2 * ref.abs()
        assert bool((err <= bound).all()), f"{name}: max err {float(err.max()):.4g} (max |ref| {float(ref.abs().max()):.4g})"


@pytest.mark.parametrize("fp8", [False, True])
def test_prompt_chunks_over_a_cached_prefix_at_serving_size(ops, fp8):
    """Four chunks of 2048 rows over 8192 cached tokens each, 32 query / 8 kv heads, head_dim 128, keys and values read
    through the block table (the shape of bench.py's paged legs).  The oracle on one sequence and the eight query
    heads of two kv heads; relocation: after moving every block to another physical position (tables rewritten) the
    output is identical bit for bit; and the packed kernel on the gathered rows gives the same bits (bf16 cache)."""
    print(f"case: paged chunks 4 x 2048 over 8192, fp8={fp8}", flush=True)
    dev = "cuda:0"
    B, chunk, ctx, Hq, Hkv, D = 4, 2048, 8192, 32, 8, 128
    nblk = ctx // 16
    g = torch.Generator(device=dev).manual_seed(77)
    pool = B * nblk + 9
    kc = (torch.randn(pool, Hkv, 16, D, device=dev, generator=g) * 0.7).to(torch.bfloat16)
    vc = (torch.randn(pool, Hkv, 16, D, device=dev, generator=g) * 0.7).to(torch.bfloat16)
    perm = torch.randperm(pool, device=dev, generator=g)
    table = perm[:B * nblk].view(B, nblk).to(torch.int32)
    lens = torch.full((B,), ctx, dtype=torch.int32, device=dev)
    cu = (torch.arange(B + 1, device=dev) * chunk).to(torch.int32)
    q = (torch.randn(B * chunk, Hq, D, device=dev, generator=g) * 0.7).to(torch.bfloat16)
    kw = {}
    kq, vq = kc, vc
    if fp8:
        kq, ks = ops.quantize_kv_cache_fp8(kc)
        vq, vs = ops.quantize_kv_cache_fp8(vc)
        kw = {"k_scale": ks, "v_scale": vs, "total_context": B * ctx}
    got = ops.flash_attn_paged_prefill(q, kq, vq, cu, table, lens, chunk, **kw)
    # oracle: sequence 2, query heads 0..7 (kv heads 0, 1), on the cache the kernel read (dequantised for fp8)
    b = 2
    ids = table[b].long()
    if fp8:
        k_seq = orc.dequantize_kv_fp8(kq[ids].cpu(), ks[ids].cpu())[:, :2]
        v_seq = orc.dequantize_kv_fp8(vq[ids].cpu(), vs[ids].cpu())[:, :2]
    else:
        k_seq, v_seq = kc[ids, :2].float().cpu(), vc[ids, :2].float().cpu()
    k_lin = k_seq.permute(1, 0, 2, 3).reshape(1, 2, ctx, D)
    v_lin = v_seq.permute(1, 0, 2, 3).reshape(1, 2, ctx, D)
    q_seq = q[b * chunk:(b + 1) * chunk, :8].transpose(0, 1)[None].cpu()
    ref = orc.prefill_reference(q_seq, k_lin, v_lin, causal=True, head_chunk=4)[0].transpose(0, 1)
    _close(got[b * chunk:(b + 1) * chunk, :8], ref)
    # relocation
    perm2 = torch.randperm(pool, device=dev, generator=g)
    k2, v2 = torch.empty_like(kq), torch.empty_like(vq)
    k2[perm2] = kq
    v2[perm2] = vq
    table2 = perm2[table.long()].to(torch.int32)
    kw2 = dict(kw)
    if fp8:
        ks2, vs2 = torch.empty_like(ks), torch.empty_like(vs)
        ks2[perm2] = ks
        vs2[perm2] = vs
        kw2.update(k_scale=ks2, v_scale=vs2)
    moved = ops.flash_attn_paged_prefill(q, k2, v2, cu, table2, lens, chunk, **kw2)
    assert torch.equal(moved, got)
    if not fp8:
        rows = kc[table.long()]                                         # (B, nblk, Hkv, 16, D) -> packed (B*ctx, Hkv, D)
        k_pack = rows.permute(0, 1, 3, 2, 4).reshape(B * ctx, Hkv, D).contiguous()
        v_pack = vc[table.long()].permute(0, 1, 3, 2, 4).reshape(B * ctx, Hkv, D).contiguous()
        cu_k = (torch.arange(B + 1, device=dev) * ctx).to(torch.int32)
        packed = ops.flash_attn_varlen_prefill(q, k_pack, v_pack, cu, cu_k, chunk, ctx, causal=True, kv_splits=1)
        assert torch.equal(packed, got)
