"""mi355_paged_decode_fwd_static (the entry point that allocates nothing: split-K partials in the library's own
device array) against mi355_paged_decode_fwd with a caller-provided workspace, through the C ABI: same kernels,
same layout, so the outputs must be equal bit for bit.  Two calls in a row share the array, the second with a
smaller problem (fewer sequences, shorter contexts, another chunk size), so leftovers of the first call are there
to be tripped over."""
import pytest
import torch

from oracle import attention_oracle as orc

pytestmark = pytest.mark.gpu


def _both(lib, _lib, case, fp8):
    dev = "cuda:0"
    q, kc, vc, bt, cl = case
    ks = vs = None
    if fp8:
        kc, ks = orc.quantize_kv_fp8(kc)
        vc, vs = orc.quantize_kv_fp8(vc)
        kc, vc = kc.view(torch.uint8), vc.view(torch.uint8)
        ks, vs = ks.to(dev), vs.to(dev)
    q, kc, vc, bt, cl = (t.to(dev) for t in (q, kc, vc, bt, cl))
    B, Hq, D = q.shape
    Hkv = kc.shape[1]
    max_ctx = bt.shape[1] * 16
    need = lib.mi355_paged_decode_workspace_bytes(B, Hq, D, max_ctx)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    out_ws = torch.full_like(q, float("nan"))
    out_static = torch.full_like(q, float("nan"))
    stream = torch.cuda.current_stream().cuda_stream
    kv = _lib.MI355_FP8_E4M3 if fp8 else _lib.MI355_BF16
    sp = (lambda t: None if t is None else t.data_ptr())
    rc = lib.mi355_paged_decode_fwd(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), out_ws.data_ptr(), bt.data_ptr(),
                                    bt.stride(0), cl.data_ptr(), sp(ks), sp(vs), ws.data_ptr(), need,
                                    B, Hq, Hkv, D, 16, kc.shape[0], max_ctx, D ** -0.5, kv, stream)
    _lib.check(rc, "mi355_paged_decode_fwd")
    rc = lib.mi355_paged_decode_fwd_static(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), out_static.data_ptr(),
                                           bt.data_ptr(), bt.stride(0), cl.data_ptr(), sp(ks), sp(vs),
                                           B, Hq, Hkv, D, 16, kc.shape[0], max_ctx, D ** -0.5, kv, stream)
    _lib.check(rc, "mi355_paged_decode_fwd_static")
    torch.cuda.synchronize()
    return out_ws, out_static, (q.cpu(), kc.cpu(), vc.cpu(), bt.cpu(), cl.cpu(), None if ks is None else ks.cpu(),
                                None if vs is None else vs.cpu())


@pytest.mark.parametrize("fp8", [False, True])
def test_static_scratch_entry_point_equals_the_workspace_one(fp8):
    import mi355_attn
    from mi355_attn import _lib
    lib = mi355_attn.load()
    print(f"case: no-alloc decode fp8={fp8}", flush=True)
    big = orc.make_paged_case(batch=16, n_q_heads=32, n_kv_heads=8, head_dim=128, block_size=16,
                              context_lens=[12000, 4097, 8192, 1, 500, 4096, 9000, 10000, 33, 7000, 5000, 11999, 16, 4095,
                                            8193, 6000], pool_factor=1.1, seed=5, dtype=torch.bfloat16)
    small = orc.make_paged_case(batch=5, n_q_heads=32, n_kv_heads=8, head_dim=128, block_size=16,
                                context_lens=[3000, 2049, 17, 2500, 1], pool_factor=1.2, seed=6, dtype=torch.bfloat16)
    for name, case in (("first call", big), ("second, smaller call", small)):
        out_ws, out_static, (q, kc, vc, bt, cl, ks, vs) = _both(lib, _lib, case, fp8)
        assert bool(torch.isfinite(out_static.float()).all()), name
        assert torch.equal(out_ws, out_static), name
        ref = orc.paged_decode_reference(q, kc, vc, bt, cl, k_scale=ks, v_scale=vs)
        err = (out_static.float().cpu() - ref).abs()
        assert bool((err <= 2e-2 + 1e-2 * ref.abs()).all()), (name, float(err.max()))


def test_static_scratch_entry_point_rejects_what_does_not_fit():
    import mi355_attn
    from mi355_attn import _lib
    lib = mi355_attn.load()
    print("case: no-alloc decode, too large", flush=True)
    q = torch.zeros(256, 64, 128, dtype=torch.bfloat16, device="cuda:0")
    kc = torch.zeros(4, 8, 16, 128, dtype=torch.bfloat16, device="cuda:0")
    bt = torch.zeros(256, 2048, dtype=torch.int32, device="cuda:0")
    cl = torch.ones(256, dtype=torch.int32, device="cuda:0")
    assert lib.mi355_paged_decode_workspace_bytes(256, 64, 128, 32768) > _lib.STATIC_SCRATCH_BYTES
    rc = lib.mi355_paged_decode_fwd_static(q.data_ptr(), kc.data_ptr(), kc.data_ptr(), q.data_ptr(), bt.data_ptr(),
                                           bt.stride(0), cl.data_ptr(), None, None, 256, 64, 8, 128, 16, 4, 32768,
                                           0.1, _lib.MI355_BF16, None)
    assert rc == -2 and b"static scratch" in lib.mi355_last_error()
    # the Python operator: needs `out`, raises on a problem that does not fit
    with pytest.raises(ValueError, match="out"):
        mi355_attn.paged_attention_decode(q, kc, kc, bt, cl, static_scratch=True)
    with pytest.raises(ValueError, match="static scratch"):
        mi355_attn.paged_attention_decode(q, kc, kc, bt, cl, static_scratch=True, out=torch.empty_like(q))
    # one chunk needs no scratch at all, whatever the batch
    out = torch.empty_like(q)
    mi355_attn.paged_attention_decode(q, kc, kc, bt[:, :4].contiguous(), cl, static_scratch=True, out=out)
    torch.cuda.synchronize()
    assert bool((out == 0).all())
