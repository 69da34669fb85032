"""CPU-side checks: the C-ABI library loads, exports what include/mi355_attn.h declares, and rejects
bad arguments before touching a GPU; host-side operator validation; workload generators."""
import ctypes as C
import os
import re

import pytest
import torch

import mi355_attn
from mi355_attn import _lib, workloads

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    return mi355_attn.load()


def declared_functions():
    text = open(os.path.join(ROOT, "include", "mi355_attn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib):
    names = declared_functions()
    assert "mi355_prefill_fwd" in names and "mi355_paged_decode_fwd" in names
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/mi355_attn.h but not exported"
    assert sorted(_lib.EXPORTS) == names


def test_version_and_workspace_queries(lib):
    assert b"gfx950" in lib.mi355_version()
    # (batch, query heads, kv heads, longest context): a batch that fills the GPU gets chunks that grow with the context
    assert lib.mi355_paged_decode_chunk_tokens(128, 32, 8, 256) == 1024
    assert lib.mi355_paged_decode_chunk_tokens(128, 32, 8, 3000) == 2048
    assert lib.mi355_paged_decode_chunk_tokens(128, 32, 8, 16384) == 4096
    # ... and a small batch shorter ones, until it has about 256 workgroups (down to 4 x 64 tokens)
    assert lib.mi355_paged_decode_chunk_tokens(1, 32, 8, 8192) == 256
    assert lib.mi355_paged_decode_chunk_tokens(1, 32, 8, 131072) == 4096
    assert lib.mi355_paged_decode_chunk_tokens(4, 32, 8, 8192) == 1024
    assert lib.mi355_paged_decode_chunk_tokens(1, 32, 8, 100) == 1024          # one chunk and no combine pass up to 1024 tokens
    assert lib.mi355_paged_decode_chunk_tokens(1, 32, 8, 1025) == 256
    assert lib.mi355_paged_decode_chunk_tokens(0, 32, 8, 100) == 0 and lib.mi355_paged_decode_chunk_tokens(1, 32, 5, 100) == 0
    # one chunk -> still a (small) partial area; grows with chunks * B * Hq * D
    small = lib.mi355_paged_decode_workspace_bytes(4, 8, 64, 256)
    big = lib.mi355_paged_decode_workspace_bytes(128, 32, 128, 16384)
    assert 0 < small < big
    chunks = (16384 + 4095) // 4096
    assert big >= 128 * 32 * chunks * (128 + 2) * 4
    assert lib.mi355_paged_decode_workspace_bytes(0, 8, 64, 256) == 0


def test_workspace_requirement_is_monotonic_in_max_ctx(lib):
    """A workspace sized for the largest batch and the longest context must serve every smaller call, although the
    chunk size (and with it the number of chunks a launch uses) changes at 2048 and 4096 tokens and shrinks for
    small batches."""
    def need(B, Hq, Hkv, D, m):          # what a launch with these bounds really lays out
        chunk = lib.mi355_paged_decode_chunk_tokens(B, Hq, Hkv, m)
        rows = B * Hq * ((m + chunk - 1) // chunk)
        return rows * D * 4 + 2 * rows * 4

    for B, Hq, Hkv, D in ((64, 16, 4, 128), (3, 8, 8, 64), (1, 32, 8, 128), (2, 64, 1, 128)):
        prev = 0
        for m in list(range(1, 9000, 7)) + [16384, 16385, 32768, 100000]:
            cur = lib.mi355_paged_decode_workspace_bytes(B, Hq, D, m)
            assert cur >= prev, (B, Hq, D, m)
            assert cur >= need(B, Hq, Hkv, D, m), (B, Hq, D, m)
            prev = cur
        # and in the batch and head counts
        assert lib.mi355_paged_decode_workspace_bytes(B - 1, Hq, D, 5000) <= lib.mi355_paged_decode_workspace_bytes(B, Hq, D, 5000)
    # every smaller call fits the workspace of the largest one
    Hq, Hkv, D = 32, 8, 128
    for B_max, m_max in ((64, 32768), (8, 4096), (256, 2000)):
        have = lib.mi355_paged_decode_workspace_bytes(B_max, Hq, D, m_max)
        for B in sorted({1, 2, 3, 5, 8, 13, 32, 63, B_max}):
            if B > B_max:
                continue
            for m in (1, 255, 257, 1000, 1025, 2047, 2048, 4095, 4096, 8191, 20000, m_max):
                if m <= m_max:
                    assert need(B, Hq, Hkv, D, m) <= have, (B_max, m_max, B, m)


def test_prefill_rejects_bad_arguments_without_a_gpu(lib):
    s3 = _lib.strides3((8, 8, 8))
    buf = C.create_string_buffer(64)
    ptr = (C.addressof(buf) + 15) & ~15

    def call(D=64, Hq=2, Hkv=2, q=ptr, mode=_lib.MASK_CAUSAL, dtype=_lib.MI355_BF16, mask=None, cu_q=None, cu_k=None,
             strides=s3):
        return lib.mi355_prefill_fwd(q, ptr, ptr, ptr, strides, s3, s3, s3, cu_q, cu_k, mask, s3,
                                     1, Hq, Hkv, 8, 8, D, 0.125, mode, dtype, None)

    assert call(D=96) == -1 and b"head_dim" in lib.mi355_last_error()
    assert call(Hq=3, Hkv=2) == -1
    assert call(q=None) == -1 and b"null" in lib.mi355_last_error()
    assert call(dtype=7) == -3
    assert call(mode=9) == -1
    assert call(mode=_lib.MASK_BOOL, mask=None) == -1
    assert call(cu_q=ptr, cu_k=None) == -1
    assert call(strides=_lib.strides3((8, 8, 4))) == -1 and b"strides" in lib.mi355_last_error()
    assert call(q=ptr + 2) == -1 and b"aligned" in lib.mi355_last_error()


def test_prefill_split_keys_rejects_bad_arguments_without_a_gpu(lib):
    s3 = _lib.strides3((8, 8, 8))
    buf = C.create_string_buffer(64)
    ptr = (C.addressof(buf) + 15) & ~15
    need = lib.mi355_prefill_splitkv_workspace_bytes(8, 2, 64, 4)
    assert need == 4 * 2 * 8 * (64 + 1) * 4
    assert lib.mi355_prefill_splitkv_workspace_bytes(8, 2, 64, 1) == 0

    def call(n_split=4, rows=8, ws=ptr, ws_bytes=need, mode=_lib.MASK_CAUSAL):
        return lib.mi355_prefill_fwd_splitkv(ptr, ptr, ptr, ptr, s3, s3, s3, s3, None, None, 1, 2, 2, 8, 8, 64, 0.125,
                                             mode, _lib.MI355_BF16, n_split, rows, ws, ws_bytes, None)

    assert call(n_split=65) == -1 and b"n_split" in lib.mi355_last_error()
    assert call(n_split=0) == -1
    assert call(rows=7) == -1 and b"total_q_rows" in lib.mi355_last_error()
    assert call(ws=None) == -1 and b"workspace" in lib.mi355_last_error()
    assert call(ws=ptr + 4) == -1
    assert call(ws_bytes=need - 1) == -2 and b"workspace" in lib.mi355_last_error()
    assert call(mode=_lib.MASK_BOOL) == -1


def test_suggested_key_splits_follow_the_measured_cases(lib):
    """The cost model against timings taken on an MI355X (256 compute units): few query rows over many keys are
    split, a launch that fills the GPU is not, and the suggestion never leaves a share fewer than two K/V tiles."""
    def n(B, Hq, Sq, Sk, causal=1):
        return lib.mi355_prefill_suggest_kv_splits(B, Hq, 128, Sq, Sk, B * Sq, causal, 256)

    assert n(8, 32, 4096, 4096) == 1                    # configs[2]: 768 workgroups
    assert n(1, 32, 2048, 2048) == 1                    # measured: 49 us unsplit (a compute unit per query tile), 80 us split in two
    assert n(8, 32, 128, 2048) == 1                     # measured: 60 us unsplit, 85 us split in two
    assert 6 <= n(1, 32, 256, 16384) <= 8               # measured best 6-8 (291 -> 80 us)
    assert 4 <= n(1, 32, 256, 8192) <= 8                # measured best 6 (150 -> 53 us)
    assert n(1, 32, 1024, 8192) == 2                    # measured best 2 (153 -> 131 us)
    assert 3 <= n(1, 32, 512, 8192) <= 4                # measured best 4 (153 -> 80 us)
    assert 8 <= n(1, 8, 512, 16384) <= 16               # measured best 12 (290 -> 60 us)
    assert 3 <= n(8, 8, 128, 2048) <= 4                 # measured best 3 (46 -> 32 us)
    assert n(1, 8, 64, 32768) >= 16                     # measured best 16-24 (566 -> 61 us)
    assert n(4, 32, 256, 4096) <= 2                     # measured: 89 us unsplit, 83 us split in two
    for Sq, Sk in ((1, 1), (64, 64), (256, 300), (100, 128)):
        assert n(1, 1, Sq, Sk) == 1 and n(1, 1, Sq, Sk, causal=0) == 1
    assert n(1, 1, 64, 100000, causal=0) == 64
    assert lib.mi355_prefill_suggest_kv_splits(0, 8, 128, 64, 64, 0, 1, 256) == 1


def test_decode_rejects_bad_arguments_without_a_gpu(lib):
    buf = C.create_string_buffer(64)
    ptr = C.addressof(buf)

    def call(Hq=8, Hkv=2, D=128, bs=16, kv=_lib.MI355_BF16, ks=None, ws=ptr, ws_bytes=1 << 30, max_ctx=64, q=ptr, nb=8):
        return lib.mi355_paged_decode_fwd(q, ptr, ptr, ptr, ptr, 4, ptr, ks, ks, ws, ws_bytes,
                                          2, Hq, Hkv, D, bs, nb, max_ctx, 0.1, kv, None)

    assert call(bs=32) == -1 and b"block_size" in lib.mi355_last_error()
    assert call(Hq=7) == -1
    assert call(D=96) == -1
    assert call(kv=5) == -3
    assert call(kv=_lib.MI355_FP8_E4M3, ks=None) == -1 and b"scale" in lib.mi355_last_error()
    assert call(kv=_lib.MI355_FP8_E4M3, ks=ptr, D=32) == -1
    assert call(q=None) == -1
    assert call(nb=0) == -1 and b"num_blocks" in lib.mi355_last_error()
    assert call(max_ctx=100000, ws_bytes=16) == -2 and b"workspace" in lib.mi355_last_error()


def test_fp8_cache_write_rejects_a_k_out_that_overlaps_k_in(lib):
    """The fp8 cache write reads the keys twice (query workgroups emit k_out, key/value workgroups quantise): k_out on
    top of k_in would hand rotated rows to the second reader.  The argument check refuses it before any launch."""
    buf = (C.c_char * 8192)()
    base = (C.addressof(buf) + 15) & ~15

    def call(k_in, k_out, T=4, Hkv=2, D=32, k_stride=64, ko_stride=64):
        return lib.mi355_rope_and_cache_fp8(base, k_in, base, base, base, base, base, base, base, base, base,
                                            8, T, 2, Hkv, D, 16, 64, k_stride, 64, 64, k_out, ko_stride, None)

    assert call(base, base) == -1 and b"overlap" in lib.mi355_last_error()
    assert call(base, base + 3 * 128 + 96) == -1                   # last 32 bytes of k_in's last row
    assert call(base + 496, base) == -1 and b"overlap" in lib.mi355_last_error()    # k_out's last 16 bytes reach into k_in
    # the same pointers with no tokens: nothing is read, nothing to refuse
    assert call(base, base, T=0) == 0


def test_host_ops_validate_before_launch():
    q = torch.zeros(2, 4, 64, dtype=torch.bfloat16)
    kc = torch.zeros(8, 2, 16, 64, dtype=torch.bfloat16)
    bt = torch.zeros(2, 4, dtype=torch.int32)
    cl = torch.ones(2, dtype=torch.int32)
    with pytest.raises(ValueError, match="GPU"):
        mi355_attn.paged_attention_decode(q, kc, kc, bt, cl)
    with pytest.raises(ValueError, match="GPU"):
        mi355_attn.flash_attn_prefill(torch.zeros(1, 2, 8, 64, dtype=torch.bfloat16),
                                      torch.zeros(1, 2, 8, 64, dtype=torch.bfloat16),
                                      torch.zeros(1, 2, 8, 64, dtype=torch.bfloat16))
    with pytest.raises(TypeError):
        mi355_attn.scaled_dot_product_attention(torch.zeros(2, 8, 64), torch.zeros(2, 8, 64), torch.zeros(2, 8, 64),
                                                mask=torch.zeros(8, 8))          # mask must be boolean


def test_missing_library_is_an_error_not_a_fallback(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libmi355attn.so")
    with pytest.raises(_lib.LibraryMissing):
        _lib.load()


def test_product_package_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "llm-systems-from-scratch_amd")
    for d, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(d, f)).read()
                assert "attention_oracle" not in text and "from oracle" not in text and "import oracle" not in text, f


def test_workload_draws_match_the_configurations():
    c3 = workloads.draw_context_lens("uniform", 128, 512, 16384, 0)
    assert c3.shape == (128,) and c3.min() >= 512 and c3.max() <= 16384
    assert torch.equal(c3, workloads.draw_context_lens("uniform", 128, 512, 16384, 0))
    c4 = workloads.draw_context_lens("loguniform", 256, 128, 32768, 0)
    assert c4.min() >= 128 and c4.max() <= 32768
    # the oracle's generator (used by the tests) and the product's draw the same lengths
    from oracle import attention_oracle as orc
    assert torch.equal(c3, orc.draw_context_lens("uniform", 128, 512, 16384, 0))
    assert torch.equal(c4, orc.draw_context_lens("loguniform", 256, 128, 32768, 0))


def test_committed_assembly_include_is_what_the_generator_writes(tmp_path):
    """csrc/prefill_w64_asm.inc is generated text that every build rewrites: the committed copy must be the generator's
    output byte for byte (a hand edit or a stale commit would otherwise be invisible), and the generator must take no
    switches from the environment."""
    import subprocess
    import sys

    csrc = os.path.join(ROOT, "llm-systems-from-scratch_amd", "csrc")
    gen = os.path.join(csrc, "gen_prefill_w64_loop.py")
    out = tmp_path / "w64.inc"
    env = dict(os.environ, W64_ABL="nobarrier,nodma,nocheck,noexp,novalu,nosum,nofma")     # must have no effect
    subprocess.run([sys.executable, gen, str(out)], check=True, capture_output=True, env=env)
    assert out.read_bytes() == open(os.path.join(csrc, "prefill_w64_asm.inc"), "rb").read()
    assert "environ" not in open(gen).read()
