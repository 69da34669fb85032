"""ctypes binding of libmi355attn.so (declarations mirror include/mi355_attn.h)."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmi355attn.so")

MI355_BF16 = 0
MI355_FP8_E4M3 = 1
MI355_FP32 = 2
MASK_NONE, MASK_CAUSAL, MASK_BOOL = 0, 1, 2
STATIC_SCRATCH_BYTES = 16 << 20          # MI355_STATIC_SCRATCH_BYTES

_i64x3 = C.c_int64 * 3
_i64x2 = C.c_int64 * 2
_lib = None

EXPORTS = (
    "mi355_prefill_fwd",
    "mi355_prefill_fwd_lse",
    "mi355_prefill_bwd",
    "mi355_prefill_fwd_mask_lse",
    "mi355_prefill_bwd_mask",
    "mi355_paged_decode_fwd",
    "mi355_paged_decode_fwd_static",
    "mi355_paged_decode_workspace_bytes",
    "mi355_paged_decode_chunk_tokens",
    "mi355_prefill_paged_fwd",
    "mi355_gather_kv_fp8",
    "mi355_prefill_fwd_splitkv",
    "mi355_prefill_splitkv_workspace_bytes",
    "mi355_prefill_suggest_kv_splits",
    "mi355_rope_and_cache",
    "mi355_rope_and_cache_fp8",
    "mi355_quantize_kv_fp8",
    "mi355_rms_norm_fwd",
    "mi355_silu_mul_fwd",
    "mi355_calib_copy",
    "mi355_last_error",
    "mi355_version",
)


class LibraryMissing(RuntimeError):
    pass


def load():
    """Loads the HIP library once.  There is no fallback: a missing library is an error."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise LibraryMissing(
            f"{LIB_PATH} is not built; run `python llm-systems-from-scratch_amd/build.py` "
            "(needs hipcc, cross-compiles for gfx950 without a GPU)")
    lib = C.CDLL(LIB_PATH)
    vp, i32, i64, f32, sz = C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_size_t
    lib.mi355_prefill_fwd.restype = i32
    lib.mi355_prefill_fwd.argtypes = [vp, vp, vp, vp, _i64x3, _i64x3, _i64x3, _i64x3, vp, vp, vp, _i64x3,
                                      i32, i32, i32, i32, i32, i32, f32, i32, i32, vp]
    lib.mi355_prefill_fwd_lse.restype = i32
    lib.mi355_prefill_fwd_lse.argtypes = [vp, vp, vp, vp, vp, _i64x3, _i64x3, _i64x3, _i64x3, _i64x2, vp, vp,
                                          i32, i32, i32, i32, i32, i32, f32, i32, i32, vp]
    lib.mi355_prefill_bwd.restype = i32
    lib.mi355_prefill_bwd.argtypes = [vp] * 10 + [_i64x3] * 8 + [_i64x2, vp, vp,
                                                                 i32, i32, i32, i32, i32, i32, f32, i32, i32, vp]
    lib.mi355_prefill_fwd_mask_lse.restype = i32
    lib.mi355_prefill_fwd_mask_lse.argtypes = [vp, vp, vp, vp, vp, _i64x3, _i64x3, _i64x3, _i64x3, _i64x2, vp, _i64x3,
                                               i32, i32, i32, i32, i32, i32, f32, i32, vp]
    lib.mi355_prefill_bwd_mask.restype = i32
    lib.mi355_prefill_bwd_mask.argtypes = [vp] * 10 + [_i64x3] * 8 + [_i64x2, vp, _i64x3,
                                                                      i32, i32, i32, i32, i32, i32, f32, i32, vp]
    lib.mi355_prefill_paged_fwd.restype = i32
    lib.mi355_prefill_paged_fwd.argtypes = [vp, vp, vp, vp, i64, i64, vp, vp, i64, i64, vp,
                                            i32, i32, i32, i32, i32, i32, i64, f32, i32, i32, i64, vp, sz, vp]
    lib.mi355_gather_kv_fp8.restype = i32
    lib.mi355_gather_kv_fp8.argtypes = [vp, vp, vp, vp, vp, i64, i64, vp, vp, vp, vp, i64, i64, i32, i32, i32, i32, i64, vp]
    lib.mi355_prefill_fwd_splitkv.restype = i32
    lib.mi355_prefill_fwd_splitkv.argtypes = [vp, vp, vp, vp, _i64x3, _i64x3, _i64x3, _i64x3, vp, vp,
                                              i32, i32, i32, i32, i32, i32, f32, i32, i32, i32, i64, vp, sz, vp]
    lib.mi355_prefill_splitkv_workspace_bytes.restype = sz
    lib.mi355_prefill_splitkv_workspace_bytes.argtypes = [i64, i32, i32, i32]
    lib.mi355_prefill_suggest_kv_splits.restype = i32
    lib.mi355_prefill_suggest_kv_splits.argtypes = [i32, i32, i32, i32, i32, i64, i32, i32]
    lib.mi355_paged_decode_fwd.restype = i32
    lib.mi355_paged_decode_fwd.argtypes = [vp, vp, vp, vp, vp, i64, vp, vp, vp, vp, sz,
                                           i32, i32, i32, i32, i32, i64, i32, f32, i32, vp]
    lib.mi355_paged_decode_fwd_static.restype = i32
    lib.mi355_paged_decode_fwd_static.argtypes = [vp, vp, vp, vp, vp, i64, vp, vp, vp,
                                                  i32, i32, i32, i32, i32, i64, i32, f32, i32, vp]
    lib.mi355_paged_decode_workspace_bytes.restype = sz
    lib.mi355_paged_decode_workspace_bytes.argtypes = [i32, i32, i32, i32]
    lib.mi355_paged_decode_chunk_tokens.restype = i32
    lib.mi355_paged_decode_chunk_tokens.argtypes = [i32, i32, i32, i32]
    lib.mi355_rope_and_cache.restype = i32
    lib.mi355_rope_and_cache.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, i32, i32, i32, i32, i32,
                                         i64, i64, i64, i64, vp, i64, vp]
    lib.mi355_rope_and_cache_fp8.restype = i32
    lib.mi355_rope_and_cache_fp8.argtypes = [vp] * 11 + [i64, i32, i32, i32, i32, i32, i64, i64, i64, i64, vp, i64, vp]
    lib.mi355_quantize_kv_fp8.restype = i32
    lib.mi355_quantize_kv_fp8.argtypes = [vp, vp, vp, i64, i32, i32, i32, vp]
    lib.mi355_rms_norm_fwd.restype = i32
    lib.mi355_rms_norm_fwd.argtypes = [vp, vp, vp, vp, vp, vp, i64, i32, i64, i64, i64, i64, f32, i32, vp]
    lib.mi355_silu_mul_fwd.restype = i32
    lib.mi355_silu_mul_fwd.argtypes = [vp, vp, vp, i64, i32, i64, i64, i64, vp]
    lib.mi355_calib_copy.restype = i32
    lib.mi355_calib_copy.argtypes = [vp, vp, sz, vp]
    lib.mi355_last_error.restype = C.c_char_p
    lib.mi355_version.restype = C.c_char_p
    _lib = lib
    return lib


def strides3(values):
    return _i64x3(*[int(v) for v in values])


def strides2(values):
    return _i64x2(*[int(v) for v in values])


def check(rc: int, what: str):
    if rc != 0:
        msg = load().mi355_last_error().decode()
        if rc < 0:
            raise ValueError(f"{what}: {msg} (code {rc})")
        raise RuntimeError(f"{what}: HIP error {rc}: {msg}")
