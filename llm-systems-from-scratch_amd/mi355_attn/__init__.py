"""MI355X-native attention hot path: HIP kernels for gfx950 behind the reference's Python API.

Drop-in surface (same names, argument meaning and tensor conventions as
llm-core/llm_core/model.py:308-325 and the SDPA slot at model.py:382):

    scaled_dot_product_attention(Q, K, V, mask=None)
    flash_attn_prefill(q, k, v, causal=True)            # f(Q, K, V, is_causal=True) slot
    flash_attn_varlen_prefill(q, k, v, cu_seqlens_q, cu_seqlens_k, ...)
    flash_attn_paged_prefill(q, k_cache, v_cache, cu_seqlens_q, block_tables, context_lens, max_seqlen_q)   # bf16 or fp8 cache
    paged_attention_decode(q, k_cache, v_cache, block_tables, context_lens, ...)
    rope_and_cache(q, k, v, positions, freq_cache, k_cache, v_cache, slot_mapping)   # cache producer
    quantize_kv_cache_fp8(cache)
    rope_and_cache_fp8(q, k, v, positions, freq_cache, k_cache8, v_cache8, k_scale, v_scale, slot_mapping)
    rms_norm(x, weight, eps, residual=None)             # RMSNorm.forward / TritonRMSNorm forward
    silu_mul(gate, up)                                  # fused kernel of FusedSwiGLU

Every function runs on the HIP library; there is no CPU or PyTorch fallback.
"""
from .ops import (  # noqa: F401
    build_rope_cache,
    quantize_kv_cache_fp8,
    rms_norm,
    rope_and_cache,
    rope_and_cache_fp8,
    silu_mul,
    flash_attn_paged_prefill,
    gather_kv_fp8,
    flash_attn_prefill,
    flash_attn_varlen_prefill,
    paged_attention_decode,
    paged_decode_workspace,
    decode_chunk_tokens,
    prefill_splitkv_workspace,
    suggest_kv_splits,
    scaled_dot_product_attention,
    sdpa_slot,
)
from .engine import BlockAllocator, OutOfBlocks, PagedAttentionEngine  # noqa: F401
from .model import CachedTransformerLM  # noqa: F401
from ._lib import LIB_PATH, LibraryMissing, load  # noqa: F401
