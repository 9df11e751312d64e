"""MI355X (gfx950) flash attention with flexible masks.

    from flash_mi355 import attention, SCORE_FUNC_MODE1_DOC
    out = attention(q, k, v, causal=True, eq=eq, ek=ek, score_func_mode=SCORE_FUNC_MODE1_DOC)

The four public names match the reference module ``flash_triton``.
"""
from .api import (SCORE_FUNC_MODE0_NOPE, SCORE_FUNC_MODE1_DOC, SCORE_FUNC_MODE2_BLOCK, FlashAttention, FlashAttentionWithLse, attention,
                  attention_varlen, attention_with_lse, mask_dump, maybe_contiguous, varlen_ids, varlen_positions)

__all__ = ["attention", "FlashAttention", "FlashAttentionWithLse", "SCORE_FUNC_MODE0_NOPE", "SCORE_FUNC_MODE1_DOC",
           "attention_with_lse", "attention_varlen", "varlen_ids", "varlen_positions", "mask_dump", "maybe_contiguous"]
