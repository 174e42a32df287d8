"""Which kernel runs an operation: chosen by dtype and shape, never silently wrong.

float32 activations always take the 32-bit kernels (plain multiply-adds, accurate
exp and sqrt). bfloat16 activations take the matrix-core kernels where the shape
fits what they are written for and the generic kernels otherwise.
"""
from __future__ import annotations

import torch

from ..csrc import lib as K

EPI_STORE, EPI_ADD, EPI_GATED = K.EPI_STORE, K.EPI_ADD, K.EPI_GATED

# switches for tests and measurements: names of fast kernels that must not be used
disabled = set()


def linear(a, w, out, epilogue=EPI_STORE):
    """out (=, +=, gated) a @ w.T."""
    if a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
        M = a.shape[0]
        if "skinny" not in disabled and K.has("gl3_gemm_skinny") and K.gemm_skinny_fits(a, w, out, epilogue):
            return K.gemm_skinny(a, w, out, epilogue)
        if "mfma" not in disabled and K.has("gl3_gemm_mfma") and K.gemm_mfma_fits(a, w, out, epilogue):
            return K.gemm_mfma(a, w, out, epilogue)
    return K.gemm_generic(a, w, out, epilogue)


def attention(ctx, q, k_cache, v_cache, block_table, out, n_heads, n_kv, head_dim, window, scale):
    page = k_cache.shape[2]          # keys are [page, kv head, position in page, head_dim]
    if q.dtype == torch.bfloat16:
        if (ctx.decode and "attn_decode" not in disabled and K.has("gl3_attention_decode")
                and K.attention_decode_fits(head_dim, n_heads, n_kv, page)):
            T = q.shape[0]
            splits = K.decode_splits(T, n_heads, n_kv, ctx.kv_len_hint)
            part_o = part_ml = None
            if splits > 1:
                part_o = ctx.buffer("attn_part_o", (T, n_heads, splits, head_dim), torch.float32)
                part_ml = ctx.buffer("attn_part_ml", (T, n_heads, splits, 2), torch.float32)
            return K.attention_decode(q, k_cache, v_cache, ctx.positions, ctx.seq_of_token, block_table, out, n_heads,
                                      n_kv, head_dim, page, window, scale, splits, part_o, part_ml)
        if (not ctx.decode and "attn_prefill" not in disabled and K.has("gl3_attention_prefill")
                and K.attention_prefill_fits(head_dim, n_heads, n_kv, page)):
            return K.attention_prefill(q, k_cache, v_cache, ctx.cu_seqlens, ctx.kv_before, block_table, out,
                                       ctx.max_q_len, n_heads, n_kv, head_dim, page, window, scale)
    return K.attention_generic(q, k_cache, v_cache, ctx.positions, ctx.seq_of_token, block_table, out, n_heads, n_kv,
                               head_dim, page, window, scale)
