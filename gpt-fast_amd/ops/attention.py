"""Attention over the paged cache: which kernel runs a step's attention.

float32 engine: the plain kernel (one workgroup per token and head, float arithmetic
in an order fixed by the token's position).  bfloat16 engine: the split-context kernel
for one-token steps, the MFMA kernel for prompts (csrc/attention_bf16.hip), and the
plain kernel for shapes those refuse.
"""
import torch

from . import kernels as K


def attention(q, k_pages, v_pages, batch, table, scale: float, window: int = 0,
              for_product: bool = False):
    """q [N, H, hd] of the step's tokens; returns [N, H, hd].  ``for_product``: the caller
    only hands the result to a few-row product of ``ops.linear`` that takes
    ``gemm_bf16.ChunkedRows`` ([N, H * hd]), and may get that instead."""
    if q.dtype == torch.bfloat16:
        from . import attention_bf16 as fast
        y = fast.attention(q, k_pages, v_pages, batch, table, scale, window, chunked=for_product)
        if y is not None:
            return y
    return K.attention_generic(q, k_pages, v_pages, batch.tok_seq, batch.tok_pos, table,
                               scale, window)
