"""Functional entry points (reference: trident/function/function.py:238-253)."""
import math

import torch

from . import operation


def scaled_dot_product_attention(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    attn_mask: torch.Tensor = None,
    dropout_p: float = 0.0,
    is_causal: bool = False,
    use_accelerator: bool = False,
):
    """
    Computes scaled dot product attention on query, key and value tensors,
    and applying dropout if a probability greater than 0.0 is specified.
    """
    return operation.Attention.apply(
        query, key, value, attn_mask, dropout_p, is_causal, 1.0 / math.sqrt(key.shape[-1]), use_accelerator
    )


def attention(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    mask: torch.Tensor = None,
    dropout_p: float = 0.0,
    is_causal: bool = False,
    softmax_scale: float = None,
):
    """Same operation with an explicit softmax scale (default 1/sqrt(head size)): the positional
    argument list of operation.Attention.apply without ``use_accelerator``."""
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(key.shape[-1])
    return operation.Attention.apply(query, key, value, mask, dropout_p, is_causal, softmax_scale, False)
