"""Functional entry points (reference: trident/function/function.py:58-67, 166-172, 238-262)."""
import math

import torch

from . import operation


def dropout(input, p=0.5, training=True):
    """
    Applies Dropout to an input.

    See Dropout for details.
    """
    if training:
        return operation.Dropout.apply(input.view(-1, input.shape[-1]), p).view(input.shape)
    else:
        return input.clone()


def masked_softmax(input: torch.Tensor, mask: torch.Tensor, dim: int):
    """
    Applies Masked Softmax to an input rescaling them so that an output lie in the range [0,1] and sum to 1.

    See MaskedSoftmax for more details.
    """
    return operation.MaskedSoftmax.apply(input, mask, dim)


def softmax(input: torch.Tensor, dim: int = None):
    """
    Applies Softmax to an input rescaling them so that an output lie in the range [0,1] and sum to 1.

    See Softmax for more details.
    """
    return operation.Softmax.apply(input, dim)


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
    return operation.Attention.call(
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
    return operation.Attention.call(query, key, value, mask, dropout_p, is_causal, softmax_scale, False)
