"""Attention autograd Function behind the reference's operator API.

Mirrors trident/operation/attention.py:23-202: the same eight positional arguments, the same
validation errors, the same saved state and the same 8-tuple returned by backward. The three
Triton launches of the reference (attention.py:109, 161, 170) become calls into
libtrident_attn.so (include/tri_attn.h).
"""
import ctypes
from typing import Any

import torch

from . import _lib, config, util


def _strides4(t: torch.Tensor):
    s = list(t.stride())
    if t.shape[-1] == 1:
        s[-1] = 1
    return s


def _dense_rows(t: torch.Tensor) -> torch.Tensor:
    """The kernels need unit stride along the last dimension and non-negative strides."""
    if t.shape[-1] != 1 and t.stride(-1) != 1:
        return t.contiguous()
    return t


def _require_same_gpu(device, **tensors):
    """Every tensor handed to the library must live on the one GPU the call runs on: the kernels
    dereference the raw pointers, so a host or other-device tensor must stop here, as an exception."""
    if device.type != "cuda":
        raise RuntimeError("trident_amd attention runs on the GPU only; got a tensor on " + str(device))
    for name, t in tensors.items():
        if t is not None and t.device != device:
            raise RuntimeError(f"trident_amd attention: {name} is on {t.device}, expected {device} "
                               "(all tensors of a call must be on the same GPU)")


def _next_seed():
    fixed = config.dropout_seed
    if fixed is None:
        return int(torch.randint(0, 2**63 - 1, (1,), dtype=torch.int64).item()), 0
    if isinstance(fixed, int):
        fixed = (fixed, 0)
    seed, offset = int(fixed[0]), int(fixed[1])
    config.dropout_seed = (seed, offset + 1)
    return seed, offset


_NO_STRIDES = (0, 0, 0, 0)


def _strides_or_zero(t):
    if t is None:
        return _NO_STRIDES
    return t.stride() if t.shape[-1] != 1 else tuple(_strides4(t))


def _make_args(query, key, value, output, log2sum, mask, dropout_p, is_causal, softmax_scale, seed, offset,
               grad_output=None, grad_query=None, grad_key=None, grad_value=None, grad_mask=None, delta=None):
    """TriAttnArgs (include/tri_attn.h) for one call, on torch's current stream of the query's device."""
    args = _lib.TriAttnArgs()
    num_batches, num_heads, y_size, x_size = query.shape
    _lib.ARGS_PACKER.pack_into(
        args, 0,
        _lib.ARGS_PACKER.size, util.dtype(query.dtype), num_batches, num_heads, y_size, x_size,
        1 if is_causal else 0, 0 if mask is None else util.dtype(mask.dtype), softmax_scale, dropout_p, seed, offset,
        query.data_ptr(), key.data_ptr(), value.data_ptr(), output.data_ptr(), log2sum.data_ptr(),
        0 if mask is None else mask.data_ptr(),
        0 if grad_output is None else grad_output.data_ptr(),
        0 if grad_query is None else grad_query.data_ptr(),
        0 if grad_key is None else grad_key.data_ptr(),
        0 if grad_value is None else grad_value.data_ptr(),
        0 if grad_mask is None else grad_mask.data_ptr(),
        0 if delta is None else delta.data_ptr(),
        *query.stride(), *key.stride(), *value.stride(), *output.stride(),
        *_strides_or_zero(grad_output), *_strides_or_zero(grad_query), *_strides_or_zero(grad_key),
        *_strides_or_zero(grad_value), *_strides_or_zero(mask), *_strides_or_zero(grad_mask),
        torch._C._cuda_getCurrentRawStream(query.device.index), 0,
    )
    return args


# Classes of a mask's 64 x 64 blocks (tri_attn_classify_mask), kept per mask tensor: the forward call computes them, the
# backward call and later calls with the same, unmodified tensor (other layers, other steps) find them here. An entry
# dies with its tensor (weak reference) and is recomputed when the tensor was written to through torch (its version
# counter moved), when another stream asks for it (no event orders the two), and it is neither made nor used while a
# stream is being captured (the classification would be recorded, not run). A write that torch does not see (through
# ``.data``, a raw pointer, a graph replay into the mask's memory) leaves stale classes behind, and the kernels skip
# tiles on their word: such callers set ``config.cache_mask_classes = False`` (every call classifies the mask again)
# or call ``forget_mask_classes()`` after the write.
_MASK_CLASSES = {}


def forget_mask_classes():
    """Drops every cached block classification (after a write to a mask's memory that torch's version counter did not see)."""
    _MASK_CLASSES.clear()


def _mask_classes(mask: torch.Tensor, args):
    """Sets args.mask_classes for the mask already described in ``args``; returns the tensor to keep alive, or None
    where the library has no use for classes (nothing is launched then)."""
    import weakref

    lib = _lib.lib()
    size = lib.tri_attn_mask_classes_size(ctypes.byref(args))
    if size <= 0:
        return None
    use_cache = config.cache_mask_classes and not torch.cuda.is_current_stream_capturing()
    key = id(mask)
    entry = _MASK_CLASSES.get(key) if use_cache else None
    signature = (mask._version, tuple(mask.shape), mask.stride(), mask.dtype, args.B, args.H, args.S, args.mask, args.stream)
    if entry is not None and entry[0]() is mask and entry[1] == signature:
        classes = entry[2]
    else:
        classes = torch.empty(size, dtype=torch.uint8, device=mask.device)
        args.mask_classes = classes.data_ptr()
        status = lib.tri_attn_classify_mask(ctypes.byref(args))
        if status in (_lib.ENOFUSE, _lib.EALIGN):
            args.mask_classes = None
            return None
        _lib.check(status)
        if use_cache:
            if len(_MASK_CLASSES) >= 64:
                _MASK_CLASSES.clear()
            _MASK_CLASSES[key] = (weakref.ref(mask, lambda _r, k=key: _MASK_CLASSES.pop(k, None)), signature, classes)
    args.mask_classes = classes.data_ptr()
    return classes


def _expand_mask(mask: torch.Tensor, shape):
    """View of the additive mask broadcast to [B,H,S,S] (stride 0 on broadcast dims)."""
    view = mask
    while view.dim() < 4:
        view = view.unsqueeze(0)
    view = view.expand(*shape)
    if view.shape[-1] != 1 and view.stride(-1) != 1:
        view = view.contiguous()
    return view


class _NoGraph:
    """Stands in for the autograd context when no gradient is asked for."""

    def save_for_backward(self, *tensors):
        pass


class Attention(torch.autograd.Function):
    @staticmethod
    def call(query, key, value, mask, dropout_p, is_causal, softmax_scale, use_accelerator):
        """``apply`` with the same arguments, checks and result; when no input asks for a gradient (or gradients are
        switched off) the forward runs without autograd's bookkeeping, which a small problem would feel."""
        if torch.is_grad_enabled() and (
            query.requires_grad or key.requires_grad or value.requires_grad or (mask is not None and mask.requires_grad)
        ):
            return Attention.apply(query, key, value, mask, dropout_p, is_causal, softmax_scale, use_accelerator)
        return Attention.forward(_NoGraph(), query, key, value, mask, dropout_p, is_causal, softmax_scale, use_accelerator)

    @staticmethod
    def forward(ctx: Any, *args: Any, **kwargs: Any):
        query, key, value, mask, dropout_p, is_causal, softmax_scale, use_accelerator = args

        if query.dim() != 4 or key.dim() != 4 or value.dim() != 4:
            raise ValueError("The dimension of query, key and value should be 4.")

        if (
            not util.is_pow2(query.shape[-1])
            or not util.is_pow2(key.shape[-1])
            or not util.is_pow2(value.shape[-1])
            or (
                config.reference_limits
                and (
                    not util.is_pow2(query.shape[-2])
                    or not util.is_pow2(key.shape[-2])
                    or not util.is_pow2(value.shape[-2])
                )
            )
        ):
            raise ValueError("Attention supports only for power of 2 size tensors.")

        if mask is not None:
            if is_causal:
                raise ValueError("Error because both attn_mask and is_causal are set.")
            if mask.dtype == torch.bool:
                if config.reference_limits:
                    raise ValueError("Boolean mask is not supported yet.")
                # torch's meaning of a boolean attn_mask: True = the key takes part in the attention (the additive
                # mask is made in the operand type: half the bytes of an fp32 one for the 16-bit kernels to stream)
                mask = torch.zeros(mask.shape, dtype=query.dtype, device=mask.device).masked_fill_(~mask, float("-inf"))

        seed, offset = _next_seed() if dropout_p > 0.0 else (0, 0)

        util.push_trace("Attention.__forward")
        output, log_sum_exp = Attention._forward(
            query, key, value, mask, dropout_p, is_causal, softmax_scale, seed, offset
        )
        util.pop_trace()

        ctx.save_for_backward(query, key, value, output, log_sum_exp)
        ctx.mask = mask
        ctx.dropout_p = dropout_p
        ctx.is_causal = is_causal
        ctx.softmax_scale = softmax_scale
        ctx.use_accelerator = use_accelerator
        ctx.seed = seed
        ctx.offset = offset

        return output

    @staticmethod
    def backward(ctx: Any, *grad_outputs: Any):
        (grad_output,) = grad_outputs
        query, key, value, output, log_sum_exp = ctx.saved_tensors

        util.push_trace("Attention.__backward")
        grad_query, grad_key, grad_value, grad_mask = Attention._backward(
            grad_output,
            query,
            key,
            value,
            output,
            log_sum_exp,
            ctx.mask,
            ctx.softmax_scale,
            ctx.dropout_p,
            ctx.is_causal,
            ctx.seed,
            ctx.offset,
            ctx.mask is not None and ctx.needs_input_grad[3],
        )
        util.pop_trace()

        return grad_query, grad_key, grad_value, grad_mask, None, None, None, None

    @staticmethod
    def _forward(query, key, value, mask, dropout_p, is_causal, softmax_scale, seed, offset):
        assert query.shape[-1] == key.shape[-1] and key.shape[-1] == value.shape[-1]
        assert key.shape[-1] in {16, 32, 64, 128}
        _require_same_gpu(query.device, key=key, value=value, mask=mask)
        if key.shape != query.shape or value.shape != query.shape:
            raise ValueError("query, key and value must have the same shape.")
        if key.dtype != query.dtype or value.dtype != query.dtype:
            raise ValueError("query, key and value must have the same dtype.")

        lib = _lib.lib()
        query, key, value = _dense_rows(query), _dense_rows(key), _dense_rows(value)
        num_batches, num_heads, y_size, x_size = query.shape
        output = torch.empty(query.shape, device=query.device, dtype=query.dtype)
        log2sum = torch.empty(num_batches, num_heads, y_size, device=query.device, dtype=torch.float32)
        mask_view = _expand_mask(mask.detach(), (num_batches, num_heads, y_size, y_size)) if mask is not None else None

        args = _make_args(query, key, value, output, log2sum, mask_view, dropout_p, is_causal, softmax_scale, seed, offset)
        classes = _mask_classes(mask, args) if mask is not None else None  # (kept alive until the call is enqueued)

        util.push_trace("kernel.Attention.forward")
        _lib.check(lib.tri_attn_fwd(ctypes.byref(args)))
        util.pop_trace()

        return output, log2sum

    @staticmethod
    def _backward(grad_output, query, key, value, output, log2sum, mask, softmax_scale, dropout_p, is_causal,
                  seed, offset, want_grad_mask, delta_out=None):
        """``delta_out``: optional fp32 [B,H,S] tensor that receives delta (the backward's intermediate,
        trident/operation/attention.py:155); allocated here when not given."""
        _require_same_gpu(query.device, key=key, value=value, mask=mask, grad_output=grad_output, output=output,
                          log_sum_exp=log2sum)
        lib = _lib.lib()
        query, key, value = _dense_rows(query), _dense_rows(key), _dense_rows(value)
        grad_output = _dense_rows(grad_output)
        num_batches, num_heads, y_size, x_size = output.shape
        grad_query = torch.empty(query.shape, device=query.device, dtype=query.dtype)
        grad_key = torch.empty(key.shape, device=key.device, dtype=key.dtype)
        grad_value = torch.empty(value.shape, device=value.device, dtype=value.dtype)
        delta = torch.empty_like(log2sum) if delta_out is None else delta_out
        full = (num_batches, num_heads, y_size, y_size)
        mask_view = _expand_mask(mask.detach(), full) if mask is not None else None
        # The mask gradient (trident/kernel/attention.py:332-335) in the mask's own shape: a full [B,H,S,S] mask gets
        # dS written in place; a broadcast mask gets a zero-filled fp32 buffer of its shape that the kernels add to
        # through strides of 0 (autograd's sum over the broadcast dimensions, without a [B,H,S,S] intermediate).
        grad_mask_buf = grad_mask_view = None
        if want_grad_mask:
            shape4 = (1,) * (4 - mask.dim()) + tuple(mask.shape)
            if shape4 == full:
                grad_mask_buf = torch.empty(full, device=mask.device, dtype=mask.dtype)
                grad_mask_view = grad_mask_buf
            else:
                grad_mask_buf = torch.zeros(shape4, device=mask.device, dtype=torch.float32)
                grad_mask_view = grad_mask_buf.expand(*full)
                if mask_view.dtype != torch.float32:  # (mask and dmask share one dtype field)
                    mask_view = _expand_mask(mask.detach().float(), full)

        args = _make_args(query, key, value, output, log2sum, mask_view, dropout_p, is_causal, softmax_scale, seed, offset,
                          grad_output, grad_query, grad_key, grad_value, grad_mask_view, delta)
        # (the classes describe the mask tensor as the kernels see it: not when it was converted to fp32 above)
        classes = _mask_classes(mask, args) if mask is not None and mask_view.dtype == mask.dtype else None

        # one call for the three backward launches (trident/operation/attention.py:161-199 launches the
        # delta pre-pass and the backward kernel): the library orders them, and where the dQ kernel can
        # compute delta on its way the pre-pass disappears into it
        util.push_trace("kernel.Attention.backward")
        _lib.check(lib.tri_attn_bwd(ctypes.byref(args)))
        util.pop_trace()

        grad_mask = None
        if grad_mask_buf is not None:
            grad_mask = grad_mask_buf.to(mask.dtype).reshape(mask.shape)

        return grad_query, grad_key, grad_value, grad_mask


from .rowops import Dropout, MaskedSoftmax, Softmax  # noqa: E402,F401  (trident.operation.Softmax etc.)
