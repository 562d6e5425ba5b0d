"""Softmax, MaskedSoftmax and Dropout autograd Functions behind the reference's operator API.

Mirror trident/operation/softmax.py:23-110, trident/operation/masked_softmax.py:23-116 and
trident/operation/dropout.py:23-79: the same positional arguments, the same saved state, the same
tuples returned by backward. The Triton launches become calls into libtrident_attn.so
(include/tri_rowops.h); the two backward launches of the softmax operations (delta, then the gradient)
are one call here.
"""
import ctypes
from typing import Any

import torch

from . import _lib, config, util

_MASK_CODES = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2, torch.int64: 3, torch.int32: 4,
               torch.uint8: 5, torch.bool: 5}


def size_and_stride(input: torch.Tensor, dim: int):
    """(y_size, x_size, y_stride, x_stride) with the operation running along x
    (trident/util/util.py:65-76 for 2-D tensors; a contiguous tensor of any rank is also taken
    along its last dimension)."""
    if input.dim() == 2:
        if dim == 0:
            x_size, y_size = input.shape
            return y_size, x_size, input.stride(1), input.stride(0)
        y_size, x_size = input.shape
        return y_size, x_size, input.stride(0), input.stride(1)
    if input.dim() >= 1 and dim in (-1, input.dim() - 1) and input.is_contiguous():
        x_size = input.shape[-1]
        return input.numel() // max(x_size, 1), x_size, x_size, 1
    raise ValueError(f"{dim} is not supported.")


def _require_gpu(input, **others):
    if input.device.type != "cuda":
        raise RuntimeError("trident_amd runs on the GPU only; got a tensor on " + str(input.device))
    for name, t in others.items():
        if t is not None and t.device != input.device:
            raise RuntimeError(f"trident_amd: {name} is on {t.device}, expected {input.device}")


def _same_layout(t: torch.Tensor, like: torch.Tensor):
    """The kernels address every tensor of a call with one stride pair (trident/kernel/softmax.py:41-44)."""
    if t.shape == like.shape and t.stride() == like.stride():
        return t
    out = torch.empty_strided(like.shape, like.stride(), dtype=t.dtype, device=t.device)
    out.copy_(t.expand(like.shape))
    return out


def _row_args(input, dim):
    args = _lib.TriRowArgs()
    args.struct_size = ctypes.sizeof(_lib.TriRowArgs)
    args.dtype = util.dtype(input.dtype)
    args.y_size, args.x_size, args.y_stride, args.x_stride = size_and_stride(input, dim)
    args.stream = torch.cuda.current_stream(input.device).cuda_stream
    return args


def _dense(input):
    """Strides the kernels can address: non-overlapping and non-negative (anything else is copied)."""
    if input.is_contiguous() or (input.dim() == 2 and input.t().is_contiguous()):
        return input
    return input.contiguous()


def _softmax_forward(input, mask, dim, trace):
    _require_gpu(input, mask=mask)
    input = _dense(input)
    output = torch.empty_like(input)  # (preserves the strides of a dense input)
    args = _row_args(input, dim)
    args.input, args.output = input.data_ptr(), output.data_ptr()
    if mask is not None:
        if mask.dtype not in _MASK_CODES:
            raise ValueError(f"Unable to convert the given input: '{mask.dtype}'.")
        mask = _same_layout(mask, input)
        args.mask, args.mask_dtype = mask.data_ptr(), _MASK_CODES[mask.dtype]
    util.push_trace(trace)
    _lib.check(_lib.lib().tri_softmax_fwd(ctypes.byref(args)))
    util.pop_trace()
    return output


def _softmax_backward(grad_output, output, dim, trace):
    _require_gpu(output, grad_output=grad_output)
    grad_output = _same_layout(grad_output, output)
    grad_input = torch.empty_like(output)
    args = _row_args(output, dim)
    args.output, args.grad_output, args.grad_input = output.data_ptr(), grad_output.data_ptr(), grad_input.data_ptr()
    util.push_trace(trace)
    _lib.check(_lib.lib().tri_softmax_bwd(ctypes.byref(args)))
    util.pop_trace()
    return grad_input


class Softmax(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, *args: Any, **kwargs: Any):
        input, dim = args

        util.push_trace("Softmax.__forward")
        output = _softmax_forward(input, None, dim, "kernel.Softmax.forward")
        util.pop_trace()

        ctx.save_for_backward(output)
        ctx.dim = dim

        return output

    @staticmethod
    def backward(ctx: Any, *grad_outputs: Any):
        (grad_output,) = grad_outputs
        (output,) = ctx.saved_tensors

        util.push_trace("Softmax.__backward")
        grad_input = _softmax_backward(grad_output, output, ctx.dim, "kernel.Softmax.backward")
        util.pop_trace()

        return grad_input, None


class MaskedSoftmax(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, *args: Any, **kwargs: Any):
        input, mask, dim = args

        util.push_trace("MaskedSoftmax.__forward")
        output = _softmax_forward(input, mask, dim, "kernel.MaskedSoftmax.forward")
        util.pop_trace()

        ctx.save_for_backward(output)
        ctx.dim = dim

        return output

    @staticmethod
    def backward(ctx: Any, *grad_outputs: Any):
        (grad_output,) = grad_outputs
        (output,) = ctx.saved_tensors

        util.push_trace("MaskedSoftmax.__backward")
        grad_input = _softmax_backward(grad_output, output, ctx.dim, "kernel.MaskedSoftmax.backward")
        util.pop_trace()

        return grad_input, None, None


def _next_seed():
    from .operation import _next_seed as attention_seed

    return attention_seed()


class Dropout(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, *args: Any, **kwargs: Any):
        input, p = args

        util.push_trace("Dropout.__forward")
        seed, offset = _next_seed()
        output = Dropout._launch(input, p, seed, offset, False)
        util.pop_trace()

        # the keep decisions are regenerated from (seed, offset, p) in backward: no tensor is saved
        # (the reference saves input and output and tests output > 0, trident/operation/dropout.py:33,
        # trident/kernel/dropout.py:128)
        ctx.p = p
        ctx.seed = seed
        ctx.offset = offset

        return output

    @staticmethod
    def backward(ctx: Any, *grad_outputs: Any):
        (grad_output,) = grad_outputs

        util.push_trace("Dropout.__backward")
        grad_input = Dropout._launch(grad_output, ctx.p, ctx.seed, ctx.offset, True)
        util.pop_trace()

        return grad_input, None

    @staticmethod
    def _launch(source, p, seed, offset, backward):
        _require_gpu(source)
        source = source.contiguous()
        result = torch.empty_like(source)
        args = _lib.TriRowArgs()
        args.struct_size = ctypes.sizeof(_lib.TriRowArgs)
        args.dtype = util.dtype(source.dtype)
        args.y_size, args.x_size = 1, source.numel()
        args.p = float(p)
        args.seed, args.offset = seed, offset
        args.stream = torch.cuda.current_stream(source.device).cuda_stream
        if source.numel() == 0:
            return result
        lib = _lib.lib()
        if backward:
            args.grad_output, args.grad_input = source.data_ptr(), result.data_ptr()
            util.push_trace("kernel.Dropout.backward")
            _lib.check(lib.tri_dropout_bwd(ctypes.byref(args)))
        else:
            args.input, args.output = source.data_ptr(), result.data_ptr()
            util.push_trace("kernel.Dropout.forward")
            _lib.check(lib.tri_dropout_fwd(ctypes.byref(args)))
        util.pop_trace()
        return result
