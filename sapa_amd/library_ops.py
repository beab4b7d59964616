"""The operators as `torch.library` custom ops, so that `torch.compile` and
`torch.export` trace through them without graph breaks.

    import sapa_amd.library_ops            # registers torch.ops.sapa_amd.*
    torch.ops.sapa_amd.qk(query, key, 5, 2)
    torch.ops.sapa_amd.sapa_fused(query, key, value, 5, 2)

Each forward op has a shape-only ("fake") implementation and an autograd
formula whose backward is itself a registered op, so forward and backward
graphs both consist of opaque `sapa_amd::*` nodes.  The eager entry points of
`sapa_amd` (qk, av, ... -- the reference's autograd.Function API,
sapa/sapa/sapa_func.py:51,96 and deformsapa/deformsapa/deform_func.py:59,114)
stay as they are; these ops call the same library functions.
"""
from typing import Tuple

import torch
from torch import Tensor
from torch.library import custom_op

from . import deform_func as _d
from . import sapa_func as _b

_NS = 'sapa_amd'


def _hi(t, s):
    return t.shape[2] * s, t.shape[3] * s


def _new_out(like, shape, *inputs):
    """Shape-only result of a SAPA-B forward op: in torch.channels_last order
    when every input is (the eager kernels serve that order without a copy and
    answer in it), contiguous otherwise."""
    cl = (not all(t.is_contiguous() for t in inputs)
          and all(t.dim() == 4 and t.is_contiguous(memory_format=torch.channels_last)
                  for t in inputs))
    return torch.empty(tuple(shape), dtype=like.dtype, device=like.device,
                       memory_format=torch.channels_last if cl else torch.contiguous_format)


def _new_grad(t):
    # a gradient comes back in the order of the tensor it belongs to (the kernels work in
    # contiguous order; channels-last operands and results are transposed around them)
    cl = t.dim() == 4 and not t.is_contiguous() and t.is_contiguous(memory_format=torch.channels_last)
    return torch.empty(t.shape, dtype=t.dtype, device=t.device,
                       memory_format=torch.channels_last if cl else torch.contiguous_format)


# ------------------------------------------------------------------ SAPA-B
@custom_op(f'{_NS}::qk', mutates_args=())
def qk(query: Tensor, key: Tensor, kernel_size: int, scale_factor: int) -> Tensor:
    with torch.no_grad():
        return _b.QKFunction.apply(query, key, kernel_size, scale_factor)


@qk.register_fake
def _(query, key, kernel_size, scale_factor):
    return _new_out(key, (key.shape[0], kernel_size ** 2) + _hi(key, scale_factor), query, key)


@custom_op(f'{_NS}::qk_backward', mutates_args=())
def qk_backward(grad_output: Tensor, query: Tensor, key: Tensor, kernel_size: int,
                scale_factor: int) -> Tuple[Tensor, Tensor]:
    return _b._qk_backward(grad_output, query, key, kernel_size, scale_factor)


@qk_backward.register_fake
def _(grad_output, query, key, kernel_size, scale_factor):
    return _new_grad(query), _new_grad(key)


def _qk_setup(ctx, inputs, output):
    query, key, ctx.kernel_size, ctx.scale_factor = inputs
    ctx.save_for_backward(query, key)


def _qk_grad(ctx, grad_output):
    query, key = ctx.saved_tensors
    gq, gk = qk_backward(grad_output, query, key, ctx.kernel_size, ctx.scale_factor)
    return gq, gk, None, None


qk.register_autograd(_qk_grad, setup_context=_qk_setup)


@custom_op(f'{_NS}::av', mutates_args=())
def av(attn: Tensor, value: Tensor, kernel_size: int, scale_factor: int) -> Tensor:
    with torch.no_grad():
        return _b.AVFunction.apply(attn, value, kernel_size, scale_factor)


@av.register_fake
def _(attn, value, kernel_size, scale_factor):
    return _new_out(value, value.shape[:2] + _hi(value, scale_factor), attn, value)


@custom_op(f'{_NS}::av_backward', mutates_args=())
def av_backward(grad_output: Tensor, attn: Tensor, value: Tensor, kernel_size: int,
                scale_factor: int) -> Tuple[Tensor, Tensor]:
    return _b._av_backward(grad_output, attn, value, kernel_size, scale_factor)


@av_backward.register_fake
def _(grad_output, attn, value, kernel_size, scale_factor):
    return _new_grad(attn), _new_grad(value)


def _av_setup(ctx, inputs, output):
    attn, value, ctx.kernel_size, ctx.scale_factor = inputs
    ctx.save_for_backward(attn, value)


def _av_grad(ctx, grad_output):
    attn, value = ctx.saved_tensors
    ga, gv = av_backward(grad_output, attn, value, ctx.kernel_size, ctx.scale_factor)
    return ga, gv, None, None


av.register_autograd(_av_grad, setup_context=_av_setup)


@custom_op(f'{_NS}::sapa_fused', mutates_args=())
def sapa_fused(query: Tensor, key: Tensor, value: Tensor, kernel_size: int,
               scale_factor: int) -> Tensor:
    with torch.no_grad():
        return _b.SAPAFusedFunction.apply(query, key, value, kernel_size, scale_factor)


@sapa_fused.register_fake
def _(query, key, value, kernel_size, scale_factor):
    return _new_out(value, value.shape[:2] + _hi(value, scale_factor), query, key, value)


@custom_op(f'{_NS}::sapa_fused_backward', mutates_args=())
def sapa_fused_backward(grad_output: Tensor, query: Tensor, key: Tensor, value: Tensor,
                        kernel_size: int, scale_factor: int) -> Tuple[Tensor, Tensor, Tensor]:
    return _b._fused_backward(grad_output, query, key, value, kernel_size, scale_factor)


@sapa_fused_backward.register_fake
def _(grad_output, query, key, value, kernel_size, scale_factor):
    return _new_grad(query), _new_grad(key), _new_grad(value)


def _fused_setup(ctx, inputs, output):
    query, key, value, ctx.kernel_size, ctx.scale_factor = inputs
    ctx.save_for_backward(query, key, value)


def _fused_grad(ctx, grad_output):
    query, key, value = ctx.saved_tensors
    gq, gk, gv = sapa_fused_backward(grad_output, query, key, value,
                                     ctx.kernel_size, ctx.scale_factor)
    return gq, gk, gv, None, None


sapa_fused.register_autograd(_fused_grad, setup_context=_fused_setup)


# ------------------------------------------------------------------ SAPA-D
@custom_op(f'{_NS}::deform_qk', mutates_args=())
def deform_qk(query: Tensor, key: Tensor, offset: Tensor, num_point: int, scale_factor: int,
              groups: int) -> Tensor:
    with torch.no_grad():
        return _d.DeformQKFunction.apply(query, key, offset, num_point, scale_factor, groups)


@deform_qk.register_fake
def _(query, key, offset, num_point, scale_factor, groups):
    return query.new_empty((query.shape[0], groups, num_point) + tuple(query.shape[2:]))


@custom_op(f'{_NS}::deform_qk_backward', mutates_args=())
def deform_qk_backward(grad_output: Tensor, query: Tensor, key: Tensor, offset: Tensor,
                       num_point: int, scale_factor: int,
                       groups: int) -> Tuple[Tensor, Tensor, Tensor]:
    return _d._deform_qk_backward(grad_output, query, key, offset, num_point, scale_factor, groups)


@deform_qk_backward.register_fake
def _(grad_output, query, key, offset, num_point, scale_factor, groups):
    return torch.empty_like(query), torch.empty_like(key), torch.empty_like(offset)


def _dqk_setup(ctx, inputs, output):
    query, key, offset, ctx.num_point, ctx.scale_factor, ctx.groups = inputs
    ctx.save_for_backward(query, key, offset)


def _dqk_grad(ctx, grad_output):
    query, key, offset = ctx.saved_tensors
    gq, gk, go = deform_qk_backward(grad_output.contiguous(), query, key, offset, ctx.num_point,
                                    ctx.scale_factor, ctx.groups)
    return gq, gk, go, None, None, None


deform_qk.register_autograd(_dqk_grad, setup_context=_dqk_setup)


@custom_op(f'{_NS}::deform_av', mutates_args=())
def deform_av(attn: Tensor, value: Tensor, offset: Tensor, num_point: int, scale_factor: int,
              groups: int) -> Tensor:
    with torch.no_grad():
        return _d.DeformAVFunction.apply(attn, value, offset, num_point, scale_factor, groups)


@deform_av.register_fake
def _(attn, value, offset, num_point, scale_factor, groups):
    return value.new_empty(value.shape[:2] + _hi(value, scale_factor))


@custom_op(f'{_NS}::deform_av_backward', mutates_args=())
def deform_av_backward(grad_output: Tensor, attn: Tensor, value: Tensor, offset: Tensor,
                       num_point: int, scale_factor: int,
                       groups: int) -> Tuple[Tensor, Tensor, Tensor]:
    return _d._deform_av_backward(grad_output, attn, value, offset, num_point, scale_factor,
                                  groups)


@deform_av_backward.register_fake
def _(grad_output, attn, value, offset, num_point, scale_factor, groups):
    return torch.empty_like(attn), torch.empty_like(value), torch.empty_like(offset)


def _dav_setup(ctx, inputs, output):
    attn, value, offset, ctx.num_point, ctx.scale_factor, ctx.groups = inputs
    ctx.save_for_backward(attn, value, offset)


def _dav_grad(ctx, grad_output):
    attn, value, offset = ctx.saved_tensors
    ga, gv, go = deform_av_backward(grad_output.contiguous(), attn, value, offset, ctx.num_point,
                                    ctx.scale_factor, ctx.groups)
    return ga, gv, go, None, None, None


deform_av.register_autograd(_dav_grad, setup_context=_dav_setup)


@custom_op(f'{_NS}::deform_sapa_fused', mutates_args=())
def deform_sapa_fused(query: Tensor, key: Tensor, value: Tensor, offset: Tensor, num_point: int,
                      scale_factor: int, groups: int, offset_layout: str = 'hires') -> Tensor:
    with torch.no_grad():
        return _d.DeformSAPAFusedFunction.apply(query, key, value, offset, num_point,
                                                scale_factor, groups, offset_layout)


@deform_sapa_fused.register_fake
def _(query, key, value, offset, num_point, scale_factor, groups, offset_layout='hires'):
    return _new_out(value, value.shape[:2] + _hi(value, scale_factor), query, key, value, offset)


@custom_op(f'{_NS}::deform_sapa_fused_backward', mutates_args=())
def deform_sapa_fused_backward(grad_output: Tensor, query: Tensor, key: Tensor, value: Tensor,
                               offset: Tensor, num_point: int, scale_factor: int, groups: int,
                               offset_layout: str) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    return _d._deform_fused_backward(grad_output, query, key, value, offset, num_point,
                                     scale_factor, groups, offset_layout)


@deform_sapa_fused_backward.register_fake
def _(grad_output, query, key, value, offset, num_point, scale_factor, groups, offset_layout):
    return _new_grad(query), _new_grad(key), _new_grad(value), _new_grad(offset)


def _dfused_setup(ctx, inputs, output):
    (query, key, value, offset, ctx.num_point, ctx.scale_factor, ctx.groups,
     ctx.offset_layout) = inputs
    ctx.save_for_backward(query, key, value, offset)


def _dfused_grad(ctx, grad_output):
    query, key, value, offset = ctx.saved_tensors
    gq, gk, gv, go = deform_sapa_fused_backward(
        grad_output, query, key, value, offset, ctx.num_point, ctx.scale_factor,
        ctx.groups, ctx.offset_layout)
    return gq, gk, gv, go, None, None, None, None


deform_sapa_fused.register_autograd(_dfused_grad, setup_context=_dfused_setup)

__all__ = ['qk', 'av', 'sapa_fused', 'deform_qk', 'deform_av', 'deform_sapa_fused',
           'qk_backward', 'av_backward', 'sapa_fused_backward', 'deform_qk_backward',
           'deform_av_backward', 'deform_sapa_fused_backward']
