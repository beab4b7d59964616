"""SAPA-D operators: autograd API of the reference on top of libsapa_hip.so.

Mirrors deformsapa/deformsapa/deform_func.py of the reference
(DeformQKFunction :7-59, DeformAVFunction :62-114): same names, argument
order, assertions, output allocation and error behaviour, so
`from deformsapa import deform_qk, deform_av` callers such as
SAPADeform.attention (sapa_deform.py:51-53) run unchanged.
`deform_sapa_fused` is an addition.
"""
import torch
import torch.nn.functional as F
from torch.autograd import Function

from . import _lib


def _compute_dtype(t):
    # 16-bit tensors that the native 16-bit backward entry points do not serve
    # (_backward_16bit) take the fp32 kernels and the gradients are rounded back
    return t.dtype if t.dtype in (torch.float32, torch.float64) else torch.float32


def _backward_16bit(entry, grad_output, a, low, offset, P, s, G, needs):
    """The gradients of one sampled operator on f16 / bf16 tensors as they are
    (sapa_deform_{qk,av}_backward_ws); None where that path does not serve the
    configuration.  a: query (deform_qk) or attn (deform_av); low: key or value."""
    if low.dtype not in (torch.float16, torch.bfloat16):
        return None
    go, a, low, off = (_lib.layout_copy(t, False) for t in (grad_output, a, low, offset))
    _lib.require_cuda_contiguous(grad_output=go, a=a, low=low, offset=off)
    n, c, h, w = low.size()
    nbytes = _lib.lib().sapa_deform_backward_workspace(n, c, h, w, P, s, G, _lib.dtype_code(low))
    if nbytes <= 0:
        return None
    ws = torch.empty(nbytes, dtype=torch.uint8, device=low.device)
    grads = [_lib.new_out(t) if need else None for t, need in ((a, needs[0]), (low, needs[1]), (off, needs[2]))]
    status = _lib.call_status(entry, low.device, _lib.ptr(go), _lib.ptr(a), _lib.ptr(low), _lib.ptr(off),
                              _lib.ptr(ws), _lib.ptr(grads[0]), _lib.ptr(grads[1]), _lib.ptr(grads[2]),
                              n, c, h, w, P, s, G, _lib.dtype_code(low))
    return None if status == _lib.UNSUPPORTED else tuple(grads)


def _deform_qk_backward(grad_output, query, key, offset, P, s, G, needs=(True, True, True)):
    native = _backward_16bit('sapa_deform_qk_backward_ws', grad_output, query, key, offset, P, s, G, needs)
    if native is not None:
        return native
    cdt = _compute_dtype(query)
    go, q, k, off = (_lib.layout_copy(t, False).to(cdt) for t in (grad_output, query, key, offset))
    gq = _lib.new_out(q) if needs[0] else None
    gk = torch.zeros_like(k) if needs[1] else None
    goff = _lib.new_out(off) if needs[2] else None
    _lib.require_cuda_contiguous(grad_output=go, query=q, key=k, offset=off)
    n, c, h, w = k.size()
    _lib.call('sapa_deform_qk_backward', k.device, _lib.ptr(go), _lib.ptr(q), _lib.ptr(k),
              _lib.ptr(off), _lib.ptr(gq), _lib.ptr(gk), _lib.ptr(goff), n, c, h, w, P, s, G,
              _lib.dtype_code(k))
    return tuple(None if g is None else g.to(t.dtype)
                 for g, t in ((gq, query), (gk, key), (goff, offset)))


def _deform_av_backward(grad_output, attn, value, offset, P, s, G, needs=(True, True, True)):
    native = _backward_16bit('sapa_deform_av_backward_ws', grad_output, attn, value, offset, P, s, G, needs)
    if native is not None:
        return native
    cdt = _compute_dtype(value)
    go, a, v, off = (_lib.layout_copy(t, False).to(cdt) for t in (grad_output, attn, value, offset))
    ga = _lib.new_out(a) if needs[0] else None
    gv = torch.zeros_like(v) if needs[1] else None
    goff = _lib.new_out(off) if needs[2] else None
    _lib.require_cuda_contiguous(grad_output=go, attn=a, value=v, offset=off)
    n, c, h, w = v.size()
    _lib.call('sapa_deform_av_backward', v.device, _lib.ptr(go), _lib.ptr(a), _lib.ptr(v),
              _lib.ptr(off), _lib.ptr(ga), _lib.ptr(gv), _lib.ptr(goff), n, c, h, w, P, s, G,
              _lib.dtype_code(v))
    return tuple(None if g is None else g.to(t.dtype)
                 for g, t in ((ga, attn), (gv, value), (goff, offset)))


class DeformQKFunction(Function):

    @staticmethod
    def forward(ctx, query, key, offset, num_point, scale_factor, groups):
        assert scale_factor >= 1
        assert query.size(0) == key.size(0)
        assert query.size(1) == key.size(1)
        assert query.size(2) == key.size(2) * scale_factor
        assert query.size(3) == key.size(3) * scale_factor
        assert offset.size(0) == key.size(0)
        assert offset.size(1) == groups * num_point * 2
        assert offset.size(2) == key.size(2) * scale_factor
        assert offset.size(3) == key.size(3) * scale_factor
        assert query.size(1) % groups == 0
        assert num_point >= 1
        ctx.num_point = num_point
        ctx.scale_factor = scale_factor
        ctx.groups = groups
        ctx.query_size = query.size()
        ctx.key_size = key.size()
        ctx.offset_size = offset.size()

        n, c, h, w = query.size()
        output = _lib.new_out(query, (n, groups, num_point, h, w))
        if query.is_cuda:
            _lib.require_cuda_contiguous(query=query, key=key, offset=offset)
            _lib.call('sapa_deform_qk_forward', query.device, _lib.ptr(query), _lib.ptr(key),
                      _lib.ptr(offset), _lib.ptr(output), n, c, key.size(2), key.size(3),
                      num_point, scale_factor, groups, _lib.dtype_code(query))
        else:
            raise NotImplementedError

        if query.requires_grad or key.requires_grad or offset.requires_grad:
            ctx.save_for_backward(query, key, offset)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        assert grad_output.is_cuda
        query, key, offset = ctx.saved_tensors
        gq, gk, goff = _deform_qk_backward(grad_output, query, key, offset, ctx.num_point,
                                           ctx.scale_factor, ctx.groups)
        return gq, gk, goff, None, None, None


deform_qk = DeformQKFunction.apply


class DeformAVFunction(Function):

    @staticmethod
    def forward(ctx, attn, value, offset, num_point, scale_factor, groups):
        assert scale_factor >= 1
        assert attn.size(0) == value.size(0)
        assert attn.size(1) == groups
        assert attn.size(2) == num_point
        assert attn.size(3) == value.size(2) * scale_factor
        assert attn.size(4) == value.size(3) * scale_factor
        assert offset.size(0) == value.size(0)
        assert offset.size(1) == groups * num_point * 2
        assert offset.size(2) == value.size(2) * scale_factor
        assert offset.size(3) == value.size(3) * scale_factor
        assert value.size(1) % groups == 0
        assert num_point >= 1
        ctx.num_point = num_point
        ctx.scale_factor = scale_factor
        ctx.groups = groups
        ctx.attn_size = attn.size()
        ctx.value_size = value.size()
        ctx.offset_size = offset.size()

        n, c, h, w = value.size()
        output = _lib.new_out(value, (n, c, scale_factor * h, scale_factor * w))
        if attn.is_cuda:
            _lib.require_cuda_contiguous(attn=attn, value=value, offset=offset)
            _lib.call('sapa_deform_av_forward', value.device, _lib.ptr(attn), _lib.ptr(value),
                      _lib.ptr(offset), _lib.ptr(output), n, c, h, w, num_point, scale_factor,
                      groups, _lib.dtype_code(value))
        else:
            raise NotImplementedError

        if attn.requires_grad or value.requires_grad or offset.requires_grad:
            ctx.save_for_backward(attn, value, offset)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        assert grad_output.is_cuda
        attn, value, offset = ctx.saved_tensors
        ga, gv, goff = _deform_av_backward(grad_output, attn, value, offset, ctx.num_point,
                                           ctx.scale_factor, ctx.groups)
        return ga, gv, goff, None, None, None


deform_av = DeformAVFunction.apply


OFFSET_LAYOUTS = {'hires': 0, 'pixel_shuffle': 1, 'nearest': 2}


def expand_offset(offset, scale_factor, layout):
    """The hi-res offset tensor [B, 2GP, sH, sW] that a low-res offset tensor
    in `layout` stands for (sapa_deform.py:44-47)."""
    if layout == 'hires':
        return offset
    if layout == 'pixel_shuffle':
        return F.pixel_shuffle(offset, scale_factor)
    if layout == 'nearest':
        return F.interpolate(offset, scale_factor=scale_factor)
    raise ValueError('offset_layout must be one of %s' % sorted(OFFSET_LAYOUTS))


def _reduce_offset_grad(grad_hi, scale_factor, layout):
    # adjoint of expand_offset
    if layout == 'hires':
        return grad_hi
    if layout == 'pixel_shuffle':
        return F.pixel_unshuffle(grad_hi, scale_factor)
    b, c, hh, hw = grad_hi.shape
    s = scale_factor
    return grad_hi.view(b, c, hh // s, s, hw // s, s).sum(dim=(3, 5))


def _native_fused_backward(grad_output, query, key, value, offset, P, s, G, needs):
    """sapa_deform_fused_backward on contiguous tensors with hi-res offsets: the whole
    chain in one call, fp32 [B,G,P,sH,sW] intermediates in a workspace, 16-bit tensors
    read and written as they are.  None where the entry point does not serve the
    configuration (fp64, up_factor 3, many points)."""
    n, c, h, w = value.size()
    shape = (n, key.size(1), c, h, w, P, s, G, _lib.dtype_code(value))
    nbytes = _lib.lib().sapa_deform_fused_backward_workspace(*shape)
    if nbytes == 0 or not all(t.dtype == value.dtype for t in (grad_output, query, key, offset)):
        return None
    ws = torch.empty(nbytes, dtype=torch.uint8, device=value.device)
    grads = [_lib.new_out(t) if need else None
             for t, need in zip((query, key, value, offset), needs)]
    _lib.call('sapa_deform_fused_backward', value.device, _lib.ptr(grad_output), _lib.ptr(query),
              _lib.ptr(key), _lib.ptr(value), _lib.ptr(offset), _lib.ptr(ws),
              *(_lib.ptr(g) if g is not None else None for g in grads), *shape)
    return grads


def _deform_fused_backward(grad_output, query, key, value, offset, P, s, G, offset_layout,
                           needs=(True, True, True, True)):
    """Gradients of deform_av(softmax(deform_qk(q, k, off), dim=2), v, off)
    with respect to q, k, v and the offset tensor in its own layout."""
    with torch.no_grad():
        # the gradient kernels take contiguous tensors: operands kept in channels-last order
        # are transposed here by the library's layout kernel, and each gradient goes back in
        # the order of the tensor it belongs to
        cl = [_lib.is_channels_last(t) for t in (query, key, value, offset)]

        def back(g, i):
            return g if g is None or not cl[i] else _lib.layout_copy(g, True)
        query, key, value = (_lib.layout_copy(t, False) for t in (query, key, value))
        grad_output = _lib.layout_copy(grad_output, False)
        offset = _lib.layout_copy(expand_offset(offset, s, offset_layout), False)
        native = _native_fused_backward(grad_output, query, key, value, offset, P, s, G, needs)
        if native is not None:
            gq, gk, gv, goff = native
            if goff is not None:
                goff = _reduce_offset_grad(goff, s, offset_layout)
            return back(gq, 0), back(gk, 1), back(gv, 2), back(goff, 3)
        # 16-bit tensors: the logits are recomputed from fp32 copies so that, like
        # the forward kernel's, they are not rounded to 16 bits before the softmax
        wide = _compute_dtype(query)
        logits = DeformQKFunction.apply(query.to(wide), key.to(wide), offset.to(wide), P, s, G)
        attn = torch.softmax(logits, dim=2).to(query.dtype)
        ga, gv, goff_av = _deform_av_backward(grad_output, attn, value, offset, P, s, G)
        a32, g32 = attn.float(), ga.float()
        grad_logits = (a32 * (g32 - (g32 * a32).sum(dim=2, keepdim=True))).to(attn.dtype)
        gq, gk, goff_qk = _deform_qk_backward(grad_logits, query, key, offset, P, s, G)
        goff = _reduce_offset_grad(goff_av + goff_qk, s, offset_layout)
    return back(gq, 0), back(gk, 1), back(gv, 2), back(goff, 3)


class DeformSAPAFusedFunction(Function):
    """deform_av(softmax(deform_qk(query, key, offset), dim=2), value, offset)
    -- SAPADeform.attention (sapa_deform.py:51-53) -- as one launch in the
    forward pass; the backward pass recomputes the weights and chains the
    three operators' gradients (the offset receives both paths' gradients).

    `offset_layout` 'pixel_shuffle' / 'nearest' takes the low-res output of the
    offset convolution itself ([B, 2GP*s*s, H, W] / [B, 2GP, H, W]) and reads it
    in place, so F.pixel_shuffle / F.interpolate (sapa_deform.py:44-47) and the
    hi-res offset tensor disappear from the forward pass."""

    @staticmethod
    def forward(ctx, query, key, value, offset, num_point, scale_factor, groups,
                offset_layout='hires', matrix_form=None):
        if offset_layout not in OFFSET_LAYOUTS:
            raise ValueError('offset_layout must be one of %s' % sorted(OFFSET_LAYOUTS))
        assert scale_factor >= 1
        assert query.size(0) == key.size(0) == value.size(0) == offset.size(0)
        assert query.size(1) == key.size(1)
        assert query.size(2) == key.size(2) * scale_factor
        assert query.size(3) == key.size(3) * scale_factor
        assert value.size(2) == key.size(2) and value.size(3) == key.size(3)
        if offset_layout == 'hires':
            assert offset.size(1) == groups * num_point * 2
            assert offset.size(2) == key.size(2) * scale_factor
            assert offset.size(3) == key.size(3) * scale_factor
        else:
            per_cell = scale_factor ** 2 if offset_layout == 'pixel_shuffle' else 1
            assert offset.size(1) == groups * num_point * 2 * per_cell
            assert offset.size(2) == key.size(2) and offset.size(3) == key.size(3)
        assert query.size(1) % groups == 0 and value.size(1) % groups == 0
        assert num_point >= 1
        ctx.num_point = num_point
        ctx.scale_factor = scale_factor
        ctx.groups = groups
        ctx.offset_layout = offset_layout

        n, c, h, w = value.size()
        if not value.is_cuda:
            raise NotImplementedError
        nhwc = _lib.memory_layout(query=query, key=key, value=value,
                                  offset=offset) == 'channels_last'
        output = _lib.new_out(value, (n, c, scale_factor * h, scale_factor * w), nhwc)
        if nhwc:
            # every tensor in torch.channels_last order: served as it is
            if offset_layout != 'hires':
                raise RuntimeError("channels_last tensors take offset_layout='hires'")
            _lib.call_nhwc('sapa_deform_fused_forward_nhwc', value.device, _lib.ptr(query),
                           _lib.ptr(key), _lib.ptr(value), _lib.ptr(offset), _lib.ptr(output), n,
                           key.size(1), c, h, w, num_point, scale_factor, groups,
                           _lib.dtype_code(value))
        else:
            # contiguous tensors: through the matrix-form kernels where they serve the
            # case (key and value go through a workspace in channels-last order),
            # else the contiguous-layout kernels
            shape = (n, key.size(1), c, h, w, num_point, scale_factor, groups, _lib.dtype_code(value))
            nbytes = _lib.lib().sapa_deform_fused_forward_workspace(*shape)
            if matrix_form is None:
                matrix_form = True      # wherever the library says it is the faster path
            elif matrix_form and nbytes == 0:
                raise _lib.SapaUnsupported('deform_sapa_fused(matrix_form=True): this configuration is served '
                                           'by the contiguous-layout kernels only')
            if matrix_form and nbytes > 0:
                ws = torch.empty(nbytes, dtype=torch.uint8, device=value.device)
                _lib.call('sapa_deform_fused_forward_ws', value.device, _lib.ptr(query),
                          _lib.ptr(key), _lib.ptr(value), _lib.ptr(offset), _lib.ptr(output),
                          _lib.ptr(ws), *shape[:-1], OFFSET_LAYOUTS[offset_layout], shape[-1])
            else:
                _lib.call('sapa_deform_fused_forward_from', value.device, _lib.ptr(query),
                          _lib.ptr(key), _lib.ptr(value), _lib.ptr(offset), _lib.ptr(output), n,
                          key.size(1), c, h, w, num_point, scale_factor, groups,
                          OFFSET_LAYOUTS[offset_layout], _lib.dtype_code(value))

        if any(t.requires_grad for t in (query, key, value, offset)):
            ctx.save_for_backward(query, key, value, offset)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        assert grad_output.is_cuda
        query, key, value, offset = ctx.saved_tensors
        gq, gk, gv, goff = _deform_fused_backward(
            grad_output, query, key, value, offset, ctx.num_point, ctx.scale_factor, ctx.groups,
            ctx.offset_layout, tuple(ctx.needs_input_grad[:4]))
        return gq, gk, gv, goff, None, None, None, None, None


def deform_sapa_fused(query, key, value, offset, num_point, scale_factor, groups,
                      offset_layout='hires', matrix_form=None):
    """deform_qk -> softmax over the points -> deform_av (sapa_deform.py:51-53) in one
    launch.  matrix_form (contiguous tensors): True = through the matrix-form kernels
    (sums per window cell: rounding-level differences from the reference's order in
    fp32, no further from the exact result; SapaUnsupported where they do not serve the
    configuration), False = the reference's order of sums, None = the matrix form
    where it is the faster path (16-bit tensors from 4 points, fp32 from 13)."""
    return DeformSAPAFusedFunction.apply(query, key, value, offset, num_point, scale_factor,
                                         groups, offset_layout, matrix_form)
