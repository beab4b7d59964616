"""SAPA-B operators: autograd API of the reference on top of libsapa_hip.so.

Mirrors sapa/sapa/sapa_func.py of the reference (QKFunction :9-51,
AVFunction :54-96): same names, argument order, assertions, output
allocation and error behaviour (CPU tensors raise NotImplementedError), so
`from sapa import qk, av` callers such as SAPA.attention (sapa_base.py:38-40)
run unchanged.  `sapa_fused`, `qk_softmax` and `softmax_k` are additions.
"""
import torch
from torch.autograd import Function

from . import _lib


def _check_odd_kernel(kernel_size):
    assert (kernel_size - 1) % 2 == 0 and kernel_size >= 1


class _MemoryOrder(Function):
    """`t` in contiguous / torch.channels_last order with the library's transposing kernel
    (_lib.layout_copy) in both passes: the gradient goes back in the order `t` had."""

    @staticmethod
    def forward(ctx, t, channels_last):
        ctx.back_to_channels_last = _lib.is_channels_last(t)
        with torch.no_grad():
            return _lib.layout_copy(t, channels_last)

    @staticmethod
    def backward(ctx, grad):
        return _lib.layout_copy(grad, ctx.back_to_channels_last), None


def in_memory_order(t, memory_format):
    """Tensor.contiguous(memory_format=...) for the feature maps of the modules: the tensor
    itself when it is in that order already, else a transposed copy made by the library's
    layout kernel (device tensors of 2- and 4-byte elements that are dense in the other order;
    anything else takes Tensor.contiguous)."""
    if t.is_contiguous(memory_format=memory_format):
        return t
    if not (t.is_cuda and t.dim() == 4 and t.element_size() in (2, 4)):
        return t.contiguous(memory_format=memory_format)
    return _MemoryOrder.apply(t, memory_format is torch.channels_last)


def _back(grad, channels_last):
    """A gradient computed in contiguous order, in the order of the tensor it belongs to."""
    return grad if grad is None or not channels_last else _lib.layout_copy(grad, True)


def _qk_backward(grad_output, query, key, kernel_size, scale_factor, need_q=True, need_k=True):
    # the gradient kernels take contiguous tensors: operands kept in
    # channels-last order are copied here (the forward pass is the zero-copy one)
    # 16-bit tensors are read and written as they are (fp32 sums inside the
    # kernels), as the reference's half dispatch does (qk_cuda_kernel.cu:139-171)
    # (_lib.layout_copy: the library's transposing kernel; the gradients go back in the order
    # of the tensors they belong to)
    cl_q, cl_k = _lib.is_channels_last(query), _lib.is_channels_last(key)
    query, key = _lib.layout_copy(query, False), _lib.layout_copy(key, False)
    grad_output = _lib.layout_copy(grad_output, False)
    grad_query = _lib.new_out(query) if need_q else None
    grad_key = _lib.new_out(key) if need_k else None
    _lib.require_cuda_contiguous(grad_output=grad_output, query=query, key=key)
    n, c, h, w = key.size()
    _lib.call('sapa_qk_backward', key.device, _lib.ptr(grad_output), _lib.ptr(query),
              _lib.ptr(key), _lib.ptr(grad_query), _lib.ptr(grad_key), n, c, h, w,
              kernel_size, scale_factor, _lib.dtype_code(key))
    return _back(grad_query, cl_q), _back(grad_key, cl_k)


def _av_backward(grad_output, attn, value, kernel_size, scale_factor, need_a=True, need_v=True):
    cl_a, cl_v = _lib.is_channels_last(attn), _lib.is_channels_last(value)
    attn, value = _lib.layout_copy(attn, False), _lib.layout_copy(value, False)
    grad_output = _lib.layout_copy(grad_output, False)
    grad_attn = _lib.new_out(attn) if need_a else None
    grad_value = _lib.new_out(value) if need_v else None
    _lib.require_cuda_contiguous(grad_output=grad_output, attn=attn, value=value)
    n, c, h, w = value.size()
    _lib.call('sapa_av_backward', value.device, _lib.ptr(grad_output), _lib.ptr(attn),
              _lib.ptr(value), _lib.ptr(grad_attn), _lib.ptr(grad_value), n, c, h, w,
              kernel_size, scale_factor, _lib.dtype_code(value))
    return _back(grad_attn, cl_a), _back(grad_value, cl_v)


class QKFunction(Function):

    @staticmethod
    def forward(ctx, query, key, kernel_size, scale_factor):
        assert scale_factor >= 1
        assert query.size(0) == key.size(0)
        assert query.size(1) == key.size(1)
        assert query.size(-1) == key.size(-1) * scale_factor
        assert query.size(-2) == key.size(-2) * scale_factor
        _check_odd_kernel(kernel_size)
        ctx.kernel_size = kernel_size
        ctx.scale_factor = scale_factor
        ctx.query_size = query.size()
        ctx.key_size = key.size()

        n, c, h, w = key.size()
        if not key.is_cuda:
            raise NotImplementedError
        nhwc = _lib.memory_layout(key=key, query=query) == 'channels_last'
        output = _lib.new_out(key, (n, kernel_size ** 2, h * scale_factor, w * scale_factor), nhwc)
        (_lib.call_nhwc if nhwc else _lib.call)(
            'sapa_qk_forward_nhwc' if nhwc else 'sapa_qk_forward', key.device, _lib.ptr(query),
            _lib.ptr(key), _lib.ptr(output), n, c, h, w, kernel_size, scale_factor,
            _lib.dtype_code(key))

        if query.requires_grad or key.requires_grad:
            ctx.save_for_backward(query, key)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        assert grad_output.is_cuda
        query, key = ctx.saved_tensors
        grad_query, grad_key = _qk_backward(grad_output, query, key, ctx.kernel_size,
                                            ctx.scale_factor)
        return grad_query, grad_key, None, None


qk = QKFunction.apply


class AVFunction(Function):

    @staticmethod
    def forward(ctx, attn, value, kernel_size, scale_factor):
        assert scale_factor >= 1
        assert attn.size(0) == value.size(0)
        assert attn.size(1) == kernel_size * kernel_size
        assert attn.size(-1) == value.size(-1) * scale_factor
        assert attn.size(-2) == value.size(-2) * scale_factor
        _check_odd_kernel(kernel_size)
        ctx.kernel_size = kernel_size
        ctx.scale_factor = scale_factor
        ctx.attn_size = attn.size()
        ctx.value_size = value.size()

        n, c, h, w = value.size()
        if not value.is_cuda:
            raise NotImplementedError
        nhwc = _lib.memory_layout(value=value, attn=attn) == 'channels_last'
        output = _lib.new_out(value, (n, c, h * scale_factor, w * scale_factor), nhwc)
        (_lib.call_nhwc if nhwc else _lib.call)(
            'sapa_av_forward_nhwc' if nhwc else 'sapa_av_forward', value.device, _lib.ptr(attn),
            _lib.ptr(value), _lib.ptr(output), n, c, h, w, kernel_size, scale_factor,
            _lib.dtype_code(value))

        if attn.requires_grad or value.requires_grad:
            ctx.save_for_backward(attn, value)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        assert grad_output.is_cuda
        attn, value = ctx.saved_tensors
        grad_attn, grad_value = _av_backward(grad_output, attn, value, ctx.kernel_size,
                                             ctx.scale_factor)
        return grad_attn, grad_value, None, None


av = AVFunction.apply


def softmax_k(logits, dim=1):
    """Softmax over `dim` with the library's kernel (no autograd): the
    stand-alone form of the F.softmax calls in sapa_base.py:39 (dim=1) and
    sapa_deform.py:52 (dim=2)."""
    if not logits.is_cuda:
        raise NotImplementedError
    _lib.require_cuda_contiguous(logits=logits)
    dim = dim % logits.dim()
    N = 1
    for v in logits.shape[:dim]:
        N *= v
    M = 1
    for v in logits.shape[dim + 1:]:
        M *= v
    out = torch.empty_like(logits)
    _lib.call('sapa_softmax_forward', logits.device, _lib.ptr(logits), _lib.ptr(out), N,
              logits.shape[dim], M, _lib.dtype_code(logits))
    return out


def _qk_softmax_forward(query, key, kernel_size, scale_factor, nhwc=False):
    n, c, h, w = key.size()
    attn = _lib.new_out(key, (n, kernel_size ** 2, h * scale_factor, w * scale_factor), nhwc)
    (_lib.call_nhwc if nhwc else _lib.call)(
        'sapa_qk_softmax_forward_nhwc' if nhwc else 'sapa_qk_softmax_forward', key.device,
        _lib.ptr(query), _lib.ptr(key), _lib.ptr(attn), n, c, h, w, kernel_size, scale_factor,
        _lib.dtype_code(key))
    return attn


def qk_softmax(query, key, kernel_size, scale_factor):
    """softmax(qk(query, key), dim=1) in one launch (no autograd)."""
    assert query.size(0) == key.size(0) and query.size(1) == key.size(1)
    assert query.size(-1) == key.size(-1) * scale_factor
    assert query.size(-2) == key.size(-2) * scale_factor
    _check_odd_kernel(kernel_size)
    if not key.is_cuda:
        raise NotImplementedError
    nhwc = _lib.memory_layout(key=key, query=query) == 'channels_last'
    return _qk_softmax_forward(query, key, kernel_size, scale_factor, nhwc)


def _fused_backward(grad_output, query, key, value, K, s, needs=(True, True, True), attn=None):
    """Gradients of av(softmax(qk(query, key)), value): the attention weights
    are recomputed (one launch) unless the forward pass kept them (`attn`, fp32),
    then the three operators' gradients chain."""
    need_q, need_k, need_v = needs
    cl = [_lib.is_channels_last(t) for t in (query, key, value)]
    if any(cl) or _lib.is_channels_last(grad_output) or _lib.is_channels_last(attn):
        # the gradient kernels take contiguous tensors: operands in channels-last order are
        # transposed by the library's layout kernel, and each gradient goes back in the order
        # of the tensor it belongs to
        grads = _fused_backward(_lib.layout_copy(grad_output, False), _lib.layout_copy(query, False),
                                _lib.layout_copy(key, False), _lib.layout_copy(value, False), K, s, needs,
                                None if attn is None else _lib.layout_copy(attn, False))
        return tuple(_back(g, c) for g, c in zip(grads, cl))
    query, key, value = query.contiguous(), key.contiguous(), value.contiguous()
    grad_output = grad_output.contiguous()
    _lib.require_cuda_contiguous(grad_output=grad_output, query=query, key=key, value=value)
    if attn is not None:
        n, c, h, w = value.size()
        nbytes = _lib.lib().sapa_fused_backward_attn_workspace(n, h, w, K, s)
        ws = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=value.device)
        grads = [_lib.new_out(t) if need else None
                 for t, need in ((query, need_q), (key, need_k), (value, need_v))]
        status = _lib.call_status('sapa_fused_backward_attn', value.device, _lib.ptr(grad_output),
                                  _lib.ptr(query), _lib.ptr(key), _lib.ptr(value), _lib.ptr(attn), _lib.ptr(ws),
                                  _lib.ptr(grads[0]), _lib.ptr(grads[1]), _lib.ptr(grads[2]), n, key.size(1),
                                  c, h, w, K, s, _lib.dtype_code(value))
        if status != _lib.UNSUPPORTED:
            return tuple(grads)
        del ws, grads
    # the whole chain in one library call where the tiled kernels cover it: 16-bit
    # tensors go in and out as they are, the [B,K*K,sH,sW] intermediates stay fp32
    n, c, h, w = value.size()
    d = key.size(1)
    nbytes = _lib.lib().sapa_fused_backward_workspace(n, h, w, K, s)
    ws = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=value.device)
    grads = [_lib.new_out(t) if need else None
             for t, need in ((query, need_q), (key, need_k), (value, need_v))]
    status = _lib.call_status('sapa_fused_backward', value.device, _lib.ptr(grad_output), _lib.ptr(query),
                              _lib.ptr(key), _lib.ptr(value), _lib.ptr(ws), _lib.ptr(grads[0]),
                              _lib.ptr(grads[1]), _lib.ptr(grads[2]), n, d, c, h, w, K, s,
                              _lib.dtype_code(value))
    if status != _lib.UNSUPPORTED:
        return tuple(grads)
    del ws, grads
    if value.dtype in (torch.float16, torch.bfloat16):
        # no one-call kernel for this (kernel_size, scale_factor): the chain below in fp32 on
        # widened copies, so that the weights and the gradient of the logits are rounded to
        # 16 bits nowhere -- each gradient is rounded once, at the end
        wide = _fused_backward(grad_output.float(), query.float(), key.float(), value.float(), K, s, needs)
        return tuple(None if t is None else t.to(value.dtype) for t in wide)
    attn = _qk_softmax_forward(query, key, K, s)
    grad_query = grad_key = grad_logits = None
    if need_q or need_k:
        # grad of the logits through av and softmax in one launch where the
        # library has it ...
        grad_output = grad_output.contiguous()
        _lib.require_cuda_contiguous(grad_output=grad_output, attn=attn, value=value)
        n, c, h, w = value.size()
        grad_logits = _lib.new_out(attn)
        status = _lib.call_status('sapa_av_backward_logits', value.device, _lib.ptr(grad_output),
                                  _lib.ptr(attn), _lib.ptr(value), _lib.ptr(grad_logits), n, c, h,
                                  w, K, s, _lib.dtype_code(value))
        if status == _lib.UNSUPPORTED:
            grad_logits = None
    grad_attn, grad_value = _av_backward(
        grad_output, attn, value, K, s,
        need_a=(need_q or need_k) and grad_logits is None, need_v=need_v)
    if need_q or need_k:
        if grad_logits is None:
            # ... else softmax backward in fp32: attn * (g_attn - sum_k g_attn * attn)
            a32, g32 = attn.float(), grad_attn.float()
            grad_logits = (a32 * (g32 - (g32 * a32).sum(dim=1, keepdim=True))).to(attn.dtype)
        grad_query, grad_key = _qk_backward(grad_logits, query, key, K, s, need_q, need_k)
    return grad_query, grad_key, grad_value


# Training steps of sapa_fused keep the fp32 attention weights between the forward and
# the backward pass (faster: one launch less per step) unless this is False or the call
# says save_attention=False (less memory: the weights are recomputed).
SAVE_ATTENTION = True


class SAPAFusedFunction(Function):
    """av(softmax(qk(query, key), dim=1), value) -- SAPA.attention
    (sapa_base.py:38-40) -- as one launch in the forward pass.  When a gradient
    is wanted and `save_attention` is set (the default, SAVE_ATTENTION), the
    forward pass runs as two launches that leave the fp32 attention weights
    [B,K*K,sH,sW] behind for the backward pass, as the reference's autograd graph
    does; otherwise the backward pass recomputes them (one launch more, nothing
    kept alive but the operands).  Then the three operators' gradients chain.

    query_bias [B, d] (optional): a per-image bias added to every query vector,
    i.e. the result for query + query_bias[:, :, None, None] -- what a 1x1
    projection with a (per-image) bias produces -- without that sum being
    written first.  The channels_last kernels add it on the fly; other layouts
    form the sum."""

    @staticmethod
    def forward(ctx, query, key, value, kernel_size, scale_factor, query_bias=None, save_attention=None):
        assert scale_factor >= 1
        assert query.size(0) == key.size(0) == value.size(0)
        assert query.size(1) == key.size(1)
        assert query.size(-1) == key.size(-1) * scale_factor
        assert query.size(-2) == key.size(-2) * scale_factor
        assert value.size(-1) == key.size(-1) and value.size(-2) == key.size(-2)
        _check_odd_kernel(kernel_size)
        ctx.kernel_size = kernel_size
        ctx.scale_factor = scale_factor

        n, d, h, w = key.size()
        c = value.size(1)
        if not value.is_cuda:
            raise NotImplementedError
        nhwc = _lib.memory_layout(value=value, key=key, query=query) == 'channels_last'
        if query_bias is not None:
            assert query_bias.shape == (n, d) and query_bias.dtype == query.dtype
        ctx.has_bias = query_bias is not None
        wants_grad = query.requires_grad or key.requires_grad or value.requires_grad or \
            (query_bias is not None and query_bias.requires_grad)
        saved = (query, key, value) + ((query_bias,) if ctx.has_bias else ())
        ctx.has_attn = False
        if query_bias is not None and not nhwc:
            query = query + query_bias[:, :, None, None]
            query_bias = None
        output = _lib.new_out(value, (n, c, h * scale_factor, w * scale_factor), nhwc)
        if wants_grad and not nhwc and (SAVE_ATTENTION if save_attention is None else save_attention):
            attn = torch.empty((n, kernel_size * kernel_size, h * scale_factor, w * scale_factor),
                               dtype=torch.float32, device=value.device)
            status = _lib.call_status('sapa_fused_forward_attn', value.device, _lib.ptr(query), _lib.ptr(key),
                                      _lib.ptr(value), _lib.ptr(attn), _lib.ptr(output), n, d, c, h, w,
                                      kernel_size, scale_factor, _lib.dtype_code(value))
            if status != _lib.UNSUPPORTED:
                ctx.has_attn = True
                ctx.save_for_backward(*(saved + (attn,)))
                return output
            del attn
        if wants_grad:
            ctx.save_for_backward(*saved)
        if query_bias is not None:
            query_bias = query_bias.contiguous()
            _lib.call_nhwc('sapa_fused_forward_nhwc_qbias', value.device, _lib.ptr(query), _lib.ptr(key),
                           _lib.ptr(value), _lib.ptr(query_bias), _lib.ptr(output), n, d, c, h, w,
                           kernel_size, scale_factor, _lib.dtype_code(value))
        else:
            (_lib.call_nhwc if nhwc else _lib.call)(
                'sapa_fused_forward_nhwc' if nhwc else 'sapa_fused_forward', value.device,
                _lib.ptr(query), _lib.ptr(key), _lib.ptr(value), _lib.ptr(output), n, d, c, h, w,
                kernel_size, scale_factor, _lib.dtype_code(value))
        return output

    @staticmethod
    def backward(ctx, grad_output):
        assert grad_output.is_cuda
        query, key, value = ctx.saved_tensors[:3]
        needs = ctx.needs_input_grad
        grad_bias = None
        if ctx.has_bias:
            query = query + ctx.saved_tensors[3][:, :, None, None]
        grad_query, grad_key, grad_value = _fused_backward(
            grad_output, query, key, value, ctx.kernel_size, ctx.scale_factor,
            (needs[0] or (ctx.has_bias and needs[5]), needs[1], needs[2]),
            attn=ctx.saved_tensors[-1] if ctx.has_attn else None)
        if ctx.has_bias and needs[5]:
            wide = torch.float32 if grad_query.dtype in (torch.float16, torch.bfloat16) else None
            grad_bias = grad_query.sum(dim=(2, 3), dtype=wide).to(grad_query.dtype)
        return (grad_query if needs[0] else None), grad_key, grad_value, None, None, grad_bias, None


def sapa_fused(query, key, value, kernel_size, scale_factor, query_bias=None, save_attention=None):
    return SAPAFusedFunction.apply(query, key, value, kernel_size, scale_factor, query_bias, save_attention)
