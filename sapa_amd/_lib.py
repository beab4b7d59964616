"""ctypes binding of libsapa_hip.so (C ABI in include/sapa_hip.h).

The library is loaded from sapa_amd/lib/, where `python -m sapa_amd.build`
puts it.  There is no fallback: if the library is missing or a call fails,
the operators raise.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# SAPA_HIP_LIBRARY points at another build of the same ABI (e.g. a tuning build)
LIB_PATH = os.environ.get('SAPA_HIP_LIBRARY') or os.path.join(_HERE, 'lib', 'libsapa_hip.so')

ABI_VERSION = 1

DTYPES = {torch.float32: 0, torch.float64: 1, torch.float16: 2, torch.bfloat16: 3}

_vp, _i, _ll = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong
# name -> argtypes, in the order of include/sapa_hip.h
SIGNATURES = {
    'sapa_fused_forward_nhwc_qbias': [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_project_nhwc': [_vp, _vp, _vp, _vp, _i, _i, _i, _ll, _i, _vp],
    'sapa_project_nchw': [_vp, _vp, _vp, _vp, _i, _i, _i, _ll, _i, _i, _vp],
    'sapa_norm_project': [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _ll, _i, ctypes.c_float, _i, _i, _i,
                          _vp],
    'sapa_channel_moments': [_vp, _vp, _vp, _i, _i, _ll, _i, _i, _vp],
    'sapa_channel_moments_static': [_vp, _vp, _i, _i, _ll, _i, _i, _vp],
    'sapa_groupnorm_fold': [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, ctypes.c_float, _i, _vp],
    'sapa_qk_forward': [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_qk_backward': [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_av_forward': [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_av_backward': [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_softmax_forward': [_vp, _vp, _ll, _i, _ll, _i, _vp],
    'sapa_fused_forward': [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_qk_softmax_forward': [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_av_backward_logits': [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_fused_backward': [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_fused_forward_attn': [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_fused_backward_attn': [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_qk_forward_nhwc': [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_qk_softmax_forward_nhwc': [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_av_forward_nhwc': [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_fused_forward_nhwc': [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_deform_qk_forward': [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_deform_qk_backward': [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_deform_av_forward': [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_deform_av_backward': [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_deform_qk_backward_ws': [_vp] * 8 + [_i] * 8 + [_vp],
    'sapa_deform_av_backward_ws': [_vp] * 8 + [_i] * 8 + [_vp],
    'sapa_deform_fused_forward': [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_deform_fused_forward_nhwc': [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_deform_fused_backward': [_vp] * 10 + [_i] * 9 + [_vp],
    'sapa_deform_fused_forward_ws': [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_deform_qk_forward_from': [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_deform_av_forward_from': [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    'sapa_stream_mix': [_vp, _vp, _ll, _i, _i, _i, _i, _vp],
    'sapa_layout_copy': [_vp, _vp, _i, _i, _ll, _i, _i, _vp],
    'sapa_deform_fused_forward_from': [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp],
}

_lib = None


class SapaHipError(RuntimeError):
    """A libsapa_hip.so entry point returned a negative status."""


class SapaUnsupported(SapaHipError):
    """SAPA_ERR_UNSUPPORTED: a valid request that this entry point has no
    kernel for.  Direct operator calls raise it; the modules catch it and take
    the next more general path (contiguous tensors, the separate operators)."""


def lib():
    """The loaded library (loaded on first use)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f'{LIB_PATH} is missing: build it with `python -m sapa_amd.build` '
                '(hipcc, gfx950).  There is no fallback implementation.')
        handle = ctypes.CDLL(LIB_PATH)
        handle.sapa_hip_abi_version.restype = _i
        handle.sapa_hip_abi_version.argtypes = []
        if handle.sapa_hip_abi_version() != ABI_VERSION:
            raise RuntimeError(f'{LIB_PATH}: ABI version {handle.sapa_hip_abi_version()}, '
                               f'this package expects {ABI_VERSION}; rebuild the library')
        handle.sapa_hip_status_string.restype = ctypes.c_char_p
        handle.sapa_hip_status_string.argtypes = [_i]
        handle.sapa_hip_last_hip_error.restype = ctypes.c_char_p
        handle.sapa_hip_last_hip_error.argtypes = []
        handle.sapa_hip_last_kernel.restype = ctypes.c_char_p
        handle.sapa_hip_last_kernel.argtypes = []
        for name, argtypes in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = _i
            fn.argtypes = argtypes
        handle.sapa_channel_moments_workspace.restype = _ll
        handle.sapa_channel_moments_workspace.argtypes = [_i, _i, _ll, _i]
        handle.sapa_norm_project_scratch.restype = _ll
        handle.sapa_norm_project_scratch.argtypes = [_i, _i, _i, _ll, _i, _i]
        handle.sapa_fused_backward_workspace.restype = _ll
        handle.sapa_fused_backward_workspace.argtypes = [_i, _i, _i, _i, _i]
        handle.sapa_fused_backward_attn_workspace.restype = _ll
        handle.sapa_fused_backward_attn_workspace.argtypes = [_i, _i, _i, _i, _i]
        handle.sapa_deform_fused_forward_workspace.restype = _ll
        handle.sapa_deform_fused_forward_workspace.argtypes = [_i] * 9
        handle.sapa_deform_fused_backward_workspace.restype = _ll
        handle.sapa_deform_fused_backward_workspace.argtypes = [_i] * 9
        handle.sapa_deform_backward_workspace.restype = _ll
        handle.sapa_deform_backward_workspace.argtypes = [_i] * 8
        handle.sapa_channel_moments_static_capacity.restype = _ll
        handle.sapa_channel_moments_static_capacity.argtypes = []
        _lib = handle
    return _lib


def last_kernel():
    """Name of the kernel behind this thread's most recent forward call."""
    return lib().sapa_hip_last_kernel().decode()


def check(status, what):
    if status == 0:
        return
    handle = lib()
    msg = handle.sapa_hip_status_string(status).decode()
    if status == -4:
        msg += ': ' + handle.sapa_hip_last_hip_error().decode()
    raise (SapaUnsupported if status == UNSUPPORTED else SapaHipError)(
        f'{what}: {msg} (status {status})')


# SAPA_AMD_POISON=1 fills every buffer the kernels are meant to overwrite with
# NaN first, so that a skipped element shows up in any comparison (test aid).
_POISON = os.environ.get('SAPA_AMD_POISON', '') not in ('', '0')


def new_out(like, shape=None, channels_last=False):
    """A buffer that a kernel overwrites completely.  The reference allocates
    these zero-filled (new_zeros, sapa/sapa/sapa_func.py:24); since every
    element is written, the fill is skipped here."""
    shape = like.shape if shape is None else shape
    fmt = torch.channels_last if channels_last else torch.contiguous_format
    out = torch.empty(tuple(shape), dtype=like.dtype, device=like.device, memory_format=fmt)
    if _POISON:
        out.fill_(float('nan'))
    return out


def ptr(t):
    return None if t is None else t.data_ptr()


def dtype_code(t):
    try:
        return DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f'unsupported dtype {t.dtype}; supported: {list(DTYPES)}') from None


def require_cuda_contiguous(**tensors):
    """The reference's CHECK_INPUT (sapa/sapa/src/cuda/qk_cuda.cpp:34-39):
    device tensors, contiguous, and here also one device and one dtype."""
    first = None
    for name, t in tensors.items():
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(f'{name} must be a CUDA tensor')
        if not t.is_contiguous():
            raise RuntimeError(f'{name} must be contiguous')
        if first is None:
            first = (name, t)
        else:
            if t.device != first[1].device:
                raise RuntimeError(f'{name} is on {t.device}, {first[0]} on {first[1].device}')
            if t.dtype != first[1].dtype:
                raise RuntimeError(f'{name} is {t.dtype}, {first[0]} is {first[1].dtype}')


def memory_layout(**tensors):
    """'contiguous' when every tensor is contiguous (what the reference
    requires), 'channels_last' when every tensor is a 4-D device tensor in
    torch.channels_last order (served without a copy by the *_nhwc entry
    points); anything else raises like the reference's CHECK_INPUT."""
    ts = [t for t in tensors.values() if t is not None]
    if all(t.is_contiguous() for t in ts):
        require_cuda_contiguous(**tensors)
        return 'contiguous'
    if all(t.dim() == 4 and t.is_contiguous(memory_format=torch.channels_last) for t in ts):
        # same device / dtype checks, on views that are contiguous
        require_cuda_contiguous(**{k: (None if t is None else t.permute(0, 2, 3, 1))
                                   for k, t in tensors.items()})
        return 'channels_last'
    bad = [k for k, t in tensors.items() if t is not None and not t.is_contiguous()]
    raise RuntimeError(f'{bad[0]} must be contiguous (or every tensor in torch.channels_last order)')


def is_channels_last(t):
    """A 4-D tensor that is dense in torch.channels_last order and not in contiguous order."""
    return (t is not None and t.dim() == 4 and not t.is_contiguous()
            and t.is_contiguous(memory_format=torch.channels_last))


def layout_copy(t, channels_last):
    """`t` (4-D, dense in the other order) in contiguous / torch.channels_last order: the
    library's transposing kernel for 2- and 4-byte elements on the device (the generic strided
    copy behind Tensor.contiguous() runs at a small fraction of the memory rate on these
    shapes), torch's copy for everything else."""
    fmt = torch.channels_last if channels_last else torch.contiguous_format
    if t.is_contiguous(memory_format=fmt):
        return t
    other = torch.contiguous_format if channels_last else torch.channels_last
    if (t.is_cuda and t.dim() == 4 and t.element_size() in (2, 4) and t.is_contiguous(memory_format=other)
            and not (t.requires_grad and torch.is_grad_enabled())):
        out = torch.empty(t.shape, dtype=t.dtype, device=t.device, memory_format=fmt)
        b, c, h, w = t.shape
        status = call_status('sapa_layout_copy', t.device, ptr(t), ptr(out), b, c, h * w,
                             1 if channels_last else 0, t.element_size())
        if status != UNSUPPORTED:
            return out
    return t.contiguous(memory_format=fmt)


def call_nhwc(name, device, *args):
    """An *_nhwc entry point; SAPA_ERR_UNSUPPORTED becomes an error that says
    what the channels-last kernels cover (there is no hidden layout copy)."""
    status = call_status(name, device, *args)
    if status == UNSUPPORTED and 'deform' in name:
        raise SapaUnsupported(
            f'{name}: channels_last tensors are served for float32 / float16 / bfloat16, '
            'scale_factor 1, 2 or 4, at most 32 points, channels per group that are multiples '
            'of 4 (at most 64 query / key channels per group); call .contiguous() on the inputs '
            'for other configurations')
    if status == UNSUPPORTED:
        raise SapaUnsupported(
            f'{name}: channels_last tensors are served for float32 / float16 / bfloat16, '
            '(kernel_size, scale_factor) in {(3,2), (5,2), (7,2), (5,4), (7,4)}, channel counts that '
            'are multiples of 4; '
            'call .contiguous() on the inputs for other configurations')


UNSUPPORTED = -2   # SAPA_ERR_UNSUPPORTED: a valid request this build has no kernel for


def call_status(name, device, *args):
    """Like `call`, but hands back SAPA_ERR_UNSUPPORTED instead of raising on
    it, for entry points that have a composite fallback."""
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device).cuda_stream
        status = getattr(lib(), name)(*args, stream)
    if status != UNSUPPORTED:
        check(status, name)
    return status


def call(name, device, *args):
    """Run entry point `name` on `device`'s current torch stream."""
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device).cuda_stream
        check(getattr(lib(), name)(*args, stream), name)


def channel_moments(x):
    """Mean and biased variance of every (image, channel) of a CUDA feature
    map x [B, C, H, W] (contiguous or channels_last; f32 / f16 / bf16), one
    pass over it: an fp32 tensor [B, C, 2].  None if the kernel does not cover
    the configuration (the caller then uses torch reductions)."""
    B, C, H, W = x.shape
    if x.dtype not in (torch.float32, torch.float16, torch.bfloat16) or x.numel() == 0:
        return None
    if x.is_contiguous():
        cl = 0
    elif x.is_contiguous(memory_format=torch.channels_last):
        cl = 1
    else:
        return None
    handle = lib()
    with torch.cuda.device(x.device):
        ws = torch.empty(max(handle.sapa_channel_moments_workspace(B, C, H * W, cl), 4),
                         dtype=torch.uint8, device=x.device)
        mv = torch.empty(B, C, 2, dtype=torch.float32, device=x.device)
        status = handle.sapa_channel_moments(x.data_ptr(), ws.data_ptr(), mv.data_ptr(), B, C, H * W, cl,
                                             DTYPES[x.dtype], torch.cuda.current_stream(x.device).cuda_stream)
    if status == UNSUPPORTED:
        return None
    check(status, 'sapa_channel_moments')
    return mv


def groupnorm_fold(mean_var, norm, conv, dtype):
    """Per-image projection weights [B, O, C] and bias [B, O] (type `dtype`) of
    conv(norm(x)) from channel_moments' [B, C, 2] tensor; None if the kernel
    does not cover the configuration."""
    B, C, _ = mean_var.shape
    O = conv.out_channels
    params = [norm.weight, norm.bias, conv.weight, conv.bias]
    if C > 8192 or any(p is not None and (p.dtype != dtype or not p.is_contiguous()) for p in params):
        return None
    ptr = lambda t: None if t is None else t.data_ptr()
    with torch.cuda.device(mean_var.device):
        w_out = torch.empty(B, O, C, dtype=dtype, device=mean_var.device)
        b_out = torch.empty(B, O, dtype=dtype, device=mean_var.device)
        status = lib().sapa_groupnorm_fold(
            mean_var.data_ptr(), ptr(norm.weight), ptr(norm.bias), conv.weight.data_ptr(), ptr(conv.bias),
            w_out.data_ptr(), b_out.data_ptr(), B, C, O, norm.num_groups, float(norm.eps), DTYPES[dtype],
            torch.cuda.current_stream(mean_var.device).cuda_stream)
    if status == UNSUPPORTED:
        return None
    check(status, 'sapa_groupnorm_fold')
    return w_out, b_out


def norm_project(x, norm, conv, channels_last_out=False, defer_bias=False):
    """conv(norm(x)) for a GroupNorm and a 1x1 convolution on a CUDA feature x [B, C, H, W]
    (contiguous or channels_last; f16 / bf16 / fp32) in one library call (moments, fold,
    projection: four launches): (out, None), or with defer_bias (out without the bias,
    per-image bias [B, O]); out is channels_last for a channels_last x or with
    channels_last_out.  None if some step has no kernel for the configuration (nothing was
    launched then; the caller takes the steps one by one)."""
    B, C, H, W = x.shape
    O = conv.out_channels
    dtype = x.dtype
    params = [norm.weight, norm.bias, conv.weight, conv.bias]
    if (dtype not in DTYPES or x.numel() == 0 or conv.weight.numel() != O * C
            or any(p is not None and (p.dtype != dtype or not p.is_contiguous()) for p in params)):
        return None
    if x.is_contiguous():
        cl = 0
    elif x.is_contiguous(memory_format=torch.channels_last):
        cl = 1
    else:
        return None
    out_cl = 1 if (cl or channels_last_out) else 0
    handle = lib()
    ptr = lambda t: None if t is None else t.data_ptr()
    with torch.cuda.device(x.device):
        nbytes = handle.sapa_norm_project_scratch(B, C, O, H * W, cl, DTYPES[dtype])
        scratch = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
        out = torch.empty(B, O, H, W, dtype=dtype, device=x.device,
                          memory_format=torch.channels_last if out_cl else torch.contiguous_format)
        b_out = torch.empty(B, O, dtype=dtype, device=x.device) if defer_bias else None
        status = handle.sapa_norm_project(
            x.data_ptr(), ptr(norm.weight), ptr(norm.bias), conv.weight.data_ptr(), ptr(conv.bias),
            scratch.data_ptr(), out.data_ptr(), ptr(b_out), B, C, O, H * W, norm.num_groups, float(norm.eps),
            cl, out_cl, DTYPES[dtype], torch.cuda.current_stream(x.device).cuda_stream)
    if status == UNSUPPORTED:
        return None
    check(status, 'sapa_norm_project')
    return out, b_out


def project_nchw(x, weight, bias=None, channels_last_out=False):
    """out[b, :, h, w] = weight[b] @ x[b, :, h, w] (+ bias[b]) for a contiguous f16 /
    bf16 / fp32 CUDA feature x [B, C, H, W] and per-image weights [B, O, C]: a contiguous
    (or, with channels_last_out, a channels_last) tensor [B, O, H, W], or None if the
    kernel does not cover the configuration (the caller then uses a library GEMM)."""
    B, C, H, W = x.shape
    O = weight.shape[1]
    assert weight.shape == (B, O, C) and (bias is None or bias.shape == (B, O)), 'per-image weights [B, O, C], bias [B, O]'
    if (x.dtype not in (torch.float16, torch.bfloat16, torch.float32) or weight.dtype != x.dtype
            or x.numel() == 0 or not x.is_contiguous()):
        return None
    weight = weight.contiguous()
    if bias is not None:
        bias = bias.to(x.dtype).contiguous()
    with torch.cuda.device(x.device):
        out = torch.empty(B, O, H, W, dtype=x.dtype, device=x.device,
                          memory_format=torch.channels_last if channels_last_out else torch.contiguous_format)
        status = lib().sapa_project_nchw(
            x.data_ptr(), weight.data_ptr(), None if bias is None else bias.data_ptr(), out.data_ptr(),
            B, C, O, H * W, 1 if channels_last_out else 0, DTYPES[x.dtype],
            torch.cuda.current_stream(x.device).cuda_stream)
    if status == UNSUPPORTED:
        return None
    check(status, 'sapa_project_nchw')
    return out


def project_nhwc(x, weight, bias=None):
    """out[b, :, h, w] = weight[b] @ x[b, :, h, w] (+ bias[b]) for a channels_last
    f16 / bf16 / fp32 CUDA feature x [B, C, H, W] and per-image weights [B, O, C]: a
    channels_last tensor [B, O, H, W], or None if the kernel does not cover the
    configuration (the caller then uses a library GEMM)."""
    B, C, H, W = x.shape
    O = weight.shape[1]
    assert weight.shape == (B, O, C) and (bias is None or bias.shape == (B, O)), 'per-image weights [B, O, C], bias [B, O]'
    if (x.dtype not in (torch.float16, torch.bfloat16, torch.float32) or weight.dtype != x.dtype
            or x.numel() == 0):
        return None
    if not x.is_contiguous(memory_format=torch.channels_last):
        return None
    weight = weight.contiguous()
    if bias is not None:
        bias = bias.to(x.dtype).contiguous()
    with torch.cuda.device(x.device):
        out = torch.empty(B, O, H, W, dtype=x.dtype, device=x.device,
                          memory_format=torch.channels_last)
        status = lib().sapa_project_nhwc(
            x.data_ptr(), weight.data_ptr(), None if bias is None else bias.data_ptr(), out.data_ptr(),
            B, C, O, H * W, DTYPES[x.dtype], torch.cuda.current_stream(x.device).cuda_stream)
    if status == UNSUPPORTED:
        return None
    check(status, 'sapa_project_nhwc')
    return out
