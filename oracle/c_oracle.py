"""ctypes front-end of the brute-force C oracle (oracle/sapa_oracle.c).

TEST INFRASTRUCTURE ONLY -- see oracle/__init__.py.

Functions take and return CPU torch tensors (NCHW-contiguous).  `mode`:
  'f32'     the reference kernels' own arithmetic: float FMA accumulation in
            the kernels' loop order (float32 in, float32 out)
  'f64'     everything in double (float64 in, float64 out)
  'f32a64'  float32 in, sums in double, float64 out (forward only)
Argument order follows the Python API of the reference
(sapa/sapa/sapa_func.py:12,57; deformsapa/deformsapa/deform_func.py:10,65).
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, '_build', 'libsapa_oracle.so')
_lib = None


def build(force=False):
    """Compile the C oracle with gcc (oracle/Makefile)."""
    if force:
        subprocess.check_call(['make', '-C', _HERE, 'clean'], stdout=subprocess.DEVNULL)
    subprocess.check_call(['make', '-C', _HERE], stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


_IN = {'f32': torch.float32, 'f64': torch.float64, 'f32a64': torch.float32}
_OUT = {'f32': torch.float32, 'f64': torch.float64, 'f32a64': torch.float64}


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _prep(mode, *ts):
    dt = _IN[mode]
    out = []
    for t in ts:
        assert t.device.type == 'cpu'
        assert t.dtype == dt, f'mode {mode} wants {dt}, got {t.dtype}'
        out.append(t.contiguous())
    return out


def _call(name, mode, *args):
    fn = getattr(lib(), f'oracle_{mode}_{name}')
    fn.restype = None
    fn(*args)


def _ints(*v):
    return [ctypes.c_int(int(x)) for x in v]


def qk(q, key, K, s, mode='f32'):
    q, key = _prep(mode, q, key)
    B, d, H, W = key.shape
    assert q.shape == (B, d, H * s, W * s)
    out = torch.empty(B, K * K, H * s, W * s, dtype=_OUT[mode])
    _call('qk_forward', mode, _p(q), _p(key), _p(out), *_ints(B, d, H, W, K, s))
    return out


def av(attn, value, K, s, mode='f32'):
    attn, value = _prep(mode, attn, value)
    B, C, H, W = value.shape
    assert attn.shape == (B, K * K, H * s, W * s)
    out = torch.empty(B, C, H * s, W * s, dtype=_OUT[mode])
    _call('av_forward', mode, _p(attn), _p(value), _p(out), *_ints(B, C, H, W, K, s))
    return out


def softmax(x, dim, mode='f32'):
    (x,) = _prep(mode, x)
    N = 1
    for v in x.shape[:dim]:
        N *= v
    R = x.shape[dim]
    M = 1
    for v in x.shape[dim + 1:]:
        M *= v
    out = torch.empty(x.shape, dtype=_OUT[mode])
    _call('softmax_forward', mode, _p(x), _p(out), ctypes.c_long(N),
          ctypes.c_int(R), ctypes.c_long(M))
    return out


def sapa_fused(q, key, value, K, s, mode='f32'):
    """qk -> softmax(dim=1) -> av (sapa_base.py:38-40).  In 'f32a64' the
    intermediate logits and weights stay in double."""
    if mode == 'f32a64':
        logits = qk(q, key, K, s, 'f32a64')
        attn = softmax(logits, 1, 'f64')
        return av(attn, value.double(), K, s, 'f64')
    return av(softmax(qk(q, key, K, s, mode), 1, mode), value, K, s, mode)


def deform_qk(q, key, offset, P, s, G, mode='f32'):
    q, key, offset = _prep(mode, q, key, offset)
    B, Cq, H, W = key.shape
    assert q.shape == (B, Cq, H * s, W * s)
    assert offset.shape == (B, 2 * G * P, H * s, W * s)
    out = torch.empty(B, G, P, H * s, W * s, dtype=_OUT[mode])
    _call('deform_qk_forward', mode, _p(q), _p(key), _p(offset), _p(out),
          *_ints(B, Cq, H, W, P, s, G))
    return out


def deform_av(attn, value, offset, P, s, G, mode='f32'):
    attn, value, offset = _prep(mode, attn, value, offset)
    B, C, H, W = value.shape
    assert attn.shape == (B, G, P, H * s, W * s)
    assert offset.shape == (B, 2 * G * P, H * s, W * s)
    out = torch.empty(B, C, H * s, W * s, dtype=_OUT[mode])
    _call('deform_av_forward', mode, _p(attn), _p(value), _p(offset), _p(out),
          *_ints(B, C, H, W, P, s, G))
    return out


def deform_sapa_fused(q, key, value, offset, P, s, G, mode='f32'):
    """deform_qk -> softmax over P -> deform_av (sapa_deform.py:51-53)."""
    assert mode in ('f32', 'f64')
    attn = softmax(deform_qk(q, key, offset, P, s, G, mode), 2, mode)
    return deform_av(attn, value, offset, P, s, G, mode)


def qk_backward(gout, q, key, K, s, mode='f64'):
    assert mode in ('f32', 'f64')
    gout, q, key = _prep(mode, gout, q, key)
    B, d, H, W = key.shape
    gq, gk = torch.zeros_like(q), torch.zeros_like(key)
    _call('qk_backward', mode, _p(gout), _p(q), _p(key), _p(gq), _p(gk),
          *_ints(B, d, H, W, K, s))
    return gq, gk


def av_backward(gout, attn, value, K, s, mode='f64'):
    assert mode in ('f32', 'f64')
    gout, attn, value = _prep(mode, gout, attn, value)
    B, C, H, W = value.shape
    ga, gv = torch.zeros_like(attn), torch.zeros_like(value)
    _call('av_backward', mode, _p(gout), _p(attn), _p(value), _p(ga), _p(gv),
          *_ints(B, C, H, W, K, s))
    return ga, gv


def deform_qk_backward(gout, q, key, offset, P, s, G, mode='f64'):
    assert mode in ('f32', 'f64')
    gout, q, key, offset = _prep(mode, gout, q, key, offset)
    B, Cq, H, W = key.shape
    gq, gk, go = torch.zeros_like(q), torch.zeros_like(key), torch.zeros_like(offset)
    _call('deform_qk_backward', mode, _p(gout), _p(q), _p(key), _p(offset),
          _p(gq), _p(gk), _p(go), *_ints(B, Cq, H, W, P, s, G))
    return gq, gk, go


def deform_av_backward(gout, attn, value, offset, P, s, G, mode='f64'):
    assert mode in ('f32', 'f64')
    gout, attn, value, offset = _prep(mode, gout, attn, value, offset)
    B, C, H, W = value.shape
    ga, gv, go = torch.zeros_like(attn), torch.zeros_like(value), torch.zeros_like(offset)
    _call('deform_av_backward', mode, _p(gout), _p(attn), _p(value), _p(offset),
          _p(ga), _p(gv), _p(go), *_ints(B, C, H, W, P, s, G))
    return ga, gv, go
