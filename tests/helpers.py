"""Shared test helpers: seeded inputs and the parity bars."""
import os

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, 'tests', 'golden', 'sapa_golden.npz')

# fp32 bar of the build's brief: |a - b| <= 1e-6 + 1e-5 * |b|
F32_RTOL, F32_ATOL = 1e-5, 1e-6
# bf16 bar: 1e-2 relative.  A pure element-wise relative error is undefined
# at near-zero outputs of a signed sum, so "relative" is taken against
# max(|b|, rms(b)): |a - b| <= 1e-2 * max(|b|, rms(b)).
BF16_REL = 1e-2
F16_REL = 2e-3


def gen(seed):
    return torch.Generator().manual_seed(seed)


def randn(g, *shape, dtype=torch.float32):
    return torch.randn(*shape, generator=g, dtype=dtype)


def golden():
    return np.load(GOLDEN)


def assert_f32_close(got, want, what=''):
    got, want = got.detach().cpu().double(), want.detach().cpu().double()
    err = (got - want).abs()
    bound = F32_ATOL + F32_RTOL * want.abs()
    bad = err > bound
    assert not bad.any(), (f'{what}: {int(bad.sum())} of {bad.numel()} outside '
                           f'{F32_ATOL}+{F32_RTOL}*|b|; max abs err {err.max().item():.3e}')


def assert_rel_rms_close(got, want, rel, what=''):
    got, want = got.detach().cpu().double(), want.detach().cpu().double()
    rms = want.pow(2).mean().sqrt()
    bound = rel * torch.maximum(want.abs(), rms)
    err = (got - want).abs()
    bad = err > bound
    assert not bad.any(), (f'{what}: {int(bad.sum())} of {bad.numel()} outside {rel}*max(|b|,rms); '
                           f'max err {err.max().item():.3e}, rms {rms.item():.3e}')


def ulp_report(got, want):
    """max |a-b| in units of fp32 spacing at |b| (for messages)."""
    got, want = got.detach().cpu().float(), want.detach().cpu().float()
    sp = torch.abs(torch.nextafter(want, torch.full_like(want, float('inf'))) - want)
    return ((got - want).abs() / sp).max().item()


def fused_backward_oracle(coracle, go, q, key, v, K, s):
    """float64 chain of the reference's backward (sapa/sapa/sapa_func.py:34-48,79-93
    under sapa_base.py:38-40): av backward, softmax backward, qk backward."""
    q, key, v, go = (t.double() for t in (q, key, v, go))
    attn = torch.softmax(coracle.qk(q, key, K, s, 'f64'), dim=1)
    ga, gv = coracle.av_backward(go, attn, v, K, s, 'f64')
    gl = attn * (ga - (ga * attn).sum(dim=1, keepdim=True))
    gq, gk = coracle.qk_backward(gl, q, key, K, s, 'f64')
    return gq, gk, gv


def deform_fused_backward_oracle(coracle, go, q, key, v, off, P, s, G):
    """deform_av_backward -> softmax backward -> deform_qk_backward in float64
    on the given values (the chain autograd runs for sapa_deform.py:51-53)."""
    go, q, key, v, off = (t.double() for t in (go, q, key, v, off))
    attn = torch.softmax(coracle.deform_qk(q, key, off, P, s, G, 'f64'), dim=2)
    ga, gv, goff_av = coracle.deform_av_backward(go, attn, v, off, P, s, G, 'f64')
    gl = attn * (ga - (ga * attn).sum(dim=2, keepdim=True))
    gq, gk, goff_qk = coracle.deform_qk_backward(gl, q, key, off, P, s, G, 'f64')
    return gq, gk, gv, goff_av + goff_qk
