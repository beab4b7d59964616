"""GPU parity of the SAPA-D operators (deform_qk, deform_av, fused) against
the CPU oracle, through the Python API and so through the C ABI.

fp32 results are compared bit-for-bit with the oracle in the reference
kernels' arithmetic: that pins the floor / guard / corner indexing exactly.
"""
import pytest
import torch
import torch.nn.functional as F

import sapa_amd
from helpers import (BF16_REL, F16_REL, assert_f32_close, assert_rel_rms_close, deform_fused_backward_oracle,
                     gen, golden, randn, ulp_report)

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'

# B, G, dq (query/key channels per group), cg (value channels per group), H, W, P, s
SHAPES = [
    (2, 4, 2, 3, 7, 9, 5, 2), (1, 2, 3, 2, 5, 5, 9, 1), (1, 4, 8, 16, 12, 20, 9, 2),
    (2, 1, 4, 5, 6, 4, 25, 2), (1, 3, 2, 2, 4, 5, 3, 3), (1, 2, 5, 9, 8, 8, 17, 2),
    (1, 1, 2, 2, 3, 3, 40, 2), (1, 4, 32, 64, 16, 16, 5, 2),
]
IDS = ['-'.join(map(str, s)) for s in SHAPES]


def dev(*ts):
    return [t.to(DEV) for t in ts]


def make(g, shape, dtype=torch.float32, off_scale=1.5):
    B, G, dq, cg, H, W, P, s = shape
    q = randn(g, B, G * dq, H * s, W * s, dtype=dtype)
    key = randn(g, B, G * dq, H, W, dtype=dtype)
    v = randn(g, B, G * cg, H, W, dtype=dtype)
    off = randn(g, B, 2 * G * P, H * s, W * s, dtype=dtype) * off_scale
    attn = randn(g, B, G, P, H * s, W * s, dtype=dtype)
    return q, key, v, off, attn


@pytest.mark.parametrize('shape', SHAPES, ids=IDS)
def test_deform_qk_av_fp32_bit_exact(coracle, shape):
    B, G, dq, cg, H, W, P, s = shape
    q, key, v, off, attn = make(gen(200), shape)
    got = sapa_amd.deform_qk(*dev(q, key, off), P, s, G).cpu()
    want = coracle.deform_qk(q, key, off, P, s, G, 'f32')
    assert got.shape == (B, G, P, H * s, W * s)
    assert torch.equal(got, want), f'deform_qk max ulp {ulp_report(got, want)}'
    got = sapa_amd.deform_av(*dev(attn, v, off), P, s, G).cpu()
    want = coracle.deform_av(attn, v, off, P, s, G, 'f32')
    assert torch.equal(got, want), f'deform_av max ulp {ulp_report(got, want)}'


@pytest.mark.parametrize('shape', SHAPES, ids=IDS)
def test_deform_fused_fp32(coracle, shape):
    B, G, dq, cg, H, W, P, s = shape
    q, key, v, off, _ = make(gen(201), shape)
    got = sapa_amd.deform_sapa_fused(*dev(q, key, v, off), P, s, G).cpu()
    assert_f32_close(got, coracle.deform_sapa_fused(q, key, v, off, P, s, G, 'f32'), 'deform fused')
    want64 = coracle.deform_sapa_fused(q.double(), key.double(), v.double(), off.double(), P, s, G, 'f64')
    torch.testing.assert_close(got.double(), want64, rtol=1e-4, atol=1e-5)


# Contiguous tensors through the matrix-form kernels (key and value copied to
# channels-last order in a workspace, q / offset / out used in place).
# B, G, dq, cg, H, W, P, s, offset scale: far offsets with 16 lanes per pixel and
# rows that are no multiple of the 4-pixel tile (26 and 6 pixels wide); 48 channels
# padded to 64 at s = 4; s = 1; three value chunks (64 + 64 + 8); groups that are
# not whole 16-byte pieces (16-bit tensors then stay on the fp32-in-LDS kernel)
MATRIX_SHAPES = [(1, 4, 32, 64, 8, 8, 25, 2, 0.75), (2, 2, 8, 16, 14, 13, 16, 2, 6.0),
                 (1, 2, 48, 24, 7, 9, 15, 4, 2.5), (2, 1, 16, 40, 11, 6, 29, 1, 3.0),
                 (1, 1, 64, 136, 5, 7, 21, 2, 1.5), (1, 2, 12, 20, 6, 5, 17, 2, 1.0)]
MATRIX_IDS = ['-'.join(map(str, s)) for s in MATRIX_SHAPES]


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('shape', MATRIX_SHAPES, ids=MATRIX_IDS)
def test_deform_fused_matrix_form_on_contiguous_tensors(coracle, shape, dtype):
    from sapa_amd import _lib
    B, G, dq, cg, H, W, P, s, oscale = shape
    q, key, v, off, _ = make(gen(230), shape[:8], off_scale=oscale)
    q, key, v, off = (t.to(dtype) for t in (q, key, v, off))
    want = coracle.deform_sapa_fused(q.float(), key.float(), v.float(), off.float(), P, s, G, 'f32')
    got = sapa_amd.deform_sapa_fused(*dev(q, key, v, off), P, s, G, matrix_form=True)
    kernel = _lib.last_kernel()
    assert got.is_contiguous() and got.dtype == dtype and got.shape == want.shape
    if dtype == torch.float32:
        assert kernel == 'deform_fused_wmat_kernel'
        if dq <= 8:
            assert_f32_close(got, want, 'matrix form')
        else:   # the reference's own check tolerance (deformsapa/deformsapa/forward_check.py)
            torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-5)
        # the reference's order of sums on request
        plain = sapa_amd.deform_sapa_fused(*dev(q, key, v, off), P, s, G, matrix_form=False)
        assert _lib.last_kernel() != kernel
        assert_f32_close(plain, want, 'reference order')
        auto = sapa_amd.deform_sapa_fused(*dev(q, key, v, off), P, s, G)
        assert _lib.last_kernel() == kernel and torch.equal(auto, got)
    else:
        assert kernel == ('deform_fused_wmat16_kernel' if dq % 8 == 0 and cg % 8 == 0 else 'deform_fused_wmat_kernel')
        assert_rel_rms_close(got.float(), want, BF16_REL if dtype == torch.bfloat16 else F16_REL, 'matrix form')
        # 16-bit tensors take it by default
        auto = sapa_amd.deform_sapa_fused(*dev(q, key, v, off), P, s, G)
        assert _lib.last_kernel() == kernel and torch.equal(auto, got)
        sapa_amd.deform_sapa_fused(*dev(q, key, v, off), P, s, G, matrix_form=False)
        assert _lib.last_kernel() != kernel
    # the offsets read in place from the low-res convolution output (sapa_deform.py:44-47)
    from sapa_amd.deform_func import expand_offset
    for layout in ('pixel_shuffle', 'nearest'):
        lo = _lowres_offsets(gen(233), shape[:8], layout, dtype=dtype).to(DEV)
        hi = expand_offset(lo, s, layout).contiguous()
        a = sapa_amd.deform_sapa_fused(*dev(q, key, v), hi, P, s, G, matrix_form=True)
        b = sapa_amd.deform_sapa_fused(*dev(q, key, v), lo, P, s, G, layout, matrix_form=True)
        assert _lib.last_kernel() == kernel and torch.equal(a, b), layout


def test_deform_fused_matrix_form_limits():
    """Too few points for the matrix form to pay, fp64, and the low-res offset
    layouts stay on the contiguous-layout kernels; asking for it explicitly raises."""
    from sapa_amd import _lib
    shape = (1, 2, 8, 8, 6, 7, 3, 2)
    q, key, v, off, _ = make(gen(231), shape)
    with pytest.raises(_lib.SapaUnsupported):
        sapa_amd.deform_sapa_fused(*dev(q, key, v, off), 3, 2, 2, matrix_form=True)
    h = sapa_amd.deform_sapa_fused(*dev(*(t.half() for t in (q, key, v, off))), 3, 2, 2)
    assert _lib.last_kernel() not in ('deform_fused_wmat_kernel', 'deform_fused_wmat16_kernel') and h.dtype == torch.float16
    q, key, v, off, _ = make(gen(232), (1, 2, 8, 8, 6, 7, 17, 2), dtype=torch.float64)
    with pytest.raises(_lib.SapaUnsupported):
        sapa_amd.deform_sapa_fused(*dev(q, key, v, off), 17, 2, 2, matrix_form=True)


def test_golden_vectors():
    G = golden()
    t = lambda a: torch.from_numpy(a)
    for tag in ('d_p5s2', 'd_p9s1'):
        B, Gr, dq, cg, H, W, P, s = (int(v) for v in G[f'{tag}.cfg'])
        q, key, v, off, attn = (t(G[f'{tag}.{n}']) for n in ('q', 'key', 'v', 'off', 'attn'))
        assert torch.equal(sapa_amd.deform_qk(*dev(q, key, off), P, s, Gr).cpu(), t(G[f'{tag}.dqk'])), tag
        assert torch.equal(sapa_amd.deform_av(*dev(attn, v, off), P, s, Gr).cpu(), t(G[f'{tag}.dav'])), tag
        assert_f32_close(sapa_amd.deform_sapa_fused(*dev(q, key, v, off), P, s, Gr).cpu(),
                         t(G[f'{tag}.dfused']), tag)


def test_regular_grid_offsets_reduce_to_sapa_b():
    """G=1, P=K*K, integer offsets on the window grid: the sampled operators
    equal the window operators bit for bit (weights are exactly 1,0,0,0)."""
    g = gen(202)
    B, d, C, H, W, K, s = 2, 6, 5, 9, 11, 5, 2
    q, key, v = randn(g, B, d, H * s, W * s), randn(g, B, d, H, W), randn(g, B, C, H, W)
    attn = randn(g, B, K * K, H * s, W * s)
    off = torch.zeros(B, 2 * K * K, H * s, W * s)
    for ky in range(K):
        for kx in range(K):
            off[:, 2 * (ky * K + kx)] = kx - K // 2
            off[:, 2 * (ky * K + kx) + 1] = ky - K // 2
    a = sapa_amd.deform_qk(*dev(q, key, off), K * K, s, 1)
    assert torch.equal(a.view(B, K * K, H * s, W * s), sapa_amd.qk(*dev(q, key), K, s))
    b = sapa_amd.deform_av(attn.view(B, 1, K * K, H * s, W * s).to(DEV), v.to(DEV), off.to(DEV), K * K, s, 1)
    assert torch.equal(b, sapa_amd.av(*dev(attn, v), K, s))
    c = sapa_amd.deform_sapa_fused(*dev(q, key, v, off), K * K, s, 1)
    assert_f32_close(c.cpu(), sapa_amd.sapa_fused(*dev(q, key, v), K, s).cpu(), 'fused families')


def test_guard_and_borders(coracle):
    """Offsets that push samples across every border, onto exact integers and
    onto the guard's edges (-1 and H): indices must still match exactly."""
    g = gen(203)
    shape = (1, 2, 3, 2, 5, 6, 8, 2)
    B, G, dq, cg, H, W, P, s = shape
    q, key, v, off, attn = make(g, shape, off_scale=4.0)
    off[:, :, ::3, ::2] = torch.round(off[:, :, ::3, ::2])          # exact integers
    off[0, 0] = -1.0 - torch.arange(W * s).div(s, rounding_mode='floor').float()  # kw == -1 exactly
    off[0, 3] = float(H)                                             # kh >= H
    got = sapa_amd.deform_qk(*dev(q, key, off), P, s, G).cpu()
    assert torch.equal(got, coracle.deform_qk(q, key, off, P, s, G, 'f32'))
    assert torch.count_nonzero(got[0, 0, 0]) == 0
    got = sapa_amd.deform_av(*dev(attn, v, off), P, s, G).cpu()
    assert torch.equal(got, coracle.deform_av(attn, v, off, P, s, G, 'f32'))


@pytest.mark.parametrize('dtype,rel', [(torch.bfloat16, BF16_REL), (torch.float16, F16_REL)])
def test_16bit_dtypes(coracle, dtype, rel):
    shape = SHAPES[2]
    B, G, dq, cg, H, W, P, s = shape
    q, key, v, off, attn = (x.to(dtype) for x in make(gen(204), shape))
    attn = F.softmax(attn.float(), 2).to(dtype)
    qf, kf, vf, of, af = (x.float() for x in (q, key, v, off, attn))
    got = sapa_amd.deform_qk(*dev(q, key, off), P, s, G)
    assert got.dtype == dtype
    assert_rel_rms_close(got.float(), coracle.deform_qk(qf, kf, of, P, s, G, 'f32a64'), rel, 'dqk')
    got = sapa_amd.deform_av(*dev(attn, v, off), P, s, G)
    assert_rel_rms_close(got.float(), coracle.deform_av(af, vf, of, P, s, G, 'f32a64'), rel, 'dav')
    got = sapa_amd.deform_sapa_fused(*dev(q, key, v, off), P, s, G)
    want = coracle.deform_sapa_fused(qf, kf, vf, of, P, s, G, 'f32')
    assert_rel_rms_close(got.float(), want, rel, 'dfused')


def test_fp64(coracle):
    shape = SHAPES[0]
    B, G, dq, cg, H, W, P, s = shape
    q, key, v, off, attn = make(gen(205), shape, dtype=torch.float64)
    assert torch.equal(sapa_amd.deform_qk(*dev(q, key, off), P, s, G).cpu(),
                       coracle.deform_qk(q, key, off, P, s, G, 'f64'))
    assert torch.equal(sapa_amd.deform_av(*dev(attn, v, off), P, s, G).cpu(),
                       coracle.deform_av(attn, v, off, P, s, G, 'f64'))
    torch.testing.assert_close(sapa_amd.deform_sapa_fused(*dev(q, key, v, off), P, s, G).cpu(),
                               coracle.deform_sapa_fused(q, key, v, off, P, s, G, 'f64'),
                               rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize('shape', [SHAPES[0], SHAPES[4]], ids=[IDS[0], IDS[4]])
def test_backward_vs_oracle(coracle, shape):
    B, G, dq, cg, H, W, P, s = shape
    for dt, tol in ((torch.float64, dict(rtol=1e-10, atol=1e-11)), (torch.float32, dict(rtol=1e-4, atol=1e-4))):
        g = gen(206)
        q, key, v, off, attn = make(g, shape, dtype=dt)
        go = randn(g, B, G, P, H * s, W * s, dtype=dt)
        qd, kd, od = (x.to(DEV).requires_grad_() for x in (q, key, off))
        sapa_amd.deform_qk(qd, kd, od, P, s, G).backward(go.to(DEV))
        gq, gk, goff = coracle.deform_qk_backward(go.double(), q.double(), key.double(), off.double(), P, s, G, 'f64')
        if dt == torch.float64:
            torch.testing.assert_close(qd.grad.cpu().double(), gq, **tol)
            torch.testing.assert_close(kd.grad.cpu().double(), gk, **tol)
            torch.testing.assert_close(od.grad.cpu().double(), goff, **tol)
        else:
            # fp32 coordinates differ from float64 ones in the last bit: compare
            # with the oracle run in fp32 arithmetic instead
            gq32, gk32, goff32 = coracle.deform_qk_backward(go, q, key, off, P, s, G, 'f32')
            torch.testing.assert_close(qd.grad.cpu(), gq32, **tol)
            torch.testing.assert_close(kd.grad.cpu(), gk32, **tol)
            torch.testing.assert_close(od.grad.cpu(), goff32, **tol)

        go = randn(g, B, G * cg, H * s, W * s, dtype=dt)
        ad, vd, od = (x.to(DEV).requires_grad_() for x in (attn, v, off))
        sapa_amd.deform_av(ad, vd, od, P, s, G).backward(go.to(DEV))
        mode = 'f64' if dt == torch.float64 else 'f32'
        ga, gv, goff = coracle.deform_av_backward(go, attn, v, off, P, s, G, mode)
        torch.testing.assert_close(ad.grad.cpu(), ga, **tol)
        torch.testing.assert_close(vd.grad.cpu(), gv, **tol)
        torch.testing.assert_close(od.grad.cpu(), goff, **tol)


SEPARATE_16BIT = [(2, 2, 8, 12, 9, 11, 9, 2, 1.0), (1, 4, 5, 3, 7, 6, 17, 2, 6.0), (1, 1, 4, 6, 5, 4, 5, 4, 2.0),
                  (1, 2, 6, 4, 10, 9, 13, 1, 1.5), (1, 2, 16, 64, 8, 10, 25, 2, 1.0)]


@pytest.mark.parametrize('dtype,rel', [(torch.bfloat16, 1.5e-2), (torch.float16, 2e-3)])
@pytest.mark.parametrize('shape', SEPARATE_16BIT, ids=['-'.join(map(str, s)) for s in SEPARATE_16BIT])
def test_separate_backward_16bit_native(coracle, shape, dtype, rel):
    """deform_qk / deform_av backward on f16 / bf16 tensors through the entry points
    that read and write them as they are (no fp32 copies of the features): every
    gradient against the float64 oracle on the rounded inputs, one rounding of the
    result; and the native path, not the widened fallback, served the call."""
    from sapa_amd import deform_func
    B, G, dq, cg, H, W, P, s, oscale = shape
    g = gen(208)
    q, key, v, off, attn = make(g, shape[:8], dtype=dtype, off_scale=oscale)
    go_qk = randn(g, B, G, P, H * s, W * s).to(dtype)
    go_av = randn(g, B, G * cg, H * s, W * s).to(dtype)
    d64 = lambda *ts: [t.double() for t in ts]

    # the native entry points take these configurations
    assert deform_func._backward_16bit('sapa_deform_qk_backward_ws', go_qk.to(DEV), q.to(DEV), key.to(DEV),
                                       off.to(DEV), P, s, G, (True, True, True)) is not None
    qd, kd, od = (x.to(DEV).requires_grad_() for x in (q, key, off))
    sapa_amd.deform_qk(qd, kd, od, P, s, G).backward(go_qk.to(DEV))
    want = coracle.deform_qk_backward(*d64(go_qk, q, key, off), P, s, G, 'f64')
    for got, w, name in zip((qd.grad, kd.grad, od.grad), want, ('grad_query', 'grad_key', 'grad_offset')):
        assert got.dtype == dtype
        assert_rel_rms_close(got.float().cpu(), w.float(), rel, f'deform_qk {name}')

    ad, vd, od = (x.to(DEV).requires_grad_() for x in (attn, v, off))
    sapa_amd.deform_av(ad, vd, od, P, s, G).backward(go_av.to(DEV))
    want = coracle.deform_av_backward(*d64(go_av, attn, v, off), P, s, G, 'f64')
    for got, w, name in zip((ad.grad, vd.grad, od.grad), want, ('grad_attn', 'grad_value', 'grad_offset')):
        assert got.dtype == dtype
        assert_rel_rms_close(got.float().cpu(), w.float(), rel, f'deform_av {name}')


# B, G, dq, cg, H, W, P, s, offset scale: partial tiles and chunks; offsets beyond the
# LDS window; s = 4 and s = 1
# (B, G, d, cg, H, W, P, s, offset scale).  The first four: one shape the matrix-form
# stage serves and three it does not (d or cg not a multiple of 4: the chain of
# separate kernels).  The rest go through the matrix-form stage: two passes over the
# tile (P > 16), s = 4 and s = 1, offsets far outside the window, odd widths (tile
# rows that are not whole vectors), two value chunks with a ragged second one, 64
# query / key channels per group, tiles that stick out of the image.
BACKWARD_SHAPES = [(2, 2, 8, 12, 9, 11, 9, 2, 1.0), (1, 4, 5, 3, 7, 6, 17, 2, 6.0),
                   (1, 1, 4, 6, 5, 4, 5, 4, 2.0), (1, 2, 6, 4, 10, 9, 13, 1, 1.5),
                   (1, 2, 16, 32, 8, 10, 25, 2, 1.0), (1, 2, 8, 8, 5, 6, 17, 4, 2.0),
                   (2, 1, 12, 20, 9, 7, 7, 1, 1.5), (1, 2, 8, 16, 7, 9, 21, 2, 7.0),
                   (1, 1, 32, 72, 6, 5, 5, 2, 1.0), (1, 1, 64, 16, 5, 7, 32, 2, 1.0),
                   (1, 3, 4, 4, 5, 5, 3, 2, 9.0)]


@pytest.mark.parametrize('dtype,tol', [(torch.float32, dict(rtol=1e-4, atol=2e-5)),
                                        (torch.bfloat16, 1.5e-2), (torch.float16, 2e-3)])
@pytest.mark.parametrize('shape', BACKWARD_SHAPES, ids=['-'.join(map(str, s)) for s in BACKWARD_SHAPES])
def test_deform_fused_backward_entry_point(coracle, shape, dtype, tol):
    """sapa_deform_fused_backward through the C ABI: the four gradients against the
    float64 oracle chain on the same (rounded) inputs; fp32 intermediates for 16-bit
    tensors, only the gradients themselves are rounded to 16 bits.  Offsets sit away
    from integers, where the bilinear sample has a kink."""
    from sapa_amd import _lib
    B, G, dq, cg, H, W, P, s, oscale = shape
    g = gen(240)
    q, key, v, off, _ = make(g, shape[:8], off_scale=oscale)
    frac = off - off.floor()
    off = off.floor() + frac.clamp(0.2, 0.8)        # the 16-bit rounding must not cross an integer
    go = randn(g, B, G * cg, H * s, W * s)
    q, key, v, off, go = (t.to(dtype) for t in (q, key, v, off, go))
    qd, kd, vd, od, god = dev(q, key, v, off, go)
    h = _lib.lib()
    args = (B, G * dq, G * cg, H, W, P, s, G, _lib.DTYPES[dtype])
    nbytes = h.sapa_deform_fused_backward_workspace(*args)
    assert nbytes > 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    grads = [torch.full_like(t, float('nan')) for t in (qd, kd, vd, od)]
    assert _lib.call_status('sapa_deform_fused_backward', DEV, _lib.ptr(god), _lib.ptr(qd), _lib.ptr(kd),
                            _lib.ptr(vd), _lib.ptr(od), _lib.ptr(ws), *(_lib.ptr(t) for t in grads), *args) == 0
    want = deform_fused_backward_oracle(coracle, go.float(), q.float(), key.float(), v.float(), off.float(), P, s, G)
    for got, w, name in zip(grads, want, ('grad_query', 'grad_key', 'grad_value', 'grad_offset')):
        assert torch.isfinite(got).all(), name
        if dtype == torch.float32:
            torch.testing.assert_close(got.cpu().double(), w, msg=lambda m: f'{name}: {m}', **tol)
        else:
            assert_rel_rms_close(got.float().cpu(), w, tol, f'{name} {dtype}')
    # only grad_key and grad_offset wanted: the other buffers stay as they are
    gq2, gv2 = torch.full_like(qd, 7.0), torch.full_like(vd, 7.0)
    gk2, go2 = torch.full_like(kd, float('nan')), torch.full_like(od, float('nan'))
    assert _lib.call_status('sapa_deform_fused_backward', DEV, _lib.ptr(god), _lib.ptr(qd), _lib.ptr(kd),
                            _lib.ptr(vd), _lib.ptr(od), _lib.ptr(ws), None, _lib.ptr(gk2), None, _lib.ptr(go2),
                            *args) == 0
    assert (gq2 == 7).all() and (gv2 == 7).all() and torch.equal(go2, grads[3])
    # float atomics: the order of the fp32 sums varies from run to run, and a 16-bit
    # result may then round to the neighbouring number
    again = dict(rtol={torch.float32: 1e-5, torch.float16: 1.1 * 2.0 ** -10, torch.bfloat16: 1.1 * 2.0 ** -7}[dtype],
                 atol=1e-6)
    torch.testing.assert_close(gk2.float(), grads[1].float(), **again)
    # the autograd route takes the same entry point, also with the offsets read in
    # place from a low-res tensor (their gradient is folded back to its layout)
    leaves = [t.clone().requires_grad_() for t in (qd, kd, vd, od)]
    sapa_amd.deform_sapa_fused(*leaves, P, s, G).backward(god)
    for leaf, got, name in zip(leaves, grads, ('grad_query', 'grad_key', 'grad_value', 'grad_offset')):
        torch.testing.assert_close(leaf.grad.float(), got.float(), msg=lambda m: f'{name}: {m}', **again)


def test_deform_fused_backward_limits():
    from sapa_amd import _lib
    h = _lib.lib()
    f32, f64 = _lib.DTYPES[torch.float32], _lib.DTYPES[torch.float64]
    assert h.sapa_deform_fused_backward_workspace(1, 8, 8, 4, 4, 9, 3, 2, f32) == 0     # up_factor 3
    assert h.sapa_deform_fused_backward_workspace(1, 8, 8, 4, 4, 9, 2, 2, f64) == 0
    assert h.sapa_deform_fused_backward_workspace(1, 8, 8, 4, 4, 49, 2, 2, f32) == 0    # many points
    x = torch.zeros(1, 8, 8, 8, device=DEV)
    lo = torch.zeros(1, 8, 4, 4, device=DEV)
    off = torch.zeros(1, 2 * 2 * 9, 12, 12, device=DEV)
    ws = torch.empty(256, dtype=torch.uint8, device=DEV)
    assert _lib.call_status('sapa_deform_fused_backward', DEV, _lib.ptr(x), _lib.ptr(x), _lib.ptr(lo), _lib.ptr(lo),
                            _lib.ptr(off), _lib.ptr(ws), _lib.ptr(x), None, None, None,
                            1, 8, 8, 4, 4, 9, 3, 2, f32) == _lib.UNSUPPORTED
    # such configurations still train through the separate backward entry points
    q = torch.randn(1, 8, 12, 12, device=DEV, requires_grad=True)
    k = torch.randn(1, 8, 4, 4, device=DEV, requires_grad=True)
    sapa_amd.deform_sapa_fused(q, k, k.detach(), off, 9, 3, 2).sum().backward()
    assert torch.isfinite(q.grad).all() and torch.isfinite(k.grad).all()


def test_gradcheck_reference_shapes():
    """deformsapa/deformsapa/grad_check.py:8-35: float64 gradcheck at its
    shapes, offsets in [0,1) so no sample sits on a bilinear kink.  The
    gradient of the sampled tensor is accumulated with atomics (as in the
    reference, deform_qk_cuda_kernel.cu:105), so two runs may differ in the
    last bits: nondet_tol allows for that."""
    from torch.autograd import gradcheck
    g = gen(207)
    b, h, w, c, P, s, G = 2, 3, 4, 16, 5, 2, 4
    r = lambda *sh: torch.rand(*sh, generator=g, dtype=torch.float64).to(DEV).requires_grad_()
    q, k, o = r(b, c, s * h, s * w), r(b, c, h, w), r(b, G * P * 2, s * h, s * w)
    assert gradcheck(sapa_amd.deform_qk, (q, k, o, P, s, G), nondet_tol=1e-10)
    a = randn(g, b, G, P, s * h, s * w, dtype=torch.float64).to(DEV).requires_grad_()
    v = randn(g, b, c, h, w, dtype=torch.float64).to(DEV).requires_grad_()
    assert gradcheck(sapa_amd.deform_av, (a, v, o, P, s, G), nondet_tol=1e-10)
    assert gradcheck(sapa_amd.deform_sapa_fused, (q, k, v, o, P, s, G), eps=1e-5, atol=1e-6,
                     nondet_tol=1e-10)


def test_sapa_deform_module(coracle):
    """SAPADeform at the module's defaults (P=9, G=4, pixel-shuffled offsets,
    sapa_deform.py:8-9,44-45), fused and three-step, against the oracle fed
    with the same projections."""
    from deformsapa import deform_av, deform_qk
    g = gen(208)
    torch.manual_seed(2)
    m = sapa_amd.SAPADeform(16, embedding_dim=8).to(DEV)
    torch.nn.init.normal_(m.offset.weight, std=0.3)   # spread the samples out
    y, x = randn(g, 2, 16, 12, 20), randn(g, 2, 16, 6, 10)
    with torch.no_grad():
        out = m(y.to(DEV), x.to(DEV))
        q, k = m.q(y.to(DEV)), m.k(x.to(DEV))
        off = F.pixel_shuffle(m.offset(x.to(DEV)), 2).contiguous()
        out3 = deform_av(F.softmax(deform_qk(q, k, off, 9, 2, 4), dim=2), x.to(DEV), off, 9, 2, 4)
    assert out.shape == (2, 16, 12, 20)
    want = coracle.deform_sapa_fused(q.cpu(), k.cpu(), x, off.cpu(), 9, 2, 4, 'f32')
    assert_f32_close(out.cpu(), want, 'SAPADeform fused')
    assert_f32_close(out3.cpu(), want, 'SAPADeform three-step')
    # nearest-interpolated offsets: the fused module reads the low-res tensor in place
    m2 = sapa_amd.SAPADeform(16, embedding_dim=8, high_offset=False, norm=False, fused=False).to(DEV)
    torch.nn.init.normal_(m2.offset.weight, std=0.3)
    with torch.no_grad():
        out2 = m2(y.to(DEV), x.to(DEV))
        m2.fused = True
        out2f = m2(y.to(DEV), x.to(DEV))
    assert out2.shape == (2, 16, 12, 20)
    assert_f32_close(out2f.cpu(), out2.cpu(), 'SAPADeform nearest offsets, fused vs three-step')


def test_module_trains():
    torch.manual_seed(3)
    m = sapa_amd.SAPADeform(16, embedding_dim=8).to(DEV)
    y = torch.randn(2, 16, 12, 16, device=DEV)
    x = torch.randn(2, 16, 6, 8, device=DEV, requires_grad=True)
    m(y, x).square().mean().backward()
    for n, p in m.named_parameters():
        assert p.grad is not None and torch.isfinite(p.grad).all(), n
    assert x.grad is not None and x.grad.abs().sum() > 0


def _lowres_offsets(g, shape, layout, dtype=torch.float32):
    B, G, dq, cg, H, W, P, s = shape
    ch = 2 * G * P * (s * s if layout == 'pixel_shuffle' else 1)
    return randn(g, B, ch, H, W, dtype=dtype) * 1.5


@pytest.mark.parametrize('layout', ['pixel_shuffle', 'nearest'])
@pytest.mark.parametrize('shape', [SHAPES[0], SHAPES[2], SHAPES[4], SHAPES[6]],
                         ids=[IDS[0], IDS[2], IDS[4], IDS[6]])
def test_offsets_read_in_place_match_materialised(layout, shape):
    """Offsets read from the low-res convolution output (sapa_deform.py:44-47)
    give the very bits of pixel_shuffle / interpolate followed by the
    hi-res-offset operators, for all three forward entry points and for both
    the LDS-windowed (s in 1, 2, 4) and the global-memory kernels (s = 3)."""
    from sapa_amd import _lib
    from sapa_amd.deform_func import OFFSET_LAYOUTS, expand_offset
    B, G, dq, cg, H, W, P, s = shape
    g = gen(300 + s)
    q, key, v, _, attn = make(g, shape)
    lo = _lowres_offsets(g, shape, layout)
    q, key, v, attn, lo = dev(q, key, v, attn, lo)
    hi = expand_offset(lo, s, layout).contiguous()
    code = OFFSET_LAYOUTS[layout]
    dt = _lib.dtype_code(q)

    want = sapa_amd.deform_qk(q, key, hi, P, s, G)
    got = torch.empty_like(want)
    _lib.call('sapa_deform_qk_forward_from', q.device, _lib.ptr(q), _lib.ptr(key), _lib.ptr(lo),
              _lib.ptr(got), B, G * dq, H, W, P, s, G, code, dt)
    assert torch.equal(got, want), 'deform_qk ' + layout

    want = sapa_amd.deform_av(attn, v, hi, P, s, G)
    got = torch.empty_like(want)
    _lib.call('sapa_deform_av_forward_from', q.device, _lib.ptr(attn), _lib.ptr(v), _lib.ptr(lo),
              _lib.ptr(got), B, G * cg, H, W, P, s, G, code, dt)
    assert torch.equal(got, want), 'deform_av ' + layout

    want = sapa_amd.deform_sapa_fused(q, key, v, hi, P, s, G)
    got = sapa_amd.deform_sapa_fused(q, key, v, lo, P, s, G, layout)
    assert torch.equal(got, want), 'fused ' + layout


def test_offsets_read_in_place_fp64_and_bf16():
    from sapa_amd.deform_func import expand_offset
    shape = SHAPES[2]
    B, G, dq, cg, H, W, P, s = shape
    for dtype in (torch.float64, torch.bfloat16):
        g = gen(310)
        q, key, v, _, _ = make(g, shape, dtype=dtype)
        lo = _lowres_offsets(g, shape, 'pixel_shuffle', dtype=dtype)
        q, key, v, lo = dev(q, key, v, lo)
        # on either kernel family (bf16: the matrix form by default) the result is the
        # same bit for bit as with the hi-res offsets written out first
        for mf in (None, False):
            want = sapa_amd.deform_sapa_fused(q, key, v, expand_offset(lo, s, 'pixel_shuffle').contiguous(),
                                              P, s, G, matrix_form=mf)
            got = sapa_amd.deform_sapa_fused(q, key, v, lo, P, s, G, 'pixel_shuffle', matrix_form=mf)
            assert torch.equal(got, want), f'{dtype} matrix_form={mf}'


@pytest.mark.parametrize('layout', ['pixel_shuffle', 'nearest'])
def test_offsets_read_in_place_gradients(layout):
    """Gradients with respect to the low-res offset tensor equal autograd
    through pixel_shuffle / interpolate into the hi-res-offset operator."""
    from sapa_amd.deform_func import expand_offset
    shape = (1, 2, 3, 2, 4, 5, 4, 2)
    B, G, dq, cg, H, W, P, s = shape
    g = gen(320)
    q, key, v, _, _ = make(g, shape, dtype=torch.float64)
    lo = _lowres_offsets(g, shape, layout, dtype=torch.float64)
    q, key, v, lo = dev(q, key, v, lo)
    up = randn(g, B, G * cg, H * s, W * s, dtype=torch.float64).to(DEV)
    grads = []
    for direct in (True, False):
        ts = [t.clone().requires_grad_(True) for t in (q, key, v, lo)]
        if direct:
            out = sapa_amd.deform_sapa_fused(ts[0], ts[1], ts[2], ts[3], P, s, G, layout)
        else:
            out = sapa_amd.deform_sapa_fused(ts[0], ts[1], ts[2],
                                             expand_offset(ts[3], s, layout).contiguous(), P, s, G)
        (out * up).sum().backward()
        grads.append([t.grad for t in ts])
    for a, b, name in zip(grads[0], grads[1], ('q', 'key', 'value', 'offset')):
        assert a.shape == b.shape
        torch.testing.assert_close(a, b, rtol=1e-10, atol=1e-12, msg=name + ' ' + layout)


def test_offset_layout_is_validated():
    g = gen(330)
    q, key, v, off, _ = make(g, SHAPES[0])
    q, key, v, off = dev(q, key, v, off)
    with pytest.raises(ValueError):
        sapa_amd.deform_sapa_fused(q, key, v, off, 5, 2, 4, 'bilinear')
    with pytest.raises(AssertionError):
        sapa_amd.deform_sapa_fused(q, key, v, off, 5, 2, 4, 'nearest')   # hi-res shape, low-res layout


# B, G, dq, cg, H, W, P, s: several tiles per image, ragged edges, every scale
# factor with an LDS instance, many points (larger dynamic LDS)
LDS_GRAD_SHAPES = [(1, 2, 5, 9, 19, 21, 9, 2), (1, 1, 3, 4, 6, 7, 25, 2), (1, 2, 4, 4, 17, 18, 4, 1),
                   (1, 2, 3, 3, 5, 6, 6, 4), (2, 4, 8, 16, 9, 9, 9, 2)]


@pytest.mark.parametrize('off_scale', [1.5, 4.0], ids=['offsets1.5', 'offsets4'])
@pytest.mark.parametrize('shape', LDS_GRAD_SHAPES, ids=['-'.join(map(str, s)) for s in LDS_GRAD_SHAPES])
def test_lds_gradient_kernels_vs_oracle(coracle, shape, off_scale):
    """fp32 gradients of both sampled operators from the LDS kernels (offset
    gradient by gather, low-res gradient by fixed-point scatter) against the
    float64 oracle; offsets of scale 4 push many taps out of the LDS window
    onto the per-term path."""
    B, G, dq, cg, H, W, P, s = shape
    g = gen(340)
    q, key, v, off, attn = make(g, shape, off_scale=off_scale)
    go_qk = randn(g, B, G, P, H * s, W * s)
    go_av = randn(g, B, G * cg, H * s, W * s)
    qd, kd, od = (x.to(DEV).requires_grad_() for x in (q, key, off))
    sapa_amd.deform_qk(qd, kd, od, P, s, G).backward(go_qk.to(DEV))
    gq, gk, goff = coracle.deform_qk_backward(go_qk.double(), q.double(), key.double(),
                                              off.double(), P, s, G, 'f64')
    tol = dict(rtol=1e-4, atol=5e-5)
    torch.testing.assert_close(qd.grad.cpu().double(), gq, **tol)
    torch.testing.assert_close(kd.grad.cpu().double(), gk, **tol)
    torch.testing.assert_close(od.grad.cpu().double(), goff, **tol)
    ad, vd, od = (x.to(DEV).requires_grad_() for x in (attn, v, off))
    sapa_amd.deform_av(ad, vd, od, P, s, G).backward(go_av.to(DEV))
    ga, gv, goff = coracle.deform_av_backward(go_av.double(), attn.double(), v.double(),
                                              off.double(), P, s, G, 'f64')
    torch.testing.assert_close(ad.grad.cpu().double(), ga, **tol)
    torch.testing.assert_close(vd.grad.cpu().double(), gv, **tol)
    torch.testing.assert_close(od.grad.cpu().double(), goff, **tol)


@pytest.mark.parametrize('magnitude', [1e-12, 1.0, 1e12])
def test_lowres_gradient_fixed_point_scaling(coracle, magnitude):
    """The fixed-point window sums rescale themselves to the data: the
    relative accuracy of grad_value does not depend on the magnitude of the
    incoming gradient, and one huge element does not wipe out the rest."""
    shape = (1, 2, 4, 8, 9, 10, 9, 2)
    B, G, dq, cg, H, W, P, s = shape
    g = gen(341)
    _, _, v, off, attn = make(g, shape)
    attn = torch.softmax(attn, dim=2)
    go = randn(g, B, G * cg, H * s, W * s) * magnitude
    go[0, 3, 5, 7] = 1e4 * magnitude
    ad, vd, od = (x.to(DEV).requires_grad_() for x in (attn, v, off))
    sapa_amd.deform_av(ad, vd, od, P, s, G).backward(go.to(DEV))
    _, gv, _ = coracle.deform_av_backward(go.double(), attn.double(), v.double(), off.double(),
                                          P, s, G, 'f64')
    got = vd.grad.cpu().double()
    scale = gv.abs().max()
    # per element: fp32 resolution of the element itself plus 2^-30 of the
    # largest magnitude in play
    err = (got - gv).abs()
    bound = 1e-5 * gv.abs() + 1e-9 * scale
    assert (err <= bound).all(), float((err - bound).max() / scale)


def test_lowres_gradient_integer_inputs_exact(coracle):
    """Integer-valued tensors with half-integer offsets: every term is a
    multiple of 1/4 and every sum is exact in fp32 and in the fixed-point
    window, so the result does not depend on the order of any add."""
    shape = (1, 2, 3, 4, 11, 13, 6, 2)
    B, G, dq, cg, H, W, P, s = shape
    g = gen(342)
    attn = torch.randint(-2, 3, (B, G, P, H * s, W * s), generator=g).float()
    go = torch.randint(-2, 3, (B, G * cg, H * s, W * s), generator=g).float()
    off = torch.randint(-7, 8, (B, 2 * G * P, H * s, W * s), generator=g).float() * 0.5
    v = torch.zeros(B, G * cg, H, W)
    runs = []
    for _ in range(2):
        ad, vd, od = (x.to(DEV) for x in (attn, v, off))
        vd.requires_grad_()
        sapa_amd.deform_av(ad, vd, od, P, s, G).backward(go.to(DEV))
        runs.append(vd.grad.cpu())
    _, gv, _ = coracle.deform_av_backward(go.double(), attn.double(), v.double(), off.double(),
                                          P, s, G, 'f64')
    assert torch.equal(runs[0].double(), gv)
    assert torch.equal(runs[0], runs[1])
