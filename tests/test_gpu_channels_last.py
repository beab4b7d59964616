"""GPU parity of the SAPA-B operators on tensors in torch.channels_last order
(served without a layout copy by the *_nhwc entry points of the C ABI) against
the CPU oracle and against the library's own contiguous path.

Bars: av bit-exact (the tap sum runs in the reference's order).  The channel
sums of the logits run in tree order, so qk / fused are compared with the
float64-accumulated oracle: within 1e-5 rel / 1e-6 abs for short sums (d <= 8);
for long sums (d = 64 ... 128, logits of magnitude 10 ... 30, whose fp32 spacing
alone is 1e-6 ... 2e-6) within 1e-5 relative to max(|b|, rms) for the logits
and within the reference's own check tolerance, allclose(atol=1e-5)
(sapa/sapa/forward_check.py:37-39), for the fused output -- the reference's
sequential fp32 sums sit at least as far from the float64 value.  16-bit
within the usual relative bars.
"""
import pytest
import torch
import torch.nn.functional as F

import sapa_amd
from helpers import BF16_REL, F16_REL, assert_f32_close, assert_rel_rms_close, gen, randn

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'
CL = torch.channels_last

# B, d, C, H, W, K, s: ragged against the 4x4-parent tiles, one / two / partial
# 64-channel chunks of key and value, every (K, s) the kernels are built for
SHAPES = [(2, 4, 8, 5, 7, 5, 2), (1, 64, 64, 8, 8, 5, 2), (1, 68, 72, 6, 9, 5, 2),
          (1, 8, 132, 3, 4, 3, 2), (2, 128, 4, 9, 5, 3, 2), (1, 16, 256, 1, 1, 5, 2),
          (1, 4, 4, 13, 2, 5, 2), (1, 8, 12, 6, 5, 7, 2), (1, 72, 68, 5, 6, 5, 4),
          (2, 4, 8, 3, 7, 7, 4), (1, 64, 64, 4, 4, 7, 4)]
IDS = ['-'.join(map(str, s)) for s in SHAPES]


def cl(*ts):
    return [t.to(DEV).contiguous(memory_format=CL) for t in ts]


def inputs(g, B, d, C, H, W, K, s=2, dtype=torch.float32):
    q, key, v = (randn(g, *sh).to(dtype) for sh in
                 ((B, d, s * H, s * W), (B, d, H, W), (B, C, H, W)))
    attn = F.softmax(randn(g, B, K * K, s * H, s * W), 1).to(dtype)
    return q, key, v, attn


@pytest.mark.parametrize('shape', SHAPES, ids=IDS)
def test_fp32_vs_oracle(coracle, shape):
    B, d, C, H, W, K, s = shape
    q, key, v, attn = inputs(gen(300), *shape)
    got = sapa_amd.qk(*cl(q, key), K, s)
    assert got.is_contiguous(memory_format=CL) and got.shape == (B, K * K, s * H, s * W)
    want = coracle.qk(q, key, K, s, 'f32a64')
    if d <= 8:
        assert_f32_close(got, want, 'qk')
    else:
        assert_rel_rms_close(got, want, 1e-5, 'qk')
    got = sapa_amd.qk_softmax(*cl(q, key), K, s)
    assert got.is_contiguous(memory_format=CL)
    torch.testing.assert_close(got.cpu(), coracle.softmax(want.float(), 1, 'f32'), rtol=1e-5,
                               atol=1e-7 if d <= 8 else 1e-5)
    got = sapa_amd.av(*cl(attn, v), K, s)
    assert got.is_contiguous(memory_format=CL) and got.shape == (B, C, s * H, s * W)
    # the sum over the K*K taps runs in the reference's order: same bits
    assert torch.equal(got.cpu(), coracle.av(attn, v, K, s, 'f32'))
    got = sapa_amd.sapa_fused(*cl(q, key, v), K, s)
    assert got.is_contiguous(memory_format=CL)
    want = coracle.sapa_fused(q, key, v, K, s, 'f32a64')
    if d <= 8:
        assert_f32_close(got, want, 'fused')
    else:
        torch.testing.assert_close(got.cpu().double(), want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize('dtype,rel', [(torch.bfloat16, BF16_REL), (torch.float16, F16_REL)])
@pytest.mark.parametrize('shape', SHAPES, ids=IDS)
def test_16bit_vs_oracle(coracle, shape, dtype, rel):
    """Shapes with d % 8 == 0 run on the 16-bit matrix-instruction kernel (16-bit
    windows in LDS, weights rounded to the tensor type before the aggregation),
    the others on the kernel that widens to fp32 in LDS."""
    B, d, C, H, W, K, s = shape
    q, key, v, attn = inputs(gen(301), *shape, dtype=dtype)
    qf, kf, vf, af = (x.float() for x in (q, key, v, attn))
    got = sapa_amd.qk(*cl(q, key), K, s)
    assert got.dtype == dtype and got.is_contiguous(memory_format=CL)
    assert_rel_rms_close(got.float(), coracle.qk(qf, kf, K, s, 'f32a64'), rel, 'qk')
    got = sapa_amd.qk_softmax(*cl(q, key), K, s)
    assert got.dtype == dtype and got.is_contiguous(memory_format=CL)
    want = coracle.softmax(coracle.qk(qf, kf, K, s, 'f32a64').float(), 1, 'f32')
    torch.testing.assert_close(got.float().cpu(), want, rtol=rel, atol=rel / 4)
    got = sapa_amd.av(*cl(attn, v), K, s)
    assert_rel_rms_close(got.float(), coracle.av(af, vf, K, s, 'f32a64'), rel, 'av')
    got = sapa_amd.sapa_fused(*cl(q, key, v), K, s)
    assert got.dtype == dtype and got.is_contiguous(memory_format=CL)
    assert_rel_rms_close(got.float(), coracle.sapa_fused(qf, kf, vf, K, s, 'f32a64'), rel, 'fused')


# Fused, channels-last 16-bit tensors, K = 5, s = 2, d and C multiples of 8, images of at least 2048 low-res
# cells: two dense products per 4 x 4 block of parents on the 16-bit matrix instructions.  (B, d, C, H, W): one
# 64-channel chunk of each; whole tiles; ragged tiles (H % 4 = 1, W % 4 = 2) and partial chunks; partial
# chunks of key and value; more than one key chunk; the FPN geometry.
DENSE16_CL_SHAPES = [(1, 8, 8, 46, 46), (2, 64, 64, 32, 64), (2, 24, 40, 45, 50), (1, 72, 136, 40, 56),
                     (1, 136, 24, 47, 44), (1, 16, 32, 100, 168)]


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('shape', DENSE16_CL_SHAPES, ids=['-'.join(map(str, s)) for s in DENSE16_CL_SHAPES])
def test_16bit_dense_window_kernel(coracle, shape, dtype):
    """Products of 16-bit values are exact in fp32, sums and softmax are fp32, the weights enter the
    aggregation as a 16-bit value plus a 16-bit remainder: what is left is the rounding of the result, at
    most half a 16-bit spacing (2^-8 resp. 2^-11 of the value) against the double-precision oracle."""
    B, d, C, H, W = shape
    g = gen(341)
    q, key, v = (randn(g, *sh).to(dtype) for sh in ((B, d, H * 2, W * 2), (B, d, H, W), (B, C, H, W)))
    half_ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
    got = sapa_amd.sapa_fused(*cl(q, key, v), 5, 2)
    assert sapa_amd._lib.last_kernel() == 'sapa_b_nhwc_wm16_kernel'
    assert got.dtype == dtype and got.shape == (B, C, 2 * H, 2 * W) and got.is_contiguous(memory_format=CL)
    exact = torch.cat([coracle.sapa_fused(q[i:i + 1].float(), key[i:i + 1].float(), v[i:i + 1].float(), 5, 2, 'f32a64')
                       for i in range(B)]).double()
    err = (got.float().cpu().double() - exact).abs()
    worst = (err / torch.maximum(exact.abs(), exact.square().mean().sqrt())).max().item()
    assert worst <= 1.05 * half_ulp, f'{shape} {dtype}: {worst / half_ulp:.2f} half-spacings'
    # zero query: every child weighs the 25 cells of its own window equally and the rest of the 8 x 8
    # window not at all -- the box filter of the value, zero padding counted.  Positive values, large on
    # the border cells, and a bar relative to each element.
    vp = v.float().abs() + 0.5
    for sl in ((slice(None), slice(None), 0), (slice(None), slice(None), -1),
               (slice(None), slice(None), slice(None), 0), (slice(None), slice(None), slice(None), -1)):
        vp[sl] *= 64.0
    vp = vp.to(dtype)
    got0 = sapa_amd.sapa_fused(*cl(torch.zeros_like(q), key, vp), 5, 2)
    assert sapa_amd._lib.last_kernel() == 'sapa_b_nhwc_wm16_kernel'
    box = F.interpolate(F.avg_pool2d(vp.double(), 5, 1, 2, count_include_pad=True), scale_factor=2)
    rel = ((got0.float().cpu().double() - box).abs() / box).max().item()
    assert rel <= 1.05 * half_ulp + 1e-6, f'{shape} {dtype} box filter: {rel / half_ulp:.2f} half-spacings'
    # a per-image bias of the query: key . (q + b) with nothing rounded in between
    if B * H * W <= 6000:
        bias = (randn(g, B, d) * 0.7).to(dtype)
        got_b = sapa_amd.sapa_fused(*cl(q, key, v), 5, 2, bias.to(DEV))
        assert sapa_amd._lib.last_kernel() == 'sapa_b_nhwc_wm16_kernel'
        qb = q.float() + bias.float()[:, :, None, None]
        exact_b = torch.cat([coracle.sapa_fused(qb[i:i + 1], key[i:i + 1].float(), v[i:i + 1].float(), 5, 2, 'f32a64')
                             for i in range(B)]).double()
        err = (got_b.float().cpu().double() - exact_b).abs()
        worst = (err / torch.maximum(exact_b.abs(), exact_b.square().mean().sqrt())).max().item()
        assert worst <= 1.05 * half_ulp, f'{shape} {dtype} with bias: {worst / half_ulp:.2f} half-spacings'


@pytest.mark.parametrize('dtype,rel', [(torch.bfloat16, BF16_REL), (torch.float16, F16_REL)])
@pytest.mark.parametrize('K,s', [(5, 2), (7, 4)])
def test_16bit_matches_contiguous_path_at_a_larger_shape(dtype, rel, K, s):
    """Several tiles per image, several images, two key chunks and a ragged
    value chunk: the 16-bit matrix-instruction kernel against the library's
    NCHW kernels on the same 16-bit values."""
    B, d, C, H, W = 3, 72, 100, 11, 14
    q, key, v, attn = inputs(gen(311), B, d, C, H, W, K, s, dtype=dtype)
    qd, kd, vd, ad = (t.to(DEV) for t in (q, key, v, attn))
    assert_rel_rms_close(sapa_amd.sapa_fused(*cl(q, key, v), K, s).float().contiguous(),
                         sapa_amd.sapa_fused(qd, kd, vd, K, s).float().cpu(), rel, 'fused')
    assert_rel_rms_close(sapa_amd.av(*cl(attn, v), K, s).float().contiguous(),
                         sapa_amd.av(ad, vd, K, s).float().cpu(), rel, 'av')
    assert_rel_rms_close(sapa_amd.qk(*cl(q, key), K, s).float().contiguous(),
                         sapa_amd.qk(qd, kd, K, s).float().cpu(), rel, 'qk')


def test_matches_contiguous_path_at_a_larger_shape():
    """Several tiles per image and several images: against the library's own
    NCHW kernels on the same values."""
    B, d, C, H, W, K = 3, 64, 96, 21, 30, 5
    q, key, v, attn = inputs(gen(302), B, d, C, H, W, K)
    qd, kd, vd, ad = (t.to(DEV) for t in (q, key, v, attn))
    torch.testing.assert_close(sapa_amd.sapa_fused(*cl(q, key, v), K, 2).contiguous(),
                               sapa_amd.sapa_fused(qd, kd, vd, K, 2), rtol=2e-5, atol=2e-5)
    assert torch.equal(sapa_amd.av(*cl(attn, v), K, 2).contiguous(), sapa_amd.av(ad, vd, K, 2))
    assert_rel_rms_close(sapa_amd.qk(*cl(q, key), K, 2), sapa_amd.qk(qd, kd, K, 2), 1e-5, 'qk')


def test_matches_contiguous_path_k7_s4():
    B, d, C, H, W, K, s = 2, 64, 80, 10, 13, 7, 4
    q, key, v, attn = inputs(gen(310), B, d, C, H, W, K, s)
    qd, kd, vd, ad = (t.to(DEV) for t in (q, key, v, attn))
    # two fp32 evaluations with different summation orders, each within 1e-5 of
    # the exact value: twice that between them
    torch.testing.assert_close(sapa_amd.sapa_fused(*cl(q, key, v), K, s).contiguous(),
                               sapa_amd.sapa_fused(qd, kd, vd, K, s), rtol=2e-5, atol=2e-5)
    assert torch.equal(sapa_amd.av(*cl(attn, v), K, s).contiguous(), sapa_amd.av(ad, vd, K, s))


def test_zero_query_is_the_box_filter():
    """q == 0: uniform weights 1/K^2, out-of-range neighbours in the denominator."""
    B, d, C, H, W, K = 1, 8, 12, 9, 10, 5
    g = gen(303)
    key, v = randn(g, B, d, H, W), randn(g, B, C, H, W)
    q = torch.zeros(B, d, 2 * H, 2 * W)
    got = sapa_amd.sapa_fused(*cl(q, key, v), K, 2).cpu()
    want = F.avg_pool2d(v.double(), K, 1, K // 2, count_include_pad=True)
    want = want.repeat_interleave(2, -2).repeat_interleave(2, -1)
    assert_f32_close(got, want, 'box filter')


def test_layout_errors():
    B, d, C, H, W, K = 1, 8, 8, 4, 4, 5
    q, key, v, attn = inputs(gen(304), B, d, C, H, W, K)
    qc, kc, vc = cl(q, key, v)
    with pytest.raises(RuntimeError, match='contiguous'):
        sapa_amd.sapa_fused(qc, key.to(DEV), vc, K, 2)            # mixed orders
    q9 = randn(gen(305), B, d, 2 * H, 2 * W)
    with pytest.raises(RuntimeError, match='channels_last'):
        sapa_amd.qk(*cl(q9, key), 9, 2)                           # no channels-last kernel for K = 9
    k6 = randn(gen(306), B, 6, H, W)
    q6 = randn(gen(307), B, 6, 2 * H, 2 * W)
    with pytest.raises(RuntimeError, match='channels_last'):
        sapa_amd.qk(*cl(q6, k6), K, 2)                            # channels not a multiple of 4


def test_backward_through_channels_last_forward():
    B, d, C, H, W, K = 2, 8, 12, 6, 7, 5
    q, key, v, _ = inputs(gen(308), B, d, C, H, W, K)
    go = randn(gen(309), B, C, 2 * H, 2 * W)
    grads = []
    for fmt in (torch.contiguous_format, CL):
        ts = [t.to(DEV).contiguous(memory_format=fmt).requires_grad_() for t in (q, key, v)]
        out = sapa_amd.sapa_fused(*ts, K, 2)
        out.backward(go.to(DEV).contiguous(memory_format=fmt))
        grads.append([t.grad for t in ts])
    for a, b, name in zip(grads[0], grads[1], ('query', 'key', 'value')):
        torch.testing.assert_close(b, a, rtol=1e-4, atol=1e-5, msg=lambda m: f'grad_{name}: {m}')


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('shape', [(2, 8, 5, 7), (1, 3, 1, 35), (3, 64, 12, 20), (2, 260, 9, 4), (1, 1, 6, 6)])
def test_layout_copy_kernel(shape, dtype):
    """sapa_layout_copy both ways, on shapes that take its 16-byte form and its element form:
    the same values as Tensor.contiguous(), in the requested order."""
    from sapa_amd import _lib
    x = randn(gen(330), *shape).to(dtype).to(DEV)
    to_cl = _lib.layout_copy(x, True)
    assert to_cl.is_contiguous(memory_format=CL) and torch.equal(to_cl, x)
    src = x.contiguous(memory_format=CL)
    back = _lib.layout_copy(src, False)
    assert back.is_contiguous() and torch.equal(back, x)
    if shape[1] > 1 and shape[2] * shape[3] > 1:
        # the library's kernel did these, not torch's copy
        out = torch.full_like(x, float('nan'))
        _lib.call('sapa_layout_copy', x.device, src.data_ptr(), out.data_ptr(), shape[0], shape[1],
                  shape[2] * shape[3], 0, x.element_size())
        assert torch.equal(out, x)


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_backward_of_channels_last_tensors_equals_contiguous(dtype):
    """The backward pass of channels_last operands runs on the contiguous kernels after the
    library's layout kernel: bit-identical gradients, each in the order of its tensor."""
    B, d, C, H, W, K = 2, 16, 24, 12, 20, 5
    q, key, v, _ = inputs(gen(331), B, d, C, H, W, K, dtype=dtype)
    go = randn(gen(332), B, C, 2 * H, 2 * W).to(dtype)
    grads = []
    for fmt in (torch.contiguous_format, CL):
        ts = [t.to(DEV).contiguous(memory_format=fmt).requires_grad_() for t in (q, key, v)]
        # (the forward kernels of the two layouts sum in different orders; the gradients are
        # taken with respect to the same operands either way)
        out = sapa_amd.sapa_fused(*ts, K, 2)
        gs = torch.autograd.grad(out, ts, go.to(DEV).contiguous(memory_format=fmt))
        grads.append(gs)
        for g in gs:
            assert g.is_contiguous(memory_format=fmt)
    for a, b, name in zip(grads[0], grads[1], ('query', 'key', 'value')):
        assert torch.equal(a, b), f'grad_{name}'


def test_module_in_channels_last_format():
    """A SAPA module in channels_last memory format: same result as the
    contiguous run, output in channels_last order, parameters get gradients."""
    torch.manual_seed(0)
    m = sapa_amd.SAPA(64, 64, up_factor=2, up_kernel_size=5, embedding_dim=32).to(DEV)
    g = gen(311)
    y, x = randn(g, 2, 64, 18, 22).to(DEV), randn(g, 2, 64, 9, 11).to(DEV)
    want = m(y, x)
    mc = m.to(memory_format=CL)
    yc, xc = y.contiguous(memory_format=CL), x.contiguous(memory_format=CL)
    got = mc(yc, xc)
    assert got.is_contiguous(memory_format=CL)
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-5)
    got.sum().backward()
    assert all(p.grad is not None for p in mc.parameters())
    unfused = sapa_amd.SAPA(64, 64, embedding_dim=32, fused=False).to(DEV)
    unfused.load_state_dict(m.state_dict())
    torch.testing.assert_close(unfused(yc, xc), want, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize('dtype,rel', [(torch.bfloat16, BF16_REL), (torch.float32, None)])
def test_heavy_tailed_query_k7_s4(coracle, dtype, rel):
    """The stress configuration in small: K = 7, s = 4, a tenth of the query
    drawn from Student-t(3) (logits with outliers), both memory orders against
    the float64-accumulated oracle on the rounded inputs."""
    B, d, C, H, W, K, s = 1, 64, 72, 6, 7, 7, 4
    g = gen(320)
    q, key, v, _ = inputs(g, B, d, C, H, W, K, s)
    z = randn(g, 4, *q.shape)
    t3 = z[0] / z[1:].pow(2).mean(0).sqrt()
    q = torch.where(torch.rand(q.shape, generator=g) < 0.1, t3, q)
    q, key, v = (t.to(dtype) for t in (q, key, v))
    want = coracle.sapa_fused(q.float(), key.float(), v.float(), K, s, 'f32a64')
    for got in (sapa_amd.sapa_fused(*cl(q, key, v), K, s),
                sapa_amd.sapa_fused(q.to(DEV), key.to(DEV), v.to(DEV), K, s)):
        if rel is None:
            torch.testing.assert_close(got.cpu().double().contiguous(), want, rtol=1e-5, atol=1e-5)
        else:
            assert_rel_rms_close(got.float(), want, rel, 'fused')


def test_random_configurations_match_contiguous_path():
    """24 seeded random shapes / window sizes / dtypes: the channels-last entry
    points (both kernels behind them) against the contiguous-layout ones."""
    import random
    rnd = random.Random(7)
    g = gen(330)
    for _ in range(24):
        K, s = rnd.choice([(3, 2), (5, 2), (7, 2), (5, 4), (7, 4)])
        B, H, W = rnd.randint(1, 2), rnd.randint(1, 13), rnd.randint(1, 14)
        d, C = 4 * rnd.randint(1, 20), 4 * rnd.randint(1, 36)
        dtype = rnd.choice([torch.float32, torch.bfloat16, torch.float16])
        q, key, v, attn = inputs(g, B, d, C, H, W, K, s, dtype=dtype)
        qd, kd, vd, ad = (t.to(DEV) for t in (q, key, v, attn))
        what = f'B{B} d{d} C{C} {H}x{W} K{K} s{s} {dtype}'
        fused_cl = sapa_amd.sapa_fused(*cl(q, key, v), K, s)
        av_cl = sapa_amd.av(*cl(attn, v), K, s)
        qk_cl = sapa_amd.qk(*cl(q, key), K, s)
        fused, av, qk = sapa_amd.sapa_fused(qd, kd, vd, K, s), sapa_amd.av(ad, vd, K, s), sapa_amd.qk(qd, kd, K, s)
        if dtype == torch.float32:
            assert torch.equal(av_cl.contiguous(), av), what
            torch.testing.assert_close(fused_cl.contiguous(), fused, rtol=2e-5, atol=2e-5, msg=what)
            assert_rel_rms_close(qk_cl, qk, 1e-5, what)
        else:
            rel = BF16_REL if dtype == torch.bfloat16 else F16_REL
            assert_rel_rms_close(av_cl.float(), av.float(), rel, what + ' av')
            assert_rel_rms_close(fused_cl.float(), fused.float(), rel, what + ' fused')
            assert_rel_rms_close(qk_cl.float(), qk.float(), rel, what + ' qk')


@pytest.mark.parametrize('dtype,tol', [(torch.float32, 1e-4), (torch.bfloat16, 6e-2)])
@pytest.mark.parametrize('norm', [True, False])
def test_module_emitting_channels_last(dtype, tol, norm):
    """SAPA(channels_last=True): projections that write q and k in
    channels_last order, the operator in that order, a channels_last result --
    same values as the default module on contiguous tensors."""
    torch.manual_seed(6)
    m = sapa_amd.SAPA(64, embedding_dim=16, norm=norm).to(DEV)
    # 16 bits: small projections, i.e. a smooth softmax -- two different 16-bit
    # pipelines for q and k are compared, and a sharp softmax would turn their
    # rounding differences into different winners
    std = 0.2 if dtype == torch.float32 else 0.03
    torch.nn.init.normal_(m.q.weight, std=std)
    torch.nn.init.normal_(m.k.weight, std=std)
    if norm:
        torch.nn.init.normal_(m.norm_y.weight, 1.0, 0.2)
        torch.nn.init.normal_(m.norm_x.bias, 0.0, 0.2)
    m = m.to(dtype)
    y = (torch.randn(2, 64, 18, 22, device=DEV) + 0.5).to(dtype)
    x = torch.randn(2, 64, 9, 11, device=DEV).to(dtype)
    with torch.no_grad():
        want = m(y, x)
        m.channels_last = True
        got = m(y, x)
        got_cl_in = m(y.contiguous(memory_format=CL), x.contiguous(memory_format=CL))
    assert got.shape == want.shape and got.is_contiguous(memory_format=CL)
    torch.testing.assert_close(got.float(), want.float(), rtol=tol, atol=tol)
    torch.testing.assert_close(got_cl_in.float(), want.float(), rtol=tol, atol=tol)


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('shape', [(2, 64, 9, 11), (1, 256, 40, 33), (3, 12, 5, 7), (2, 36, 1, 1),
                                   (1, 8, 130, 129)])
def test_channel_moments_kernel(dtype, shape):
    """The one-pass per-(image, channel) mean / variance kernel behind the folded
    GroupNorm, both memory orders, against float64 reductions of the same values
    (including a feature whose mean is far from zero)."""
    from sapa_amd import _lib
    B, C, H, W = shape
    x = (randn(gen(340), B, C, H, W) * 1.7 + 25.0).to(dtype)
    ref = x.double()
    want_mean, want_var = ref.mean(dim=(2, 3)), ref.var(dim=(2, 3), unbiased=False)
    for t in (x.to(DEV), x.to(DEV).contiguous(memory_format=CL)):
        got = _lib.channel_moments(t)
        if C % 4 != 0 and not t.is_contiguous():
            assert got is None                      # channels-last needs whole channel quads
            continue
        assert got.shape == (B, C, 2) and got.dtype == torch.float32
        mean, var = got[..., 0], got[..., 1]
        torch.testing.assert_close(mean.cpu().double(), want_mean, rtol=1e-6, atol=1e-6)
        torch.testing.assert_close(var.cpu().double(), want_var, rtol=2e-5, atol=1e-6)


@pytest.mark.parametrize('dtype,tol', [(torch.float32, 2e-5), (torch.bfloat16, 2e-2), (torch.float16, 3e-3)])
def test_groupnorm_fold_kernel(dtype, tol):
    """Per-image folded projection weights / bias from the moments, against
    float64 arithmetic on the same parameters."""
    from sapa_amd import _lib
    torch.manual_seed(9)
    B, C, O, G = 3, 64, 24, 32
    x = (torch.randn(B, C, 7, 9) * 1.3 + 0.4).to(dtype).to(DEV)
    norm = torch.nn.GroupNorm(G, C).to(DEV)
    torch.nn.init.normal_(norm.weight, 1.0, 0.3)
    torch.nn.init.normal_(norm.bias, 0.0, 0.3)
    conv = torch.nn.Conv2d(C, O, 1).to(DEV)
    norm, conv = norm.to(dtype), conv.to(dtype)
    mom = _lib.channel_moments(x)
    w_b, b_b = _lib.groupnorm_fold(mom, norm, conv, dtype)
    assert w_b.shape == (B, O, C) and b_b.shape == (B, O) and w_b.dtype == dtype
    xd = x.double().cpu().reshape(B, G, -1)
    mean, var = xd.mean(2), xd.var(2, unbiased=False)
    rstd = (var + norm.eps).rsqrt().repeat_interleave(C // G, 1)
    mean_c = mean.repeat_interleave(C // G, 1)
    gamma, beta = norm.weight.double().cpu(), norm.bias.double().cpu()
    w = conv.weight.double().cpu().reshape(O, C)
    scale = gamma * rstd
    want_w = w.unsqueeze(0) * scale.unsqueeze(1)
    want_b = conv.bias.double().cpu() + torch.einsum('oc,bc->bo', w, beta - mean_c * scale)
    torch.testing.assert_close(w_b.double().cpu(), want_w, rtol=tol, atol=tol * 0.1)
    torch.testing.assert_close(b_b.double().cpu(), want_b, rtol=tol, atol=tol)


@pytest.mark.parametrize('dtype,rel', [(torch.float32, None), (torch.bfloat16, BF16_REL), (torch.float16, F16_REL)])
@pytest.mark.parametrize('shape', [(2, 64, 40, 9, 11, 5, 2), (1, 72, 36, 5, 6, 7, 4), (2, 12, 8, 6, 7, 3, 2)],
                         ids=['d64', 'd72-k7s4', 'd12'])
def test_fused_with_query_bias(coracle, dtype, rel, shape):
    """sapa_fused(q, k, v, K, s, query_bias) = sapa_fused(q + bias, k, v, K, s): the
    channels-last kernels add the per-image bias on the fly (16-bit: as four more
    matrix instructions per tap group), the contiguous path forms the sum."""
    B, d, C, H, W, K, s = shape
    g = gen(350)
    q, key, v, _ = inputs(g, B, d, C, H, W, K, s, dtype=dtype)
    bias = (randn(g, B, d) * 0.7).to(dtype)
    qb = q.float() + bias.float()[:, :, None, None]
    want = coracle.sapa_fused(qb, key.float(), v.float(), K, s, 'f32a64')
    # the contiguous path writes the sum in the tensors' type first: one more rounding
    want_rounded = coracle.sapa_fused(qb.to(dtype).float(), key.float(), v.float(), K, s, 'f32a64')
    got_cl = sapa_amd.sapa_fused(*cl(q, key, v), K, s, bias.to(DEV))
    got = sapa_amd.sapa_fused(q.to(DEV), key.to(DEV), v.to(DEV), K, s, bias.to(DEV))
    assert got_cl.is_contiguous(memory_format=CL)
    for out, want in ((got_cl, want), (got, want_rounded)):
        if rel is None:
            torch.testing.assert_close(out.cpu().double().contiguous(), want, rtol=1e-5, atol=1e-5)
        else:
            assert_rel_rms_close(out.float(), want, rel, 'fused with bias')


def test_fused_with_query_bias_gradients():
    """Gradients through the biased call equal those of the explicit sum."""
    g = gen(351)
    B, d, C, H, W, K, s = 2, 8, 12, 5, 6, 5, 2
    q, key, v, _ = inputs(g, B, d, C, H, W, K, s)
    bias = randn(g, B, d) * 0.5
    go = randn(g, B, C, s * H, s * W).to(DEV)
    grads = []
    for biased in (True, False):
        leaves = [t.to(DEV).contiguous(memory_format=CL).requires_grad_() for t in (q, key, v)]
        bl = bias.to(DEV).requires_grad_()
        if biased:
            out = sapa_amd.sapa_fused(*leaves, K, s, bl)
        else:
            out = sapa_amd.sapa_fused(leaves[0] + bl[:, :, None, None], leaves[1], leaves[2], K, s)
        grads.append(torch.autograd.grad(out, leaves + [bl], go))
    for a, b in zip(*grads):
        torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize('dtype,tol', [(torch.bfloat16, 2e-2), (torch.float16, 3e-3)])
@pytest.mark.parametrize('shape', [(2, 256, 64, 9, 11), (1, 128, 32, 40, 33), (3, 64, 64, 5, 7),
                                   (1, 512, 64, 4, 4), (2, 256, 128, 1, 1), (1, 256, 64, 130, 129)])
def test_projection_kernel(dtype, tol, shape):
    """The streaming 1x1 projection with per-image weights on a channels_last
    16-bit feature (ragged last pixel tile, one pixel, several images) against
    float64 arithmetic on the same values; None for shapes it is not built for."""
    from sapa_amd import _lib
    B, C, O, H, W = shape
    g = gen(360)
    x = randn(g, B, C, H, W).to(dtype).to(DEV).contiguous(memory_format=CL)
    w = (randn(g, B, O, C) * 0.1).to(dtype).to(DEV)
    b = randn(g, B, O).to(dtype).to(DEV)
    want = torch.einsum('boc,bchw->bohw', w.double().cpu(), x.double().cpu())
    for bias in (None, b):
        out = _lib.project_nhwc(x, w, bias)
        assert out is not None and out.shape == (B, O, H, W) and out.is_contiguous(memory_format=CL)
        ref = want if bias is None else want + bias.double().cpu()[:, :, None, None]
        torch.testing.assert_close(out.double().cpu(), ref, rtol=tol, atol=tol)
    assert _lib.project_nhwc(x[:, :48].contiguous(memory_format=CL), w[:, :, :48].contiguous()) is None
    assert _lib.project_nhwc(x.double(), w.double()) is None


@pytest.mark.parametrize('shape', [(2, 256, 64, 9, 11), (1, 128, 32, 40, 33), (3, 64, 64, 5, 7), (1, 512, 32, 4, 4),
                                   (2, 256, 32, 1, 1), (1, 256, 64, 130, 129), (2, 64, 32, 17, 3)])
def test_projection_kernel_fp32(shape):
    """The fp32 form of the streaming projection: every product as six products of bf16
    pieces on the matrix instruction, fp32 sums.  Against float64 arithmetic on the same
    values it must stand where an fp32 dot product stands: the bound is the error of
    torch's own fp32 product on these values (with a factor for its different order of
    summation) and, outright, the stated 1e-5 relative to the operands' scale."""
    from sapa_amd import _lib
    B, C, O, H, W = shape
    g = gen(361)
    x = (randn(g, B, C, H, W) * 3 + 0.5).to(DEV).contiguous(memory_format=CL)
    w = (randn(g, B, O, C) * 0.1).to(DEV)
    b = randn(g, B, O).to(DEV)
    want = torch.einsum('boc,bchw->bohw', w.double().cpu(), x.double().cpu())
    e32 = (torch.einsum('boc,bchw->bohw', w.cpu(), x.cpu()).double() - want).abs().max().item()
    # sum over c of |w x|: what the rounding of an fp32 dot product scales with
    scale = torch.einsum('boc,bchw->bohw', w.double().abs().cpu(), x.double().abs().cpu()).max().item()
    for bias in (None, b):
        out = _lib.project_nhwc(x, w, bias)
        assert out is not None and out.dtype == torch.float32 and out.shape == (B, O, H, W)
        assert out.is_contiguous(memory_format=CL)
        ref = want if bias is None else want + bias.double().cpu()[:, :, None, None]
        err = (out.double().cpu() - ref).abs().max().item()
        assert err <= max(3 * e32, 1e-6 * scale), (err, e32, scale)
        assert err <= 1e-5 * scale
    # pairs whose three weight planes do not fit the LDS go to the caller's library GEMM
    if C == 256 and O == 64:
        w2 = torch.cat([w, w], 1).contiguous()
        assert _lib.project_nhwc(x, w2) is None


@pytest.mark.parametrize('shape', [(2, 256, 64, 9, 12), (1, 128, 32, 40, 33), (3, 64, 64, 5, 8), (1, 512, 32, 4, 4),
                                   (2, 256, 32, 1, 4), (1, 256, 64, 130, 129), (2, 64, 32, 17, 3)])
def test_projection_kernel_fp32_contiguous_feature(shape):
    """The fp32 projection reading a contiguous feature (planes), writing a channels_last
    or a contiguous result (the latter for plane sizes that are multiples of 4; None
    otherwise): same bound as the channels_last form, and the two results bit for bit
    the same (one arithmetic, two store patterns)."""
    from sapa_amd import _lib
    B, C, O, H, W = shape
    g = gen(362)
    x = (randn(g, B, C, H, W) * 3 + 0.5).to(DEV)
    w = (randn(g, B, O, C) * 0.1).to(DEV)
    b = randn(g, B, O).to(DEV)
    want = torch.einsum('boc,bchw->bohw', w.double().cpu(), x.double().cpu())
    e32 = (torch.einsum('boc,bchw->bohw', w.cpu(), x.cpu()).double() - want).abs().max().item()
    scale = torch.einsum('boc,bchw->bohw', w.double().abs().cpu(), x.double().abs().cpu()).max().item()
    for bias in (None, b):
        ref = want if bias is None else want + bias.double().cpu()[:, :, None, None]
        out_cl = _lib.project_nchw(x, w, bias, channels_last_out=True)
        assert out_cl is not None and out_cl.shape == (B, O, H, W) and out_cl.is_contiguous(memory_format=CL)
        err = (out_cl.double().cpu() - ref).abs().max().item()
        assert err <= max(3 * e32, 1e-6 * scale) and err <= 1e-5 * scale, (err, e32, scale)
        out = _lib.project_nchw(x, w, bias)
        if (H * W) % 4:
            assert out is None
        else:
            assert out.is_contiguous() and torch.equal(out, out_cl)
        # ... and the same bits as the channels_last feature's kernel
        assert torch.equal(_lib.project_nhwc(x.contiguous(memory_format=CL), w, bias), out_cl)
    assert _lib.project_nchw(x.double(), w.double()) is None
    assert _lib.project_nchw(x.contiguous(memory_format=CL), w) is None


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('shape', [(2, 256, 64, 9, 16), (1, 128, 32, 40, 34), (3, 64, 64, 5, 8), (2, 64, 48, 6, 8)])
def test_norm_project_in_one_call(dtype, shape):
    """Moments, fold and projection through the single entry point: the same bits as the
    three entry points one after the other (it launches the same kernels), for both
    memory orders of the feature, with the bias added and with it handed back; None --
    and nothing launched -- for a channel pair without a projection kernel."""
    from sapa_amd import _lib
    B, C, O, H, W = shape
    torch.manual_seed(11)
    norm = torch.nn.GroupNorm(32, C).to(DEV).to(dtype)
    conv = torch.nn.Conv2d(C, O, 1).to(DEV).to(dtype)
    torch.nn.init.normal_(norm.weight, 1.0, 0.2)
    torch.nn.init.normal_(norm.bias, 0.0, 0.2)
    x = (randn(gen(364), B, C, H, W) * 1.5 + 0.3).to(dtype).to(DEV)
    for feat, cl_out in ((x, False), (x, True), (x.contiguous(memory_format=CL), True)):
        got = _lib.norm_project(feat, norm, conv, channels_last_out=cl_out)
        got_d = _lib.norm_project(feat, norm, conv, channels_last_out=cl_out, defer_bias=True)
        if O == 48:
            assert got is None and got_d is None
            continue
        w_b, b_b = _lib.groupnorm_fold(_lib.channel_moments(feat), norm, conv, dtype)
        if feat.is_contiguous():
            want, want_d = (_lib.project_nchw(feat, w_b, b, channels_last_out=cl_out) for b in (b_b, None))
        else:
            want, want_d = (_lib.project_nhwc(feat, w_b, b) for b in (b_b, None))
        assert got[1] is None and torch.equal(got[0], want) and got[0].stride() == want.stride()
        assert torch.equal(got_d[0], want_d) and torch.equal(got_d[1], b_b)
        # and the composition it stands for
        ref = conv(norm(x)).float()
        tol = 2e-4 if dtype == torch.float32 else 6e-2 if dtype == torch.bfloat16 else 1e-2
        torch.testing.assert_close(got[0].float(), ref, rtol=tol, atol=tol)


@pytest.mark.parametrize('dtype,tol', [(torch.bfloat16, 2e-2), (torch.float16, 3e-3)])
@pytest.mark.parametrize('shape', [(2, 256, 64, 9, 16), (1, 128, 32, 40, 34), (3, 64, 64, 5, 8), (1, 512, 32, 4, 4),
                                   (2, 256, 32, 1, 8), (1, 256, 64, 130, 132), (2, 64, 32, 17, 3)])
def test_projection_kernel_16bit_contiguous_feature(dtype, tol, shape):
    """The 16-bit projection reading a contiguous feature (planes of a multiple of 8
    pixels; None otherwise), writing a channels_last or a contiguous result: against
    float64 arithmetic on the same values, the two results bit for bit the same, and the
    same bits as the channels_last feature's kernel gives (fp32 sums in the same order
    would not be needed for that bar; they are what the kernels do)."""
    from sapa_amd import _lib
    B, C, O, H, W = shape
    g = gen(363)
    x = randn(g, B, C, H, W).to(dtype).to(DEV)
    w = (randn(g, B, O, C) * 0.1).to(dtype).to(DEV)
    b = randn(g, B, O).to(dtype).to(DEV)
    want = torch.einsum('boc,bchw->bohw', w.double().cpu(), x.double().cpu())
    for bias in (None, b):
        out_cl = _lib.project_nchw(x, w, bias, channels_last_out=True)
        out = _lib.project_nchw(x, w, bias)
        if (H * W) % 8:
            assert out_cl is None and out is None
            continue
        assert out_cl.is_contiguous(memory_format=CL) and out.is_contiguous() and out.dtype == dtype
        ref = want if bias is None else want + bias.double().cpu()[:, :, None, None]
        torch.testing.assert_close(out_cl.double().cpu(), ref, rtol=tol, atol=tol)
        assert torch.equal(out, out_cl)
        torch.testing.assert_close(_lib.project_nhwc(x.contiguous(memory_format=CL), w, bias).float(), out_cl.float(),
                                   rtol=2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10, atol=1e-6)
