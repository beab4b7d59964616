"""GPU parity of the SAPA-B operators (qk, softmax, av, fused) against the
CPU oracle, through the Python API and so through the C ABI.

Bars: fp32 qk/av bit-exact against the oracle in the reference kernels' own
arithmetic (same FMA order); fused fp32 within 1e-5 rel / 1e-6 abs; bf16
within 1e-2 (relative to max(|b|, rms)); integer-valued inputs exact.
"""
import pytest
import torch
import torch.nn.functional as F

import sapa_amd
from helpers import (BF16_REL, F16_REL, assert_f32_close, assert_rel_rms_close, fused_backward_oracle, gen, golden,
                     randn, ulp_report)

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'

# B, d, C, H, W, K, s -- K=5,s=2 takes the LDS-tiled kernels, the rest the
# generic ones; extents are ragged against the 16x16 and 16x8 tiles
SHAPES = [
    (2, 6, 5, 9, 19, 5, 2), (1, 32, 64, 32, 32, 5, 2), (2, 8, 8, 16, 16, 5, 2),
    (1, 3, 2, 1, 1, 5, 2), (1, 9, 7, 17, 33, 5, 2), (3, 64, 16, 24, 40, 5, 2),
    (1, 4, 3, 5, 6, 3, 3), (1, 3, 2, 6, 7, 7, 1), (2, 5, 4, 4, 4, 1, 1),
    (1, 4, 6, 7, 5, 9, 2), (1, 2, 2, 3, 3, 11, 4), (1, 3, 3, 8, 8, 3, 2),
    # the matrix-pipe kernel: K in {3,5,7} x s in {2,4} except K=5, s=2
    (1, 5, 6, 9, 37, 7, 2), (2, 4, 5, 7, 18, 3, 4), (1, 6, 8, 6, 35, 5, 4), (1, 4, 9, 5, 17, 7, 4),
    (2, 9, 13, 11, 34, 3, 2), (1, 64, 40, 16, 16, 7, 4),
]
IDS = ['-'.join(map(str, s)) for s in SHAPES]


def dev(*ts):
    return [t.to(DEV) for t in ts]


@pytest.mark.parametrize('shape', SHAPES, ids=IDS)
def test_qk_fp32_bit_exact(coracle, shape):
    B, d, C, H, W, K, s = shape
    g = gen(100)
    q, key = randn(g, B, d, H * s, W * s), randn(g, B, d, H, W)
    got = sapa_amd.qk(*dev(q, key), K, s).cpu()
    want = coracle.qk(q, key, K, s, 'f32')
    assert got.shape == want.shape and got.dtype == torch.float32
    assert torch.equal(got, want), f'max ulp {ulp_report(got, want)}'
    if d <= 9:  # short sums: also within the bar of the float64-accumulated value
        assert_f32_close(got, coracle.qk(q, key, K, s, 'f32a64'), 'qk vs f64 accumulation')


@pytest.mark.parametrize('shape', SHAPES, ids=IDS)
def test_av_fp32_bit_exact(coracle, shape):
    B, d, C, H, W, K, s = shape
    g = gen(101)
    attn, v = randn(g, B, K * K, H * s, W * s), randn(g, B, C, H, W)
    got = sapa_amd.av(*dev(attn, v), K, s).cpu()
    want = coracle.av(attn, v, K, s, 'f32')
    assert torch.equal(got, want), f'max ulp {ulp_report(got, want)}'


@pytest.mark.parametrize('shape', SHAPES, ids=IDS)
def test_fused_fp32(coracle, shape):
    B, d, C, H, W, K, s = shape
    g = gen(102)
    q, key, v = randn(g, B, d, H * s, W * s), randn(g, B, d, H, W), randn(g, B, C, H, W)
    got = sapa_amd.sapa_fused(*dev(q, key, v), K, s).cpu()
    assert_f32_close(got, coracle.sapa_fused(q, key, v, K, s, 'f32'), 'fused vs kernel-arithmetic oracle')
    # against the float64-accumulated value the distance is fp32 summation
    # error itself (the reference's fp32 kernels sit just as far away), so the
    # bound here is the reference's own check tolerance, allclose(atol=1e-5)
    torch.testing.assert_close(got.double(), coracle.sapa_fused(q, key, v, K, s, 'f32a64'),
                               rtol=1e-5, atol=1e-5)
    # and the attention weights on their own
    attn = sapa_amd.qk_softmax(*dev(q, key), K, s).cpu()
    want = coracle.softmax(coracle.qk(q, key, K, s, 'f32'), 1, 'f32')
    torch.testing.assert_close(attn, want, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(attn.sum(1), torch.ones(B, H * s, W * s), rtol=1e-5, atol=0)


@pytest.mark.parametrize('shape', SHAPES, ids=IDS)
def test_integer_inputs_exact(coracle, shape):
    """Integer-valued tensors: every product and sum is exact in fp32, so any
    indexing error is a hard mismatch whatever the summation order."""
    B, d, C, H, W, K, s = shape
    g = gen(103)
    ri = lambda *sh: torch.randint(-4, 5, sh, generator=g).float()
    q, key, v, attn = ri(B, d, H * s, W * s), ri(B, d, H, W), ri(B, C, H, W), ri(B, K * K, H * s, W * s)
    assert torch.equal(sapa_amd.qk(*dev(q, key), K, s).cpu(), coracle.qk(q, key, K, s, 'f32a64').float())
    assert torch.equal(sapa_amd.av(*dev(attn, v), K, s).cpu(), coracle.av(attn, v, K, s, 'f32a64').float())


def test_golden_vectors():
    G = golden()
    t = lambda a: torch.from_numpy(a)
    for tag in ('b_k5s2', 'b_k3s3', 'b_k7s1'):
        B, d, C, H, W, K, s = (int(v) for v in G[f'{tag}.cfg'])
        q, key, v, attn = (t(G[f'{tag}.{n}']) for n in ('q', 'key', 'v', 'attn'))
        assert torch.equal(sapa_amd.qk(*dev(q, key), K, s).cpu(), t(G[f'{tag}.qk'])), tag
        assert torch.equal(sapa_amd.av(*dev(attn, v), K, s).cpu(), t(G[f'{tag}.av'])), tag
        got = sapa_amd.sapa_fused(*dev(q, key, v), K, s).cpu()
        assert_f32_close(got, t(G[f'{tag}.fused']), tag)
        torch.testing.assert_close(got.double(), t(G[f'{tag}.fused64']), rtol=1e-5, atol=1e-5)


def test_reference_forward_check_shape(coracle):
    """sapa/sapa/forward_check.py:27-46 with its own tolerance (atol=1e-5),
    against the unfold-based restatement."""
    from oracle import torch_oracle as T
    g = gen(104)
    b, h, w, c, K, s = 4, 10, 12, 8, 5, 2
    q, k = randn(g, b, c, s * h, s * w), randn(g, b, c, h, w)
    assert torch.allclose(T.qk(q, k, K, s), sapa_amd.qk(*dev(q, k), K, s).cpu(), atol=1e-5)
    attn, v = randn(g, b, K * K, s * h, s * w), randn(g, b, c, h, w)
    assert torch.allclose(T.av(attn, v, K, s), sapa_amd.av(*dev(attn, v), K, s).cpu(), atol=1e-5)


def test_softmax_kernel(coracle):
    g = gen(105)
    x = randn(g, 2, 25, 14, 22) * 4
    got = sapa_amd.softmax_k(x.to(DEV), 1).cpu()
    torch.testing.assert_close(got, coracle.softmax(x, 1, 'f32'), rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(got, F.softmax(x.double(), 1).float(), rtol=1e-5, atol=1e-7)
    x5 = randn(g, 2, 4, 9, 6, 10)
    got = sapa_amd.softmax_k(x5.to(DEV), 2).cpu()
    torch.testing.assert_close(got, F.softmax(x5, 2), rtol=1e-5, atol=1e-7)
    xd = x.double()
    torch.testing.assert_close(sapa_amd.softmax_k(xd.to(DEV), 1).cpu(), F.softmax(xd, 1), rtol=1e-12, atol=1e-15)


def test_fused_zero_query_box_filter():
    """q == 0: uniform weights 1/K^2 everywhere, out-of-range neighbours
    included in the denominator: the zero-padded box filter of the value."""
    g = gen(106)
    B, d, C, H, W, K, s = 2, 8, 6, 21, 37, 5, 2
    key, v = randn(g, B, d, H, W), randn(g, B, C, H, W)
    q = torch.zeros(B, d, H * s, W * s)
    got = sapa_amd.sapa_fused(*dev(q, key, v), K, s).cpu()
    want = F.avg_pool2d(v.double(), K, 1, K // 2, count_include_pad=True)
    want = want.repeat_interleave(s, -2).repeat_interleave(s, -1)
    assert_f32_close(got, want, 'box filter')


@pytest.mark.parametrize('dtype,rel', [(torch.bfloat16, BF16_REL), (torch.float16, F16_REL)])
@pytest.mark.parametrize('shape', [SHAPES[0], SHAPES[5], SHAPES[6], SHAPES[9], SHAPES[12], SHAPES[15]],
                         ids=[IDS[0], IDS[5], IDS[6], IDS[9], IDS[12], IDS[15]])
def test_16bit_dtypes(coracle, shape, dtype, rel):
    """Oracle = fp32-input, float64-accumulated math on the rounded inputs."""
    B, d, C, H, W, K, s = shape
    g = gen(107)
    q, key, v = (randn(g, *sh).to(dtype) for sh in
                 ((B, d, H * s, W * s), (B, d, H, W), (B, C, H, W)))
    attn = F.softmax(randn(g, B, K * K, H * s, W * s), 1).to(dtype)
    qf, kf, vf, af = (x.float() for x in (q, key, v, attn))
    got = sapa_amd.qk(*dev(q, key), K, s)
    assert got.dtype == dtype
    assert_rel_rms_close(got.float(), coracle.qk(qf, kf, K, s, 'f32a64'), rel, 'qk')
    got = sapa_amd.av(*dev(attn, v), K, s)
    assert_rel_rms_close(got.float(), coracle.av(af, vf, K, s, 'f32a64'), rel, 'av')
    got = sapa_amd.sapa_fused(*dev(q, key, v), K, s)
    assert got.dtype == dtype
    assert_rel_rms_close(got.float(), coracle.sapa_fused(qf, kf, vf, K, s, 'f32a64'), rel, 'fused')


# K = 5, s = 2, W a multiple of 4 and at least 32: the 16-bit kernels built on
# the two-term dot product instructions.  Several tiles in x and y, ragged
# edges, odd channel counts (the last channel pair / value chunk is partial).
DOT2_SHAPES = [(2, 7, 11, 13, 36, 5, 2), (1, 16, 8, 8, 32, 5, 2), (1, 33, 20, 9, 68, 5, 2),
               (1, 5, 3, 3, 100, 5, 2), (1, 1, 1, 1, 32, 5, 2), (2, 18, 70, 17, 44, 5, 2)]


@pytest.mark.parametrize('dtype,rel', [(torch.bfloat16, BF16_REL), (torch.float16, F16_REL)])
@pytest.mark.parametrize('shape', DOT2_SHAPES, ids=['-'.join(map(str, s)) for s in DOT2_SHAPES])
def test_16bit_dot_product_kernels(coracle, shape, dtype, rel):
    B, d, C, H, W, K, s = shape
    g = gen(117)
    q, key, v = (randn(g, *sh).to(dtype) for sh in
                 ((B, d, H * s, W * s), (B, d, H, W), (B, C, H, W)))
    attn = F.softmax(randn(g, B, K * K, H * s, W * s), 1).to(dtype)
    qf, kf, vf, af = (x.float() for x in (q, key, v, attn))
    got = sapa_amd.qk(*dev(q, key), K, s)
    assert got.dtype == dtype
    # products of 16-bit values are exact in fp32 and the sums are fp32: only
    # the final rounding to the 16-bit type separates the result from the oracle
    want = coracle.qk(qf, kf, K, s, 'f32a64')
    assert_rel_rms_close(got.float(), want, rel, 'qk')
    if d <= 8:
        # at most one unit in the last place of the 16-bit type
        torch.testing.assert_close(got.float().cpu(), want.to(dtype).float(),
                                   rtol=2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10, atol=1e-6)
    got = sapa_amd.qk_softmax(*dev(q, key), K, s)
    want = coracle.softmax(coracle.qk(qf, kf, K, s, 'f32a64').float(), 1, 'f32')
    assert_rel_rms_close(got.float(), want, rel, 'qk_softmax')
    got = sapa_amd.av(*dev(attn, v), K, s)
    assert_rel_rms_close(got.float(), coracle.av(af, vf, K, s, 'f32a64'), rel, 'av')
    got = sapa_amd.sapa_fused(*dev(q, key, v), K, s)
    assert got.dtype == dtype
    assert_rel_rms_close(got.float(), coracle.sapa_fused(qf, kf, vf, K, s, 'f32a64'), rel, 'fused')


# Fused, contiguous 16-bit tensors, K = 5, s = 2, W even and at least 16: two dense products per 4 x 4 block
# of parents on the 16-bit matrix instructions (small shapes of the lists above reach it as well).  (B, d, C, H, W): one tile of 8 blocks; ragged tile rows, d and C off the 16-channel chunks;
# a single tile of 13 blocks; 7 tiles in x; two unequal tiles; the FPN geometry (3 tiles of 14 blocks) with
# odd channel counts; rows that end inside a block and inside a 16-byte piece (W = 42: one tile, W = 70: two).
DENSE16_SHAPES = [(1, 3, 5, 2, 16), (13, 16, 16, 32, 32), (2, 24, 40, 79, 80), (5, 40, 24, 51, 52), (1, 64, 48, 30, 420),
                  (3, 32, 16, 66, 68), (1, 17, 19, 100, 168), (13, 20, 24, 25, 42), (2, 8, 8, 100, 70)]


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('shape', DENSE16_SHAPES, ids=['-'.join(map(str, s)) for s in DENSE16_SHAPES])
def test_16bit_dense_window_kernel(coracle, shape, dtype):
    """Products of 16-bit values are exact in fp32, sums and softmax are fp32, the weights enter the
    aggregation as a 16-bit value plus a 16-bit remainder: what is left is the rounding of the result, at
    most half a 16-bit spacing (2^-8 resp. 2^-11 of the value) against the double-precision oracle."""
    B, d, C, H, W = shape
    g = gen(131)
    q, key, v = (randn(g, *sh).to(dtype) for sh in ((B, d, H * 2, W * 2), (B, d, H, W), (B, C, H, W)))
    half_ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
    got = sapa_amd.sapa_fused(*dev(q, key, v), 5, 2)
    assert sapa_amd._lib.last_kernel() == 'sapa_b_wmat16_kernel'
    assert got.dtype == dtype and got.shape == (B, C, 2 * H, 2 * W)
    exact = torch.cat([coracle.sapa_fused(q[i:i + 1].float(), key[i:i + 1].float(), v[i:i + 1].float(), 5, 2, 'f32a64')
                       for i in range(B)]).double()
    err = (got.float().cpu().double() - exact).abs()
    worst = (err / torch.maximum(exact.abs(), exact.square().mean().sqrt())).max().item()
    assert worst <= 1.05 * half_ulp, f'{shape} {dtype}: {worst / half_ulp:.2f} half-spacings'
    # zero query: every child weighs the 25 cells of its own window equally and the rest of the 8 x 8
    # window not at all -- the box filter of the value, zero padding counted.  Positive values, large on
    # the border cells, and a bar relative to each element: a cell too many or too few at an edge, a
    # shifted window row or column shows at once.
    vp = v.float().abs() + 0.5
    for sl in ((slice(None), slice(None), 0), (slice(None), slice(None), -1),
               (slice(None), slice(None), slice(None), 0), (slice(None), slice(None), slice(None), -1)):
        vp[sl] *= 64.0
    vp = vp.to(dtype)
    got0 = sapa_amd.sapa_fused(torch.zeros_like(q).to(DEV), key.to(DEV), vp.to(DEV), 5, 2)
    assert sapa_amd._lib.last_kernel() == 'sapa_b_wmat16_kernel'
    box = F.interpolate(F.avg_pool2d(vp.double(), 5, 1, 2, count_include_pad=True), scale_factor=2)
    rel = ((got0.float().cpu().double() - box).abs() / box).max().item()
    assert rel <= 1.05 * half_ulp + 1e-6, f'{shape} {dtype} box filter: {rel / half_ulp:.2f} half-spacings'


@pytest.mark.parametrize('shape', [SHAPES[0], SHAPES[6]], ids=[IDS[0], IDS[6]])
def test_fp64(coracle, shape):
    B, d, C, H, W, K, s = shape
    g = gen(108)
    q, key, v = (randn(g, *sh, dtype=torch.float64) for sh in
                 ((B, d, H * s, W * s), (B, d, H, W), (B, C, H, W)))
    attn = randn(g, B, K * K, H * s, W * s, dtype=torch.float64)
    assert torch.equal(sapa_amd.qk(*dev(q, key), K, s).cpu(), coracle.qk(q, key, K, s, 'f64'))
    assert torch.equal(sapa_amd.av(*dev(attn, v), K, s).cpu(), coracle.av(attn, v, K, s, 'f64'))
    torch.testing.assert_close(sapa_amd.sapa_fused(*dev(q, key, v), K, s).cpu(),
                               coracle.sapa_fused(q, key, v, K, s, 'f64'), rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize('shape', [SHAPES[0], SHAPES[6], SHAPES[7]], ids=[IDS[0], IDS[6], IDS[7]])
def test_backward_vs_oracle(coracle, shape):
    B, d, C, H, W, K, s = shape
    g = gen(109)
    for dt, tol in ((torch.float64, dict(rtol=1e-11, atol=1e-12)), (torch.float32, dict(rtol=1e-4, atol=1e-5))):
        q = randn(g, B, d, H * s, W * s, dtype=dt)
        key = randn(g, B, d, H, W, dtype=dt)
        go = randn(g, B, K * K, H * s, W * s, dtype=dt)
        qd, kd = (x.to(DEV).requires_grad_() for x in (q, key))
        sapa_amd.qk(qd, kd, K, s).backward(go.to(DEV))
        gq, gk = coracle.qk_backward(go.double(), q.double(), key.double(), K, s, 'f64')
        torch.testing.assert_close(qd.grad.cpu().double(), gq, **tol)
        torch.testing.assert_close(kd.grad.cpu().double(), gk, **tol)

        attn = randn(g, B, K * K, H * s, W * s, dtype=dt)
        v = randn(g, B, C, H, W, dtype=dt)
        go = randn(g, B, C, H * s, W * s, dtype=dt)
        ad, vd = (x.to(DEV).requires_grad_() for x in (attn, v))
        sapa_amd.av(ad, vd, K, s).backward(go.to(DEV))
        ga, gv = coracle.av_backward(go.double(), attn.double(), v.double(), K, s, 'f64')
        torch.testing.assert_close(ad.grad.cpu().double(), ga, **tol)
        torch.testing.assert_close(vd.grad.cpu().double(), gv, **tol)


# B, d, C, H, W, K: more than one tile in x and y, ragged edges, channel counts
# that are not a multiple of the kernel's chunk, channel slicing (few tiles,
# many channels)
LOWGRAD_SHAPES = [(2, 5, 11, 19, 45, 5), (1, 40, 70, 9, 17, 5), (1, 3, 9, 21, 70, 3),
                  (2, 16, 8, 8, 32, 5), (1, 2, 1, 1, 1, 5)]


@pytest.mark.parametrize('shape', LOWGRAD_SHAPES, ids=['-'.join(map(str, s)) for s in LOWGRAD_SHAPES])
def test_tiled_lowres_gradients_vs_oracle(coracle, shape):
    """grad_key / grad_value from the tiled scatter kernel (fp32, s = 2)
    against the float64 oracle, twice in a row into dirty buffers' successors
    (the kernel zero-fills its output itself)."""
    B, d, C, H, W, K = shape
    s = 2
    g = gen(150)
    q, key = randn(g, B, d, H * s, W * s), randn(g, B, d, H, W)
    go = randn(g, B, K * K, H * s, W * s)
    attn, v = randn(g, B, K * K, H * s, W * s), randn(g, B, C, H, W)
    go2 = randn(g, B, C, H * s, W * s)
    _, gk = coracle.qk_backward(go.double(), q.double(), key.double(), K, s, 'f64')
    _, gv = coracle.av_backward(go2.double(), attn.double(), v.double(), K, s, 'f64')
    from sapa_amd import _lib
    qd, kd, god, ad, vd, go2d = dev(q, key, go, attn, v, go2)
    for fill in (7.0, -3.0):
        out_k = torch.full_like(kd, fill)
        _lib.call('sapa_qk_backward', kd.device, _lib.ptr(god), _lib.ptr(qd), _lib.ptr(kd), None,
                  _lib.ptr(out_k), B, d, H, W, K, s, 0)
        torch.testing.assert_close(out_k.cpu().double(), gk, rtol=1e-4, atol=2e-5)
        out_v = torch.full_like(vd, fill)
        _lib.call('sapa_av_backward', vd.device, _lib.ptr(go2d), _lib.ptr(ad), _lib.ptr(vd), None,
                  _lib.ptr(out_v), B, C, H, W, K, s, 0)
        torch.testing.assert_close(out_v.cpu().double(), gv, rtol=1e-4, atol=2e-5)


# the first shape takes the gather, the others the lane-exchange form (several
# tiles in x and y, ragged edges, channels not a multiple of the chunk)
@pytest.mark.parametrize('shape', [(2, 10, 13, 37, 5), (2, 10, 24, 50, 5), (1, 7, 21, 70, 3), (1, 3, 12, 12, 5)],
                         ids=['gather-13x37', 'shift-24x50', 'shift-21x70-k3', 'shift-12x12'])
def test_tiled_lowres_gradient_integer_inputs_exact(shape):
    """Integer-valued inputs make every product and sum exact in fp32, so any
    order of the sums gives the same bits: an index error cannot hide."""
    g = gen(151)
    B, C, H, W, K = shape
    s = 2
    attn = torch.randint(-3, 4, (B, K * K, H * s, W * s), generator=g).float()
    go = torch.randint(-3, 4, (B, C, H * s, W * s), generator=g).float()
    v = torch.zeros(B, C, H, W)
    ad, vd, god = dev(attn, v, go)
    ad.requires_grad_(False)
    vd.requires_grad_()
    sapa_amd.av(ad, vd, K, s).backward(god)
    want = torch.zeros(B, C, H, W, dtype=torch.float64)
    r = K // 2
    a6 = attn.double().view(B, K, K, H, s, W, s)
    g6 = go.double().view(B, C, H, s, W, s)
    for ky in range(K):
        for kx in range(K):
            contrib = torch.einsum('bhiwj,bchiwj->bchw', a6[:, ky, kx], g6)   # per parent
            dy, dx = ky - r, kx - r                                          # cell = parent + (dy, dx)
            ys, xs = slice(max(0, -dy), H - max(0, dy)), slice(max(0, -dx), W - max(0, dx))
            yd, xd = slice(max(0, dy), H + min(0, dy)), slice(max(0, dx), W + min(0, dx))
            want[:, :, yd, xd] += contrib[:, :, ys, xs]
    assert torch.equal(vd.grad.cpu().double(), want)


def test_backward_16bit_tensors():
    """16-bit tensors: gradients come back in the tensors' dtype and agree
    with the fp32 gradients at the same (rounded) inputs."""
    g = gen(152)
    B, d, C, H, W, K, s = 1, 8, 12, 10, 20, 5, 2
    q, key, v = randn(g, B, d, H * s, W * s), randn(g, B, d, H, W), randn(g, B, C, H, W)
    go = randn(g, B, C, H * s, W * s)
    for dt, rel in ((torch.bfloat16, 3e-2), (torch.float16, 5e-3)):
        ts = [t.to(DEV).to(dt).requires_grad_() for t in (q, key, v)]
        sapa_amd.sapa_fused(*ts, K, s).backward(go.to(DEV).to(dt))
        ref = [t.detach().float().requires_grad_() for t in ts]
        sapa_amd.sapa_fused(*ref, K, s).backward(go.to(DEV).to(dt).float())
        for a, b in zip(ts, ref):
            assert a.grad.dtype == dt
            assert_rel_rms_close(a.grad.float().cpu(), b.grad.cpu(), rel, str(dt))


@pytest.mark.parametrize('K,s', [(7, 4), (3, 2), (5, 4)])
@pytest.mark.parametrize('dt,rel', [(torch.bfloat16, 1e-2), (torch.float16, 2e-3)])
def test_backward_16bit_tensors_other_windows(coracle, K, s, dt, rel):
    """(kernel_size, scale_factor) pairs that the one-call backward does not cover:
    the chain runs in fp32 on widened copies, so the 16-bit gradients are the
    rounded float64 chain on the rounded inputs (one rounding, at the end)."""
    g = gen(154)
    B, d, C, H, W = 1, 8, 12, 6, 9
    q, key, v = (randn(g, B, d, H * s, W * s).to(dt), randn(g, B, d, H, W).to(dt), randn(g, B, C, H, W).to(dt))
    go = randn(g, B, C, H * s, W * s).to(dt)
    ts = [t.to(DEV).requires_grad_() for t in (q, key, v)]
    sapa_amd.sapa_fused(*ts, K, s).backward(go.to(DEV))
    q64, k64, v64, go64 = (t.double() for t in (q, key, v, go))
    attn = coracle.softmax(coracle.qk(q64, k64, K, s, 'f64'), 1, 'f64')
    ga, gv = coracle.av_backward(go64, attn, v64, K, s, 'f64')
    gl = attn * (ga - (ga * attn).sum(1, keepdim=True))
    gq, gk = coracle.qk_backward(gl, q64, k64, K, s, 'f64')
    for a, want, name in zip(ts, (gq, gk, gv), ('grad_query', 'grad_key', 'grad_value')):
        assert a.grad.dtype == dt
        assert_rel_rms_close(a.grad.float().cpu(), want.float(), rel, f'{name} {dt} K={K} s={s}')


# 16-bit tensors take the lane-exchange form in rows of 32 lanes (30x70, 33x47 with
# K = 3) or of 16 (25x42); each shape spans several tiles with ragged edges
@pytest.mark.parametrize('shape', [(1, 6, 30, 70, 5), (2, 5, 25, 42, 5), (1, 5, 33, 47, 3)],
                         ids=['rows32-30x70', 'rows16-25x42', 'rows32-33x47-k3'])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_lowres_gradients_16bit_integer_inputs_exact(shape, dtype):
    """Small integers are exact in 16 bits, and so is every product and sum in the
    kernels' fp32: grad_value of 16-bit tensors must equal the integer result bit for
    bit whichever form and tile geometry serves the shape."""
    g = gen(153)
    B, C, H, W, K = shape
    s = 2
    attn = torch.randint(-2, 3, (B, K * K, H * s, W * s), generator=g).float()
    go = torch.randint(-2, 3, (B, C, H * s, W * s), generator=g).float()
    from sapa_amd import _lib
    ad, god = attn.to(DEV).to(dtype), go.to(DEV).to(dtype)
    vd = torch.zeros(B, C, H, W, device=DEV, dtype=dtype)
    out = torch.full_like(vd, 9.0)
    _lib.call('sapa_av_backward', vd.device, _lib.ptr(god), _lib.ptr(ad), _lib.ptr(vd), None, _lib.ptr(out),
              B, C, H, W, K, s, _lib.DTYPES[dtype])
    want = torch.zeros(B, C, H, W, dtype=torch.float64)
    r = K // 2
    a6 = attn.double().view(B, K, K, H, s, W, s)
    g6 = go.double().view(B, C, H, s, W, s)
    for ky in range(K):
        for kx in range(K):
            contrib = torch.einsum('bhiwj,bchiwj->bchw', a6[:, ky, kx], g6)   # per parent
            dy, dx = ky - r, kx - r                                          # cell = parent + (dy, dx)
            ys, xs = slice(max(0, -dy), H - max(0, dy)), slice(max(0, -dx), W - max(0, dx))
            yd, xd = slice(max(0, dy), H + min(0, dy)), slice(max(0, dx), W + min(0, dx))
            want[:, :, yd, xd] += contrib[:, :, ys, xs]
    assert want.abs().max() < 256          # exactly representable in bf16 as well
    assert torch.equal(out.double().cpu(), want)


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
def test_fused_training_step_keeps_attention(dtype):
    """sapa_fused with gradients wanted: the forward pass that keeps the fp32 attention
    weights (two launches) against the one-launch forward whose backward recomputes them:
    the same gradients bit for bit (the kept weights are the recomputed ones), the same
    output to the type's rounding; one more saved tensor, [B,K*K,sH,sW] fp32.  K = 3 is
    not covered by the pair of entry points and silently takes the other path."""
    g = gen(154)
    for (B, d, C, H, W, K) in ((2, 16, 24, 13, 22, 5), (1, 8, 12, 9, 14, 3)):
        s = 2
        q, key, v = randn(g, B, d, H * s, W * s), randn(g, B, d, H, W), randn(g, B, C, H, W)
        go = randn(g, B, C, H * s, W * s).to(DEV).to(dtype)
        res = {}
        for keep in (True, False):
            saved = []
            ts = [t.to(DEV).to(dtype).requires_grad_() for t in (q, key, v)]
            with torch.autograd.graph.saved_tensors_hooks(lambda t: saved.append(tuple(t.shape)) or t, lambda t: t):
                out = sapa_amd.sapa_fused(*ts, K, s, save_attention=keep)
            out.backward(go)
            res[keep] = (out.detach(), [t.grad for t in ts], saved)
        kept = (B, K * K, H * s, W * s) in res[True][2]
        assert kept == (K == 5) and (B, K * K, H * s, W * s) not in res[False][2]
        for a, b in zip(res[True][1], res[False][1]):
            assert torch.equal(a, b)
        if dtype == torch.float32:
            assert_f32_close(res[True][0], res[False][0], 'output with kept weights')
        else:
            assert_rel_rms_close(res[True][0].float(), res[False][0].float(), 2 ** -7 if dtype == torch.bfloat16 else 2 ** -10,
                                 f'output with kept weights {dtype}')


@pytest.mark.parametrize('dtype,tol', [(torch.float32, dict(rtol=1e-4, atol=1e-5)),
                                        (torch.bfloat16, 1.5e-2), (torch.float16, 2e-3)])
def test_fused_backward_entry_point(coracle, dtype, tol):
    """sapa_fused_backward through the C ABI: all three gradients against the
    float64 oracle chain on the same (rounded) inputs, fp32 intermediates for
    16-bit tensors (only the gradients themselves are rounded to 16 bits);
    outputs that are not wanted are not touched; K = 3 is left to the caller."""
    from sapa_amd import _lib
    g = gen(170)
    B, d, C, H, W, K, s = 2, 16, 24, 21, 36, 5, 2      # W % 4 == 0, W >= 32: the dot-product stages for 16-bit
    q, key, v = (randn(g, *sh).to(dtype) for sh in ((B, d, H * s, W * s), (B, d, H, W), (B, C, H, W)))
    go = randn(g, B, C, H * s, W * s).to(dtype)
    qd, kd, vd, god = dev(q, key, v, go)
    h = _lib.lib()
    ws = torch.empty(h.sapa_fused_backward_workspace(B, H, W, K, s) // 4, device=DEV)
    gq, gk, gv = (torch.full_like(t, float('nan')) for t in (qd, kd, vd))
    args = (B, d, C, H, W, K, s, _lib.DTYPES[dtype])
    assert _lib.call_status('sapa_fused_backward', DEV, _lib.ptr(god), _lib.ptr(qd), _lib.ptr(kd), _lib.ptr(vd),
                            _lib.ptr(ws), _lib.ptr(gq), _lib.ptr(gk), _lib.ptr(gv), *args) == 0
    want = fused_backward_oracle(coracle, go.float(), q.float(), key.float(), v.float(), K, s)
    for got, w, name in zip((gq, gk, gv), want, ('grad_query', 'grad_key', 'grad_value')):
        assert torch.isfinite(got).all(), name
        if dtype == torch.float32:
            torch.testing.assert_close(got.cpu().double(), w, msg=lambda m: f'{name}: {m}', **tol)
        else:
            assert_rel_rms_close(got.float().cpu(), w, tol, f'{name} {dtype}')
    # only grad_key wanted: the other buffers stay as they are
    gq2, gv2 = torch.full_like(qd, 7.0), torch.full_like(vd, 7.0)
    gk2 = torch.full_like(kd, float('nan'))
    assert _lib.call_status('sapa_fused_backward', DEV, _lib.ptr(god), _lib.ptr(qd), _lib.ptr(kd), _lib.ptr(vd),
                            _lib.ptr(ws), None, _lib.ptr(gk2), None, *args) == 0
    assert torch.equal(gk2, gk) and (gq2 == 7).all() and (gv2 == 7).all()
    # the autograd route takes the same entry point
    leaves = [t.clone().requires_grad_() for t in (qd, kd, vd)]
    sapa_amd.sapa_fused(*leaves, K, s).backward(god)
    for leaf, got in zip(leaves, (gq, gk, gv)):
        assert torch.equal(leaf.grad, got)
    # K = 3: no tiled kernels behind this call
    assert _lib.call_status('sapa_fused_backward', DEV, _lib.ptr(god), _lib.ptr(qd), _lib.ptr(kd), _lib.ptr(vd),
                            _lib.ptr(ws), _lib.ptr(gq), _lib.ptr(gk), _lib.ptr(gv), B, d, C, H, W, 3, s,
                            _lib.DTYPES[dtype]) == _lib.UNSUPPORTED


def test_gradcheck_reference_shapes():
    """sapa/sapa/grad_check.py:8-33: float64 gradcheck at its shapes."""
    from torch.autograd import gradcheck
    g = gen(110)
    b, h, w, c, K, s = 2, 3, 4, 16, 5, 2
    q = torch.rand(b, c, s * h, s * w, generator=g, dtype=torch.float64).to(DEV).requires_grad_()
    k = torch.rand(b, c, h, w, generator=g, dtype=torch.float64).to(DEV).requires_grad_()
    assert gradcheck(sapa_amd.qk, (q, k, K, s))
    a = randn(g, b, K * K, s * h, s * w, dtype=torch.float64).to(DEV).requires_grad_()
    v = randn(g, b, c, h, w, dtype=torch.float64).to(DEV).requires_grad_()
    assert gradcheck(sapa_amd.av, (a, v, K, s), eps=1e-4)
    v3 = randn(g, b, 3, h, w, dtype=torch.float64).to(DEV).requires_grad_()
    assert gradcheck(sapa_amd.sapa_fused, (q, k, v3, K, s), eps=1e-5, atol=1e-6)


def test_fused_backward_matches_composition():
    g = gen(111)
    B, d, C, H, W, K, s = 2, 6, 5, 9, 11, 5, 2
    q, key, v = randn(g, B, d, H * s, W * s), randn(g, B, d, H, W), randn(g, B, C, H, W)
    go = randn(g, B, C, H * s, W * s).to(DEV)
    a = [x.to(DEV).requires_grad_() for x in (q, key, v)]
    b = [x.to(DEV).requires_grad_() for x in (q, key, v)]
    sapa_amd.sapa_fused(*a, K, s).backward(go)
    sapa_amd.av(F.softmax(sapa_amd.qk(b[0], b[1], K, s), dim=1), b[2], K, s).backward(go)
    for x, y in zip(a, b):
        torch.testing.assert_close(x.grad, y.grad, rtol=1e-4, atol=1e-5)


def test_error_behaviour_on_device():
    """qk_cuda.cpp:34-39: non-contiguous tensors are refused, not copied."""
    q = torch.randn(1, 4, 8, 16, device=DEV)[:, :, :, ::2]
    k = torch.randn(1, 4, 4, 4, device=DEV)
    with pytest.raises(RuntimeError):
        sapa_amd.qk(q, k, 5, 2)
    with pytest.raises(RuntimeError):
        sapa_amd.qk(torch.randn(1, 4, 8, 8, device=DEV).double(), k, 5, 2)  # dtype mismatch
    out = sapa_amd.qk(torch.randn(1, 4, 8, 8, device=DEV), k, 5, 2)
    assert out.shape == (1, 25, 8, 8) and out.dtype == torch.float32 and out.is_cuda


def test_sapa_module_forward_and_drop_in_import(coracle):
    """The reference's own caller pattern: `from sapa import qk, av`, then
    av(softmax(qk(q, k)), v) (sapa_base.py:4,38-40); and the SAPA module at
    BASELINE config 1 (1x64x32x32 -> 64x64, d=32, K=5)."""
    from sapa import av, qk
    g = gen(112)
    torch.manual_seed(0)
    m = sapa_amd.SAPA(64, embedding_dim=32).to(DEV)
    y, x = randn(g, 1, 64, 64, 64), randn(g, 1, 64, 32, 32)
    with torch.no_grad():
        out = m(y.to(DEV), x.to(DEV))
        qd, kd = m.q(m.norm_y(y.to(DEV))), m.k(m.norm_x(x.to(DEV)))
        out3 = av(F.softmax(qk(qd, kd, 5, 2), dim=1), x.to(DEV), 5, 2)
    assert out.shape == (1, 64, 64, 64)
    want = coracle.sapa_fused(qd.cpu(), kd.cpu(), x, 5, 2, 'f32')
    assert_f32_close(out.cpu(), want, 'SAPA module (fused)')
    assert_f32_close(out3.cpu(), want, 'reference three-step composition')
    m.fused = False
    with torch.no_grad():
        assert_f32_close(m(y.to(DEV), x.to(DEV)).cpu(), want, 'SAPA module (three-step)')


def test_module_trains():
    torch.manual_seed(1)
    m = sapa_amd.SAPA(32, embedding_dim=16).to(DEV)
    y = torch.randn(2, 32, 16, 24, device=DEV)
    x = torch.randn(2, 32, 8, 12, device=DEV, requires_grad=True)
    m(y, x).square().mean().backward()
    for n, p in m.named_parameters():
        assert p.grad is not None and torch.isfinite(p.grad).all(), n
    assert x.grad is not None and x.grad.abs().sum() > 0


@pytest.mark.parametrize('C', [32, 64, 100, 260])
def test_fused_and_av_with_sliced_value_channels(coracle, C):
    """Few tiles and many value channels: the launcher slices the channels
    over several workgroups per tile (ragged last slice at C=100, 260)."""
    B, d, H, W, K, s = 1, 8, 10, 20, 5, 2
    g = gen(113)
    q, key, v = randn(g, B, d, H * s, W * s), randn(g, B, d, H, W), randn(g, B, C, H, W)
    attn = F.softmax(randn(g, B, K * K, H * s, W * s), 1)
    got = sapa_amd.sapa_fused(*dev(q, key, v), K, s).cpu()
    assert_f32_close(got, coracle.sapa_fused(q, key, v, K, s, 'f32'), f'fused C={C}')
    assert torch.equal(sapa_amd.av(*dev(attn, v), K, s).cpu(), coracle.av(attn, v, K, s, 'f32'))


@pytest.mark.parametrize('W', [20, 22, 21, 36, 34, 33])
def test_window_staging_vector_widths(coracle, W):
    """Row lengths that are multiples of 4, of 2 only, and odd select the
    4-, 2- and 1-element staging loads of the tiled kernel; a sliced view
    shifts the base pointer off 16-byte alignment."""
    B, d, C, H, K, s = 2, 8, 8, 9, 5, 2
    g = gen(114)
    q, key, v = randn(g, B, d, H * s, W * s), randn(g, B, d, H, W), randn(g, B, C + 1, H, W)
    vd = v.to(DEV)[:, 1:].contiguous()
    got = sapa_amd.sapa_fused(q.to(DEV), key.to(DEV), vd, K, s).cpu()
    assert_f32_close(got, coracle.sapa_fused(q, key, v[:, 1:].contiguous(), K, s, 'f32'), f'W={W}')
    # an unaligned (but contiguous) value tensor: flat storage offset of one element
    flat = torch.empty(B * C * H * W + 1, device=DEV)
    vu = flat[1:].view(B, C, H, W)
    vu.copy_(v[:, 1:])
    got = sapa_amd.sapa_fused(q.to(DEV), key.to(DEV), vu, K, s).cpu()
    assert_f32_close(got, coracle.sapa_fused(q, key, v[:, 1:].contiguous(), K, s, 'f32'), f'W={W} unaligned')
    logits = sapa_amd.qk(q.to(DEV), key.to(DEV), K, s).cpu()
    assert torch.equal(logits, coracle.qk(q, key, K, s, 'f32'))


# (B, d, C, H, W): rows that are multiples of 4 elements at 16-byte aligned tensors, one case per tile
# geometry the launcher picks for fp32 (32 x 8 tiles; 16 x 16; 16 x 8; the two-waves-per-band
# geometry of small problems), with ragged tiles, channel counts off the chunk size and a sliced
# value tensor
LDS_DIRECT_SHAPES = [(2, 13, 21, 100, 168), (5, 9, 10, 128, 48), (4, 9, 10, 136, 48), (3, 20, 37, 19, 44),
                     (1, 3, 2, 1, 4), (1, 64, 260, 10, 20)]


@pytest.mark.parametrize('shape', LDS_DIRECT_SHAPES, ids=['-'.join(map(str, s)) for s in LDS_DIRECT_SHAPES])
def test_windows_loaded_straight_into_lds(coracle, shape):
    """fp32 windows whose rows allow 16-byte vectors go from global memory straight into LDS
    (zero padding = the hardware's zero for an out-of-range offset): qk and av stay bit-exact,
    the fused result within the stated bar, values at the image border included."""
    B, d, C, H, W = shape
    K, s = 5, 2
    g = gen(121)
    q, key, v = randn(g, B, d, H * s, W * s), randn(g, B, d, H, W), randn(g, B, C, H, W)
    attn = F.softmax(randn(g, B, K * K, H * s, W * s), 1)
    # large values on the border cells: a wrong padding or a shifted window row shows at once
    # (in the two bit-exact comparisons only: in the fused one they would turn the bar, which
    # is relative to the result, into one on cancelling terms 64 times its size)
    def border(t, f):
        t = t.clone()
        t[:, :, 0, :] *= f
        t[:, :, -1, :] *= f
        t[:, :, :, 0] *= f
        t[:, :, :, -1] *= f
        return t
    kb, vb = border(key, 64.0), border(v, 64.0)
    assert torch.equal(sapa_amd.qk(*dev(q, kb), K, s).cpu(), coracle.qk(q, kb, K, s, 'f32'))
    assert torch.equal(sapa_amd.av(*dev(attn, vb), K, s).cpu(), coracle.av(attn, vb, K, s, 'f32'))
    got = sapa_amd.sapa_fused(*dev(q, key, v), K, s).cpu()
    assert_f32_close(got, coracle.sapa_fused(q, key, v, K, s, 'f32'), f'fused {shape}')
    assert sapa_amd._lib.last_kernel().startswith('sapa_b_tiled_kernel') or B * H * W <= 12288


def test_module_with_folded_groupnorm_matches_two_step():
    """SAPA(fold_norm=True) = the same module with GroupNorm and the 1x1
    projections as separate steps (sapa_base.py:26-36), up to rounding."""
    torch.manual_seed(5)
    m = sapa_amd.SAPA(64, embedding_dim=16).to(DEV)
    torch.nn.init.normal_(m.norm_y.weight, 1.0, 0.2)
    torch.nn.init.normal_(m.norm_x.bias, 0.0, 0.2)
    torch.nn.init.normal_(m.q.weight, std=0.2)
    torch.nn.init.normal_(m.k.weight, std=0.2)
    y = torch.randn(2, 64, 18, 22, device=DEV) + 0.5
    x = torch.randn(2, 64, 9, 11, device=DEV)
    with torch.no_grad():
        want = m(y, x)
        m.fold_norm = True
        got = m(y, x)
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-4)
    md = sapa_amd.SAPADeform(64, embedding_dim=8, norm=True).to(DEV)
    torch.nn.init.normal_(md.offset.weight, std=0.1)
    with torch.no_grad():
        want = md(y, x)
        md.fold_norm = True
        got = md(y, x)
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-4)


def test_av_backward_logits_entry_point(coracle):
    """sapa_av_backward_logits = softmax backward applied to the grad_attn of
    the aggregation, against float64 arithmetic on the oracle's grad_attn."""
    from sapa_amd import _lib
    g = gen(160)
    B, C, H, W, K, s = 2, 11, 9, 21, 5, 2
    attn = torch.softmax(randn(g, B, K * K, H * s, W * s) * 2, dim=1)
    v, go = randn(g, B, C, H, W), randn(g, B, C, H * s, W * s)
    ga, _ = coracle.av_backward(go.double(), attn.double(), v.double(), K, s, 'f64')
    a64 = attn.double()
    want = a64 * (ga - (ga * a64).sum(dim=1, keepdim=True))
    ad, vd, god = dev(attn, v, go)
    got = torch.full_like(ad, float('nan'))
    status = _lib.call_status('sapa_av_backward_logits', ad.device, _lib.ptr(god), _lib.ptr(ad),
                              _lib.ptr(vd), _lib.ptr(got), B, C, H, W, K, s, 0)
    assert status == 0
    torch.testing.assert_close(got.cpu().double(), want, rtol=1e-4, atol=1e-5)
    # no register-tiled instance for K = 7, s = 1: the caller is told so
    a7 = torch.softmax(randn(g, 1, 49, 6, 7), dim=1).to(DEV)
    out7 = torch.empty_like(a7)
    status = _lib.call_status('sapa_av_backward_logits', a7.device, _lib.ptr(randn(g, 1, 3, 6, 7).to(DEV)),
                              _lib.ptr(a7), _lib.ptr(randn(g, 1, 3, 6, 7).to(DEV)), _lib.ptr(out7),
                              1, 3, 6, 7, 7, 1, 0)
    assert status == _lib.UNSUPPORTED
