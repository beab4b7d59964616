"""Pins the CPU oracle before anything is compared with it.

The reference holds no golden vectors for this path (its checks are
relational, on unseeded data), so each oracle function is pinned by
  * two independent restatements agreeing (library routines in
    oracle/torch_oracle.py vs brute-force loops in oracle/sapa_oracle.c vs
    pure-Python loops written here from the kernels' index math),
  * closed forms and special cases that reduce to textbook/library routines,
  * integer-valued inputs, on which every product and sum is exact in fp32,
    so that any index error is a hard mismatch whatever the summation order.
"""
import itertools

import pytest
import torch
import torch.nn.functional as F

from oracle import torch_oracle as T


def gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def randn(g, *shape, dtype=torch.float64):
    return torch.randn(*shape, generator=g, dtype=dtype)


def randint(g, lo, hi, *shape, dtype=torch.float32):
    return torch.randint(lo, hi, shape, generator=g).to(dtype)


SHAPES = [  # B, d, H, W, K, s
    (2, 3, 4, 5, 1, 1), (2, 3, 4, 5, 3, 1), (2, 3, 4, 5, 5, 2),
    (1, 4, 3, 7, 3, 3), (2, 2, 6, 4, 7, 2), (1, 5, 2, 2, 5, 4),
]


# ---------------------------------------------------------------- python loops
def qk_loops(q, key, K, s):
    """qk_cuda_kernel.cu:41-66, one output element at a time."""
    B, d, H, W = key.shape
    r = (K - 1) // 2
    out = torch.zeros(B, K * K, H * s, W * s, dtype=q.dtype)
    for n, k, ph, pw in itertools.product(range(B), range(K * K), range(H * s), range(W * s)):
        dh = ph // s - r + k // K
        dw = pw // s - r + k % K
        if dh < 0 or dh > H - 1 or dw < 0 or dw > W - 1:
            continue
        out[n, k, ph, pw] = sum(key[n, c, dh, dw] * q[n, c, ph, pw] for c in range(d))
    return out


def av_loops(attn, v, K, s):
    """av_cuda_kernel.cu:39-73."""
    B, C, H, W = v.shape
    r = (K - 1) // 2
    out = torch.zeros(B, C, H * s, W * s, dtype=v.dtype)
    for n, c, ph, pw in itertools.product(range(B), range(C), range(H * s), range(W * s)):
        acc = 0.0
        for iy in range(ph // s - r, ph // s + r + 1):
            for ix in range(pw // s - r, pw // s + r + 1):
                if iy < 0 or iy > H - 1 or ix < 0 or ix > W - 1:
                    continue
                mc = (iy - ph // s + r) * K + (ix - pw // s + r)
                acc += v[n, c, iy, ix] * attn[n, mc, ph, pw]
        out[n, c, ph, pw] = acc
    return out


def bilinear_loops(plane, h, w):
    """deform_qk_cuda_kernel.cu:23-68 on python floats."""
    import math
    H, W = plane.shape
    hl, wl = math.floor(h), math.floor(w)
    hh_, wh = hl + 1, wl + 1
    lh, lw = h - hl, w - wl
    v = [0.0] * 4
    if hl >= 0 and wl >= 0:
        v[0] = plane[hl, wl].item()
    if hl >= 0 and wh <= W - 1:
        v[1] = plane[hl, wh].item()
    if hh_ <= H - 1 and wl >= 0:
        v[2] = plane[hh_, wl].item()
    if hh_ <= H - 1 and wh <= W - 1:
        v[3] = plane[hh_, wh].item()
    return (1 - lh) * (1 - lw) * v[0] + (1 - lh) * lw * v[1] + lh * (1 - lw) * v[2] + lh * lw * v[3]


def deform_qk_loops(q, key, off, P, s, G):
    """deform_qk_cuda_kernel.cu:152-195."""
    B, Cq, H, W = key.shape
    d = Cq // G
    out = torch.zeros(B, G, P, H * s, W * s, dtype=q.dtype)
    for b, g, p, qh, qw in itertools.product(range(B), range(G), range(P), range(H * s), range(W * s)):
        ow = off[b, 2 * (g * P + p), qh, qw].item()
        oh = off[b, 2 * (g * P + p) + 1, qh, qw].item()
        kh, kw = qh // s + oh, qw // s + ow
        if kh > -1 and kh < H and kw > -1 and kw < W:
            out[b, g, p, qh, qw] = sum(
                q[b, g * d + c, qh, qw].item() * bilinear_loops(key[b, g * d + c], kh, kw)
                for c in range(d))
    return out


def deform_av_loops(attn, v, off, P, s, G):
    """deform_av_cuda_kernel.cu:152-193."""
    B, C, H, W = v.shape
    out = torch.zeros(B, C, H * s, W * s, dtype=v.dtype)
    for b, c, qh, qw in itertools.product(range(B), range(C), range(H * s), range(W * s)):
        g = c // (C // G)
        acc = 0.0
        for p in range(P):
            ow = off[b, 2 * (g * P + p), qh, qw].item()
            oh = off[b, 2 * (g * P + p) + 1, qh, qw].item()
            kh, kw = qh // s + oh, qw // s + ow
            if kh > -1 and kh < H and kw > -1 and kw < W:
                acc += attn[b, g, p, qh, qw].item() * bilinear_loops(v[b, c], kh, kw)
        out[b, c, qh, qw] = acc
    return out


def up_nearest(x, s):
    return x.repeat_interleave(s, dim=-2).repeat_interleave(s, dim=-1)


def shift2d(x, dy, dx):
    """y[..., i, j] = x[..., i+dy, j+dx], zero outside."""
    H, W = x.shape[-2:]
    y = torch.zeros_like(x)
    ys = slice(max(0, -dy), min(H, H - dy))
    xs = slice(max(0, -dx), min(W, W - dx))
    yd = slice(max(0, -dy) + dy, min(H, H - dy) + dy)
    xd = slice(max(0, -dx) + dx, min(W, W - dx) + dx)
    y[..., ys, xs] = x[..., yd, xd]
    return y


# ------------------------------------------------------------------------- qk
@pytest.mark.parametrize('B,d,H,W,K,s', SHAPES)
def test_qk_three_restatements_agree(coracle, B, d, H, W, K, s):
    g = gen(1)
    q, key = randn(g, B, d, H * s, W * s), randn(g, B, d, H, W)
    ref = qk_loops(q, key, K, s)
    torch.testing.assert_close(T.qk(q, key, K, s), ref, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(coracle.qk(q, key, K, s, 'f64'), ref, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize('B,d,H,W,K,s', SHAPES)
def test_qk_integer_inputs_exact_in_fp32(coracle, B, d, H, W, K, s):
    g = gen(2)
    q, key = randint(g, -4, 5, B, d, H * s, W * s), randint(g, -4, 5, B, d, H, W)
    a = coracle.qk(q, key, K, s, 'f32')
    assert torch.equal(a, T.qk(q, key, K, s))
    assert torch.equal(a.double(), coracle.qk(q, key, K, s, 'f32a64'))
    assert torch.equal(a, qk_loops(q, key, K, s))


def test_qk_closed_forms(coracle):
    g = gen(3)
    B, d, H, W = 2, 6, 5, 7
    # K=1, s=1: plain channel dot product
    q, key = randn(g, B, d, H, W), randn(g, B, d, H, W)
    torch.testing.assert_close(coracle.qk(q, key, 1, 1, 'f64'),
                               (q * key).sum(1, keepdim=True), rtol=1e-12, atol=1e-12)
    # q == 1: windows of the channel-summed key, nearest-upsampled
    K, s = 5, 2
    key = randn(g, B, d, H, W)
    ones = torch.ones(B, d, H * s, W * s, dtype=torch.float64)
    want = up_nearest(F.unfold(key.sum(1, keepdim=True), K, padding=K // 2).reshape(B, K * K, H, W), s)
    torch.testing.assert_close(coracle.qk(ones, key, K, s, 'f64'), want, rtol=1e-12, atol=1e-12)
    # q one-hot in channel c0: plane k is key[:, c0] shifted by (ky-r, kx-r)
    c0 = 4
    q = torch.zeros(B, d, H * s, W * s, dtype=torch.float64)
    q[:, c0] = 1
    got = coracle.qk(q, key, K, s, 'f64')
    for ky in range(K):
        for kx in range(K):
            want = up_nearest(shift2d(key[:, c0], ky - 2, kx - 2), s)
            assert torch.equal(got[:, ky * K + kx], want), (ky, kx)


def test_qk_invariants(coracle):
    g = gen(4)
    B, d, H, W, K, s = 1, 3, 4, 4, 5, 2
    q, key = randn(g, B, d, H * s, W * s), randn(g, B, d, H, W)
    out = coracle.qk(q, key, K, s, 'f64')
    # bilinear in (q, key)
    q2, key2 = randn(g, *q.shape), randn(g, *key.shape)
    torch.testing.assert_close(coracle.qk(q + 2 * q2, key, K, s, 'f64'),
                               out + 2 * coracle.qk(q2, key, K, s, 'f64'), rtol=1e-11, atol=1e-11)
    torch.testing.assert_close(coracle.qk(q, key - 3 * key2, K, s, 'f64'),
                               out - 3 * coracle.qk(q, key2, K, s, 'f64'), rtol=1e-11, atol=1e-11)
    # out-of-range neighbours are exact zeros: top-left pixel, ky<r or kx<r
    for ky in range(K):
        for kx in range(K):
            if ky < 2 or kx < 2:
                assert out[0, ky * K + kx, 0, 0] == 0
            else:
                assert out[0, ky * K + kx, 0, 0] != 0
    # the s*s children of one cell see the same key window: equal q => equal logits
    qc = up_nearest(randn(g, B, d, H, W), s)
    o = coracle.qk(qc, key, K, s, 'f64').reshape(B, K * K, H, s, W, s)
    assert torch.equal(o[:, :, :, 0, :, 0], o[:, :, :, 1, :, 1])
    assert torch.equal(o[:, :, :, 0, :, 1], o[:, :, :, 1, :, 0])


# -------------------------------------------------------------------- softmax
def test_softmax(coracle):
    g = gen(5)
    x = randn(g, 2, 25, 6, 4) * 3
    y = coracle.softmax(x, 1, 'f64')
    torch.testing.assert_close(y, F.softmax(x, dim=1), rtol=1e-13, atol=1e-15)
    torch.testing.assert_close(y.sum(1), torch.ones(2, 6, 4, dtype=torch.float64), rtol=1e-13, atol=0)
    torch.testing.assert_close(coracle.softmax(x + 7.5, 1, 'f64'), y, rtol=1e-12, atol=1e-15)
    x5 = randn(g, 2, 4, 9, 3, 5)
    torch.testing.assert_close(coracle.softmax(x5, 2, 'f64'), F.softmax(x5, dim=2), rtol=1e-13, atol=1e-15)
    xf = x.float()
    torch.testing.assert_close(coracle.softmax(xf, 1, 'f32'), F.softmax(xf, dim=1), rtol=1e-5, atol=1e-7)


def test_softmax_oob_logits_take_weight(coracle):
    """A zero logit (out-of-range neighbour) is a real participant, not -inf."""
    x = torch.tensor([0.0, 1.0, 0.0, -2.0], dtype=torch.float64).view(1, 4, 1)
    y = coracle.softmax(x, 1, 'f64').view(-1)
    z = torch.exp(x.view(-1) - 1.0)
    torch.testing.assert_close(y, z / z.sum(), rtol=1e-14, atol=0)
    assert y[0] > 0.1


# ------------------------------------------------------------------------- av
@pytest.mark.parametrize('B,C,H,W,K,s', SHAPES)
def test_av_three_restatements_agree(coracle, B, C, H, W, K, s):
    g = gen(6)
    attn, v = randn(g, B, K * K, H * s, W * s), randn(g, B, C, H, W)
    ref = av_loops(attn, v, K, s)
    torch.testing.assert_close(T.av(attn, v, K, s), ref, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(coracle.av(attn, v, K, s, 'f64'), ref, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize('B,C,H,W,K,s', SHAPES)
def test_av_integer_inputs_exact_in_fp32(coracle, B, C, H, W, K, s):
    g = gen(7)
    attn, v = randint(g, -3, 4, B, K * K, H * s, W * s), randint(g, -3, 4, B, C, H, W)
    a = coracle.av(attn, v, K, s, 'f32')
    assert torch.equal(a, T.av(attn, v, K, s))
    assert torch.equal(a.double(), coracle.av(attn, v, K, s, 'f32a64'))
    assert torch.equal(a, av_loops(attn, v, K, s))


def test_av_closed_forms(coracle):
    g = gen(8)
    B, C, H, W, K, s = 2, 3, 6, 5, 5, 2
    v = randn(g, B, C, H, W)
    # one-hot attention at k: nearest-upsample of v shifted by (ky-r, kx-r)
    for k in (0, 7, 12, 24):
        attn = torch.zeros(B, K * K, H * s, W * s, dtype=torch.float64)
        attn[:, k] = 1
        want = up_nearest(shift2d(v, k // K - 2, k % K - 2), s)
        assert torch.equal(coracle.av(attn, v, K, s, 'f64'), want), k
    # uniform attention: box filter that counts the zero padding
    attn = torch.full((B, K * K, H * s, W * s), 1.0 / (K * K), dtype=torch.float64)
    want = up_nearest(F.avg_pool2d(v, K, 1, K // 2, count_include_pad=True), s)
    torch.testing.assert_close(coracle.av(attn, v, K, s, 'f64'), want, rtol=1e-12, atol=1e-13)


def test_fused_zero_query_is_box_filter(coracle):
    """q == 0: all logits 0, including the out-of-range ones, so attention is
    uniform 1/K^2 everywhere (borders too) and the result is the box filter."""
    g = gen(9)
    B, d, C, H, W, K, s = 1, 4, 3, 5, 6, 5, 2
    key, v = randn(g, B, d, H, W), randn(g, B, C, H, W)
    q = torch.zeros(B, d, H * s, W * s, dtype=torch.float64)
    want = up_nearest(F.avg_pool2d(v, K, 1, K // 2, count_include_pad=True), s)
    torch.testing.assert_close(coracle.sapa_fused(q, key, v, K, s, 'f64'), want, rtol=1e-12, atol=1e-13)
    torch.testing.assert_close(T.sapa_fused(q, key, v, K, s), want, rtol=1e-12, atol=1e-13)


def test_fused_is_composition(coracle):
    g = gen(10)
    B, d, C, H, W, K, s = 2, 5, 4, 4, 6, 3, 2
    q, key, v = randn(g, B, d, H * s, W * s), randn(g, B, d, H, W), randn(g, B, C, H, W)
    want = T.av(F.softmax(T.qk(q, key, K, s), dim=1), v, K, s)
    torch.testing.assert_close(coracle.sapa_fused(q, key, v, K, s, 'f64'), want, rtol=1e-11, atol=1e-12)
    torch.testing.assert_close(coracle.sapa_fused(q.float(), key.float(), v.float(), K, s, 'f32a64'),
                               T.sapa_fused(q.float().double(), key.float().double(), v.float().double(), K, s),
                               rtol=1e-11, atol=1e-12)


# --------------------------------------------------------------------- deform
DSHAPES = [  # B, G, d, H, W, P, s
    (2, 2, 3, 4, 5, 3, 2), (1, 4, 2, 3, 4, 5, 2), (1, 1, 4, 5, 3, 4, 3), (2, 2, 2, 3, 3, 2, 1),
]


@pytest.mark.parametrize('B,G,d,H,W,P,s', DSHAPES)
def test_deform_qk_three_restatements_agree(coracle, B, G, d, H, W, P, s):
    g = gen(11)
    q, key = randn(g, B, G * d, H * s, W * s), randn(g, B, G * d, H, W)
    off = randn(g, B, 2 * G * P, H * s, W * s) * 1.5
    ref = deform_qk_loops(q, key, off, P, s, G)
    torch.testing.assert_close(coracle.deform_qk(q, key, off, P, s, G, 'f64'), ref, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(T.deform_qk(q, key, off, P, s, G), ref, rtol=1e-9, atol=1e-10)


@pytest.mark.parametrize('B,G,d,H,W,P,s', DSHAPES)
def test_deform_av_three_restatements_agree(coracle, B, G, d, H, W, P, s):
    g = gen(12)
    C = G * d
    attn, v = randn(g, B, G, P, H * s, W * s), randn(g, B, C, H, W)
    off = randn(g, B, 2 * G * P, H * s, W * s) * 1.5
    ref = deform_av_loops(attn, v, off, P, s, G)
    torch.testing.assert_close(coracle.deform_av(attn, v, off, P, s, G, 'f64'), ref, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(T.deform_av(attn, v, off, P, s, G), ref, rtol=1e-9, atol=1e-10)


def regular_grid_offsets(B, K, sH, sW, dtype):
    """Offsets that turn the sampled ops into the KxK-window ops: point
    p = ky*K+kx sits at (dy, dx) = (ky-r, kx-r); channel 2p = dx, 2p+1 = dy."""
    r = (K - 1) // 2
    off = torch.zeros(B, 2 * K * K, sH, sW, dtype=dtype)
    for ky in range(K):
        for kx in range(K):
            p = ky * K + kx
            off[:, 2 * p] = kx - r
            off[:, 2 * p + 1] = ky - r
    return off


@pytest.mark.parametrize('K,s', [(3, 2), (5, 2), (5, 1), (3, 3)])
def test_deform_on_regular_grid_is_sapa_b(coracle, K, s):
    """G=1, P=K*K, integer offsets on the window grid: deform_qk == qk and
    deform_av == av exactly (cross-pins the two operator families)."""
    g = gen(13)
    B, d, C, H, W = 2, 4, 3, 5, 6
    q, key, v = randn(g, B, d, H * s, W * s), randn(g, B, d, H, W), randn(g, B, C, H, W)
    attn = randn(g, B, K * K, H * s, W * s)
    off = regular_grid_offsets(B, K, H * s, W * s, torch.float64)
    a = coracle.deform_qk(q, key, off, K * K, s, 1, 'f64')
    assert torch.equal(a.reshape(B, K * K, H * s, W * s), coracle.qk(q, key, K, s, 'f64'))
    b = coracle.deform_av(attn.reshape(B, 1, K * K, H * s, W * s), v, off, K * K, s, 1, 'f64')
    assert torch.equal(b, coracle.av(attn, v, K, s, 'f64'))
    # same in the kernels' fp32 arithmetic: integer offsets give weights 1,0,0,0
    a32 = coracle.deform_qk(q.float(), key.float(), off.float(), K * K, s, 1, 'f32')
    assert torch.equal(a32.reshape(B, K * K, H * s, W * s), coracle.qk(q.float(), key.float(), K, s, 'f32'))


def test_deform_closed_forms(coracle):
    g = gen(14)
    B, G, d, H, W, P, s = 1, 2, 3, 4, 5, 2, 2
    q, key = randn(g, B, G * d, H * s, W * s), randn(g, B, G * d, H, W)
    # zero offsets: per-group dot of q with the nearest-upsampled key
    off = torch.zeros(B, 2 * G * P, H * s, W * s, dtype=torch.float64)
    want = (q * up_nearest(key, s)).reshape(B, G, 1, d, H * s, W * s).sum(3).expand(B, G, P, H * s, W * s)
    torch.testing.assert_close(coracle.deform_qk(q, key, off, P, s, G, 'f64'), want, rtol=1e-12, atol=1e-12)
    # half-integer offsets: mean of the 2 (dx) or 4 (dx, dy) neighbours, zero padded
    v = randn(g, B, G, H, W)          # C = G: one channel per group
    attn = torch.ones(B, G, 1, H * s, W * s, dtype=torch.float64)
    off = torch.zeros(B, 2 * G, H * s, W * s, dtype=torch.float64)
    off[:, 0::2] = 0.5
    want = up_nearest(0.5 * (v + shift2d(v, 0, 1)), s)
    torch.testing.assert_close(coracle.deform_av(attn, v, off, 1, s, G, 'f64'), want, rtol=1e-13, atol=1e-13)
    off[:, 1::2] = -0.5
    want = up_nearest(0.25 * (v + shift2d(v, 0, 1) + shift2d(v, -1, 0) + shift2d(v, -1, 1)), s)
    torch.testing.assert_close(coracle.deform_av(attn, v, off, 1, s, G, 'f64'), want, rtol=1e-13, atol=1e-13)


def test_deform_guard_and_negative_floor(coracle):
    """Strict guard kh > -1, kh < H (deform_qk_cuda_kernel.cu:187) and floor of
    negative coordinates: a sample at -0.25 keeps 0.75 of row 0."""
    B, G, H, W, s, P = 1, 1, 3, 3, 1, 1
    v = torch.arange(1.0, 10.0, dtype=torch.float64).view(1, 1, 3, 3)
    attn = torch.ones(B, G, P, H, W, dtype=torch.float64)

    def run(dx, dy):
        off = torch.zeros(B, 2, H, W, dtype=torch.float64)
        off[:, 0], off[:, 1] = dx, dy
        return coracle.deform_av(attn, v, off, P, s, G, 'f64')[0, 0]

    out = run(0.0, -0.25)
    assert out[0, 0].item() == 0.75 * 1.0           # row -1 is padding
    assert out[1, 1].item() == 0.25 * 2.0 + 0.75 * 5.0
    out = run(-1.0, 0.0)                            # kw == -1 at column 0: guard fails
    assert out[0, 0].item() == 0.0 and out[0, 1].item() == 1.0
    out = run(-3.0, 0.0)
    assert torch.count_nonzero(out) == 0
    out = run(0.0, 1.0)                             # last row: kh == H, guard fails
    assert out[2, 0].item() == 0.0 and out[1, 0].item() == 7.0
    out = run(0.75, 0.0)                            # last column keeps 0.25 of itself
    assert out[0, 2].item() == 0.25 * 3.0


def test_deform_group_mapping(coracle):
    """g(c) = c // (C/G): attention that is non-zero in one group only lights
    exactly that group's channels."""
    g = gen(15)
    B, G, cg, H, W, P, s = 1, 4, 3, 3, 3, 2, 2
    v = randn(g, B, G * cg, H, W) + 5
    off = torch.zeros(B, 2 * G * P, H * s, W * s, dtype=torch.float64)
    for gi in range(G):
        attn = torch.zeros(B, G, P, H * s, W * s, dtype=torch.float64)
        attn[:, gi] = 1
        out = coracle.deform_av(attn, v, off, P, s, G, 'f64')
        lit = (out.abs().sum(dim=(0, 2, 3)) > 0).nonzero().view(-1).tolist()
        assert lit == list(range(gi * cg, (gi + 1) * cg))


def test_deform_offset_channel_layout(coracle):
    """Channel 2*(g*P+p) is dx (width), +1 is dy (height)."""
    B, G, P, H, W, s = 1, 2, 2, 4, 4, 1
    v = torch.zeros(B, G, H, W, dtype=torch.float64)
    v[0, 1, 1, 2] = 1.0                              # group 1: a dot at (y=1, x=2)
    attn = torch.zeros(B, G, P, H, W, dtype=torch.float64)
    attn[0, 1, 1] = 1.0                              # only point p=1 of group 1
    off = torch.zeros(B, 2 * G * P, H, W, dtype=torch.float64)
    off[0, 2 * (1 * P + 1)] = 2.0                    # dx = +2
    off[0, 2 * (1 * P + 1) + 1] = 1.0                # dy = +1
    out = coracle.deform_av(attn, v, off, P, s, G, 'f64')
    assert out[0, 1, 0, 0] == 1.0 and out[0, 1].sum() == 1.0 and out[0, 0].sum() == 0.0


# ------------------------------------------------------------------- backward
def test_backward_oracles_match_autograd(coracle):
    """The scatter-form backward transcriptions equal autograd through the
    library restatement (float64)."""
    g = gen(16)
    B, d, C, H, W, K, s = 2, 3, 4, 4, 5, 5, 2
    q = randn(g, B, d, H * s, W * s).requires_grad_()
    key = randn(g, B, d, H, W).requires_grad_()
    go = randn(g, B, K * K, H * s, W * s)
    T.qk(q, key, K, s).backward(go)
    gq, gk = coracle.qk_backward(go, q.detach(), key.detach(), K, s, 'f64')
    torch.testing.assert_close(gq, q.grad, rtol=1e-11, atol=1e-12)
    torch.testing.assert_close(gk, key.grad, rtol=1e-11, atol=1e-12)

    attn = randn(g, B, K * K, H * s, W * s).requires_grad_()
    v = randn(g, B, C, H, W).requires_grad_()
    go = randn(g, B, C, H * s, W * s)
    T.av(attn, v, K, s).backward(go)
    ga, gv = coracle.av_backward(go, attn.detach(), v.detach(), K, s, 'f64')
    torch.testing.assert_close(ga, attn.grad, rtol=1e-11, atol=1e-12)
    torch.testing.assert_close(gv, v.grad, rtol=1e-11, atol=1e-12)


def test_deform_backward_oracles_match_autograd(coracle):
    g = gen(17)
    B, G, d, H, W, P, s = 2, 2, 3, 4, 5, 3, 2
    q = randn(g, B, G * d, H * s, W * s).requires_grad_()
    key = randn(g, B, G * d, H, W).requires_grad_()
    # offsets in (0,1) like the reference's grad check: away from bilinear kinks
    off = (torch.rand(B, 2 * G * P, H * s, W * s, generator=g, dtype=torch.float64) * 0.9 + 0.05).requires_grad_()
    go = randn(g, B, G, P, H * s, W * s)
    T.deform_qk(q, key, off, P, s, G).backward(go)
    gq, gk, goff = coracle.deform_qk_backward(go, q.detach(), key.detach(), off.detach(), P, s, G, 'f64')
    torch.testing.assert_close(gq, q.grad, rtol=1e-9, atol=1e-10)
    torch.testing.assert_close(gk, key.grad, rtol=1e-9, atol=1e-10)
    torch.testing.assert_close(goff, off.grad, rtol=1e-8, atol=1e-9)

    attn = randn(g, B, G, P, H * s, W * s).requires_grad_()
    v = randn(g, B, G * d, H, W).requires_grad_()
    off = off.detach().clone().requires_grad_()
    go = randn(g, B, G * d, H * s, W * s)
    T.deform_av(attn, v, off, P, s, G).backward(go)
    ga, gv, goff = coracle.deform_av_backward(go, attn.detach(), v.detach(), off.detach(), P, s, G, 'f64')
    torch.testing.assert_close(ga, attn.grad, rtol=1e-9, atol=1e-10)
    torch.testing.assert_close(gv, v.grad, rtol=1e-9, atol=1e-10)
    torch.testing.assert_close(goff, off.grad, rtol=1e-8, atol=1e-9)


def test_reference_forward_check_shape(coracle):
    """The reference's own check shape (sapa/sapa/forward_check.py:29-46,
    deformsapa/deformsapa/forward_check.py:45-64) at its own tolerance:
    library restatement vs kernel-arithmetic oracle, fp32."""
    g = gen(18)
    b, h, w, c, K, s, P, G = 4, 10, 12, 8, 5, 2, 5, 4
    q, k = randn(g, b, c, s * h, s * w, dtype=torch.float32), randn(g, b, c, h, w, dtype=torch.float32)
    assert torch.allclose(T.qk(q, k, K, s), coracle.qk(q, k, K, s, 'f32'), atol=1e-5)
    attn, v = randn(g, b, K * K, s * h, s * w, dtype=torch.float32), randn(g, b, c, h, w, dtype=torch.float32)
    assert torch.allclose(T.av(attn, v, K, s), coracle.av(attn, v, K, s, 'f32'), atol=1e-5)
    off = randn(g, b, G * P * 2, s * h, s * w, dtype=torch.float32)
    assert torch.allclose(T.deform_qk(q, k, off, P, s, G), coracle.deform_qk(q, k, off, P, s, G, 'f32'), atol=1e-5)
    attn = randn(g, b, G, P, s * h, s * w, dtype=torch.float32)
    assert torch.allclose(T.deform_av(attn, v, off, P, s, G), coracle.deform_av(attn, v, off, P, s, G, 'f32'), atol=1e-5)
