"""GPU: every benchmark configuration at its own parameters.

  c2  SegFormer-style chain  B8  C256 d32  K5 s2  16^2 -> 32^2 -> 64^2 -> 128^2,
      query / key from the module's 1x1 projections (normal_(std=.02))
  c3  FPN levels             B16 C256 d64  K5 s2  25x42, 50x84, 100x168 -> x2,
      keys scaled per channel ~U(0.5, 2); fp32 and bf16
  c4  SAPA-D                 B8  C256 d32 G4  64^2 -> 128^2, P in {25, 9, 5},
      offsets clamp(0.75 randn, +-4); with a sigmoid gate on the logits
  c5  stress                 B4  C512 d64  K7 s4  64^2 -> 256^2, bf16, 10 % of
      the query elements Student-t(3)

One or two full-resolution images are compared with the C oracle (the
reference kernels' arithmetic, qk_cuda_kernel.cu:39-67, av_cuda_kernel.cu:37-74,
deform_*_cuda_kernel.cu:139-197, composed as sapa_base.py:38-40 /
sapa_deform.py:51-53); the full batch goes through properties a wrong tile,
channel slice or batch stride breaks: the batch result equals the per-image
results bit for bit, a zero query gives the box filter, integer-valued inputs
give exact logits and sums.  Contiguous and channels_last tensors both.
The backward passes likewise: c3's low-res gradients on integer-valued tensors
at the levels' own sizes, bit for bit; the fused backward of one image per
level against the float64 chain, the batch against its images.

Bars: fp32 |a-b| <= 1e-6 + 1e-5 |b| against the reference-order ('f32')
oracle; bf16 |a-b| <= 1e-2 max(|b|, rms(b)) against the oracle with double
sums on the bf16-rounded inputs.  The channels_last fp32 kernel sums the
channels of a logit in tree order, not the reference's sequential order: its
bar is that it is no further from the exact (double) result than the
reference order is: RMS error, number of elements outside the fp32 bar and
largest error (assert_no_worse_than_reference_order).
"""
from concurrent.futures import ThreadPoolExecutor

import pytest
import torch
import torch.nn.functional as F

import sapa_amd
from helpers import (BF16_REL, F32_ATOL, F32_RTOL, assert_f32_close, assert_rel_rms_close,
                     deform_fused_backward_oracle, fused_backward_oracle, gen, randn)

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'
CL = torch.channels_last


def dev(*ts):
    return [t.to(DEV) for t in ts]


def as_cl(*ts):
    return [t.contiguous(memory_format=CL) for t in ts]


def per_image(fn, tensors, *args, images=None):
    """fn on single images in host threads (the C oracle is single-threaded and
    ctypes releases the GIL), concatenated."""
    idx = list(range(tensors[0].shape[0])) if images is None else list(images)
    with ThreadPoolExecutor(max_workers=min(8, len(idx))) as ex:
        outs = list(ex.map(lambda i: fn(*[t[i:i + 1].contiguous() for t in tensors], *args), idx))
    return torch.cat(outs)


def assert_batch_equals_images(fn, tensors, what, images=None):
    """fn(batch)[i] == fn(image i), bit for bit."""
    full = fn(*tensors)
    B = tensors[0].shape[0]
    for i in (range(B) if images is None else images):
        one = fn(*[t[i:i + 1] for t in tensors])
        assert torch.equal(full[i:i + 1], one), f'{what}: image {i} differs between batch and single call'
    return full


# bounds on the literal comparison of a re-ordered fp32 sum with the reference-order result
LITERAL_BAR_MAX_FRACTION = 0.02


def assert_no_worse_than_reference_order(got, ref32, exact, what):
    """`got` (fp32 sums in another order) against the exact (double) result,
    next to the reference-order fp32 result `ref32` against the same: its RMS
    error is not larger, no more of its elements lie outside the fp32 bar
    1e-6 + 1e-5 |b|, and its largest error is not larger (the maximum over 1e7
    elements of two independent rounding errors is a noisy statistic: 25 %
    slack on that one, 1 % on the other two).

    The literal comparison is stated too: how many elements of `got` lie
    outside 1e-6 + 1e-5 |b| of the reference-order fp32 result itself.  Two
    fp32 orders of one sum differ by their rounding errors, which that bar
    (one fp32 spacing near 0.1) does not absorb where terms cancel, so the
    count is not zero for either order against the other; it is printed and
    held below LITERAL_BAR_MAX_FRACTION of the elements (the largest
    difference is printed too; it is bounded by the two errors against the
    exact result, which are held above)."""
    got, ref32, exact = got.double().cpu(), ref32.double().cpu(), exact.double().cpu()
    e_got, e_ref = (got - exact).abs(), (ref32 - exact).abs()
    bar = F32_ATOL + F32_RTOL * exact.abs()
    e_lit = (got - ref32).abs()
    st = dict(rms=e_got.square().mean().sqrt().item(), rms_ref=e_ref.square().mean().sqrt().item(),
              max=e_got.max().item(), max_ref=e_ref.max().item(),
              outside=int((e_got > bar).sum()), outside_ref=int((e_ref > bar).sum()), n=exact.numel(),
              literal_outside=int((e_lit > F32_ATOL + F32_RTOL * ref32.abs()).sum()),
              literal_max=e_lit.max().item())
    print(what, ' '.join(f'{k}={v:.3e}' if isinstance(v, float) else f'{k}={v}' for k, v in st.items()))
    # (1 % slack on the two averages: where both orders are equally good -- SAPA-D,
    # whose error is the fp32 rounding of the sample coordinates in either order --
    # they differ by sampling noise only)
    assert st['rms'] <= 1.01 * st['rms_ref'], f"{what}: rms error {st['rms']:.3e} > reference order {st['rms_ref']:.3e}"
    assert st['outside'] <= 1.01 * st['outside_ref'] + 10, \
        f"{what}: {st['outside']} elements outside the fp32 bar, reference order {st['outside_ref']}"
    assert st['max'] <= 1.25 * st['max_ref'], \
        f"{what}: max error {st['max']:.3e} > 1.25 x reference order {st['max_ref']:.3e}"
    assert st['literal_outside'] <= LITERAL_BAR_MAX_FRACTION * st['n'], \
        f"{what}: {st['literal_outside']} of {st['n']} elements outside 1e-6 + 1e-5 |b| of the reference-order result"
    return st


# ---------------------------------------------------------------- c3: FPN levels

C3_LEVELS = [(25, 42), (50, 84), (100, 168)]


def c3_inputs(B, H, W, seed):
    g = gen(seed)
    scale = torch.rand(64, generator=g) * 1.5 + 0.5
    q = randn(g, B, 64, 2 * H, 2 * W)
    key = randn(g, B, 64, H, W) * scale[None, :, None, None]
    v = randn(g, B, 256, H, W)
    return q, key, v


@pytest.mark.parametrize('H,W', C3_LEVELS)
def test_c3_fpn_fp32_against_oracle(coracle, H, W):
    q, key, v = c3_inputs(2, H, W, 300 + H)
    ref32 = per_image(coracle.sapa_fused, (q, key, v), 5, 2, 'f32')
    exact = per_image(coracle.sapa_fused, (q, key, v), 5, 2, 'f32a64')
    got = sapa_amd.sapa_fused(*dev(q, key, v), 5, 2).cpu()
    assert_f32_close(got, ref32, f'c3 {H}x{W} fp32 contiguous')
    got_cl = sapa_amd.sapa_fused(*as_cl(*dev(q, key, v)), 5, 2)
    assert got_cl.is_contiguous(memory_format=CL)
    assert_no_worse_than_reference_order(got_cl, ref32, exact, f'c3 {H}x{W} fp32 channels_last')
    # the separate operators at this shape: reference arithmetic bit for bit
    logits = sapa_amd.qk(*dev(q[:1], key[:1]), 5, 2)
    assert torch.equal(logits.cpu(), coracle.qk(q[:1], key[:1], 5, 2, 'f32'))
    attn = torch.softmax(logits, 1)
    assert torch.equal(sapa_amd.av(attn, v[:1].to(DEV), 5, 2).cpu(), coracle.av(attn.cpu(), v[:1], 5, 2, 'f32'))


@pytest.mark.parametrize('dtype,rel', [(torch.bfloat16, BF16_REL), (torch.float16, 2e-3)])
@pytest.mark.parametrize('H,W', C3_LEVELS)
def test_c3_fpn_16bit_against_oracle(coracle, H, W, dtype, rel):
    """Inputs rounded to the 16-bit type, the oracle with double sums on those
    values: the kernels keep every intermediate in fp32, so only the rounding of
    the result (at most 2^-8 relative for bf16) is left of the bar."""
    q, key, v = (t.to(dtype) for t in c3_inputs(2, H, W, 300 + H))
    exact = per_image(coracle.sapa_fused, (q.float(), key.float(), v.float()), 5, 2, 'f32a64')
    got = sapa_amd.sapa_fused(*dev(q, key, v), 5, 2)
    assert got.dtype == dtype
    assert_rel_rms_close(got.float(), exact, rel, f'c3 {H}x{W} {dtype} contiguous')
    got_cl = sapa_amd.sapa_fused(*as_cl(*dev(q, key, v)), 5, 2)
    assert got_cl.is_contiguous(memory_format=CL)
    assert_rel_rms_close(got_cl.float(), exact, rel, f'c3 {H}x{W} {dtype} channels_last')
    # the rounding of the result is all that is left: at most half the 16-bit
    # spacing at the exact value (2^-8 resp. 2^-11 of it) plus fp32 noise
    half_ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
    for name, o in (('contiguous', got), ('channels_last', got_cl)):
        err = (o.float().cpu().double() - exact).abs()
        rms = exact.square().mean().sqrt()
        worst = (err / torch.maximum(exact.abs(), rms)).max().item()
        assert worst <= 1.05 * half_ulp, f'c3 {H}x{W} {dtype} {name}: {worst / half_ulp:.2f} half-ulps'


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('layout', ['contiguous', 'channels_last'])
def test_c3_full_batch_properties(layout, dtype):
    """B = 16 at the largest level."""
    H, W = 100, 168
    q, key, v = (t.to(dtype) for t in c3_inputs(16, H, W, 333))
    conv = (lambda *ts: as_cl(*dev(*ts))) if layout == 'channels_last' else dev
    qd, kd, vd = conv(q, key, v)
    fused = lambda a, b, c: sapa_amd.sapa_fused(a, b, c, 5, 2)
    out = assert_batch_equals_images(fused, (qd, kd, vd), f'c3 fused {layout} {dtype}', images=(0, 7, 15))
    assert torch.isfinite(out).all()
    # zero query: uniform weights, the result is the 5x5 box filter of the value
    # (zero padding counted in the mean), nearest-upsampled
    box = F.interpolate(F.avg_pool2d(vd.float().contiguous(), 5, 1, 2, count_include_pad=True), scale_factor=2)
    got0 = fused(torch.zeros_like(qd), kd, vd).float()
    if dtype == torch.float32:
        assert_f32_close(got0, box, f'c3 box filter {layout}')
    else:
        assert_rel_rms_close(got0, box, BF16_REL, f'c3 box filter {layout} bf16')


@pytest.mark.parametrize('layout', ['contiguous', 'channels_last'])
def test_c3_full_batch_integer_inputs_exact(layout):
    """Integer-valued tensors make every product and sum exact in fp32 whatever
    the order: qk and av over the whole batch equal the unfold + einsum
    restatement (sapa/sapa/forward_check.py:9-24) bit for bit."""
    B, H, W, K, s = 16, 100, 168, 5, 2
    g = gen(334)
    ri = lambda *shape: torch.randint(-3, 4, shape, generator=g).float()
    q, key, v = ri(B, 64, s * H, s * W), ri(B, 64, H, W), ri(B, 256, H, W)
    attn = torch.randint(0, 3, (B, K * K, s * H, s * W), generator=g).float()
    conv = (lambda *ts: as_cl(*dev(*ts))) if layout == 'channels_last' else dev
    qd, kd, vd, ad = conv(q, key, v, attn)
    logits = sapa_amd.qk(qd, kd, K, s)
    out = sapa_amd.av(ad, vd, K, s)
    for i in range(0, B, 4):    # the restatement in slices of 4 images (unfold of v: 1.7 GB each)
        sl = slice(i, i + 4)
        ku = F.unfold(kd[sl].contiguous(), K, padding=K // 2).view(4, 64, K * K, H, W)
        want = torch.einsum('bckhw,bchiwj->bkhiwj', ku, qd[sl].contiguous().view(4, 64, H, s, W, s))
        assert torch.equal(logits[sl].contiguous(), want.reshape(4, K * K, s * H, s * W))
        vu = F.unfold(vd[sl].contiguous(), K, padding=K // 2).view(4, 256, K * K, H, W)
        want = torch.einsum('bckhw,bkhiwj->bchiwj', vu, ad[sl].contiguous().view(4, K * K, H, s, W, s))
        assert torch.equal(out[sl].contiguous(), want.reshape(4, 256, s * H, s * W))


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('H,W', C3_LEVELS)
def test_c3_lowres_gradients_integer_inputs_exact(H, W, dtype):
    """grad_value and grad_key at the FPN levels' own sizes (C = 256 / d = 64, four
    images) with small integers in every tensor: products and sums are exact in the
    kernels' fp32 and in the 16-bit result, whatever form, tile geometry and order
    serve the shape, so they must equal the shifted sums of the per-parent products
    (av_cuda_kernel.cu:128-145, qk_cuda_kernel.cu:120-135 written as 25 shifts) bit
    for bit."""
    B, K, s = 4, 5, 2
    g = gen(335)
    r = K // 2
    from sapa_amd import _lib

    def shifted_sums(w, hi):
        C = hi.shape[1]
        w6 = w.double().view(B, K, K, H, s, W, s)
        h6 = hi.double().view(B, C, H, s, W, s)
        want = torch.zeros(B, C, H, W, dtype=torch.float64, device=hi.device)
        for ky in range(K):
            for kx in range(K):
                contrib = torch.einsum('bhiwj,bchiwj->bchw', w6[:, ky, kx], h6)   # per parent
                dy, dx = ky - r, kx - r                                          # cell = parent + (dy, dx)
                ys, xs = slice(max(0, -dy), H - max(0, dy)), slice(max(0, -dx), W - max(0, dx))
                yd, xd = slice(max(0, dy), H + min(0, dy)), slice(max(0, dx), W + min(0, dx))
                want[:, :, yd, xd] += contrib[:, :, ys, xs]
        return want

    for C, entry in ((256, 'sapa_av_backward'), (64, 'sapa_qk_backward')):
        w = torch.randint(-2, 3, (B, K * K, s * H, s * W), generator=g).float().to(DEV)
        hi = torch.randint(-2, 3, (B, C, s * H, s * W), generator=g).float().to(DEV)
        want = shifted_sums(w, hi)
        assert want.abs().max() < 256          # exact in bf16 as well
        wd, hid = w.to(dtype), hi.to(dtype)
        low = torch.zeros(B, C, H, W, device=DEV, dtype=dtype)
        out = torch.full_like(low, 9.0)
        if entry == 'sapa_av_backward':     # (grad_out, attn, value, grad_attn, grad_value)
            _lib.call(entry, low.device, _lib.ptr(hid), _lib.ptr(wd), _lib.ptr(low), None, _lib.ptr(out),
                      B, C, H, W, K, s, _lib.DTYPES[dtype])
        else:                               # (grad_logits, query, key, grad_query, grad_key)
            _lib.call(entry, low.device, _lib.ptr(wd), _lib.ptr(hid), _lib.ptr(low), None, _lib.ptr(out),
                      B, C, H, W, K, s, _lib.DTYPES[dtype])
        assert torch.equal(out.double(), want), f'{entry} {H}x{W} {dtype}'


@pytest.mark.parametrize('H,W', C3_LEVELS)
def test_c3_fused_backward_against_oracle(coracle, H, W):
    """One image of each FPN level through sapa_fused(...).backward(): all
    three gradients against the float64 chain of the reference's backward functions on
    the same values; the full batch of the level equals its images bit for bit (the
    kernels have no atomics).  Bar: |a - b| <= 1e-4 max(|b|, rms(b)) -- fp32 sums of up
    to 6400 products against double sums."""
    q, key, v = c3_inputs(4, H, W, 336)
    go = randn(gen(337), 4, 256, 2 * H, 2 * W)

    def grads(qi, ki, vi, gi):
        ts = [t.clone().requires_grad_() for t in (qi, ki, vi)]
        sapa_amd.sapa_fused(*ts, 5, 2).backward(gi)
        return [t.grad for t in ts]

    qd, kd, vd, god = dev(q, key, v, go)
    full = grads(qd, kd, vd, god)
    for i in (0, 3):
        one = grads(qd[i:i + 1], kd[i:i + 1], vd[i:i + 1], god[i:i + 1])
        for name, a, b in zip(('grad_query', 'grad_key', 'grad_value'), full, one):
            assert torch.equal(a[i:i + 1], b), f'{name}: image {i} differs between batch and single call'
    want = fused_backward_oracle(coracle, go[:1], q[:1], key[:1], v[:1], 5, 2)
    for name, a, b in zip(('grad_query', 'grad_key', 'grad_value'), full, want):
        assert_rel_rms_close(a[:1].cpu().double(), b, 1e-4, f'c3 {H}x{W} {name}')


# ---------------------------------------------------------------- c2: SegFormer-style chain

def test_c2_segformer_chain_module_and_operators(coracle):
    """Three stages 16^2 -> 32^2 -> 64^2 -> 128^2; each stage's output is the next
    stage's low-res feature; SAPA(256, embedding_dim=32) with GroupNorm(32) and
    1x1 projections ~N(0, .02) (sapa_base.py:17-22,42-46)."""
    B = 8
    torch.manual_seed(2)
    g = gen(200)
    stages = [sapa_amd.SAPA(256, embedding_dim=32).to(DEV) for _ in range(3)]
    x = randn(g, B, 256, 16, 16).to(DEV)
    with torch.no_grad():
        for m, h in zip(stages, (16, 32, 64)):
            y = randn(g, B, 256, 2 * h, 2 * h).to(DEV)
            out = m(y, x)
            assert out.shape == (B, 256, 2 * h, 2 * h)
            q, k = m.q(m.norm_y(y)), m.k(m.norm_x(x))
            # raw operators, fused and the reference's three steps (sapa_base.py:38-40)
            fused = lambda a, b, c: sapa_amd.sapa_fused(a, b, c, 5, 2)
            raw = assert_batch_equals_images(fused, (q, k, x), f'c2 {h} fused')
            assert torch.equal(raw, out)
            three = sapa_amd.av(F.softmax(sapa_amd.qk(q, k, 5, 2), dim=1), x, 5, 2)
            want = per_image(coracle.sapa_fused, (q.cpu(), k.cpu(), x.cpu()), 5, 2, 'f32', images=(0, B - 1))
            for got, name in ((out, 'module'), (three, 'three-step')):
                assert_f32_close(got[[0, B - 1]].cpu(), want, f'c2 {h}->{2 * h} {name}')
            # the module's other forward routes on the same features
            m.fold_norm = True
            torch.testing.assert_close(m(y, x), out, rtol=1e-4, atol=1e-5)
            m.fold_norm, m.channels_last = False, True
            out_cl = m(*as_cl(y, x))
            assert out_cl.is_contiguous(memory_format=CL)
            torch.testing.assert_close(out_cl.contiguous(), out, rtol=1e-4, atol=1e-5)
            m.channels_last = False
            # channels_last operator on the same projections: within the fp32 bar of the oracle
            got_cl = sapa_amd.sapa_fused(*as_cl(q, k, x), 5, 2)
            assert_f32_close(got_cl[[0, B - 1]].cpu(), want, f'c2 {h}->{2 * h} channels_last')
            x = out


@pytest.mark.parametrize('h', [16, 32, 64])
def test_c2_segformer_stage_backward(coracle, h):
    """One stage of the chain at its own size (B = 8, C = 256, d = 32, projections
    ~N(0, .02) of GroupNorm-ed features): the gradients of the fused operator for query,
    key and value -- batch equal to its images bit for bit, image 0 against the float64
    chain of the reference's backward functions, |a - b| <= 1e-4 max(|b|, rms(b)) --
    with the attention weights kept by the forward pass and recomputed (same bits)."""
    B = 8
    torch.manual_seed(3)
    g = gen(201)
    m = sapa_amd.SAPA(256, embedding_dim=32).to(DEV)
    x, y = randn(g, B, 256, h, h).to(DEV), randn(g, B, 256, 2 * h, 2 * h).to(DEV)
    go = randn(g, B, 256, 2 * h, 2 * h).to(DEV)
    with torch.no_grad():
        q, k = m.q(m.norm_y(y)).contiguous(), m.k(m.norm_x(x)).contiguous()

    def grads(qi, ki, vi, gi, keep=True):
        ts = [t.clone().requires_grad_() for t in (qi, ki, vi)]
        sapa_amd.sapa_fused(*ts, 5, 2, save_attention=keep).backward(gi)
        return [t.grad for t in ts]

    full = grads(q, k, x, go)
    for a, b in zip(full, grads(q, k, x, go, keep=False)):
        assert torch.equal(a, b)
    for i in (0, B - 1):
        one = grads(q[i:i + 1], k[i:i + 1], x[i:i + 1], go[i:i + 1])
        for name, a, b in zip(('grad_query', 'grad_key', 'grad_value'), full, one):
            assert torch.equal(a[i:i + 1], b), f'c2 {h}: {name} of image {i} differs between batch and single call'
    want = fused_backward_oracle(coracle, go[:1].cpu(), q[:1].cpu(), k[:1].cpu(), x[:1].cpu(), 5, 2)
    for name, a, b in zip(('grad_query', 'grad_key', 'grad_value'), full, want):
        assert_rel_rms_close(a[:1].cpu().double(), b, 1e-4, f'c2 {h}->{2 * h} {name}')


# ---------------------------------------------------------------- c4: SAPA-D

def c4_inputs(B, P, seed, G=4):
    g = gen(seed)
    q = randn(g, B, 128, 128, 128)
    key = randn(g, B, 128, 64, 64)
    v = randn(g, B, 256, 64, 64)
    off = (0.75 * randn(g, B, 2 * G * P, 128, 128)).clamp(-4, 4)
    gate = torch.sigmoid(randn(g, B, 1, 1, 128, 128))
    return q, key, v, off, gate


@pytest.mark.parametrize('P', [25, 9, 5])
def test_c4_deform_against_oracle(coracle, P):
    """B = 8, G = 4, d = 32 per group, C = 256, 64^2 -> 128^2.  The sigmoid gate
    of the benchmark description has no counterpart in sapa_deform.py: it is
    input conditioning, applied to the logits in the same way on both sides
    (separate operators); the fused operator is compared without it."""
    B, s, G = 8, 2, 4
    q, key, v, off, gate = c4_inputs(B, P, 400 + P)
    qd, kd, vd, od, gd = dev(q, key, v, off, gate)
    imgs = (0, B - 1)
    sub = lambda *ts: [t[list(imgs)] for t in ts]
    # separate operators: bit for bit the reference arithmetic
    logits = sapa_amd.deform_qk(qd, kd, od, P, s, G)
    want_logits = per_image(coracle.deform_qk, sub(q, key, off), P, s, G, 'f32')
    assert torch.equal(logits[list(imgs)].cpu(), want_logits)
    attn = torch.softmax(logits * gd, dim=2)
    want_attn = torch.softmax(want_logits * gate[list(imgs)], dim=2)
    torch.testing.assert_close(attn[list(imgs)].cpu(), want_attn, rtol=1e-5, atol=1e-7)
    out = sapa_amd.deform_av(attn, vd, od, P, s, G)
    want = per_image(coracle.deform_av, [attn[list(imgs)].cpu()] + sub(v, off), P, s, G, 'f32')
    assert torch.equal(out[list(imgs)].cpu(), want)
    # fused, both memory orders
    fused = lambda a, b, c, o: sapa_amd.deform_sapa_fused(a, b, c, o, P, s, G)
    fused_r = lambda a, b, c, o: sapa_amd.deform_sapa_fused(a, b, c, o, P, s, G, matrix_form=False)
    got = assert_batch_equals_images(fused_r, (qd, kd, vd, od), f'c4 P={P} fused', images=(0, 3, B - 1))
    want_f = per_image(coracle.deform_sapa_fused, sub(q, key, v, off), P, s, G, 'f32')
    assert_f32_close(got[list(imgs)].cpu(), want_f, f'c4 P={P} fused, reference order')
    got_cl = assert_batch_equals_images(fused, as_cl(qd, kd, vd, od), f'c4 P={P} fused channels_last',
                                        images=(0, 3, B - 1))
    exact = per_image(coracle.deform_sapa_fused, [t.double() for t in sub(q, key, v, off)], P, s, G, 'f64')
    assert_no_worse_than_reference_order(got_cl[list(imgs)], want_f, exact, f'c4 P={P} fused channels_last')
    # contiguous tensors, the default route: the matrix-form kernel from 13 points on (key and
    # value via a workspace), the reference's order of sums below
    got_m = assert_batch_equals_images(fused, (qd, kd, vd, od), f'c4 P={P} fused default', images=(0, 3, B - 1))
    assert got_m.is_contiguous()
    if P >= 13:
        from sapa_amd import _lib
        assert _lib.last_kernel() == 'deform_fused_wmat_kernel'
        assert_no_worse_than_reference_order(got_m[list(imgs)], want_f, exact, f'c4 P={P} fused matrix form')
    else:
        assert torch.equal(got_m, got)
    # 16-bit tensors, contiguous and channels_last
    hq, hk, hv, ho = (t.to(torch.bfloat16) for t in (qd, kd, vd, od))
    exact16 = per_image(coracle.deform_sapa_fused, [t[list(imgs)].double().cpu() for t in (hq, hk, hv, ho)],
                        P, s, G, 'f64')
    assert_rel_rms_close(fused(hq, hk, hv, ho)[list(imgs)].float(), exact16, BF16_REL, f'c4 P={P} bf16')
    assert_rel_rms_close(fused(*as_cl(hq, hk, hv, ho))[list(imgs)].float(), exact16, BF16_REL,
                         f'c4 P={P} bf16 channels_last')


@pytest.mark.parametrize('dtype,P', [(torch.float32, 25), (torch.float32, 9), (torch.bfloat16, 25)])
def test_c4_deform_backward_against_oracle(coracle, dtype, P):
    """The training step of config 4 at its own sizes: the gradients of
    sum(out * grad_out) through deform_sapa_fused (one sapa_deform_fused_backward call:
    the matrix-form kernel for the per-pixel part, the matrix-product scatter for the
    low-res gradients) against the float64 oracle chain on two images, and the whole
    batch against the same call image by image -- bit for bit where no atomics are
    involved (grad_query, grad_offset), to fp32 rounding where the order of the sums
    varies (grad_key, grad_value)."""
    B, s, G = 8, 2, 4
    q, key, v, off, _ = c4_inputs(B, P, 450 + P)
    frac = off - off.floor()
    off = off.floor() + frac.clamp(0.2, 0.8)        # 16-bit rounding must not cross a bilinear kink
    go = randn(gen(460 + P), B, 256, 128, 128)
    q, key, v, off, go = (t.to(dtype) for t in (q, key, v, off, go))

    def grads(*ts):
        leaves = [t.clone().requires_grad_() for t in ts[:4]]
        sapa_amd.deform_sapa_fused(*leaves, P, s, G).backward(ts[4])
        return [t.grad for t in leaves]

    def grads_separate(*ts):
        leaves = [t.clone().requires_grad_() for t in ts[:4]]
        a, b, c, o = leaves
        attn = torch.softmax(sapa_amd.deform_qk(a, b, o, P, s, G), dim=2)
        sapa_amd.deform_av(attn, c, o, P, s, G).backward(ts[4])
        return [t.grad for t in leaves]

    full = grads(*dev(q, key, v, off, go))
    names = ('grad_query', 'grad_key', 'grad_value', 'grad_offset')
    for n in (0, B - 1):
        one = grads(*dev(*(t[n:n + 1] for t in (q, key, v, off, go))))
        for name, a, b in zip(names, full, one):
            if name in ('grad_query', 'grad_offset'):
                assert torch.equal(a[n:n + 1], b), f'{name}: image {n} of the batch differs from the image alone'
            else:
                torch.testing.assert_close(a[n:n + 1].float(), b.float(), msg=lambda m: f'{name} image {n}: {m}',
                                           rtol=1e-5 if dtype == torch.float32 else 2.0 ** -7, atol=1e-5)
        want = deform_fused_backward_oracle(coracle, *(t[n:n + 1].float() for t in (go, q, key, v, off)), P, s, G)
        if dtype == torch.float32:
            # fp32: sums per window cell instead of per point and channel -- no further
            # from the double-precision result than the chain of the separate operators,
            # whose kernels keep the reference's order
            ref = grads_separate(*dev(*(t[n:n + 1] for t in (q, key, v, off, go))))
            for name, got, r, w in zip(names, full, ref, want):
                assert_no_worse_than_reference_order(got[n:n + 1], r, w, f'c4 backward P={P} {name} image {n}')
        else:
            for name, got, w in zip(names, full, want):
                assert_rel_rms_close(got[n:n + 1].float().cpu().double(), w, 1.5e-2,
                                     f'c4 backward P={P} bf16 {name} image {n}')


def test_c4_regular_grid_offsets_reduce_to_sapa_b():
    """P = 25 regular-grid integer offsets, G = 1: SAPA-D is SAPA-B with K = 5,
    at the full c4 extent (cross-check between the two operator families)."""
    B, d, C, H, W, K, s = 8, 32, 256, 64, 64, 5, 2
    g = gen(440)
    q, key, v = randn(g, B, d, s * H, s * W), randn(g, B, d, H, W), randn(g, B, C, H, W)
    off = torch.empty(B, 2 * K * K, s * H, s * W)
    for ky in range(K):
        for kx in range(K):
            off[:, 2 * (ky * K + kx)] = kx - K // 2         # width offset first
            off[:, 2 * (ky * K + kx) + 1] = ky - K // 2
    qd, kd, vd, od = dev(q, key, v, off)
    assert torch.equal(sapa_amd.deform_qk(qd, kd, od, K * K, s, 1).squeeze(1), sapa_amd.qk(qd, kd, K, s))
    want = sapa_amd.sapa_fused(qd, kd, vd, K, s)
    assert_f32_close(sapa_amd.deform_sapa_fused(qd, kd, vd, od, K * K, s, 1, matrix_form=False), want,
                     'regular grid, contiguous, reference order')
    exact = sapa_amd.sapa_fused(qd.double(), kd.double(), vd.double(), K, s)
    assert_no_worse_than_reference_order(sapa_amd.deform_sapa_fused(qd, kd, vd, od, K * K, s, 1), want, exact,
                                         'regular grid, contiguous, matrix form')
    assert_no_worse_than_reference_order(sapa_amd.deform_sapa_fused(*as_cl(qd, kd, vd, od), K * K, s, 1), want,
                                         exact, 'regular grid, channels_last')


# ---------------------------------------------------------------- c5: stress

def c5_inputs(B, seed):
    g = gen(seed)
    q = randn(g, B, 64, 256, 256)
    heavy = torch.rand(q.shape, generator=g) < 0.1
    # Student-t(3) = normal / sqrt(chi2_3 / 3), drawn from the seeded generator
    t3 = randn(g, *q.shape) / (randn(g, 3, *q.shape).square().sum(0) / 3).sqrt()
    q = torch.where(heavy, t3, q)
    key = randn(g, B, 64, 64, 64)
    v = randn(g, B, 512, 64, 64)
    return q, key, v


def test_c5_stress_bf16_against_oracle(coracle):
    """B = 4, C = 512, d = 64, K = 7, s = 4, 64^2 -> 256^2, bf16, heavy-tailed query."""
    B, K, s = 4, 7, 4
    q, key, v = (t.to(torch.bfloat16) for t in c5_inputs(B, 500))
    qd, kd, vd = dev(q, key, v)
    fused = lambda a, b, c: sapa_amd.sapa_fused(a, b, c, K, s)
    got = assert_batch_equals_images(fused, (qd, kd, vd), 'c5 contiguous')
    got_cl = assert_batch_equals_images(fused, as_cl(qd, kd, vd), 'c5 channels_last')
    exact = per_image(coracle.sapa_fused, (q.float(), key.float(), v.float()), K, s, 'f32a64', images=(0, B - 1))
    assert_rel_rms_close(got[[0, B - 1]].float(), exact, BF16_REL, 'c5 bf16 contiguous')
    assert_rel_rms_close(got_cl[[0, B - 1]].float(), exact, BF16_REL, 'c5 bf16 channels_last')
    # fp32 at the same extent, one image: the reference-order bar
    q32, k32, v32 = q[:1].float(), key[:1].float(), v[:1].float()
    want = coracle.sapa_fused(q32, k32, v32, K, s, 'f32')
    assert_f32_close(sapa_amd.sapa_fused(*dev(q32, k32, v32), K, s).cpu(), want, 'c5 fp32 contiguous')
    exact1 = exact[:1]
    assert_no_worse_than_reference_order(sapa_amd.sapa_fused(*as_cl(*dev(q32, k32, v32)), K, s), want, exact1,
                                         'c5 fp32 channels_last')
