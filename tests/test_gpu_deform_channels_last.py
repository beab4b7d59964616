"""GPU parity of the fused SAPA-D forward on tensors in torch.channels_last
order (sapa_deform_fused_forward_nhwc) against the CPU oracle and against the
library's contiguous path.

The oracle runs the reference kernels' fp32 arithmetic (same index math, same
guard).  The logits' channel sums run in tree order here, so the comparison
uses the reference's own check tolerance, allclose(atol=1e-5)
(deformsapa/deformsapa/forward_check.py), tightened to 1e-5 rel / 1e-6 abs for
short sums; 16-bit within the usual relative bars.
"""
import pytest
import torch

import sapa_amd
from helpers import BF16_REL, F16_REL, assert_f32_close, assert_rel_rms_close, gen, randn

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'
CL = torch.channels_last

# B, G, d (q/k channels per group), cg (value channels per group), H, W, P, s, offset scale
SHAPES = [(2, 2, 4, 8, 5, 7, 9, 2, 1.0), (1, 4, 32, 64, 8, 8, 25, 2, 0.75), (1, 1, 64, 72, 6, 5, 4, 2, 1.5),
          (1, 2, 8, 132, 4, 6, 16, 1, 1.0), (2, 3, 4, 4, 3, 5, 17, 4, 1.0), (1, 2, 8, 8, 9, 9, 32, 2, 1.0),
          (1, 1, 4, 4, 1, 1, 1, 2, 1.0),
          # offsets far beyond the +-4 cells of the LDS window: the global-memory path
          (1, 2, 8, 12, 14, 13, 7, 2, 6.0), (1, 2, 8, 12, 14, 13, 9, 2, 6.0),
          # more than 7 points take the matrix formulation: the same far offsets; 64 and 48
          # query / key channels per group (the padded instance), a ragged second value
          # chunk (72 = 64 + 8) and a short single one (20); s = 4 and s = 1 with part of
          # the samples outside the window; odd extents
          (1, 2, 8, 12, 14, 13, 16, 2, 6.0), (1, 1, 64, 72, 6, 5, 20, 2, 1.5), (1, 2, 48, 20, 7, 9, 13, 4, 2.5),
          (2, 1, 12, 36, 11, 6, 29, 1, 3.0),
          # channels per group in whole 16-byte pieces: 16-bit tensors take the 16-bit matrix
          # instructions -- far offsets with 16 lanes per pixel, 48 channels padded to 64 at
          # s = 4, s = 1, the full 32 points over three groups, three value chunks (64 + 64 + 8)
          (1, 2, 8, 16, 14, 13, 16, 2, 6.0), (1, 2, 48, 24, 7, 9, 13, 4, 2.5), (2, 1, 16, 40, 11, 6, 29, 1, 3.0),
          (2, 3, 24, 8, 9, 11, 32, 2, 1.0), (1, 1, 64, 136, 5, 7, 21, 2, 1.5)]
IDS = ['-'.join(map(str, s)) for s in SHAPES]


def cl(*ts):
    return [t.to(DEV).contiguous(memory_format=CL) for t in ts]


def inputs(g, B, G, d, cg, H, W, P, s, oscale, dtype=torch.float32):
    q = randn(g, B, G * d, s * H, s * W).to(dtype)
    key = randn(g, B, G * d, H, W).to(dtype)
    v = randn(g, B, G * cg, H, W).to(dtype)
    off = (randn(g, B, 2 * G * P, s * H, s * W) * oscale).to(dtype)
    return q, key, v, off


@pytest.mark.parametrize('shape', SHAPES, ids=IDS)
def test_fp32_vs_oracle(coracle, shape):
    B, G, d, cg, H, W, P, s, _ = shape
    q, key, v, off = inputs(gen(500), *shape)
    got = sapa_amd.deform_sapa_fused(*cl(q, key, v, off), P, s, G)
    assert got.is_contiguous(memory_format=CL) and got.shape == (B, G * cg, s * H, s * W)
    want = coracle.deform_sapa_fused(q, key, v, off, P, s, G, 'f32')
    if d <= 8:
        assert_f32_close(got, want, 'fused')
    else:
        torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize('dtype,rel', [(torch.bfloat16, BF16_REL), (torch.float16, F16_REL)])
@pytest.mark.parametrize('shape', SHAPES[:4] + SHAPES[7:], ids=IDS[:4] + IDS[7:])  # incl. the matrix-formulation shapes
def test_16bit_vs_oracle(coracle, shape, dtype, rel):
    B, G, d, cg, H, W, P, s, _ = shape
    q, key, v, off = inputs(gen(501), *shape, dtype=dtype)
    got = sapa_amd.deform_sapa_fused(*cl(q, key, v, off), P, s, G)
    assert got.dtype == dtype and got.is_contiguous(memory_format=CL)
    want = coracle.deform_sapa_fused(q.float(), key.float(), v.float(), off.float(), P, s, G, 'f32')
    assert_rel_rms_close(got.float(), want, rel, 'fused')


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('layout', ['contiguous', 'channels_last'])
def test_matrix_form_carries_non_finite_logits(coracle, layout, dtype):
    """A NaN or +inf in the query makes the logits of that pixel and group
    non-finite; softmax then gives NaN for every point and the reference's
    attn * val (deform_av_cuda_kernel.cu:185-190) puts NaN into every channel
    of the group at that pixel.  The matrix form builds its weight matrix from
    integers, which cannot carry a NaN: such pixels take the per-sample path."""
    B, G, d, cg, H, W, P, s = 2, 2, 8, 16, 9, 11, 16, 2
    q, key, v, off = inputs(gen(503), B, G, d, cg, H, W, P, s, 1.0, dtype=dtype)
    q[0, 3, 5, 7] = float('nan')            # group 0
    q[1, d + 2, 10, 3] = float('inf')       # group 1
    q[1, 1, 0, 0] = float('inf')            # a corner pixel: part of its samples fail the guard
    want = coracle.deform_sapa_fused(q.float(), key.float(), v.float(), off.float(), P, s, G, 'f32')
    bad = ~torch.isfinite(want)
    assert bad.any() and bad.sum() <= 3 * cg, 'whole groups of three pixels at most'
    args = cl(q, key, v, off) if layout == 'channels_last' else [t.to(DEV) for t in (q, key, v, off)]
    got = sapa_amd.deform_sapa_fused(*args, P, s, G, matrix_form=True).float().cpu()
    assert torch.equal(torch.isnan(got), torch.isnan(want))
    fin = ~bad
    if dtype == torch.float32:
        torch.testing.assert_close(got[fin], want[fin], rtol=1e-5, atol=1e-5)
    else:
        assert_rel_rms_close(torch.where(fin, got, 0), torch.where(fin, want, 0), BF16_REL, 'finite part')


def test_matches_contiguous_path_at_a_larger_shape():
    B, G, d, cg, H, W, P, s = 2, 4, 32, 64, 19, 22, 25, 2
    q, key, v, off = inputs(gen(502), B, G, d, cg, H, W, P, s, 0.75)
    off = off.clamp(-4, 4)
    want = sapa_amd.deform_sapa_fused(*(t.to(DEV) for t in (q, key, v, off)), P, s, G)
    got = sapa_amd.deform_sapa_fused(*cl(q, key, v, off), P, s, G)
    torch.testing.assert_close(got.contiguous(), want, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize('P', [5, 9, 17])   # the gather kernel / the matrix formulation (16 and 32 lanes per pixel)
def test_guard_failures_and_image_border(P):
    """Offsets that push most points out of the image: those points keep logit
    0, take part in the softmax and contribute nothing."""
    B, G, d, cg, H, W, s = 1, 2, 4, 8, 6, 7, 2
    g = gen(503)
    q, key, v, off = inputs(g, B, G, d, cg, H, W, P, s, 1.0)
    off = off + 5.0 * torch.sign(randn(g, *off.shape))      # +-5 cells: in or out of a 6x7 image
    want_shape = (B, G * cg, s * H, s * W)
    got = sapa_amd.deform_sapa_fused(*cl(q, key, v, off), P, s, G)
    assert got.shape == want_shape
    want = sapa_amd.deform_sapa_fused(*(t.to(DEV) for t in (q, key, v, off)), P, s, G)
    torch.testing.assert_close(got.contiguous(), want, rtol=1e-5, atol=1e-6)
    # every point outside: uniform weights over nothing -> exact zeros
    off_far = torch.full_like(off, 100.0)
    got = sapa_amd.deform_sapa_fused(*cl(q, key, v, off_far), P, s, G)
    assert torch.count_nonzero(got) == 0


@pytest.mark.parametrize('dtype,rel', [(torch.bfloat16, BF16_REL), (torch.float16, F16_REL)])
def test_guard_failures_on_the_16bit_matrix_kernel(coracle, dtype, rel):
    """The same border case where 16-bit tensors take the 16-bit matrix
    instructions (8 channels per group, 17 points), and the name of the
    kernel that ran."""
    from sapa_amd import _lib
    B, G, d, cg, H, W, P, s = 1, 2, 8, 8, 6, 7, 17, 2
    g = gen(505)
    q, key, v, off = inputs(g, B, G, d, cg, H, W, P, s, 1.0, dtype=dtype)
    off = (off.float() + 5.0 * torch.sign(randn(g, *off.shape))).to(dtype)
    got = sapa_amd.deform_sapa_fused(*cl(q, key, v, off), P, s, G)
    assert _lib.last_kernel() == 'deform_fused_wmat16_kernel'
    want = coracle.deform_sapa_fused(q.float(), key.float(), v.float(), off.float(), P, s, G, 'f32')
    assert_rel_rms_close(got.float(), want, rel, 'fused')
    got = sapa_amd.deform_sapa_fused(*cl(q, key, v, torch.full_like(off, 100.0)), P, s, G)
    assert torch.count_nonzero(got) == 0
    # groups that are not whole 16-byte pieces stay on the kernel for any channel count
    q, key, v, off = inputs(g, B, G, 4, 12, H, W, P, s, 1.0, dtype=dtype)
    sapa_amd.deform_sapa_fused(*cl(q, key, v, off), P, s, G)
    assert _lib.last_kernel() == 'deform_fused_wmat_kernel'


def test_layout_errors_and_backward():
    B, G, d, cg, H, W, P, s = 1, 2, 4, 8, 5, 6, 9, 2
    q, key, v, off = inputs(gen(504), B, G, d, cg, H, W, P, s, 1.0)
    qc, kc, vc, oc = cl(q, key, v, off)
    with pytest.raises(RuntimeError, match='contiguous'):
        sapa_amd.deform_sapa_fused(qc, kc, vc, off.to(DEV), P, s, G)          # mixed orders
    q6 = randn(gen(505), B, G * 3, s * H, s * W)
    k6 = randn(gen(506), B, G * 3, H, W)
    with pytest.raises(RuntimeError, match='channels_last'):
        sapa_amd.deform_sapa_fused(*cl(q6, k6, v, off), P, s, G)              # 3 channels per group
    q68, k68 = randn(gen(508), B, G * 68, s * H, s * W), randn(gen(509), B, G * 68, H, W)
    with pytest.raises(RuntimeError, match='channels_last'):
        sapa_amd.deform_sapa_fused(*cl(q68, k68, v, off), P, s, G)            # 68 channels per group
    grads = []
    go = randn(gen(507), B, G * cg, s * H, s * W)
    for fmt in (torch.contiguous_format, CL):
        ts = [t.to(DEV).contiguous(memory_format=fmt).requires_grad_() for t in (q, key, v, off)]
        out = sapa_amd.deform_sapa_fused(*ts, P, s, G)
        out.backward(go.to(DEV).contiguous(memory_format=fmt))
        grads.append([t.grad for t in ts])
    for a, b, name in zip(grads[0], grads[1], ('query', 'key', 'value', 'offset')):
        torch.testing.assert_close(b, a, rtol=1e-4, atol=1e-5, msg=lambda m: f'grad_{name}: {m}')


def test_module_in_channels_last_format():
    torch.manual_seed(1)
    m = sapa_amd.SAPADeform(64, 64, up_factor=2, num_point=9, groups=4, embedding_dim=32).to(DEV)
    g = gen(510)
    y, x = randn(g, 2, 64, 18, 22).to(DEV), randn(g, 2, 64, 9, 11).to(DEV)
    want = m(y, x)
    mc = m.to(memory_format=CL)
    got = mc(y.contiguous(memory_format=CL), x.contiguous(memory_format=CL))
    assert got.is_contiguous(memory_format=CL)
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-5)
    got.sum().backward()
    assert all(p.grad is not None for p in mc.parameters())


@pytest.mark.parametrize('norm', [False, True])
def test_module_emitting_channels_last(norm):
    """SAPADeform(channels_last=True): projections that write q, k and the
    offsets in channels_last order, the fused operator in that order -- same
    values as the default module on contiguous tensors."""
    import sapa_amd
    torch.manual_seed(8)
    m = sapa_amd.SAPADeform(64, embedding_dim=8, norm=norm).to(DEV)
    torch.nn.init.normal_(m.offset.weight, std=0.1)
    torch.nn.init.normal_(m.q.weight, std=0.2)
    torch.nn.init.normal_(m.k.weight, std=0.2)
    y = torch.randn(2, 64, 18, 22, device=DEV) + 0.5
    x = torch.randn(2, 64, 9, 11, device=DEV)
    with torch.no_grad():
        want = m(y, x)
        m.channels_last = True
        got = m(y, x)
        got_cl_in = m(y.contiguous(memory_format=torch.channels_last),
                      x.contiguous(memory_format=torch.channels_last))
    assert got.shape == want.shape and got.is_contiguous(memory_format=torch.channels_last)
    torch.testing.assert_close(got, want, rtol=2e-4, atol=2e-4)
    torch.testing.assert_close(got_cl_in, want, rtol=2e-4, atol=2e-4)
