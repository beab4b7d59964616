"""GPU: the SAPA / SAPADeform modules beyond the plain forward pass --
parameter gradients with frozen features, configurations that the
channels-last and fused kernels do not cover (the modules fall back, the
operators raise), and non-finite values in the softmax and the sampled
gradients (torch.softmax / the reference's atomicAdd semantics)."""
import pytest
import torch
import torch.nn.functional as F

import sapa_amd
from sapa_amd import _lib
from helpers import gen, randn

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'


def _param_grads(m, y, x):
    m.zero_grad(set_to_none=True)
    out = m(y, x)
    out.float().square().mean().backward()
    return out.detach(), {n: p.grad.detach().clone() for n, p in m.named_parameters()
                          if p.grad is not None}


@pytest.mark.parametrize('kind', ['sapa', 'deform'])
@pytest.mark.parametrize('mode', ['fold_norm', 'channels_last'])
def test_parameters_train_with_frozen_features(kind, mode):
    """Features from a frozen backbone (requires_grad=False) with grad mode on:
    the folded / channels_last forward must still record the graph of
    norm_y / norm_x / q / k / offset (sapa_base.py:26-36 trains them), and the
    gradients must equal the two-step module's."""
    torch.manual_seed(11)
    if kind == 'sapa':
        m = sapa_amd.SAPA(64, embedding_dim=16).to(DEV)
    else:
        m = sapa_amd.SAPADeform(64, embedding_dim=8, norm=True).to(DEV)
        torch.nn.init.normal_(m.offset.weight, std=0.1)
    torch.nn.init.normal_(m.norm_y.weight, 1.0, 0.2)
    torch.nn.init.normal_(m.norm_x.bias, 0.0, 0.2)
    torch.nn.init.normal_(m.q.weight, std=0.2)
    torch.nn.init.normal_(m.k.weight, std=0.2)
    y = torch.randn(2, 64, 16, 24, device=DEV) + 0.3
    x = torch.randn(2, 64, 8, 12, device=DEV)
    assert not x.requires_grad and not y.requires_grad and torch.is_grad_enabled()
    want_out, want = _param_grads(m, y, x)
    assert set(want) == {n for n, _ in m.named_parameters()}
    setattr(m, mode, True)
    got_out, got = _param_grads(m, y, x)
    torch.testing.assert_close(got_out.contiguous(), want_out, rtol=1e-4, atol=1e-4)
    assert set(got) == set(want), f'parameters without a gradient: {set(want) - set(got)}'
    for n in want:
        scale = want[n].abs().max().item()
        assert scale > 0, n
        torch.testing.assert_close(got[n], want[n], rtol=2e-3, atol=2e-4 * scale, msg=lambda s: f'{n}: {s}')


def _two_step(m, y, x):
    """sapa_base.py:26-40 on contiguous tensors with the separate operators."""
    q, k = (m.q(m.norm_y(y)), m.k(m.norm_x(x))) if m.norm else (m.q(y), m.k(x))
    K, s = m.up_kernel_size, m.up_factor
    return sapa_amd.av(F.softmax(sapa_amd.qk(q, k, K, s), dim=1), x, K, s)


@pytest.mark.parametrize('cfg', [
    dict(C=64, K=5, s=2, dtype=torch.float64),      # no float64 channels-last kernel
    dict(C=64, K=5, s=3, dtype=torch.float32),      # up_factor 3
    dict(C=64, K=1, s=2, dtype=torch.float32),      # kernel size 1
    dict(C=66, K=5, s=2, dtype=torch.float32, norm=False),   # channels not a multiple of 4
    dict(C=32, K=13, s=2, dtype=torch.float32),     # K*K > 121: beyond the fused kernels
])
def test_sapa_module_falls_back_where_kernels_do_not_cover(cfg):
    """A default module fed channels_last features works for every
    configuration the contiguous operators serve; the operator itself still
    says what it does not cover."""
    torch.manual_seed(12)
    C, K, s, dt = cfg['C'], cfg['K'], cfg['s'], cfg['dtype']
    m = sapa_amd.SAPA(C, up_factor=s, up_kernel_size=K, embedding_dim=8,
                      norm=cfg.get('norm', True)).to(DEV).to(dt)
    torch.nn.init.normal_(m.q.weight, std=0.3)
    torch.nn.init.normal_(m.k.weight, std=0.3)
    y = torch.randn(2, C, 7 * s, 9 * s, device=DEV, dtype=dt)
    x = torch.randn(2, C, 7, 9, device=DEV, dtype=dt)
    with torch.no_grad():
        want = _two_step(m, y, x)
        got = m(y, x)                                               # contiguous features
        ycl, xcl = (t.contiguous(memory_format=torch.channels_last) for t in (y, x))
        got_cl = m(ycl, xcl)                                        # channels_last features
        m.channels_last = True
        got_cl2 = m(ycl, xcl)
    tol = dict(rtol=1e-9, atol=1e-9) if dt == torch.float64 else dict(rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(got, want, **tol)
    torch.testing.assert_close(got_cl.contiguous(), want, **tol)
    assert got_cl.is_contiguous(memory_format=torch.channels_last)
    torch.testing.assert_close(got_cl2.contiguous(), want, rtol=1e-4, atol=1e-4)
    # the operator called directly on such tensors raises rather than copying
    if K * K <= 121:
        q = torch.randn(2, 8, 7 * s, 9 * s, device=DEV, dtype=dt).contiguous(memory_format=torch.channels_last)
        k = torch.randn(2, 8, 7, 9, device=DEV, dtype=dt).contiguous(memory_format=torch.channels_last)
        with pytest.raises(_lib.SapaUnsupported):
            sapa_amd.sapa_fused(q, k, xcl, K, s)
    else:
        q, k = torch.randn(2, 8, 7 * s, 9 * s, device=DEV), torch.randn(2, 8, 7, 9, device=DEV)
        with pytest.raises(_lib.SapaUnsupported):
            sapa_amd.sapa_fused(q, k, x, K, s)


@pytest.mark.parametrize('cfg', [
    dict(P=9, dtype=torch.float64),     # no float64 channels-last kernel
    dict(P=40, dtype=torch.float32),    # more than 32 points: contiguous fused kernel
    dict(P=70, dtype=torch.float32),    # more than 64 points: the separate operators
])
def test_deform_module_falls_back_where_kernels_do_not_cover(cfg):
    torch.manual_seed(13)
    P, dt = cfg['P'], cfg['dtype']
    m = sapa_amd.SAPADeform(32, num_point=P, groups=2, embedding_dim=8).to(DEV).to(dt)
    torch.nn.init.normal_(m.offset.weight, std=0.1)
    torch.nn.init.normal_(m.q.weight, std=0.3)
    torch.nn.init.normal_(m.k.weight, std=0.3)
    y = torch.randn(1, 32, 12, 16, device=DEV, dtype=dt)
    x = torch.randn(1, 32, 6, 8, device=DEV, dtype=dt)
    with torch.no_grad():
        m.fused = False
        want = m(y, x)                  # sapa_deform.py:36-53 on the separate operators
        m.fused = True
        got = m(y, x)
        ycl, xcl = (t.contiguous(memory_format=torch.channels_last) for t in (y, x))
        got_cl = m(ycl, xcl)
        m.channels_last = True
        got_cl2 = m(ycl, xcl)
    tol = dict(rtol=1e-9, atol=1e-9) if dt == torch.float64 else dict(rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(got, want, **tol)
    torch.testing.assert_close(got_cl.contiguous(), want, **tol)
    assert got_cl.is_contiguous(memory_format=torch.channels_last)
    torch.testing.assert_close(got_cl2.contiguous(), want, rtol=1e-4, atol=1e-4)


def test_softmax_of_minus_infinity_is_zero():
    """A -inf logit gets weight 0 (torch.softmax, sapa_base.py:39), not NaN."""
    g = gen(14)
    x = randn(g, 2, 25, 6, 10)
    x[0, 3] = float('-inf')
    x[1, :24, 2, 5] = float('-inf')     # a single finite logit left
    got = sapa_amd.softmax_k(x.to(DEV), 1).cpu()
    want = torch.softmax(x, 1)
    assert torch.isfinite(got).all()
    assert (got[0, 3] == 0).all() and got[1, 24, 2, 5] == 1
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-7)
    x5 = randn(g, 1, 2, 9, 6, 10)
    x5[0, 1, 4] = float('-inf')
    got5 = sapa_amd.softmax_k(x5.to(DEV), 2).cpu()
    assert (got5[0, 1, 4] == 0).all()
    torch.testing.assert_close(got5, torch.softmax(x5, 2), rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize('C', [16, 128])
@pytest.mark.parametrize('bad', [float('inf'), float('nan')])
def test_sampled_gradients_carry_non_finite_values(coracle, bad, C):
    """An inf / NaN in grad_output reaches grad_value through the sampled
    aggregation's gradient, as it does through the reference's atomicAdd
    (deform_av_cuda_kernel.cu:230-292): overflow detection of a loss scaler
    relies on it.  Finite entries stay within the usual bar.  C = 16 is served
    by the LDS-window scatter, C = 128 (9 points x 64 channels per group) by
    the matrix-product scatter; one of the bad pixels has an attention weight
    of exactly 0, where the reference's 0 * inf gives NaN."""
    g = gen(15)
    B, H, W, P, s, G = 1, 12, 12, 9, 2, 2
    attn = torch.softmax(randn(g, B, G, P, H * s, W * s), dim=2)
    v = randn(g, B, C, H, W)
    off = (0.75 * randn(g, B, 2 * G * P, H * s, W * s)).clamp(-4, 4)
    go = randn(g, B, C, H * s, W * s)
    go[0, 3, 10, 9] = bad
    go[0, C - 4, 2, 20] = bad
    attn[0, 0, 4, 10, 9] = 0.0          # group of channel 3
    attn_d, v_d, off_d = (t.to(DEV) for t in (attn, v, off))
    v_d.requires_grad_(True)
    out = sapa_amd.deform_av(attn_d, v_d, off_d, P, s, G)
    out.backward(go.to(DEV))
    got = v_d.grad.cpu()
    _, want, _ = coracle.deform_av_backward(go.double(), attn.double(), v.double(), off.double(),
                                            P, s, G, 'f64')
    fin = torch.isfinite(want)
    assert not fin.all(), 'the case must produce non-finite gradients'
    assert torch.equal(torch.isfinite(got), fin)
    if bad == float('inf'):
        assert torch.equal(torch.isnan(got), torch.isnan(want))
        assert torch.equal(got[~fin & ~torch.isnan(want)], want[~fin & ~torch.isnan(want)].float())
    # channels 3 and C - 4 only: every other channel is untouched by the bad values
    torch.testing.assert_close(got[fin], want[fin].float(), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize('bad', [float('inf'), float('nan')])
def test_fused_sampled_backward_carries_non_finite_values(coracle, bad):
    """The same through the one-call backward of the fused operator
    (sapa_deform_fused_backward: matrix-product scatter, channels-last
    accumulation): grad_value against the float64 chain."""
    g = gen(16)
    B, C, d, H, W, P, s, G = 1, 128, 8, 12, 12, 9, 2, 2
    q, key = randn(g, B, G * d, H * s, W * s), randn(g, B, G * d, H, W)
    v = randn(g, B, C, H, W)
    off = (0.75 * randn(g, B, 2 * G * P, H * s, W * s)).clamp(-4, 4)
    go = randn(g, B, C, H * s, W * s)
    go[0, 3, 10, 9] = bad
    go[0, C - 4, 2, 20] = bad
    leaves = [t.to(DEV).requires_grad_(True) for t in (q, key, v, off)]
    sapa_amd.deform_sapa_fused(*leaves, P, s, G).backward(go.to(DEV))
    got = leaves[2].grad.cpu()
    attn = coracle.softmax(coracle.deform_qk(q.double(), key.double(), off.double(), P, s, G, 'f64'), 2, 'f64')
    _, want, _ = coracle.deform_av_backward(go.double(), attn, v.double(), off.double(), P, s, G, 'f64')
    fin = torch.isfinite(want)
    assert not fin.all()
    assert torch.equal(torch.isfinite(got), fin)
    if bad == float('inf'):
        assert torch.equal(torch.isnan(got), torch.isnan(want))
    torch.testing.assert_close(got[fin], want[fin].float(), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize('dtype,mode', [(torch.bfloat16, 'channels_last'), (torch.float32, 'fold_norm'),
                                        (torch.float32, 'channels_last')])
def test_module_forward_replays_from_a_hip_graph(dtype, mode):
    """The folded module forward (moments, fold, projections, fused operator: library
    launches and tensor allocations only) captured once into a HIP graph: every replay,
    with new feature values and eager work in between, gives the bits of the eager
    forward on the same values."""
    torch.manual_seed(17)
    B, C, d, H, W = 4, 256, 32, 12, 20
    m = sapa_amd.SAPA(C, embedding_dim=d).to(DEV).to(dtype)
    m.channels_last, m.fold_norm = mode == 'channels_last', mode == 'fold_norm'
    fmt = torch.channels_last if mode == 'channels_last' else torch.contiguous_format
    ys = torch.randn(B, C, 2 * H, 2 * W, device=DEV).to(dtype).contiguous(memory_format=fmt)
    xs = torch.randn(B, C, H, W, device=DEV).to(dtype).contiguous(memory_format=fmt)
    with torch.no_grad():
        for _ in range(2):
            m(ys, xs)                      # first-call set-up happens outside the capture
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = m(ys, xs)
        for _ in range(3):
            ys.copy_(torch.randn_like(ys))
            xs.copy_(torch.randn_like(xs))
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, m(ys, xs))
