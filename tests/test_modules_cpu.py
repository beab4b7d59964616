"""Host-side logic of the modules that needs no GPU: the GroupNorm-folded
projections against GroupNorm followed by Conv2d (sapa_base.py:26-36)."""
import pytest
import torch
import torch.nn as nn

from sapa_amd.modules import norm_project


@pytest.mark.parametrize('dtype,tol', [(torch.float64, 1e-12), (torch.float32, 2e-5)])
def test_norm_project_equals_groupnorm_then_conv(dtype, tol):
    torch.manual_seed(0)
    B, C, H, W = 3, 64, 7, 9
    x = (torch.randn(B, C, H, W) * 2 + 0.7).to(dtype)
    norm = nn.GroupNorm(32, C).to(dtype)
    nn.init.normal_(norm.weight, 1.0, 0.3)
    nn.init.normal_(norm.bias, 0.0, 0.3)
    convs = [nn.Conv2d(C, 16, 1).to(dtype), nn.Conv2d(C, 40, 1, bias=False).to(dtype)]
    with torch.no_grad():
        want = [c(norm(x)) for c in convs]
        got = norm_project(x, norm, *convs)
    for g, w in zip(got, want):
        assert g.shape == w.shape and g.is_contiguous()
        # statistics are taken in fp32 (as GroupNorm does), so fp64 agrees to
        # fp32 resolution of the statistics only
        torch.testing.assert_close(g, w, rtol=max(tol, 1e-5), atol=max(tol, 1e-5))


def test_norm_project_gradients_match():
    torch.manual_seed(1)
    B, C, H, W = 2, 32, 5, 6
    norm = nn.GroupNorm(32, C)
    conv = nn.Conv2d(C, 8, 1)
    grads = []
    for folded in (False, True):
        x = torch.randn(B, C, H, W, generator=torch.Generator().manual_seed(2)).requires_grad_()
        for p in list(norm.parameters()) + list(conv.parameters()):
            p.grad = None
        out = norm_project(x, norm, conv)[0] if folded else conv(norm(x))
        out.square().sum().backward()
        grads.append([x.grad] + [p.grad.clone() for p in list(norm.parameters()) + list(conv.parameters())])
    for a, b in zip(*grads):
        torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize('x_order', ['contiguous', 'channels_last'])
@pytest.mark.parametrize('out_cl', [False, True])
def test_norm_project_memory_orders(x_order, out_cl):
    """Either memory order of the feature is read in place, and the
    projection can be asked for a channels_last result: same values."""
    torch.manual_seed(3)
    B, C, H, W = 2, 64, 6, 5
    x = torch.randn(B, C, H, W) * 1.5 - 0.3
    if x_order == 'channels_last':
        x = x.contiguous(memory_format=torch.channels_last)
    norm = nn.GroupNorm(32, C)
    nn.init.normal_(norm.weight, 1.0, 0.3)
    nn.init.normal_(norm.bias, 0.0, 0.3)
    conv = nn.Conv2d(C, 24, 1)
    with torch.no_grad():
        (got,) = norm_project(x, norm, conv, channels_last=out_cl)
        (plain,) = norm_project(x, None, conv, channels_last=out_cl)
        want, want_plain = conv(norm(x)), conv(x)
    for g in (got, plain):
        assert g.shape == (B, 24, H, W)
        assert g.is_contiguous(memory_format=torch.channels_last if out_cl else torch.contiguous_format)
    torch.testing.assert_close(got, want, rtol=2e-5, atol=2e-5)
    torch.testing.assert_close(plain, want_plain, rtol=2e-5, atol=2e-5)
