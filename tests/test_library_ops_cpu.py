"""torch.library registration of the operators: schemas and shape-only
implementations (no GPU needed; the kernels themselves are not called)."""
import pytest
import torch

import sapa_amd.library_ops as ops


def meta(*shape, dtype=torch.float32):
    return torch.empty(*shape, device='meta', dtype=dtype)


def test_ops_are_registered():
    for name in ops.__all__:
        assert hasattr(torch.ops.sapa_amd, name), name


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_fake_shapes_sapa_b(dtype):
    B, d, C, H, W, K, s = 2, 8, 16, 5, 7, 5, 2
    q, key, v = meta(B, d, H * s, W * s, dtype=dtype), meta(B, d, H, W, dtype=dtype), meta(B, C, H, W, dtype=dtype)
    logits = torch.ops.sapa_amd.qk(q, key, K, s)
    assert logits.shape == (B, K * K, H * s, W * s) and logits.dtype == dtype
    out = torch.ops.sapa_amd.av(logits, v, K, s)
    assert out.shape == (B, C, H * s, W * s) and out.dtype == dtype
    assert torch.ops.sapa_amd.sapa_fused(q, key, v, K, s).shape == (B, C, H * s, W * s)
    gq, gk = torch.ops.sapa_amd.qk_backward(logits, q, key, K, s)
    assert gq.shape == q.shape and gk.shape == key.shape
    ga, gv = torch.ops.sapa_amd.av_backward(out, logits, v, K, s)
    assert ga.shape == logits.shape and gv.shape == v.shape
    assert [t.shape for t in torch.ops.sapa_amd.sapa_fused_backward(out, q, key, v, K, s)] == \
        [q.shape, key.shape, v.shape]


def test_fake_shapes_sapa_d():
    B, G, dq, cg, H, W, P, s = 2, 4, 3, 5, 6, 4, 9, 2
    q, key, v = meta(B, G * dq, H * s, W * s), meta(B, G * dq, H, W), meta(B, G * cg, H, W)
    off = meta(B, 2 * G * P, H * s, W * s)
    logits = torch.ops.sapa_amd.deform_qk(q, key, off, P, s, G)
    assert logits.shape == (B, G, P, H * s, W * s)
    assert torch.ops.sapa_amd.deform_av(logits, v, off, P, s, G).shape == (B, G * cg, H * s, W * s)
    assert torch.ops.sapa_amd.deform_sapa_fused(q, key, v, off, P, s, G).shape == \
        (B, G * cg, H * s, W * s)
    lo = meta(B, 2 * G * P * s * s, H, W)
    out = torch.ops.sapa_amd.deform_sapa_fused(q, key, v, lo, P, s, G, 'pixel_shuffle')
    assert out.shape == (B, G * cg, H * s, W * s)
    grads = torch.ops.sapa_amd.deform_sapa_fused_backward(out, q, key, v, lo, P, s, G,
                                                          'pixel_shuffle')
    assert [t.shape for t in grads] == [q.shape, key.shape, v.shape, lo.shape]


def test_compile_traces_without_graph_breaks_on_fake_inputs():
    """make_fx over fake tensors records the ops as single nodes, forward and
    backward: what torch.compile needs to keep a model in one graph."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.fx.experimental.proxy_tensor import make_fx

    def f(q, key, v):
        out = torch.ops.sapa_amd.sapa_fused(q, key, v, 5, 2)
        return torch.autograd.grad(out.sum(), (q, key, v))

    with FakeTensorMode():
        q = torch.empty(1, 4, 8, 8, requires_grad=True)
        key = torch.empty(1, 4, 4, 4, requires_grad=True)
        v = torch.empty(1, 6, 4, 4, requires_grad=True)
        gm = make_fx(f)(q, key, v)
    targets = [str(n.target) for n in gm.graph.nodes if n.op == 'call_function']
    assert any('sapa_fused.default' in t for t in targets)
    assert any('sapa_fused_backward' in t for t in targets)
