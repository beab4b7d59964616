"""The torch.library ops on the GPU: same bits as the eager API, usable under
torch.compile (aot_eager backend: tracing and autograd partitioning without a
code generator), and torch.library.opcheck's schema / fake / autograd checks."""
import pytest
import torch

import sapa_amd
import sapa_amd.library_ops  # noqa: F401  (registers torch.ops.sapa_amd.*)
from helpers import gen, randn

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'


def _b_inputs(dtype=torch.float32):
    g = gen(400)
    return [randn(g, 2, 6, 8, 12, dtype=dtype).to(DEV), randn(g, 2, 6, 4, 6, dtype=dtype).to(DEV),
            randn(g, 2, 10, 4, 6, dtype=dtype).to(DEV)]


def _d_inputs(dtype=torch.float32):
    g = gen(401)
    B, G, dq, cg, H, W, P, s = 1, 2, 3, 4, 5, 6, 4, 2
    return [randn(g, B, G * dq, H * s, W * s, dtype=dtype).to(DEV),
            randn(g, B, G * dq, H, W, dtype=dtype).to(DEV),
            randn(g, B, G * cg, H, W, dtype=dtype).to(DEV),
            (randn(g, B, 2 * G * P, H * s, W * s, dtype=dtype) * 1.5).to(DEV)], (P, s, G)


def test_ops_match_eager_api():
    q, key, v = _b_inputs()
    assert torch.equal(torch.ops.sapa_amd.qk(q, key, 5, 2), sapa_amd.qk(q, key, 5, 2))
    attn = torch.softmax(sapa_amd.qk(q, key, 5, 2), dim=1)
    assert torch.equal(torch.ops.sapa_amd.av(attn, v, 5, 2), sapa_amd.av(attn, v, 5, 2))
    assert torch.equal(torch.ops.sapa_amd.sapa_fused(q, key, v, 5, 2),
                       sapa_amd.sapa_fused(q, key, v, 5, 2))
    (dq, dk, dv, off), (P, s, G) = _d_inputs()
    assert torch.equal(torch.ops.sapa_amd.deform_qk(dq, dk, off, P, s, G),
                       sapa_amd.deform_qk(dq, dk, off, P, s, G))
    assert torch.equal(torch.ops.sapa_amd.deform_sapa_fused(dq, dk, dv, off, P, s, G),
                       sapa_amd.deform_sapa_fused(dq, dk, dv, off, P, s, G))


def test_compiled_module_matches_eager_forward_and_backward():
    def attention(q, key, v):
        attn = torch.softmax(torch.ops.sapa_amd.qk(q, key, 5, 2), dim=1)
        return torch.ops.sapa_amd.av(attn, v, 5, 2) + torch.ops.sapa_amd.sapa_fused(q, key, v, 5, 2)

    compiled = torch.compile(attention, backend='aot_eager', fullgraph=True)
    results = []
    for fn in (attention, compiled):
        ts = [t.clone().requires_grad_(True) for t in _b_inputs(torch.float64)]
        out = fn(*ts)
        out.square().sum().backward()
        results.append([out] + [t.grad for t in ts])
    for a, b in zip(*results):
        torch.testing.assert_close(a, b, rtol=1e-12, atol=1e-12)


def test_compiled_deform_matches_eager():
    (dq, dk, dv, off), (P, s, G) = _d_inputs(torch.float64)

    def attention(q, key, v, o):
        return torch.ops.sapa_amd.deform_sapa_fused(q, key, v, o, P, s, G)

    compiled = torch.compile(attention, backend='aot_eager', fullgraph=True)
    results = []
    for fn in (attention, compiled):
        ts = [t.clone().requires_grad_(True) for t in (dq, dk, dv, off)]
        out = fn(*ts)
        out.square().sum().backward()
        results.append([out] + [t.grad for t in ts])
    for a, b in zip(*results):
        torch.testing.assert_close(a, b, rtol=1e-9, atol=1e-10)   # atomics: order varies


def test_channels_last_ops_and_compile():
    """Channels-last operands: the ops answer in channels-last order, the
    shape-only implementations agree with that, and a compiled graph matches."""
    CL = torch.channels_last
    q, key, v = (t.contiguous(memory_format=CL) for t in _b_inputs())   # channel counts 6, 6, 10
    q, key, v = (torch.cat([t, t], 1).contiguous(memory_format=CL) for t in (q, key, v))  # 12, 12, 20
    out = torch.ops.sapa_amd.sapa_fused(q, key, v, 5, 2)
    assert out.is_contiguous(memory_format=CL)
    assert torch.equal(out, sapa_amd.sapa_fused(q, key, v, 5, 2))
    tests = ('test_schema', 'test_faketensor', 'test_autograd_registration')
    torch.library.opcheck(torch.ops.sapa_amd.sapa_fused.default, (q, key, v, 5, 2), test_utils=tests)
    torch.library.opcheck(torch.ops.sapa_amd.qk.default, (q, key, 5, 2), test_utils=tests)

    def attention(q, key, v):
        return torch.ops.sapa_amd.sapa_fused(q, key, v, 5, 2)
    compiled = torch.compile(attention, backend='aot_eager', fullgraph=True)
    leaves = [t.clone().requires_grad_() for t in (q, key, v)]
    ref_leaves = [t.clone().requires_grad_() for t in (q, key, v)]
    y, y_ref = compiled(*leaves), attention(*ref_leaves)
    assert torch.equal(y, y_ref)
    go = torch.randn_like(y_ref)
    y.backward(go)
    y_ref.backward(go)
    for a, b in zip(leaves, ref_leaves):
        assert torch.equal(a.grad, b.grad)
    # the gradient ops answer in the order of their operands, and their shape-only
    # implementations say so
    gq, gk, gv = torch.ops.sapa_amd.sapa_fused_backward(go, q, key, v, 5, 2)
    assert all(t.is_contiguous(memory_format=CL) for t in (gq, gk, gv))
    torch.library.opcheck(torch.ops.sapa_amd.sapa_fused_backward.default, (go, q, key, v, 5, 2),
                          test_utils=('test_schema', 'test_faketensor'))
    # SAPA-D: 4 channels per group so that the channels-last kernel takes it
    g = gen(402)
    B, G, H, W, P, s = 1, 2, 5, 6, 4, 2
    dq, dk = randn(g, B, G * 4, H * s, W * s).to(DEV), randn(g, B, G * 4, H, W).to(DEV)
    dv, off = randn(g, B, G * 8, H, W).to(DEV), randn(g, B, 2 * G * P, H * s, W * s).to(DEV)
    dq, dk, dv, off = (t.contiguous(memory_format=CL) for t in (dq, dk, dv, off))
    out = torch.ops.sapa_amd.deform_sapa_fused(dq, dk, dv, off, P, s, G)
    assert out.is_contiguous(memory_format=CL)
    assert torch.equal(out, sapa_amd.deform_sapa_fused(dq, dk, dv, off, P, s, G))
    torch.library.opcheck(torch.ops.sapa_amd.deform_sapa_fused.default, (dq, dk, dv, off, P, s, G),
                          test_utils=tests)


def test_opcheck():
    q, key, v = [t.requires_grad_(True) for t in _b_inputs(torch.float64)]
    tests = ('test_schema', 'test_faketensor', 'test_autograd_registration')
    torch.library.opcheck(torch.ops.sapa_amd.qk.default, (q, key, 5, 2), test_utils=tests)
    torch.library.opcheck(torch.ops.sapa_amd.sapa_fused.default, (q, key, v, 5, 2),
                          test_utils=tests)
    (dq, dk, dv, off), (P, s, G) = _d_inputs(torch.float64)
    torch.library.opcheck(torch.ops.sapa_amd.deform_sapa_fused.default,
                          (dq.requires_grad_(True), dk, dv, off, P, s, G), test_utils=tests)
