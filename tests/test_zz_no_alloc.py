"""GPU: sapa_channel_moments_static, the entry point that allocates nothing
(partial sums in a fixed array inside the library), against
sapa_channel_moments with a caller-provided workspace: bit for bit, on two
calls in a row, the second on a smaller input."""
import pytest
import torch

from sapa_amd import _lib

pytestmark = pytest.mark.gpu


def _both(x, cl):
    """(workspace form, static form) of the [B, C, 2] statistics of x, through the C ABI."""
    B, C, H, W = x.shape
    h = _lib.lib()
    code = _lib.DTYPES[x.dtype]
    with torch.cuda.device(x.device):
        st = torch.cuda.current_stream(x.device).cuda_stream
        need = h.sapa_channel_moments_workspace(B, C, H * W, cl)
        assert 0 < need <= h.sapa_channel_moments_static_capacity()
        ws = torch.empty(need, dtype=torch.uint8, device=x.device)
        want = torch.full((B, C, 2), float('nan'), device=x.device)
        got = torch.full((B, C, 2), float('nan'), device=x.device)
        assert h.sapa_channel_moments(x.data_ptr(), ws.data_ptr(), want.data_ptr(), B, C, H * W, cl, code, st) == 0
        assert h.sapa_channel_moments_static(x.data_ptr(), got.data_ptr(), B, C, H * W, cl, code, st) == 0
        torch.cuda.synchronize()
    return want, got


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('cl', [0, 1])
def test_static_scratch_matches_workspace_form(cl, dtype):
    dev = torch.device('cuda:0')
    g = torch.Generator(device=dev).manual_seed(5)
    # several chunks per image in both layouts, then a smaller input on the same array
    for shape in ((3, 64, 96, 160), (2, 32, 40, 52)):
        x = (torch.randn(shape, generator=g, device=dev) * 2 + 0.5).to(dtype)
        if cl:
            x = x.contiguous(memory_format=torch.channels_last)
        want, got = _both(x, cl)
        assert torch.isfinite(got).all()
        assert torch.equal(got, want), f'{shape}: max diff {(got - want).abs().max().item()}'
        # and both agree with torch's own statistics
        xf = x.float()
        ref = torch.stack([xf.mean((2, 3)), xf.var((2, 3), unbiased=False)], -1)
        assert torch.allclose(got, ref, rtol=1e-4, atol=1e-5)


def test_static_scratch_refuses_what_does_not_fit():
    h = _lib.lib()
    dev = torch.device('cuda:0')
    x = torch.zeros(16, device=dev)
    mv = torch.zeros(16, device=dev)
    B, C, HW = 2, 1024, 1 << 22
    assert h.sapa_channel_moments_workspace(B, C, HW, 1) > h.sapa_channel_moments_static_capacity()
    # refused on the extents alone: the pointers are never dereferenced
    assert h.sapa_channel_moments_static(x.data_ptr(), mv.data_ptr(), B, C, HW, 1, 0, None) == -3


def test_static_scratch_under_graph_capture():
    """The call allocates nothing and can be recorded into a HIP graph: after one
    eager call (the library looks its array's address up on the first call on a
    device, which must therefore happen outside a capture), the call is captured,
    the allocator's byte count is unchanged, and every replay -- on fresh input,
    with eager work and synchronisations in between -- equals the workspace form
    bit for bit."""
    h = _lib.lib()
    dev = torch.device('cuda:0')
    g = torch.Generator(device=dev).manual_seed(6)
    B, C, H, W = 2, 48, 60, 84
    x = torch.randn(B, C, H, W, generator=g, device=dev)
    got = torch.full((B, C, 2), float('nan'), device=dev)
    need = h.sapa_channel_moments_workspace(B, C, H * W, 0)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    want = torch.empty_like(got)
    st = torch.cuda.current_stream(dev).cuda_stream
    assert h.sapa_channel_moments_static(x.data_ptr(), got.data_ptr(), B, C, H * W, 0, 0, st) == 0
    torch.cuda.synchronize()
    def allocator():
        st = torch.cuda.memory_stats(dev)
        return torch.cuda.memory_allocated(dev), st['allocation.all.allocated'], st['segment.all.allocated']
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        # (torch's own capture set-up allocates; the count is taken around the call alone)
        cst = torch.cuda.current_stream(dev).cuda_stream
        before = allocator()
        assert h.sapa_channel_moments_static(x.data_ptr(), got.data_ptr(), B, C, H * W, 0, 0, cst) == 0
        assert allocator() == before
    before = torch.cuda.memory_allocated(dev)
    for rep in range(3):
        x.copy_(torch.randn(B, C, H, W, generator=g, device=dev) * (rep + 1) - rep)
        got.fill_(float('nan'))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert h.sapa_channel_moments(x.data_ptr(), ws.data_ptr(), want.data_ptr(), B, C, H * W, 0, 0, st) == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want), f'replay {rep}: max diff {(got - want).abs().max().item()}'
    assert torch.cuda.memory_allocated(dev) == before
