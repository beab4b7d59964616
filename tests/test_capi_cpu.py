"""CPU: the C-ABI library loads, exports every symbol include/sapa_hip.h
declares, validates arguments without touching a GPU, and the Python mirror
of the reference API keeps its error behaviour."""
import ctypes
import os
import re

import pytest
import torch

import sapa_amd
from sapa_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, 'include', 'sapa_hip.h')


def declared_functions():
    src = open(HEADER).read()
    src = re.sub(r'/\*.*?\*/', '', src, flags=re.S)
    return sorted(set(re.findall(r'\b(sapa_\w+)\s*\(', src)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 15, names
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(handle, n), f'{n} declared in include/sapa_hip.h but not exported'
    # and the Python binding covers every operator entry point
    # (the workspace query returns a size, not a status: bound separately)
    ops = [n for n in names if not n.startswith('sapa_hip_')
           and n not in ('sapa_channel_moments_workspace', 'sapa_channel_moments_static_capacity',
                         'sapa_norm_project_scratch',
                         'sapa_fused_backward_workspace', 'sapa_fused_backward_attn_workspace',
                         'sapa_deform_fused_forward_workspace',
                         'sapa_deform_fused_backward_workspace', 'sapa_deform_backward_workspace')]
    assert sorted(ops) == sorted(_lib.SIGNATURES)
    h = _lib.lib()
    assert h.sapa_channel_moments_workspace(16, 256, 67200, 0) > 0
    assert h.sapa_channel_moments_workspace(0, 256, 67200, 1) == 0
    assert h.sapa_channel_moments_static_capacity() == 8 << 20
    assert h.sapa_fused_backward_workspace(2, 10, 12, 5, 2) == 2 * 2 * 25 * 20 * 24 * 4
    assert h.sapa_fused_backward_attn_workspace(2, 10, 12, 5, 2) == 2 * 25 * 20 * 24 * 4
    # key [8,128,64,64] + value [8,256,64,64] in bf16; fp32 with few points and fp64: not served
    assert h.sapa_deform_fused_forward_workspace(8, 128, 256, 64, 64, 25, 2, 4, _lib.DTYPES[torch.bfloat16]) == 8 * 4096 * (128 + 256) * 2
    assert h.sapa_deform_fused_forward_workspace(8, 128, 256, 64, 64, 5, 2, 4, _lib.DTYPES[torch.float32]) == 0
    assert h.sapa_deform_fused_forward_workspace(8, 128, 256, 64, 64, 25, 2, 4, _lib.DTYPES[torch.float64]) == 0
    # fp32 copy of the per-point tensor + fp32 accumulator of the low-res gradient; 16-bit tensors only
    assert (h.sapa_deform_backward_workspace(8, 128, 64, 64, 25, 2, 4, _lib.DTYPES[torch.bfloat16])
            == 8 * 4 * 25 * 128 * 128 * 4 + 8 * 128 * 4096 * 4)
    assert h.sapa_deform_backward_workspace(8, 128, 64, 64, 25, 2, 4, _lib.DTYPES[torch.float32]) == 0
    assert h.sapa_deform_backward_workspace(8, 128, 64, 64, 25, 3, 4, _lib.DTYPES[torch.float16]) == 0
    # the point counts from which the path serves, as include/sapa_hip.h states them:
    # 16-bit tensors from 4 points, fp32 from 13
    bf, f32 = _lib.DTYPES[torch.bfloat16], _lib.DTYPES[torch.float32]
    assert h.sapa_deform_fused_forward_workspace(8, 128, 256, 64, 64, 3, 2, 4, bf) == 0
    assert h.sapa_deform_fused_forward_workspace(8, 128, 256, 64, 64, 4, 2, 4, bf) == 8 * 4096 * (128 + 256) * 2
    assert h.sapa_deform_fused_forward_workspace(8, 128, 256, 64, 64, 12, 2, 4, f32) == 0
    assert h.sapa_deform_fused_forward_workspace(8, 128, 256, 64, 64, 13, 2, 4, f32) == 8 * 4096 * (128 + 256) * 4
    # two fp32 [B,G,P,sH,sW] tensors, fp32 accumulators of the two low-res gradients and
    # channels-last copies of key and value for the matrix-form stage.  Groups that stage does not
    # serve (5 channels): no copies, but half of grad_offset in fp32 for 16-bit tensors
    per_point = 8 * 4 * 25 * 128 * 128 * 4
    low = 8 * 4096 * (128 + 256)
    assert h.sapa_deform_fused_backward_workspace(8, 128, 256, 64, 64, 25, 2, 4, _lib.DTYPES[torch.float32]) == 2 * per_point + low * 4 + low * 4
    assert (h.sapa_deform_fused_backward_workspace(8, 128, 256, 64, 64, 25, 2, 4, _lib.DTYPES[torch.bfloat16])
            == 2 * per_point + low * 4 + low * 2)
    low5 = 8 * 4096 * (20 + 256)
    assert h.sapa_deform_fused_backward_workspace(8, 20, 256, 64, 64, 25, 2, 4, _lib.DTYPES[torch.float32]) == 2 * per_point + low5 * 4
    assert (h.sapa_deform_fused_backward_workspace(8, 20, 256, 64, 64, 25, 2, 4, _lib.DTYPES[torch.bfloat16])
            == 4 * per_point + low5 * 4)
    assert h.sapa_deform_fused_backward_workspace(8, 128, 256, 64, 64, 25, 3, 4, _lib.DTYPES[torch.float32]) == 0


def test_abi_version_and_status_strings():
    h = _lib.lib()
    assert h.sapa_hip_abi_version() == _lib.ABI_VERSION
    assert h.sapa_hip_status_string(0) == b'ok'
    for code in (-1, -2, -3, -4):
        assert h.sapa_hip_status_string(code) not in (b'ok', b'unknown status')
    assert h.sapa_hip_status_string(-99) == b'unknown status'
    assert h.sapa_hip_last_hip_error() == b''
    assert h.sapa_hip_last_kernel() == b''


def test_argument_validation_returns_codes():
    """Rejected before any HIP call, so this runs without a GPU."""
    h = _lib.lib()
    p = ctypes.c_void_p(16)  # never dereferenced: the calls below fail validation
    # even kernel size
    assert h.sapa_qk_forward(p, p, p, 1, 4, 8, 8, 4, 2, 0, None) == -1
    # bad dtype, scale < 1, non-positive extents
    assert h.sapa_qk_forward(p, p, p, 1, 4, 8, 8, 5, 2, 7, None) == -1
    assert h.sapa_av_forward(p, p, p, 1, 4, 8, 8, 5, 0, 0, None) == -1
    assert h.sapa_av_forward(p, p, p, 1, 0, 8, 8, 5, 2, 0, None) == -1
    assert h.sapa_fused_forward(p, p, p, p, 1, 4, 4, -1, 8, 5, 2, 0, None) == -1
    # null pointers
    assert h.sapa_qk_forward(None, p, p, 1, 4, 8, 8, 5, 2, 0, None) == -1
    assert h.sapa_fused_forward(p, p, None, p, 1, 4, 4, 8, 8, 5, 2, 0, None) == -1
    # empty batch is a no-op
    assert h.sapa_qk_forward(None, None, None, 0, 4, 8, 8, 5, 2, 0, None) == 0
    # fused window beyond 11x11: unsupported; index range: too large
    assert h.sapa_fused_forward(p, p, p, p, 1, 4, 4, 8, 8, 13, 2, 0, None) == -2
    assert h.sapa_qk_forward(p, p, p, 1, 4, 1 << 23, 8, 5, 2, 0, None) == -3
    # deform: channels not divisible by groups, P < 1, fused P > 64, 16-bit backward
    assert h.sapa_deform_qk_forward(p, p, p, p, 1, 6, 8, 8, 5, 2, 4, 0, None) == -1
    assert h.sapa_deform_av_forward(p, p, p, p, 1, 8, 8, 8, 0, 2, 4, 0, None) == -1
    assert h.sapa_deform_fused_forward(p, p, p, p, p, 1, 8, 8, 8, 8, 65, 2, 4, 0, None) == -2
    assert h.sapa_deform_qk_backward(p, p, p, p, p, p, p, 1, 8, 8, 8, 5, 2, 4, 3, None) == -2
    assert h.sapa_softmax_forward(p, p, 4, 0, 4, 0, None) == -1
    # channels-last entry points: the same checks in front of the kernels
    assert h.sapa_fused_forward_nhwc(p, p, p, p, 1, 4, 4, 8, 8, 4, 2, 0, None) == -1
    assert h.sapa_fused_forward_nhwc(p, p, None, p, 1, 4, 4, 8, 8, 5, 2, 0, None) == -1
    assert h.sapa_qk_forward_nhwc(None, None, None, 0, 4, 8, 8, 5, 2, 0, None) == 0
    # channel moments: extents, dtype (no fp64 kernel), null pointers, empty batch
    assert h.sapa_channel_moments(p, p, p, 1, 0, 64, 0, 0, None) == -1
    assert h.sapa_channel_moments(p, p, p, 1, 8, 0, 1, 0, None) == -1
    assert h.sapa_channel_moments(p, p, p, 1, 8, 64, 0, 1, None) == -2
    assert h.sapa_channel_moments(p, None, p, 1, 8, 64, 0, 0, None) == -1
    assert h.sapa_channel_moments(None, None, None, 0, 8, 64, 0, 0, None) == 0
    # the form without a workspace: same validation, and extents whose partial
    # sums exceed the library's fixed array are refused before any HIP call
    assert h.sapa_channel_moments_static(p, p, 1, 0, 64, 0, 0, None) == -1
    assert h.sapa_channel_moments_static(p, p, 1, 8, 64, 0, 1, None) == -2
    assert h.sapa_channel_moments_static(None, p, 1, 8, 64, 0, 0, None) == -1
    assert h.sapa_channel_moments_static(None, None, 0, 8, 64, 0, 0, None) == 0
    big = (2, 1024, 1 << 22, 1)
    assert h.sapa_channel_moments_workspace(*big) > h.sapa_channel_moments_static_capacity()
    assert h.sapa_channel_moments_static(p, p, big[0], big[1], big[2], big[3], 0, None) == -3
    # projection: extents, null pointers, fp64 (no kernel), empty batch
    assert h.sapa_project_nhwc(p, p, p, p, 1, 0, 64, 100, 3, None) == -1
    assert h.sapa_project_nhwc(p, None, p, p, 1, 256, 64, 100, 3, None) == -1
    assert h.sapa_project_nhwc(p, p, None, p, 1, 256, 64, 100, 1, None) == -2
    assert h.sapa_project_nhwc(None, None, None, None, 0, 256, 64, 100, 3, None) == 0
    assert h.sapa_project_nchw(p, p, p, p, 1, 256, 0, 100, 0, 0, None) == -1
    assert h.sapa_project_nchw(p, p, p, None, 1, 256, 64, 100, 1, 0, None) == -1
    assert h.sapa_project_nchw(p, p, None, p, 1, 256, 64, 100, 0, 1, None) == -2     # fp64
    assert h.sapa_project_nchw(p, p, None, p, 1, 256, 64, 100, 0, 3, None) == -2     # 16-bit planes of 100 pixels
    assert h.sapa_project_nchw(p, p, None, p, 1, 256, 64, 102, 0, 0, None) == -2     # planes of 102 pixels
    assert h.sapa_project_nchw(None, None, None, None, 0, 256, 64, 100, 1, 0, None) == 0
    # moments + fold + projection in one call: scratch = moments workspace + [B,C,2] fp32 + folded
    # weights + folded bias, each rounded to 256 bytes; extents, null pointers; configurations without
    # a kernel are refused before anything is launched
    assert (h.sapa_norm_project_scratch(16, 256, 64, 67200, 1, 3)
            == (h.sapa_channel_moments_workspace(16, 256, 67200, 1) + 255) // 256 * 256
            + 16 * 256 * 8 + 16 * 64 * 256 * 2 + 16 * 64 * 2)
    assert h.sapa_norm_project_scratch(0, 256, 64, 67200, 1, 3) == 0
    assert h.sapa_norm_project(p, p, p, p, p, p, p, p, 1, 256, 64, 100, 0, 1e-5, 1, 1, 3, None) == -1
    assert h.sapa_norm_project(p, p, p, p, p, None, p, p, 1, 256, 64, 100, 32, 1e-5, 1, 1, 3, None) == -1
    assert h.sapa_norm_project(p, p, p, p, p, p, p, p, 1, 256, 64, 100, 32, 1e-5, 1, 1, 1, None) == -2     # fp64
    assert h.sapa_norm_project(p, p, p, p, p, p, p, p, 1, 256, 48, 100, 32, 1e-5, 1, 1, 3, None) == -2     # no (256, 48)
    assert h.sapa_norm_project(p, p, p, p, p, p, p, p, 1, 256, 64, 100, 32, 1e-5, 0, 0, 3, None) == -2     # 16-bit planes of 100
    assert h.sapa_norm_project(p, p, p, p, p, p, p, p, 1, 256, 64, 100, 48, 1e-5, 1, 1, 3, None) == -2     # 256 % 48
    assert h.sapa_norm_project(None, None, None, None, None, None, None, None, 0, 256, 64, 100, 32, 1e-5, 1, 1, 3, None) == 0
    # layout copy: element size, negative extents, null / misaligned pointers, empty tensors,
    # more rows than the tiled side holds
    assert h.sapa_layout_copy(p, p, 1, 8, 64, 1, 3, None) == -1
    assert h.sapa_layout_copy(p, p, 1, -1, 64, 1, 4, None) == -1
    assert h.sapa_layout_copy(None, p, 1, 8, 64, 0, 4, None) == -1
    assert h.sapa_layout_copy(ctypes.c_void_p(18), p, 1, 8, 64, 0, 4, None) == -1
    assert h.sapa_layout_copy(None, None, 0, 8, 64, 1, 2, None) == 0
    assert h.sapa_layout_copy(p, p, 1, 4, 5000000, 0, 4, None) == -2
    # GroupNorm fold: channels not divisible by the groups, null weight, empty batch
    assert h.sapa_groupnorm_fold(p, p, p, p, p, p, p, 1, 10, 4, 4, 1e-5, 0, None) == -1
    assert h.sapa_groupnorm_fold(p, p, p, None, p, p, p, 1, 8, 4, 4, 1e-5, 0, None) == -1
    assert h.sapa_groupnorm_fold(None, None, None, None, None, None, None, 0, 8, 4, 4, 1e-5, 0, None) == 0


def test_python_api_surface():
    for name in ('qk', 'av', 'sapa_fused', 'deform_qk', 'deform_av', 'deform_sapa_fused',
                 'SAPA', 'SAPADeform'):
        assert hasattr(sapa_amd, name)
    import deformsapa
    import sapa
    assert sapa.qk is sapa_amd.qk and sapa.av is sapa_amd.av
    assert deformsapa.deform_qk is sapa_amd.deform_qk
    assert deformsapa.deform_av is sapa_amd.deform_av


def test_cpu_tensors_raise_not_implemented():
    """sapa/sapa/sapa_func.py:27-28, deform_func.py:33-34: no CPU path."""
    q, k, v = torch.randn(1, 4, 8, 8), torch.randn(1, 4, 4, 4), torch.randn(1, 3, 4, 4)
    with pytest.raises(NotImplementedError):
        sapa_amd.qk(q, k, 5, 2)
    with pytest.raises(NotImplementedError):
        sapa_amd.av(torch.randn(1, 25, 8, 8), v, 5, 2)
    with pytest.raises(NotImplementedError):
        sapa_amd.sapa_fused(q, k, v, 5, 2)
    off = torch.randn(1, 2 * 2 * 3, 8, 8)
    with pytest.raises(NotImplementedError):
        sapa_amd.deform_qk(q, k, off, 3, 2, 2)
    with pytest.raises(NotImplementedError):
        sapa_amd.deform_av(torch.randn(1, 2, 3, 8, 8), torch.randn(1, 4, 4, 4), off, 3, 2, 2)


def test_shape_assertions_match_reference():
    """sapa_func.py:13-17,58-62; deform_func.py:11-21,66-76."""
    k = torch.randn(2, 4, 4, 4)
    with pytest.raises(AssertionError):
        sapa_amd.qk(torch.randn(2, 4, 8, 9), k, 5, 2)       # width mismatch
    with pytest.raises(AssertionError):
        sapa_amd.qk(torch.randn(1, 4, 8, 8), k, 5, 2)       # batch mismatch
    with pytest.raises(AssertionError):
        sapa_amd.qk(torch.randn(2, 4, 8, 8), k, 4, 2)       # even kernel
    with pytest.raises(AssertionError):
        sapa_amd.qk(torch.randn(2, 4, 8, 8), k, 5, 0)       # scale < 1
    with pytest.raises(AssertionError):
        sapa_amd.av(torch.randn(2, 9, 8, 8), k, 5, 2)       # attn channels != K*K
    off = torch.randn(2, 2 * 2 * 3, 8, 8)
    with pytest.raises(AssertionError):
        sapa_amd.deform_qk(torch.randn(2, 4, 8, 8), k, off, 3, 2, 4)    # offset ch != 2GP
    with pytest.raises(AssertionError):
        sapa_amd.deform_qk(torch.randn(2, 4, 8, 8), k, off[:, :6], 1, 2, 3)  # C % G
    with pytest.raises(AssertionError):
        sapa_amd.deform_av(torch.randn(2, 2, 4, 8, 8), k, off, 3, 2, 2)  # attn P mismatch


def test_module_parameter_names_match_reference():
    """state_dict keys of sapa_base.py / sapa_deform.py, so checkpoints load."""
    m = sapa_amd.SAPA(64, embedding_dim=32)
    assert sorted(m.state_dict()) == sorted(
        ['norm_y.weight', 'norm_y.bias', 'norm_x.weight', 'norm_x.bias',
         'q.weight', 'q.bias', 'k.weight', 'k.bias'])
    assert m.q.weight.shape == (32, 64, 1, 1)
    md = sapa_amd.SAPADeform(16, num_point=9, groups=4, embedding_dim=8)
    assert sorted(md.state_dict()) == sorted(
        ['q.weight', 'q.bias', 'k.weight', 'k.bias', 'offset.weight', 'offset.bias'])
    assert md.offset.weight.shape == (4 * 9 * 2 * 4, 16, 1, 1)
    assert md.q.weight.shape == (32, 16, 1, 1)
    md2 = sapa_amd.SAPADeform(16, high_offset=False, norm=False)
    assert md2.offset.weight.shape[0] == 4 * 9 * 2
    assert float(m.q.bias.detach().abs().sum()) == 0.0
    assert 0.01 < float(m.q.weight.detach().std()) < 0.03
