"""SAPA / SAPADeform upsampling modules on the HIP operators.

Same constructor arguments, forward(y, x) contract and parameter names
(norm_y, norm_x, q, k, offset) as the reference's sapa_base.py:7-49 and
sapa_deform.py:7-62, so its checkpoints load.  `x` is the low-res feature
(source of key and value), `y` the high-res guide (source of the query).
`fused=True` (default) runs attention as the single fused launch; False
runs the reference's three-step composition on the separate operators.
"""
import torch.nn as nn
import torch.nn.functional as F

from .deform_func import deform_av, deform_qk, deform_sapa_fused
from .sapa_func import av, qk, sapa_fused


def _init_projection(m):
    # sapa_base.py:42-46: 1x1 projections ~ N(0, 0.02), zero bias
    if isinstance(m, nn.Conv2d):
        nn.init.normal_(m.weight, std=.02)
        if m.bias is not None:
            nn.init.constant_(m.bias, 0)


class SAPA(nn.Module):
    def __init__(self, dim_y, dim_x=None, up_factor=2, up_kernel_size=5, embedding_dim=32,
                 qkv_bias=True, norm=True, fused=True):
        super().__init__()
        dim_x = dim_y if dim_x is None else dim_x
        self.up_factor = up_factor
        self.up_kernel_size = up_kernel_size
        self.embedding_dim = embedding_dim
        self.norm = norm
        self.fused = fused
        if norm:
            self.norm_y = nn.GroupNorm(32, dim_y)
            self.norm_x = nn.GroupNorm(32, dim_x)
        self.q = nn.Conv2d(dim_y, embedding_dim, kernel_size=1, bias=qkv_bias)
        self.k = nn.Conv2d(dim_x, embedding_dim, kernel_size=1, bias=qkv_bias)
        self.apply(_init_projection)

    def forward(self, y, x):
        # the value is the un-normalised x; only the key sees norm_x(x)
        x_ = self.norm_x(x) if self.norm else x
        if self.norm:
            y = self.norm_y(y)
        return self.attention(self.q(y), self.k(x_), x)

    def attention(self, q, k, v):
        K, s = self.up_kernel_size, self.up_factor
        if self.fused:
            return sapa_fused(q.contiguous(), k.contiguous(), v.contiguous(), K, s)
        attn = F.softmax(qk(q, k, K, s), dim=1)
        return av(attn, v, K, s)


class SAPADeform(nn.Module):
    def __init__(self, dim_y, dim_x=None, up_factor=2, num_point=9, groups=4, embedding_dim=32,
                 qkv_bias=True, high_offset=True, norm=False, fused=True):
        super().__init__()
        dim_x = dim_y if dim_x is None else dim_x
        self.up_factor = up_factor
        self.num_point = num_point
        self.groups = groups
        self.embedding_dim = embedding_dim
        self.high_offset = high_offset
        self.norm = norm
        self.fused = fused
        if norm:
            self.norm_y = nn.GroupNorm(32, dim_y)
            self.norm_x = nn.GroupNorm(32, dim_x)
        self.q = nn.Conv2d(dim_y, groups * embedding_dim, kernel_size=1, bias=qkv_bias)
        self.k = nn.Conv2d(dim_x, groups * embedding_dim, kernel_size=1, bias=qkv_bias)
        # high_offset: one offset pair per high-res child, produced at low
        # resolution and pixel-shuffled up (sapa_deform.py:27-31,44-47)
        offset_dim = groups * num_point * 2 * (up_factor ** 2 if high_offset else 1)
        self.offset = nn.Conv2d(dim_x, offset_dim, kernel_size=1, bias=qkv_bias)
        self.apply(_init_projection)

    def forward(self, y, x):
        x_ = self.norm_x(x) if self.norm else x
        if self.norm:
            y = self.norm_y(y)
        q, k = self.q(y), self.k(x_)
        if self.fused:
            # the kernel reads the offset convolution's output in place
            return deform_sapa_fused(q.contiguous(), k.contiguous(), x.contiguous(),
                                     self.offset(x_).contiguous(), self.num_point,
                                     self.up_factor, self.groups,
                                     'pixel_shuffle' if self.high_offset else 'nearest')
        if self.high_offset:
            offset = F.pixel_shuffle(self.offset(x_), upscale_factor=self.up_factor)
        else:
            offset = F.interpolate(self.offset(x_), scale_factor=self.up_factor)
        return self.attention(q, k, x, offset)

    def attention(self, q, k, x, offset):
        P, s, G = self.num_point, self.up_factor, self.groups
        offset = offset.contiguous()
        if self.fused:
            return deform_sapa_fused(q.contiguous(), k.contiguous(), x.contiguous(), offset,
                                     P, s, G)
        attn = F.softmax(deform_qk(q, k, offset, P, s, G), dim=2)
        return deform_av(attn, x, offset, P, s, G)
