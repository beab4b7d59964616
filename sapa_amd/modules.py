"""SAPA / SAPADeform upsampling modules on the HIP operators.

Same constructor arguments, forward(y, x) contract and parameter names
(norm_y, norm_x, q, k, offset) as the reference's sapa_base.py:7-49 and
sapa_deform.py:7-62, so its checkpoints load.  `x` is the low-res feature
(source of key and value), `y` the high-res guide (source of the query).
`fused=True` (default) runs attention as the single fused launch; False
runs the reference's three-step composition on the separate operators.
`fold_norm=True` folds the GroupNorms into the 1x1 projections (one batched
GEMM per projection straight from the un-normalised feature);
`channels_last=True` (both modules) additionally has those GEMMs write q and
k (and the offsets) in channels_last order and runs the fused operator in
that order.
"""
import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _lib
from .deform_func import deform_av, deform_qk, deform_sapa_fused
from .sapa_func import av, in_memory_order, qk, sapa_fused


def _needs_grad(*mods):
    """True when autograd is recording and a parameter of `mods` requires grad."""
    return torch.is_grad_enabled() and any(
        p.requires_grad for m in mods if m is not None for p in m.parameters())


def norm_project(x, norm, *convs, channels_last=False, defer_bias=False):
    """conv(norm(x)) for a GroupNorm and one or more 1x1 convolutions fed by
    it (sapa_base.py:26-36: norm_y -> q, norm_x -> k) without materialising
    norm(x): the normalisation is affine per (image, channel), so it folds into
    per-image projection weights

        W'[b,o,c] = W[o,c] * gamma[c] * rstd[b,g(c)]
        b'[b,o]   = bias[o] + sum_c W[o,c] * (beta[c] - gamma[c] * mean[b,g(c)] * rstd[b,g(c)])

    and each projection becomes one batched GEMM  W'[b] @ x[b]  reading x
    directly.  That removes the write and re-read of norm(x) (2.2 GB for the
    largest FPN level in fp32).  Exact in real arithmetic; in floating point it
    differs from the two-step form by rounding only, with one caveat: the mean
    is subtracted after the GEMM instead of before it, so it loses accuracy if
    |mean| exceeds the standard deviation of a group by many orders of magnitude.
    Statistics are taken in fp32, like GroupNorm's.  `norm` may be None (plain
    1x1 convolutions).  x may be contiguous or in channels_last order; either
    way it is read in place.  Returns a list, one output per convolution, each
    [B, out, H, W]: contiguous, or -- channels_last=True -- in channels_last
    order (the GEMM is then written as x[b]^T @ W'[b]^T, whose result is the
    channels-last tensor: the layout the operators are fastest in costs the
    projection nothing).  defer_bias=True: the per-image biases [B, out] are not
    added; the list holds (output without bias, bias) pairs (for an operator
    that adds the bias itself)."""
    B, C, H, W = x.shape
    x_cl = not x.is_contiguous() and x.is_contiguous(memory_format=torch.channels_last)
    if (norm is not None and len(convs) == 1 and x.is_cuda and not torch.is_grad_enabled()
            and convs[0].kernel_size == (1, 1) and convs[0].groups == 1 and (channels_last or not x_cl)):
        # inference on the GPU, one projection of the feature: moments, fold and projection in one
        # library call (the same four launches as below, a third of the host time)
        res = _lib.norm_project(x, norm, convs[0], channels_last_out=channels_last, defer_bias=defer_bias)
        if res is not None:
            return [res if defer_bias else res[0]]
    if norm is not None:
        G = norm.num_groups
        per_c = C // G
        # inference on the GPU: one pass of the library's moments kernel over x
        # (it has no backward, so tensors that need gradients take the torch path)
        mom = None
        # statistics and folded weights in fp32 like GroupNorm's (fp64 for fp64 tensors)
        acc = torch.float64 if x.dtype == torch.float64 else torch.float32
        if x.is_cuda and not (torch.is_grad_enabled() and x.requires_grad):
            mom = _lib.channel_moments(x)
        # the per-(image, channel) scale and shift of the normalisation as torch tensors: only the
        # projections that do not go through the library's fold kernel below need them (a dozen
        # small launches otherwise spent for nothing)
        def affine():
            if mom is not None:
                mean_ch, var_ch = (mom[..., i].reshape(B, G, per_c) for i in (0, 1))
                mean = mean_ch.mean(dim=2)
                var = (var_ch + (mean_ch - mean.unsqueeze(2)).square()).mean(dim=2)
            elif x_cl:
                # per-channel moments, then per group: no layout copy of x
                m1 = x.mean(dim=(2, 3), dtype=acc).reshape(B, G, per_c)
                m2 = (torch.linalg.vector_norm(x, dim=(2, 3), dtype=acc).square()
                      / (H * W)).reshape(B, G, per_c)
                mean = m1.mean(dim=2)
                var = (m2.mean(dim=2) - mean * mean).clamp_min(0)
            else:
                xg = x.reshape(B, G, -1)
                if x.dtype in (torch.float16, torch.bfloat16):
                    # fp32 accumulation straight from the 16-bit tensor (no fp32 copy)
                    mean = xg.mean(dim=2, dtype=torch.float32)
                    sq = torch.linalg.vector_norm(xg, dim=2, dtype=torch.float32).square() / xg.shape[2]
                    var = (sq - mean * mean).clamp_min(0)
                else:
                    var, mean = torch.var_mean(xg.to(acc), dim=2, unbiased=False)
            rstd = torch.rsqrt(var + norm.eps)
            rstd_c = rstd.repeat_interleave(per_c, dim=1)                    # [B, C]
            mean_c = mean.repeat_interleave(per_c, dim=1)
            gamma = norm.weight.to(acc) if norm.weight is not None else x.new_ones(C, dtype=acc)
            beta = norm.bias.to(acc) if norm.bias is not None else x.new_zeros(C, dtype=acc)
            scale = gamma.unsqueeze(0) * rstd_c                              # [B, C]
            shift = beta.unsqueeze(0) - mean_c * scale                       # [B, C]
            return scale, shift
    else:
        mom = None
        acc = torch.float64 if x.dtype == torch.float64 else torch.float32

        def affine():
            return x.new_ones(B, C, dtype=acc), x.new_zeros(B, C, dtype=acc)
    scale_shift = None
    # [B, C, HW] view of x in either memory order
    x3 = x.permute(0, 2, 3, 1).reshape(B, H * W, C).transpose(1, 2) if x_cl else x.reshape(B, C, H * W)
    outs = []
    for conv in convs:
        assert conv.kernel_size == (1, 1) and conv.groups == 1
        O = conv.out_channels
        folded = None
        if norm is not None and mom is not None and not _needs_grad(norm, conv):
            # the per-image weights and bias in one small kernel launch (the kernel
            # has no backward: parameters that train take the torch expressions below)
            folded = _lib.groupnorm_fold(mom, norm, conv, x.dtype)
        if folded is not None:
            w_b, b_b = folded
        else:
            if scale_shift is None:
                scale_shift = affine()
            scale, shift = scale_shift
            w = conv.weight.reshape(O, C).to(acc)
            w_b = (w.unsqueeze(0) * scale.unsqueeze(1)).to(x.dtype)      # [B, O, C]
            b_b = torch.einsum('oc,bc->bo', w, shift)
            if conv.bias is not None:
                b_b = b_b + conv.bias.to(acc).unsqueeze(0)
            b_b = b_b.to(x.dtype)
        # GEMM, then the bias in place: measurably faster than baddbmm here, which
        # first spreads the bias over the whole output
        if channels_last:
            # a channels_last feature (f16 / bf16 / fp32) that needs no gradient: the
            # library's streaming projection kernel (bias in its epilogue); else a
            # library GEMM
            out = None
            if x.is_cuda and not torch.is_grad_enabled():
                if x_cl:
                    out = _lib.project_nhwc(x, w_b, None if defer_bias else b_b)
                else:
                    # (a contiguous feature: the same kernels reading planes)
                    out = _lib.project_nchw(x, w_b, None if defer_bias else b_b, channels_last_out=True)
            if out is None:
                out = torch.bmm(x3.transpose(1, 2), w_b.transpose(1, 2))      # [B, HW, O]
                if not defer_bias:
                    out.add_(b_b.unsqueeze(1))
                out = out.view(B, H, W, O).permute(0, 3, 1, 2)
        else:
            out = None
            if x.is_cuda and not x_cl and not torch.is_grad_enabled():
                out = _lib.project_nchw(x, w_b, None if defer_bias else b_b)
            if out is None:
                out = torch.bmm(w_b, x3)                                 # [B, O, HW]
                if not defer_bias:
                    out.add_(b_b.unsqueeze(2))
                out = out.view(B, O, H, W)
        outs.append((out, b_b) if defer_bias else out)
    return outs


def _init_projection(m):
    # sapa_base.py:42-46: 1x1 projections ~ N(0, 0.02), zero bias
    if isinstance(m, nn.Conv2d):
        nn.init.normal_(m.weight, std=.02)
        if m.bias is not None:
            nn.init.constant_(m.bias, 0)


class SAPA(nn.Module):
    def __init__(self, dim_y, dim_x=None, up_factor=2, up_kernel_size=5, embedding_dim=32,
                 qkv_bias=True, norm=True, fused=True, fold_norm=False, channels_last=False):
        super().__init__()
        dim_x = dim_y if dim_x is None else dim_x
        self.up_factor = up_factor
        self.up_kernel_size = up_kernel_size
        # channels_last: the projections emit q and k in channels_last order
        # (free: norm_project) and the operator runs in that order, its fastest;
        # the value is used as it is if it already is channels_last, else copied
        # once (a low-res tensor); the result is a channels_last tensor
        self.channels_last = channels_last
        self.embedding_dim = embedding_dim
        self.norm = norm
        self.fused = fused
        # fold_norm: GroupNorm folded into the q / k projections (norm_project)
        self.fold_norm = fold_norm
        if norm:
            self.norm_y = nn.GroupNorm(32, dim_y)
            self.norm_x = nn.GroupNorm(32, dim_x)
        self.q = nn.Conv2d(dim_y, embedding_dim, kernel_size=1, bias=qkv_bias)
        self.k = nn.Conv2d(dim_x, embedding_dim, kernel_size=1, bias=qkv_bias)
        self.apply(_init_projection)

    def forward(self, y, x):
        # the value is the un-normalised x; only the key sees norm_x(x)
        if self.channels_last:
            ny, nx = (self.norm_y, self.norm_x) if self.norm else (None, None)
            # the query's bias goes into the fused operator instead of a pass of its
            # own over the hi-res query tensor
            ((q, q_bias),) = norm_project(y, ny, self.q, channels_last=True, defer_bias=True)
            if not self.fused:
                q, q_bias = q.add_(q_bias[:, :, None, None]), None
            (k,) = norm_project(x, nx, self.k, channels_last=True)
            return self.attention(q, k, in_memory_order(x, torch.channels_last), q_bias)
        if self.norm and self.fold_norm:
            (q,), (k,) = norm_project(y, self.norm_y, self.q), norm_project(x, self.norm_x, self.k)
            return self.attention(q, k, x)
        x_ = self.norm_x(x) if self.norm else x
        if self.norm:
            y = self.norm_y(y)
        return self.attention(self.q(y), self.k(x_), x)

    def attention(self, q, k, v, q_bias=None):
        K, s = self.up_kernel_size, self.up_factor
        # the operators take one memory order for all their tensors: the value's
        # (the caller's feature map) decides, so a channels-last model stays
        # channels-last end to end; for tensors already in that order these
        # calls return the tensor itself
        fmt = (torch.channels_last
               if not v.is_contiguous() and v.is_contiguous(memory_format=torch.channels_last)
               else torch.contiguous_format)
        q, k, v = (in_memory_order(t, fmt) for t in (q, k, v))
        try:
            return self._attend(q, k, v, q_bias, fmt)
        except _lib.SapaUnsupported:
            if fmt is not torch.channels_last:
                raise
        # a configuration the channels-last kernels do not cover (float64, other
        # (kernel, scale) pairs, channel counts that are no multiple of 4): one
        # layout copy each way and the contiguous kernels, which serve them all
        out = self._attend(*(in_memory_order(t, torch.contiguous_format) for t in (q, k, v)), q_bias,
                           torch.contiguous_format)
        return in_memory_order(out, torch.channels_last)

    def _attend(self, q, k, v, q_bias, fmt):
        K, s = self.up_kernel_size, self.up_factor
        if self.fused:
            try:
                return sapa_fused(q, k, v, K, s, q_bias)
            except _lib.SapaUnsupported:
                if fmt is torch.channels_last:
                    raise
            # kernel sizes beyond the fused kernel's register budget: the three
            # operators, which take any odd kernel size
        if q_bias is not None:
            q = q + q_bias[:, :, None, None]
        attn = F.softmax(qk(q, k, K, s), dim=1).contiguous(memory_format=fmt)
        return av(attn, v, K, s)


class SAPADeform(nn.Module):
    def __init__(self, dim_y, dim_x=None, up_factor=2, num_point=9, groups=4, embedding_dim=32,
                 qkv_bias=True, high_offset=True, norm=False, fused=True, fold_norm=False,
                 channels_last=False):
        super().__init__()
        dim_x = dim_y if dim_x is None else dim_x
        self.fold_norm = fold_norm
        # channels_last: as for SAPA -- q, k and the offsets leave their projections
        # in channels_last order, the fused operator runs in that order
        self.channels_last = channels_last
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
        if self.channels_last and self.fused:
            (q,) = norm_project(y, self.norm_y if self.norm else None, self.q, channels_last=True)
            k, offset_lo = norm_project(x, self.norm_x if self.norm else None, self.k, self.offset,
                                        channels_last=True)
            if self.high_offset:
                offset = F.pixel_shuffle(offset_lo, upscale_factor=self.up_factor)
            else:
                offset = F.interpolate(offset_lo, scale_factor=self.up_factor)
            return self.attention(q, k, in_memory_order(x, torch.channels_last), offset)
        if self.norm and self.fold_norm:
            (q,) = norm_project(y, self.norm_y, self.q)
            k, offset_lo = norm_project(x, self.norm_x, self.k, self.offset)
        else:
            x_ = self.norm_x(x) if self.norm else x
            if self.norm:
                y = self.norm_y(y)
            q, k, offset_lo = self.q(y), self.k(x_), self.offset(x_)
        if self.fused and (x.is_contiguous()
                           or not x.is_contiguous(memory_format=torch.channels_last)):
            # the kernel reads the offset convolution's output in place
            try:
                return deform_sapa_fused(*(in_memory_order(t, torch.contiguous_format) for t in (q, k, x)),
                                         offset_lo.contiguous(), self.num_point,
                                         self.up_factor, self.groups,
                                         'pixel_shuffle' if self.high_offset else 'nearest')
            except _lib.SapaUnsupported:
                pass    # more points than the fused kernel holds: attention() below
        if self.high_offset:
            offset = F.pixel_shuffle(offset_lo, upscale_factor=self.up_factor)
        else:
            offset = F.interpolate(offset_lo, scale_factor=self.up_factor)
        return self.attention(q, k, x, offset)

    def attention(self, q, k, x, offset):
        P, s, G = self.num_point, self.up_factor, self.groups
        if self.fused:
            # one memory order for all tensors, the value's: a channels-last
            # model stays channels-last (the fused kernel serves that order)
            cl = not x.is_contiguous() and x.is_contiguous(memory_format=torch.channels_last)
            fmt = torch.channels_last if cl else torch.contiguous_format
            q, k, x, offset = (in_memory_order(t, fmt) for t in (q, k, x, offset))
            try:
                return deform_sapa_fused(q, k, x, offset, P, s, G)
            except _lib.SapaUnsupported:
                pass
            # not covered in this memory order (float64, more than 32 points,
            # channel counts that are no multiple of 4 ...) or at all (more than 64
            # points): contiguous tensors, then the separate operators
            q, k, x, offset = (in_memory_order(t, torch.contiguous_format) for t in (q, k, x, offset))
            try:
                out = deform_sapa_fused(q, k, x, offset, P, s, G)
            except _lib.SapaUnsupported:
                attn = F.softmax(deform_qk(q, k, offset, P, s, G), dim=2)
                out = deform_av(attn, x, offset, P, s, G)
            return in_memory_order(out, fmt)
        # the separate operators take contiguous tensors only
        q, k, x, offset = (in_memory_order(t, torch.contiguous_format) for t in (q, k, x, offset))
        attn = F.softmax(deform_qk(q, k, offset, P, s, G), dim=2)
        return deform_av(attn, x, offset, P, s, G)
