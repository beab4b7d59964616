"""Library-routine restatement of SAPA's operators on the CPU (torch).

TEST INFRASTRUCTURE ONLY -- see oracle/__init__.py.  This is the "unfold-based
PyTorch math" of the reference's own forward checks, restated:

  * qk / av           follow sapa/sapa/forward_check.py:9-24 (F.unfold + einsum)
  * softmax axis      follows sapa_base.py:39 (dim=1 over K*K) and
                      sapa_deform.py:52 (dim=2 over the P points of a group)
  * sampled variants  follow deformsapa/deformsapa/forward_check.py:6-40
                      (F.grid_sample, bilinear, zero padding,
                      align_corners=False)

Every function works in the dtype of its inputs; pass float64 tensors for a
high-precision value.  It is also the CPU baseline that bench.py times.

Tensor names use the shapes, not the reference's letters: `q` is the
high-res query [B,d,sH,sW]; `key`/`value` are low-res [B,d|C,H,W].
"""
import torch
import torch.nn.functional as F


def _windows(low, K):
    """[B,C,H,W] -> [B,C,K*K,H,W]: the zero-padded KxK neighbourhood of every
    low-res cell, neighbour index k = ky*K + kx (row offset major), which is
    both F.unfold's ordering and the kernels' (qk_cuda_kernel.cu:50-53)."""
    B, C, H, W = low.shape
    return F.unfold(low, kernel_size=K, padding=K // 2).reshape(B, C, K * K, H, W)


def qk(q, key, K, s):
    """logits[b,k,ph,pw] = sum_c key[b,c,ph//s-r+ky,pw//s-r+kx] * q[b,c,ph,pw],
    out-of-range neighbours count as zero (forward_check.py:9-15,
    qk_cuda_kernel.cu:55-66)."""
    B, d, H, W = key.shape
    assert q.shape == (B, d, H * s, W * s)
    win = _windows(key, K)                       # b c k h w
    q6 = q.reshape(B, d, H, s, W, s)             # b c h i w j
    out = torch.einsum('bchiwj,bckhw->bkhiwj', q6, win)
    return out.reshape(B, K * K, H * s, W * s)


def av(attn, value, K, s):
    """out[b,c,ph,pw] = sum_k value[b,c,ph//s-r+ky,pw//s-r+kx] * attn[b,k,ph,pw]
    (forward_check.py:18-24, av_cuda_kernel.cu:56-73)."""
    B, C, H, W = value.shape
    assert attn.shape == (B, K * K, H * s, W * s)
    win = _windows(value, K)
    a6 = attn.reshape(B, K * K, H, s, W, s)
    out = torch.einsum('bkhiwj,bckhw->bchiwj', a6, win)
    return out.reshape(B, C, H * s, W * s)


def sapa_fused(q, key, value, K, s):
    """qk -> softmax over the K*K axis -> av (sapa_base.py:38-40)."""
    return av(F.softmax(qk(q, key, K, s), dim=1), value, K, s)


def _sample(low, offset, P, s, G):
    """Bilinear samples of every group of `low` at parent + offset.

    low [B,G*cg,H,W], offset [B,2*G*P,sH,sW] with channel 2*(g*P+p) = dx and
    +1 = dy in low-res pixels (deform_qk_cuda_kernel.cu:172-183).  Returns
    [B,G,P,cg,sH,sW].  The sample position of query (ph,pw) is
    (ph//s + dy, pw//s + dx) in pixel-index coordinates; grid_sample with
    align_corners=False puts index i at normalised (2i+1)/N - 1.
    """
    B, C, H, W = low.shape
    cg = C // G
    sH, sW = H * s, W * s
    off = offset.reshape(B, G, P, 2, sH, sW)
    py = (torch.arange(sH) // s).to(low.dtype).view(1, 1, 1, sH, 1)
    px = (torch.arange(sW) // s).to(low.dtype).view(1, 1, 1, 1, sW)
    gx = (2 * (px + off[:, :, :, 0]) + 1) / W - 1      # B G P sH sW
    gy = (2 * (py + off[:, :, :, 1]) + 1) / H - 1
    grid = torch.stack((gx, gy), dim=-1)               # B G P sH sW 2
    src = low.reshape(B * G, cg, H, W)
    out = low.new_empty(B, G, P, cg, sH, sW)
    for p in range(P):
        smp = F.grid_sample(src, grid[:, :, p].reshape(B * G, sH, sW, 2),
                            mode='bilinear', padding_mode='zeros',
                            align_corners=False)
        out[:, :, p] = smp.reshape(B, G, cg, sH, sW)
    return out


def deform_qk(q, key, offset, P, s, G):
    """out[b,g,p,qh,qw] = sum_{c<d} q[b,g*d+c,qh,qw] * bilinear(key[b,g*d+c])
    (deformsapa/forward_check.py:19-26, deform_qk_cuda_kernel.cu:151-196)."""
    B, C, sH, sW = q.shape
    d = C // G
    smp = _sample(key, offset, P, s, G)                # B G P d sH sW
    return (q.reshape(B, G, 1, d, sH, sW) * smp).sum(dim=3)


def deform_av(attn, value, offset, P, s, G):
    """out[b,c,qh,qw] = sum_p attn[b,g(c),p,qh,qw] * bilinear(value[b,c]),
    g(c) = c // (C/G) (deformsapa/forward_check.py:29-38,
    deform_av_cuda_kernel.cu:151-194)."""
    B, C, H, W = value.shape
    smp = _sample(value, offset, P, s, G)              # B G P cg sH sW
    out = (attn.unsqueeze(3) * smp).sum(dim=2)         # B G cg sH sW
    return out.reshape(B, C, H * s, W * s)


def deform_sapa_fused(q, key, value, offset, P, s, G):
    """deform_qk -> softmax over the P axis -> deform_av (sapa_deform.py:51-53)."""
    attn = F.softmax(deform_qk(q, key, offset, P, s, G), dim=2)
    return deform_av(attn, value, offset, P, s, G)
