"""Writes tests/golden/sapa_golden.npz: seeded inputs and the outputs of this
repository's own CPU oracle (oracle/sapa_oracle.c in the reference kernels'
fp32 arithmetic, float64 where noted).  The reference ships no golden vectors
for this path, and nothing of the reference is read or run here.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import c_oracle as O  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'sapa_golden.npz')


def main():
    g = torch.Generator().manual_seed(20240521)
    r = lambda *s: torch.randn(*s, generator=g)
    d = {}
    # SAPA-B: B, d, C, H, W, K, s  (ragged against the 16x16 / 16x8 tiles)
    for tag, (B, dd, C, H, W, K, s) in {
        'b_k5s2': (2, 6, 5, 9, 19, 5, 2),
        'b_k3s3': (1, 4, 3, 5, 6, 3, 3),
        'b_k7s1': (1, 3, 2, 6, 7, 7, 1),
    }.items():
        q, key, v = r(B, dd, H * s, W * s), r(B, dd, H, W), r(B, C, H, W)
        attn = r(B, K * K, H * s, W * s)
        d[f'{tag}.cfg'] = np.array([B, dd, C, H, W, K, s])
        d[f'{tag}.q'], d[f'{tag}.key'], d[f'{tag}.v'], d[f'{tag}.attn'] = (
            t.numpy() for t in (q, key, v, attn))
        d[f'{tag}.qk'] = O.qk(q, key, K, s, 'f32').numpy()
        d[f'{tag}.av'] = O.av(attn, v, K, s, 'f32').numpy()
        d[f'{tag}.fused'] = O.sapa_fused(q, key, v, K, s, 'f32').numpy()
        d[f'{tag}.fused64'] = O.sapa_fused(q, key, v, K, s, 'f32a64').numpy()
    # SAPA-D: B, G, dq, cg, H, W, P, s
    for tag, (B, G, dq, cg, H, W, P, s) in {
        'd_p5s2': (2, 4, 2, 3, 7, 9, 5, 2),
        'd_p9s1': (1, 2, 3, 2, 5, 5, 9, 1),
    }.items():
        q, key, v = r(B, G * dq, H * s, W * s), r(B, G * dq, H, W), r(B, G * cg, H, W)
        off = r(B, 2 * G * P, H * s, W * s) * 1.5
        attn = r(B, G, P, H * s, W * s)
        d[f'{tag}.cfg'] = np.array([B, G, dq, cg, H, W, P, s])
        d[f'{tag}.q'], d[f'{tag}.key'], d[f'{tag}.v'], d[f'{tag}.off'], d[f'{tag}.attn'] = (
            t.numpy() for t in (q, key, v, off, attn))
        d[f'{tag}.dqk'] = O.deform_qk(q, key, off, P, s, G, 'f32').numpy()
        d[f'{tag}.dav'] = O.deform_av(attn, v, off, P, s, G, 'f32').numpy()
        d[f'{tag}.dfused'] = O.deform_sapa_fused(q, key, v, off, P, s, G, 'f32').numpy()
    np.savez_compressed(OUT, **d)
    print(OUT, os.path.getsize(OUT), 'bytes')


if __name__ == '__main__':
    main()
