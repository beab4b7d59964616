"""CPU: the committed golden vectors are what the oracle computes today, and
the two oracle implementations agree on them."""
import torch

from helpers import assert_f32_close, golden
from oracle import torch_oracle as T


def t(a):
    return torch.from_numpy(a)


def test_golden_sapa_b(coracle):
    G = golden()
    for tag in ('b_k5s2', 'b_k3s3', 'b_k7s1'):
        B, d, C, H, W, K, s = (int(v) for v in G[f'{tag}.cfg'])
        q, key, v, attn = (t(G[f'{tag}.{n}']) for n in ('q', 'key', 'v', 'attn'))
        assert torch.equal(coracle.qk(q, key, K, s, 'f32'), t(G[f'{tag}.qk']))
        assert torch.equal(coracle.av(attn, v, K, s, 'f32'), t(G[f'{tag}.av']))
        assert_f32_close(coracle.sapa_fused(q, key, v, K, s, 'f32'), t(G[f'{tag}.fused']), tag)
        # library-routine restatement in float64 against the stored float64 value
        want = T.sapa_fused(q.double(), key.double(), v.double(), K, s)
        torch.testing.assert_close(t(G[f'{tag}.fused64']), want, rtol=1e-11, atol=1e-12)
        assert_f32_close(t(G[f'{tag}.fused']), want, tag)
        assert_f32_close(t(G[f'{tag}.qk']), T.qk(q.double(), key.double(), K, s), tag)


def test_golden_sapa_d(coracle):
    G = golden()
    for tag in ('d_p5s2', 'd_p9s1'):
        B, Gr, dq, cg, H, W, P, s = (int(v) for v in G[f'{tag}.cfg'])
        q, key, v, off, attn = (t(G[f'{tag}.{n}']) for n in ('q', 'key', 'v', 'off', 'attn'))
        assert torch.equal(coracle.deform_qk(q, key, off, P, s, Gr, 'f32'), t(G[f'{tag}.dqk']))
        assert torch.equal(coracle.deform_av(attn, v, off, P, s, Gr, 'f32'), t(G[f'{tag}.dav']))
        assert_f32_close(coracle.deform_sapa_fused(q, key, v, off, P, s, Gr, 'f32'),
                         t(G[f'{tag}.dfused']), tag)
        want = T.deform_qk(q.double(), key.double(), off.double(), P, s, Gr)
        torch.testing.assert_close(t(G[f'{tag}.dqk']).double(), want, rtol=1e-4, atol=1e-5)
        want = T.deform_sapa_fused(q.double(), key.double(), v.double(), off.double(), P, s, Gr)
        torch.testing.assert_close(t(G[f'{tag}.dfused']).double(), want, rtol=1e-4, atol=1e-5)
