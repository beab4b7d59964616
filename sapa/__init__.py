"""Drop-in for the reference's `sapa` package (sapa/sapa/__init__.py:1-3):
`from sapa import qk, av` resolves to the MI355X HIP operators."""
from sapa_amd.sapa_func import av, qk, qk_softmax, sapa_fused, softmax_k

__all__ = ['qk', 'av', 'sapa_fused', 'qk_softmax', 'softmax_k']
