"""Drop-in for the reference's `deformsapa` package
(deformsapa/deformsapa/__init__.py:1-3): `from deformsapa import deform_qk,
deform_av` resolves to the MI355X HIP operators."""
from sapa_amd.deform_func import deform_av, deform_qk, deform_sapa_fused

__all__ = ['deform_qk', 'deform_av', 'deform_sapa_fused']
