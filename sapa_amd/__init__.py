"""SAPA upsampling operators for AMD MI355X (gfx950): hand-written HIP
kernels behind the reference's Python autograd API.

    from sapa_amd import qk, av, sapa_fused                 # SAPA-B
    from sapa_amd import deform_qk, deform_av, deform_sapa_fused  # SAPA-D
    from sapa_amd import SAPA, SAPADeform                   # nn.Modules

The top-level `sapa` and `deformsapa` packages re-export the operators under
the reference's import paths.
"""
from .deform_func import (DeformAVFunction, DeformQKFunction, DeformSAPAFusedFunction,
                          deform_av, deform_qk, deform_sapa_fused)
from .modules import SAPA, SAPADeform
from .sapa_func import (AVFunction, QKFunction, SAPAFusedFunction, av, qk, qk_softmax,
                        sapa_fused, softmax_k)

__all__ = ['qk', 'av', 'sapa_fused', 'qk_softmax', 'softmax_k', 'deform_qk', 'deform_av',
           'deform_sapa_fused', 'SAPA', 'SAPADeform', 'QKFunction', 'AVFunction',
           'SAPAFusedFunction', 'DeformQKFunction', 'DeformAVFunction',
           'DeformSAPAFusedFunction']
