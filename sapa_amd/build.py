"""Builds libsapa_hip.so from sapa_amd/csrc/*.hip with hipcc for gfx950.

    python -m sapa_amd.build          # compile and link in-tree

The library lands in sapa_amd/lib/ so that it travels with the source tree.
Nothing is compiled at import time: sapa_amd loads what this step built.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
OBJ = os.path.join(CSRC, '_obj')
LIBDIR = os.path.join(HERE, 'lib')
LIB = os.path.join(LIBDIR, 'libsapa_hip.so')
SOURCES = ['capi.hip', 'sapa_b_generic.hip', 'sapa_b_tiled.hip', 'sapa_b_dot2.hip', 'sapa_b_wmat16.hip', 'sapa_b_nhwc.hip', 'sapa_b_nhwc_mm.hip', 'sapa_b_nhwc16.hip', 'sapa_b_nhwc_wm16.hip', 'sapa_b_mfma.hip', 'sapa_b_lowgrad.hip', 'sapa_d.hip', 'sapa_d_lowgrad.hip', 'sapa_d_nhwc.hip', 'sapa_d_wmat16.hip', 'sapa_d_backward.hip', 'sapa_d_bwdmat.hip', 'sapa_d_scatter.hip', 'sapa_moments.hip', 'sapa_project.hip', 'sapa_layout.hip', 'sapa_stream.hip',
           'sapa_d_lds.hip']

HIPCC = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
# packed-fp32 VALU ops are switched off for every kernel in this library
FLAGS = ['-O3', '-std=c++17', '--offload-arch=gfx950', '-fPIC', '-fno-gpu-rdc',
         '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
         '-Wall', '-Wno-unused-function']
# sapa_b_wmat16 / sapa_b_nhwc / sapa_b_nhwc_mm / sapa_b_nhwc16 / sapa_d_nhwc / sapa_d_wmat16 / sapa_d_bwdmat / sapa_d_scatter keep their MFMA accumulators in ordinary VGPRs: left to itself the
# compiler moves them to the accumulation registers on top of an already full
# VGPR budget, which costs the kernels a wave per SIMD
SOURCE_FLAGS = {'sapa_b_wmat16.hip': ['-mllvm', '-amdgpu-mfma-vgpr-form'],
                'sapa_b_nhwc_wm16.hip': ['-mllvm', '-amdgpu-mfma-vgpr-form'],
                'sapa_b_nhwc.hip': ['-mllvm', '-amdgpu-mfma-vgpr-form'],
                'sapa_b_nhwc_mm.hip': ['-mllvm', '-amdgpu-mfma-vgpr-form'],
                'sapa_b_nhwc16.hip': ['-mllvm', '-amdgpu-mfma-vgpr-form'],
                'sapa_d_nhwc.hip': ['-mllvm', '-amdgpu-mfma-vgpr-form'],
                'sapa_d_wmat16.hip': ['-mllvm', '-amdgpu-mfma-vgpr-form'],
                'sapa_d_bwdmat.hip': ['-mllvm', '-amdgpu-mfma-vgpr-form'],
                'sapa_d_scatter.hip': ['-mllvm', '-amdgpu-mfma-vgpr-form']}


def _compile(src, extra):
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + '.o')
    cmd = [HIPCC] + FLAGS + SOURCE_FLAGS.get(src, []) + extra + ['-c', os.path.join(CSRC, src), '-o', obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = '\n'.join(l for l in r.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if r.returncode != 0:
        raise RuntimeError(f'hipcc failed on {src}:\n{out}')
    return obj, out


def build(verbose=False, extra_flags=()):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 1)) as ex:
        results = list(ex.map(lambda s: _compile(s, list(extra_flags)), SOURCES))
    for _, out in results:
        if verbose and out.strip():
            print(out)
    cmd = [HIPCC, '--offload-arch=gfx950', '-shared', '-fPIC', '-o', LIB] + [o for o, _ in results]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f'link failed:\n{r.stdout}')
    return LIB


if __name__ == '__main__':
    print(build(verbose=True, extra_flags=sys.argv[1:]))
