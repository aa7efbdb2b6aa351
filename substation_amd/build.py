"""Builds libsubstation_amd.so (HIP, gfx950 only) in-tree with hipcc.

    python -m substation_amd.build

The library is prebuilt once; unlike the reference, which shells out to nvcc for
every new configuration (pytorch_module/encoder.py:378-390), nothing is compiled
when an Encoder is constructed.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
OBJ = os.path.join(CSRC, 'build')
LIB_DIR = os.path.join(HERE, 'lib')
LIB = os.path.join(LIB_DIR, 'libsubstation_amd.so')
SOURCES = ['encoder.hip', 'k_rows.hip', 'k_elem.hip', 'k_cols.hip', 'k_lnbwd.hip', 'k_attn.hip', 'k_mha.hip', 'k_relayout.hip', 'k_probe.hip', 'k_gemm.hip']
FLAGS = ['--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC', '-Wall', '-Wno-unused-function',
         # packed-fp32 VALU forms are switched off for every kernel of this library
         '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops']
# The attention kernels work on the MFMA results with vector instructions right
# away: keep those results in ordinary vector registers (the default puts them
# in accumulator registers and copies every value out and back in).
EXTRA_FLAGS = {'k_mha.hip': ['-mllvm', '-amdgpu-mfma-vgpr-form=1']}


def _hipcc():
    for cand in (os.environ.get('HIPCC'), '/opt/rocm/bin/hipcc', 'hipcc'):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return 'hipcc'


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = '\n'.join(l for l in r.stdout.splitlines()
                    if 'packed-fp32-ops' not in l and 'is not a recognized feature' not in l)
    if r.returncode != 0:
        raise RuntimeError('command failed: ' + ' '.join(cmd) + '\n' + out)
    return out


def build(verbose=False, jobs=8):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = _hipcc()

    def compile_one(src):
        obj = os.path.join(OBJ, src.replace('.hip', '.o'))
        out = _run([hipcc, *FLAGS, *EXTRA_FLAGS.get(src, []), '-c', os.path.join(CSRC, src), '-o', obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    _run([hipcc, '--offload-arch=gfx950', '-shared', '-fPIC', *objs, '-o', LIB])
    return LIB


if __name__ == '__main__':
    print(build(verbose='-v' in sys.argv))
