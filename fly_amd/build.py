"""Build step: compiles the HIP sources under ``csrc/`` for gfx950 into ``libflyhip.so`` next to
this file.  Run as ``python -m fly_amd.build``; hipcc cross-compiles without a GPU."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
LIB = os.path.join(HERE, 'libflyhip.so')
SOURCES = ['api.cpp', 'sblocal.hip', 'sblocal_prep.hip', 'blocksparse.hip']
# packed-fp32 VALU forms are switched off for every kernel of this library; MFMA accumulators stay in
# ordinary VGPRs (the softmax arithmetic reads them between products, and every trip through the
# accumulation registers costs a move per value)
FLAGS = ['--offload-arch=gfx950', '-O3', '-fPIC', '-std=c++17',
         '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
         '-mllvm', '-amdgpu-mfma-vgpr-form=1']


def _hipcc():
    for cand in (os.environ.get('HIPCC'), '/opt/rocm/bin/hipcc', 'hipcc'):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError('hipcc not found')


def build(verbose=False):
    hipcc = _hipcc()
    # extra compiler flags for measurement builds (e.g. -DFLY_BF16_WIDE=0: the 16-queries-per-wave bfloat16 band kernel everywhere)
    extra = os.environ.get('FLYHIP_EXTRA_FLAGS', '').split()
    objdir = os.path.join(HERE, 'build')
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(objdir, os.path.splitext(src)[0] + '.o')
        cmd = [hipcc] + FLAGS + extra + ['-x', 'hip', '-c', os.path.join(CSRC, src), '-o', obj]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f'hipcc failed on {src}:\n{res.stderr}')
        if verbose:
            print(' '.join(cmd))
        return obj

    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    cmd = [hipcc, '--offload-arch=gfx950', '-shared', '-fPIC', '-o', LIB] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f'link failed:\n{res.stderr}')
    return LIB


if __name__ == '__main__':
    print(build(verbose='-v' in sys.argv))
