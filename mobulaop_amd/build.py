"""Ahead-of-time build of the HIP launcher library for gfx950.

    python -m mobulaop_amd.build          # compile csrc/*.hip + opzoo/*/*.hip

One shared object, `csrc/libmobula_hip.so`, holds the runtime and every
operator's entry points.  It stays in the source tree (next to the code that
loads it).  Replaces the per-call JIT of the reference
(mobula/building/build.py:64-146) with one explicit hipcc invocation.
"""
import glob
import os
import shutil
import subprocess
import sys

from .config import config

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, 'csrc')
LIB_PATH = os.path.join(CSRC, 'libmobula_hip.so')


def sources():
    return sorted(glob.glob(os.path.join(CSRC, '*.hip')) +
                  glob.glob(os.path.join(_HERE, 'opzoo', '*', '*.hip')))


def hipcc_flags():
    flags = [
        '--offload-arch=' + config.OFFLOAD_ARCH, '-std=c++17', '-O3', '-fPIC', '-shared',
        # fp32 expressions are evaluated as written: no fused multiply-add unless
        # the source asks for one, IEEE division and square root.
        '-ffp-contract=off', '-fhip-fp32-correctly-rounded-divide-sqrt',
        # hardware fp32 atomic add on global and LDS memory
        '-munsafe-fp-atomics',
        # keep scalar fp32 code scalar (no packed-fp32 instruction selection)
        '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
        '-Wall', '-Wno-unused-function', '-Wno-unknown-warning-option',
        '-I' + CSRC,
        # modules compiled on load name the library by this, wherever the tree lies
        '-Wl,-soname,libmobula_hip.so',
    ]
    if config.DEBUG:
        flags.append('-g')
    return flags


def build_library(verbose=False):
    hipcc = shutil.which(config.HIPCC) or '/opt/rocm/bin/hipcc'
    if not os.path.exists(hipcc):
        raise RuntimeError('hipcc not found: the HIP launcher library cannot be built here')
    tmp = LIB_PATH + '.tmp.{}'.format(os.getpid())
    cmd = [hipcc] + hipcc_flags() + ['-o', tmp] + sources()
    if verbose or config.SHOW_BUILDING_COMMAND:
        print(' '.join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the packed-fp32 target feature: harmless
    noise = ("is not a recognized feature for this target", )
    log = '\n'.join(l for l in proc.stdout.splitlines() if not any(n in l for n in noise))
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise RuntimeError('hipcc failed:\n' + log)
    if verbose and log.strip():
        print(log)
    os.replace(tmp, LIB_PATH)  # atomic: concurrent loaders never see a partial file
    return LIB_PATH


if __name__ == '__main__':
    print(build_library(verbose=True))
    sys.exit(0)
