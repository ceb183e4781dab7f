"""Build libkfac_hip.so (hand-written HIP for gfx950) in-tree with hipcc.

    python pytorch-sso_amd/build_ext.py

The library lands next to the Python package (torchsso/libkfac_hip.so) so that
it travels with the source tree; there is no JIT step at import time.
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
OUT = os.path.join(HERE, 'torchsso', 'libkfac_hip.so')

HIPCC_FLAGS = [
    '-O3', '-std=c++17', '--offload-arch=gfx950', '-fPIC', '-shared',
    # packed fp32 VALU forms are kept off for every kernel of this library
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    '-Wno-unused-command-line-argument',
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, '*.hip')))


def build(verbose=True):
    hipcc = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
    objs = []
    procs = []
    for src in sources():
        obj = src[:-4] + '.o'
        cmd = [hipcc] + [f for f in HIPCC_FLAGS if f != '-shared'] + ['-c', src, '-o', obj]
        if verbose:
            print(' '.join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        objs.append(obj)
    for src, p in procs:
        out, _ = p.communicate()
        text = out.decode(errors='replace')
        # hipcc's host pass says it does not know the packed-fp32 feature: harmless
        text = '\n'.join(l for l in text.splitlines() if 'packed-fp32-ops' not in l)
        if p.returncode != 0:
            raise RuntimeError('hipcc failed on %s:\n%s' % (src, text))
        if verbose and text.strip():
            print(text)
    cmd = [hipcc, '--offload-arch=gfx950', '-shared', '-fPIC'] + objs + ['-o', OUT]
    if verbose:
        print(' '.join(cmd), flush=True)
    subprocess.check_call(cmd)
    return OUT


if __name__ == '__main__':
    build()
    sys.exit(0)
