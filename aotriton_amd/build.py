"""Builds libaotriton_amd.so in-tree with hipcc for gfx950 (cross-compiles without a GPU).

Usage: python -m aotriton_amd.build [-j N] [--force]
"""
import argparse
import concurrent.futures
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
ROOT = os.path.dirname(HERE)
OBJ = os.path.join(CSRC, 'obj')
LIB = os.path.join(HERE, 'libaotriton_amd.so')
HIPCC = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')

COMMON = [
    '--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC', '-fvisibility=hidden',
    '-I', os.path.join(ROOT, 'include'), '-I', CSRC,
    # packed fp32 VALU ops are kept off on this target
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    '-Wno-unused-command-line-argument',
]


# Per-file additions.  The dQ kernels post-process MFMA results with the vector ALU; letting
# the register allocator keep those results in VGPRs saves the AGPR read per element.
EXTRA = {
    'fa_bwd_dq_d64.hip': ['-mllvm', '-amdgpu-mfma-vgpr-form'],
    'fa_bwd_dq_d128.hip': ['-mllvm', '-amdgpu-mfma-vgpr-form'],
}

# The per-head-dim kernel files are compiled a second time with FA_PADDED=1: the copies that
# serve head dims rounded up to the compiled one.
PADDED_RE = re.compile(r'fa_(fwd|bwd_dkdv|bwd_dq|bwd_fused)_d\d+\.hip$')


def sources():
    """(source file, extra defines, object name) per compilation."""
    out = []
    for f in sorted(os.listdir(CSRC)):
        if not (f.endswith('.hip') or f.endswith('.cpp')):
            continue
        out.append((f, [], f + '.o'))
        if PADDED_RE.match(f):
            out.append((f, ['-DFA_PADDED=1'], f + '.padded.o'))
    return out


def headers():
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith('.h')]
    hs.append(os.path.join(ROOT, 'include', 'aotriton_amd', 'flash.h'))
    return hs


def _compile(unit, force):
    src, defines, objname = unit
    obj = os.path.join(OBJ, objname)
    path = os.path.join(CSRC, src)
    newest = max(os.path.getmtime(p) for p in [path] + headers())
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= newest:
        return obj, '', 0
    cmd = [HIPCC] + COMMON + EXTRA.get(src, []) + defines + ['-x', 'hip', '-c', path, '-o', obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the packed-fp32 feature name; that note is noise
    err = '\n'.join(l for l in r.stderr.splitlines() if 'packed-fp32-ops' not in l)
    return obj, err, r.returncode


def build(jobs=8, force=False, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    objs = []
    failed = False
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for obj, err, rc in ex.map(lambda s: _compile(s, force), srcs):
            objs.append(obj)
            if err.strip() and (rc != 0 or verbose):
                sys.stderr.write(err + '\n')
            failed |= rc != 0
    if failed:
        raise RuntimeError('hipcc failed')
    cmd = [HIPCC, '--offload-arch=gfx950', '-shared', '-fPIC', '-o', LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stderr)
        raise RuntimeError('link failed')
    return LIB


if __name__ == '__main__':
    ap = argparse.ArgumentParser()
    ap.add_argument('-j', type=int, default=8)
    ap.add_argument('--force', action='store_true')
    a = ap.parse_args()
    print(build(a.j, a.force))
