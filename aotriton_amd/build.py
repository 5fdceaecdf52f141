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
    # the ILP-first scheduling strategy: dK/dV kernel of the headline shape -1..2 % (same-box A/B,
    # no spills either way); level on the forward and the dQ-from-dS kernel, which keep the default
    'fa_bwd_dkdv_d128.hip': ['-mllvm', '-amdgpu-sched-strategy=max-ilp'],
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
    hs.append(os.path.join(ROOT, 'include', 'aotriton_amd', 'probe.h'))
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


_WATERFALL = re.compile(r'v_readfirstlane_b32[^\n]*\n(?:[^\n]*\n){0,24}?[^\n]*s_and_saveexec_b64[^\n]*\n'
                        r'(?:[^\n]*\n){0,24}?[^\n]*buffer_(?:load|store)[^\n]*\n(?:[^\n]*\n){0,4}?'
                        r'[^\n]*s_xor_b64 exec, exec[^\n]*\n[^\n]*s_cbranch_execnz')


def scan(jobs=8):
    """Compiles every kernel file to assembly and reports per-descriptor loops around buffer
    accesses ("waterfall" loops: readfirstlane, compare, masked issue, repeat while lanes are left).
    The compiler emits them when it takes a buffer descriptor for divergent, e.g. one built from
    threadIdx.x >> 6.  They cost time, and hipcc 7.2 has placed a register spill in the block such
    a loop exits to, before exec is restored: the store runs with no lane enabled and the reload
    later returns whatever the slot held.  The kernels here are written so that none is emitted;
    returns the list of (file, loops, functions left out of line) that have some of either."""
    import tempfile
    tmpdir = tempfile.TemporaryDirectory(prefix='fa_scan_')
    tmp = tmpdir.name

    def one(unit):
        src, defines, objname = unit
        if not src.endswith('.hip'):
            return src, 0, 0
        out = os.path.join(tmp, objname + '.s')
        cmd = [HIPCC] + COMMON + EXTRA.get(src, []) + defines + ['-x', 'hip', '--cuda-device-only', '-S',
                                                                 os.path.join(CSRC, src), '-o', out]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError('hipcc failed on ' + src)
        text = open(out).read()
        # a device function left out of line (a lambda the inliner gave up on) keeps its captures in
        # memory and reads them back with flat loads; every kernel here is meant to be one function
        outlined = len(re.findall(r'^\s*\.type\s+\S+,@function', text, re.M)) - text.count('.amdhsa_kernel ')
        return objname, len(_WATERFALL.findall(text)), outlined

    with tmpdir, concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        return [(n, c, o) for n, c, o in ex.map(one, sources()) if c or o]


if __name__ == '__main__':
    ap = argparse.ArgumentParser()
    ap.add_argument('-j', type=int, default=8)
    ap.add_argument('--force', action='store_true')
    ap.add_argument('--scan', action='store_true', help='compile to assembly and look for per-descriptor loops')
    a = ap.parse_args()
    if a.scan:
        found = scan(a.j)
        print('per-descriptor loops / functions left out of line:', found if found else 'none')
        sys.exit(1 if found else 0)
    print(build(a.j, a.force))
