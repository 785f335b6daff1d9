"""Builds libasdl_amd.so (every HIP source under csrc/) for gfx950 with hipcc, in-tree."""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
LIB_DIR = os.path.join(HERE, 'lib')
LIB_PATH = os.path.join(LIB_DIR, 'libasdl_amd.so')

HIPCC = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
FLAGS = ['--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC', '-fno-gpu-rdc',
         '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
         '-Wno-unused-result', '-Wno-unknown-attributes', '-Wno-align-mismatch']


def sources():
    return sorted(glob.glob(os.path.join(CSRC, '*.hip')))


def build(verbose=True, jobs=8):
    """AK_TUNING_HOOKS=1 in the environment adds the ak_debug_set_* / ak_debug_force_* setters (tuning runs only)."""
    flags = FLAGS + (['-DAK_TUNING_HOOKS'] if os.environ.get('AK_TUNING_HOOKS') == '1' else [])
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(LIB_DIR, 'obj')
    os.makedirs(obj_dir, exist_ok=True)
    procs = []
    objs = []
    for src in sources():
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + '.o')
        objs.append(obj)
        cmd = [HIPCC] + flags + ['-c', src, '-o', obj]
        if verbose:
            print(' '.join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        while sum(p.poll() is None for _, p in procs) >= jobs:
            procs[0][1].wait()
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = '\n'.join(l for l in out.splitlines() if 'packed-fp32-ops' not in l and l.strip())
        if p.returncode != 0:
            failed = True
            print(f'FAILED {src}\n{out}', file=sys.stderr)
        elif verbose and out:
            print(out)
    if failed:
        raise RuntimeError('hipcc failed')
    cmd = [HIPCC, '--offload-arch=gfx950', '-shared', '-fPIC', '-o', LIB_PATH] + objs
    if verbose:
        print(' '.join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB_PATH


if __name__ == '__main__':
    build()
