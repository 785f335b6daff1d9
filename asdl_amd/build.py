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
         '-Wno-unused-result', '-Wno-unknown-attributes', '-Wno-align-mismatch',
         '-Rpass-analysis=kernel-resource-usage']
RESOURCE_REPORT = os.path.join(LIB_DIR, 'kernel_resources.txt')     # one line per kernel: registers, scratch, LDS


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
    report = []
    for src, p in procs:
        out, _ = p.communicate()
        report += _resource_lines(os.path.basename(src), out)
        out = '\n'.join(l for l in out.splitlines()
                        if 'packed-fp32-ops' not in l and 'kernel-resource-usage' not in l and l.strip())
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
    with open(RESOURCE_REPORT, 'w') as fh:
        fh.write('# file kernel VGPRs AGPRs scratch_bytes_per_lane occupancy_waves_per_simd lds_bytes\n')
        fh.write('\n'.join(report) + '\n')
    return LIB_PATH


def _resource_lines(src_name, compiler_output):
    """The compiler's per-kernel resource remarks as 'file kernel VGPRs AGPRs scratch occupancy lds' lines: a kernel
    that starts to spill (scratch > 0) after a change shows up here, and tests/test_host_cpu.py reads the file."""
    lines, cur = [], None
    for l in compiler_output.splitlines():
        if 'kernel-resource-usage' not in l or 'remark:' not in l:
            continue
        text = l.split('remark:', 1)[1].replace('[-Rpass-analysis=kernel-resource-usage]', '').strip()
        key, _, value = text.partition(':')
        key, value = key.strip(), value.strip()
        if key == 'Function Name':
            cur = dict(name=value)
        elif cur is not None:
            cur[key] = value
            if key == 'LDS Size [bytes/block]':
                lines.append(' '.join([src_name, cur['name'], cur.get('VGPRs', '?'), cur.get('AGPRs', '?'),
                                       cur.get('ScratchSize [bytes/lane]', '?'),
                                       cur.get('Occupancy [waves/SIMD]', '?'), value]))
                cur = None
    return lines


if __name__ == '__main__':
    build()
