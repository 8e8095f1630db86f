"""Build step: compile kerops_amd/csrc/*.hip for gfx950 into kerops_amd/_C/libkerops_hip.so.

    python -m kerops_amd.build            # compile every source, link
    python -m kerops_amd.build --verbose

hipcc cross-compiles without a GPU.  Packed-fp32 instructions are disabled for all
device code (-Xclang -target-feature -Xclang -packed-fp32-ops).  The library has
no libtorch / C++-ABI dependency; it needs only the HIP runtime, which the process
that loads it (PyTorch-ROCm) has already mapped.
"""
import argparse
import glob
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
OUT_DIR = os.path.join(HERE, '_C')
OBJ_DIR = os.path.join(OUT_DIR, 'obj')
LIB_PATH = os.path.join(OUT_DIR, 'libkerops_hip.so')

ARCH = 'gfx950'
HIPCC = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
COMMON_FLAGS = [
    '-O3', '-std=c++17', '-fPIC', f'--offload-arch={ARCH}',
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    # a*b+c is fused only where the source says fmaf: the quantisers and the backward
    # formulas are defined step by step in IEEE fp32
    '-ffp-contract=off',
    '-Wno-unused-command-line-argument',
]
# Extra flags per source file.  The load/store optimizer pairs 8-byte LDS reads into ds_read2_b64, which gfx950 runs
# at a fraction of the rate of two ds_read_b64: the kernels that read their operands 8 bytes wide are built without it.
PER_FILE_FLAGS = {
    'dwconv_wgrad_dma.hip': ['-Xclang', '-target-feature', '-Xclang', '-load-store-opt'],
    'dwconv_bwd_dma.hip': ['-Xclang', '-target-feature', '-Xclang', '-load-store-opt'],
}


def sources():
    return sorted(glob.glob(os.path.join(CSRC, '*.hip')))


def _compile(src, verbose):
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + '.o')
    cmd = [HIPCC] + COMMON_FLAGS + PER_FILE_FLAGS.get(os.path.basename(src), []) + ['-c', src, '-o', obj]
    if verbose:
        print(' '.join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    err = '\n'.join(l for l in res.stderr.splitlines() if 'packed-fp32-ops' not in l and 'load-store-opt' not in l)
    if res.returncode != 0:
        raise RuntimeError(f'hipcc failed for {src}:\n{err}')
    if verbose and err.strip():
        print(err)
    return obj


def build(verbose=False, jobs=None):
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f'no .hip sources under {CSRC}')
    jobs = jobs or min(len(srcs), os.cpu_count() or 1, 8)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, verbose), srcs))
    cmd = [HIPCC, '-shared', '-fPIC', f'--offload-arch={ARCH}', '-o', LIB_PATH] + objs
    if verbose:
        print(' '.join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB_PATH


if __name__ == '__main__':
    ap = argparse.ArgumentParser()
    ap.add_argument('--verbose', action='store_true')
    ap.add_argument('-j', '--jobs', type=int, default=None)
    args = ap.parse_args()
    print(build(verbose=args.verbose, jobs=args.jobs))
