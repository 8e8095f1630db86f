"""Build step for the CPU oracle (test infrastructure, never the product path).

`python oracle/build_oracle.py` compiles oracle/kerops_oracle.c with gcc into
oracle/_build/liboracle.so.  -ffp-contract=off keeps every fp32 step of the
quantisers a separate IEEE operation; no -march flag is used so the library
runs on whatever host the tree is copied to.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, 'kerops_oracle.c')
OUT_DIR = os.path.join(HERE, '_build')
OUT = os.path.join(OUT_DIR, 'liboracle.so')


def build(verbose=False):
    os.makedirs(OUT_DIR, exist_ok=True)
    cmd = [
        'gcc', '-O2', '-fopenmp', '-fPIC', '-shared', '-std=c11',
        '-ffp-contract=off', '-fno-fast-math', '-Wall', '-Wextra',
        SRC, '-o', OUT, '-lm',
    ]
    if verbose:
        print(' '.join(cmd))
    subprocess.run(cmd, check=True)
    return OUT


if __name__ == '__main__':
    print(build(verbose=True))
    sys.exit(0)
