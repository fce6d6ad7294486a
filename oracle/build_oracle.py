"""TEST INFRASTRUCTURE ONLY - compiles oracle/fp8_gemm_oracle.c with gcc into oracle/_build/."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
OUT_DIR = os.path.join(HERE, '_build')
LIB_PATH = os.path.join(OUT_DIR, 'libfp8_gemm_oracle.so')


def build_oracle() -> str:
    os.makedirs(OUT_DIR, exist_ok=True)
    cmd = ['gcc', '-O2', '-fno-fast-math', '-ffp-contract=off', '-shared', '-fPIC', '-o', LIB_PATH,
           os.path.join(HERE, 'fp8_gemm_oracle.c'), '-lm']
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f'gcc failed:\n{res.stdout}{res.stderr}')
    return LIB_PATH


if __name__ == '__main__':
    print(build_oracle())
