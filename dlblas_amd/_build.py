"""Builds the HIP shared library of this package for gfx950 with hipcc (in-tree, next to this file)."""
import os
import shutil
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(PKG_DIR, 'csrc')
LIB_NAME = 'libdlblas_fp8_gemm.so'
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)
SOURCES = ['dlblas_fp8_gemm.hip', 'dlblas_fp8_moe.hip']

# packed fp32 VALU forms are switched off for every device compile of this library
HIPCC_FLAGS = [
    '-O3', '-std=c++17', '--offload-arch=gfx950', '-shared', '-fPIC', '-Xclang', '-target-feature', '-Xclang',
    '-packed-fp32-ops', '-mllvm', '-amdgpu-mfma-vgpr-form=1', '-Wall', '-Wno-unused-function'
]


def find_hipcc() -> str:
    for cand in (os.environ.get('HIPCC'), shutil.which('hipcc'), '/opt/rocm/bin/hipcc'):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError('hipcc not found (set HIPCC or put /opt/rocm/bin on PATH)')


def build_library(verbose: bool = False, defines=(), out_path: str = LIB_PATH) -> str:
    """Compile csrc/*.hip into libdlblas_fp8_gemm.so; always recompiles. Returns the library path.
    `defines` / `out_path`: measurement builds kept apart from the library (the DLB_ABLATE_* switches of the ring kernels'
    K step, loaded through the DLBLAS_AMD_LIB environment variable)."""
    cmd = [find_hipcc()] + HIPCC_FLAGS + [f'-D{d}' for d in defines] + ['-o', out_path] + [os.path.join(CSRC_DIR, s) for s in SOURCES]
    res = subprocess.run(cmd, cwd=CSRC_DIR, capture_output=True, text=True)
    log = '\n'.join(line for line in (res.stdout + res.stderr).splitlines() if 'packed-fp32-ops' not in line)
    if res.returncode != 0:
        raise RuntimeError(f'hipcc failed ({res.returncode}):\n{log}')
    if verbose and log.strip():
        print(log)
    return out_path


if __name__ == '__main__':
    import argparse
    ap = argparse.ArgumentParser()
    ap.add_argument('--define', action='append', default=[], help='preprocessor symbol of a measurement build, e.g. DLB_ABLATE_VMCNT')
    ap.add_argument('--out', default=LIB_PATH, help='output path (default: the library next to this file)')
    a = ap.parse_args()
    print(build_library(verbose=True, defines=a.define, out_path=a.out))
