"""Builds ``cabi_gpu_check``, the plain-C caller of ``libmlora.so`` that ``tests/test_gpu_cabi_program.py`` runs:
gcc over the HIP runtime API header and ``include/mlora.h``, linked against the library where it lies in the tree."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
SRC = os.path.join(HERE, "cabi_gpu_check.c")
EXE = os.path.join(HERE, "cabi_gpu_check")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


def build() -> str:
    cmd = ["gcc", "-std=c99", "-O1", "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__", f"-I{ROCM}/include",
           f"-I{os.path.join(ROOT, 'include')}", SRC, "-o", EXE, f"-L{os.path.join(ROOT, 'valora_amd')}", "-lmlora",
           f"-L{ROCM}/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN/../../valora_amd", f"-Wl,-rpath,{ROCM}/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("gcc failed on tests/cabi/cabi_gpu_check.c:\n" + r.stderr)
    return EXE


if __name__ == "__main__":
    print(build())
