"""Builds the C oracle (oracle/_build/libmoye_oracle.so) with gcc.  Test infrastructure only.

No reference build exists beside it: the reference is Julia source with no C/C++ files, and no
Julia toolchain is present, so `oracle/_ref/` stays empty.
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "_build", "libmoye_oracle.so")


def build(force=False):
    src = os.path.join(HERE, "gemm_oracle.c")
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    if not force and os.path.exists(OUT) and os.path.getmtime(OUT) >= os.path.getmtime(src):
        return OUT
    cmd = ["gcc", "-O2", "-ffp-contract=off", "-fopenmp", "-shared", "-fPIC", "-o", OUT, src]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("gcc failed:\n" + r.stdout + r.stderr)
    return OUT


if __name__ == "__main__":
    print(build(force=True))
