"""Builds libmoye_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python moye.jl_amd/build.py [--force]

Objects go to csrc/build/, the library next to the Python mirror as moye_hip/libmoye_hip.so.
"""
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "moye_hip", "libmoye_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

COMMON = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# source -> extra flags
SOURCES = {
    "capi.hip": [],
    "copy_kernels.hip": [],
    # the epilogue's alpha * acc + beta * c is two products and a sum, each rounded (the oracle composes it from axpby!):
    # never contracted into fused operations
    "gemm_mfma.hip": ["-ffp-contract=off"],
    "gemm_mfma128.hip": ["-ffp-contract=off"],
    "gemm_mfma256.hip": ["-ffp-contract=off"],
    "gemm_mfma256pp.hip": ["-ffp-contract=off"],
    "gemm_mfma256w4.hip": ["-ffp-contract=off"],
    "gemm_mfma_skinny.hip": ["-ffp-contract=off"],
    "mfma_ceiling.hip": [],
    "elementwise.hip": ["-ffp-contract=off"],      # axpby!: rounded products, unfused sum
    "gemm_universal.hip": ["-ffp-contract=off"],   # UniversalFMA: mul then add, never fused
    "layout_host.cpp": ["-x", "hip"],
    "tiled_host.cpp": ["-x", "hip"],
}


def _headers():
    return [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hpp", ".h"))] + \
        [os.path.join(HERE, "..", "include", "moye_hip.h")]


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(item, force):
    src, extra = item
    path = os.path.join(CSRC, src)
    obj = os.path.join(CSRC, "build", os.path.splitext(src)[0] + ".o")
    if not force and not _stale(obj, [path] + _headers()):
        return obj, ""
    cmd = [HIPCC] + COMMON + extra + ["-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "not a recognized feature for this target"
    err = "\n".join(l for l in (r.stdout + r.stderr).splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj, err


# Kernels whose MFMAs are inline assembly: the compiler does not know how long their results take, so any
# instruction of its own that touches an accumulator register next to them (a copy made by the register
# allocator, an epilogue read scheduled upwards) would read a value that is not there yet, silently.
ASM_MFMA_SOURCES = ["gemm_mfma256w4.hip"]


def check_accumulator_hazards(src, force=False):
    """Compile `src` to assembly and fail if, in any basic block that holds v_mfma instructions, something
    other than a v_mfma names an AccVGPR before the kernel's `MOYE_ACC_SETTLED` marker."""
    path = os.path.join(CSRC, src)
    asm = os.path.join(CSRC, "build", os.path.splitext(src)[0] + ".s")
    if not force and not _stale(asm, [path] + _headers()):
        return
    cmd = [HIPCC] + COMMON + SOURCES.get(src, []) + ["-S", "--cuda-device-only", path, "-o", asm]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc -S failed for %s:\n%s" % (src, r.stdout + r.stderr))
    fn, block, bad = None, [], []

    def flush():
        if fn and any("v_mfma" in c.split(";")[0] for _, c in block):
            settled = False
            for ln, c in block:
                settled = settled or "MOYE_ACC_SETTLED" in c
                code = c.split(";")[0]
                if "v_mfma" in code or settled:
                    continue
                if re.search(r"\ba(\[\d+:\d+\]|\d+)\b", code):
                    bad.append("%s:%d: %s   [%s]" % (os.path.basename(asm), ln, code.strip(), fn[:60]))
        del block[:]

    with open(asm) as f:
        for ln, line in enumerate(f, 1):
            m = re.match(r"^(_Z\w+):", line)
            if m:
                flush()
                fn = m.group(1)
                continue
            if fn is None:
                continue
            if re.match(r"^\.LBB\w+:", line):
                flush()
            block.append((ln, line))
            if re.search(r"\bs_(cbranch|branch|endpgm)", line):
                flush()
                if "s_endpgm" in line:
                    fn = None
    if bad:
        os.remove(asm)
        raise RuntimeError("accumulator registers are touched next to inline-assembly MFMAs:\n" + "\n".join(bad[:20]))


def build(force=False, verbose=True):
    os.makedirs(os.path.join(CSRC, "build"), exist_ok=True)
    items = [(s, f) for s, f in SOURCES.items() if os.path.exists(os.path.join(CSRC, s))]
    with ThreadPoolExecutor(max_workers=min(8, len(items))) as ex:
        results = list(ex.map(lambda it: _compile(it, force), items))
    for src in ASM_MFMA_SOURCES:
        check_accumulator_hazards(src, force)
    objs = [o for o, _ in results]
    for (src, _), (_, msg) in zip(items, results):
        if msg.strip() and verbose:
            print("[%s]\n%s" % (src, msg))
    if force or _stale(OUT, objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    return OUT


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
