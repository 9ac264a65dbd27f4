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
    "gemm_mfma256_atom32.hip": ["-ffp-contract=off"],
    "gemm_mfma256pp.hip": ["-ffp-contract=off"],
    "gemm_mfma256w4.hip": ["-ffp-contract=off"],
    "gemm_mfma256w4_majors.hip": ["-ffp-contract=off"],
    "gemm_mfma256w4_ops.hip": ["-ffp-contract=off"],
    "gemm_mfma256w4_persist.hip": ["-ffp-contract=off"],
    "gemm_mfma128w4.hip": ["-ffp-contract=off"],
    "gemm_mfma128w4_majors.hip": ["-ffp-contract=off"],
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
ASM_MFMA_SOURCES = ["gemm_mfma256w4.hip", "gemm_mfma256w4_majors.hip", "gemm_mfma256w4_ops.hip", "gemm_mfma256w4_persist.hip", "gemm_mfma128w4.hip", "gemm_mfma128w4_majors.hip"]


def check_accumulator_hazards(src, force=False):
    """Compile `src` to assembly and fail if, in any basic block that holds v_mfma instructions, something
    other than a v_mfma names an AccVGPR before the kernel's `MOYE_ACC_SETTLED` marker, or something other than a
    v_mfma or a fragment read (ds_read_b128, ds_read_b64_tr_b16, ds_read_b64_tr_b8, ds_read_b32) names a register that the fragment reads of such blocks
    write."""
    path = os.path.join(CSRC, src)
    asm = os.path.join(CSRC, "build", os.path.splitext(src)[0] + ".s")
    if not force and not _stale(asm, [path] + _headers()):
        return
    cmd = [HIPCC] + COMMON + SOURCES.get(src, []) + ["-S", "--cuda-device-only", path, "-o", asm]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc -S failed for %s:\n%s" % (src, r.stdout + r.stderr))
    with open(asm) as f:
        acc_bad, frag_bad = asm_mfma_hazards(f, os.path.basename(asm))
    if acc_bad:
        os.remove(asm)
        raise RuntimeError("accumulator registers are touched next to inline-assembly MFMAs:\n" + "\n".join(acc_bad[:20]))
    if frag_bad:
        os.remove(asm)
        raise RuntimeError("fragment registers of inline-assembly LDS reads are touched between the MFMAs:\n" + "\n".join(frag_bad[:20]))


# the LDS reads that fill MFMA operand fragments in these kernels: whole pieces, the transposing reads of M- / N-major
# 16-bit and 8-bit operands, single values of M- / N-major fp32 operands
FRAG_READ = re.compile(r"\s*ds_read_(?:b128|b64_tr_b16|b64_tr_b8|b32)\s+(v\[\d+:\d+\]|v\d+\b)")


def asm_mfma_hazards(lines, name="asm"):
    """The analysis of check_accumulator_hazards on the lines of an assembly listing: (accumulator findings, fragment
    findings), each a list of 'file:line: instruction [function]'."""
    fn, block, bad = None, [], []
    mfma_blocks = []   # (function, [(line number, text)]) of every block that holds MFMAs, for the fragment check below

    def flush():
        if fn and any("v_mfma" in c.split(";")[0] for _, c in block):
            mfma_blocks.append((fn, list(block)))
            settled = False
            for ln, c in block:
                settled = settled or "MOYE_ACC_SETTLED" in c
                code = c.split(";")[0]
                if "v_mfma" in code or settled:
                    continue
                if re.search(r"\ba(\[\d+:\d+\]|\d+)\b", code):
                    bad.append("%s:%d: %s   [%s]" % (name, ln, code.strip(), fn[:60]))
        del block[:]

    if True:
        for ln, line in enumerate(lines, 1):
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
    acc_bad, bad = bad, []
    # The fragment registers: written by inline-assembly ds_read_b128 whose results the compiler believes are there at
    # once; the kernel's own s_waitcnt come before the MFMAs that read them.  Anything else that names such a register
    # between the MFMAs (a copy made by the register allocator, a spill) could read it before the data has arrived.
    def vregs(text):
        out = set()
        for a, b in re.findall(r"\bv\[(\d+):(\d+)\]", text):
            out.update(range(int(a), int(b) + 1))
        out.update(int(a) for a in re.findall(r"\bv(\d+)\b", text))
        return out

    frags = {}
    for f, blk in mfma_blocks:
        for _, c in blk:
            code = c.split(";")[0]
            m = FRAG_READ.match(code)
            if m:
                frags.setdefault(f, set()).update(vregs(m.group(1)))
    # Per block: a register counts as a fragment from the block's start (the reads of an earlier block or trip may still
    # be in flight) until something other than a fragment read writes it (the fragment is dead then and the register has
    # a new owner); a fragment read makes it one again.
    no_dest = re.compile(r"\s*(global_store|buffer_store|ds_write|global_load_lds|s_|v_cmp|v_readfirstlane|v_readlane)")
    for f, blk in mfma_blocks:
        pending = set(frags.get(f, set()))
        settled = False
        for ln, c in blk:
            settled = settled or "MOYE_ACC_SETTLED" in c
            code = c.split(";")[0]
            if settled or not code.strip() or code.lstrip().startswith(".") or "v_mfma" in code:
                continue
            m = FRAG_READ.match(code)
            if m:
                pending |= vregs(m.group(1))
                continue
            ops = code.strip().split(None, 1)
            operands = ops[1].split(",") if len(ops) > 1 else []
            dest = set() if (no_dest.match(code) or not operands) else vregs(operands[0])
            srcs = vregs(",".join(operands[1:] if dest else operands))
            if srcs & pending:
                bad.append("%s:%d: %s   [%s]" % (name, ln, code.strip(), f[:60]))
            pending -= dest
    return acc_bad, bad


def build(force=False, verbose=True):
    os.makedirs(os.path.join(CSRC, "build"), exist_ok=True)
    items = [(s, f) for s, f in SOURCES.items() if os.path.exists(os.path.join(CSRC, s))]
    # (the hazard checks compile their sources to assembly: they run beside the object compiles, the longest jobs first)
    order = sorted(items, key=lambda it: it[0] not in ASM_MFMA_SOURCES)
    with ThreadPoolExecutor(max_workers=8) as ex:
        checks = [ex.submit(check_accumulator_hazards, src, force) for src in ASM_MFMA_SOURCES]
        compiled = dict(zip([it[0] for it in order], ex.map(lambda it: _compile(it, force), order)))
        for c in checks:
            c.result()
    results = [compiled[it[0]] for it in items]
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
