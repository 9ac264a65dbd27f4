"""Device loops behind the C ABI: copyto! and gemm! on flattened descriptors."""
import ctypes as C

from . import _lib
from ._lib import TiledCopy, TiledMMA, check, lib


def version():
    return lib().moye_version().decode()


def device_info():
    name = C.create_string_buffer(256)
    cu, khz, mem = C.c_int32(), C.c_int32(), C.c_size_t()
    check(lib().moye_device_info(name, 256, C.byref(cu), C.byref(khz), C.byref(mem)))
    return {"name": name.value.decode(), "compute_units": cu.value, "clock_khz": khz.value,
            "total_mem": mem.value}


def tiled_mma_desc(atom, atom_layout=(1, 1, 1), tile=(0, 0, 0), cta_tile=(0, 0, 0), stages=0, split_k=0,
                   flags=0):
    """A moye_tiled_mma: what `make_tiled_mma(op, atom_layout, permutations)` (src/atom/mma.jl:193-233)
    plus the kernel's shared-memory tile (bM, bN, bK) boil down to."""
    d = TiledMMA()
    d.atom = atom
    for i in range(3):
        d.atom_layout_mnk[i] = atom_layout[i] if i < len(atom_layout) else 1
        d.tile_mnk[i] = tile[i]
        d.cta_tile_mnk[i] = cta_tile[i]
    d.stages, d.split_k, d.flags = stages, split_k, flags
    return d


def tiled_copy_desc(op=_lib.COPY_UNIVERSAL, vec_bits=0, thr_shape=(0, 0), val_shape=(0, 0), tiler=(0, 0),
                    flags=0):
    """A moye_tiled_copy: `make_tiled_copy(atom, thr_layout, val_layout)` (src/atom/copy.jl:249-258)."""
    d = TiledCopy()
    d.op, d.vec_bits, d.flags = op, vec_bits, flags
    for i in range(2):
        d.thr_shape[i], d.val_shape[i], d.tiler_mn[i] = thr_shape[i], val_shape[i], tiler[i]
    return d


def _ref(x):
    return C.byref(x) if x is not None else None


def copyto_(dst, src, tiled_copy=None, stream=None):
    """copyto!(dst, src) / copyto!(tiled_copy, dst, src) on moye_tensor descriptors; returns dst."""
    check(lib().moye_copy(_ref(tiled_copy), C.byref(dst), C.byref(src), stream))
    return dst


def copyto_if_(dst, src, mask, stream=None):
    """copyto_if!(dst, src, mask) (src/algorithm/copy.jl:4-16) on moye_tensor descriptors; the mask holds one byte per
    logical element, nonzero = move."""
    check(lib().moye_copy_if(C.byref(dst), C.byref(src), C.byref(mask), stream))
    return dst


def gemm_(mma, D, A, B, C_=None, alpha=1.0, stream=None):
    """gemm!(mma, D, A, B, C): D = alpha * A * B' + C with A:(M,K), B:(N,K), C,D:(M,N)."""
    check(lib().moye_gemm(C.byref(mma), C.byref(D), C.byref(A), C.byref(B), _ref(C_), alpha, stream))


def gemm_epilogue(alpha=1.0, beta=0.0, op=_lib.MAP_IDENTITY, operand=None, scalar=0.0):
    """A moye_gemm_epilogue: D = op(alpha * A * B' + beta * C, operand or scalar), every step rounded in fp32.
    Keeps `operand` (a moye_tensor) alive through the attribute `_operand`."""
    e = _lib.GemmEpilogue()
    e.alpha, e.beta, e.op, e.scalar = alpha, beta, op, scalar
    if operand is not None:
        e._operand = operand
        e.operand = C.pointer(operand)
    return e


def gemm_ex_(mma, D, A, B, C_=None, epilogue=None, workspace=None, workspace_bytes=0, stream=None):
    """gemm! with a fused epilogue and a caller-provided workspace (a device pointer as int, or None); never
    allocates."""
    ep = epilogue if epilogue is not None else gemm_epilogue()
    check(lib().moye_gemm_ex(C.byref(mma), C.byref(D), C.byref(A), C.byref(B), _ref(C_), C.byref(ep), workspace,
                             workspace_bytes, stream))


NOALLOC_SCRATCH_BYTES = 32 << 20


def gemm_noalloc_(mma, D, A, B, C_=None, alpha=1.0, stream=None):
    """gemm! whose workspace is the library's static device array (moye_gemm_noalloc): allocates nothing; fails when
    the call needs more than NOALLOC_SCRATCH_BYTES."""
    check(lib().moye_gemm_noalloc(C.byref(mma), C.byref(D), C.byref(A), C.byref(B), _ref(C_), alpha, stream))


def gemm_release_workspace():
    """Frees the per-stream workspaces moye_gemm keeps (waits for the device first)."""
    check(lib().moye_gemm_release_workspace())


def gemm_workspace_size(mma, D, A, B, epilogue=None):
    """Bytes of library-owned device workspace this gemm! call needs (K-major copies of operands that are not K-major,
    partial products of a split-K call); 0 for a plain TN call.  With `epilogue` (a moye_gemm_epilogue): for the
    moye_gemm_ex call with that epilogue."""
    n = C.c_size_t()
    if epilogue is None:
        check(lib().moye_gemm_workspace_size(C.byref(mma), C.byref(D), C.byref(A), C.byref(B), C.byref(n)))
    else:
        check(lib().moye_gemm_ex_workspace_size(C.byref(mma), C.byref(D), C.byref(A), C.byref(B), C.byref(epilogue), C.byref(n)))
    return n.value


def gemm_explain(mma, D, A, B, C_=None, epilogue=None, compute_units=0):
    """The launches a gemm! call would make (moye_gemm_explain): a list of dicts, one per step, with the step's `what`
    ("kernel", "kmajor_copy", "splitk_reduce"), the kernel's `name` and the `key=value` fields of its line (integers where
    they are integers), plus the first line's `workspace` bytes under the key "plan".  Host arithmetic only: the data
    pointers of the descriptors are never dereferenced."""
    buf = C.create_string_buffer(1 << 16)
    check(lib().moye_gemm_explain(C.byref(mma), C.byref(D), C.byref(A), C.byref(B), _ref(C_),
                                  C.byref(epilogue) if epilogue is not None else None, compute_units, buf, len(buf)))
    return parse_plan(buf.value.decode())


def parse_plan(text):
    """moye_gemm_explain's text as {"workspace": bytes, "cus": n, "xcds": n, "steps": [dict, ...], "text": text}."""
    lines = text.strip().splitlines()
    head = lines[0].split()
    plan = {"workspace": int(head[4]), "cus": int(head[6]), "xcds": int(head[9]), "steps": [], "text": text}
    for line in lines[1:]:
        body = line.split(": ", 1)[1]
        what, rest = body.split(" ", 1)
        step = {"what": what}
        if what == "kernel":
            name, _, rest = rest.partition(" ")
            step["name"] = name
            step["family"] = name.split("<")[0]
        for tok in rest.split():
            if "=" in tok:
                k, v = tok.split("=", 1)
                try:
                    step[k] = int(v)
                except ValueError:
                    step[k] = v
        if "flags" in step:
            step["flags"] = set() if step["flags"] in ("0", 0) else set(str(step["flags"]).split("|"))
        plan["steps"].append(step)
    return plan


def time_gemm(mma, D, A, B, C_=None, alpha=1.0, stream=None, warmup=2, iters=10):
    """Average milliseconds per launch (HIP events on `stream`)."""
    ms = C.c_float()
    check(lib().moye_time_gemm(C.byref(mma), C.byref(D), C.byref(A), C.byref(B), _ref(C_), alpha, stream,
                               warmup, iters, C.byref(ms)))
    return ms.value


def time_copy(dst, src, tiled_copy=None, stream=None, warmup=2, iters=10):
    ms = C.c_float()
    check(lib().moye_time_copy(_ref(tiled_copy), C.byref(dst), C.byref(src), stream, warmup, iters, C.byref(ms)))
    return ms.value


def mma_atom_probe(atom, a_ptr, b_ptr, d_ptr, stream=None):
    """One wave executes the atom once through its (thr,val) tables: D(M,N) = A(M,K) * B(N,K)',
    all dense column-major device buffers (raw pointers)."""
    f = lib().moye_mma_atom_probe
    f.argtypes = [C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    check(f(atom, a_ptr, b_ptr, d_ptr, stream))


def axpby_(a, x, b, y, stream=None):
    """axpby!(a, X, b, Y) on raw descriptors."""
    f = lib().moye_axpby
    f.argtypes = [C.c_double, C.c_void_p, C.c_double, C.c_void_p, C.c_void_p]
    check(f(a, C.byref(x), b, C.byref(y), stream))


def fill_(x, value, stream=None):
    f = lib().moye_fill
    f.argtypes = [C.c_void_p, C.c_double, C.c_void_p]
    check(f(C.byref(x), value, stream))


def map_(op, dst, a, b=None, scalar=0.0, stream=None):
    """dst .= op.(a, b) / op.(a, scalar) on raw descriptors (moye_map)."""
    f = lib().moye_map
    f.argtypes = [C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_double, C.c_void_p]
    check(f(op, C.byref(dst), C.byref(a), C.byref(b) if b is not None else None, scalar, stream))


def mfma_ceiling(in_dtype, random_operands=True, seconds=0.3, stream=None):
    """(TFLOP/s, clock GHz) of an MFMA-only loop on every CU: the matrix pipe's sustained rate on this part."""
    f = lib().moye_mfma_ceiling
    f.argtypes = [C.c_int32, C.c_int32, C.c_float, C.POINTER(C.c_float), C.POINTER(C.c_float), C.c_void_p]
    tf, ghz = C.c_float(), C.c_float()
    check(f(in_dtype, 1 if random_operands else 0, seconds, C.byref(tf), C.byref(ghz), stream))
    return tf.value, ghz.value
