"""ctypes binding of include/fp8_block_gemm.h.

`gemm(a, b, a_scale, b_scale, c, m, n, k)` keeps the reference launcher's argument order
(/root/reference/check.cu:113, mn_large.hip:11).  Arguments are torch CUDA tensors (or raw
integer device pointers); only their data_ptr() crosses the boundary.
"""
import ctypes as C
import os
import re
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

KERNEL_AUTO, KERNEL_SCALAR, KERNEL_LARGE, KERNEL_SPLITK, KERNEL_SKINNY = range(5)
DTYPE_BF16, DTYPE_F32, DTYPE_BF16_F32MATH = 0, 1, 2
FLAG_WORKSPACE_ZEROED = 1
WORKSPACE_HEADER_BYTES = 16 << 20


class Options(C.Structure):
    """fp8gemm_options of the header: per-call kernel choice for gemm_ex"""
    _fields_ = [("kernel", C.c_int), ("tile_variant", C.c_int), ("ksplit", C.c_int), ("persistent", C.c_int),
                ("flags", C.c_int)]

    def __init__(self, kernel=KERNEL_AUTO, tile_variant=-1, ksplit=0, persistent=-1, flags=0):
        super().__init__(kernel, tile_variant, ksplit, persistent, flags)


class Fp8GemmError(RuntimeError):
    def __init__(self, code, where):
        self.code = code
        super().__init__(f"{where}: {error_string(code)} (code {code})")


def lib_path():
    return os.path.join(_HERE, "libfp8gemm.so")


def build(force=True):
    """Compile the HIP library for gfx950 (hipcc cross-compiles without a GPU)."""
    cmd = ["make", "-C", _HERE, "-j8"] + (["-B"] if force else [])
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL)


def abi_symbols():
    """Function names declared in include/fp8_block_gemm.h."""
    hdr = os.path.join(_HERE, "..", "include", "fp8_block_gemm.h")
    text = open(hdr).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fp8_[a-z0-9_]+)\s*\(", text)))


def lib():
    global _LIB
    if _LIB is not None:
        return _LIB
    path = lib_path()
    if not os.path.exists(path):
        raise FileNotFoundError(
            f"{path} is missing: build it with __graft_entry__.build() or `make -C {_HERE}`")
    L = C.CDLL(path)
    vp, fp, i, sz = C.c_void_p, C.c_void_p, C.c_int, C.c_size_t
    L.fp8_block_gemm.restype = i
    L.fp8_block_gemm.argtypes = [vp, vp, fp, fp, vp, i, i, i]
    L.fp8_block_gemm_stream.restype = i
    L.fp8_block_gemm_stream.argtypes = [vp, vp, fp, fp, vp, i, i, i, vp]
    L.fp8_block_gemm_ex.restype = i
    L.fp8_block_gemm_ex.argtypes = [vp, vp, fp, fp, vp, i, i, i, C.POINTER(Options), vp, sz, vp]
    L.fp8_block_gemm_ws.restype = i
    L.fp8_block_gemm_ws.argtypes = [vp, vp, fp, fp, vp, i, i, i, vp, sz, vp]
    L.fp8_block_gemm_workspace_bytes_ex.restype = sz
    L.fp8_block_gemm_workspace_bytes_ex.argtypes = [i, i, i, C.POINTER(Options), i]
    L.fp8_block_gemm_grouped_workspace_bytes.restype = sz
    L.fp8_block_gemm_grouped_workspace_bytes.argtypes = [i, C.POINTER(C.c_int), i, i]
    L.fp8_block_gemm_grouped_workspace_bytes_ex.restype = sz
    L.fp8_block_gemm_grouped_workspace_bytes_ex.argtypes = [i, C.POINTER(C.c_int), i, i, C.POINTER(Options)]
    L.fp8_block_gemm_grouped_ex.restype = i
    L.fp8_block_gemm_grouped_ex.argtypes = [i, vp, vp, vp, vp, vp, vp, i, i, C.POINTER(Options), vp, sz, vp]
    L.fp8_block_gemm_noalloc.restype = i
    L.fp8_block_gemm_noalloc.argtypes = [vp, vp, fp, fp, vp, i, i, i, vp]
    L.fp8_block_gemm_scalar.restype = i
    L.fp8_block_gemm_scalar.argtypes = [vp, vp, fp, fp, vp, i, i, i, vp]
    L.fp8_block_gemm_select.restype = i
    L.fp8_block_gemm_select.argtypes = [i]
    L.fp8_block_gemm_force_config.restype = i
    L.fp8_block_gemm_force_config.argtypes = [i, i]
    L.fp8_block_gemm_grouped.restype = i
    L.fp8_block_gemm_grouped.argtypes = [i, vp, vp, vp, vp, vp, vp, i, i, vp]
    L.fp8_block_gemm_set_persistent.restype = i
    L.fp8_block_gemm_set_persistent.argtypes = [i]
    L.fp8_block_gemm_set_fused_reduction.restype = i
    L.fp8_block_gemm_set_fused_reduction.argtypes = [i]
    L.fp8_block_gemm_plan.restype = i
    L.fp8_block_gemm_plan.argtypes = [i, i, i, C.c_char_p, sz]
    L.fp8_block_gemm_last_kernel.restype = C.c_char_p
    L.fp8_block_gemm_last_kernel.argtypes = []
    L.fp8_block_gemm_workspace_bytes.restype = sz
    L.fp8_block_gemm_workspace_bytes.argtypes = [i, i, i]
    L.fp8_block_gemm_set_workspace.restype = i
    L.fp8_block_gemm_set_workspace.argtypes = [vp, sz]
    L.fp8_block_gemm_release.restype = i
    L.fp8_block_gemm_release.argtypes = []
    L.fp8_block_gemm_workspace_growth.restype = sz
    L.fp8_block_gemm_workspace_growth.argtypes = [sz, sz]
    L.fp8_convert_f32_to_e4m3fn.restype = i
    L.fp8_convert_f32_to_e4m3fn.argtypes = [vp, vp, sz, vp]
    L.fp8_quantize_a_1x128.restype = i
    L.fp8_quantize_a_1x128.argtypes = [vp, i, vp, fp, i, i, vp]
    L.fp8_quantize_b_128x128.restype = i
    L.fp8_quantize_b_128x128.argtypes = [vp, i, vp, fp, i, i, vp]
    L.fp8_block_gemm_error_string.restype = C.c_char_p
    L.fp8_block_gemm_error_string.argtypes = [i]
    L.fp8_block_gemm_abi_version.restype = i
    L.fp8_block_gemm_abi_version.argtypes = []
    L.fp8_gemm_host.restype = i
    L.fp8_gemm_host.argtypes = [vp, vp, vp, vp, vp, sz, sz, sz, i]
    _LIB = L
    return L


def error_string(code):
    return lib().fp8_block_gemm_error_string(int(code)).decode()


def _ptr(x):
    if x is None:
        return None
    if isinstance(x, int):
        return x
    return x.data_ptr()


def _check(rc, where):
    if rc != 0:
        raise Fp8GemmError(rc, where)


def gemm(a, b, a_scale, b_scale, c, m, n, k, stream=None):
    """C[m,n] bf16 = block-scaled A.B^T.  `stream` is a raw hipStream_t (int) or None for the
    null stream."""
    L = lib()
    if stream is None:
        rc = L.fp8_block_gemm(_ptr(a), _ptr(b), _ptr(a_scale), _ptr(b_scale), _ptr(c), m, n, k)
    else:
        rc = L.fp8_block_gemm_stream(_ptr(a), _ptr(b), _ptr(a_scale), _ptr(b_scale), _ptr(c), m, n, k,
                                     stream)
    _check(rc, "fp8_block_gemm")


def gemm_ex(a, b, a_scale, b_scale, c, m, n, k, options=None, workspace=None, workspace_bytes=0, stream=None):
    """Per-call form: `options` (Options or None = automatic), `workspace` (device tensor / pointer or
    None) of `workspace_bytes`.  Allocates nothing, reads no process-wide switch."""
    opt = C.byref(options) if options is not None else None
    rc = lib().fp8_block_gemm_ex(_ptr(a), _ptr(b), _ptr(a_scale), _ptr(b_scale), _ptr(c), m, n, k, opt,
                                 _ptr(workspace), workspace_bytes, stream)
    _check(rc, "fp8_block_gemm_ex")


NOALLOC_MAX_BYTES = 32 << 20


def gemm_noalloc(a, b, a_scale, b_scale, c, m, n, k, stream=None):
    """fp8_block_gemm_stream with the library's fixed in-image workspace: allocates nothing; plans that
    need more than NOALLOC_MAX_BYTES raise (code -4)."""
    _check(lib().fp8_block_gemm_noalloc(_ptr(a), _ptr(b), _ptr(a_scale), _ptr(b_scale), _ptr(c), m, n, k,
                                        stream), "fp8_block_gemm_noalloc")


def workspace_bytes_ex(m, n, k, options=None, any_alignment=False):
    opt = C.byref(options) if options is not None else None
    return int(lib().fp8_block_gemm_workspace_bytes_ex(m, n, k, opt, 1 if any_alignment else 0))


def grouped_workspace_bytes(m, n, k, options=None, per_call=False):
    """Workspace bound of gemm_grouped (process-wide switches), or of gemm_grouped_ex under `options`
    when options is given or per_call is set."""
    ms = (C.c_int * len(m))(*[int(v) for v in m])
    if options is None and not per_call:
        return int(lib().fp8_block_gemm_grouped_workspace_bytes(len(m), ms, n, k))
    opt = C.byref(options) if options is not None else None
    return int(lib().fp8_block_gemm_grouped_workspace_bytes_ex(len(m), ms, n, k, opt))


def gemm_scalar(a, b, a_scale, b_scale, c, m, n, k, stream=None):
    rc = lib().fp8_block_gemm_scalar(_ptr(a), _ptr(b), _ptr(a_scale), _ptr(b_scale), _ptr(c), m, n, k,
                                     stream)
    _check(rc, "fp8_block_gemm_scalar")


def select(kernel_id):
    _check(lib().fp8_block_gemm_select(kernel_id), "fp8_block_gemm_select")


def force_config(tile_variant=-1, ksplit=0):
    _check(lib().fp8_block_gemm_force_config(tile_variant, ksplit), "fp8_block_gemm_force_config")


def gemm_grouped(a, b, a_scale, b_scale, c, m, n, k, stream=None):
    """Grouped GEMM: lists of per-group tensors (or raw device pointers) and a list of per-group m;
    all groups share n and k.  One persistent launch when every m is a multiple of 16."""
    groups = len(m)
    if not (len(a) == len(b) == len(a_scale) == len(b_scale) == len(c) == groups):
        raise ValueError("one entry per group in every list")
    ptrs = lambda xs: (C.c_void_p * groups)(*[_ptr(x) for x in xs])
    ms = (C.c_int * groups)(*[int(v) for v in m])
    _check(lib().fp8_block_gemm_grouped(groups, ptrs(a), ptrs(b), ptrs(a_scale), ptrs(b_scale), ptrs(c),
                                        ms, n, k, stream), "fp8_block_gemm_grouped")


def gemm_grouped_ex(a, b, a_scale, b_scale, c, m, n, k, options=None, workspace=None, workspace_bytes=0, stream=None):
    """Per-call form of gemm_grouped: `options` and `workspace` as for gemm_ex; allocates nothing and
    reads no process-wide switch."""
    groups = len(m)
    if not (len(a) == len(b) == len(a_scale) == len(b_scale) == len(c) == groups):
        raise ValueError("one entry per group in every list")
    ptrs = lambda xs: (C.c_void_p * groups)(*[_ptr(x) for x in xs])
    ms = (C.c_int * groups)(*[int(v) for v in m])
    opt = C.byref(options) if options is not None else None
    _check(lib().fp8_block_gemm_grouped_ex(groups, ptrs(a), ptrs(b), ptrs(a_scale), ptrs(b_scale), ptrs(c), ms, n, k,
                                           opt, _ptr(workspace), workspace_bytes, stream), "fp8_block_gemm_grouped_ex")


def set_persistent(mode=-1):
    """-1: persistent tile kernel when tiles outnumber the CUs, 0: never, 1: whenever possible"""
    _check(lib().fp8_block_gemm_set_persistent(mode), "fp8_block_gemm_set_persistent")


def set_fused_reduction(mode=-1):
    """K splits added inside the GEMM kernel: -1 by cost, 0 never (reduction kernel), 1 whenever possible"""
    _check(lib().fp8_block_gemm_set_fused_reduction(mode), "fp8_block_gemm_set_fused_reduction")


def plan(m, n, k):
    """Name of the kernel plan the dispatcher picks for this shape (no device access)."""
    buf = C.create_string_buffer(64)
    _check(lib().fp8_block_gemm_plan(m, n, k, buf, 64), "fp8_block_gemm_plan")
    return buf.value.decode()


def last_kernel():
    return lib().fp8_block_gemm_last_kernel().decode()


def workspace_bytes(m, n, k):
    return int(lib().fp8_block_gemm_workspace_bytes(m, n, k))


def set_workspace(ptr, nbytes):
    _check(lib().fp8_block_gemm_set_workspace(_ptr(ptr), nbytes), "fp8_block_gemm_set_workspace")


def release():
    _check(lib().fp8_block_gemm_release(), "fp8_block_gemm_release")


def convert_f32_to_e4m3fn(src, dst, count, stream=None):
    _check(lib().fp8_convert_f32_to_e4m3fn(_ptr(src), _ptr(dst), count, stream),
           "fp8_convert_f32_to_e4m3fn")


def quantize_a_1x128(x, a, a_scale, m, k, dtype=DTYPE_BF16, stream=None):
    """x [m][k] row-major (bf16 bits or fp32) -> a (fp8, element (m,k) at m + k*M) and
    a_scale ([k/128][m]): to_float8_rowwise_scale of /root/reference/quantize.py:43-67 written
    in the GEMM's layouts."""
    _check(lib().fp8_quantize_a_1x128(_ptr(x), dtype, _ptr(a), _ptr(a_scale), m, k, stream),
           "fp8_quantize_a_1x128")


def quantize_b_128x128(x, b, b_scale, n, k, dtype=DTYPE_BF16, stream=None):
    """x [n][k] row-major -> b (fp8 at n + k*N) and b_scale ([k/128][ceil(n/128)]):
    to_float8_block_scale of /root/reference/quantize.py:16-41 written in the GEMM's layouts."""
    _check(lib().fp8_quantize_b_128x128(_ptr(x), dtype, _ptr(b), _ptr(b_scale), n, k, stream),
           "fp8_quantize_b_128x128")


def custom_kernel(data, stream=None):
    """The operator form the reference's kernels were written for (the challenge harness named in
    /root/reference/README.md:13 hands over torch tensors and expects c back):

        a        [m, k]           fp8 e4m3fn (or its uint8 view), strides (1, m)   -- column-major
        b        [n, k]           fp8 e4m3fn (or its uint8 view), strides (1, n)
        a_scale  [m, k/128]       float32, strides (1, m)
        b_scale  [n/128, k/128]   float32, strides (1, ceil(n/128))
        c        [m, n]           bfloat16, contiguous (row-major), overwritten and returned

    Those strides are exactly the memory layouts of the C ABI (check.cu:42-48), so only the
    pointers cross the boundary.  Runs on torch's current stream unless `stream` is given."""
    import torch
    a, b, a_scale, b_scale, c = data
    m, k = a.shape
    n = b.shape[0]
    sn = (n + 127) // 128
    if b.shape[1] != k or tuple(c.shape) != (m, n) or k % 128:
        raise ValueError(f"inconsistent shapes: a {tuple(a.shape)}, b {tuple(b.shape)}, c {tuple(c.shape)}")
    if tuple(a_scale.shape) != (m, k // 128) or tuple(b_scale.shape) != (sn, k // 128):
        raise ValueError(f"scale shapes {tuple(a_scale.shape)}, {tuple(b_scale.shape)} do not match "
                         f"({m}, {k // 128}) and ({sn}, {k // 128})")

    def col_major(t, lead):
        return t.stride(0) == 1 and (t.shape[1] == 1 or t.stride(1) == lead)

    if not (col_major(a, m) and col_major(b, n) and col_major(a_scale, m) and col_major(b_scale, sn)):
        raise ValueError("a, b, a_scale and b_scale must be column-major (stride 1 along their first axis)")
    if not c.is_contiguous() or c.dtype != torch.bfloat16:
        raise ValueError("c must be a contiguous bfloat16 tensor")
    if a.element_size() != 1 or b.element_size() != 1 or a_scale.dtype != torch.float32 \
            or b_scale.dtype != torch.float32:
        raise ValueError("a and b must be 1-byte fp8 tensors, the scales float32")
    if stream is None:
        stream = torch.cuda.current_stream().cuda_stream
    gemm(a, b, a_scale, b_scale, c, m, n, k, stream)
    return c
