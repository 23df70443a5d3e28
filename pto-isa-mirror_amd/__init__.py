"""Python host side of the MI355X (gfx950) backend for the PTO tile-matmul hot path.

Thin ctypes binding of the C ABI in ``include/ptoamd.h`` (``lib/libptoamd.so``).  PyTorch is used for device memory
and streams only; every operator below hands raw device pointers and sizes to the library, which runs hand-written
HIP kernels.  There is no CPU or PyTorch fallback: if the library is missing, importing this package raises.

Operator names and argument meaning mirror the reference's tile instructions for this path
(``TMATMUL`` / ``TMATMUL_ACC`` / ``TMATMUL_MX`` / ``TQUANT`` / ``TDEQUANT``, reference ``include/pto/common/pto_instr.hpp``).
"""
import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libptoamd.so")

# element types (include/ptoamd.h)
F32, F16, BF16, I32, I8, U8, E4M3, E5M2, E2M1, E1M2, I16, HIF8 = range(12)
RELU, SATURATE_INF = 1, 2  # flags of the `relu` argument
B_ND, B_DN = 0, 1
MX_A_ZZ, MX_A_ND, MX_A_DN, MX_B_NN, MX_B_ND, MX_B_DN = range(6)
OCP_MXFP8, NV_MXFP8, OCP_MXFP4, NV_MXFP4 = range(4)


class PtoAmdError(RuntimeError):
    pass


if not os.path.exists(LIB_PATH):
    raise ImportError(f"{LIB_PATH} is missing: build it with `make -C pto-isa-mirror_amd -j8` "
                      "(or __graft_entry__.build()); this package has no fallback path")

_lib = C.CDLL(LIB_PATH)
_lib.ptoamd_last_error.restype = C.c_char_p
_lib.ptoamd_last_kernel.restype = C.c_char_p
_lib.ptoamd_gemm_mx_workspace_bytes.restype = C.c_size_t
_lib.ptoamd_gemm_mx_workspace_bytes_b_nd.restype = C.c_size_t
_lib.ptoamd_gemm_workspace_bytes.restype = C.c_size_t
_lib.ptoamd_gemv_mxfp4_packed_bytes.restype = C.c_size_t

EXPORTS = [
    "ptoamd_init", "ptoamd_finalize", "ptoamd_last_error", "ptoamd_device_info", "ptoamd_malloc", "ptoamd_free",
    "ptoamd_malloc_host", "ptoamd_free_host", "ptoamd_memcpy", "ptoamd_memcpy_async", "ptoamd_memset",
    "ptoamd_stream_create", "ptoamd_stream_destroy", "ptoamd_stream_synchronize", "ptoamd_event_create",
    "ptoamd_event_destroy", "ptoamd_event_record", "ptoamd_event_synchronize", "ptoamd_event_elapsed_ms",
    "ptoamd_gemm", "ptoamd_gemm_bias", "ptoamd_gemm_ws", "ptoamd_gemm_workspace_bytes", "ptoamd_gemm_fp8", "ptoamd_gemm_requant", "ptoamd_gemm_atomic_add", "ptoamd_gemm_w8a8", "ptoamd_gemm_mx", "ptoamd_gemm_mx_bias",
    "ptoamd_gemm_mx_ws",
    "ptoamd_gemm_mx_workspace_bytes", "ptoamd_gemm_mx_workspace_bytes_b_nd", "ptoamd_gemm_mx_static", "ptoamd_gemv_mxfp4", "ptoamd_gemv_mxfp4_packed_bytes", "ptoamd_gemv_mxfp4_pack", "ptoamd_gemv_mxfp4_packed", "ptoamd_tquant_int8",
    "ptoamd_tquant_int8_para", "ptoamd_tquant_mx", "ptoamd_tdequant", "ptoamd_tdequant_para", "ptoamd_mx_scale_relayout",
    "ptoamd_last_kernel", "ptoamd_reload_options",
]


def lib():
    return _lib


def _check(rc, what):
    if rc != 0:
        raise PtoAmdError(f"{what} failed ({rc}): {_lib.ptoamd_last_error().decode()}")


def last_kernel():
    return _lib.ptoamd_last_kernel().decode()


def init(device=0):
    _check(_lib.ptoamd_init(int(device)), "ptoamd_init")


def reload_options():
    """Re-reads the PTOAMD_* environment switches (the library reads them once per process otherwise)."""
    _check(_lib.ptoamd_reload_options(), "ptoamd_reload_options")


def _ptr(t, strided=False):
    """Device address of a tensor.  Operands must be contiguous; strided=True also takes a 2-D view with unit column
    stride, and is passed only where the call forwards the view's row pitch (stride(0)) as a leading dimension."""
    if t is None:
        return C.c_void_p(0)
    assert t.is_cuda, "operands must be device tensors"
    if strided:
        assert t.is_contiguous() or (t.dim() == 2 and t.stride(1) == 1), "operand must be contiguous or row-strided"
    else:
        assert t.is_contiguous(), "operand must be contiguous (this argument has no leading-dimension parameter)"
    return C.c_void_p(t.data_ptr())


def _cin(c_in, out):
    """The accumulator input is read at the output's row pitch (the C ABI has one ldc for both)."""
    if c_in is None:
        return C.c_void_p(0)
    assert c_in.dim() == 2 and c_in.stride(0) == out.stride(0), "c_in must have the output's row pitch"
    return _ptr(c_in, True)


def _stream(stream):
    s = stream if stream is not None else torch.cuda.current_stream()
    return C.c_void_p(s.cuda_stream)


_TORCH_OUT = {F32: torch.float32, F16: torch.float16, BF16: torch.bfloat16, I32: torch.int32}


def gemm_workspace_bytes(n, k, ab_type, b_layout):
    return int(_lib.ptoamd_gemm_workspace_bytes(n, k, ab_type, b_layout))


def gemm(a, b, ab_type, c_type=F32, b_layout=B_DN, c_in=None, relu=False, m=None, n=None, k=None, stream=None, out=None,
         bias=None, workspace=None):
    """TLOAD -> TMATMUL / TMATMUL_ACC / TMATMUL_BIAS -> TSTORE.  a: [m, k]; b: [n, k] (B_DN) or [k, n] (B_ND), raw-typed
    tensors; bias: [n] of the accumulator type; workspace: a uint8 device tensor of gemm_workspace_bytes(...) bytes into
    which a row-major b is re-ordered (without one it is transposed inside the loader)."""
    m = a.shape[0] if m is None else m
    k = a.shape[1] if k is None else k
    n = (b.shape[0] if b_layout == B_DN else b.shape[1]) if n is None else n
    if out is None:
        out = torch.empty((m, n), dtype=_TORCH_OUT[c_type], device=a.device)
    if workspace is not None:
        _check(_lib.ptoamd_gemm_ws(_ptr(out, True), c_type, _ptr(a, True), _ptr(b, True), ab_type, _cin(c_in, out), _ptr(bias), m, n, k,
                                   a.stride(0), b.stride(0), out.stride(0), b_layout, int(relu), _ptr(workspace),
                                   C.c_size_t(workspace.numel() * workspace.element_size()), _stream(stream)), "ptoamd_gemm_ws")
        return out
    if bias is not None:
        _check(_lib.ptoamd_gemm_bias(_ptr(out, True), c_type, _ptr(a, True), _ptr(b, True), ab_type, _cin(c_in, out), _ptr(bias), m, n, k,
                                     a.stride(0), b.stride(0), out.stride(0), b_layout, int(relu), _stream(stream)),
               "ptoamd_gemm_bias")
        return out
    _check(_lib.ptoamd_gemm(_ptr(out, True), c_type, _ptr(a, True), _ptr(b, True), ab_type, _cin(c_in, out), m, n, k, a.stride(0), b.stride(0),
                            out.stride(0), b_layout, int(relu), _stream(stream)), "ptoamd_gemm")
    return out


def gemm_fp8(a, b, a_type, b_type, c_type=F32, b_layout=B_DN, c_in=None, bias=None, relu=False, stream=None, out=None):
    """TMATMUL on an fp8 pair whose two types may differ (E4M3 / E5M2)."""
    m, k = a.shape
    n = b.shape[0] if b_layout == B_DN else b.shape[1]
    if out is None:
        out = torch.empty((m, n), dtype=_TORCH_OUT[c_type], device=a.device)
    _check(_lib.ptoamd_gemm_fp8(_ptr(out, True), c_type, _ptr(a, True), a_type, _ptr(b, True), b_type, _cin(c_in, out), _ptr(bias), m, n, k,
                                a.stride(0), b.stride(0), out.stride(0), b_layout, int(relu), _stream(stream)), "ptoamd_gemm_fp8")
    return out


def gemm_atomic_add(out, a, b, ab_type, b_layout=B_DN, stream=None):
    """out += A . B through TSTORE<AtomicAdd> (out: f32 for float inputs, int32 for int8)."""
    m, k = a.shape
    n = out.shape[1]
    c_type = F32 if out.dtype == torch.float32 else I32
    _check(_lib.ptoamd_gemm_atomic_add(_ptr(out, True), c_type, _ptr(a, True), _ptr(b, True), ab_type, m, n, k, a.stride(0), b.stride(0),
                                       out.stride(0), b_layout, _stream(stream)), "ptoamd_gemm_atomic_add")
    return out


def gemm_requant(a, b, ab_type, c_type, quant_words, per_column=False, b_layout=B_DN, c_in=None, bias=None, relu=False,
                 n=None, stream=None, out=None):
    """TLOAD -> TMATMUL -> TSTORE through the fix-pipe quantiser.  quant_words: int64 / uint64 device tensor holding one
    word, or one word per column; c_type: I8, U8, F16, BF16 or (int8 operands) I16."""
    m, k = a.shape
    n = (b.shape[0] if b_layout == B_DN else b.shape[1]) if n is None else n
    if out is None:
        out = torch.empty((m, n), dtype={I8: torch.int8, U8: torch.uint8, F16: torch.float16, BF16: torch.bfloat16, I16: torch.int16}[c_type], device=a.device)
    _check(_lib.ptoamd_gemm_requant(_ptr(out, True), c_type, _ptr(a, True), _ptr(b, True), ab_type, _cin(c_in, out), _ptr(bias), _ptr(quant_words),
                                    int(per_column), m, n, k, a.stride(0), b.stride(0), out.stride(0), b_layout, int(relu),
                                    _stream(stream)), "ptoamd_gemm_requant")
    return out


def gemm_w8a8(a, b, scale_a, scale_b, b_layout=B_DN, want_acc=False, stream=None, out=None):
    """int8 x int8 -> int32 accumulate with the fused dequantising drain to bf16."""
    m, k = a.shape
    n = b.shape[0] if b_layout == B_DN else b.shape[1]
    if out is None:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=a.device)
    acc = torch.empty((m, n), dtype=torch.int32, device=a.device) if want_acc else None
    _check(_lib.ptoamd_gemm_w8a8(_ptr(out, True), _ptr(acc), _ptr(a, True), _ptr(b, True), _ptr(scale_a), _ptr(scale_b), m, n, k,
                                 a.stride(0), b.stride(0), out.stride(0), b_layout, _stream(stream)), "ptoamd_gemm_w8a8")
    return (out, acc) if want_acc else out


STATIC_SCRATCH_BYTES = 4 * 1024 * 1024


def gemm_mx_static(a, b, sa, sb, m, n, k, a_type, b_type, out, sa_layout=MX_A_ND, sb_layout=MX_B_DN, b_layout=B_DN, c_in=None,
                   stream=None):
    """TMATMUL_MX into a caller-provided `out`, re-laying scales in the library's static device array: nothing is
    allocated, here or in the library.  Calls that overlap in time on one GPU race on that array."""
    c_type = {v: key for key, v in _TORCH_OUT.items()}[out.dtype]
    lda = k
    ldb = k if b_layout == B_DN else n
    _check(_lib.ptoamd_gemm_mx_static(_ptr(out, True), c_type, _ptr(a), _ptr(b), a_type, b_type, _ptr(sa), _ptr(sb), sa_layout,
                                      sb_layout, _cin(c_in, out), m, n, k, lda, ldb, out.stride(0), b_layout, _stream(stream)),
           "ptoamd_gemm_mx_static")
    return out


def gemm_mx_workspace_bytes(m, n, k, sa_layout=MX_A_ND, sb_layout=MX_B_DN, b_layout=B_DN, b_type=E4M3):
    """Bytes of workspace gemm_mx(..., workspace=...) needs; with b_layout=B_ND it includes the room for a transposed
    copy of a row-major fp8 B, which lets the direct-to-LDS kernels run."""
    if b_layout == B_ND:
        return int(_lib.ptoamd_gemm_mx_workspace_bytes_b_nd(m, n, k, sa_layout, sb_layout, b_type))
    return int(_lib.ptoamd_gemm_mx_workspace_bytes(m, n, k, sa_layout, sb_layout))


def gemm_mx(a, b, sa, sb, m, n, k, a_type, b_type, c_type=F32, sa_layout=MX_A_ND, sb_layout=MX_B_DN, b_layout=B_DN,
            c_in=None, stream=None, out=None, workspace=None, bias=None):
    """TMATMUL_MX.  a / b hold element codes (uint8; fp4 packed two per byte); sa / sb hold E8M0 bytes.  workspace: a
    uint8 device tensor of gemm_mx_workspace_bytes(...) bytes selects the form that allocates nothing."""
    if out is None:
        out = torch.empty((m, n), dtype=_TORCH_OUT[c_type], device=a.device)
    lda = k
    ldb = k if b_layout == B_DN else n
    if workspace is not None:
        _check(_lib.ptoamd_gemm_mx_ws(_ptr(out, True), c_type, _ptr(a), _ptr(b), a_type, b_type, _ptr(sa), _ptr(sb), sa_layout,
                                      sb_layout, _cin(c_in, out), m, n, k, lda, ldb, out.stride(0), b_layout, _ptr(workspace),
                                      C.c_size_t(workspace.numel() * workspace.element_size()), _stream(stream)),
               "ptoamd_gemm_mx_ws")
        return out
    if bias is not None:
        _check(_lib.ptoamd_gemm_mx_bias(_ptr(out, True), c_type, _ptr(a), _ptr(b), a_type, b_type, _ptr(sa), _ptr(sb), sa_layout,
                                        sb_layout, _cin(c_in, out), _ptr(bias), m, n, k, lda, ldb, out.stride(0), b_layout,
                                        _stream(stream)), "ptoamd_gemm_mx_bias")
        return out
    _check(_lib.ptoamd_gemm_mx(_ptr(out, True), c_type, _ptr(a), _ptr(b), a_type, b_type, _ptr(sa), _ptr(sb), sa_layout,
                               sb_layout, _cin(c_in, out), m, n, k, lda, ldb, out.stride(0), b_layout, _stream(stream)),
           "ptoamd_gemm_mx")
    return out


def gemv_mxfp4(a_bf16, w, sw, n, k, c_type=F32, stream=None, out=None):
    """Decode GEMV: bf16 activations [m <= 16, k] times MXFP4 weights [n, k/2] with E8M0 scales [n, k/32]."""
    m = a_bf16.shape[0]
    if out is None:
        out = torch.empty((m, n), dtype=_TORCH_OUT[c_type], device=w.device)
    _check(_lib.ptoamd_gemv_mxfp4(_ptr(out, True), c_type, _ptr(a_bf16, True), _ptr(w), _ptr(sw), m, n, k, a_bf16.stride(0), k,
                                  out.stride(0), _stream(stream)), "ptoamd_gemv_mxfp4")
    return out


def gemv_mxfp4_pack(w, sw, n, k, stream=None):
    """MXFP4 weights [n, k/2] + E8M0 scales [n, k/32] -> the packed buffer gemv_mxfp4_packed consumes (k % 2048 == 0)."""
    size = int(_lib.ptoamd_gemv_mxfp4_packed_bytes(n, k))
    if size == 0:
        raise PtoAmdError(f"gemv_mxfp4_pack: k = {k} must be a positive multiple of 2048")
    packed = torch.empty(size, dtype=torch.uint8, device=w.device)
    _check(_lib.ptoamd_gemv_mxfp4_pack(_ptr(packed), _ptr(w), _ptr(sw), n, k, k, _stream(stream)), "ptoamd_gemv_mxfp4_pack")
    return packed


def gemv_mxfp4_packed(a_bf16, packed, n, k, c_type=F32, stream=None, out=None):
    """Decode GEMV on weights packed by gemv_mxfp4_pack: the same sums in the same order as gemv_mxfp4."""
    m = a_bf16.shape[0]
    if out is None:
        out = torch.empty((m, n), dtype=_TORCH_OUT[c_type], device=packed.device)
    _check(_lib.ptoamd_gemv_mxfp4_packed(_ptr(out, True), c_type, _ptr(a_bf16, True), _ptr(packed), m, n, k, a_bf16.stride(0),
                                         out.stride(0), _stream(stream)), "ptoamd_gemv_mxfp4_packed")
    return out


def tquant_int8(src, scale, offset=None, stream=None, out=None):
    """scale / offset: one value per row (1-D), or a 2-D parameter tile [para_rows][para_ld]: column 0 is read and rows
    past the tile's last repeat it (the reference's GetParamValue)."""
    rows, cols = src.shape
    if out is None:
        out = torch.empty((rows, cols), dtype=torch.int8 if offset is None else torch.uint8, device=src.device)
    if scale.dim() == 2:
        assert offset is None or offset.stride(0) == scale.stride(0), "scale and offset tiles share one row pitch"
        _check(_lib.ptoamd_tquant_int8_para(_ptr(out), _ptr(src), _ptr(scale, True), _ptr(offset, True), rows, cols, scale.shape[0],
                                            scale.stride(0), _stream(stream)), "ptoamd_tquant_int8_para")
        return out
    _check(_lib.ptoamd_tquant_int8(_ptr(out), _ptr(src), _ptr(scale), _ptr(offset), rows, cols, _stream(stream)),
           "ptoamd_tquant_int8")
    return out


_SRC_TYPE = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}


def tquant_mx(src, alg, axis=1, want_aux=True, stream=None, out=None):
    """TQUANT<MXFP8 | MXFP4_E2M1>: returns (codes, exp[, max, scaling]).  out: (codes, exp) tensors to write into."""
    rows, cols = src.shape
    fp4 = alg in (OCP_MXFP4, NV_MXFP4)
    gshape = (rows, cols // 32) if axis == 1 else (rows // 32, cols)
    if out is not None:
        codes, exp = out
    else:
        codes = torch.empty((rows, cols // 2 if fp4 else cols), dtype=torch.uint8, device=src.device)
        exp = torch.empty(gshape, dtype=torch.uint8, device=src.device)
    mx = torch.empty(gshape, dtype=torch.float32, device=src.device) if want_aux else None
    sc = torch.empty(gshape, dtype=torch.float32, device=src.device) if want_aux else None
    _check(_lib.ptoamd_tquant_mx(_ptr(codes), _ptr(exp), _ptr(mx), _ptr(sc), _ptr(src), _SRC_TYPE[src.dtype], rows, cols,
                                 alg, axis, _stream(stream)), "ptoamd_tquant_mx")
    return (codes, exp, mx, sc) if want_aux else (codes, exp)


_INT_TYPE = {torch.int8: I8, torch.int16: I16, torch.int32: I32}


def tdequant(src, scale, offset, stream=None, out=None):
    """scale / offset: one value per row (1-D), or a 2-D parameter tile [rows][para_cols]: element (r, c) reads parameter
    column min(c, para_cols - 1)."""
    rows, cols = src.shape
    if out is None:
        out = torch.empty((rows, cols), dtype=torch.float32, device=src.device)
    if scale.dim() == 2:
        assert offset.stride(0) == scale.stride(0), "scale and offset tiles share one row pitch"
        _check(_lib.ptoamd_tdequant_para(_ptr(out), _ptr(src), _INT_TYPE[src.dtype], _ptr(scale, True), _ptr(offset, True), rows, cols,
                                         scale.shape[1], scale.stride(0), _stream(stream)), "ptoamd_tdequant_para")
        return out
    _check(_lib.ptoamd_tdequant(_ptr(out), _ptr(src), _INT_TYPE[src.dtype], _ptr(scale), _ptr(offset), rows, cols,
                                _stream(stream)), "ptoamd_tdequant")
    return out


def mx_scale_relayout(src, src_layout, dst_layout, rows, cols, stream=None):
    out = torch.empty_like(src)
    _check(_lib.ptoamd_mx_scale_relayout(_ptr(out), dst_layout, _ptr(src), src_layout, rows, cols, _stream(stream)),
           "ptoamd_mx_scale_relayout")
    return out
