"""ctypes bindings for the test-only checkers (TEST INFRASTRUCTURE, never imported by the product package).

``Oracle``  -> oracle/libptooracle.so   (plain-C restatement, pto_oracle.c)
``RefLib``  -> oracle/_ref/libptoref.so (the reference CPU simulator compiled from its own headers; present
               only where it was built, i.e. where the reference tree is mounted, or as a prebuilt file)
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

E4M3, E5M2, E2M1, E1M2, E8M0 = 0, 1, 2, 3, 4
ND, DN, NZ, MX_A_ZZ, MX_A_ND, MX_A_DN, MX_B_NN, MX_B_ND, MX_B_DN = range(9)
ST_F32, ST_F16, ST_BF16, ST_I32, ST_I8, ST_U8, ST_I16 = range(7)
OCP_FP8, NV_FP8, OCP_FP4, NV_FP4 = range(4)
SRC_F32, SRC_F16, SRC_BF16 = range(3)


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    return None if a is None else np.ascontiguousarray(a, dtype=dt)


class Oracle:
    def __init__(self, path=None):
        path = path or os.path.join(_HERE, "libptooracle.so")
        if not os.path.exists(path):
            raise FileNotFoundError(f"{path} missing: run `make -C oracle libptooracle.so` (or __graft_entry__.build())")
        L = self.lib = C.CDLL(path)
        L.pto_f16_to_f32.restype = C.c_float
        L.pto_f16_to_f32.argtypes = [C.c_uint16]
        L.pto_f32_to_f16.restype = C.c_uint16
        L.pto_f32_to_f16.argtypes = [C.c_float]
        L.pto_f32_to_bf16.restype = C.c_uint16
        L.pto_f32_to_bf16.argtypes = [C.c_float]
        L.pto_mx_decode.restype = C.c_double
        L.pto_mx_decode.argtypes = [C.c_int, C.c_uint]
        L.pto_mx_encode_trunc.restype = C.c_uint
        L.pto_mx_encode_trunc.argtypes = [C.c_int, C.c_double]
        L.pto_fp8_encode_round.restype = C.c_uint
        L.pto_fp8_encode_round.argtypes = [C.c_int, C.c_double, C.c_int, C.c_int]
        L.pto_fp4_encode_round.restype = C.c_uint
        L.pto_fp4_encode_round.argtypes = [C.c_int, C.c_double, C.c_int]
        L.pto_mx_scale_offset.restype = C.c_int64
        L.pto_mx_scale_offset.argtypes = [C.c_int] * 5
        L.pto_quant_word_scale.restype = C.c_float
        L.pto_quant_word_scale.argtypes = [C.c_uint64, C.c_int]
        L.pto_encode_e4m3fn.restype = C.c_uint
        L.pto_encode_e4m3fn.argtypes = [C.c_float, C.c_int]
        L.pto_encode_e2m1_magic.restype = C.c_uint
        L.pto_encode_e2m1_magic.argtypes = [C.c_float]
        L.pto_shared_exponent.restype = C.c_uint
        L.pto_shared_exponent.argtypes = [C.c_int, C.c_float]
        L.pto_hif8_to_f64.restype = C.c_double
        L.pto_hif8_to_f64.argtypes = [C.c_uint]
        L.pto_group_scaling.restype = C.c_float
        L.pto_group_scaling.argtypes = [C.c_int, C.c_float, C.c_uint]
        L.pto_tile_offset.restype = C.c_int64
        L.pto_global_offset.restype = C.c_int64
        L.pto_global_offset.argtypes = [C.c_int, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p]
        L.pto_layout_2d.restype = C.c_int
        L.pto_layout_2d.argtypes = [C.c_int, C.c_int64, C.c_int64, C.c_int, C.c_void_p, C.c_void_p]
        L.pto_sim_gemm_tiled.restype = C.c_int
        L.pto_sim_gemm_mx_tiled.restype = C.c_int

    # -- element types -----------------------------------------------------------------------
    def f32_to_f16(self, x):
        x = np.asarray(x, np.float32).ravel()
        return np.array([self.lib.pto_f32_to_f16(float(v)) for v in x], np.uint16)

    def f32_to_bf16(self, x):
        x = np.asarray(x, np.float32).ravel()
        return np.array([self.lib.pto_f32_to_bf16(float(v)) for v in x], np.uint16)

    def mx_decode_table(self, typ):
        return np.array([self.lib.pto_mx_decode(typ, c) for c in range(256)], np.float64)

    # -- addressing --------------------------------------------------------------------------
    class _TileLayout(C.Structure):
        _fields_ = [(n, C.c_int) for n in ("rows", "cols", "row_major", "sfractal", "inner_rows", "inner_cols")]

    def tile_offsets(self, rows, cols, row_major, sfractal, sfractal_size, elem_bytes, packed2=0):
        t = self._TileLayout()
        self.lib.pto_tile_layout_init(C.byref(t), rows, cols, int(row_major), sfractal, sfractal_size, elem_bytes,
                                      packed2)
        out = np.empty((rows, cols), np.int64)
        for r in range(rows):
            for c in range(cols):
                out[r, c] = self.lib.pto_tile_offset(C.byref(t), r, c)
        return out

    def mx_scale_offsets(self, layout, rows, cols):
        return np.array([[self.lib.pto_mx_scale_offset(layout, rows, cols, r, c) for c in range(cols)]
                         for r in range(rows)], np.int64)

    def global_offsets(self, layout, shape, stride, rows, cols):
        """Element offsets of the rows x cols logical view of a 5-D GlobalTensor (ND, DN or NZ)."""
        sh = np.ascontiguousarray(shape, np.int64)
        st = np.ascontiguousarray(stride, np.int64)
        return np.array([[self.lib.pto_global_offset(layout, r, c, _p(sh), _p(st)) for c in range(cols)]
                         for r in range(rows)], np.int64)

    def layout_2d(self, layout, rows, cols, c0=8):
        sh, st = np.zeros(5, np.int64), np.zeros(5, np.int64)
        assert self.lib.pto_layout_2d(layout, rows, cols, c0, _p(sh), _p(st)) == 0
        return sh, st

    def reorder_exp_zz(self, exp):
        exp = np.ascontiguousarray(exp, np.uint8)
        out = np.empty(exp.size, np.uint8)
        self.lib.pto_reorder_exp_zz(_p(out), _p(exp), exp.shape[0], exp.shape[1])
        return out

    # -- matmul ------------------------------------------------------------------------------
    def _mm(self, fn, out_dt, in_dt, a, b, cin, bias, b_dn):
        a = _c(a, in_dt)
        b = _c(b, in_dt)
        m, k = a.shape
        n = b.shape[0] if b_dn else b.shape[1]
        assert (b.shape[1] if b_dn else b.shape[0]) == k
        out = np.empty((m, n), out_dt)
        cin = _c(cin, out_dt)
        bias = _c(bias, out_dt)
        fn(_p(out), _p(a), _p(b), _p(cin), _p(bias), m, k, n, k, b.shape[1], n, int(b_dn))
        return out

    def matmul_f16(self, a, b, cin=None, bias=None, b_dn=False):
        return self._mm(self.lib.pto_matmul_f16, np.float32, np.uint16, a, b, cin, bias, b_dn)

    def matmul_bf16(self, a, b, cin=None, bias=None, b_dn=False):
        return self._mm(self.lib.pto_matmul_bf16, np.float32, np.uint16, a, b, cin, bias, b_dn)

    def matmul_f32(self, a, b, cin=None, bias=None, b_dn=False):
        return self._mm(self.lib.pto_matmul_f32, np.float32, np.float32, a, b, cin, bias, b_dn)

    def matmul_i8(self, a, b, cin=None, bias=None, b_dn=False):
        return self._mm(self.lib.pto_matmul_i8, np.int32, np.int8, a, b, cin, bias, b_dn)

    def matmul_fp8(self, a, b, cin=None, bias=None, b_dn=False, a_type=E4M3, b_type=E4M3):
        a = _c(a, np.uint8)
        b = _c(b, np.uint8)
        m, k = a.shape
        n = b.shape[0] if b_dn else b.shape[1]
        out = np.empty((m, n), np.float32)
        cin = _c(cin, np.float32)
        bias = _c(bias, np.float32)
        self.lib.pto_matmul_fp8(_p(out), _p(a), _p(b), _p(cin), _p(bias), m, k, n, k, b.shape[1], n, int(b_dn),
                                a_type, b_type)
        return out

    def matmul_mx(self, a, b, sa, sb, m, k, n, a_type, b_type, sa_layout=MX_A_ND, sb_layout=MX_B_DN, b_dn=True,
                  cin=None, bias=None):
        """a, b: uint8 code buffers (fp4 packed two per byte); leading dims are k (A) and k or n (B), in elements."""
        a = _c(a, np.uint8)
        b = _c(b, np.uint8)
        sa = _c(sa, np.uint8)
        sb = _c(sb, np.uint8)
        out = np.empty((m, n), np.float32)
        cin = _c(cin, np.float32)
        bias = _c(bias, np.float32)
        self.lib.pto_matmul_mx(_p(out), _p(a), _p(b), _p(sa), _p(sb), _p(cin), _p(bias), m, k, n, k,
                               k if b_dn else n, n, int(b_dn), a_type, b_type, sa_layout, sb_layout)
        return out

    # -- store -------------------------------------------------------------------------------
    _ST_DT = {ST_F32: np.float32, ST_F16: np.uint16, ST_BF16: np.uint16, ST_I32: np.int32, ST_I8: np.int8,
              ST_U8: np.uint8, ST_I16: np.int16}

    def store_f32(self, acc, dst_kind, relu=False):
        acc = _c(acc, np.float32)
        m, n = acc.shape
        out = np.empty((m, n), self._ST_DT[dst_kind])
        self.lib.pto_store_f32(_p(out), dst_kind, _p(acc), m, n, n, n, int(relu))
        return out

    def hif8_table(self):
        """The 256 HiFloat8 values as float64."""
        return np.array([self.lib.pto_hif8_to_f64(c) for c in range(256)], np.float64)

    def matmul_hif8(self, a, b, b_dn=False):
        """hif8 x hif8 TMATMUL: every code is an exact float, then the f32 product (sequential fma, k ascending)."""
        t = self.hif8_table().astype(np.float32)
        return self.matmul_f32(t[np.asarray(a, np.uint8)], t[np.asarray(b, np.uint8)], b_dn=b_dn)

    def store_quant(self, acc, dst_kind, words, per_column, relu=False, saturate_inf=0):
        words = _c(words, np.uint64)
        m, n = acc.shape
        out = np.empty((m, n), self._ST_DT[dst_kind])
        if acc.dtype == np.int32:
            acc = _c(acc, np.int32)
            self.lib.pto_store_quant_i32(_p(out), dst_kind, _p(acc), m, n, _p(words), int(per_column), int(relu))
        else:
            acc = _c(acc, np.float32)
            self.lib.pto_store_quant_f32(_p(out), dst_kind, _p(acc), m, n, _p(words), int(per_column), int(relu),
                                         int(saturate_inf))
        return out

    # -- quant / dequant ---------------------------------------------------------------------
    def tquant_int8(self, src, scale, offset=None):
        src = _c(src, np.float32)
        scale = _c(scale, np.float32)
        r, c = src.shape
        if offset is None:
            out = np.empty((r, c), np.int8)
            self.lib.pto_tquant_int8_sym(_p(out), _p(src), _p(scale), r, c)
        else:
            offset = _c(offset, np.float32)
            out = np.empty((r, c), np.uint8)
            self.lib.pto_tquant_int8_asym(_p(out), _p(src), _p(scale), _p(offset), r, c)
        return out

    def tquant_mx(self, src, alg, axis=1, src_kind=SRC_F32):
        src = _c(src, np.float32)
        r, c = src.shape
        fp4 = alg in (OCP_FP4, NV_FP4)
        dst = np.zeros(r * c // 2 if fp4 else r * c, np.uint8)
        gshape = (r, c // 32) if axis == 1 else (r // 32, c)
        exp = np.empty(gshape, np.uint8)
        mx = np.empty(gshape, np.float32)
        sc = np.empty(gshape, np.float32)
        self.lib.pto_tquant_mx(_p(dst), _p(exp), _p(mx), _p(sc), _p(src), r, c, alg, axis, src_kind)
        return (dst.reshape(r, c // 2) if fp4 else dst.reshape(r, c)), exp, mx, sc

    def tdequant(self, src, scale, offset):
        kind = {np.dtype(np.int8): 0, np.dtype(np.int16): 1, np.dtype(np.int32): 2}[src.dtype]
        src = np.ascontiguousarray(src)
        r, c = src.shape
        out = np.empty((r, c), np.float32)
        self.lib.pto_tdequant(_p(out), _p(src), kind, _p(_c(scale, np.float32)), _p(_c(offset, np.float32)), r, c)
        return out

    def tdequant_para(self, src, scale, offset):
        """scale / offset: [rows][para_cols]; element (r, c) uses parameter column min(c, para_cols - 1)."""
        kind = {np.dtype(np.int8): 0, np.dtype(np.int16): 1, np.dtype(np.int32): 2}[src.dtype]
        src = np.ascontiguousarray(src)
        scale, offset = _c(scale, np.float32), _c(offset, np.float32)
        r, c = src.shape
        out = np.empty((r, c), np.float32)
        self.lib.pto_tdequant_para(_p(out), _p(src), kind, _p(scale), _p(offset), r, c, scale.shape[1], scale.shape[1])
        return out

    def tquant_int8_para(self, src, scale, offset=None, para_ld=1):
        """scale / offset: [para_rows * para_ld] flat; row r uses element min(r, para_rows - 1) * para_ld."""
        src = _c(src, np.float32)
        scale = _c(scale, np.float32)
        r, c = src.shape
        out = np.empty((r, c), np.uint8)
        off = None if offset is None else _p(_c(offset, np.float32))
        self.lib.pto_tquant_int8_para(_p(out), _p(src), _p(scale), off, r, c, scale.size // para_ld, para_ld)
        return out if offset is not None else out.view(np.int8)

    # -- CPU-simulator-shaped baseline --------------------------------------------------------
    def sim_gemm_tiled(self, a, b, dtype, out_kind, b_dn, max_threads=0):
        a = np.ascontiguousarray(a)
        b = np.ascontiguousarray(b)
        m, k = a.shape
        n = b.shape[0] if b_dn else b.shape[1]
        out = np.empty((m, n), np.int32 if dtype == 2 else self._ST_DT[out_kind])
        threads = self.lib.pto_sim_gemm_tiled(_p(out), _p(a), _p(b), m, k, n, int(b_dn), dtype, out_kind, max_threads)
        return out, threads

    def sim_gemm_mx_tiled(self, a, b, sa, sb, m, k, n, a_type, b_type, out_kind, max_threads=0):
        out = np.empty((m, n), self._ST_DT[out_kind])
        threads = self.lib.pto_sim_gemm_mx_tiled(_p(out), out_kind, _p(_c(a, np.uint8)), _p(_c(b, np.uint8)),
                                                 _p(_c(sa, np.uint8)), _p(_c(sb, np.uint8)), m, k, n, a_type, b_type,
                                                 max_threads)
        return out, threads


class RefLib:
    """The compiled reference CPU simulator (oracle/_ref/libptoref.so)."""

    @staticmethod
    def path():
        return os.path.join(_HERE, "_ref", "libptoref.so")

    @classmethod
    def available(cls):
        return os.path.exists(cls.path())

    def __init__(self):
        L = self.lib = C.CDLL(self.path())
        L.ref_init(1)
        L.ref_mx_decode.restype = C.c_double
        L.ref_mx_decode.argtypes = [C.c_int, C.c_uint]
        L.ref_mx_encode_trunc.restype = C.c_uint
        L.ref_mx_encode_trunc.argtypes = [C.c_int, C.c_double]
        L.ref_mx_encode_round.restype = C.c_uint
        L.ref_mx_encode_round.argtypes = [C.c_int, C.c_double, C.c_int, C.c_int]
        L.ref_encode_e4m3fn.restype = C.c_uint
        L.ref_encode_e4m3fn.argtypes = [C.c_float, C.c_int]
        L.ref_encode_e2m1_magic.restype = C.c_uint
        L.ref_encode_e2m1_magic.argtypes = [C.c_float]
        L.ref_shared_exponent.restype = C.c_uint
        L.ref_shared_exponent.argtypes = [C.c_int, C.c_float]
        L.ref_group_scaling.restype = C.c_float
        L.ref_group_scaling.argtypes = [C.c_int, C.c_float, C.c_uint]
        L.ref_extract_m1.restype = C.c_float
        L.ref_extract_m1.argtypes = [C.c_uint64, C.c_int]
        L.ref_tile_offset.restype = C.c_int64
        L.ref_mx_scale_offset.restype = C.c_int64
        L.ref_global_offset.restype = C.c_int64
        L.ref_global_offset.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]

    def gemm(self, kind, a, b, cin=None, b_dn=False, kstep=0):
        fn, in_dt, out_dt = {
            "f16": (self.lib.ref_gemm_f16, np.uint16, np.float32),
            "f32": (self.lib.ref_gemm_f32, np.float32, np.float32),
            "i8": (self.lib.ref_gemm_i8, np.int8, np.int32),
            "e4m3": (self.lib.ref_gemm_e4m3, np.uint8, np.float32),
            "e5m2": (self.lib.ref_gemm_e5m2, np.uint8, np.float32),
        }[kind]
        a = _c(a, in_dt)
        b = _c(b, in_dt)
        m, k = a.shape
        n = b.shape[0] if b_dn else b.shape[1]
        out = np.empty((m, n), out_dt)
        rc = fn(_p(out), _p(a), _p(b), _p(_c(cin, out_dt)), m, k, n, int(b_dn), kstep)
        assert rc == 0, rc
        return out

    def gemm_f16_out_f16(self, a, b, b_dn=False, kstep=0, relu=False):
        a = _c(a, np.uint16)
        b = _c(b, np.uint16)
        m, k = a.shape
        n = b.shape[0] if b_dn else b.shape[1]
        out = np.empty((m, n), np.uint16)
        rc = self.lib.ref_gemm_f16_out_f16(_p(out), _p(a), _p(b), m, k, n, int(b_dn), kstep, int(relu))
        assert rc == 0, rc
        return out

    def gemm_mx(self, a, b, sa, sb, m, k, n, dtype, scale_fmt, b_dn, cin=None):
        out = np.empty((m, n), np.float32)
        rc = self.lib.ref_gemm_mx(_p(out), _p(_c(a, np.uint8)), _p(_c(b, np.uint8)), _p(_c(sa, np.uint8)),
                                  _p(_c(sb, np.uint8)), _p(_c(cin, np.float32)), m, k, n, dtype, scale_fmt, int(b_dn))
        assert rc == 0, rc
        return out

    def hif8_table(self):
        out = np.empty(256, np.float64)
        self.lib.ref_hif8_table(_p(out))
        return out

    def store_quant(self, acc, dst, words, per_column, relu=False, saturate_inf=0):
        """saturate_inf sets bit 48 of the simulator's task cookie for the call (cpu/common.hpp:146)."""
        self.lib.ref_set_task_cookie(C.c_uint64((1 << 48) if saturate_inf else 0))
        try:
            return self._store_quant(acc, dst, words, per_column, relu)
        finally:
            self.lib.ref_set_task_cookie(C.c_uint64(0))

    def _store_quant(self, acc, dst, words, per_column, relu=False):
        words = _c(words, np.uint64)
        m, n = acc.shape
        key = ("i32" if acc.dtype == np.int32 else "f32") + "_" + dst
        out_dt = {"i8": np.int8, "u8": np.uint8, "f16": np.uint16, "i16": np.int16}[dst]
        out = np.empty((m, n), out_dt)
        acc = np.ascontiguousarray(acc)
        rc = getattr(self.lib, "ref_store_" + key)(_p(out), _p(acc), m, n, _p(words), int(per_column), int(relu))
        assert rc == 0, rc
        return out

    def global_offsets(self, which, rows, cols):
        """(offsets[rows][cols], shape[5], stride[5]) of ref_global_offset's tensor `which`."""
        sh, st = np.zeros(5, np.int64), np.zeros(5, np.int64)
        out = np.array([[self.lib.ref_global_offset(which, r, c, _p(sh), _p(st)) for c in range(cols)]
                        for r in range(rows)], np.int64)
        return out, sh, st

    def layout_2d(self, layout, rows, cols):
        sh, st = np.zeros(5, np.int64), np.zeros(5, np.int64)
        assert self.lib.ref_layout_2d(layout, rows, cols, _p(sh), _p(st)) == 0
        return sh, st

    def reorder_exp_zz(self, exp):
        exp = np.ascontiguousarray(exp, np.uint8)
        out = np.empty(exp.size, np.uint8)
        self.lib.ref_reorder_exp_zz(_p(out), _p(exp), exp.shape[0], exp.shape[1])
        return out

    def shape(self, shape_id):
        r, c = C.c_int(), C.c_int()
        assert self.lib.ref_shape(shape_id, C.byref(r), C.byref(c)) == 0
        return r.value, c.value

    def tquant_int8(self, shape_id, src, scale, offset=None):
        r, c = self.shape(shape_id)
        out = np.empty((r, c), np.uint8)
        rc = self.lib.ref_tquant_int8(shape_id, int(offset is not None), _p(out), _p(_c(src, np.float32)),
                                      _p(_c(scale, np.float32)), _p(_c(offset, np.float32)))
        assert rc == 0, rc
        return out

    def tquant_mx(self, shape_id, src, alg, axis=1, src_f16=False):
        r, c = self.shape(shape_id)
        fp4 = alg in (OCP_FP4, NV_FP4)
        dst = np.zeros(r * c // 2 if fp4 else r * c, np.uint8)
        gshape = (r, c // 32) if axis == 1 else (r // 32, c)
        exp = np.empty(gshape, np.uint8)
        mx = np.empty(gshape, np.float32)
        sc = np.empty(gshape, np.float32)
        rc = self.lib.ref_tquant_mx(shape_id, alg, axis, int(src_f16), _p(dst), _p(exp), _p(mx), _p(sc),
                                    _p(_c(src, np.float32)))
        assert rc == 0, rc
        return (dst.reshape(r, c // 2) if fp4 else dst.reshape(r, c)), exp, mx, sc

    def tdequant_para(self, src, scale, offset):
        """16 x 64 int8 source, scale / offset [16][para_cols] with para_cols 1, 3 or 8."""
        out = np.empty((16, 64), np.float32)
        scale, offset = _c(scale, np.float32), _c(offset, np.float32)
        rc = self.lib.ref_tdequant_para(scale.shape[1], _p(out), _p(_c(src, np.int8)), _p(scale), _p(offset))
        assert rc == 0, rc
        return out

    def tquant_int8_para(self, src, scale, offset=None):
        """16 x 64 f32 source, scale / offset [para_rows] with para_rows 1, 5 or 16."""
        out = np.empty((16, 64), np.uint8)
        scale = _c(scale, np.float32)
        off = _c(np.zeros_like(scale) if offset is None else offset, np.float32)
        rc = self.lib.ref_tquant_int8_para(scale.size, int(offset is not None), _p(out), _p(_c(src, np.float32)), _p(scale), _p(off))
        assert rc == 0, rc
        return out if offset is not None else out.view(np.int8)

    def tdequant(self, shape_id, src, scale, offset):
        r, c = self.shape(shape_id)
        kind = {np.dtype(np.int8): 0, np.dtype(np.int16): 1, np.dtype(np.int32): 2}[src.dtype]
        out = np.empty((r, c), np.float32)
        rc = self.lib.ref_tdequant(shape_id, kind, _p(out), _p(np.ascontiguousarray(src)), _p(_c(scale, np.float32)),
                                   _p(_c(offset, np.float32)))
        assert rc == 0, rc
        return out
