"""ctypes bindings for the CPU checker -- TEST INFRASTRUCTURE ONLY.

Two libraries are exposed:

* ``Oracle``  -- this repository's scalar restatement (oracle/w8a8_oracle.c).
* ``Reference`` -- the reference's own kernels compiled from its sources
  (oracle/_ref/libvxref.so), when that build exists.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import
this module.  The shipped package (volvoxai_amd) never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
DTYPE_U8 = 5
DTYPE_I8 = 6
OP_PACKED_LINEAR = 1036  # src/generated/operator_vocabulary.h:127
OP_ROTARY_EMBEDDING = 1030  # src/generated/operator_vocabulary.h:121

_f32p = C.POINTER(C.c_float)
_i32p = C.POINTER(C.c_int32)
_u32p = C.POINTER(C.c_uint32)
_i8p = C.POINTER(C.c_int8)
_u8p = C.POINTER(C.c_uint8)


def _ptr(a, ty=C.c_void_p):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be C-contiguous"
    return a.ctypes.data_as(ty)


def _f(v) -> float:
    return float(np.float32(v))


def np_dtype(code: int):
    return np.int8 if code == DTYPE_I8 else np.uint8


def build(force: bool = False) -> None:
    """Compile libvxoracle.so (and _ref/libvxref.so when the tree is there)."""
    if force or not (HERE / "libvxoracle.so").exists():
        subprocess.check_call(["make", "-C", str(HERE), "oracle"])
    if force and Path("/root/reference/native/src/kernels/kernels.c").exists():
        subprocess.check_call(["make", "-C", str(HERE), "ref"])


class Oracle:
    def __init__(self):
        path = HERE / "libvxoracle.so"
        if not path.exists():
            build()
        self.lib = L = C.CDLL(str(path))
        L.vxo_round_ties_even.restype = C.c_int32
        L.vxo_round_ties_even.argtypes = [C.c_float]
        L.vxo_requantize.restype = C.c_int32
        L.vxo_requantize.argtypes = [C.c_float, C.c_int32, C.c_int32, C.c_int32]
        L.vxo_transform_accumulator.restype = C.c_float
        L.vxo_transform_accumulator.argtypes = [C.c_int64, C.c_float, C.c_int32]
        L.vxo_multiplier.restype = C.c_int
        L.vxo_multiplier.argtypes = [C.c_float, C.c_float, C.c_float, _f32p]
        L.vxo_packed_round_i8.restype = C.c_int32
        L.vxo_packed_round_i8.argtypes = [C.c_float]
        L.vxo_qlinear_i8u8.restype = C.c_int
        L.vxo_qlinear_i8u8.argtypes = [
            C.c_void_p, C.c_void_p, _i32p, _f32p, _i32p, C.c_void_p, _i32p,
            C.c_uint32, C.c_uint32, C.c_uint32, C.c_float, C.c_int32,
            C.c_float, C.c_int32, C.c_uint32, C.c_uint32, C.c_uint32]
        L.vxo_qlinear_rowscale_i8u8.restype = C.c_int
        L.vxo_qlinear_rowscale_i8u8.argtypes = [
            _i8p, C.c_void_p, _i32p, _f32p, _f32p, _i32p, C.c_void_p, _i32p,
            C.c_uint32, C.c_uint32, C.c_uint32, _f32p, C.c_float, C.c_int32,
            C.c_uint32, C.c_uint32]
        L.vxo_packed_prepare_i8.restype = C.c_int
        L.vxo_packed_prepare_i8.argtypes = [_f32p, C.c_uint32, _i8p, _f32p]
        L.vxo_packed_linear_forward.restype = C.c_int
        L.vxo_packed_linear_forward.argtypes = [
            _f32p, _u32p, _f32p, _f32p, _f32p, C.c_uint64, C.c_uint32,
            C.c_uint32, C.c_uint32]
        L.vxo_packed_linear_a8.restype = C.c_int
        L.vxo_packed_linear_a8.argtypes = [
            _i8p, _f32p, _u8p, _u32p, _f32p, _f32p, _f32p, _i32p, C.c_uint64,
            C.c_uint32, C.c_uint32, C.c_uint32]
        L.vxo_quantize_linear.restype = C.c_int
        L.vxo_quantize_linear.argtypes = [
            _f32p, C.c_uint32, C.c_void_p, C.c_float, C.c_int32, C.c_uint32]
        L.vxo_requantize_linear.restype = C.c_int
        L.vxo_requantize_linear.argtypes = [C.c_void_p, C.c_uint32, C.c_float, C.c_int32, C.c_float, C.c_int32,
                                            C.c_uint32, C.c_uint32, C.c_void_p]
        L.vxo_dequantize_linear.restype = C.c_int
        L.vxo_dequantize_linear.argtypes = [
            C.c_void_p, C.c_uint32, C.c_float, C.c_int32, C.c_uint32, _f32p]
        L.vxo_ptq_symmetric_scale.restype = C.c_int
        L.vxo_ptq_symmetric_scale.argtypes = [_f32p, C.c_int64, _f32p]
        L.vxo_ptq_quantize_i8.restype = C.c_int
        L.vxo_ptq_quantize_i8.argtypes = [_f32p, C.c_int64, C.c_float, C.c_int32, _i8p]
        L.vxo_ptq_pack_bias_i32.restype = C.c_int
        L.vxo_ptq_pack_bias_i32.argtypes = [_f32p, C.c_int32, C.c_float, _f32p, _i32p]
        L.vxo_pack_w8_words.restype = None
        L.vxo_pack_w8_words.argtypes = [_i8p, C.c_uint32, C.c_uint32, _u32p]
        L.vxo_pack_w4_words.restype = None
        L.vxo_pack_w4_words.argtypes = [_i8p, C.c_uint32, C.c_uint32, _u32p]
        L.vxo_packed_linear_forward_bits.restype = C.c_int
        L.vxo_packed_linear_forward_bits.argtypes = (
            list(L.vxo_packed_linear_forward.argtypes) + [C.c_uint32])
        L.vxo_packed_linear_forward_window.restype = C.c_int
        L.vxo_packed_linear_forward_window.argtypes = (
            list(L.vxo_packed_linear_forward.argtypes) + [C.c_uint32, C.c_uint64, C.c_uint64])
        L.vxo_packed_linear_a8_bits.restype = C.c_int
        L.vxo_packed_linear_a8_bits.argtypes = (
            list(L.vxo_packed_linear_a8.argtypes) + [C.c_uint32])

    # -- scalar helpers ---------------------------------------------------
    def round_ties_even(self, v):
        return int(self.lib.vxo_round_ties_even(_f(v)))

    def requantize(self, v, lo, hi, nan_value):
        return int(self.lib.vxo_requantize(_f(v), lo, hi, nan_value))

    def multiplier(self, s_in, s_w, s_out):
        out = C.c_float(0)
        ok = self.lib.vxo_multiplier(_f(s_in), _f(s_w),
                                     _f(s_out), C.byref(out))
        return (bool(ok), np.float32(out.value))

    def packed_round_i8(self, v):
        return int(self.lib.vxo_packed_round_i8(_f(v)))

    # -- QLinear ----------------------------------------------------------
    def qlinear(self, x, w, bias, w_scales, w_zps, s_in, zp_in, s_out, zp_out,
                in_dtype, w_dtype, out_dtype, want_acc=False):
        rows, k = x.shape
        n = w.shape[0]
        y = np.zeros((rows, n), dtype=np_dtype(out_dtype))
        acc = np.zeros((rows, n), dtype=np.int32) if want_acc else None
        ok = self.lib.vxo_qlinear_i8u8(
            _ptr(x), _ptr(w), _ptr(bias, _i32p), _ptr(w_scales, _f32p),
            _ptr(w_zps, _i32p), _ptr(y), _ptr(acc, _i32p), rows, k, n,
            _f(s_in), int(zp_in), _f(s_out), int(zp_out),
            in_dtype, w_dtype, out_dtype)
        return (int(ok), y, acc) if want_acc else (int(ok), y)

    def qlinear_rowscale(self, x, w, w_scales, w_zps, row_scales, s_out, zp_out,
                         w_dtype=DTYPE_I8, out_dtype=DTYPE_I8, bias_i32=None,
                         bias_f32=None):
        rows, k = x.shape
        n = w.shape[0]
        y = np.zeros((rows, n), dtype=np_dtype(out_dtype))
        acc = np.zeros((rows, n), dtype=np.int32)
        ok = self.lib.vxo_qlinear_rowscale_i8u8(
            _ptr(x, _i8p), _ptr(w), _ptr(bias_i32, _i32p), _ptr(bias_f32, _f32p),
            _ptr(w_scales, _f32p), _ptr(w_zps, _i32p), _ptr(y), _ptr(acc, _i32p),
            rows, k, n, _ptr(row_scales, _f32p), _f(s_out), int(zp_out),
            w_dtype, out_dtype)
        return int(ok), y, acc

    # -- PackedLinear -----------------------------------------------------
    def packed_prepare(self, x):
        rows, k = x.shape
        a = np.zeros((rows, k), dtype=np.int8)
        s = np.zeros(rows, dtype=np.float32)
        fin = np.zeros(rows, dtype=np.uint8)
        for r in range(rows):
            sc = C.c_float(0)
            fin[r] = self.lib.vxo_packed_prepare_i8(
                _ptr(x[r], _f32p), k, _ptr(a[r], _i8p), C.byref(sc))
            s[r] = sc.value
        return a, s, fin

    def packed_linear(self, x, packed, scales, bias, n, group, bits=8):
        rows, k = x.shape
        y = np.zeros((rows, n), dtype=np.float32)
        st = self.lib.vxo_packed_linear_forward_bits(
            _ptr(x, _f32p), _ptr(packed, _u32p), _ptr(scales, _f32p),
            _ptr(bias, _f32p), _ptr(y, _f32p), rows, k, n, group, bits)
        return st, y

    def packed_linear_window(self, x, packed, scales, bias, out, group, first_unit, unit_count, bits=8):
        """Writes the window's elements of `out` [rows, n] in place; returns the status."""
        rows, k = x.shape
        return self.lib.vxo_packed_linear_forward_window(
            _ptr(x, _f32p), _ptr(packed, _u32p), _ptr(scales, _f32p), _ptr(bias, _f32p), _ptr(out, _f32p),
            rows, k, out.shape[1], group, bits, int(first_unit), int(unit_count))

    def packed_linear_a8(self, a, row_scales, packed, scales, bias, n, group,
                         row_finite=None, bits=8):
        rows, k = a.shape
        y = np.zeros((rows, n), dtype=np.float32)
        acc = np.zeros((rows, n), dtype=np.int32)
        st = self.lib.vxo_packed_linear_a8_bits(
            _ptr(a, _i8p), _ptr(row_scales, _f32p), _ptr(row_finite, _u8p),
            _ptr(packed, _u32p), _ptr(scales, _f32p), _ptr(bias, _f32p),
            _ptr(y, _f32p), _ptr(acc, _i32p), rows, k, n, group, bits)
        return st, y, acc

    def pack_low_bit_words(self, w, bits):
        n, k = w.shape
        words = (k // 32) * bits + ((k % 32) * bits + 31) // 32
        out = np.zeros((n, words), dtype=np.uint32)
        self.lib.vxo_pack_low_bit_words.restype = None
        self.lib.vxo_pack_low_bit_words(_ptr(w, _i8p), C.c_uint32(n), C.c_uint32(k), C.c_uint32(bits),
                                        _ptr(out, _u32p))
        return out

    def pack_w4_words(self, w):
        n, k = w.shape
        words = (k // 32) * 4 + ((k % 32) * 4 + 31) // 32
        out = np.zeros((n, words), dtype=np.uint32)
        self.lib.vxo_pack_w4_words(_ptr(w, _i8p), n, k, _ptr(out, _u32p))
        return out

    def pack_w8_words(self, w):
        n, k = w.shape
        out = np.zeros((n, (k + 3) // 4), dtype=np.uint32)
        self.lib.vxo_pack_w8_words(_ptr(w, _i8p), n, k, _ptr(out, _u32p))
        return out

    # -- boundaries / PTQ ---------------------------------------------------
    def quantize(self, x, scale, zp, dtype):
        out = np.zeros(x.shape, dtype=np_dtype(dtype))
        ok = self.lib.vxo_quantize_linear(_ptr(x, _f32p), x.size, _ptr(out),
                                          _f(scale), int(zp), dtype)
        return int(ok), out

    def dequantize(self, q, scale, zp, dtype):
        out = np.zeros(q.shape, dtype=np.float32)
        ok = self.lib.vxo_dequantize_linear(_ptr(q), q.size, _f(scale),
                                            int(zp), dtype, _ptr(out, _f32p))
        return int(ok), out

    def requantize_linear(self, q, s_in, zp_in, s_out, zp_out, in_dtype, out_dtype):
        out = np.zeros(q.shape, dtype=np_dtype(out_dtype))
        ok = self.lib.vxo_requantize_linear(_ptr(q), q.size, _f(s_in), int(zp_in), _f(s_out), int(zp_out),
                                            in_dtype, out_dtype, _ptr(out))
        return int(ok), out

    def ptq_symmetric_scale(self, x):
        s = C.c_float(0)
        st = self.lib.vxo_ptq_symmetric_scale(_ptr(x, _f32p), x.size, C.byref(s))
        assert st == 0
        return np.float32(s.value)

    def ptq_quantize_i8(self, x, scale, zp=0):
        out = np.zeros(x.shape, dtype=np.int8)
        st = self.lib.vxo_ptq_quantize_i8(_ptr(x, _f32p), x.size, _f(scale),
                                          int(zp), _ptr(out, _i8p))
        assert st == 0
        return out

    def embedding(self, tokens, table):
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        out = np.zeros((tokens.size, table.shape[1]), dtype=np.float32)
        self.lib.vxo_embedding_f32.restype = None
        self.lib.vxo_embedding_f32(tokens.ctypes.data_as(C.c_void_p), _ptr(table, _f32p), _ptr(out, _f32p),
                                   C.c_uint32(tokens.size), C.c_uint32(table.shape[1]))
        return out

    def argmax_rows(self, x):
        out = np.zeros(x.shape[0], dtype=np.int32)
        self.lib.vxo_argmax_rows_f32.restype = None
        self.lib.vxo_argmax_rows_f32(_ptr(x, _f32p), C.c_uint32(x.shape[0]), C.c_uint32(x.shape[1]),
                                     _ptr(out, _i32p))
        return out

    def ptq_pack_bias(self, b, s_in, w_scales):
        out = np.zeros(b.shape, dtype=np.int32)
        st = self.lib.vxo_ptq_pack_bias_i32(_ptr(b, _f32p), b.size, _f(s_in),
                                            _ptr(w_scales, _f32p), _ptr(out, _i32p))
        return st, out


def packed_linear_a8_blocked(a8, row_scales, w, scales, bias, group):
    """PackedLinear / DYNAMIC_I8 from prepared activations, vectorised for shapes the scalar C
    restatement would take minutes on (TEST INFRASTRUCTURE like the rest of this module).

    The same rule as vxo_packed_linear_a8 (src/kernels/packed_linear_ops.inc:1498-1504, :1533):
    per storage group g in ascending order  sum = f32(sum + f32(f32(dot_g) * f32(s_a * s_w[n][g]))),
    then  y = f32(sum + bias[n]).  The group dots are exact: int8 products summed in float64
    through BLAS stay below 2^53 by a wide margin (|dot_g| <= 256 * 127 * 128).  numpy's float32
    arithmetic is one IEEE rounding per operation and never fused.

    a8 int8 [rows, k], row_scales f32 [rows], w int8 [n, k] (the signed weights, not the packed
    words), scales f32 [n, ceil(k/group)], bias f32 [n] or None.  Returns (y f32 [rows, n],
    acc int64 [rows, n] = the full-K sums).  Rows with a NaN scale give NaN rows."""
    rows, k = a8.shape
    n = w.shape[0]
    groups = (k + group - 1) // group
    assert scales.shape == (n, groups)
    total = np.zeros((rows, n), dtype=np.float32)
    acc = np.zeros((rows, n), dtype=np.int64)
    rs = row_scales.astype(np.float32)[:, None]
    with np.errstate(invalid="ignore"):
        for g in range(groups):
            lo, hi = g * group, min(k, (g + 1) * group)
            dot = a8[:, lo:hi].astype(np.float64) @ w[:, lo:hi].astype(np.float64).T
            acc += dot.astype(np.int64)
            gs = (rs * scales[None, :, g].astype(np.float32)).astype(np.float32)
            term = (dot.astype(np.float32) * gs).astype(np.float32)
            total = (total + term).astype(np.float32)
        if bias is not None:
            total = (total + bias.astype(np.float32)[None, :]).astype(np.float32)
    total[np.isnan(row_scales)] = np.nan
    return total, acc


class _LLMOpArgs(C.Structure):
    """Field order of VxLLMOpArgs (src/kernels/llm_ops.h:38-53)."""
    _fields_ = [(n, C.c_int32) for n in (
        "kind", "batch", "sequence", "keys", "heads", "kv_heads", "key_dim",
        "value_dim", "streams", "groups", "rate", "window", "top_k",
        "iterations", "index_heads", "index_dim", "rotary_dim", "rotary_offset",
        "normalize", "causal", "interleaved", "mask_mode")] + [
        ("eps", C.c_float), ("hc_eps", C.c_float), ("scale", C.c_float),
        ("x", C.c_void_p * 8), ("y", C.c_void_p * 3),
        ("mask", C.c_void_p), ("positions", C.c_void_p),
        ("x_elements", C.c_uint64 * 8), ("y_elements", C.c_uint64 * 3),
        ("mask_elements", C.c_uint64), ("position_elements", C.c_uint64),
        ("query_offset", C.c_int32),
        ("first_unit", C.c_uint64), ("unit_count", C.c_uint64)]


class _Scope(C.Structure):
    _fields_ = [("previous", C.c_void_p), ("bound", C.c_void_p), ("retained", C.c_int)]


class Reference:
    """The reference's own C kernels (compiled from its sources into _ref/)."""

    PATH = HERE / "_ref" / "libvxref.so"

    @classmethod
    def available(cls) -> bool:
        return cls.PATH.exists()

    def __init__(self):
        self.lib = L = C.CDLL(str(self.PATH))
        sig = [C.c_void_p, C.c_void_p, _i32p, _f32p, _i32p, C.c_void_p,
               C.c_uint32, C.c_uint32, C.c_uint32, C.c_float, C.c_int32,
               C.c_float, C.c_int32, C.c_uint32, C.c_uint32, C.c_uint32]
        for name in ("qlinear_i8u8", "vx_qlinear_i8u8_native", "vx_qlinear_i8u8_packed"):
            fn = getattr(L, name)
            fn.restype = C.c_int
            fn.argtypes = sig
        L.vx_packed_q8_weight_size.restype = C.c_uint32
        L.vx_packed_q8_weight_size.argtypes = [C.c_uint32, C.c_uint32]
        L.vx_pack_q8_weight.restype = C.c_int
        L.vx_pack_q8_weight.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p,
                                        C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32]
        L.vx_packed_q8_preferred_for_native_w8a8.restype = C.c_int
        L.vx_packed_q8_preferred_for_native_w8a8.argtypes = [
            C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_int]
        L.vx_llm_forward_f32.restype = C.c_int
        L.vx_llm_forward_f32.argtypes = [C.POINTER(_LLMOpArgs)]
        L.quantize_linear_typed.restype = C.c_int
        L.quantize_linear_typed.argtypes = [_f32p, _f32p, C.c_void_p, C.c_uint32,
                                            C.c_void_p, C.c_uint32, C.c_uint32]
        L.dequantize_linear_typed.restype = C.c_int
        L.dequantize_linear_typed.argtypes = [C.c_void_p, C.c_int, _f32p, C.c_void_p,
                                              C.c_int, _f32p, C.c_int]
        L.requantize_linear_i8u8.restype = C.c_int
        L.requantize_linear_i8u8.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_float, C.c_int32, C.c_float,
                                             C.c_int32, C.c_uint32, C.c_uint32]
        L.vx_kernel_thread_pool_create.restype = C.c_void_p
        L.vx_kernel_thread_pool_create.argtypes = [C.c_int]
        L.vx_kernel_thread_pool_destroy.argtypes = [C.c_void_p]
        L.vx_kernel_thread_pool_scope_enter.restype = _Scope
        L.vx_kernel_thread_pool_scope_enter.argtypes = [C.c_void_p]
        L.vx_kernel_thread_pool_scope_leave.argtypes = [_Scope]
        L.vx_kernels_thread_count.restype = C.c_int
        L.volvoxai_ptq_pack_bias_i32.restype = C.c_int
        L.volvoxai_ptq_pack_bias_i32.argtypes = [_f32p, C.c_int32, C.c_float,
                                                 _f32p, C.c_int32, _i32p]
        self._pool = None
        self._scope = None

    # thread pool (src/kernels/thread_pool.h:20-54) -------------------------
    def enter_pool(self, threads: int) -> int:
        self.leave_pool()
        self._pool = self.lib.vx_kernel_thread_pool_create(threads)
        if not self._pool:
            return 1
        self._scope = self.lib.vx_kernel_thread_pool_scope_enter(self._pool)
        return int(self.lib.vx_kernels_thread_count())

    def leave_pool(self):
        if self._scope is not None:
            self.lib.vx_kernel_thread_pool_scope_leave(self._scope)
            self._scope = None
        if self._pool:
            self.lib.vx_kernel_thread_pool_destroy(self._pool)
            self._pool = None

    # QLinear --------------------------------------------------------------
    def _qcall(self, fn, x, w, bias, w_scales, w_zps, s_in, zp_in, s_out, zp_out,
               in_dtype, w_dtype, out_dtype):
        rows, k = x.shape
        n = w_scales.shape[0]
        y = np.zeros((rows, n), dtype=np_dtype(out_dtype))
        ok = fn(_ptr(x), _ptr(w), _ptr(bias, _i32p), _ptr(w_scales, _f32p),
                _ptr(w_zps, _i32p), _ptr(y), rows, k, n, _f(s_in),
                int(zp_in), _f(s_out), int(zp_out), in_dtype, w_dtype,
                out_dtype)
        return int(ok), y

    def qlinear_portable(self, *a):
        return self._qcall(self.lib.qlinear_i8u8, *a)

    def qlinear_native(self, *a):
        return self._qcall(self.lib.vx_qlinear_i8u8_native, *a)

    def pack_q8(self, w, w_dtype):
        n, k = w.shape
        size = self.lib.vx_packed_q8_weight_size(k, n)
        buf = np.zeros(size, dtype=np.uint8)
        ok = self.lib.vx_pack_q8_weight(_ptr(buf), size, _ptr(w), k, n, w_dtype, 1)
        assert ok, "reference pack failed"
        return buf

    def qlinear_packed(self, x, packed, bias, w_scales, w_zps, *rest):
        return self._qcall(self.lib.vx_qlinear_i8u8_packed, x, packed, bias,
                           w_scales, w_zps, *rest)

    def requantize_linear(self, q, s_in, zp_in, s_out, zp_out, in_dtype, out_dtype):
        """requantize_linear_i8u8 of the reference build (portable_inference_kernels.inc:2437-2463)."""
        out = np.zeros(q.shape, dtype=np_dtype(out_dtype))
        ok = self.lib.requantize_linear_i8u8(_ptr(q), _ptr(out), q.size, _f(s_in), int(zp_in), _f(s_out), int(zp_out),
                                             in_dtype, out_dtype)
        return int(ok), out

    def packed_preferred(self, rows, k, n, w_dtype, zero_zp):
        return int(self.lib.vx_packed_q8_preferred_for_native_w8a8(
            rows, k, n, w_dtype, int(zero_zp)))

    # PackedLinear -----------------------------------------------------------
    def packed_linear(self, x, packed, scales, bias, n, group, bits=8, first_unit=0, unit_count=0, out=None):
        """vx_llm_forward_f32 on a PackedLinear node; with `out` given it is written in place, so a
        window (first_unit, unit_count) shows what the reference leaves untouched."""
        rows, k = x.shape
        y = np.zeros((rows, n), dtype=np.float32) if out is None else out
        a = _LLMOpArgs()
        a.first_unit, a.unit_count = int(first_unit), int(unit_count)
        a.kind = OP_PACKED_LINEAR
        a.batch, a.sequence = 1, rows
        a.key_dim, a.value_dim = k, n
        a.groups, a.rate, a.normalize = bits, group, 8
        a.x[0] = x.ctypes.data
        a.x[1] = packed.ctypes.data
        a.x[2] = scales.ctypes.data
        a.x[3] = bias.ctypes.data if bias is not None else None
        a.y[0] = y.ctypes.data
        a.x_elements[0] = x.size
        a.x_elements[1] = packed.size
        a.x_elements[2] = scales.size
        a.x_elements[3] = bias.size if bias is not None else 0
        a.y_elements[0] = y.size
        st = self.lib.vx_llm_forward_f32(C.byref(a))
        return int(st), y

    # decoder glue ----------------------------------------------------------------
    def rmsnorm(self, x, gain, eps):
        """rmsnorm_f32 (src/kernels/softmax_rmsnorm.inc:3-17)."""
        out = np.zeros_like(x)
        self.lib.rmsnorm_f32.restype = None
        self.lib.rmsnorm_f32.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_double]
        self.lib.rmsnorm_f32(_ptr(x, _f32p), _ptr(gain, _f32p), _ptr(out, _f32p), x.shape[0], x.shape[1], float(eps))
        return out

    def silu_mul(self, gate, up):
        """silu_f32 then mul_f32 (src/kernels/elementwise_f32.inc:153-165): the SiLU and Mul nodes of a SwiGLU."""
        gate, up = np.ascontiguousarray(gate), np.ascontiguousarray(up)
        act, out = np.zeros_like(gate), np.zeros_like(gate)
        self.lib.silu_f32.restype = None
        self.lib.silu_f32.argtypes = [_f32p, _f32p, C.c_int]
        self.lib.silu_f32(_ptr(gate, _f32p), _ptr(act, _f32p), gate.size)
        self.lib.mul_f32.restype = None
        self.lib.mul_f32.argtypes = [_f32p, _f32p, _f32p, C.c_int]
        self.lib.mul_f32(_ptr(act, _f32p), _ptr(up, _f32p), _ptr(out, _f32p), gate.size)
        return out

    def rotary(self, x, cos, sin):
        """The RotaryEmbedding operator of vx_llm_forward_f32 (src/kernels/llm_math.h:256-274), half-split
        pairs over the whole head: x [tokens, heads, d], cos and sin [tokens, d]."""
        tokens, heads, d = x.shape
        y = np.zeros_like(x)
        a = _LLMOpArgs()
        a.kind = OP_ROTARY_EMBEDDING
        a.batch, a.sequence, a.heads, a.key_dim = 1, tokens, heads, d
        a.rotary_dim, a.rotary_offset, a.interleaved = d, 0, 0
        a.x[0], a.x[1], a.x[2] = x.ctypes.data, cos.ctypes.data, sin.ctypes.data
        a.y[0] = y.ctypes.data
        a.x_elements[0], a.x_elements[1], a.x_elements[2] = x.size, cos.size, sin.size
        a.y_elements[0] = y.size
        st = self.lib.vx_llm_forward_f32(C.byref(a))
        return int(st), y

    def attention(self, q, k, v, q_heads, kv_heads, head_dim, causal):
        """cross_sdpa_gqa_f32 (src/kernels/cross_sdpa.inc:53) with scale f32(1/sqrt(head_dim)), no mask."""
        out = np.zeros((q.shape[0], q_heads * head_dim), dtype=np.float32)
        self.lib.cross_sdpa_gqa_f32.restype = None
        self.lib.cross_sdpa_gqa_f32.argtypes = [_f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                                C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_int, C.c_int]
        self.lib.cross_sdpa_gqa_f32(_ptr(q, _f32p), _ptr(k, _f32p), _ptr(v, _f32p), _ptr(out, _f32p), q.shape[0], k.shape[0],
                                    q.shape[1], k.shape[1], q_heads, kv_heads, head_dim,
                                    float(np.float32(1.0 / np.sqrt(head_dim))), None, 0, int(causal))
        return out

    def embedding(self, tokens, table):
        """embedding_f32 (src/kernels/embedding.inc:5-16); pointers travel as integers."""
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        out = np.zeros((tokens.size, table.shape[1]), dtype=np.float32)
        self.lib.embedding_f32.restype = None
        self.lib.embedding_f32(C.c_size_t(tokens.ctypes.data), C.c_size_t(table.ctypes.data),
                               C.c_size_t(out.ctypes.data), C.c_int(tokens.size), C.c_int(table.shape[1]))
        return out

    def argmax_rows(self, x):
        """argmax_f32 (src/kernels/reduction_argmax.inc:237-240): indices come back as f32."""
        out = np.zeros(x.shape[0], dtype=np.float32)
        self.lib.argmax_f32.restype = None
        self.lib.argmax_f32(_ptr(x, _f32p), _ptr(out, _f32p), C.c_int(x.shape[0]), C.c_int(x.shape[1]))
        return out.astype(np.int32)

    def ptq_pack_bias(self, b, s_in, w_scales):
        out = np.zeros(b.shape, dtype=np.int32)
        st = self.lib.volvoxai_ptq_pack_bias_i32(
            _ptr(b, _f32p), b.size, _f(s_in), _ptr(w_scales, _f32p),
            b.size, _ptr(out, _i32p))
        return int(st), out
