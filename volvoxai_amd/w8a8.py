"""Host-side mirror of the reference's W8A8 device-op interface over the C ABI.

Names and argument order follow the reference slots they stand in for:
``qlinear_i8u8`` is VxQLinearI8U8Fn (native/src/backends/w8a8_device_ops.h:15-17),
``quantize_typed_f32_i8u8`` / ``dequantize_typed_i8u8_f32`` are :31-32, and
``packed_linear_f32`` takes the PackedLinear fields of VxLLMOpArgs
(native/src/kernels/llm_ops.h:22-32).  Resident classes (Context, QLinear,
PackedLinear) take torch CUDA tensors, which only supply device addresses.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from ._lib import library

DTYPE_U8 = 5
DTYPE_I8 = 6


class VxHipError(RuntimeError):
    pass


def _err() -> str:
    return library().vxhip_last_error().decode(errors="replace")


def _check(status: int, what: str) -> None:
    if status != 0:
        raise VxHipError(f"{what} failed with status {status}: {_err()}")


def _np(a, dtype=None):
    a = np.ascontiguousarray(a if dtype is None else np.asarray(a, dtype=dtype))
    return a


def _hp(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _dp(t, name="tensor", dtype=None, shape=None, numel=None, min_numel=None):
    """Device address of a contiguous torch tensor, after checking what the library cannot: it
    receives a bare address, so a tensor of the wrong type or extent would be read or written out
    of bounds on the device.  `dtype` is a torch dtype or a tuple of them."""
    if t is None:
        return None
    if not (t.is_cuda and t.is_contiguous()):
        raise ValueError(f"{name}: expected a contiguous device tensor")
    if dtype is not None and t.dtype not in (dtype if isinstance(dtype, tuple) else (dtype,)):
        raise ValueError(f"{name}: dtype {t.dtype}, expected {dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name}: shape {tuple(t.shape)}, expected {tuple(shape)}")
    if numel is not None and t.numel() != numel:
        raise ValueError(f"{name}: {t.numel()} elements, expected {numel}")
    if min_numel is not None and t.numel() < min_numel:
        raise ValueError(f"{name}: {t.numel()} elements, at least {min_numel} are needed")
    return C.c_void_p(t.data_ptr())


def _byte_dtype(code, name):
    if code not in (DTYPE_I8, DTYPE_U8):
        raise ValueError(f"{name}: dtype id {code} is neither I8 ({DTYPE_I8}) nor U8 ({DTYPE_U8})")
    return _torch_dtype(code)


def _torch_dtype(code):
    import torch
    return torch.int8 if code == DTYPE_I8 else torch.uint8


class Context:
    """Context scope: one stream plus mutable scratch (one thread at a time)."""

    def __init__(self, device: int = 0, stream=None):
        self._h = C.c_void_p()
        self._stream = stream
        if stream is not None:  # borrow the caller's stream (handle 0 is the default stream)
            raw, flags = C.c_void_p(stream.cuda_stream), 1
        else:
            raw, flags = None, 0
        _check(library().vxhip_context_create(device, raw, flags, C.byref(self._h)), "vxhip_context_create")

    def close(self):
        if self._h:
            library().vxhip_context_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def synchronize(self):
        _check(library().vxhip_context_synchronize(self._h), "vxhip_context_synchronize")

    @property
    def last_variant(self) -> str:
        return library().vxhip_context_last_variant(self._h).decode()

    def set_activation_layout(self, operand_order: bool):
        """Prepared activations of calls with up to 32 rows in the GEMV's operand order (True) or
        row major (False, the default); see vxhip_context_set_activation_layout."""
        _check(library().vxhip_context_set_activation_layout(self._h, 1 if operand_order else 0),
               "vxhip_context_set_activation_layout")

    def prepared_buffer(self, rows: int, k: int, device):
        """An int8 buffer for the prepared codes of rows x k in this context's layout: [rows, k] row
        major, or flat (32 * ceil(k/16) * 16 bytes) in operand order."""
        import torch
        nbytes = library().vxhip_context_prepared_bytes(self._h, rows, k)
        if nbytes == rows * k:
            return torch.empty((rows, k), dtype=torch.int8, device=device)
        return torch.empty((nbytes,), dtype=torch.int8, device=device)

    def fault_flags(self) -> int:
        v = C.c_uint32(0)
        _check(library().vxhip_context_fault_flags(self._h, C.byref(v)), "vxhip_context_fault_flags")
        return v.value

    def clear_fault_flags(self):
        _check(library().vxhip_context_clear_fault_flags(self._h), "vxhip_context_clear_fault_flags")

    def begin_recording(self):
        """From here to end_recording() the launches of this context's entry points are recorded, not run."""
        _check(library().vxhip_context_begin_recording(self._h), "context_begin_recording")

    def end_recording(self) -> "Replay":
        handle = C.c_void_p()
        _check(library().vxhip_context_end_recording(self._h, C.byref(handle)), "context_end_recording")
        return Replay(handle)

    def reserve_scratch(self, nbytes: int):
        _check(library().vxhip_context_reserve_scratch(self._h, int(nbytes)), "vxhip_context_reserve_scratch")

    def probe_mfma_rate(self, rounds=128, random_operands=True, k64=False) -> dict:
        """Register-only MFMA loop: the int8 rate, shader clock and time it reached (k64: on the
        16x16x64 instruction instead of the 32x32x32 one)."""
        tops, mhz, us = C.c_double(0), C.c_double(0), C.c_double(0)
        _check(library().vxhip_probe_mfma_rate(self._h, int(rounds), (1 if random_operands else 0) | (2 if k64 else 0), C.byref(tops),
                                               C.byref(mhz), C.byref(us)), "vxhip_probe_mfma_rate")
        return {"tops": tops.value, "shader_mhz": mhz.value, "microseconds": us.value}

    def probe_mfma_valu_overlap(self, rounds=2000, constant_operands=False) -> dict:
        """Time and clock of the MFMAs alone, the folds alone, both in every wave, and split over
        alternate waves (vxhip_probe_mfma_valu_overlap), on random operand bytes or on ones."""
        us, mhz = (C.c_double * 4)(), (C.c_double * 4)()
        _check(library().vxhip_probe_mfma_valu_overlap(self._h, rounds, 1 if constant_operands else 0, us, mhz),
               "vxhip_probe_mfma_valu_overlap")
        names = ("mfma_only", "folds_only", "both_in_every_wave", "mfma_waves_beside_fold_waves_half_the_work_each")
        return {n: {"microseconds": us[i], "shader_mhz": mhz[i]} for i, n in enumerate(names)}

    def probe_stream_read(self, buffers, launches=60) -> dict:
        """A kernel that only reads, one whole buffer (device tensors of equal size, rotated) per
        launch: the rate and time per launch the memory system gives a kernel of that size."""
        nbytes = buffers[0].numel() * buffers[0].element_size()
        if any(b.numel() * b.element_size() != nbytes for b in buffers):
            raise ValueError("probe_stream_read: buffers differ in size")
        pointers = (C.c_void_p * len(buffers))(*[b.data_ptr() for b in buffers])
        gbs, us = C.c_double(0), C.c_double(0)
        _check(library().vxhip_probe_stream_read(self._h, pointers, len(buffers), nbytes, int(launches), C.byref(gbs),
                                                 C.byref(us)), "vxhip_probe_stream_read")
        return {"GBs": gbs.value, "microseconds": us.value, "bytes": nbytes // 16 * 16, "buffers_rotated": len(buffers)}


class QLinear:
    """Compiled scope of one QLinear/QMatMul/QGemm node: prepacked weights."""

    def __init__(self, weight, weight_scales, weight_zero_points, bias=None, weight_dtype=DTYPE_I8):
        w = _np(weight)
        assert w.ndim == 2 and w.dtype in (np.int8, np.uint8)
        self.d_out, self.d_in = w.shape
        s = _np(weight_scales, np.float32)
        z = _np(weight_zero_points, np.int32)
        b = None if bias is None else _np(bias, np.int32)
        self._h = C.c_void_p()
        _check(library().vxhip_qlinear_create(_hp(w), _hp(s), _hp(z), _hp(b), self.d_in, self.d_out,
                                               weight_dtype, C.byref(self._h)), "vxhip_qlinear_create")

    def close(self):
        if self._h:
            library().vxhip_qlinear_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def resident_bytes(self) -> int:
        return int(library().vxhip_qlinear_resident_bytes(self._h))

    def forward(self, ctx: Context, x, input_scale, input_zero_point, output_scale,
                output_zero_point, input_dtype=DTYPE_I8, output_dtype=DTYPE_I8, out=None,
                want_accumulators=False, accumulators=None):
        import torch
        if x.ndim != 2 or x.shape[1] != self.d_in:
            raise ValueError(f"x: shape {tuple(x.shape)}, expected [rows, {self.d_in}]")
        rows = x.shape[0]
        in_t, out_t = _byte_dtype(input_dtype, "input_dtype"), _byte_dtype(output_dtype, "output_dtype")
        if out is None:
            out = torch.empty((rows, self.d_out), dtype=out_t, device=x.device)
        if want_accumulators and accumulators is None:
            accumulators = torch.empty((rows, self.d_out), dtype=torch.int32, device=x.device)
        ok = library().vxhip_qlinear_forward(
            ctx._h, self._h, _dp(x, "x", in_t), _dp(out, "out", out_t, (rows, self.d_out)),
            _dp(accumulators, "accumulators", torch.int32, (rows, self.d_out)), rows, float(np.float32(input_scale)),
            int(input_zero_point), float(np.float32(output_scale)), int(output_zero_point),
            input_dtype, output_dtype)
        return (ok, out, accumulators) if want_accumulators else (ok, out)

    def forward_dequantized(self, ctx: Context, x, input_scale, input_zero_point, output_scale, output_zero_point,
                            input_dtype=DTYPE_I8, output_dtype=DTYPE_I8, dequant_scale=None, dequant_zero_point=None,
                            out=None, want_bytes=False):
        """QLinear and the DequantizeLinear behind it in one launch: returns (ok, f32 [rows, d_out][, bytes]).
        The dequantization parameters default to the output's own."""
        import torch
        if x.ndim != 2 or x.shape[1] != self.d_in:
            raise ValueError(f"x: shape {tuple(x.shape)}, expected [rows, {self.d_in}]")
        rows = x.shape[0]
        in_t, out_t = _byte_dtype(input_dtype, "input_dtype"), _byte_dtype(output_dtype, "output_dtype")
        if out is None:
            out = torch.empty((rows, self.d_out), dtype=torch.float32, device=x.device)
        q = torch.empty((rows, self.d_out), dtype=out_t, device=x.device) if want_bytes else None
        ok = library().vxhip_qlinear_forward_dequantized(
            ctx._h, self._h, _dp(x, "x", in_t), _dp(out, "out", torch.float32, (rows, self.d_out)),
            _dp(q, "bytes", out_t, (rows, self.d_out)), rows, float(np.float32(input_scale)), int(input_zero_point),
            float(np.float32(output_scale)), int(output_zero_point), input_dtype, output_dtype,
            float(np.float32(output_scale if dequant_scale is None else dequant_scale)),
            int(output_zero_point if dequant_zero_point is None else dequant_zero_point))
        return (ok, out, q) if want_bytes else (ok, out)

    def forward_f32(self, ctx: Context, x, input_scale, input_zero_point, output_scale, output_zero_point,
                    input_dtype=DTYPE_I8, output_dtype=DTYPE_I8, want_f32=True, want_bytes=False):
        """QuantizeLinear -> QLinear [-> DequantizeLinear] on f32 rows x [rows, d_in]:
        returns (ok, f32 or None, bytes or None)."""
        import torch
        if x.ndim != 2 or x.shape[1] != self.d_in:
            raise ValueError(f"x: shape {tuple(x.shape)}, expected [rows, {self.d_in}]")
        rows = x.shape[0]
        _byte_dtype(input_dtype, "input_dtype")
        out_t = _byte_dtype(output_dtype, "output_dtype")
        y = torch.empty((rows, self.d_out), dtype=torch.float32, device=x.device) if want_f32 else None
        q = torch.empty((rows, self.d_out), dtype=out_t, device=x.device) if want_bytes else None
        ok = library().vxhip_qlinear_forward_f32(
            ctx._h, self._h, _dp(x, "x", torch.float32), _dp(y, "out", torch.float32, (rows, self.d_out)),
            _dp(q, "bytes", out_t, (rows, self.d_out)), rows, float(np.float32(input_scale)), int(input_zero_point),
            float(np.float32(output_scale)), int(output_zero_point), input_dtype, output_dtype,
            float(np.float32(output_scale)), int(output_zero_point))
        return ok, y, q

    def forward_rowscale(self, ctx: Context, x, row_scales, output_scale, output_zero_point=0,
                         output_dtype=DTYPE_I8, bias_f32=None, out=None, want_accumulators=False,
                         accumulators=None):
        import torch
        if x.ndim != 2 or x.shape[1] != self.d_in:
            raise ValueError(f"x: shape {tuple(x.shape)}, expected [rows, {self.d_in}]")
        rows = x.shape[0]
        out_t = _byte_dtype(output_dtype, "output_dtype")
        if out is None:
            out = torch.empty((rows, self.d_out), dtype=out_t, device=x.device)
        if want_accumulators and accumulators is None:
            accumulators = torch.empty((rows, self.d_out), dtype=torch.int32, device=x.device)
        ok = library().vxhip_qlinear_forward_rowscale(
            ctx._h, self._h, _dp(x, "x", torch.int8), _dp(row_scales, "row_scales", torch.float32, numel=rows),
            _dp(bias_f32, "bias_f32", torch.float32, numel=self.d_out), _dp(out, "out", out_t, (rows, self.d_out)),
            _dp(accumulators, "accumulators", torch.int32, (rows, self.d_out)), rows,
            float(np.float32(output_scale)), int(output_zero_point), output_dtype)
        return (ok, out, accumulators) if want_accumulators else (ok, out)


class Replay:
    """Launches recorded on a context (Context.begin_recording / end_recording), instantiated for replay."""

    def __init__(self, handle):
        self._h = handle

    def launch(self, ctx: Context):
        _check(library().vxhip_replay_launch(ctx._h, self._h), "replay_launch")

    def close(self):
        if self._h:
            library().vxhip_replay_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


ROW_OP_NONE, ROW_OP_RMSNORM, ROW_OP_SWIGLU = 0, 1, 2


class PackedLinear:
    """Compiled scope of one PackedLinear node (weight_bits=8, DYNAMIC_I8)."""

    def __init__(self, packed_words, scales, bias, k, n, group_size, weight_bits=8):
        pw = _np(packed_words, np.uint32)
        sc = _np(scales, np.float32)
        b = None if bias is None else _np(bias, np.float32)
        self.k, self.n, self.group_size = int(k), int(n), int(group_size)
        self._h = C.c_void_p()
        _check(library().vxhip_packed_linear_create(_hp(pw), _hp(sc), _hp(b), self.k, self.n,
                                                     self.group_size, weight_bits, C.byref(self._h)),
               "vxhip_packed_linear_create")

    def close(self):
        if self._h:
            library().vxhip_packed_linear_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def resident_bytes(self) -> int:
        return int(library().vxhip_packed_linear_resident_bytes(self._h))

    def forward_f32(self, ctx: Context, x, out=None, no_alloc=False):
        """no_alloc=True takes the entry point that stages in the library's fixed scratch array and
        allocates nothing (`out` must then be given)."""
        import torch
        if x.ndim != 2 or x.shape[1] != self.k:
            raise ValueError(f"x: shape {tuple(x.shape)}, expected [rows, {self.k}]")
        rows = x.shape[0]
        if out is None:
            if no_alloc:
                raise ValueError("out: the entry point that allocates nothing needs the output tensor from its caller")
            out = torch.empty((rows, self.n), dtype=torch.float32, device=x.device)
        entry = library().vxhip_packed_linear_forward_f32_noalloc if no_alloc else library().vxhip_packed_linear_forward_f32
        st = entry(ctx._h, self._h, _dp(x, "x", torch.float32), _dp(out, "out", torch.float32, (rows, self.n)), rows)
        return st, out

    def forward_f32_window(self, ctx: Context, x, out, first_unit, unit_count):
        """Writes units [first_unit, first_unit + unit_count) of the row-major `out` [rows, n] (0 units:
        all of it) and leaves the rest of it alone: the reference's first_unit / unit_count."""
        import torch
        if x.ndim != 2 or x.shape[1] != self.k:
            raise ValueError(f"x: shape {tuple(x.shape)}, expected [rows, {self.k}]")
        rows = x.shape[0]
        return library().vxhip_packed_linear_forward_f32_window(
            ctx._h, self._h, _dp(x, "x", torch.float32), _dp(out, "out", torch.float32, (rows, self.n)), rows,
            int(first_unit), int(unit_count))

    def fused_takes(self, ctx: Context, rows, row_op=ROW_OP_NONE, with_residual=False) -> bool:
        """Whether forward_fused would run a call of this description on ctx (nothing is launched)."""
        return bool(library().vxhip_packed_linear_fused_takes(ctx._h, self._h, int(rows), int(row_op), 1 if with_residual else 0))

    def forward_fused(self, ctx: Context, x, row_op=ROW_OP_NONE, gain=None, eps=0.0, add_to=None, out=None):
        """One or two f32 rows through [RMSNorm | SwiGLU] -> preparation -> linear [-> residual add] in one
        launch.  x is [rows, k], or [rows, 2k] = [gate | up] for ROW_OP_SWIGLU; add_to [rows, n] may be
        `out` itself.  Returns (handled, out): handled 0 means nothing ran and the caller takes the
        separate launches."""
        import torch
        width = 2 * self.k if row_op == ROW_OP_SWIGLU else self.k
        if row_op not in (ROW_OP_NONE, ROW_OP_RMSNORM, ROW_OP_SWIGLU):
            raise ValueError(f"row_op: {row_op}")
        if x.ndim != 2 or x.shape[1] != width:
            raise ValueError(f"x: shape {tuple(x.shape)}, expected [rows, {width}]")
        rows = x.shape[0]
        if row_op == ROW_OP_RMSNORM and gain is None:
            raise ValueError("gain: RMSNorm needs its gain vector")
        if out is None:
            out = torch.empty((rows, self.n), dtype=torch.float32, device=x.device)
        # every workgroup reads the whole input rows while others already store: the input may not share
        # memory with the output or the residual (add_to may be `out` itself)
        x0, x1 = x.data_ptr(), x.data_ptr() + x.numel() * 4
        for name, other in (("out", out), ("add_to", add_to)):
            if other is not None and x0 < other.data_ptr() + other.numel() * 4 and other.data_ptr() < x1:
                raise ValueError(f"x: overlaps {name}")
        handled = library().vxhip_packed_linear_forward_fused(
            ctx._h, self._h, _dp(x, "x", torch.float32), rows, row_op,
            _dp(gain if row_op == ROW_OP_RMSNORM else None, "gain", torch.float32, numel=self.k), float(eps),
            _dp(add_to, "add_to", torch.float32, (rows, self.n)), _dp(out, "out", torch.float32, (rows, self.n)))
        if handled < 0:
            raise RuntimeError(library().vxhip_last_error().decode())
        return handled, out

    def forward_a8(self, ctx: Context, a8, row_scales, out=None, want_accumulators=False,
                   accumulators=None):
        import torch
        if row_scales.ndim != 1:
            raise ValueError(f"row_scales: shape {tuple(row_scales.shape)}, expected [rows]")
        rows = row_scales.shape[0]  # (a8 is flat when the context exchanges operand-order activations)
        need = library().vxhip_context_prepared_bytes(ctx._h, rows, self.k)
        if a8.ndim == 2 and tuple(a8.shape) != (rows, self.k):
            raise ValueError(f"a8: shape {tuple(a8.shape)}, expected ({rows}, {self.k}) or the flat operand-order buffer")
        if out is None:
            out = torch.empty((rows, self.n), dtype=torch.float32, device=a8.device)
        if want_accumulators and accumulators is None:
            accumulators = torch.empty((rows, self.n), dtype=torch.int32, device=a8.device)
        st = library().vxhip_packed_linear_forward_a8(
            ctx._h, self._h, _dp(a8, "a8", torch.int8, numel=need), _dp(row_scales, "row_scales", torch.float32),
            _dp(out, "out", torch.float32, (rows, self.n)),
            _dp(accumulators, "accumulators", torch.int32, (rows, self.n)), rows)
        return (st, out, accumulators) if want_accumulators else (st, out)


def rmsnorm_prepare_i8(ctx: Context, x, gain, eps, want_normalized=False):
    """RMSNorm then activation preparation of x [rows, d]; returns (codes int8, row scales[, normalized f32])."""
    import torch
    rows, d = x.shape
    a8 = ctx.prepared_buffer(rows, d, x.device)
    scales = torch.empty((rows,), dtype=torch.float32, device=x.device)
    normalized = torch.empty((rows, d), dtype=torch.float32, device=x.device) if want_normalized else None
    _check(library().vxhip_rmsnorm_prepare_i8(ctx._h, _dp(x, "x", torch.float32), _dp(gain, "gain", torch.float32, numel=d),
                                              rows, d, float(eps), _dp(a8), _dp(scales), _dp(normalized)),
           "vxhip_rmsnorm_prepare_i8")
    return (a8, scales, normalized) if want_normalized else (a8, scales)


def add_rmsnorm_prepare_i8(ctx: Context, residual, delta, gain, eps):
    """residual += delta in place, then RMSNorm and preparation of the updated rows."""
    import torch
    rows, d = residual.shape
    a8 = ctx.prepared_buffer(rows, d, residual.device)
    scales = torch.empty((rows,), dtype=torch.float32, device=residual.device)
    _check(library().vxhip_add_rmsnorm_prepare_i8(ctx._h, _dp(residual, "residual", torch.float32),
                                                  _dp(delta, "delta", torch.float32, (rows, d)),
                                                  _dp(gain, "gain", torch.float32, numel=d), rows, d, float(eps),
                                                  _dp(a8), _dp(scales)), "vxhip_add_rmsnorm_prepare_i8")
    return a8, scales


def swiglu_prepare_i8(ctx: Context, gate_up, want_activated=False):
    """silu(gate) * up of gate_up [rows, 2*inter], then activation preparation."""
    import torch
    rows, two = gate_up.shape
    if two % 2:
        raise ValueError(f"gate_up: shape {tuple(gate_up.shape)}, the last extent must be even")
    inter = two // 2
    a8 = ctx.prepared_buffer(rows, inter, gate_up.device)
    scales = torch.empty((rows,), dtype=torch.float32, device=gate_up.device)
    act = torch.empty((rows, inter), dtype=torch.float32, device=gate_up.device) if want_activated else None
    _check(library().vxhip_swiglu_prepare_i8(ctx._h, _dp(gate_up, "gate_up", torch.float32), rows, inter, _dp(a8),
                                             _dp(scales), _dp(act)),
           "vxhip_swiglu_prepare_i8")
    return (a8, scales, act) if want_activated else (a8, scales)


def _check_caches(k_cache, v_cache, cos, sin, rows, kv_heads, head_dim):
    """Shapes the attention entry points index by: caches [rows, kv_heads, max_seq, head_dim] f32,
    rotary tables [max_seq, head_dim] f32.  Returns max_seq."""
    import torch
    if k_cache.ndim != 4 or tuple(k_cache.shape[:2]) != (rows, kv_heads) or k_cache.shape[3] != head_dim:
        raise ValueError(f"k_cache: shape {tuple(k_cache.shape)}, expected [{rows}, {kv_heads}, max_seq, {head_dim}]")
    max_seq = k_cache.shape[2]
    _dp(k_cache, "k_cache", torch.float32)
    _dp(v_cache, "v_cache", torch.float32, tuple(k_cache.shape))
    for name, table in (("cos", cos), ("sin", sin)):
        if table is not None:
            _dp(table, name, torch.float32, (max_seq, head_dim))
    return max_seq


def rope_append_kv(ctx: Context, qkv, cos, sin, positions, q_heads, kv_heads, head_dim, k_cache, v_cache):
    """qkv [rows, t, (q+2kv)*d]; caches [rows, kv_heads, max_seq, d] updated in place; returns rotated q."""
    import torch
    rows, t, _ = qkv.shape
    max_seq = _check_caches(k_cache, v_cache, cos, sin, rows, kv_heads, head_dim)
    q = torch.empty((rows, t, q_heads, head_dim), dtype=torch.float32, device=qkv.device)
    _check(library().vxhip_rope_append_kv(ctx._h, _dp(qkv, "qkv", torch.float32, (rows, t, (q_heads + 2 * kv_heads) * head_dim)),
                                          _dp(cos), _dp(sin), _dp(positions, "positions", torch.int64, numel=t), rows, t, q_heads,
                                          kv_heads, head_dim, max_seq, _dp(q), _dp(k_cache), _dp(v_cache)),
           "vxhip_rope_append_kv")
    return q


def gqa_attention(ctx: Context, q, k_cache, v_cache, positions):
    """q [rows, t, q_heads, d] over caches [rows, kv_heads, max_seq, d]; returns [rows, t, q_heads*d]."""
    import torch
    rows, t, q_heads, head_dim = q.shape
    if k_cache.ndim != 4:
        raise ValueError(f"k_cache: shape {tuple(k_cache.shape)}, expected [rows, kv_heads, max_seq, head_dim]")
    max_seq = _check_caches(k_cache, v_cache, None, None, rows, k_cache.shape[1], head_dim)
    out = torch.empty((rows, t, q_heads * head_dim), dtype=torch.float32, device=q.device)
    _check(library().vxhip_gqa_attention(ctx._h, _dp(q, "q", torch.float32), _dp(k_cache), _dp(v_cache),
                                         _dp(positions, "positions", torch.int64, numel=t), rows, t, q_heads,
                                         k_cache.shape[1], head_dim, max_seq, _dp(out)),
           "vxhip_gqa_attention")
    return out


def rope_gqa_attention_decode(ctx: Context, qkv, cos, sin, position, q_heads, kv_heads, head_dim, k_cache, v_cache):
    """One decode step: qkv [rows, (q+2kv)*d]; rotary, cache append at slot position[0] and attention
    in one launch; returns [rows, q_heads*d]."""
    import torch
    rows = qkv.shape[0]
    max_seq = _check_caches(k_cache, v_cache, cos, sin, rows, kv_heads, head_dim)
    out = torch.empty((rows, q_heads * head_dim), dtype=torch.float32, device=qkv.device)
    _check(library().vxhip_rope_gqa_attention_decode(ctx._h, _dp(qkv, "qkv", torch.float32, (rows, (q_heads + 2 * kv_heads) * head_dim)),
                                                     _dp(cos), _dp(sin), _dp(position, "position", torch.int64, min_numel=1),
                                                     rows, q_heads, kv_heads, head_dim, max_seq, _dp(k_cache), _dp(v_cache),
                                                     _dp(out)),
           "vxhip_rope_gqa_attention_decode")
    return out


def embedding_gather(ctx: Context, tokens_i32, table, out=None):
    """out[i] = table[tokens_i32[i]]; tokens int32 of any shape, table [vocab, d] f32."""
    import torch
    count = tokens_i32.numel()
    vocab, d = table.shape
    if out is None:
        out = torch.empty((count, d), dtype=torch.float32, device=table.device)
    _check(library().vxhip_embedding_gather_f32(ctx._h, _dp(tokens_i32, "tokens", torch.int32),
                                                _dp(table, "table", torch.float32), count, d, vocab,
                                                _dp(out, "out", torch.float32, numel=count * d)),
           "vxhip_embedding_gather_f32")
    return out


def argmax_rows(ctx: Context, x, out=None, advance=None):
    """First index of the row maximum of x [rows, n] as int32 [rows]; `advance` (int64 tensor of up
    to 64 counters) is incremented by one in the same launch."""
    import torch
    rows, n = x.shape
    if out is None:
        out = torch.empty((rows,), dtype=torch.int32, device=x.device)
    if advance is not None and advance.numel() > 64:
        raise ValueError("advance: at most 64 counters")
    _check(library().vxhip_argmax_rows_f32(ctx._h, _dp(x, "x", torch.float32), rows, n,
                                           _dp(out, "out", torch.int32, numel=rows), _dp(advance, "advance", torch.int64),
                                           0 if advance is None else advance.numel()),
           "vxhip_argmax_rows_f32")
    return out


def operand_order_codes(a8):
    """Row-major int8 codes [rows <= 32, k] (numpy) re-ordered the way a context with
    set_activation_layout(True) exchanges them: flat, 32 * ceil(k/16) * 16 bytes, code j of row r
    at ((j // 16) * 32 + r) * 16 + j % 16, zeros elsewhere."""
    a8 = np.ascontiguousarray(a8, dtype=np.int8)
    rows, k = a8.shape
    if rows > 32:
        raise ValueError("operand order holds at most 32 rows")
    chunks = (k + 15) // 16
    padded = np.zeros((rows, chunks * 16), np.int8)
    padded[:, :k] = a8
    out = np.zeros((chunks, 32, 16), np.int8)
    out[:, :rows] = padded.reshape(rows, chunks, 16).transpose(1, 0, 2)
    return out.reshape(-1)


def packed_prepare_i8(ctx: Context, x):
    import torch
    rows, k = x.shape
    a8 = ctx.prepared_buffer(rows, k, x.device)
    scales = torch.empty((rows,), dtype=torch.float32, device=x.device)
    _check(library().vxhip_packed_prepare_i8(ctx._h, _dp(x, "x", torch.float32), rows, k, _dp(a8), _dp(scales)),
           "vxhip_packed_prepare_i8")
    return a8, scales


# ---- host-pointer drop-ins (numpy in, numpy out) -------------------------------

def qlinear_i8u8(input, weight, weight_scales, weight_zero_points, bias, rows, d_in, d_out,
                 input_scale, input_zero_point, output_scale, output_zero_point, input_dtype,
                 weight_dtype, output_dtype):
    """VxQLinearI8U8Fn with the output returned: (handled, output[rows, d_out])."""
    x = _np(input)
    w = _np(weight)
    s = _np(weight_scales, np.float32)
    z = _np(weight_zero_points, np.int32)
    b = None if bias is None else _np(bias, np.int32)
    out = np.zeros((rows, d_out), dtype=np.int8 if output_dtype == DTYPE_I8 else np.uint8)
    ok = library().vxhip_qlinear_i8u8(_hp(x), _hp(w), _hp(s), _hp(z), _hp(b), _hp(out), rows, d_in,
                                      d_out, float(np.float32(input_scale)), int(input_zero_point),
                                      float(np.float32(output_scale)), int(output_zero_point),
                                      input_dtype, weight_dtype, output_dtype)
    return int(ok), out


def packed_linear_f32(x, packed_weight, scale, bias, key_dim, value_dim, rate, groups=8, normalize=8,
                      first_unit=0, unit_count=0, out=None):
    """vx_llm_forward_f32 for a PackedLinear node: (status, out[rows, value_dim]).  first_unit /
    unit_count: the reference's output window in elements of the row-major output (0 units = all);
    `out`, when given, is written in place and keeps every element outside the window."""
    xx = _np(x, np.float32)
    rows = xx.shape[0]
    pw = _np(packed_weight, np.uint32)
    sc = _np(scale, np.float32)
    b = None if bias is None else _np(bias, np.float32)
    if out is None:
        out = np.zeros((rows, value_dim), dtype=np.float32)
    elif out.dtype != np.float32 or out.shape != (rows, value_dim) or not out.flags.c_contiguous:
        raise ValueError("out: a C-contiguous float32 array [rows, value_dim]")
    st = library().vxhip_packed_linear_f32(_hp(xx), _hp(pw), _hp(sc), _hp(b), _hp(out), rows,
                                           key_dim, value_dim, rate, groups, normalize, int(first_unit), int(unit_count))
    return int(st), out


def quantize_typed_f32_i8u8(input, scale, zero_point, output_dtype):
    x = _np(input, np.float32)
    out = np.zeros(x.shape, dtype=np.int8 if output_dtype == DTYPE_I8 else np.uint8)
    ok = library().vxhip_quantize_typed_f32_i8u8(_hp(x), x.size, _hp(out), float(np.float32(scale)),
                                                 int(zero_point), output_dtype)
    return int(ok), out


def dequantize_typed_i8u8_f32(input, scale, zero_point, input_dtype):
    q = _np(input)
    out = np.zeros(q.shape, dtype=np.float32)
    ok = library().vxhip_dequantize_typed_i8u8_f32(_hp(q), q.size, float(np.float32(scale)),
                                                   int(zero_point), input_dtype, _hp(out))
    return int(ok), out


def requantize_linear_i8u8(input, input_scale, input_zero_point, output_scale, output_zero_point, input_dtype,
                           output_dtype):
    """RequantizeLinear on host arrays (the drop-in slot): (ok, bytes)."""
    q = _np(input)
    out = np.zeros(q.shape, dtype=np.int8 if output_dtype == DTYPE_I8 else np.uint8)
    ok = library().vxhip_requantize_linear_i8u8(_hp(q), q.size, _hp(out), out.size, float(np.float32(input_scale)),
                                                int(input_zero_point), float(np.float32(output_scale)),
                                                int(output_zero_point), input_dtype, output_dtype)
    return int(ok), out


def requantize_forward(ctx: Context, x, input_scale, input_zero_point, output_scale, output_zero_point, input_dtype,
                       output_dtype, out=None):
    """RequantizeLinear on a resident byte tensor: (ok, bytes)."""
    import torch
    in_t, out_t = _byte_dtype(input_dtype, "input_dtype"), _byte_dtype(output_dtype, "output_dtype")
    if out is None:
        out = torch.empty(x.shape, dtype=out_t, device=x.device)
    ok = library().vxhip_requantize_forward(ctx._h, _dp(x, "x", in_t), x.numel(), _dp(out, "out", out_t, tuple(x.shape)),
                                            float(np.float32(input_scale)), int(input_zero_point),
                                            float(np.float32(output_scale)), int(output_zero_point), input_dtype, output_dtype)
    return int(ok), out


class _Variant(C.Structure):
    _fields_ = [("id", C.c_char_p), ("backend", C.c_int32), ("operator_kind", C.c_int32),
                ("entrypoint_id", C.c_char_p), ("predicate_id", C.c_char_p),
                ("required_features", C.c_char_p), ("priority", C.c_int32)]


def kernel_variants():
    n = C.c_size_t(0)
    p = library().vxhip_kernel_variants(C.byref(n))
    arr = C.cast(p, C.POINTER(_Variant))
    return [dict(id=arr[i].id.decode(), backend=arr[i].backend, operator_kind=arr[i].operator_kind,
                 entrypoint_id=arr[i].entrypoint_id.decode(), predicate_id=arr[i].predicate_id.decode(),
                 required_features=arr[i].required_features.decode(), priority=arr[i].priority)
            for i in range(n.value)]


def force_variant(prefix: str | None):
    library().vxhip_force_variant((prefix or "").encode())
