"""The ctypes wrappers hand bare device addresses to the library, so they must refuse a tensor of
the wrong type or extent themselves, with a Python error, before anything is launched.  Real CPU
tensors stand in for device tensors here (a subclass that claims to be on the device); every
refusal happens before the library is called, which a null handle would make fatal otherwise."""
import ctypes as C

import pytest

torch = pytest.importorskip("torch")


class FakeDevice(torch.Tensor):
    @property
    def is_cuda(self):
        return True


def fake(*shape, dtype=torch.float32):
    return torch.zeros(shape, dtype=dtype).as_subclass(FakeDevice)


def test_device_pointer_checks():
    from volvoxai_amd.w8a8 import _dp
    assert _dp(None) is None
    assert _dp(fake(3, 4), "x", torch.float32, (3, 4)).value
    with pytest.raises(ValueError, match="contiguous device"):
        _dp(torch.zeros(4), "x")                       # a host tensor
    with pytest.raises(ValueError, match="contiguous device"):
        _dp(fake(4, 4).t(), "x")                       # not contiguous
    with pytest.raises(ValueError, match="dtype"):
        _dp(fake(4, dtype=torch.float64), "x", torch.float32)
    with pytest.raises(ValueError, match="shape"):
        _dp(fake(4, 5), "x", torch.float32, (4, 6))
    with pytest.raises(ValueError, match="elements"):
        _dp(fake(7), "x", torch.float32, numel=8)
    with pytest.raises(ValueError, match="at least"):
        _dp(fake(0, dtype=torch.int64), "x", torch.int64, min_numel=1)


def _qlinear(d_in, d_out):
    from volvoxai_amd.w8a8 import QLinear
    lin = QLinear.__new__(QLinear)
    lin.d_in, lin.d_out, lin._h = d_in, d_out, C.c_void_p()
    return lin


def _packed(k, n):
    from volvoxai_amd.w8a8 import PackedLinear
    pl = PackedLinear.__new__(PackedLinear)
    pl.k, pl.n, pl.group_size, pl._h = k, n, 128, C.c_void_p()
    return pl


class NullContext:
    _h = C.c_void_p()


def test_qlinear_wrappers_refuse_wrong_tensors():
    lin, ctx = _qlinear(64, 32), NullContext()
    x8 = fake(5, 64, dtype=torch.int8)
    with pytest.raises(ValueError, match=r"expected \[rows, 64\]"):
        lin.forward(ctx, fake(5, 48, dtype=torch.int8), 0.1, 0, 0.1, 0)
    with pytest.raises(ValueError, match="dtype"):
        lin.forward(ctx, fake(5, 64, dtype=torch.uint8), 0.1, 0, 0.1, 0)           # I8 call, U8 bytes
    with pytest.raises(ValueError, match="out: shape"):
        lin.forward(ctx, x8, 0.1, 0, 0.1, 0, out=fake(5, 16, dtype=torch.int8))
    y8 = fake(5, 32, dtype=torch.int8)  # (outputs are passed in: the wrappers would allocate them on x.device)
    with pytest.raises(ValueError, match="accumulators: dtype"):
        lin.forward(ctx, x8, 0.1, 0, 0.1, 0, out=y8, accumulators=fake(5, 32, dtype=torch.int64))
    with pytest.raises(ValueError, match="neither I8"):
        lin.forward(ctx, x8, 0.1, 0, 0.1, 0, output_dtype=1)
    with pytest.raises(ValueError, match="row_scales"):
        lin.forward_rowscale(ctx, x8, fake(4), 0.05, out=y8)                          # one scale short
    with pytest.raises(ValueError, match="bias_f32"):
        lin.forward_rowscale(ctx, x8, fake(5), 0.05, bias_f32=fake(31), out=y8)
    with pytest.raises(ValueError, match="x: dtype"):
        lin.forward_rowscale(ctx, fake(5, 64, dtype=torch.uint8), fake(5), 0.05, out=y8)
    # the forms that carry their boundary operators
    with pytest.raises(ValueError, match=r"expected \[rows, 64\]"):
        lin.forward_dequantized(ctx, fake(5, 48, dtype=torch.int8), 0.1, 0, 0.1, 0)
    with pytest.raises(ValueError, match="x: dtype"):
        lin.forward_dequantized(ctx, fake(5, 64), 0.1, 0, 0.1, 0, out=fake(5, 32))    # f32 rows where bytes are due
    with pytest.raises(ValueError, match="out: shape"):
        lin.forward_dequantized(ctx, x8, 0.1, 0, 0.1, 0, out=fake(5, 16))
    with pytest.raises(ValueError, match="out: dtype"):
        lin.forward_dequantized(ctx, x8, 0.1, 0, 0.1, 0, out=y8)                      # the output is f32
    with pytest.raises(ValueError, match=r"expected \[rows, 64\]"):
        lin.forward_f32(ctx, fake(5, 63), 0.1, 0, 0.1, 0)
    with pytest.raises(ValueError, match="neither I8"):
        lin.forward_f32(ctx, fake(5, 64), 0.1, 0, 0.1, 0, input_dtype=3)


def test_packed_linear_wrappers_refuse_wrong_tensors():
    pl, ctx = _packed(128, 40), NullContext()
    with pytest.raises(ValueError, match=r"expected \[rows, 128\]"):
        pl.forward_f32(ctx, fake(3, 100))
    with pytest.raises(ValueError, match="x: dtype"):
        pl.forward_f32(ctx, fake(3, 128, dtype=torch.float64), out=fake(3, 40))
    with pytest.raises(ValueError, match="out: shape"):
        pl.forward_f32(ctx, fake(3, 128), out=fake(3, 39))
    with pytest.raises(ValueError, match="a8: shape"):
        pl.forward_a8(ctx, fake(3, 127, dtype=torch.int8), fake(3))
    with pytest.raises(ValueError, match="a8"):
        pl.forward_a8(ctx, fake(3 * 128 - 1, dtype=torch.int8), fake(3), out=fake(3, 40))  # flat and too short
    with pytest.raises(ValueError, match="row_scales"):
        pl.forward_a8(ctx, fake(3, 128, dtype=torch.int8), fake(3, 1))
    # the fused single-row forms
    from volvoxai_amd.w8a8 import ROW_OP_NONE, ROW_OP_RMSNORM, ROW_OP_SWIGLU
    with pytest.raises(ValueError, match=r"expected \[rows, 256\]"):
        pl.forward_fused(ctx, fake(1, 128), ROW_OP_SWIGLU)                       # [gate | up] is 2k wide
    with pytest.raises(ValueError, match="gain"):
        pl.forward_fused(ctx, fake(1, 128), ROW_OP_RMSNORM, out=fake(1, 40))     # RMSNorm without its gain
    with pytest.raises(ValueError, match="gain"):
        pl.forward_fused(ctx, fake(1, 128), ROW_OP_RMSNORM, gain=fake(127), out=fake(1, 40))
    with pytest.raises(ValueError, match="add_to: shape"):
        pl.forward_fused(ctx, fake(2, 128), ROW_OP_NONE, add_to=fake(1, 40), out=fake(2, 40))
    with pytest.raises(ValueError, match="row_op"):
        pl.forward_fused(ctx, fake(1, 128), 7, out=fake(1, 40))
    # an input that shares memory with the output or the residual would be read half updated
    shared = fake(1, 128)
    with pytest.raises(ValueError, match="overlaps out"):
        pl.forward_fused(ctx, shared, ROW_OP_NONE, out=shared[:, :40].contiguous().set_(shared.untyped_storage(), 0, (1, 40)))
    with pytest.raises(ValueError, match="overlaps add_to"):
        pl.forward_fused(ctx, shared, ROW_OP_NONE, add_to=torch.Tensor().set_(shared.untyped_storage(), 8, (1, 40)).as_subclass(FakeDevice),
                         out=fake(1, 40))


def test_attention_wrappers_refuse_wrong_shapes():
    from volvoxai_amd import w8a8
    ctx = NullContext()
    rows, qh, kvh, d, max_seq = 2, 4, 2, 64, 16
    k, v = fake(rows, kvh, max_seq, d), fake(rows, kvh, max_seq, d)
    cos, sin = fake(max_seq, d), fake(max_seq, d)
    qkv = fake(rows, (qh + 2 * kvh) * d)
    pos = fake(1, dtype=torch.int64)
    with pytest.raises(ValueError, match="cos"):
        w8a8.rope_gqa_attention_decode(ctx, qkv, fake(max_seq - 1, d), sin, pos, qh, kvh, d, k, v)
    with pytest.raises(ValueError, match="v_cache"):
        w8a8.rope_gqa_attention_decode(ctx, qkv, cos, sin, pos, qh, kvh, d, k, fake(rows, kvh, max_seq - 1, d))
    with pytest.raises(ValueError, match="k_cache"):
        w8a8.rope_gqa_attention_decode(ctx, qkv, cos, sin, pos, qh, kvh, d, fake(rows, kvh + 1, max_seq, d), v)
    with pytest.raises(ValueError, match="qkv"):
        w8a8.rope_gqa_attention_decode(ctx, fake(rows, qh * d), cos, sin, pos, qh, kvh, d, k, v)
    with pytest.raises(ValueError, match="position"):
        w8a8.rope_gqa_attention_decode(ctx, qkv, cos, sin, fake(1, dtype=torch.int32), qh, kvh, d, k, v)
    with pytest.raises(ValueError, match="positions"):
        w8a8.rope_append_kv(ctx, fake(rows, 3, (qh + 2 * kvh) * d), cos, sin, fake(2, dtype=torch.int64), qh, kvh, d, k, v)
    with pytest.raises(ValueError, match="positions"):
        w8a8.gqa_attention(ctx, fake(rows, 3, qh, d), k, v, fake(4, dtype=torch.int64))
    with pytest.raises(ValueError, match="tokens"):
        w8a8.embedding_gather(ctx, fake(3, dtype=torch.int64), fake(10, 8))
    with pytest.raises(ValueError, match="gain"):
        class Ctx(NullContext):
            def prepared_buffer(self, rows, k, device):
                return fake(rows, k, dtype=torch.int8)
        w8a8.rmsnorm_prepare_i8(Ctx(), fake(2, 8), fake(7), 1e-6)
