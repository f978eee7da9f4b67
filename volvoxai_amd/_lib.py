"""Locates, builds and loads libvxhip_w8a8.so.  There is no fallback path: a
missing library raises, it never degrades to a CPU implementation."""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

ROOT = Path(__file__).resolve().parent
HEADER = ROOT.parent / "include" / "vxhip_w8a8.h"


class LibraryMissing(RuntimeError):
    pass


def library_path() -> Path:
    return ROOT / "lib" / "libvxhip_w8a8.so"


def build_library(clean: bool = False) -> Path:
    """Compile the HIP sources for gfx950 (cross-compiles without a GPU)."""
    if clean:
        subprocess.check_call(["make", "-C", str(ROOT / "csrc"), "clean"])
    subprocess.check_call(["make", "-C", str(ROOT / "csrc"), "-j8"])
    return library_path()


_lib = None


def library() -> C.CDLL:
    global _lib
    if _lib is None:
        path = library_path()
        if not path.exists():
            raise LibraryMissing(
                f"{path} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C volvoxai_amd/csrc`. This package has no non-HIP path.")
        # PyTorch bundles its own libamdhip64 under the same soname as /opt/rocm's.  Whichever
        # is mapped first serves the whole process, and torch does not find the GPU when the
        # system copy got there first -- so where torch exists, let it load its runtime first.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        _lib = C.CDLL(str(path))
        _declare(_lib)
    return _lib


def _declare(L: C.CDLL) -> None:
    vp, u32, i32, f32, sz, u64 = C.c_void_p, C.c_uint32, C.c_int32, C.c_float, C.c_size_t, C.c_uint64
    pp = C.POINTER(C.c_void_p)
    sig = {
        "vxhip_abi_version": (u32, []),
        "vxhip_device_count": (i32, []),
        "vxhip_device_name": (i32, [i32, C.c_char_p, sz]),
        "vxhip_last_error": (C.c_char_p, []),
        "vxhip_context_create": (i32, [i32, vp, u32, pp]),
        "vxhip_context_destroy": (None, [vp]),
        "vxhip_context_synchronize": (i32, [vp]),
        "vxhip_context_last_variant": (C.c_char_p, [vp]),
        "vxhip_context_fault_flags": (i32, [vp, C.POINTER(u32)]),
        "vxhip_context_clear_fault_flags": (i32, [vp]),
        "vxhip_context_reserve_scratch": (i32, [vp, sz]),
        "vxhip_rmsnorm_prepare_i8": (i32, [vp, vp, vp, u32, u32, C.c_double, vp, vp, vp]),
        "vxhip_add_rmsnorm_prepare_i8": (i32, [vp, vp, vp, vp, u32, u32, C.c_double, vp, vp]),
        "vxhip_swiglu_prepare_i8": (i32, [vp, vp, u32, u32, vp, vp, vp]),
        "vxhip_rope_append_kv": (i32, [vp, vp, vp, vp, vp, u32, u32, u32, u32, u32, u32, vp, vp, vp]),
        "vxhip_gqa_attention": (i32, [vp, vp, vp, vp, vp, u32, u32, u32, u32, u32, u32, vp]),
        "vxhip_rope_gqa_attention_decode": (i32, [vp, vp, vp, vp, vp, u32, u32, u32, u32, u32, vp, vp, vp]),
        "vxhip_embedding_gather_f32": (i32, [vp, vp, vp, u32, u32, u32, vp]),
        "vxhip_argmax_rows_f32": (i32, [vp, vp, u32, u32, vp, vp, u32]),
        "vxhip_probe_mfma_rate": (i32, [vp, u32, u32, C.POINTER(C.c_double), C.POINTER(C.c_double),
                                        C.POINTER(C.c_double)]),
        "vxhip_probe_stream_read": (i32, [vp, C.POINTER(C.c_void_p), u32, sz, u32, C.POINTER(C.c_double),
                                          C.POINTER(C.c_double)]),
        "vxhip_probe_mfma_valu_overlap": (i32, [vp, u32, u32, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
        "vxhip_context_set_activation_layout": (i32, [vp, u32]),
        "vxhip_context_prepared_bytes": (sz, [vp, u32, u32]),
        "vxhip_device_malloc": (i32, [sz, pp]),
        "vxhip_device_free": (None, [vp]),
        "vxhip_memcpy_to_device": (i32, [vp, vp, vp, sz]),
        "vxhip_memcpy_to_host": (i32, [vp, vp, vp, sz]),
        "vxhip_qlinear_create": (i32, [vp, vp, vp, vp, u32, u32, u32, pp]),
        "vxhip_qlinear_destroy": (None, [vp]),
        "vxhip_qlinear_resident_bytes": (u64, [vp]),
        "vxhip_qlinear_admits": (C.c_int, [vp, f32, i32, f32, i32, u32, u32]),
        "vxhip_qlinear_forward": (C.c_int, [vp, vp, vp, vp, vp, u32, f32, i32, f32, i32, u32, u32]),
        "vxhip_qlinear_forward_dequantized": (C.c_int, [vp, vp, vp, vp, vp, u32, f32, i32, f32, i32, u32, u32, f32, i32]),
        "vxhip_qlinear_forward_f32": (C.c_int, [vp, vp, vp, vp, vp, u32, f32, i32, f32, i32, u32, u32, f32, i32]),
        "vxhip_qlinear_forward_rowscale": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, u32, f32, i32, u32]),
        "vxhip_qlinear_i8u8": (C.c_int, [vp, vp, vp, vp, vp, vp, u32, u32, u32, f32, i32, f32, i32,
                                         u32, u32, u32]),
        "vxhip_packed_linear_create": (i32, [vp, vp, vp, u32, u32, u32, u32, pp]),
        "vxhip_packed_linear_destroy": (None, [vp]),
        "vxhip_packed_linear_resident_bytes": (u64, [vp]),
        "vxhip_packed_prepare_i8": (i32, [vp, vp, u32, u32, vp, vp]),
        "vxhip_packed_linear_forward_f32": (C.c_int, [vp, vp, vp, vp, u32]),
        "vxhip_packed_linear_forward_f32_noalloc": (C.c_int, [vp, vp, vp, vp, u32]),
        "vxhip_packed_linear_forward_fused": (C.c_int, [vp, vp, vp, u32, u32, vp, C.c_double, vp, vp]),
        "vxhip_packed_linear_fused_takes": (C.c_int, [vp, vp, u32, u32, C.c_int]),
        "vxhip_packed_linear_forward_a8": (C.c_int, [vp, vp, vp, vp, vp, vp, u32]),
        "vxhip_packed_linear_f32": (C.c_int, [vp, vp, vp, vp, vp, u64, i32, i32, i32, i32, i32, u64, u64]),
        "vxhip_packed_linear_forward_f32_window": (C.c_int, [vp, vp, vp, vp, u32, u64, u64]),
        "vxhip_quantize_typed_f32_i8u8": (C.c_int, [vp, u32, vp, f32, i32, u32]),
        "vxhip_dequantize_typed_i8u8_f32": (C.c_int, [vp, u32, f32, i32, u32, vp]),
        "vxhip_quantize_forward": (C.c_int, [vp, vp, u32, vp, f32, i32, u32]),
        "vxhip_dequantize_forward": (C.c_int, [vp, vp, u32, f32, i32, u32, vp]),
        "vxhip_context_begin_recording": (C.c_int, [vp]),
        "vxhip_context_end_recording": (C.c_int, [vp, C.POINTER(vp)]),
        "vxhip_replay_launch": (C.c_int, [vp, vp]),
        "vxhip_replay_destroy": (None, [vp]),
        "vxhip_resident_weights_clear": (None, []),
        "vxhip_resident_weights_bytes": (C.c_uint64, []),
        "vxhip_requantize_linear_i8u8": (C.c_int, [vp, u32, vp, u32, f32, i32, f32, i32, u32, u32]),
        "vxhip_requantize_forward": (C.c_int, [vp, vp, u32, vp, f32, i32, f32, i32, u32, u32]),
        "vxhip_kernel_variants": (vp, [C.POINTER(sz)]),
        "vxhip_force_variant": (None, [C.c_char_p]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args


def declared_symbols() -> list[str]:
    """Every entry point the public header declares (parsed from the header)."""
    import re
    text = HEADER.read_text()
    return sorted(set(re.findall(r"\b(vxhip_[a-z0-9_]+)\s*\(", text)))
