"""ctypes binding of ``liblucid_hip.so`` - the only crossing point between the
Python host code and HIP.

Plays the role of Lucid's pybind11 boundary (``lucid/_C/bindings/bind.cpp``):
one thin layer, no tensor logic.  Status codes are turned into exception
classes named after Lucid's own (``lucid/_C/core/Error.h:63-495``,
``lucid/_C/bindings/bind_errors.cpp``).

There is no CPU fallback: if the library is missing or no gfx950 device is
visible, loading / initialising raises.
"""

from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "liblucid_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "lucid_hip.h")


# ---------------------------------------------------------------- errors
class LucidError(RuntimeError):
    """Base of every error raised by the backend."""


class OutOfMemory(LucidError):
    pass


class ShapeMismatch(LucidError):
    pass


class DtypeMismatch(LucidError):
    pass


class DeviceMismatch(LucidError):
    pass


class GpuNotAvailable(LucidError):
    pass


_STATUS_TO_EXC = {
    1: ValueError,
    2: ShapeMismatch,
    3: DtypeMismatch,
    4: DeviceMismatch,
    5: OutOfMemory,
    6: GpuNotAvailable,
    7: NotImplementedError,
    8: LucidError,
}

# lucid/_C/core/Dtype.h enum order
BOOL, I8, I16, I32, I64, F16, F32, F64, C64, BF16, C128 = range(11)

OUT_ACC_I32, OUT_F32, OUT_F16, OUT_REQUANT_I8, OUT_FAKEQUANT_F32 = range(5)

_vp, _sz, _i, _f, _u64 = C.c_void_p, C.c_size_t, C.c_int, C.c_float, C.c_uint64

# name -> argtypes; every function returns int status unless listed in _RESTYPE
_SIGNATURES = {
    "lq_version": [],
    "lq_last_tile_config": [],
    "lq_device_memory_info": [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
    "lq_tune_export": [C.c_char_p, _sz, C.POINTER(C.c_size_t)],
    "lq_tune_import": [C.c_char_p, C.POINTER(C.c_int)],
    "lq_last_error": [],
    "lq_device_count": [C.POINTER(_i)],
    "lq_init": [_i],
    "lq_device_name": [C.c_char_p, _sz],
    "lq_alloc": [C.POINTER(_vp), _sz],
    "lq_free": [_vp],
    "lq_empty_cache": [],
    "lq_memory_stats": [C.POINTER(_sz), C.POINTER(_sz)],
    "lq_graph_begin": [_vp, C.POINTER(_i)],
    "lq_graph_end": [_vp, _i],
    "lq_graph_launch": [_i, _vp],
    "lq_graph_destroy": [_i],
    "lq_h2d": [_vp, _vp, _sz, _vp],
    "lq_d2h": [_vp, _vp, _sz, _vp],
    "lq_d2d": [_vp, _vp, _sz, _vp],
    "lq_d2d_rows": [_vp, _sz, _vp, _sz, _sz, _sz, _vp],
    "lq_fill_bytes": [_vp, _i, _sz, _vp],
    "lq_sync": [_vp],
    "lq_stream_create": [C.POINTER(_vp)],
    "lq_stream_create_nonblocking": [C.POINTER(_vp)],
    "lq_stream_destroy": [_vp],
    "lq_event_create": [C.POINTER(_vp)],
    "lq_event_destroy": [_vp],
    "lq_event_record": [_vp, _vp],
    "lq_event_sync": [_vp],
    "lq_stream_wait_event": [_vp, _vp],
    "lq_event_elapsed_ms": [_vp, _vp, C.POINTER(_f)],
    "lq_op_count": [],
    "lq_op_info": [_i, C.POINTER(C.c_char_p), C.POINTER(_i), C.POINTER(_i)],
    "lq_fill_normal": [_vp, _sz, _u64, _f, _f, _vp],
    "lq_fill_uniform_i8": [_vp, _sz, _u64, _i, _i, _vp],
    "lq_index_minmax": [_vp, _i, _sz, _vp, _vp],
    "lq_embedding_i8": [_vp, _vp, _vp, _i, _i, _vp, _i, _sz, _i, _vp, _vp],
    "lq_embedding_bag_i8": [_vp, _vp, _vp, _i, _i, _vp, _i, _sz, _vp, _i, _i, _i, _i, _i, _vp, _vp],
    "lq_act_f32": [_i, _f, _vp, _vp, _sz, _i, _vp, _vp, _i, _i, _vp],
    "lq_act_requant_i8": [_i, _f, _vp, _i, _vp, _vp, _sz, _vp, _vp, _i, _i, _i, _vp, _vp],
    "lq_dilate_nhwc_i8": [_vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp],
    "lq_lstm_cell_f32": [_vp, _sz, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _sz, _vp],
    "lq_layernorm_stats_f32": [_vp, _vp, _vp, C.c_long, _i, C.c_float, _vp, _vp, _vp],
    "lq_layernorm_quantize_i8": [_vp, _vp, _vp, _vp, C.c_long, _i, _vp, _vp, _i, _i, _i, _vp, _vp],
    "lq_conv2d_f32": [_vp, _vp, _vp, _vp] + [_i] * 14 + [_vp],
    "lq_quantize_tensor_dynamic_i8": [_vp, _sz, _i, _i, _i, _i, C.c_float, _i, _vp, _vp, _vp, _vp, _vp, _vp],
    "lq_quantize_rows_dynamic_i8": [_vp, _sz, _sz, _i, _i, _i, _i, C.c_float, _i, _vp, _vp, _vp, _vp, _vp, _vp],
    "lq_dynamic_linear_small_f32": [_vp, _i, _i, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, C.c_float, _i, _vp, _vp],
    "lq_dynamic_mlp2_small_f32": [_vp, _i, _i, _vp, _i, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i,
                                  C.c_float, _i, _vp, _vp],
    "lq_selftest_requant_route": [C.c_float, C.c_float, _i, _i, _i, C.c_ulonglong, C.c_ulonglong, _vp, _vp, _vp],
    "lq_probe_mfma_i8": [_vp, _vp, _sz, _i, _vp, C.POINTER(C.c_double), _vp],
    "lq_probe_mfma_i8_k64": [_vp, _vp, _sz, _i, _vp, C.POINTER(C.c_double), _vp],
    "lq_copy_kernel": [_vp, _vp, _sz, _vp],
    "lq_minmax": [_vp, _sz, _sz, _sz, _vp, _vp, _vp],
    "lq_minmax_noalloc": [_vp, _sz, _sz, _sz, _vp, _vp, _vp],
    "lq_calc_qparams": [_vp, _vp, _sz, _i, _i, _i, _i, _f, _vp, _vp, _vp],
    "lq_quantize": [_vp, _vp, _i, _i, _sz, _sz, _sz, _vp, _vp, _i, _i, _i, _vp],
    "lq_dequantize": [_vp, _i, _i, _vp, _sz, _sz, _sz, _vp, _vp, _i, _vp],
    "lq_fake_quantize": [_vp, _vp, _sz, _sz, _sz, _vp, _vp, _i, _i, _i, _vp],
}


class JoinArgs(C.Structure):
    """``lq_join_args`` of ``include/lucid_hip.h``."""

    _fields_ = [
        ("q", _vp), ("ld", C.c_long), ("offset", _i), ("scale", _vp), ("zp", _vp), ("relu", _i),
        ("out_scale", _vp), ("out_zp", _vp), ("out_qmin", _i), ("out_qmax", _i), ("out_offset", _i),
    ]


class QLinearArgs(C.Structure):
    """``lq_qlinear_args`` of ``include/lucid_hip.h``."""

    _fields_ = [
        ("a", _vp), ("w", _vp), ("M", _i), ("N", _i), ("K", _i),
        ("wsum", _vp), ("a_zp", _i), ("a_zp_dev", _vp),
        ("a_scale", _vp), ("a_scale_per_row", _i), ("w_scale", _vp),
        ("bias", _vp), ("bias_dtype", _i), ("relu", _i), ("out_mode", _i),
        ("out_scale", _vp), ("out_zp", _vp),
        ("out_qmin", _i), ("out_qmax", _i), ("out_offset", _i),
        ("out", _vp), ("ldo", C.c_long), ("force_path", _i), ("tile_config", _i),
        ("residual", _vp), ("ldr", C.c_long), ("join", JoinArgs), ("gelu", _i), ("range", _vp),
        ("w_zp", _vp),
    ]


_SIGNATURES["lq_relu_f32"] = [_vp, _vp, _sz, _vp]
_SIGNATURES["lq_minmax_fold"] = [_vp, _vp, _vp, _vp, _sz, _i, _vp, _vp, _vp]
_SIGNATURES["lq_add_requant_i8"] = [_vp, _i, _vp, _vp, _vp, _i, _vp, _vp, _sz, _i, _vp, _vp, _i, _i,
                                    _i, _vp, _vp]
_SIGNATURES["lq_global_avgpool_nhwc_i8"] = [_vp, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp]
_SIGNATURES["lq_qlinear_w8a32"] = [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _i, _i, _vp,
                                   _vp]
_l = C.c_long
_SIGNATURES["lq_layernorm_f32"] = [_vp, _vp, _vp, _vp, _l, _i, _f, _vp, _vp]
_SIGNATURES["lq_gelu_f32"] = [_vp, _vp, _sz, _vp, _vp]
_SIGNATURES["lq_add_f32"] = [_vp, _vp, _vp, _sz, _vp]
_SIGNATURES["lq_attention_f32"] = [_vp, _vp, _i, _i, _i, _i, _f, _vp, _vp]
_SIGNATURES["lq_gather_rows_f32"] = [_vp, _sz, _vp, _sz, _sz, _vp]
_SIGNATURES["lq_range_buffer_bytes"] = []
_SIGNATURES["lq_calc_qparams_from_range"] = [_vp, _i, _i, _i, _i, _f, _vp, _vp, _vp, _vp, _vp]
_SIGNATURES["lq_patchify_f32"] = [_vp, _vp, _i, _i, _i, _i, _i, _vp]
_SIGNATURES["lq_sgemm_nt_f32"] = [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]
_SIGNATURES["lq_assemble_tokens_f32"] = [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]
_SIGNATURES["lq_patch_embed_f32"] = [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]
_SIGNATURES["lq_pad_nhwc_i8"] = [_vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp]
_SIGNATURES["lq_pad_planes_f32"] = [_vp, _vp, _sz, _i, _i, _i, _i, _i, _i, _i, _vp]
_SIGNATURES["lq_binary_requant_i8"] = [_i, _vp, _i, _vp, _vp, _vp, _i, _vp, _vp, _f, _sz, _i, _vp, _vp, _i, _i,
                                       _i, _vp, _vp]
_SIGNATURES["lq_requant_rows_i8"] = [_vp, _i, _vp, _vp, _sz, _sz, _vp, _sz, _vp, _vp, _i, _i, _i, _vp]
_SIGNATURES["lq_minmax_ema"] = [_vp, _vp, _vp, _vp, _sz, _i, _i, _f, _vp, _vp, _vp]
_SIGNATURES["lq_histc_f32"] = [_vp, _sz, C.c_double, C.c_double, _i, _vp, _vp]
_SIGNATURES["lq_wq_quantize"] = [_vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp]
_SIGNATURES["lq_wq_dequantize"] = [_vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp]
_SIGNATURES["lq_wq_matmul"] = [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp]
_SIGNATURES["lq_bias_act_f32"] = [_vp, _vp, _sz, _i, _i, _vp]
_SIGNATURES["lq_rowsum_i8"] = [_vp, _vp, _i, _i, _vp]
for _name in ("sub", "mul", "div", "maximum", "minimum"):
    _SIGNATURES[f"lq_{_name}_f32"] = [_vp, _vp, _vp, _sz, _vp]
_SIGNATURES["lq_round_f32"] = [_vp, _vp, _sz, _vp]
_SIGNATURES["lq_clip_f32"] = [_vp, _vp, _sz, C.c_double, C.c_double, _vp]
_SIGNATURES["lq_astype"] = [_vp, _i, _vp, _i, _sz, _vp]
_SIGNATURES["lq_broadcast_f32"] = [_vp, _vp, _sz, _sz, _sz, _vp]
_SIGNATURES["lq_reduce_minmax"] = [_vp, C.POINTER(C.c_int64), _i, C.POINTER(C.c_int), _i, _vp, _vp, _vp]
_SIGNATURES["lq_batchnorm_eval_f32"] = [_vp, _vp, _sz, _i, _sz, _vp, _vp, _vp, _vp, C.c_double, _vp]
_SIGNATURES["lq_qlinear_i8"] = [C.POINTER(QLinearArgs), _vp]
_SIGNATURES["lq_qlinear_i8_n"] = [C.POINTER(QLinearArgs), _i, _vp]



class QConv2dArgs(C.Structure):
    """``lq_qconv2d_args`` of ``include/lucid_hip.h``."""

    _fields_ = [
        ("x", _vp), ("w", _vp),
        ("B", _i), ("H", _i), ("W", _i), ("Cin", _i), ("Cout", _i), ("KH", _i), ("KW", _i),
        ("stride_h", _i), ("stride_w", _i), ("pad_h_lo", _i), ("pad_h_hi", _i), ("pad_w_lo", _i),
        ("pad_w_hi", _i), ("dil_h", _i), ("dil_w", _i), ("groups", _i),
        ("wsum", _vp), ("a_zp", _i), ("a_scale", _vp), ("w_scale", _vp),
        ("bias", _vp), ("bias_dtype", _i), ("relu", _i), ("out_mode", _i),
        ("out_scale", _vp), ("out_zp", _vp),
        ("out_qmin", _i), ("out_qmax", _i), ("out_offset", _i),
        ("out", _vp), ("force_path", _i), ("tile_config", _i), ("join", JoinArgs),
        ("w_zp", _vp),
    ]


_SIGNATURES["lq_qconv2d_i8"] = [C.POINTER(QConv2dArgs), _vp]


class QConv3dArgs(C.Structure):
    """``lq_qconv3d_args`` of ``include/lucid_hip.h``."""

    _fields_ = [
        ("x", _vp), ("w", _vp),
        ("B", _i), ("D", _i), ("H", _i), ("W", _i), ("Cin", _i), ("Cout", _i), ("KD", _i), ("KH", _i), ("KW", _i),
        ("stride", _i * 3), ("pad_lo", _i * 3), ("pad_hi", _i * 3), ("dilation", _i * 3), ("groups", _i),
        ("wsum", _vp), ("a_zp", _i), ("a_scale", _vp), ("w_scale", _vp),
        ("bias", _vp), ("bias_dtype", _i), ("relu", _i), ("out_mode", _i),
        ("out_scale", _vp), ("out_zp", _vp),
        ("out_qmin", _i), ("out_qmax", _i), ("out_offset", _i),
        ("out", _vp), ("tile_config", _i), ("w_zp", _vp),
    ]


_SIGNATURES["lq_qconv3d_i8"] = [C.POINTER(QConv3dArgs), _vp]
_SIGNATURES["lq_quantize_nchw_to_nhwc"] = [_vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _i, _i, _vp]
_SIGNATURES["lq_qconv2d_packed4_geometry"] = [C.POINTER(QConv2dArgs), C.POINTER(_i), C.POINTER(_i), C.POINTER(_i)]
_SIGNATURES["lq_quantize_nchw_to_packed4"] = [_vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _i, _i, _i, _vp]
_SIGNATURES["lq_pack4_filter_i8"] = [_vp, _vp, _i, _i, _i, _i, _vp]
_SIGNATURES["lq_dequantize_nhwc_to_nchw"] = [_vp, _i, _vp, _i, _i, _i, _i, _vp, _vp, _vp]
_SIGNATURES["lq_repack_oihw_to_ohwi_i8"] = [_vp, _vp, _i, _i, _i, _i, _vp]
_SIGNATURES["lq_im2col_ndhwc_i8"] = [_vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp]
_SIGNATURES["lq_transpose_i8"] = [_vp, _vp, _i, _sz, _sz, _sz, _sz, _vp]
_SIGNATURES["lq_maxpool2d_nhwc_i8"] = [_vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp]

_RESTYPE = {"lq_last_error": C.c_char_p, "lq_range_buffer_bytes": C.c_size_t}
_NO_STATUS = {"lq_version", "lq_last_error", "lq_op_count", "lq_range_buffer_bytes", "lq_last_tile_config"}

_lib = None
_initialised_device = None


ABI_VERSION = 3  # LQ_VERSION of include/lucid_hip.h this binding was written against


def load() -> C.CDLL:
    """dlopen the library and declare every signature.  Does not touch the GPU."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise GpuNotAvailable(
                f"{LIB_PATH} is missing: build it with `make -C lucid_amd/csrc` "
                "(hipcc --offload-arch=gfx950).  There is no CPU fallback."
            )
        lib = C.CDLL(LIB_PATH)
        lib.lq_version.restype = C.c_int
        if lib.lq_version() != ABI_VERSION:
            raise GpuNotAvailable(
                f"{LIB_PATH} has ABI version {lib.lq_version()}, this binding needs {ABI_VERSION}: "
                "rebuild it with `make -C lucid_amd/csrc` (argument structs differ between versions)")
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is not exported
            fn.argtypes = argtypes
            fn.restype = _RESTYPE.get(name, C.c_int)
        _lib = lib
    return _lib


def check(status: int) -> None:
    if status != 0:
        msg = load().lq_last_error().decode("utf-8", "replace")
        raise _STATUS_TO_EXC.get(status, LucidError)(msg)


_current_stream = None  # lq_stream used when a caller passes None; None = the default stream


def current_stream():
    return _current_stream


def set_current_stream(stream) -> None:
    global _current_stream
    _current_stream = stream


def _stream_last() -> frozenset:
    """Names of the entry points whose last parameter is the stream."""
    global _STREAM_LAST
    if _STREAM_LAST is None:
        import re

        text = re.sub(r"/\*.*?\*/", "", open(HEADER_PATH).read(), flags=re.S)
        _STREAM_LAST = frozenset(re.findall(r"\b(lq_[a-z0-9_]+)\s*\([^;{}]*lq_stream\s+stream\s*\)", text))
    return _STREAM_LAST


_STREAM_LAST = None


def call(name: str, *args):
    """Call an ABI function and raise on a non-zero status.  A ``None`` stream
    argument means the current stream (see ``set_current_stream``)."""
    fn = getattr(load(), name)
    if _current_stream is not None and args and args[-1] is None and name in _stream_last():
        args = args[:-1] + (_current_stream,)
    rc = fn(*args)
    if name not in _NO_STATUS:
        check(rc)
    return rc


def init(device: int = 0) -> None:
    """Select the device and allocate the library workspace (idempotent)."""
    global _initialised_device
    if _initialised_device != device:
        call("lq_init", device)
        _initialised_device = device


def is_available() -> bool:
    """True when the library loads and sees at least one device."""
    try:
        n = C.c_int(0)
        rc = load().lq_device_count(C.byref(n))
        return rc == 0 and n.value > 0
    except (OSError, LucidError):
        return False


def range_buffer_words() -> int:
    """float32 words of a kept-range buffer (``lq_range_buffer_bytes``)."""
    return int(load().lq_range_buffer_bytes()) // 4


def device_name() -> str:
    buf = C.create_string_buffer(256)
    call("lq_device_name", buf, 256)
    return buf.value.decode()


def op_registry() -> list[tuple[str, int, bool]]:
    """``(name, version, deterministic)`` rows, as ``op_registry_all`` in Lucid
    (``lucid/_C/bindings/bind_op_registry.cpp``)."""
    out = []
    for i in range(load().lq_op_count()):
        name, ver, det = C.c_char_p(), C.c_int(), C.c_int()
        call("lq_op_info", i, C.byref(name), C.byref(ver), C.byref(det))
        out.append((name.value.decode(), ver.value, bool(det.value)))
    return out


def declared_symbols() -> list[str]:
    """Function names declared in ``include/lucid_hip.h``."""
    import re

    text = open(HEADER_PATH).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lq_[a-z0-9_]+)\s*\(", text)))
