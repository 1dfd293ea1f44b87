"""The C-ABI library loads without a GPU and exports every symbol that
``include/lucid_hip.h`` declares; error paths that need no device behave."""

import ctypes as C

import pytest

import lucid_amd as L
from lucid_amd import _C


def test_library_exports_every_declared_symbol():
    lib = _C.load()
    declared = _C.declared_symbols()
    assert len(declared) >= 25
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in lucid_hip.h but not exported"
    assert set(declared) == set(_C._SIGNATURES), "binding table and header disagree"


def test_inline_assembly_mfma_loop_is_clean():
    """The one-wavefront-per-SIMD GEMM kernel issues its MFMAs from inline assembly, so the
    compiler must not touch an accumulator inside the k loop (it would read a register an MFMA is
    still writing).  `make check` compiles the kernel to ISA (cached after a build) and verifies
    that the loop holds no register move or spill."""
    import os
    import subprocess
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "lucid_amd", "csrc")
    r = subprocess.run(["make", "-C", csrc, "check"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count("clean") >= 2 and "NOT CLEAN" not in r.stdout


def test_version_and_registry():
    assert _C.load().lq_version() == _C.ABI_VERSION == 3
    ops = dict((n, (v, d)) for n, v, d in _C.op_registry())
    for name in ("quantize", "dequantize", "fake_quantize", "minmax", "calc_qparams"):
        assert ops[name] == (1, True)


def test_status_codes_map_to_lucid_error_names():
    # lucid/_C/core/Error.h:63-495 / bindings/bind_errors.cpp
    for cls in (L.OutOfMemory, L.ShapeMismatch, L.DtypeMismatch, L.DeviceMismatch,
                L.GpuNotAvailable):
        assert issubclass(cls, L.LucidError) and issubclass(cls, RuntimeError)


def test_argument_errors_need_no_device():
    lib = _C.load()
    assert lib.lq_device_count(None) == 1  # ValueError status
    assert b"NULL" in lib.lq_last_error()
    name = C.c_char_p()
    assert lib.lq_op_info(10_000, C.byref(name), None, None) == 1
    with pytest.raises(ValueError):
        _C.call("lq_op_info", -1, C.byref(name), None, None)


def test_cpu_tensors_are_containers_only():
    import numpy as np
    import lucid_amd.quantization as Q
    x = L.tensor([1.0, 2.0])
    assert x.device == "cpu" and x.dtype is L.float32
    assert np.array_equal(x.numpy(), np.array([1, 2], np.float32))
    with pytest.raises(L.DeviceMismatch):
        Q.quantize(x, 0.1, 0.0, Q.qint8)
    with pytest.raises(ValueError):
        L.tensor([1.0], device="metal")


def test_qdtype_and_qscheme_surface():
    # lucid/test/unit/quantization/test_functional.py:10-32
    import lucid_amd.quantization as Q
    assert (Q.qint8.quant_min, Q.qint8.quant_max) == (-128, 127)
    assert (Q.quint8.quant_min, Q.quint8.quant_max) == (0, 255)
    assert (Q.qint4.quant_min, Q.qint4.quant_max) == (-8, 7)
    assert Q.qint8.signed and not Q.quint8.signed
    for qd in (Q.qint8, Q.quint8, Q.qint32, Q.qint4):
        assert isinstance(getattr(L, qd.storage), L.dtype)
    assert repr(Q.qint8) == "lucid.quantization.qint8"
    assert Q.quint8.storage == "int16"
    assert Q.per_channel_symmetric.is_per_channel and not Q.per_tensor_affine.is_per_channel
    assert Q.per_tensor_symmetric.is_symmetric and not Q.per_channel_affine.is_symmetric
    assert Q.per_channel_symmetric is Q.QScheme.PER_CHANNEL_SYMMETRIC
