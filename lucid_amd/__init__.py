"""lucid_amd - MI355X (gfx950) backend for Lucid's int8 quantized-inference path.

The package mirrors the slice of Lucid's Python surface that the path uses
(``lucid.tensor``, dtypes, ``lucid.quantization``, ``lucid.nn.quantized``,
``lucid.backends.quantized``) on a third device, ``"hip"``.  All compute goes
through the C ABI of ``liblucid_hip.so``; there is no CPU fallback and no
dependency on PyTorch.
"""

from . import _C
from ._C import (
    DeviceMismatch,
    DtypeMismatch,
    GpuNotAvailable,
    LucidError,
    OutOfMemory,
    ShapeMismatch,
)
from ._tensor import (
    Tensor,
    bool_,
    dtype,
    float16,
    float32,
    float64,
    int8,
    int16,
    int32,
    int64,
    is_floating_point,
    synchronize,
    tensor,
)
from ._engine_ops import (add, amax, amin, clip, div, maximum, minimum, mul, round, sub)  # noqa: A004
from . import quantization
from . import nn
from . import backends
from . import graph
from . import serialization
from .serialization import load, save

__version__ = "0.1.0"


def is_available() -> bool:
    """True when the HIP library loads and a device is visible."""
    return _C.is_available()
