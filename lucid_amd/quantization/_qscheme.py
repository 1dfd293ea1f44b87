"""Quantization schemes and integer-grid descriptors.

Mirrors ``lucid/quantization/_qscheme.py:25-245``: same enum members, module
aliases, ``QDtype`` fields, bounds, storage dtypes (``quint8`` is held in
``int16`` because Lucid's dtype enum has no uint8) and ``repr``.
"""

from __future__ import annotations

import enum
from dataclasses import dataclass


class QScheme(enum.Enum):
    PER_TENSOR_AFFINE = "per_tensor_affine"
    PER_TENSOR_SYMMETRIC = "per_tensor_symmetric"
    PER_CHANNEL_AFFINE = "per_channel_affine"
    PER_CHANNEL_SYMMETRIC = "per_channel_symmetric"

    @property
    def is_per_channel(self) -> bool:
        return self in (QScheme.PER_CHANNEL_AFFINE, QScheme.PER_CHANNEL_SYMMETRIC)

    @property
    def is_symmetric(self) -> bool:
        return self in (QScheme.PER_TENSOR_SYMMETRIC, QScheme.PER_CHANNEL_SYMMETRIC)


per_tensor_affine: QScheme = QScheme.PER_TENSOR_AFFINE
per_tensor_symmetric: QScheme = QScheme.PER_TENSOR_SYMMETRIC
per_channel_affine: QScheme = QScheme.PER_CHANNEL_AFFINE
per_channel_symmetric: QScheme = QScheme.PER_CHANNEL_SYMMETRIC


@dataclass(frozen=True)
class QDtype:
    name: str
    bits: int
    signed: bool
    quant_min: int
    quant_max: int
    storage: str

    def __repr__(self) -> str:
        return f"lucid.quantization.{self.name}"

    # grid descriptors are singletons (code compares them with ``is``)
    def __copy__(self) -> "QDtype":
        return self

    def __deepcopy__(self, memo) -> "QDtype":
        return self


qint8: QDtype = QDtype("qint8", 8, True, -128, 127, "int8")
quint8: QDtype = QDtype("quint8", 8, False, 0, 255, "int16")
qint32: QDtype = QDtype("qint32", 32, True, -(2**31), 2**31 - 1, "int32")
qint4: QDtype = QDtype("qint4", 4, True, -8, 7, "int8")
