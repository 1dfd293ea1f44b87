"""``lucid.backends.quantized`` - quantized-GEMM engine selection
(``lucid/backends/__init__.py:57-97``), with the value this backend adds.

* ``"auto"``      - use the HIP int8 kernels when the library and a device are there.
* ``"hip"``       - require them (raises ``GpuNotAvailable`` otherwise).
* ``"mlx_group"`` - ``convert`` / ``quantize_dynamic`` build the group-wise
  weight-only ``QuantizedLinearMLX`` (int4 / int8 weights, float activations) for
  the Linear family, as Lucid does when its MLX engine is active; the kernels are
  the HIP ones.  Unlike Lucid, ``"auto"`` does not pick this form: the default here
  is the int8 x int8 integer GEMM.
* ``"reference"`` - Lucid's dequantize-to-float engine; accepted so that code
  written against Lucid keeps working, but modules built by this package always
  run the HIP kernels.
"""

from __future__ import annotations

from .. import _C


class _QuantizedBackend:
    _engine: str = "auto"

    @property
    def available(self) -> bool:
        """True when ``liblucid_hip.so`` loads and a device is visible."""
        return _C.is_available()

    @property
    def engine(self) -> str:
        return self._engine

    @engine.setter
    def engine(self, value: str) -> None:
        if value not in ("auto", "mlx_group", "reference", "hip"):
            raise ValueError(
                f"quantized.engine must be 'auto'/'mlx_group'/'reference'/'hip', got {value!r}")
        self._engine = value

    def use_mlx(self) -> bool:
        """Whether ``convert`` / ``quantize_dynamic`` route the Linear family to the
        group-wise weight-only form (only when asked for by name)."""
        if self._engine == "mlx_group":
            if not self.available:
                raise _C.GpuNotAvailable("quantized.engine = 'mlx_group' but no HIP device / library")
            return True
        return False

    def use_hip(self) -> bool:
        """Whether the HIP kernels should run given the current mode."""
        if self._engine == "hip":
            if not self.available:
                raise _C.GpuNotAvailable("quantized.engine = 'hip' but no HIP device / library")
            return True
        if self._engine == "auto":
            return self.available
        return False


quantized = _QuantizedBackend()

__all__ = ["quantized"]
