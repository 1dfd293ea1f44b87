"""Model-level workflow: ``prepare`` / ``convert`` / ``quantize_dynamic``
(``lucid/quantization/_quantize.py:204-311,314-419,429-554,684-699``).

Same control flow and warning texts as Lucid.  ``convert`` installs the hip
int8 modules; calibration itself (a float forward through the prepared model)
belongs to Lucid's float backends, so observers here are fed either by that
float model's activations moved to ``"hip"`` or through fixed qparams.
"""

from __future__ import annotations

import copy
import warnings

from .. import backends, nn
from ..nn import intrinsic as nni
from ..nn import quantized as nnq
from ..nn.quantized import dynamic as nnqd
from ._qscheme import QDtype, qint8
from .qconfig import QConfig, get_default_qconfig


def _observed_types() -> tuple[type, ...]:
    return (nn.Linear, nn.Conv1d, nn.Conv2d, nn.Conv3d, nni.LinearReLU, nni.ConvReLU1d, nni.ConvReLU2d, nni.ConvReLU3d, nnq.QuantStub,
            nnq.FloatFunctional, nn.ConvTranspose1d, nn.ConvTranspose2d, nn.ConvTranspose3d, nn.Sigmoid, nn.Hardswish, nn.Hardsigmoid, nn.Tanh, nn.ELU, nn.LeakyReLU)


def _quant_mapping() -> dict[type, object]:
    m = {
        nn.Linear: nnq.Linear.from_float,
        nni.LinearReLU: nnq.LinearReLU.from_float,
        nnq.QuantStub: nnq.Quantize.from_float,
        nnq.DeQuantStub: nnq.DeQuantize.from_float,
        nnq.FloatFunctional: nnq.QFunctional.from_float,
        nn.ConvTranspose2d: nnq.ConvTranspose2d.from_float,
        nn.ConvTranspose1d: nnq.ConvTranspose1d.from_float,
        nn.ConvTranspose3d: nnq.ConvTranspose3d.from_float,
        nn.Embedding: nnq.Embedding.from_float,
        nn.EmbeddingBag: nnq.EmbeddingBag.from_float,
        nn.Sigmoid: nnq.Sigmoid.from_float,
        nn.Hardswish: nnq.Hardswish.from_float,
        nn.Hardsigmoid: nnq.Hardsigmoid.from_float,
        nn.Tanh: nnq.Tanh.from_float,
        nn.ELU: nnq.ELU.from_float,
        nn.LeakyReLU: nnq.LeakyReLU.from_float,
    }
    if hasattr(nnq, "Conv2d"):
        m[nn.Conv2d] = nnq.Conv2d.from_float
        m[nn.Conv1d] = nnq.Conv1d.from_float
        m[nn.Conv3d] = nnq.Conv3d.from_float
        m[nni.ConvReLU2d] = nnq.ConvReLU2d.from_float
        m[nni.ConvReLU1d] = nnq.ConvReLU1d.from_float
        m[nni.ConvReLU3d] = nnq.ConvReLU3d.from_float
    return m


def _dynamic_mapping() -> dict[type, object]:
    return {nn.Linear: nnqd.Linear.from_float, nn.LSTM: nnqd.LSTM.from_float}


def _mlx_weight_bits(mod) -> int:
    """4 or 8, from the weight observer's dtype (``_quantize.py:116-123``)."""
    qcfg = getattr(mod, "qconfig", None)
    if qcfg is not None:
        bits = getattr(getattr(qcfg.weight(), "qdtype", None), "bits", None)
        if isinstance(bits, int) and bits in (4, 8):
            return bits
    return 8


def _mlx_group_size(in_features: int):
    """First of 64 / 128 / 32 that divides ``in_features``, else None
    (``_quantize.py:126-137``)."""
    for gs in (64, 128, 32):
        if in_features % gs == 0:
            return gs
    return None


def _mlx_linear_builder(relu: bool):
    """``convert`` builder for the group-wise weight-only Linear
    (``_quantize.py:140-163``); a layer no group size divides keeps the int8 form."""
    fallback = nnq.LinearReLU.from_float if relu else nnq.Linear.from_float

    def build(child):
        inner = child[0] if relu else child
        gs = _mlx_group_size(inner.in_features)
        if gs is None:
            return fallback(child)
        return nnq.QuantizedLinearMLX.from_float(
            inner, bits=_mlx_weight_bits(child), group_size=gs, relu=relu)

    return build


def _mlx_dynamic_builder():
    """``quantize_dynamic`` builder for the same (``_quantize.py:166-179``)."""

    def build(child, dtype):
        gs = _mlx_group_size(child.in_features)
        if gs is None:
            return nnqd.Linear.from_float(child, dtype)
        return nnq.QuantizedLinearMLX.from_float(child, bits=dtype.bits, group_size=gs, relu=False)

    return build


def _make_observer_hook(obs):
    def hook(_module, _args, output):
        obs(output)
    return hook


def prepare(model, qconfig: QConfig | None = None, inplace: bool = False):
    """Attach an activation observer (as a forward hook) and the ``qconfig`` to
    every quantizable module (``_quantize.py:204-311``)."""
    qcfg = qconfig if qconfig is not None else get_default_qconfig()
    model = model if inplace else copy.deepcopy(model)
    model.eval()
    observed = _observed_types()
    n_matched = 0
    for _name, mod in model.named_modules():
        if not isinstance(mod, observed):
            continue
        # the Linear / Conv inside a fused pair is observed through the pair
        mod.qconfig = qcfg
        obs = qcfg.activation()
        mod.activation_post_process = obs
        mod.register_forward_hook(_make_observer_hook(obs))
        n_matched += 1
    if n_matched == 0:
        warnings.warn(
            "prepare(): the QConfigMapping matched no quantizable modules — "
            "convert() will leave this model unchanged.",
            stacklevel=2,
        )
    return model


def _qat_mapping() -> dict[type, object]:
    """Float module type -> its QAT form (``_quantize.py:557-573``)."""
    import lucid_amd.nn.qat as nnqat
    return {nn.Linear: nnqat.Linear.from_float, nni.LinearReLU: nnqat.LinearReLU.from_float,
            nn.Conv1d: nnqat.Conv1d.from_float, nn.Conv2d: nnqat.Conv2d.from_float, nn.Conv3d: nnqat.Conv3d.from_float,
            nn.Embedding: nnqat.Embedding.from_float,
            nni.ConvReLU1d: nnqat.ConvReLU1d.from_float, nni.ConvReLU2d: nnqat.ConvReLU2d.from_float,
            nni.ConvReLU3d: nnqat.ConvReLU3d.from_float}


def _prepare_qat_recursive(module, qcfg, qat_map) -> int:
    n = 0
    for name, child in list(module.named_children()):
        build = qat_map.get(type(child))
        if build is not None:
            child.qconfig = qcfg
            module._modules[name] = build(child)
            n += 1
        elif isinstance(child, nnq.QuantStub):
            child.qconfig = qcfg
            child.activation_post_process = qcfg.activation()
            n += 1
        else:
            n += _prepare_qat_recursive(child, qcfg, qat_map)
    return n


def prepare_qat(model, qconfig: QConfig | None = None, inplace: bool = False):
    """Swap the weighted layers for their QAT forms and put a ``FakeQuantize`` on every
    ``QuantStub`` (``_quantize.py:575-700``).  The result runs the simulated-quantization
    forward on the device and converts with ``convert``; fine-tuning it is Lucid's job."""
    from .qconfig import get_default_qat_qconfig
    qcfg = qconfig if qconfig is not None else get_default_qat_qconfig()
    model = model if inplace else copy.deepcopy(model)
    if _prepare_qat_recursive(model, qcfg, _qat_mapping()) == 0:
        warnings.warn("prepare_qat(): no module of this model has a QAT form here", stacklevel=2)
    return model


def _convert_recursive(module, mapping, always) -> None:
    for name, child in list(module.named_children()):
        build = mapping.get(type(child))
        convertible = build is not None and (
            isinstance(child, always) or hasattr(child, "activation_post_process"))
        if convertible:
            module._modules[name] = build(child)  # keep the child's position
        else:
            _convert_recursive(child, mapping, always)


def convert(model, inplace: bool = False):
    """Swap every calibrated module for its quantized form
    (``_quantize.py:314-419``)."""
    model = model if inplace else copy.deepcopy(model)
    mapping = _quant_mapping()
    import lucid_amd.nn.qat as nnqat
    mapping[nnqat.Linear] = nnq.Linear.from_float
    mapping[nnqat.LinearReLU] = nnq.LinearReLU.from_float
    mapping[nnqat.Conv2d] = nnq.Conv2d.from_float
    mapping[nnqat.ConvReLU2d] = nnq.ConvReLU2d.from_float
    mapping[nnqat.Conv1d] = nnq.Conv1d.from_float
    mapping[nnqat.Conv3d] = nnq.Conv3d.from_float
    mapping[nnqat.ConvReLU1d] = nnq.ConvReLU1d.from_float
    mapping[nnqat.ConvReLU3d] = nnq.ConvReLU3d.from_float
    mapping[nnqat.Embedding] = nnq.Embedding.from_float
    import lucid_amd.nn.intrinsic.qat as nniqat
    for _cls in (nniqat.ConvBn1d, nniqat.ConvBn2d, nniqat.ConvBn3d, nniqat.ConvBnReLU1d, nniqat.ConvBnReLU2d,
                 nniqat.ConvBnReLU3d):
        mapping[_cls] = nniqat.convbn_to_quantized
    if backends.quantized.use_mlx():
        mapping[nn.Linear] = _mlx_linear_builder(relu=False)
        mapping[nni.LinearReLU] = _mlx_linear_builder(relu=True)
    # DeQuantStub and the embedding tables convert without calibration (_quantize.py:414-417)
    _convert_recursive(model, mapping, always=(nnq.DeQuantStub, nn.Embedding, nn.EmbeddingBag))
    model.eval()
    return model


def _swap_dynamic(module, mapping, types, dtype) -> None:
    for name, child in list(module.named_children()):
        build = mapping.get(type(child))
        if build is not None and type(child) in types:
            module._modules[name] = build(child, dtype)
        else:
            _swap_dynamic(child, mapping, types, dtype)


def quantize_dynamic(model, qconfig_spec=None, dtype: QDtype = qint8, inplace: bool = False):
    """Calibration-free dynamic quantization of every ``nn.Linear``
    (``_quantize.py:429-539``)."""
    model = model if inplace else copy.deepcopy(model)
    model.eval()
    mapping = _dynamic_mapping()
    if backends.quantized.use_mlx():
        mapping[nn.Linear] = _mlx_dynamic_builder()
    types = qconfig_spec if qconfig_spec is not None else set(mapping)
    if not any(type(m) in types for m in model.modules()):
        warnings.warn(
            "quantize_dynamic(): no module of a targeted type "
            f"({', '.join(sorted(t.__name__ for t in types))}) found — "
            "the model is returned unchanged.",
            stacklevel=2,
        )
    build = mapping.get(type(model))
    if build is not None and type(model) in types:
        return build(model, dtype)
    _swap_dynamic(model, mapping, types, dtype)
    return model
