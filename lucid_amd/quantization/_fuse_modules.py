"""``fuse_modules``: collapse Conv/BN/ReLU and Linear/ReLU runs before
``prepare`` (``lucid/quantization/fuse_modules.py:92-185``).  The first member
of each run is replaced by the fused module, the rest by ``Identity``."""

from __future__ import annotations

import copy
from typing import Sequence

from .. import nn
from ..nn import intrinsic as nni
from ..nn.utils.fusion import fuse_conv_bn_eval


def _get(model, dotted: str):
    mod = model
    for part in dotted.split("."):
        mod = mod._modules[part]
    return mod


def _set(model, dotted: str, new) -> None:
    parts = dotted.split(".")
    parent = model
    for part in parts[:-1]:
        parent = parent._modules[part]
    parent._modules[parts[-1]] = new


_CONV_TYPES = (nn.Conv1d, nn.Conv2d, nn.Conv3d)
_BN_TYPES = (nn.BatchNorm1d, nn.BatchNorm2d, nn.BatchNorm3d)


def _conv_relu(conv, relu):
    return {nn.Conv1d: nni.ConvReLU1d, nn.Conv2d: nni.ConvReLU2d, nn.Conv3d: nni.ConvReLU3d}[type(conv)](conv, relu)


def _fuse_run(mods):
    """Replacements for a fusible run: the fused module first, ``Identity`` for the rest
    (``fuse_modules.py:60-84``)."""
    ids = [nn.Identity() for _ in range(len(mods) - 1)]
    first = mods[0]
    if isinstance(first, _CONV_TYPES):
        rest = list(mods[1:])
        conv = first
        if rest and isinstance(rest[0], _BN_TYPES):
            conv = fuse_conv_bn_eval(first, rest.pop(0))
        if rest and isinstance(rest[0], nn.ReLU):
            rest.pop(0)
            conv = _conv_relu(conv, nn.ReLU())
        if not rest:
            return [conv, *ids]
    if isinstance(first, nn.Linear) and len(mods) == 2 and isinstance(mods[1], nn.ReLU):
        return [nni.LinearReLU(first, nn.ReLU()), *ids]
    raise ValueError(f"fuse_modules: unsupported fusion pattern {[type(m).__name__ for m in mods]}")


def fuse_modules(model, modules_to_fuse: Sequence[Sequence[str]], inplace: bool = False):
    model = model if inplace else copy.deepcopy(model)
    for group in modules_to_fuse:
        mods = [_get(model, name) for name in group]
        for name, new in zip(group, _fuse_run(mods)):
            _set(model, name, new)
    return model


def _fuse_run_qat(mods, qconfig):
    """QAT replacements (``fuse_modules.py:186-216``): a Conv + BN (+ ReLU) run becomes the
    ``nn.intrinsic.qat`` module that folds the BatchNorm on every forward; runs without a
    BatchNorm become the plain fused marker that ``prepare_qat`` then swaps."""
    from ..nn.intrinsic import qat as nniqat
    ids = [nn.Identity() for _ in range(len(mods) - 1)]
    first = mods[0]
    if isinstance(first, _CONV_TYPES):
        rank = _CONV_TYPES.index(type(first)) + 1
        rest = list(mods[1:])
        if rest and isinstance(rest[0], _BN_TYPES):
            bn = rest.pop(0)
            relu = bool(rest and isinstance(rest[0], nn.ReLU))
            plain = (nniqat.ConvBn1d, nniqat.ConvBn2d, nniqat.ConvBn3d)[rank - 1]
            fused = (nniqat.ConvBnReLU1d, nniqat.ConvBnReLU2d, nniqat.ConvBnReLU3d)[rank - 1]
            return [(fused if relu else plain)(first, bn, qconfig=qconfig), *ids]
        if rest and isinstance(rest[0], nn.ReLU):
            return [_conv_relu(first, nn.ReLU()), *ids]
        return [first, *ids]
    if isinstance(first, nn.Linear) and len(mods) == 2 and isinstance(mods[1], nn.ReLU):
        return [nni.LinearReLU(first, nn.ReLU()), *ids]
    raise ValueError(f"fuse_modules_qat: unsupported pattern {[type(m).__name__ for m in mods]}")


def fuse_modules_qat(model, modules_to_fuse: Sequence[Sequence[str]], qconfig, inplace: bool = False):
    """``fuse_modules`` for the QAT workflow (``fuse_modules.py:219-330``), run before
    ``prepare_qat``."""
    model = model if inplace else copy.deepcopy(model)
    for group in modules_to_fuse:
        mods = [_get(model, name) for name in group]
        for name, new in zip(group, _fuse_run_qat(mods, qconfig)):
            _set(model, name, new)
    return model
