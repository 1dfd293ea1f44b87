"""Benchmark / test workloads built on the quantized modules: the int8
static-quantized ResNet-50 of the benchmark configuration.

Topology is torchvision-style ResNet-50 v1.5, as Lucid's zoo builds it
(``lucid/models/vision/resnet/_model.py:109-210,255-299``): 7x7/2 stem,
3x3/2 max-pool, bottleneck stages [3, 4, 6, 3] with the stride on the 3x3
convolution, 1x1 projection shortcuts, global average pool, 1000-way
classifier.  Weights are random He-normal (fan-out), BatchNorm at its initial
state (gamma 1, beta 0, running mean 0, running var 1) folded into the
convolutions (``lucid/nn/utils/fusion.py:103-139``).  conv1 / conv2 of a
bottleneck are ConvReLU2d, conv3 and the projection plain Conv2d, the join is
``QFunctional.add_relu``.  Activation grids are fixed calibration ranges
(``FixedQParamsObserver`` semantics) read from a committed fixture.
"""

from __future__ import annotations

import json
import os

import numpy as np

import lucid_amd as L
import lucid_amd.nn as nn
import lucid_amd.nn.intrinsic as nni
import lucid_amd.nn.quantized as nnq
import lucid_amd.quantization as Q

ROOT = os.path.dirname(os.path.abspath(__file__))
CALIBRATION_FIXTURE = os.path.join(ROOT, "tests", "golden", "resnet50_calibration.json")
BN_EPS = 1e-5
STAGES = ((64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2))  # (planes, blocks, stride)


def resnet50_convs():
    """``(name, cin, cout, k, stride, pad, relu)`` for the 53 convolutions, in
    execution order."""
    convs = [("conv1", 3, 64, 7, 2, 3, True)]
    inplanes = 64
    for si, (planes, blocks, stride) in enumerate(STAGES, start=1):
        for b in range(blocks):
            s = stride if b == 0 else 1
            p = f"layer{si}.{b}"
            convs.append((f"{p}.conv1", inplanes, planes, 1, 1, 0, True))
            convs.append((f"{p}.conv2", planes, planes, 3, s, 1, True))
            convs.append((f"{p}.conv3", planes, planes * 4, 1, 1, 0, False))
            if b == 0:
                convs.append((f"{p}.downsample", inplanes, planes * 4, 1, s, 0, False))
            inplanes = planes * 4
    return convs


def resnet50_float_params(seed: int = 0):
    """Folded float parameters: name -> (weight OIHW float32, bias float32)."""
    rng = np.random.default_rng(seed)
    fold = np.float32(1.0 / np.sqrt(1.0 + BN_EPS))  # gamma / sqrt(var + eps), fusion.py:103-139
    params = {}
    for name, cin, cout, k, _s, _p, _r in resnet50_convs():
        std = np.sqrt(2.0 / (cout * k * k))  # He normal, fan-out
        w = (rng.standard_normal((cout, cin, k, k)) * std).astype(np.float32)
        params[name] = (w * fold, np.zeros(cout, np.float32))
    wfc = (rng.standard_normal((1000, 2048)) * 0.01).astype(np.float32)
    params["fc"] = (wfc, np.zeros(1000, np.float32))
    return params


def load_calibration(path: str = CALIBRATION_FIXTURE) -> dict:
    """Observer point -> [min, max] of the float activation there."""
    with open(path) as f:
        return json.load(f)["ranges"]


def _fixed_qconfig(lo: float, hi: float) -> Q.QConfig:
    """Activation grid fixed to the calibrated range; per-channel symmetric
    int8 weights (Lucid's default weight observer)."""
    def act():
        obs = Q.MinMaxObserver()
        obs.register_buffer("min_val", L.tensor(np.float32(lo), device="hip"))
        obs.register_buffer("max_val", L.tensor(np.float32(hi), device="hip"))
        return obs
    return Q.QConfig(activation=act, weight=Q.get_default_qconfig().weight)


def _qconv(name, spec, params, calib):
    _n, cin, cout, k, s, p, relu = spec
    w, b = params[name]
    conv = nn.Conv2d(cin, cout, k, stride=s, padding=p, bias=True)
    conv.register_buffer("weight", L.tensor(w))
    conv.register_buffer("bias", L.tensor(b))
    lo, hi = calib[name]
    holder = nni.ConvReLU2d(conv, nn.ReLU()) if relu else conv
    holder.qconfig = _fixed_qconfig(lo, hi)
    holder.activation_post_process = holder.qconfig.activation()
    return (nnq.ConvReLU2d if relu else nnq.Conv2d).from_float(holder)


def _qfunctional(name, calib):
    ff = nnq.FloatFunctional()
    ff.qconfig = _fixed_qconfig(*calib[name])
    ff.activation_post_process = ff.qconfig.activation()
    return nnq.QFunctional.from_float(ff)


class QBottleneck(nn.Module):
    def __init__(self, prefix, specs, params, calib, has_down):
        super().__init__()
        self.conv1 = _qconv(f"{prefix}.conv1", specs[f"{prefix}.conv1"], params, calib)
        self.conv2 = _qconv(f"{prefix}.conv2", specs[f"{prefix}.conv2"], params, calib)
        self.conv3 = _qconv(f"{prefix}.conv3", specs[f"{prefix}.conv3"], params, calib)
        self.downsample = (_qconv(f"{prefix}.downsample", specs[f"{prefix}.downsample"], params,
                                  calib) if has_down else None)
        self.skip_add = _qfunctional(f"{prefix}.add", calib)

    def forward(self, x):
        identity = x if self.downsample is None else self.downsample(x)
        out = self.conv3(self.conv2(self.conv1(x)))
        return self.skip_add.add_relu(out, identity)


class QResNet50(nn.Module):
    """Statically quantized ResNet-50; input float32 NCHW on the hip device,
    output float32 logits (on the classifier's output grid)."""

    def __init__(self, params=None, calib=None, seed: int = 0):
        super().__init__()
        params = params if params is not None else resnet50_float_params(seed)
        calib = calib if calib is not None else load_calibration()
        specs = {c[0]: c for c in resnet50_convs()}
        stub = nnq.QuantStub()
        stub.qconfig = _fixed_qconfig(*calib["input"])
        stub.activation_post_process = stub.qconfig.activation()
        self.quant = nnq.Quantize.from_float(stub)
        self.conv1 = _qconv("conv1", specs["conv1"], params, calib)
        self.maxpool = nn.MaxPool2d(3, 2, 1)
        blocks = []
        for si, (_planes, nblocks, _stride) in enumerate(STAGES, start=1):
            for b in range(nblocks):
                blocks.append(QBottleneck(f"layer{si}.{b}", specs, params, calib, has_down=(b == 0)))
        self.blocks = nn.Sequential(*blocks)
        self.avgpool = nn.AdaptiveAvgPool2d(1)
        self.flatten = nn.Flatten()
        wfc, bfc = params["fc"]
        fc = nn.Linear(2048, 1000)
        fc.register_buffer("weight", L.tensor(wfc))
        fc.register_buffer("bias", L.tensor(bfc))
        fc.qconfig = _fixed_qconfig(*calib["fc"])
        fc.activation_post_process = fc.qconfig.activation()
        self.fc = nnq.Linear.from_float(fc)
        self.dequant = nnq.DeQuantize()

    def forward(self, x):
        x = self.maxpool(self.conv1(self.quant(x)))
        x = self.blocks(x)
        return self.dequant(self.fc(self.flatten(self.avgpool(x))))


def resnet50_conv_gmacs(batch: int, size: int = 224) -> float:
    """Multiply-accumulates of the 53 convolutions + classifier, in units of 1e9."""
    total, h = 0, size
    hw = {}
    h = (size + 6 - 7) // 2 + 1
    hw["conv1"] = h
    h = (h + 2 - 3) // 2 + 1
    cur = h
    for name, cin, cout, k, s, p, _r in resnet50_convs():
        if name == "conv1":
            out = hw["conv1"]
            total += out * out * cout * cin * k * k
            continue
        if name.endswith("conv1"):
            block_in = cur
            out = cur
        elif name.endswith("conv2"):
            out = (cur + 2 * p - k) // s + 1
            cur = out
        elif name.endswith("conv3"):
            out = cur
        else:  # downsample sees the block input
            out = (block_in + 2 * p - k) // s + 1
        total += out * out * cout * cin * k * k
    total += 2048 * 1000
    return batch * total / 1e9
