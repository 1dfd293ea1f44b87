"""Benchmark / test workloads built on the quantized modules: the int8
static-quantized ResNet-50 and the dynamic-quantized ViT-B/16 of the benchmark
configurations.

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

    fuse_join = True  # conv3 applies skip_add.add_relu in its epilogue (same bits, one kernel less)

    def forward(self, x):
        identity = x if self.downsample is None else self.downsample(x)
        h = self.conv2(self.conv1(x))
        if self.fuse_join:
            return self.conv3(h, join=(identity, self.skip_add, True))
        return self.skip_add.add_relu(self.conv3(h), identity)


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
        x = self.maxpool(self.conv1(x, quantize=self.quant))  # = conv1(quant(x)), quantized into the stem's packed image
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


# ---------------------------------------------------------------- ViT-B/16, dynamic int8 Linears
# Topology as Lucid's zoo builds it (``lucid/models/vision/vit/_model.py``): 16x16
# patch convolution, class token + position table, pre-norm blocks (LayerNorm eps
# 1e-6, packed qkv attention, 4x GELU MLP), final LayerNorm, class-token pooling,
# Linear head.  Every ``nn.Linear`` goes through ``quantize_dynamic`` (W8A8: weights
# per-output-channel symmetric qint8, activations per-tensor affine quint8 from the
# runtime min / max); patch embedding, LayerNorm, attention, GELU and the residual
# adds stay float32.
VIT_B16 = dict(image=224, patch=16, dim=768, depth=12, heads=12, mlp=3072, classes=1000)


def vit_float_params(cfg=VIT_B16, seed: int = 0) -> dict:
    """Random N(0, 0.02) weights (biases too, so that every term is exercised),
    LayerNorm at gamma = 1 + N(0, 0.02), beta = N(0, 0.02)."""
    rng = np.random.default_rng(seed)
    d, m = cfg["dim"], cfg["mlp"]
    n = lambda *s: (rng.standard_normal(s) * 0.02).astype(np.float32)
    tokens = (cfg["image"] // cfg["patch"]) ** 2 + 1
    p = {"patch.weight": n(d, 3, cfg["patch"], cfg["patch"]), "patch.bias": n(d), "cls": n(d),
         "pos": n(tokens, d), "norm.weight": 1 + n(d), "norm.bias": n(d),
         "head.weight": n(cfg["classes"], d), "head.bias": n(cfg["classes"])}
    for i in range(cfg["depth"]):
        b = f"blocks.{i}."
        p[b + "norm1.weight"], p[b + "norm1.bias"] = 1 + n(d), n(d)
        p[b + "norm2.weight"], p[b + "norm2.bias"] = 1 + n(d), n(d)
        p[b + "qkv.weight"], p[b + "qkv.bias"] = n(3 * d, d), n(3 * d)
        p[b + "proj.weight"], p[b + "proj.bias"] = n(d, d), n(d)
        p[b + "fc1.weight"], p[b + "fc1.bias"] = n(m, d), n(m)
        p[b + "fc2.weight"], p[b + "fc2.bias"] = n(d, m), n(d)
    return p


def _float_linear(w, b):
    lin = nn.Linear(w.shape[1], w.shape[0])
    lin.register_buffer("weight", L.tensor(w))
    lin.register_buffer("bias", L.tensor(b))
    return lin


def _layer_norm(w, b, eps=1e-6, track_range=True):
    ln = nn.LayerNorm(w.shape[0], eps=eps, track_range=track_range)
    ln.register_buffer("weight", L.tensor(w, device="hip"))
    ln.register_buffer("bias", L.tensor(b, device="hip"))
    return ln


class ViTBlock(nn.Module):
    fuse_gelu = True
    fuse_ln_quant = True  # LayerNorm writes the next Linear's int8 codes, not float32 (same bits)

    def __init__(self, prefix, p, heads):
        super().__init__()
        self.heads = heads
        self.norm1 = _layer_norm(p[prefix + "norm1.weight"], p[prefix + "norm1.bias"])
        self.norm2 = _layer_norm(p[prefix + "norm2.weight"], p[prefix + "norm2.bias"])
        self.qkv = _float_linear(p[prefix + "qkv.weight"], p[prefix + "qkv.bias"])
        self.proj = _float_linear(p[prefix + "proj.weight"], p[prefix + "proj.bias"])
        self.fc1 = _float_linear(p[prefix + "fc1.weight"], p[prefix + "fc1.bias"])
        self.fc2 = _float_linear(p[prefix + "fc2.weight"], p[prefix + "fc2.bias"])

    def forward(self, x):
        import lucid_amd.nn.functional as F

        # every float32 kernel that feeds a dynamic-quantized Linear keeps the range of
        # what it writes; the residual adds ride in the epilogues of proj and fc2
        a = F.scaled_dot_product_attention_qkv(self._norm_linear(self.norm1, self.qkv, x), self.heads,
                                               track_range=True)
        x = self.proj(a, residual=x)
        if self.fuse_gelu:  # GELU and the range of its result in fc1's epilogue (same bits, one kernel less)
            h = self._norm_linear(self.norm2, self.fc1, x, activation="gelu", track_range=True)
        else:
            h = F.gelu(self._norm_linear(self.norm2, self.fc1, x), track_range=True)
        return self.fc2(h, residual=x)

    def _norm_linear(self, norm, lin, x, **kw):
        """``lin(norm(x))``; with ``fuse_ln_quant`` the normalized activation goes to the Linear
        as codes without a float32 copy in between."""
        import lucid_amd.nn.functional as F

        if self.fuse_ln_quant:
            r = F.layer_norm_dynamic_quantize(x, norm.normalized_shape, norm.weight, norm.bias, norm.eps,
                                              lin.act_qdtype)
            if r is not None:
                return lin.forward_quantized(r[0], r[1], r[2], x.shape[:-1], **kw)
        return lin(norm(x), **kw)


class QViT(nn.Module):
    """ViT for image classification with dynamic-quantized Linears; input float32
    NCHW images on the hip device, output float32 logits."""

    def __init__(self, cfg=VIT_B16, params=None, seed: int = 0):
        super().__init__()
        p = params if params is not None else vit_float_params(cfg, seed)
        self.cfg = dict(cfg)
        d = cfg["dim"]
        self.register_buffer("patch_weight", L.tensor(p["patch.weight"].reshape(d, -1), device="hip"))
        self.register_buffer("patch_bias", L.tensor(p["patch.bias"], device="hip"))
        self.register_buffer("cls_token", L.tensor(p["cls"], device="hip"))
        self.register_buffer("pos_embed", L.tensor(p["pos"], device="hip"))
        self.blocks = nn.Sequential(*[ViTBlock(f"blocks.{i}.", p, cfg["heads"]) for i in range(cfg["depth"])])
        self.norm = _layer_norm(p["norm.weight"], p["norm.bias"], track_range=False)
        self.head = _float_linear(p["head.weight"], p["head.bias"])
        Q.quantize_dynamic(self, inplace=True)

    def forward(self, x):
        from lucid_amd import _C
        import lucid_amd.nn.functional as F

        cfg = self.cfg
        B, C, H, W = x.shape
        ps, d = cfg["patch"], cfg["dim"]
        n = (H // ps) * (W // ps)
        # patch rows, their Linear, the class token and the position table in one launch
        tok = L.Tensor.empty((B, n + 1, d), L.float32, "hip")
        _C.call("lq_patch_embed_f32", x.data_ptr, self.patch_weight.data_ptr, self.patch_bias.data_ptr,
                self.cls_token.data_ptr, self.pos_embed.data_ptr, tok.data_ptr, B, C, H, W, ps, d, None)
        tok = self.norm(self.blocks(tok))
        # class-token pooling: row 0 of every image
        cls = L.Tensor.empty((B, d), L.float32, "hip")
        _C.call("lq_gather_rows_f32", tok.data_ptr, (n + 1) * d, cls.data_ptr, B, d, None)
        return self.head(cls)


def vit_linear_gops(cfg=VIT_B16, batch: int = 1) -> float:
    """int8 operations (2 per multiply-accumulate) of the quantized Linears, in 1e9."""
    t = (cfg["image"] // cfg["patch"]) ** 2 + 1
    d, m = cfg["dim"], cfg["mlp"]
    per_block = 2.0 * t * (d * 3 * d + d * d + 2 * d * m)
    return batch * (cfg["depth"] * per_block + 2.0 * d * cfg["classes"]) / 1e9
