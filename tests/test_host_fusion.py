"""Conv + BatchNorm folding and ``fuse_modules`` (host-side, no GPU):
lucid/test/unit/quantization/test_static_ptq.py:88-111."""

import numpy as np
import pytest

import lucid_amd as L
import lucid_amd.nn as nn
import lucid_amd.nn.intrinsic as nni
import lucid_amd.quantization as Q
from lucid_amd.nn.utils import fuse_conv_bn_eval


def _net(rng):
    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.conv = nn.Conv2d(3, 8, 3, padding=1, bias=False)
            self.bn = nn.BatchNorm2d(8)
            self.relu = nn.ReLU()
            self.fc = nn.Linear(8, 10)
            self.act = nn.ReLU()
    net = Net()
    net.bn.register_buffer("weight", L.tensor(rng.uniform(0.5, 1.5, 8).astype(np.float32)))
    net.bn.register_buffer("bias", L.tensor(rng.standard_normal(8).astype(np.float32)))
    net.bn.register_buffer("running_mean", L.tensor(rng.standard_normal(8).astype(np.float32)))
    net.bn.register_buffer("running_var", L.tensor(rng.uniform(0.2, 2.0, 8).astype(np.float32)))
    return net


def test_conv_bn_fold_matches_unfused():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(1)
    net = _net(rng)
    fused = fuse_conv_bn_eval(net.conv, net.bn)
    x = torch.from_numpy(rng.standard_normal((2, 3, 8, 8)).astype(np.float32))
    F = torch.nn.functional
    w = torch.from_numpy(net.conv.weight.numpy())
    y_ref = F.batch_norm(F.conv2d(x, w, None, 1, 1), torch.from_numpy(net.bn.running_mean.numpy()),
                         torch.from_numpy(net.bn.running_var.numpy()),
                         torch.from_numpy(net.bn.weight.numpy()), torch.from_numpy(net.bn.bias.numpy()),
                         False, 0.0, net.bn.eps)
    y = F.conv2d(x, torch.from_numpy(fused.weight.numpy()), torch.from_numpy(fused.bias.numpy()), 1, 1)
    assert np.allclose(y.numpy(), y_ref.numpy(), atol=1e-4)      # test_static_ptq.py:90-99
    # closed form, float32
    scale = net.bn.weight.numpy() / np.sqrt(net.bn.running_var.numpy() + np.float32(net.bn.eps))
    assert np.allclose(fused.weight.numpy(), net.conv.weight.numpy() * scale[:, None, None, None],
                       rtol=1e-6, atol=0)
    assert np.allclose(fused.bias.numpy(),
                       (0 - net.bn.running_mean.numpy()) * scale + net.bn.bias.numpy(), rtol=1e-5, atol=1e-7)
    assert net.conv.bias is None                                 # the original is untouched


def test_fuse_modules_patterns():
    net = _net(np.random.default_rng(2))
    fused = Q.fuse_modules(net, [["conv", "bn"]])
    assert isinstance(fused.conv, nn.Conv2d) and isinstance(fused.bn, nn.Identity)
    assert isinstance(net.bn, nn.BatchNorm2d)
    fused = Q.fuse_modules(net, [["conv", "bn", "relu"], ["fc", "act"]])
    assert isinstance(fused.conv, nni.ConvReLU2d) and isinstance(fused.bn, nn.Identity)
    assert isinstance(fused.relu, nn.Identity)
    assert isinstance(fused.fc, nni.LinearReLU) and isinstance(fused.act, nn.Identity)
    with pytest.raises(ValueError):
        Q.fuse_modules(net, [["fc", "bn"]])
