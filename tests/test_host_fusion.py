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


def _randomize_bn(bn, rng):
    n = bn.num_features
    bn.register_buffer("weight", L.tensor(rng.uniform(0.5, 1.5, n).astype(np.float32)))
    bn.register_buffer("bias", L.tensor(rng.standard_normal(n).astype(np.float32)))
    bn.register_buffer("running_mean", L.tensor(rng.standard_normal(n).astype(np.float32)))
    bn.register_buffer("running_var", L.tensor(rng.uniform(0.2, 2.0, n).astype(np.float32)))


@pytest.mark.parametrize("rank", [1, 3])
def test_conv_bn_fold_in_one_and_three_dimensions(rank):
    """fusion.py:27-28 accepts Conv1d/2d/3d with BatchNorm1d/2d/3d: the fold equals
    bn(conv(x)) computed by torch in float64 on the same parameters."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(10 + rank)
    conv = (nn.Conv1d(4, 6, 3, padding=1) if rank == 1 else nn.Conv3d(4, 6, 3, padding=1))
    bn = nn.BatchNorm1d(6) if rank == 1 else nn.BatchNorm3d(6)
    _randomize_bn(bn, rng)
    fused = fuse_conv_bn_eval(conv, bn)
    assert type(fused) is type(conv) and fused.weight.shape == conv.weight.shape
    shape = (2, 4, 9) if rank == 1 else (2, 4, 5, 6, 7)
    x = torch.from_numpy(rng.standard_normal(shape)).double()
    F = torch.nn.functional
    cf = F.conv1d if rank == 1 else F.conv3d
    t = lambda a: torch.from_numpy(a.numpy()).double()
    y_ref = F.batch_norm(cf(x, t(conv.weight), t(conv.bias), 1, 1), t(bn.running_mean), t(bn.running_var),
                         t(bn.weight), t(bn.bias), False, 0.0, bn.eps)
    y = cf(x, t(fused.weight), t(fused.bias), 1, 1)
    assert np.allclose(y.numpy(), y_ref.numpy(), atol=1e-5)
    with pytest.raises(TypeError):
        fuse_conv_bn_eval(nn.Linear(4, 4), bn)
    with pytest.raises(TypeError):
        fuse_conv_bn_eval(conv, nn.ReLU())


def test_fold_without_affine_parameters():
    rng = np.random.default_rng(3)
    conv = nn.Conv2d(3, 5, 1)
    bn = nn.BatchNorm2d(5, affine=False)
    bn.register_buffer("running_mean", L.tensor(rng.standard_normal(5).astype(np.float32)))
    bn.register_buffer("running_var", L.tensor(rng.uniform(0.2, 2.0, 5).astype(np.float32)))
    fused = fuse_conv_bn_eval(conv, bn)
    inv = 1.0 / np.sqrt(bn.running_var.numpy().astype(np.float64) + bn.eps)
    assert np.allclose(fused.weight.numpy(), conv.weight.numpy() * inv[:, None, None, None], rtol=1e-6)
    assert np.allclose(fused.bias.numpy(), (conv.bias.numpy() - bn.running_mean.numpy()) * inv, rtol=1e-5, atol=1e-7)


def test_fuse_modules_in_one_and_three_dimensions():
    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.c1, self.b1, self.r1 = nn.Conv1d(2, 4, 3), nn.BatchNorm1d(4), nn.ReLU()
            self.c3, self.b3, self.r3 = nn.Conv3d(2, 4, 3), nn.BatchNorm3d(4), nn.ReLU()
    fused = Q.fuse_modules(Net(), [["c1", "b1", "r1"], ["c3", "b3", "r3"]])
    assert isinstance(fused.c1, nni.ConvReLU1d) and isinstance(fused.c3, nni.ConvReLU3d)
    assert all(isinstance(m, nn.Identity) for m in (fused.b1, fused.r1, fused.b3, fused.r3))
    fused = Q.fuse_modules(Net(), [["c1", "b1"], ["c3", "r3"]])
    assert isinstance(fused.c1, nn.Conv1d) and isinstance(fused.c3, nni.ConvReLU3d)
