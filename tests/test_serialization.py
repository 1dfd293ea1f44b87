"""Checkpoint wire formats (host-side; no GPU needed): the ``.lucid`` container and
SafeTensors with Lucid's 0-d convention."""

import io
import pickle

import numpy as np
import pytest

import lucid_amd as L
from lucid_amd import serialization as S


def _state():
    rng = np.random.default_rng(0)
    return {
        "fc1.weight_int8": L.tensor(rng.integers(-128, 128, (5, 7)).astype(np.int8)),
        "fc1.weight_scale": L.tensor(rng.uniform(0.01, 0.1, 5).astype(np.float32)),
        "fc1.weight_zero_point": L.tensor(np.zeros(5, np.float32)),
        "fc1.bias": L.tensor(rng.standard_normal(5).astype(np.float32)),
        "fc1.scale": L.tensor(np.float32(0.037)),
        "fc1.zero_point": L.tensor(np.float32(128.0)),
    }


def _same(a, b):
    assert a.keys() == b.keys()
    for k in a:
        assert a[k].shape == b[k].shape and a[k].dtype == b[k].dtype, k
        assert a[k].numpy().tobytes() == b[k].numpy().tobytes(), k


def test_zero_d_tensors_stay_zero_d():
    t = L.tensor(np.float32(0.5))
    assert t.shape == () and t.numel == 1 and t.item() == 0.5


def test_lucid_container_round_trip_and_layout(tmp_path):
    sd = _state()
    path = str(tmp_path / "q.lucid")
    L.save(sd, path)
    back = L.load(path)
    _same(sd, back)
    assert back["fc1.weight_int8"].dtype is L.int8  # test_static_ptq.py:139
    assert back["fc1.scale"].shape == ()

    # the stream is what lucid/serialization/__init__.py:75-84,170-176 describes
    seen = []

    class Peek(pickle.Unpickler):
        def persistent_load(self, pid):
            seen.append(pid)
            return None

    with open(path, "rb") as fp:
        container = Peek(fp).load()
    assert container["_lucid_format"] == 2 and set(container["obj"]) == set(sd)
    tag, shape, dtype_name, device, raw = seen[0]
    assert (tag, shape, dtype_name, device) == ("tensor_v3", [5, 7], "int8", "cpu")
    assert raw == sd["fc1.weight_int8"].numpy().tobytes()


def test_lucid_load_refuses_anything_but_containers_and_tensors(tmp_path):
    class Evil:
        def __reduce__(self):
            return (print, ("should never run",))

    path = str(tmp_path / "evil.lucid")
    with open(path, "wb") as fp:
        pickle.dump({"_lucid_format": 2, "obj": Evil()}, fp)
    with pytest.raises(pickle.UnpicklingError):
        L.load(path)
    with open(path, "wb") as fp:
        pickle.dump({"not": "a checkpoint"}, fp)
    with pytest.raises(RuntimeError):
        L.load(path)


def test_safetensors_interoperates_with_the_safetensors_package(tmp_path):
    st = pytest.importorskip("safetensors.numpy")
    sd = _state()
    path = str(tmp_path / "q.safetensors")
    S.save_safetensors(sd, path, metadata={"model": "mlp"})
    theirs = st.load_file(path)
    for k, t in sd.items():
        exp = t.numpy().reshape((1,)) if t.shape == () else t.numpy()  # 0-d stored as (1,)
        assert theirs[k].dtype == exp.dtype and np.array_equal(theirs[k], exp)
    from safetensors import safe_open

    with safe_open(path, framework="np") as f:
        meta = f.metadata()
    assert meta["model"] == "mlp"
    assert set(meta["__lucid_scalar_keys__"].split(",")) == {"fc1.scale", "fc1.zero_point"}
    _same(sd, S.load_safetensors(path))
    _same(sd, L.load(path))  # load() dispatches on the suffix, serialization/__init__.py:221-223

    # and a file written by the package, with Lucid's scalar convention, reads back 0-d
    path2 = str(tmp_path / "theirs.safetensors")
    st.save_file({"w": np.arange(6, dtype=np.int8).reshape(2, 3), "s": np.array([0.25], np.float32)}, path2,
                 metadata={"__lucid_scalar_keys__": "s"})
    back = S.load_safetensors(path2)
    assert back["w"].dtype is L.int8 and back["w"].shape == (2, 3)
    assert back["s"].shape == () and back["s"].item() == 0.25


def test_save_safetensors_wants_tensors():
    with pytest.raises(TypeError):
        S.save_safetensors({"x": 3}, "/tmp/never-written.safetensors")
