"""Minimal ``nn.Module`` for the quantized-inference path.

Keeps the part of Lucid's module contract the path relies on
(``lucid/nn/modules`` + ``lucid/quantization/_quantize.py``): ordered
``_modules`` / ``_buffers`` registries, ``named_children`` / ``named_modules``,
``register_buffer``, ``state_dict`` / ``load_state_dict`` with dotted names,
``eval`` and forward hooks (observers are attached as forward hooks by
``prepare``).  Parameters of float modules are plain tensors here - there is
no autograd on this path.
"""

from __future__ import annotations

from collections import OrderedDict

from .._tensor import Tensor


class Module:
    def __init__(self) -> None:
        object.__setattr__(self, "_modules", OrderedDict())
        object.__setattr__(self, "_buffers", OrderedDict())
        object.__setattr__(self, "_forward_hooks", [])
        object.__setattr__(self, "training", True)

    # -- registration
    def register_buffer(self, name: str, tensor: Tensor | None) -> None:
        self.__dict__.pop(name, None)
        self._buffers[name] = tensor

    def register_forward_hook(self, hook) -> None:
        self._forward_hooks.append(hook)

    def __setattr__(self, name, value) -> None:
        if isinstance(value, Module):
            self.__dict__.pop(name, None)
            self._buffers.pop(name, None)
            self._modules[name] = value
        elif name in self.__dict__.get("_buffers", ()):
            self._buffers[name] = value
        else:
            self.__dict__.get("_modules", {}).pop(name, None)
            object.__setattr__(self, name, value)

    def __getattr__(self, name):
        d = self.__dict__
        if name in d.get("_modules", ()):
            return d["_modules"][name]
        if name in d.get("_buffers", ()):
            return d["_buffers"][name]
        raise AttributeError(f"{type(self).__name__!r} object has no attribute {name!r}")

    # -- traversal
    def named_children(self):
        return list(self._modules.items())

    def children(self):
        return list(self._modules.values())

    def named_modules(self, prefix: str = ""):
        yield prefix, self
        for name, child in self._modules.items():
            yield from child.named_modules(f"{prefix}.{name}" if prefix else name)

    def modules(self):
        return [m for _, m in self.named_modules()]

    def named_buffers(self, prefix: str = ""):
        for name, mod in self.named_modules(prefix):
            for bname, buf in mod._buffers.items():
                if buf is not None:
                    yield (f"{name}.{bname}" if name else bname), buf

    def parameters(self):
        return [b for _, b in self.named_buffers()]

    # -- state
    def state_dict(self) -> "OrderedDict[str, Tensor]":
        return OrderedDict(self.named_buffers())

    def load_state_dict(self, state, strict: bool = True) -> None:
        own = dict(self.named_buffers())
        missing = [k for k in own if k not in state]
        unexpected = [k for k in state if k not in own]
        if strict and (missing or unexpected):
            raise KeyError(f"state_dict mismatch: missing {missing}, unexpected {unexpected}")
        for name, mod in self.named_modules():
            for bname in list(mod._buffers):
                key = f"{name}.{bname}" if name else bname
                if key in state:
                    old, new = mod._buffers[bname], state[key]
                    # a checkpoint holds host tensors: keep each buffer on the device it lives on
                    if old is not None and isinstance(new, Tensor) and new.device != old.device:
                        new = new.to(old.device)
                    mod._buffers[bname] = new
                    mod._state_loaded(bname)

    def _state_loaded(self, name: str) -> None:
        """Called after a buffer was replaced by ``load_state_dict``."""

    def eval(self) -> "Module":
        return self.train(False)

    def train(self, mode: bool = True) -> "Module":
        for m in self.modules():
            object.__setattr__(m, "training", bool(mode))
        return self

    def to(self, device) -> "Module":
        for m in self.modules():
            for k, b in list(m._buffers.items()):
                if b is not None:
                    m._buffers[k] = b.to(device)
                    m._state_loaded(k)
        return self

    # -- call
    def forward(self, *args, **kwargs):
        raise NotImplementedError

    def __call__(self, *args, **kwargs):
        out = self.forward(*args, **kwargs)
        for hook in self._forward_hooks:
            hook(self, args, out)
        return out

    def extra_repr(self) -> str:
        return ""

    def __repr__(self) -> str:
        lines = [f"{type(self).__name__}({self.extra_repr()}"]
        for name, child in self._modules.items():
            child_repr = repr(child).replace("\n", "\n  ")
            lines.append(f"  ({name}): {child_repr}")
        return (lines[0] + ")") if len(lines) == 1 else "\n".join(lines) + "\n)"
