"""nn.Module for the hip device: a registry of parameters and child modules behind the method names
of the reference's class (axono/python/axono/nn/module.py).

What callers rely on: assigning a Module, a non-empty list / tuple of Modules, or a Tensor to an
attribute registers it (list items as `name.<index>`); `parameters()` / `state_dict()` return one flat
dict with dotted names; `load_state_dict` copies into the existing tensors, so device and dtype stay;
`cast_linear_fp16()` replaces the weight and bias of every Linear in the tree by FLOAT16 copies
(nn/module.py:158-184 of the reference)."""
from __future__ import annotations

from typing import Iterator

import numpy as np

from ..core.tensor import Tensor
from ..core.types import DataType

_NUMPY_OF = {DataType.FLOAT16: np.float16, DataType.FLOAT32: np.float32}


class Module:
    def __init__(self):
        self._parameters: dict = {}
        self._submodules: dict = {}
        self._is_training = True
        self._name = type(self).__name__

    # ---- registration ------------------------------------------------------------------------
    def _register(self, name: str, value) -> None:
        children = self.__dict__.get("_submodules")
        if children is None:  # attribute set before Module.__init__ ran
            return
        if isinstance(value, Module):
            children[name] = value
        elif isinstance(value, Tensor):
            self.__dict__["_parameters"][name] = value
        elif isinstance(value, (list, tuple)) and len(value) and all(isinstance(v, Module) for v in value):
            children.update({f"{name}.{i}": v for i, v in enumerate(value)})

    def __setattr__(self, name: str, value):
        if not name.startswith("_") and name != "training":
            self._register(name, value)
        object.__setattr__(self, name, value)

    def add_submodule(self, name: str, module: "Module") -> "Module":
        if not isinstance(module, Module):
            raise TypeError(f"add_submodule: expected a Module, got {type(module).__name__}")
        self._submodules[name] = module
        return module

    def add_weight(self, name: str, tensor: Tensor) -> None:
        if not isinstance(tensor, Tensor):
            raise TypeError(f"add_weight: expected a Tensor, got {type(tensor).__name__}")
        self._parameters[name] = tensor

    # ---- traversal ---------------------------------------------------------------------------
    def _walk(self, prefix: str = "") -> Iterator[tuple]:
        """(dotted prefix, module) for this module and everything below it, parents first."""
        yield prefix, self
        for child_name, child in self._submodules.items():
            yield from child._walk(f"{prefix}{child_name}.")

    def parameters(self) -> dict:
        return {prefix + pname: t for prefix, mod in self._walk() for pname, t in mod._parameters.items()}

    def weights(self) -> list:
        return [t for t in self.parameters().values() if t is not None]

    def state_dict(self) -> dict:
        return self.parameters()

    @property
    def weight(self) -> Tensor:
        return self._parameters["weight"]

    @property
    def bias(self):
        return self._parameters["bias"]

    # ---- loading and casting -----------------------------------------------------------------
    def load_state_dict(self, sd: dict, strict: bool = True) -> None:
        """`sd` maps flat names to Tensors or ndarrays.  Values are copied into the registered tensors;
        ndarrays are converted to the parameter's dtype first.  strict: a registered parameter without
        an entry raises KeyError (entries without a parameter are ignored)."""
        absent = []
        for name, dst in self.parameters().items():
            if dst is None:
                continue
            src = sd.get(name)
            if src is None:
                absent.append(name)
            elif isinstance(src, Tensor):
                dst.copy_from(src)
            else:
                host = np.ascontiguousarray(src, dtype=_NUMPY_OF.get(dst.dtype, np.float32))
                dst.copy_from_numpy(host.reshape(dst.shape))
        if strict and absent:
            raise KeyError(f"load_state_dict: no entry for {absent}")

    def cast_linear_fp16(self) -> None:
        from .layers import Linear

        for _, mod in self._walk():
            if isinstance(mod, Linear):
                for pname, t in mod._parameters.items():
                    if t is not None and t.dtype != DataType.FLOAT16:
                        mod._parameters[pname] = t.cast_to(DataType.FLOAT16)

    # ---- calling -----------------------------------------------------------------------------
    def train(self, mode: bool = True) -> "Module":
        self._is_training = bool(mode)
        return self

    def eval(self) -> "Module":
        return self.train(False)

    def forward(self, *args, **kwargs):
        raise NotImplementedError(f"{type(self).__name__} does not define forward()")

    def __call__(self, *args, **kwargs):
        return self.forward(*args, **kwargs)

    def __repr__(self) -> str:
        shown = ", ".join(f"{k}={v}" for k, v in getattr(self, "_init_args", {}).items())
        return f"{type(self).__name__}({shown})"
