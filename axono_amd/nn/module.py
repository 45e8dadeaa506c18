"""nn.Module: parameter / submodule registry with the reference's semantics
(axono/python/axono/nn/module.py): attribute assignment registers submodules (also lists of them,
as `name.i`) and Tensor parameters; `parameters()` / `state_dict()` give flat dotted names;
`load_state_dict` copies in place; `cast_linear_fp16()` turns every Linear's weight and bias into
resident FLOAT16 tensors."""
from __future__ import annotations

import numpy as np

from ..core.tensor import Tensor
from ..core.types import DataType


class Module:
    def __init__(self):
        self._parameters: dict = {}
        self._submodules: dict = {}
        self._is_training = True
        self._name = self.__class__.__name__

    def add_submodule(self, name: str, module: "Module") -> "Module":
        if not isinstance(module, Module):
            raise TypeError(f"add_submodule 需要 Module, 得到 {type(module)}")
        self._submodules[name] = module
        return module

    def __setattr__(self, name: str, value):
        if name.startswith("_") or name in ("training",):
            object.__setattr__(self, name, value)
            return
        submods = self.__dict__.get("_submodules")
        if submods is not None:
            if isinstance(value, Module):
                submods[name] = value
            elif isinstance(value, (list, tuple)) and value and all(isinstance(v, Module) for v in value):
                for i, v in enumerate(value):
                    submods[f"{name}.{i}"] = v
            elif isinstance(value, Tensor):
                params = self.__dict__.get("_parameters")
                if params is not None:
                    params[name] = value
        object.__setattr__(self, name, value)

    def add_weight(self, name: str, tensor: Tensor) -> None:
        if not isinstance(tensor, Tensor):
            raise TypeError(f"add_weight 需要 axono.Tensor, 得到 {type(tensor)}")
        self._parameters[name] = tensor

    def parameters(self) -> dict:
        out = dict(self._parameters)
        for sub_name, sub in self._submodules.items():
            for pname, pt in sub.parameters().items():
                out[f"{sub_name}.{pname}"] = pt
        return out

    def weights(self):
        ws = [t for t in self._parameters.values() if t is not None]
        for sub in self._submodules.values():
            ws.extend(sub.weights())
        return ws

    @property
    def weight(self) -> Tensor:
        return self._parameters["weight"]

    @property
    def bias(self):
        return self._parameters["bias"]

    def state_dict(self) -> dict:
        return dict(self.parameters())

    def load_state_dict(self, sd: dict, strict: bool = True) -> None:
        """{flat name: Tensor | ndarray} -> in-place copies that keep each parameter's device.
        ndarrays are converted to the parameter's dtype (FLOAT32 or FLOAT16)."""
        missing = []
        for name, t in self.parameters().items():
            if t is None:
                continue
            if name not in sd:
                missing.append(name)
                continue
            v = sd[name]
            if isinstance(v, Tensor):
                t.copy_from(v)
                continue
            want = np.float16 if t.dtype == DataType.FLOAT16 else np.float32
            t.copy_from_numpy(np.ascontiguousarray(v, dtype=want).reshape(t.shape))
        if strict and missing:
            raise KeyError(f"state_dict 缺少参数: {missing}")

    def cast_linear_fp16(self) -> None:
        """Every Linear in this module tree: weight / bias -> FLOAT16 (round-to-nearest-even), in
        place in the registry (axono/python/axono/nn/module.py:158-184)."""
        from .layers import Linear

        stack = [self]
        while stack:
            m = stack.pop()
            stack.extend(m._submodules.values())
            if not isinstance(m, Linear):
                continue
            for pname, t in list(m._parameters.items()):
                if t is None or t.dtype == DataType.FLOAT16:
                    continue
                m._parameters[pname] = t.cast_to(DataType.FLOAT16)

    def train(self, mode: bool = True) -> "Module":
        self._is_training = mode
        return self

    def eval(self) -> "Module":
        return self.train(False)

    def forward(self, *args, **kwargs):
        raise NotImplementedError("Module 子类需实现 forward()")

    def __call__(self, *args, **kwargs):
        return self.forward(*args, **kwargs)

    def __repr__(self) -> str:
        init_args = [f"{k}={v}" for k, v in getattr(self, "_init_args", {}).items()]
        return f"{self.__class__.__name__}({', '.join(init_args)})"
