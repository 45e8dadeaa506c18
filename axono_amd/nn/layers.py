"""Layers on the decode path: Linear, RMSNorm, Embedding (axono/python/axono/nn/layers.py)."""
from __future__ import annotations

import numpy as np

from .. import libaxono as _l
from ..core.tensor import Tensor, get_default_device
from ..core.types import DataType
from .module import Module


class Linear(Module):
    """y = x @ W^T + b.  Weights are created FLOAT32 like the reference's and forward then runs the plain fp32
    operator; after `cast_linear_fp16()` (on the layer or any parent) it runs the fp16-weight kernels of the
    decode path over a packed copy of the weight."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device: str | None = None):
        super().__init__()
        device = device or get_default_device()
        self._init_args = {"in_features": in_features, "out_features": out_features, "bias": bias,
                           "device": device}
        self.in_features = in_features
        self.out_features = out_features
        self.device = device
        scale = np.sqrt(2.0 / in_features)
        w = np.random.normal(0.0, scale, size=(out_features, in_features)).astype(np.float32)
        self.add_weight("weight", Tensor.from_numpy_ref(w).to(device))
        if bias:
            self.add_weight("bias", Tensor.from_numpy_ref(np.zeros(out_features, np.float32)).to(device))
        else:
            self._parameters["bias"] = None

    def forward(self, x: Tensor) -> Tensor:
        w = self._parameters["weight"]
        b = self._parameters["bias"]
        if w.is_hip and w.dtype == DataType.FLOAT16 and x.num_elements:
            # The kernels read a packed copy of the weight.  It is made on first use and again whenever
            # the weight's storage was replaced or written since (load_state_dict, copy_from,
            # copy_from_numpy and fill* write in place and bump the storage's version), so forward
            # always multiplies by the live weight, as the reference's Linear does (nn/layers.py:72-80).
            key = (w._st, w._st.version)
            held = self.__dict__.get("_packed_key")
            packed = self.__dict__.get("_packed")
            if packed is None or held is None or held[0] is not key[0] or held[1] != key[1]:
                packed = _l.pack_linear_weight(w)
                object.__setattr__(self, "_packed", packed)
                object.__setattr__(self, "_packed_key", key)
            return _l.linear_packed(x, packed, self.out_features, b)
        return _l.linear(x, w, b) if b is not None else _l.linear_nobias(x, w)


class RMSNorm(Module):
    def __init__(self, normalized_shape: int, eps: float = 1e-6, device: str | None = None):
        super().__init__()
        device = device or get_default_device()
        self._init_args = {"normalized_shape": normalized_shape, "eps": eps}
        self.normalized_shape = normalized_shape
        self.eps = eps
        self.add_weight("weight", Tensor.ones((normalized_shape,), device=device))

    def forward(self, x: Tensor) -> Tensor:
        return _l.rms_norm(x, self._parameters["weight"], self.eps)


class Embedding(Module):
    def __init__(self, num_embeddings: int, embedding_dim: int, device: str | None = None):
        super().__init__()
        device = device or get_default_device()
        self._init_args = {"num_embeddings": num_embeddings, "embedding_dim": embedding_dim}
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        self.add_weight("weight", Tensor.randn((num_embeddings, embedding_dim), device=device))

    def forward(self, ids: Tensor) -> Tensor:
        return _l.embedding(ids, self._parameters["weight"])
