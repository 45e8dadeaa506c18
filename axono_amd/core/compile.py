"""`compile(model)`: capture the model's forward into a hipGraph keyed by the call signature and
replay it afterwards.  Mirrors axono/python/axono/core/compile.py:52-174 (mode "normal"): the first
call with a new signature runs the model once eagerly (warm-up), captures it with the inputs of
that call as static buffers, and every call refreshes those buffers in place and replays.
Outputs are the captured call's tensors and are overwritten by the next replay.
"""
from __future__ import annotations

from .. import libaxono as _l
from .hip_graph import HIPGraph


class _TensorArg:
    __slots__ = ("tensor",)

    def __init__(self, tensor):
        self.tensor = tensor

    def copy_in(self, value):
        if value is not self.tensor:
            self.tensor.copy_from(value)


def _is_tensor(a):
    return hasattr(a, "shape") and hasattr(a, "dtype")


def _sig_of(args, kwargs):
    parts = []
    for a in args:
        parts.append(("T", tuple(a.shape), str(a.dtype), str(a.device)) if _is_tensor(a) else ("S", repr(a)))
    for k in sorted(kwargs):
        v = kwargs[k]
        parts.append((k, "T", tuple(v.shape), str(v.dtype), str(v.device)) if _is_tensor(v) else (k, "S", repr(v)))
    return tuple(parts)


class CompiledModel:
    def __init__(self, model, mode: str = "normal"):
        if mode != "normal":
            raise ValueError(f"axono.compile: 暂不支持 mode={mode!r} (目前只有 'normal')")
        if not _l.hip_available():
            raise RuntimeError("axono.compile 需要可用的 HIP 设备")
        self._model = model
        self._mode = mode
        self._graphs = {}

    def __getattr__(self, name):
        return getattr(object.__getattribute__(self, "_model"), name)

    def __setattr__(self, name, value):
        if name.startswith("_"):
            object.__setattr__(self, name, value)
        else:
            setattr(object.__getattribute__(self, "_model"), name, value)

    def _build(self, args, kwargs):
        static_args = [_TensorArg(a) if _is_tensor(a) else a for a in args]
        static_kwargs = {k: (_TensorArg(v) if _is_tensor(v) else v) for k, v in kwargs.items()}
        g = HIPGraph()
        g.capture(lambda: self._model(
            *[s.tensor if isinstance(s, _TensorArg) else s for s in static_args],
            **{k: (s.tensor if isinstance(s, _TensorArg) else s) for k, s in static_kwargs.items()}))
        return g, static_args, static_kwargs

    def __call__(self, *args, **kwargs):
        sig = _sig_of(args, kwargs)
        entry = self._graphs.get(sig)
        if entry is None:
            self._model(*args, **kwargs)  # warm-up on the real inputs
            entry = self._build(args, kwargs)
            self._graphs[sig] = entry
        g, static_args, static_kwargs = entry
        for s, a in zip(static_args, args):
            if isinstance(s, _TensorArg):
                s.copy_in(a)
        for k, s in static_kwargs.items():
            if isinstance(s, _TensorArg):
                s.copy_in(kwargs[k])
        g.replay()
        outs = g.outputs
        return outs[0] if len(outs) == 1 else tuple(outs)

    def forward(self, *args, **kwargs):
        return self(*args, **kwargs)

    def __repr__(self):
        inner = repr(object.__getattribute__(self, "_model"))
        return f"CompiledModel(mode={self._mode!r}, graphs={len(self._graphs)}, model={inner})"


def compile(model, mode: str = "normal"):  # noqa: A001 - the reference's name
    return CompiledModel(model, mode=mode)
