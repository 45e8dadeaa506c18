"""`compile(model)`: the model's forward as a replayed hipGraph.

Behaviour follows axono/python/axono/core/compile.py:52-174 (mode "normal"): calls are told apart
by the shapes, dtypes and devices of their tensor arguments and the values of the others; the first
call of a kind runs the model once as it is, then captures it with that call's tensors as the
graph's fixed input buffers; every call of that kind copies its tensors into those buffers (unless
they are the buffers) and replays.  The results are the captured call's output tensors: the next
replay overwrites them.
"""
from __future__ import annotations

from .. import libaxono as _table
from .hip_graph import HIPGraph


def _tensor_like(value) -> bool:
    return hasattr(value, "shape") and hasattr(value, "dtype")


def _describe(value):
    """What distinguishes one call from another: a tensor's geometry, anything else by its repr."""
    if _tensor_like(value):
        return "tensor", tuple(value.shape), str(value.dtype), str(value.device)
    return "value", repr(value)


def _call_key(args, kwargs) -> tuple:
    return tuple(_describe(a) for a in args) + tuple((name,) + _describe(kwargs[name]) for name in sorted(kwargs))


class _CapturedCall:
    """The graph of one kind of call and the tensors it reads its inputs from."""

    def __init__(self, model, args, kwargs):
        self.positional = list(args)
        self.named = dict(kwargs)
        self.graph = HIPGraph()
        self.graph.capture(lambda: model(*self.positional, **self.named))

    def run(self, args, kwargs):
        for fixed, given in zip(self.positional, args):
            if _tensor_like(fixed) and given is not fixed:
                fixed.copy_from(given)
        for name, fixed in self.named.items():
            if _tensor_like(fixed) and kwargs[name] is not fixed:
                fixed.copy_from(kwargs[name])
        self.graph.replay()
        results = self.graph.outputs
        return results[0] if len(results) == 1 else tuple(results)


class CompiledModel:
    def __init__(self, model, mode: str = "normal"):
        if mode != "normal":
            raise ValueError(f"axono.compile: mode {mode!r} is not supported (only 'normal')")
        if not _table.hip_available():
            raise RuntimeError("axono.compile needs a HIP device")
        self._model = model
        self._mode = mode
        self._graphs = {}  # call key -> _CapturedCall

    # everything that is not the wrapper's own state is the model's
    def __getattr__(self, name):
        return getattr(object.__getattribute__(self, "_model"), name)

    def __setattr__(self, name, value):
        if name.startswith("_"):
            object.__setattr__(self, name, value)
        else:
            setattr(object.__getattribute__(self, "_model"), name, value)

    def __call__(self, *args, **kwargs):
        key = _call_key(args, kwargs)
        captured = self._graphs.get(key)
        if captured is None:
            self._model(*args, **kwargs)  # once as it is: lazy initialisation happens outside the capture
            captured = self._graphs[key] = _CapturedCall(self._model, args, kwargs)
        return captured.run(args, kwargs)

    def forward(self, *args, **kwargs):
        return self(*args, **kwargs)

    def __repr__(self):
        return f"CompiledModel(mode={self._mode!r}, graphs={len(self._graphs)}, model={self._model!r})"


def compile(model, mode: str = "normal"):  # noqa: A001 - the reference's name
    return CompiledModel(model, mode=mode)
