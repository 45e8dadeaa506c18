"""hipGraph capture for the Python surface: the reference's `CUDAGraph` / `cuda_graph`
(axono/python/axono/core/cuda_graph.py:54-190) on HIP.  Same life cycle: capture (warm-up run, then
the recorded run) -> replay any number of times -> reset.  Constraints are the reference's: host
<-> device copies and synchronisation stay outside the captured body; inputs are refreshed in
place (copy_from / copy_from_numpy) because the graph reads fixed addresses.
"""
from __future__ import annotations

from .. import libaxono as _l


class HIPGraph:
    def __init__(self) -> None:
        if not _l.hip_available():
            raise RuntimeError("HIP Graph 需要可用的 HIP 设备")
        self._impl = _l.HIPGraph()
        self._outputs = []
        self._output = None

    def capture(self, fn) -> "HIPGraph":
        holder = {}

        def _body():
            holder["out"] = fn()

        self._impl.capture(_body)
        self._set_outputs(holder.get("out"))
        return self

    def _set_outputs(self, value) -> None:
        self._outputs = list(value) if isinstance(value, (tuple, list)) else [value]
        self._output = self._outputs[0] if self._outputs else None

    def replay(self) -> "HIPGraph":
        """Launches the graph and waits for it (the reference's replay is launch + stream sync,
        src/core/cuda/graph.cu:123-139)."""
        self._impl.replay()
        return self

    def launch(self) -> "HIPGraph":
        """Enqueues one replay without waiting."""
        self._impl.launch()
        return self

    def launch_async(self) -> "HIPGraph":
        """Enqueues one replay on the graph's own stream only; see libaxono.HIPGraph.launch_async."""
        self._impl.launch_async()
        return self

    @property
    def output(self):
        return self._output

    @output.setter
    def output(self, value):
        self._set_outputs(value)

    @property
    def outputs(self):
        return list(self._outputs)

    @outputs.setter
    def outputs(self, values):
        self._set_outputs(values)

    def sync(self) -> "HIPGraph":
        self._impl.sync()
        return self

    def reset(self) -> None:
        """Releases the graph and the blocks its kernels write to; earlier outputs become invalid."""
        self._impl.reset()
        self._outputs, self._output = [], None

    @property
    def is_captured(self) -> bool:
        return self._impl.is_captured

    @property
    def num_nodes(self) -> int:
        return self._impl.num_nodes


class hip_graph:  # noqa: N801 - context manager, lower case like the reference's cuda_graph
    """`with hip_graph() as g: ...` captures the block as it runs (no warm-up, no second run)."""

    def __init__(self) -> None:
        if not _l.hip_available():
            raise RuntimeError("HIP Graph 需要可用的 HIP 设备")
        self.graph = HIPGraph()
        self._stream = None

    def __enter__(self) -> HIPGraph:
        self._stream = _l._graph_begin_capture()
        return self.graph

    def __exit__(self, exc_type, exc, tb) -> bool:
        if exc_type is not None:
            _l._graph_abort_capture(self._stream)
            return False
        _l._graph_end_capture(self._stream, self.graph._impl)
        return False


# the reference's names, so code written against it keeps working
CUDAGraph = HIPGraph
cuda_graph = hip_graph
