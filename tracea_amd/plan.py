"""Execution plans: a fused operator graph compiled by ``tracea_plan_compile`` into
launches over one arena, run from Python on torch tensors.

Counterpart of the reference's GraphCompiler / ExecutionPlan / executor chain
(src/runtime/compiler.rs:100-156, src/runtime/plan.rs:10-53) for the operators
of the dense-contraction path.  The arena is one torch byte tensor; a plan can
be captured into a HIP graph (``capture``) and replayed without any host work
per launch.
"""
import ctypes as C
import json

import torch

from . import capi

_DT = {torch.float16: capi.F16, torch.bfloat16: capi.BF16}
_TENSOR_DT = {torch.float16: capi.F16, torch.bfloat16: capi.BF16, torch.float32: capi.F32}


class Plan:
    def __init__(self, graph, dtype=torch.float16, device="cuda:0"):
        """``graph``: GraphTopology dict (see tracea_amd.graph), normally already fused."""
        if dtype not in _DT:
            raise TypeError("plan dtype must be torch.float16 or torch.bfloat16")
        self.dtype = dtype
        self._h = capi.lib().tracea_plan_compile(json.dumps(graph).encode(), _DT[dtype])
        if not self._h:
            raise ValueError(capi.last_error())
        self.device = torch.device(device)
        self._keep = {}
        self._arena = None
        self._graph = None

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            try:
                capi.lib().tracea_plan_destroy(h)
            except Exception:  # interpreter shutdown: the module globals are already gone
                pass

    @property
    def arena_size(self):
        return int(capi.lib().tracea_plan_arena_size(self._h))

    def describe(self):
        return json.loads(capi.take_string(capi.lib().tracea_plan_describe(self._h)))

    def bind(self, op_id, tensor, slot="input"):
        """Attach device memory: an Input node's tensor, or a contraction's weights
        (slot "weight", "weight_rsck", "weight_t").  The tensor is kept alive by the plan."""
        if not tensor.is_cuda or not tensor.is_contiguous():
            raise ValueError("plan tensors must be contiguous device tensors")
        # with its extent and element type: a tensor that is too small or of another type than the plan
        # reads is refused here instead of being read out of bounds by a later run
        capi.check("tracea_plan_bind", capi.lib().tracea_plan_bind_sized(
            self._h, op_id, slot.encode(), tensor.data_ptr(), tensor.numel() * tensor.element_size(),
            _TENSOR_DT.get(tensor.dtype, -1)))
        self._keep[(op_id, slot)] = tensor
        return self

    def arena(self):
        if self._arena is None:
            # 256-byte alignment: torch's allocator hands out 512-byte aligned blocks
            self._arena = torch.empty(max(self.arena_size, 256), dtype=torch.uint8, device=self.device)
            assert self._arena.data_ptr() % 256 == 0
        return self._arena

    def run(self, stream=None):
        """Launches every step on ``stream`` (default: torch's current stream)."""
        s = stream if stream is not None else torch.cuda.current_stream(self.device)
        st = capi.lib().tracea_plan_run(self._h, self.arena().data_ptr(), self.device.index or 0,
                                        C.c_void_p(s.cuda_stream))
        capi.check("tracea_plan_run", st)
        return self

    def output(self, op_id, shape=None):
        """View of a node's result inside the arena (valid until a later run overwrites it; the
        bytes of an intermediate are reused after its last consumer)."""
        off, size = C.c_size_t(), C.c_size_t()
        capi.check("tracea_plan_output", capi.lib().tracea_plan_output(self._h, op_id, C.byref(off), C.byref(size)))
        t = self.arena()[off.value:off.value + size.value].view(self.dtype)
        return t.view(*shape) if shape is not None else t

    def capture(self):
        """Records one run into a HIP graph; ``replay()`` then re-issues it.  Everything a run
        touches (arena, bound tensors) must stay where it is."""
        # First-use work happens outside the capture and on the capture's own stream: kernel
        # attributes, and the split-K scratch buffer, which the library keeps per stream and
        # never allocates while a stream is being captured.
        side = torch.cuda.Stream(self.device)
        side.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(side):
            self.run()
        torch.cuda.synchronize(self.device)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            self.run()
        self._graph = g
        return self

    def replay(self):
        if self._graph is None:
            raise RuntimeError("capture() first")
        self._graph.replay()
        return self
