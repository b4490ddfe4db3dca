"""Two mixers as branches of one input: each branch's output is RMS-normed over the model
width with a weight of its own, and the mean of the two joins the residual rows:
    x += 1/2 (rms(left(h)) w_left + rms(right(h)) w_right)
One branch may ask for keys and values, the other for state; the layer call's cache entry and
state entry serve them."""
from __future__ import annotations

import torch

from ..weights import TensorSpec
from .base import Mixer, Runtime
from .calls import NormedSumArgs, emit_library_call


class ParallelMixer(Mixer):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, left: Mixer, right: Mixer, left_norm: str, right_norm: str, hidden_size: int, eps: float):
        self.left, self.right, self.D, self.eps = left, right, hidden_size, float(eps)
        self.names = (left_norm, right_norm)
        self.w_left = self.w_right = None
        lk, ls = left.cache_requests()
        rk, rs = right.cache_requests()
        if (lk is not None and rk is not None) or (ls is not None and rs is not None):
            raise ValueError("two branches that both keep keys and values, or both keep state, need a cache entry each")
        self._requests = (lk or rk, ls or rs)

    def children(self):
        return [self.left, self.right]

    def tensor_specs(self):
        return [TensorSpec(n, (self.D,), init="ones") for n in self.names]

    def load(self, fetch, runtime: Runtime) -> None:
        self.w_left, self.w_right = (fetch.get(n).to(torch.float32).contiguous() for n in self.names)

    def cache_requests(self):
        return self._requests

    def prepare(self, runtime: Runtime, max_positions: int) -> None:
        self.left.prepare(runtime, max_positions)
        self.right.prepare(runtime, max_positions)

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0) -> None:
        a = b.buffer("branch.left", self.D, torch.float32)
        c = b.buffer("branch.right", self.D, torch.float32)
        self.left.emit(b, src, a, accumulate=False)
        self.right.emit(b, src, c, accumulate=False)
        emit_library_call(b, "normed_sum", NormedSumArgs(b._ptr(self.w_left), b._ptr(self.w_right), self.D, self.eps, 0.5), x, inp=a,
                          extra=[c])
