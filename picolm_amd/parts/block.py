"""Arrangements of norm, mixer and feed-forward in a layer.  PreNormBlock is picolm's
(picolm/model_core.c:1841, :2151, :2160, :2204): x += mixer(norm(x)); x += ffn(norm(x));
a block without a feed-forward skips the second half, as picolm does when the three
matrices are absent (:2159)."""
from __future__ import annotations

from .base import Block, FeedForward, Mixer, Norm


def norm_ref_of(norm):
    """The norm as the product before it may prepare it, or None for a norm of another kind."""
    f = getattr(norm, "norm_ref", None)
    return f() if f is not None else None


class PreNormBlock(Block):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm | None, ffn: FeedForward | None):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def children(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def first_norm(self):
        """The norm this block applies to the residual stream on entry: the block before may
        have it prepared."""
        return self.mixer_norm

    def emit(self, b, x: int, after=None, after_when: int = 0) -> None:
        """x += mixer(norm(x)); x += ffn(norm(x)) over the residual rows in buffer `x`, as operations
        of a launch program.  `after`: the RMSNorm that meets x after this block (after_when = 1: only
        in steps that want every row's logits), so that the block's last product can prepare it.
        Every part emits what it is: the engine's operations, or a call of its `forward`."""
        if type(self).forward is not Block.forward and type(self).emit is PreNormBlock.emit:
            return Block.emit(self, b, x, after, after_when)       # a subclass with an arrangement of its own
        src = self.mixer_norm.emit(b, x)
        if self.ffn is None:
            self.mixer.emit(b, src, x, after, after_when)
            return
        self.mixer.emit(b, src, x, norm_ref_of(self.ffn_norm), 0)
        self.ffn.emit(b, self.ffn_norm.emit(b, x), x, after, after_when)


class _NoMixer(Mixer):
    """The mixer of a block that has none: it asks nothing of the cache."""


class LoopEntry(Block):
    """What runs before pass `number` over a looped stretch of layers:
    x <- W_in [x ; x0] + step[number], with x0 the embedding's output (which the embedding keeps,
    `TokenEmbedding(keeps_output=True)`), W_in [D, 2 D] and step [passes, D].  The passes of one
    loop share the two tensors; each pass is a part of its own because its vector differs."""
    graph_safe = True      # launches depend on device memory only

    def __init__(self, w_in, step_name: str, hidden_size: int, passes: int, number: int):
        """`w_in`: the `Linear` [D, 2 D] that the passes share."""
        if not 0 <= number < passes:
            raise ValueError(f"pass {number} of {passes}")
        self.D, self.passes, self.number = hidden_size, passes, number
        self.step_name = step_name
        self.w_in = w_in
        self.mixer = _NoMixer()
        self.step = None

    def children(self):
        return [self.w_in]

    def tensor_specs(self):
        from ..weights import TensorSpec
        return [TensorSpec(self.step_name, (self.passes, self.D))]

    def load(self, fetch, runtime) -> None:
        import torch
        self.step = fetch.get(self.step_name).to(torch.float32).contiguous()

    def emit(self, b, x: int, after=None, after_when: int = 0) -> None:
        import torch
        from .. import kernels
        from .calls import LoopInputArgs, emit_library_call
        if self.step is None:
            raise ValueError(f"loop entry {self.step_name} has no weights loaded")
        first = b.buffer("embed.out", self.D, torch.float32)
        joined = b.buffer("loop.joined", 2 * self.D, b.dtype)
        row = self.step[self.number]
        emit_library_call(b, "loop_input", LoopInputArgs(b._ptr(row), self.D), x, inp=first, extra=[joined])
        self.w_in.emit(b, joined, x, kernels.EPI_ACCUMULATE, out_norm=after, out_norm_when=after_when)
