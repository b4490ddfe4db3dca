"""Causal softmax attention without rotation whose scores get a learned bias by distance and
whose denominator holds one more term per head, a sink; queries and keys are RMS-normed per head,
values may have a size of their own, and the heads are gated before the output projection.

    q, k, v, g = W h;  q <- rms(q) w_q,  k <- rms(k) w_k               per head, over the head's size
    s_ij = scale (q_i . k_j) + rel[bucket(i - j)][head]                j <= i
    p_ij = exp(s_ij) / (exp(sink_head) + sum_j' exp(s_ij'))            the sink is a term of the denominator only
    out  = W_o (concat_heads(sum_j p_ij v_j) * sigmoid(g))

The bias table has B rows: one per distance below B/2, then rows spaced evenly in the logarithm of
the distance up to `bias_max`, the last row for everything beyond.  It is expanded once, at load,
into one entry per distance up to `bias_max` and per head; the attention kernels index that by
min(distance, last).
"""
from __future__ import annotations

import math

import torch

from .. import kernels
from ..weights import TensorSpec
from .base import KVRequest, Mixer, Runtime
from .calls import SinkAttentionArgs, emit_library_call
from .linear import Linear


def distance_rows(n_rows: int, bias_max: float) -> list[int]:
    """For every distance 0 .. ceil(bias_max) the row of a table of `n_rows` that holds its bias."""
    half = n_rows // 2
    last = int(math.ceil(bias_max))
    if n_rows > 1 and not bias_max > half:
        raise ValueError(f"a bias table of {n_rows} rows needs bias_max above {half}, got {bias_max}")
    rows = []
    for n in range(last + 1):
        if n < half or n_rows == 1:
            rows.append(min(n, n_rows - 1))
        else:
            steps = math.log(n / half) / math.log(bias_max / half) * (n_rows - half)
            rows.append(min(n_rows - 1, half + int(math.floor(steps))))
    return rows


class SinkAttention(Mixer):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int, v_head_dim: int,
                 scale: float, eps: float, bias_rows: int | None = None, bias_max: float = 0.0, has_bias: bool = False,
                 qk_norm: bool = True, sink: bool = True, gate: bool = True):
        """`has_bias`: scores get the bias by distance, from a table of `bias_rows` rows (None: as many
        as the checkpoint's tensor has) that reaches to `bias_max`."""
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} heads do not split over {n_kv_heads} KV heads")
        self.prefix, self.D = prefix, hidden_size
        self.H, self.G, self.d, self.dv = n_heads, n_kv_heads, head_dim, v_head_dim
        self.scale, self.eps = float(scale), float(eps)
        self.has_bias = bool(has_bias or bias_rows)
        self.bias_rows, self.bias_max = (None if bias_rows is None else int(bias_rows)), float(bias_max)
        if self.has_bias and not self.bias_max > 0:
            raise ValueError("a bias by distance needs bias_max, the distance its last row starts at")
        self.qk_norm, self.has_sink, self.has_gate = qk_norm, sink, gate
        names = [prefix + "q", prefix + "k", prefix + "v"] + ([prefix + "g"] if gate else [])
        sizes = [n_heads * head_dim, n_kv_heads * head_dim, n_kv_heads * v_head_dim] + ([n_heads * v_head_dim] if gate else [])
        self.proj = Linear(names, sizes, hidden_size)
        self.o = Linear([prefix + "o"], [hidden_size], n_heads * v_head_dim)
        self.q_norm = self.k_norm = self.bias = self.sink = None

    def children(self):
        return [self.proj, self.o]

    def tensor_specs(self):
        specs = []
        if self.qk_norm:
            specs += [TensorSpec(self.prefix + "q.norm", (self.d,), init="ones"), TensorSpec(self.prefix + "k.norm", (self.d,), init="ones")]
        if self.has_bias:       # (-1: any number of rows; random weights need the number)
            specs.append(TensorSpec(self.prefix + "rel", (self.bias_rows if self.bias_rows is not None else -1, self.H)))
        if self.has_sink:
            specs.append(TensorSpec(self.prefix + "sink", (self.H,)))
        return specs

    def load(self, fetch, runtime: Runtime) -> None:
        f32 = lambda name: fetch.get(self.prefix + name).to(torch.float32).contiguous()
        if self.qk_norm:
            self.q_norm, self.k_norm = f32("q.norm"), f32("k.norm")
        if self.has_bias:
            rel = f32("rel")
            rows = distance_rows(rel.shape[0], self.bias_max)
            self.bias = rel[torch.tensor(rows, device=rel.device)].t().contiguous()   # [H, distances]
        if self.has_sink:
            self.sink = f32("sink")

    def cache_requests(self):
        return KVRequest(self.G, self.d, 0, self.dv), None

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0, accumulate: bool = True) -> None:
        """x (+)= o(gate * attention) for the rows h of `src`, as operations of a launch program."""
        H, G, d, dv = self.H, self.G, self.d, self.dv
        width = self.proj.out_size
        rows = b.buffer("sink_attn.in", width, torch.float32)
        self.proj.emit(b, src, rows, kernels.EPI_STORE)
        q = b.buffer("sink_attn.q", H * d, b.dtype)
        out = b.buffer("sink_attn.out", H * dv, b.dtype)
        q_off, k_off, v_off = 0, H * d, H * d + G * d
        args = SinkAttentionArgs(H, G, d, dv, width, q_off, k_off, v_off, v_off + G * dv if self.has_gate else -1, self.scale, self.eps,
                                 b._ptr(self.q_norm), b._ptr(self.k_norm), b._ptr(self.bias),
                                 0 if self.bias is None else self.bias.shape[1], b._ptr(self.sink))
        lib = kernels.lib()
        on_matrix_cores = b.dtype == torch.bfloat16 and lib.picolm_attn_plain_mfma_takes(d, dv)
        emit_library_call(b, "sink_attention", args, out, inp=rows, extra=[q], uses_kv=True, attends=True,
                          tile_rows=lib.picolm_attn_plain_mfma_tile_rows() if on_matrix_cores else kernels.attn_prefill_tile_rows(),
                          partial_floats=H * (dv + 2))
        if accumulate:
            self.o.emit(b, out, x, kernels.EPI_ACCUMULATE, out_norm=out_norm, out_norm_when=out_norm_when)
        else:
            self.o.emit(b, out, x, kernels.EPI_STORE)
