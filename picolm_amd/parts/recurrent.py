"""Mixers that carry a matrix state per head from token to token, and the short convolution over
time in front of them.  The state (float) and the convolution's last inputs live in the state
entry of the layer call: per slot `[(taps - 1) channels | heads key_dim value_dim]` floats, zero
when a sequence starts.

GatedDeltaRule, per head with key head floor(h / (heads / key_heads)):
    q, k, v = silu(conv(W h));  q <- q / |q| / sqrt(key_dim),  k <- k / |k|
    S <- a S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q          (o is read after the update)
    a = exp(-exp(A_log) softplus(W_a h + dt_bias)),  beta = sigmoid(W_b h)
    out = W_o (rms(o) w_norm silu(W_g h))                                 rms per head

Mamba2 (state-space duality), W_in h = [z | x | B | C | dt]:
    x, B, C = silu(conv([x | B | C]) + b);  dt <- softplus(dt + dt_bias)
    S <- exp(-exp(A_log) dt) S + dt B x^T;  y = S^T C + D x
    out = W_o (rms_parts(y silu(z)) w_norm)                               gated first, then normed

Mamba1 (selective scan), W_in h = [x | z], a state S [state] per channel:
    x = silu(conv(x) + b);  [dt_low | B | C] = W_x x;  dt = softplus(W_dt dt_low + dt_bias)   per channel
    S_c <- exp(dt_c A_c) S_c + dt_c x_c B;  y_c = S_c . C + D_c x_c;  A = -exp(A_log) [channels, state]
    out = W_o (y silu(z))

HGRN2, per head a state S [key_dim][value_dim] whose forget gate also weighs what is written:
    q = silu(W_q h);  v = W_v h;  f = lower + (1 - lower) sigmoid(W_f h + b)                  per head and key channel
    S <- diag(f) S + (1 - f) v^T;  o = S^T q;  out = W_o (rms(o) w_norm)                      rms per head

A mixer's state may lie behind other floats of the layer call's state entry (`state_base`): a
block that keeps a row of its own there says where the mixer's begins.
"""
from __future__ import annotations

import torch

from .. import kernels
from ..weights import TensorSpec
from .base import Mixer, Runtime, StateRequest
from .calls import (DECAY_EXPONENTIAL, DECAY_PER_ROW, DECAY_SCAN_MAX_KEY_DIM, GATE_NONE, GATE_SILU, RULE_DELTA, RULE_OUTER_PRODUCT,
                    SHORT_CONV_MAX_TAPS, STATE_SCAN_MAX_KEY_DIM, DecayScanArgs, ForgetGatesArgs, GatedNormArgs, GateRowsArgs,
                    ShortConvArgs, StateScanArgs, emit_library_call)
from .linear import Linear


def _check_sizes(key_dim: int, taps: int) -> None:
    if not 1 <= key_dim <= STATE_SCAN_MAX_KEY_DIM:
        raise ValueError(f"a state with keys of {key_dim}: the kernel takes 1 to {STATE_SCAN_MAX_KEY_DIM}")
    if not 1 <= taps <= SHORT_CONV_MAX_TAPS:
        raise ValueError(f"a convolution of {taps} taps: the kernel takes 1 to {SHORT_CONV_MAX_TAPS}")


class GatedDeltaRule(Mixer):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, n_key_heads: int, key_dim: int, value_dim: int, taps: int,
                 eps: float, unit_eps: float = 1e-6):
        if n_heads % n_key_heads:
            raise ValueError(f"{n_heads} heads do not split over {n_key_heads} key heads")
        _check_sizes(key_dim, taps)
        self.prefix, self.D = prefix, hidden_size
        self.H, self.G, self.dk, self.dv, self.taps = n_heads, n_key_heads, key_dim, value_dim, taps
        self.eps, self.unit_eps = float(eps), float(unit_eps)
        qk, vv = n_key_heads * key_dim, n_heads * value_dim
        self.channels = 2 * qk + vv
        # one product: [q | k | v | gate | decay | strength]
        self.proj = Linear([prefix + n for n in ("q", "k", "v", "g", "a", "b")], [qk, qk, vv, vv, n_heads, n_heads], hidden_size)
        self.o = Linear([prefix + "o"], [hidden_size], vv)
        self.conv = self.A_log = self.dt_bias = self.norm = None

    def children(self):
        return [self.proj, self.o]

    def tensor_specs(self):
        p, qk, vv = self.prefix, self.G * self.dk, self.H * self.dv
        return [TensorSpec(p + "q.conv", (qk, self.taps)), TensorSpec(p + "k.conv", (qk, self.taps)),
                TensorSpec(p + "v.conv", (vv, self.taps)), TensorSpec(p + "A_log", (self.H,)), TensorSpec(p + "dt_bias", (self.H,)),
                TensorSpec(p + "norm", (self.dv,), init="ones")]

    def load(self, fetch, runtime: Runtime) -> None:
        f32 = lambda name: fetch.get(self.prefix + name).to(torch.float32)
        self.conv = torch.cat([f32("q.conv"), f32("k.conv"), f32("v.conv")], dim=0).contiguous()
        self.A_log, self.dt_bias, self.norm = f32("A_log").contiguous(), f32("dt_bias").contiguous(), f32("norm").contiguous()

    def state_floats(self) -> int:
        return (self.taps - 1) * self.channels + self.H * self.dk * self.dv

    def cache_requests(self):
        return None, StateRequest((self.state_floats(),), torch.float32)

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0, accumulate: bool = True) -> None:
        """x (+)= o(norm(scan) * silu(g)) for the rows h of `src`, as operations of a launch program."""
        H, qk, vv, C = self.H, self.G * self.dk, self.H * self.dv, self.channels
        width = self.proj.out_size
        rows = b.buffer("delta.in", width, torch.float32)
        self.proj.emit(b, src, rows, kernels.EPI_STORE)
        qkv = b.buffer("scan.qkv", C, torch.float32)
        emit_library_call(b, "short_conv", ShortConvArgs(b._ptr(self.conv), None, C, self.taps, width, 0, C, 0, 0, 1), qkv, inp=rows,
                          uses_state=True)
        aw = b.buffer("scan.aw", 2 * H, torch.float32)
        y = b.buffer("scan.out", vv, torch.float32)
        scan = StateScanArgs(RULE_DELTA, H, self.G, self.dk, self.dv, width, C + vv, C + vv + H, C, 0, qk, 2 * qk,
                             b._ptr(self.A_log), b._ptr(self.dt_bias), None, 1, self.unit_eps, float(self.dk) ** -0.5,
                             (self.taps - 1) * C)
        emit_library_call(b, "state_scan", scan, y, inp=rows, extra=[qkv, aw], uses_state=True)
        gated = b.buffer("scan.gated", vv, b.dtype)
        emit_library_call(b, "gated_norm", GatedNormArgs(b._ptr(self.norm), self.dv, vv, self.dv, self.eps, 0, width, C), gated, inp=y,
                          extra=[rows])
        self.o.emit(b, gated, x, kernels.EPI_ACCUMULATE if accumulate else kernels.EPI_STORE,
                    **({"out_norm": out_norm, "out_norm_when": out_norm_when} if accumulate else {}))


class Mamba2(Mixer):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, value_dim: int, state_dim: int, groups: int, taps: int,
                 norm_groups: int, eps: float):
        if n_heads % groups:
            raise ValueError(f"{n_heads} heads do not split over {groups} groups")
        inner = n_heads * value_dim
        if norm_groups < 1 or inner % norm_groups:
            raise ValueError(f"an inner width of {inner} does not split into {norm_groups} parts")
        _check_sizes(state_dim, taps)
        self.prefix, self.D = prefix, hidden_size
        self.H, self.P, self.N, self.G, self.taps, self.parts = n_heads, value_dim, state_dim, groups, taps, norm_groups
        self.inner, self.eps = inner, float(eps)
        self.channels = inner + 2 * groups * state_dim
        self.proj = Linear([prefix + "in"], [2 * inner + 2 * groups * state_dim + n_heads], hidden_size)
        self.o = Linear([prefix + "o"], [hidden_size], inner)
        self.conv = self.conv_bias = self.A_log = self.dt_bias = self.skip = self.norm = None

    def children(self):
        return [self.proj, self.o]

    def tensor_specs(self):
        p = self.prefix
        return [TensorSpec(p + "conv", (self.channels, self.taps)), TensorSpec(p + "conv.b", (self.channels,)),
                TensorSpec(p + "dt_bias", (self.H,)), TensorSpec(p + "A_log", (self.H,)), TensorSpec(p + "D", (self.H,), init="ones"),
                TensorSpec(p + "norm", (self.inner,), init="ones")]

    def load(self, fetch, runtime: Runtime) -> None:
        f32 = lambda name: fetch.get(self.prefix + name).to(torch.float32).contiguous()
        self.conv, self.conv_bias = f32("conv"), f32("conv.b")
        self.A_log, self.dt_bias, self.skip, self.norm = f32("A_log"), f32("dt_bias"), f32("D"), f32("norm")

    def state_floats(self) -> int:
        return (self.taps - 1) * self.channels + self.H * self.N * self.P

    def cache_requests(self):
        return None, StateRequest((self.state_floats(),), torch.float32)

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0, accumulate: bool = True) -> None:
        """x (+)= o(norm(scan * silu(z))) for the rows h of `src`, as operations of a launch program."""
        H, inner, GN, C = self.H, self.inner, self.G * self.N, self.channels
        width = self.proj.out_size
        rows = b.buffer("mamba.in", width, torch.float32)
        self.proj.emit(b, src, rows, kernels.EPI_STORE)
        xbc = b.buffer("scan.qkv", C, torch.float32)
        emit_library_call(b, "short_conv", ShortConvArgs(b._ptr(self.conv), b._ptr(self.conv_bias), C, self.taps, width, inner, C, 0, 0, 1),
                          xbc, inp=rows, uses_state=True)
        aw = b.buffer("scan.aw", 2 * H, torch.float32)
        y = b.buffer("scan.out", inner, torch.float32)
        dt_off = 2 * inner + 2 * GN
        # keys are B, queries C, values x; decay and strength both come from dt
        scan = StateScanArgs(RULE_OUTER_PRODUCT, H, self.G, self.N, self.P, width, dt_off, dt_off, C, inner + GN, inner, 0,
                             b._ptr(self.A_log), b._ptr(self.dt_bias), b._ptr(self.skip), 0, 0.0, 1.0, (self.taps - 1) * C)
        emit_library_call(b, "state_scan", scan, y, inp=rows, extra=[xbc, aw], uses_state=True)
        gated = b.buffer("scan.gated", inner, b.dtype)
        emit_library_call(b, "gated_norm", GatedNormArgs(b._ptr(self.norm), inner, inner, inner // self.parts, self.eps, 1, width, 0),
                          gated, inp=y, extra=[rows])
        self.o.emit(b, gated, x, kernels.EPI_ACCUMULATE if accumulate else kernels.EPI_STORE,
                    **({"out_norm": out_norm, "out_norm_when": out_norm_when} if accumulate else {}))


def _cast_rows(b, src: int, src_stride: int, src_off: int, width: int, name: str) -> int:
    """Columns of float rows as rows of the engine's dtype, for a product to read."""
    from ..engine.program import _DT, F32
    out = b.buffer(name, width, b.dtype)
    emit_library_call(b, "gate_rows", GateRowsArgs(width, GATE_NONE, src_stride, src_off, F32, 0, 0, _DT[b.dtype], None), out, inp=src)
    return out


class Mamba1(Mixer):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, prefix: str, hidden_size: int, inner: int, state_dim: int, dt_rank: int, taps: int):
        if not 1 <= state_dim <= DECAY_SCAN_MAX_KEY_DIM:
            raise ValueError(f"a state of {state_dim} a channel: the kernel takes 1 to {DECAY_SCAN_MAX_KEY_DIM}")
        if not 1 <= taps <= SHORT_CONV_MAX_TAPS:
            raise ValueError(f"a convolution of {taps} taps: the kernel takes 1 to {SHORT_CONV_MAX_TAPS}")
        self.prefix, self.D = prefix, hidden_size
        self.inner, self.N, self.R, self.taps = inner, state_dim, dt_rank, taps
        self.state_base = 0
        self.proj = Linear([prefix + "in"], [2 * inner], hidden_size)
        self.x_proj = Linear([prefix + "x"], [dt_rank + 2 * state_dim], inner)
        self.dt_proj = Linear([prefix + "dt"], [inner], dt_rank)
        self.o = Linear([prefix + "o"], [hidden_size], inner)
        self.conv = self.conv_bias = self.A = self.dt_bias = self.skip = None

    def children(self):
        return [self.proj, self.x_proj, self.dt_proj, self.o]

    def tensor_specs(self):
        p = self.prefix
        return [TensorSpec(p + "conv", (self.inner, self.taps)), TensorSpec(p + "conv.b", (self.inner,)),
                TensorSpec(p + "dt.b", (self.inner,)), TensorSpec(p + "A_log", (self.inner, self.N)),
                TensorSpec(p + "D", (self.inner,), init="ones")]

    def load(self, fetch, runtime: Runtime) -> None:
        f32 = lambda name: fetch.get(self.prefix + name).to(torch.float32).contiguous()
        self.conv, self.conv_bias, self.dt_bias, self.skip = f32("conv"), f32("conv.b"), f32("dt.b"), f32("D")
        self.A = (-torch.exp(f32("A_log"))).contiguous()

    def state_floats(self) -> int:
        return (self.taps - 1) * self.inner + self.inner * self.N

    def cache_requests(self):
        return None, StateRequest((self.state_floats(),), torch.float32)

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0, accumulate: bool = True) -> None:
        """x (+)= o(scan * silu(z)) for the rows h of `src`, as operations of a launch program."""
        inner, N, R = self.inner, self.N, self.R
        xz = b.buffer("mamba1.in", 2 * inner, torch.float32)
        self.proj.emit(b, src, xz, kernels.EPI_STORE)
        xc = b.buffer("scan.x", inner, torch.float32)
        emit_library_call(b, "short_conv", ShortConvArgs(b._ptr(self.conv), b._ptr(self.conv_bias), inner, self.taps, 2 * inner, 0, inner, 0,
                                                         self.state_base, 1), xc, inp=xz, uses_state=True)
        low = b.buffer("mamba1.low", R + 2 * N, torch.float32)
        self.x_proj.emit(b, _cast_rows(b, xc, inner, 0, inner, "scan.x.rows"), low, kernels.EPI_STORE)
        dt = b.buffer("mamba1.dt", inner, torch.float32)
        self.dt_proj.emit(b, _cast_rows(b, low, R + 2 * N, 0, R, "mamba1.dt.rows"), dt, kernels.EPI_STORE)
        y = b.buffer("scan.out", inner, torch.float32)
        # one head whose values are the channels: keys are B, queries C, both shared by all channels
        scan = DecayScanArgs(DECAY_EXPONENTIAL, 1, 1, N, inner, R + 2 * N, R + N, R, 0, inner, 0, inner, 0, b._ptr(self.dt_bias),
                             b._ptr(self.A), b._ptr(self.skip), self.state_base + (self.taps - 1) * inner)
        emit_library_call(b, "decay_scan", scan, y, inp=xc, extra=[low, dt], uses_state=True)
        from ..engine.program import _DT, F32
        gated = b.buffer("scan.gated", inner, b.dtype)
        emit_library_call(b, "gate_rows", GateRowsArgs(inner, GATE_SILU, inner, 0, F32, 2 * inner, inner, _DT[b.dtype], None), gated, inp=y,
                          extra=[xz])
        self.o.emit(b, gated, x, kernels.EPI_ACCUMULATE if accumulate else kernels.EPI_STORE,
                    **({"out_norm": out_norm, "out_norm_when": out_norm_when} if accumulate else {}))


class HGRN2(Mixer):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, key_dim: int, value_dim: int, eps: float):
        if not 1 <= key_dim <= DECAY_SCAN_MAX_KEY_DIM:
            raise ValueError(f"a state with keys of {key_dim}: the kernel takes 1 to {DECAY_SCAN_MAX_KEY_DIM}")
        self.prefix, self.D = prefix, hidden_size
        self.H, self.dk, self.dv, self.eps = n_heads, key_dim, value_dim, float(eps)
        self.state_base = 0
        qk, vv = n_heads * key_dim, n_heads * value_dim
        self.proj = Linear([prefix + n for n in ("q", "f", "v")], [qk, qk, vv], hidden_size)
        self.o = Linear([prefix + "o"], [hidden_size], vv)
        self.f_bias = self.lower = self.norm = None

    def children(self):
        return [self.proj, self.o]

    def tensor_specs(self):
        p, qk = self.prefix, self.H * self.dk
        return [TensorSpec(p + "f.b", (qk,)), TensorSpec(p + "lower", (qk,)), TensorSpec(p + "norm", (self.dv,), init="ones")]

    def load(self, fetch, runtime: Runtime) -> None:
        f32 = lambda name: fetch.get(self.prefix + name).to(torch.float32).contiguous()
        self.f_bias, self.lower, self.norm = f32("f.b"), f32("lower"), f32("norm")

    def state_floats(self) -> int:
        return self.H * self.dk * self.dv

    def cache_requests(self):
        return None, StateRequest((self.state_floats(),), torch.float32)

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0, accumulate: bool = True) -> None:
        """x (+)= o(norm(scan)) for the rows h of `src`, as operations of a launch program."""
        H, qk, vv = self.H, self.H * self.dk, self.H * self.dv
        width = self.proj.out_size
        rows = b.buffer("hgrn2.in", width, torch.float32)
        self.proj.emit(b, src, rows, kernels.EPI_STORE)
        gates = b.buffer("scan.qka", 3 * qk, torch.float32)
        emit_library_call(b, "forget_gates", ForgetGatesArgs(b._ptr(self.lower), b._ptr(self.f_bias), qk, width, 0, qk), gates, inp=rows)
        y = b.buffer("scan.out", vv, torch.float32)
        scan = DecayScanArgs(DECAY_PER_ROW, H, H, self.dk, self.dv, 3 * qk, 0, qk, 2 * qk, width, 2 * qk, 0, 0, None, None, None,
                             self.state_base)
        emit_library_call(b, "decay_scan", scan, y, inp=rows, extra=[gates], uses_state=True)
        normed = b.buffer("scan.gated", vv, b.dtype)
        emit_library_call(b, "gated_norm", GatedNormArgs(b._ptr(self.norm), self.dv, vv, self.dv, self.eps, 0, 0, 0), normed, inp=y)
        self.o.emit(b, normed, x, kernels.EPI_ACCUMULATE if accumulate else kernels.EPI_STORE,
                    **({"out_norm": out_norm, "out_norm_when": out_norm_when} if accumulate else {}))
