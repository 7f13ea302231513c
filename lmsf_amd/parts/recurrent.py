"""Mixers whose memory of a request is a state of fixed size: the selective scan and a matrix memory with
exponential gates, and the short causal convolution that both they and some attention layers put behind a
projection.

A request's state is one row of float32 numbers in the engine's state slots (``StateSpec``); a mixer says how
many it needs and gets ``binding.state`` [slots, that many]. The engine clears a row when a request takes it, so
"zeros before the sequence's start" and "the state starts at zero" need no code here. Everything that enters a
recurrence is float32 (csrc/recurrent.hip); the projections run in the run's dtype. The reference has no mixer
with state (its only one is attention over a paged cache, core/src/model_executor/layers/attention.rs:91-231).
"""
from typing import Callable, Dict, Optional, Sequence, Tuple

import torch

from .base import CacheBinding, Mixer, Part, Runtime, StateSpec, TensorDecl, register_part
from .linear import FusedLinear, Linear


class ShortConv(Part):
    """Causal convolution over time, a filter of ``taps`` per channel: y_t = sum_j w[:, j] u_(t - taps + 1 + j)
    (+ bias), zeros before a request's start. ``sources``: (checkpoint name under the prefix, channels) of the
    filters, laid side by side as one [C, taps] tensor; ``bias_name``: the name of a bias of C entries, or None.
    The last taps - 1 inputs of every request are its state: ``state_floats`` numbers."""

    graph_safe = True
    recordable = False

    def __init__(self, prefix: str, rt: Runtime, sources: Sequence[Tuple[str, int]], taps: int,
                 bias_name: Optional[str] = None, activation: Optional[str] = None):
        super().__init__(prefix, rt)
        self.sources = [(str(n), int(c)) for n, c in sources]
        self.channels = sum(c for _, c in self.sources)
        self.taps = int(taps)
        if self.taps < 1:
            raise ValueError("%s: a convolution needs at least one tap" % prefix)
        self.bias_name = bias_name
        self.activation = activation
        self.state_floats = self.channels * (self.taps - 1)
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def _full(self, name: str) -> str:
        return "%s.%s" % (self.prefix, name)

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        out = {self._full(n): TensorDecl((c, self.taps), init="normal:0.3") for n, c in self.sources}
        if self.bias_name:
            out[self._full(self.bias_name)] = TensorDecl((self.channels,), init="zeros")
        return out

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        parts = [fetch(self._full(n)) for n, _ in self.sources]
        self.weight = (parts[0] if len(parts) == 1 else torch.cat(parts, 0)).to(self.rt.dtype).contiguous()
        if self.bias_name:
            self.bias = fetch(self._full(self.bias_name)).to(self.rt.dtype).contiguous()

    def forward(self, u: torch.Tensor, ctx, state: Optional[torch.Tensor]) -> torch.Tensor:
        return self.rt.ops.short_conv(u, self.weight, self.bias, state, ctx, self.activation)


class FloatVector(Part):
    """A checkpoint tensor that is kept in float32 whatever the run's dtype (what enters a recurrence)."""

    graph_safe = True

    def __init__(self, name: str, rt: Runtime, shape: Tuple[int, ...], init: str = "normal"):
        super().__init__(name, rt)
        self.shape, self.init = tuple(shape), init
        self.weight: Optional[torch.Tensor] = None

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        return {self.prefix: TensorDecl(self.shape, init=self.init, keeps_float32=True)}

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        self.weight = fetch(self.prefix).to(torch.float32).contiguous()


@register_part("mixer", "selective_scan")
class SelectiveScan(Mixer):
    """Mamba's mixer. [x | z] = W_in h; x <- silu(conv(x) + b); [dt | B | C] = W_x x; dt <- softplus(W_dt dt + b_dt);
    A = -exp(A_log);  S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;  y_c = sum_n S[c, n] C_n + D_c x_c;
    out = W_o (y * silu(z)). State of a request: S [inner, state] and the convolution's last taps - 1 inputs."""

    graph_safe = True
    recordable = False

    def __init__(self, prefix: str, rt: Runtime, hidden_size: int, inner: int, state: int, dt_rank: int, conv: int,
                 names: Optional[Dict[str, str]] = None):
        super().__init__(prefix, rt)
        self.inner, self.n, self.rank, self.taps = int(inner), int(state), int(dt_rank), int(conv)
        if min(self.inner, self.n, self.rank, self.taps) < 1:
            raise ValueError("%s: sizes must be positive" % prefix)
        nm = dict(in_proj="in", conv="conv", conv_bias="conv.b", x_proj="x", dt_proj="dt", a_log="A_log", d="D", out="o")
        nm.update(names or {})
        self.in_proj = Linear(prefix, rt, nm["in_proj"], hidden_size, 2 * self.inner, bare_names=True)
        self.conv = ShortConv(prefix, rt, [(nm["conv"], self.inner)], self.taps, bias_name=nm["conv_bias"],
                              activation="silu")
        self.x_proj = Linear(prefix, rt, nm["x_proj"], self.inner, self.rank + 2 * self.n, bare_names=True)
        self.dt_proj = Linear(prefix, rt, nm["dt_proj"], self.rank, self.inner, bias=True, bare_names=True, bias_name="b")
        self.a_log = FloatVector("%s.%s" % (prefix, nm["a_log"]), rt, (self.inner, self.n), init="const:0.0")
        self.d = FloatVector("%s.%s" % (prefix, nm["d"]), rt, (self.inner,), init="ones")
        self.o = Linear(prefix, rt, nm["out"], self.inner, hidden_size, bare_names=True)
        self.scan_floats = self.inner * self.n

    def children(self):
        return [self.in_proj, self.conv, self.x_proj, self.dt_proj, self.a_log, self.d, self.o]

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec((self.scan_floats + self.conv.state_floats,), torch.float32)

    def forward(self, h: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        ops = self.rt.ops
        st = binding.state
        xz = self.in_proj.forward(h)                                            # [N, 2 inner]
        x = self.conv.forward(xz[:, :self.inner], ctx, st[:, self.scan_floats:] if self.taps > 1 else None)
        low = self.x_proj.forward(x)                                            # [N, rank + 2 n]: dt, B, C
        dt = ops.linear_wide(low[:, :self.rank], self.dt_proj.weight, self.dt_proj.bias)   # float32: a step size
        y = ops.selective_scan(x, dt, low, self.rank, self.rank + self.n, xz[:, self.inner:], self.a_log.weight,
                               self.d.weight, st, ctx)
        return self.o.forward(y)


@register_part("mixer", "matrix_memory")
class MatrixMemory(Mixer):
    """The matrix memory of xLSTM (mLSTM). q = W_q h * dim^-1/2, k = W_k h, v = W_v h per head; log gates
    i = cap tanh((W_i h + b_i) / cap), f = logsigmoid(cap tanh((W_f h + b_f) / cap)); with a running maximum m that
    starts at 0:  m' = max(f + m, i);  S <- exp(f + m - m') S + exp(i - m') k v^T;  n likewise with k alone;
    o = S^T q / (max(|n . q|, exp(-m')) + 1e-6). Every head's o over its root mean square, times a weight over all
    heads, times sigmoid(W_g h), then W_o. State of a request: S, n and m of every head."""

    graph_safe = True
    recordable = False

    def __init__(self, prefix: str, rt: Runtime, hidden_size: int, heads: int, dim: int, vdim: int, gate_cap: float,
                 eps: float, names: Optional[Dict[str, str]] = None):
        super().__init__(prefix, rt)
        self.H, self.d, self.dv = int(heads), int(dim), int(vdim)
        self.cap, self.eps = float(gate_cap), float(eps)
        if not self.cap > 0:
            raise ValueError("%s: gate_cap must be > 0" % prefix)
        nm = dict(q="q", k="k", v="v", g="g", i="i", f="f", norm="norm", out="o")
        nm.update(names or {})
        H, d, dv = self.H, self.d, self.dv
        self.qkvg = FusedLinear(prefix, rt, hidden_size, [(nm["q"], H * d), (nm["k"], H * d), (nm["v"], H * dv),
                                                          (nm["g"], H * dv)], bare_names=True)
        self.gates = FusedLinear(prefix, rt, hidden_size, [(nm["i"], H), (nm["f"], H)], bias=True, bare_names=True,
                                 bias_name="b")
        self.norm = FloatVector("%s.%s" % (prefix, nm["norm"]), rt, (H * dv,), init="ones")
        self.o = Linear(prefix, rt, nm["out"], H * dv, hidden_size, bare_names=True)
        sizer = getattr(rt.ops, "mlstm_state_floats", None)
        self.state_floats = int(sizer(H, d, dv)) if sizer is not None else H * d * (dv + 1) + H

    def children(self):
        return [self.qkvg, self.gates, self.norm, self.o]

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec((self.state_floats,), torch.float32)

    def forward(self, h: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        ops = self.rt.ops
        H, d, dv = self.H, self.d, self.dv
        p = self.qkvg.forward(h)
        gates = ops.linear_wide(h, self.gates.weight, self.gates.bias)                         # float32 [N, 2 H]
        o = ops.mlstm(p[:, :H * d], p[:, H * d:2 * H * d], p[:, 2 * H * d:2 * H * d + H * dv], gates,
                      p[:, 2 * H * d + H * dv:], self.norm.weight, binding.state, ctx, H, d, dv, d ** -0.5, self.cap,
                      self.eps)
        return self.o.forward(o)
