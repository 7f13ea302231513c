"""Softmax attention over the paged cache whose keys and values have sizes of their own, with optional extras.

H query heads and G key/value heads (query head h uses key/value head h // (H / G)), ``dim`` entries a query
or key, ``vdim`` a value. In the order in which they act, each optional:

- biases on q, k and v;
- a short causal convolution over time on every channel of q, k and v, directly after the projection (its last
  taps - 1 inputs per request are state);
- q and k divided by their root mean square over the head (a norm without a weight);
- rotary positions on the first ``rotary_dim`` entries of q and k, pairs (i, i + rotary_dim / 2);
- a query temperature: q times 1 + coef ln(floor((p + 1) / every) + 1) at position p;
- score = q . k * scale; causal, within a window of the last positions, or within the query's own chunk of
  ``chunk`` positions (chunks counted from position 0 of the request);
- the concatenated heads times sigmoid(W_g h), elementwise, before the output projection.

The attention kernels take one head size: the cache holds keys and values padded with zeros to
D = max(dim, vdim) rounded up to 16 (zeros in a key change no score; the outputs that padded values give are
dropped). Keys and values are written to the pages before any query reads, so every way of cutting a request
into steps is one case. The reference's attention has one head size and none of the extras
(core/src/model_executor/layers/attention.rs:91-231).
"""
from typing import Dict, Optional

import torch

from .base import (CacheBinding, CacheSpec, Mixer, PartSpec, PositionEncoding, Runtime, StateSpec, build_part,
                   register_part)
from .linear import FusedLinear, Linear
from .recurrent import ShortConv


@register_part("mixer", "flex_attention")
class FlexAttention(Mixer):
    graph_safe = True
    recordable = False

    def __init__(self, prefix: str, rt: Runtime, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 v_head_dim: int, scale: float, position: Optional[PartSpec] = None, qkv_bias: bool = False,
                 conv_taps: int = 0, unit_norm_eps: Optional[float] = None, temp_coef: float = 0.0, temp_every: int = 0,
                 window: Optional[int] = None, chunk: Optional[int] = None, output_gate: bool = False,
                 names: Optional[Dict[str, str]] = None, bias_name: str = "b"):
        super().__init__(prefix, rt)
        self.H, self.G, self.dim, self.vdim = int(num_heads), int(num_kv_heads), int(head_dim), int(v_head_dim)
        if self.H % self.G:
            raise ValueError("%s: heads %d is not a multiple of kv_heads %d" % (prefix, self.H, self.G))
        if window and chunk:
            raise ValueError("%s: a window or a chunk, not both" % prefix)
        self.scale = float(scale)
        self.window = int(window) if window else None
        self.chunk = int(chunk) if chunk else None
        self.unit_norm_eps = None if unit_norm_eps is None else float(unit_norm_eps)
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every or 0)
        self.D = (max(self.dim, self.vdim) + 15) // 16 * 16
        check = getattr(rt.ops, "check_head_dim", None)
        if check is not None:
            check(self.D, 1024)
        nm = dict(q="q", k="k", v="v", g="g", o="o", conv="conv")
        nm.update(names or {})
        H, G = self.H, self.G
        self.n_qkv = (H + G) * self.dim + G * self.vdim
        sources = [(nm["q"], H * self.dim), (nm["k"], G * self.dim), (nm["v"], G * self.vdim)]
        self.has_gate = bool(output_gate)
        if self.has_gate:
            sources.append((nm["g"], H * self.vdim))
        bias = [nm["q"], nm["k"], nm["v"]] if qkv_bias else False
        self.proj = FusedLinear(prefix, rt, hidden_size, sources, bias=bias, bare_names=True, bias_name=bias_name)
        self.conv: Optional[ShortConv] = None
        if conv_taps and int(conv_taps) >= 1:          # (one tap: a weight per channel, and no state)
            self.conv = ShortConv(prefix, rt, [("%s.%s" % (nm[x], nm["conv"]), n) for x, n in zip("qkv", (
                H * self.dim, G * self.dim, G * self.vdim))], int(conv_taps))
        self.o = Linear(prefix, rt, nm["o"], H * self.vdim, hidden_size, bare_names=True)
        self.position: Optional[PositionEncoding] = build_part("position", position, prefix, rt) if position else None

    def children(self):
        return [p for p in (self.proj, self.conv, self.o, self.position) if p is not None]

    def cache_spec(self) -> Optional[CacheSpec]:
        return CacheSpec(num_kv_heads=self.G, head_dim=self.D, window=self.window)

    def state_spec(self) -> Optional[StateSpec]:
        if self.conv is None or self.conv.state_floats == 0:
            return None
        return StateSpec((self.conv.state_floats,), torch.float32)

    def forward(self, h: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        ops = self.rt.ops
        H, G, dim, vdim, D = self.H, self.G, self.dim, self.vdim, self.D
        group = ctx.groups[binding.group]
        table = None
        if self.position is not None:
            rotary = self.position.rotary_table()
            if rotary is None or not rotary[2]:
                raise ValueError("%s rotates pairs (i, i + rot/2) from a table" % self.prefix)
            table = rotary[0]
        p = self.proj.forward(h)                                   # [N, q | k | v (| g)]
        qkv = p[:, :self.n_qkv]
        if self.conv is not None:
            qkv = self.conv.forward(qkv, ctx, binding.state)
        q, k, v = qkv[:, :H * dim], qkv[:, H * dim:(H + G) * dim], qkv[:, (H + G) * dim:]
        slots = group.slots if binding.writes_cache else None
        qa = ops.attn_prepare(q, k, v, H, G, dim, vdim, D, ctx.positions, slots, binding.k_pages, binding.v_pages,
                              table=table, unit_norm_eps=self.unit_norm_eps, temp_coef=self.temp_coef,
                              temp_every=self.temp_every)
        a = ops.paged_attention(qa, binding.k_pages, binding.v_pages, group.block_tables, ctx.seg_of_token,
                                ctx.positions, H, G, D, self.scale, self.window or 0, batch=ctx, chunk=self.chunk or 0)
        if self.has_gate or D != vdim:
            a = ops.head_gate(a, D, H, vdim, gate=p[:, self.n_qkv:] if self.has_gate else None)
        return self.o.forward(a)
