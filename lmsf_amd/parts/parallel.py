"""Two mixers side by side: both read the same input, each output is RMS-normed over the model width with a
weight of its own, and the result is a fixed multiple of their sum (half of it: the mean).

The pair is itself a mixer: its paged cache is that of the one child that has one, its state the children's
states one behind the other in a request's slot. The reference has no such arrangement
(core/src/model_executor/models/llama/llama.rs:276-385 is its only block).
"""
from typing import Callable, Dict, Optional

import torch

from .base import CacheBinding, CacheSpec, Mixer, PartSpec, Runtime, StateSpec, build_part, register_part
from .recurrent import FloatVector


@register_part("mixer", "parallel_pair")
class ParallelPair(Mixer):
    graph_safe = True
    recordable = False

    def __init__(self, prefix: str, rt: Runtime, hidden_size: int, left: PartSpec, right: PartSpec, eps: float,
                 scale: float = 0.5, left_prefix: str = "left", right_prefix: str = "right", out_name: str = "out"):
        super().__init__(prefix, rt)
        self.eps, self.scale = float(eps), float(scale)
        self.left: Mixer = build_part("mixer", left, "%s.%s" % (prefix, left_prefix), rt)
        self.right: Mixer = build_part("mixer", right, "%s.%s" % (prefix, right_prefix), rt)
        self.left_out = FloatVector("%s.%s.%s" % (prefix, left_prefix, out_name), rt, (int(hidden_size),), init="ones")
        self.right_out = FloatVector("%s.%s.%s" % (prefix, right_prefix, out_name), rt, (int(hidden_size),), init="ones")
        if self.left.cache_spec() is not None and self.right.cache_spec() is not None:
            raise ValueError("%s: at most one of two mixers side by side may keep a paged cache" % prefix)
        self._sizes = []
        for m in (self.left, self.right):
            sp = m.state_spec()
            if sp is not None and (sp.dtype != torch.float32 or len(sp.shape) != 1):
                raise ValueError("%s: mixers side by side keep their state as a row of float32 numbers" % prefix)
            self._sizes.append(0 if sp is None else int(sp.shape[0]))

    def children(self):
        return [self.left, self.right, self.left_out, self.right_out]

    def cache_spec(self) -> Optional[CacheSpec]:
        return self.left.cache_spec() or self.right.cache_spec()

    def state_spec(self) -> Optional[StateSpec]:
        total = sum(self._sizes)
        return StateSpec((total,), torch.float32) if total else None

    def _child_binding(self, binding: CacheBinding, which: int) -> CacheBinding:
        a = sum(self._sizes[:which])
        n = self._sizes[which]
        return CacheBinding(group=binding.group, k_pages=binding.k_pages, v_pages=binding.v_pages,
                            writes_cache=binding.writes_cache,
                            state=binding.state[:, a:a + n] if n and binding.state is not None else None)

    def forward(self, h: torch.Tensor, ctx, binding: CacheBinding) -> torch.Tensor:
        a = self.left.forward(h, ctx, self._child_binding(binding, 0))
        b = self.right.forward(h, ctx, self._child_binding(binding, 1))
        return self.rt.ops.rms_pair(a, b, self.left_out.weight, self.right_out.weight, self.eps, self.scale)
