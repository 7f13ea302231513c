"""Feed-forward of experts that a table assigns: token id t runs the ``top`` experts table[t, :], each a gated
feed-forward Wd_e (act(Wg_e h) * (Wu_e h)), each weighted 1/top; an expert that every token runs (``shared``)
is added. There is no router to compute: the choice depends on the token id alone, and is read on the device
from the step's token ids (csrc/moe.hip), so that a decode step replays from a graph.

The reference has dense feed-forwards only (core/src/model_executor/models/llama/llama.rs:223-274).
"""
from typing import Callable, Dict, Optional

import torch

from .base import FeedForward, PartSpec, Runtime, TensorDecl, build_part, register_part


@register_part("feed_forward", "table_moe")
class TableMoE(FeedForward):
    graph_safe = True
    recordable = False
    needs_token_ids = True      # forward takes the step's token ids

    def __init__(self, prefix: str, rt: Runtime, hidden_size: int, expert_size: int, num_experts: int, top: int,
                 vocab_size: int, shared: Optional[PartSpec] = None, expert_prefix: str = "e", table_name: str = "table",
                 gate_name: str = "gate", up_name: str = "up", down_name: str = "down"):
        super().__init__(prefix, rt)
        self.W, self.F, self.E, self.top, self.V = int(hidden_size), int(expert_size), int(num_experts), int(top), \
            int(vocab_size)
        if not (0 < self.top <= self.E):
            raise ValueError("%s: %d of %d experts" % (prefix, self.top, self.E))
        self.names = [("%s.%s%d" % (prefix, expert_prefix, e), gate_name, up_name, down_name) for e in range(self.E)]
        self.table_name = "%s.%s" % (prefix, table_name)
        self.shared = build_part("feed_forward", shared, "%s.%s" % (prefix, shared.params.get("prefix", "shared")), rt) \
            if shared is not None else None
        self.w_gate_up: Optional[torch.Tensor] = None     # [E, 2F, W]
        self.w_down: Optional[torch.Tensor] = None        # [E, W, F]
        self.table: Optional[torch.Tensor] = None         # int32 [V, top]

    def children(self):
        return [self.shared] if self.shared is not None else []

    def tensors(self):
        return [t for t in (self.w_gate_up, self.w_down, self.table) if t is not None]

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        out = {self.table_name: TensorDecl((self.V, self.top), kind="int", init="choices:%d" % self.E)}
        for p, g, u, d in self.names:
            out["%s.%s" % (p, g)] = TensorDecl((self.F, self.W))
            out["%s.%s" % (p, u)] = TensorDecl((self.F, self.W))
            out["%s.%s" % (p, d)] = TensorDecl((self.W, self.F))
        return out

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        gu = torch.empty((self.E, 2 * self.F, self.W), dtype=self.rt.dtype, device=self.rt.device)
        dn = torch.empty((self.E, self.W, self.F), dtype=self.rt.dtype, device=self.rt.device)
        for e, (p, g, u, d) in enumerate(self.names):
            gu[e, :self.F].copy_(fetch("%s.%s" % (p, g)))
            gu[e, self.F:].copy_(fetch("%s.%s" % (p, u)))
            dn[e].copy_(fetch("%s.%s" % (p, d)))
        self.w_gate_up, self.w_down = gu, dn
        self.table = fetch(self.table_name).to(torch.int32).contiguous()

    def forward(self, h: torch.Tensor, token_ids: Optional[torch.Tensor] = None) -> torch.Tensor:
        if token_ids is None:
            raise ValueError("table_moe needs the step's token ids")
        base = self.shared.forward(h) if self.shared is not None else None
        return self.rt.ops.table_moe(h, self.w_gate_up, self.w_down, token_ids, self.table, 1.0 / self.top, base=base)


@register_part("feed_forward", "none")
class NoFeedForward(FeedForward):
    """A layer without a feed-forward sublayer; its block skips the sublayer and its norms."""

    graph_safe = True
    absent = True

    def __init__(self, prefix: str, rt: Runtime):
        super().__init__(prefix, rt)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        raise ValueError("%s has no feed-forward" % self.prefix)
