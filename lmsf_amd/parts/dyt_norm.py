"""Dynamic Tanh in the place of a norm: y = tanh(alpha x) * w + b.

alpha is one learned number, w and b are vectors; no mean and no variance are computed, so the "norm" is
elementwise and has no eps. All arithmetic is float32 (csrc/dyt_norm.hip); like RMSNorm it carries out the
addition of the branch before it into the float32 stream. The reference's only norm is RMSNorm
(vllm/kernels/layernorm_kernels.cu:13-38).
"""
from typing import Callable, Dict, Optional

import torch

from .base import Norm, Runtime, TensorDecl, register_part


@register_part("norm", "dynamic_tanh")
class DynamicTanh(Norm):
    """``weight_name``, ``bias_name`` and ``alpha_name`` are appended to the prefix with a dot ("": the tensor is the
    prefix itself)."""

    graph_safe = True
    recordable = False

    def __init__(self, prefix: str, rt: Runtime, size: int, weight_name: str = "weight", bias_name: str = "bias",
                 alpha_name: str = "alpha", alpha_init: float = 0.5):
        super().__init__(prefix, rt)
        self.size = int(size)
        self.alpha_init = float(alpha_init)

        def full(name: str) -> str:
            return "%s.%s" % (prefix, name) if name else prefix

        self.weight_name, self.bias_name, self.alpha_name = full(weight_name), full(bias_name), full(alpha_name)
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None
        self.alpha: Optional[torch.Tensor] = None

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        return {self.weight_name: TensorDecl((self.size,), init="ones", keeps_float32=True),
                self.bias_name: TensorDecl((self.size,), init="zeros", keeps_float32=True),
                self.alpha_name: TensorDecl((), init="const:%r" % self.alpha_init, keeps_float32=True)}

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        self.weight = fetch(self.weight_name).to(torch.float32).contiguous()
        self.bias = fetch(self.bias_name).to(torch.float32).contiguous()
        self.alpha = fetch(self.alpha_name).to(torch.float32).reshape(1).contiguous()

    def tensors(self):
        return [t for t in (self.weight, self.bias, self.alpha) if t is not None]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.dtype == torch.float32:
            return self.rt.ops.dyt_norm(None, x, self.weight, self.bias, self.alpha, self.rt.dtype)
        return self.rt.ops.dyt_norm(x, None, self.weight, self.bias, self.alpha, self.rt.dtype)

    def forward_add(self, branch: Optional[torch.Tensor], residual: torch.Tensor,
                    rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        return self.rt.ops.dyt_norm(branch, residual, self.weight, self.bias, self.alpha, self.rt.dtype, rows=rows)
