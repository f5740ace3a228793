"""Root-mean-square norm: ``y = x / sqrt(mean(x^2) + eps) * gain`` in 32-bit
(rocml-kernels/kernels/rmsnorm.hip:18-42); reads the 32-bit residual stream and writes
the activation type.  With ``unit_offset`` the checkpoint stores ``gain - 1``: one is added in
32-bit when the weight is bound, and the kernels see the gain.  A norm that is not ``learned`` has no
weight: its gain is a vector of ones made here."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import NormSpec
from .base import BuildContext, Norm, NormHint, ParamSpec
from .registry import register_norm


class RMSNorm(Norm):
    prompt_graph_safe = True

    def __init__(self, spec: NormSpec, ctx: BuildContext):
        self.size = spec.size
        self.eps = float(spec.eps)
        self.unit_offset = bool(getattr(spec, "unit_offset", False))
        self.learned = bool(getattr(spec, "learned", True))
        self.gain: Optional[torch.Tensor] = None
        if not self.learned and torch.device(ctx.device).type != "meta":
            self.gain = torch.ones(self.size, dtype=torch.float32, device=ctx.device)

    def param_specs(self) -> Dict[str, ParamSpec]:
        if not self.learned:
            return {}
        return {"weight": ParamSpec((self.size,), role="gain", init="offset" if self.unit_offset else "gain")}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        if not self.learned:
            return
        self.gain = tensors["weight"] + 1.0 if self.unit_offset else tensors["weight"]

    fuses_pending = True      # forward() can add a deferred product's partial sums to x itself

    def prescale_hint(self) -> Optional[NormHint]:
        return None if self.gain is None else NormHint(self.gain, self.eps, self.size)

    def forward(self, x: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None,
                pending: Optional[torch.Tensor] = None) -> None:
        ops.rmsnorm(x, self.gain, self.eps, out, rows, partials=pending)


register_norm("rmsnorm", RMSNorm)
