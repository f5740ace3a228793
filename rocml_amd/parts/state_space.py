"""A mixer that carries a state of fixed size from token to token: the recurrence with one scalar
decay per head (state-space duality).

The input projection gives ``[z | x | B | C | dt]``; x, B and C pass a short causal convolution per
channel and silu; per head ``S <- exp(-exp(A_log) dt) S + dt B x^T`` and ``y = S^T C + D x`` with
``dt = softplus(dt + dt_bias)``; ``y * silu(z)`` is normed in equal parts and projected back.  The
projections are products in the compute type with 32-bit sums; everything between them (the
convolution, step sizes, decays, the state, the gate and the norm) is 32-bit.  The cache holds two
things per sequence, both zero at its start: the state ``[heads, head size, state]`` and the
convolution's last ``taps - 1`` inputs.  A prompt step and a step of one token run the same kernels.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import StateSpaceSpec
from ..errors import ConfigError
from .base import BuildContext, CompositeRequest, Mixer, ParamSpec, StateRequest
from .registry import register_mixer
from .residual import stream


class StateSpaceMixer(Mixer):
    adds_only = True
    prompt_graph_safe = True
    kernel_families = ("recurrent",)

    def __init__(self, spec: StateSpaceSpec, ctx: BuildContext):
        if spec.n_heads % spec.groups != 0:
            raise ConfigError(f"{spec.n_heads} heads do not fall into {spec.groups} equal groups")
        self.inner = spec.n_heads * spec.head_dim
        if self.inner % spec.norm_groups != 0:
            raise ConfigError(f"{self.inner} values do not fall into {spec.norm_groups} equal parts for the norm")
        if not 1 <= spec.conv <= 8:
            raise ConfigError(f"the convolution has {spec.conv} taps; 1 to 8 are supported")
        if spec.state > 256:
            raise ConfigError(f"a state of {spec.state} per head exceeds the 256 the recurrence kernel keeps in registers")
        self.spec = spec
        self.dtype = ctx.dtype
        self.bc = spec.groups * spec.state
        self.conv_channels = self.inner + 2 * self.bc
        self.proj_dim = 2 * self.inner + 2 * self.bc + spec.n_heads
        self.w_in: Optional[torch.Tensor] = None
        self.w_out: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        s = self.spec
        return {"in_proj.weight": ParamSpec((self.proj_dim, s.hidden)),
                "conv.weight": ParamSpec((self.conv_channels, s.conv), role="gain", init="normal"),
                "conv.bias": ParamSpec((self.conv_channels,), role="gain", init="normal"),
                "dt_bias": ParamSpec((s.n_heads,), role="gain", init="normal"),
                "A_log": ParamSpec((s.n_heads,), role="gain", init="normal"),
                "D": ParamSpec((s.n_heads,), role="gain", init="gain"),
                "norm.weight": ParamSpec((self.inner,), role="gain", init="gain"),
                "out_proj.weight": ParamSpec((s.hidden, self.inner))}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_in, self.w_out = tensors["in_proj.weight"], tensors["out_proj.weight"]
        # stored [channels, taps]; the kernels read a tap's weights of neighbouring channels side by side
        self.conv_w, self.conv_b = tensors["conv.weight"].t().contiguous(), tensors["conv.bias"]
        self.dt_bias, self.a_log, self.d_skip = tensors["dt_bias"], tensors["A_log"], tensors["D"]
        self.norm_gain = tensors["norm.weight"]

    def cache_request(self) -> CompositeRequest:
        s = self.spec
        return CompositeRequest((StateRequest((s.n_heads, s.head_dim, s.state)),
                                 StateRequest((max(s.conv - 1, 0), self.conv_channels))))

    def flops(self, new_counts, starts) -> int:
        # the products with the weights; per token and head the state's update and its read
        s = self.spec
        return 2 * sum(new_counts) * (self.matrix_elements() + 2 * s.n_heads * s.head_dim * s.state)

    def activation_bytes(self, n_tokens: int) -> int:
        size = 2 if self.dtype == torch.bfloat16 else 4
        return n_tokens * ((self.proj_dim + self.conv_channels + self.inner) * 4 + self.inner * size)

    def input_weight(self) -> Optional[torch.Tensor]:
        return self.w_in

    def adopt_input_weight(self, view: torch.Tensor) -> None:
        self.w_in = view

    def forward(self, step, xn, x_accum, cache, owns_cache: bool, projected=None) -> None:
        if not owns_cache:
            raise ConfigError("a recurrent layer cannot run on another layer's state")
        s = self.spec
        n = step.n_tokens
        ws = step.workspace
        state, conv_state = cache.parts
        if projected is not None:        # the projection is columns c0 .. of a product shared with other mixers
            proj, c0 = projected
        else:
            proj, c0 = ws.get("ssm.proj", (n, self.proj_dim), torch.float32), 0
            ops.gemm(xn, self.w_in, proj, workspace=ws.scratch())
        xbc = ws.get("ssm.xbc", (n, self.conv_channels), torch.float32)
        ops.causal_conv(proj, c0 + self.inner, self.conv_channels, self.conv_w, self.conv_b, conv_state.state, step.token_seq,
                        step.cu_seqlens, step.seq_slots, xbc, silu=True)
        y = ws.get("ssm.y", (n, self.inner), torch.float32)
        ops.ssd_scan(xbc, proj, c0 + 2 * self.inner + 2 * self.bc, self.dt_bias, self.a_log, self.d_skip, state.state,
                     step.cu_seqlens, step.seq_slots, y, s.n_heads, s.head_dim, s.state, s.groups)
        gated = ws.get("ssm.gated", (n, self.inner), self.dtype)
        ops.gated_part_norm(y, proj, c0, self.norm_gain, gated, s.norm_groups, s.eps)
        stream(step).add_product(gated, self.w_out, x_accum)


register_mixer("state_space", StateSpaceMixer)
