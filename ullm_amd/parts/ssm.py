"""A selective state-space mixer (the Mamba-2 form) over per-request state.

The input projection's rows are z | x | B | C | dt (z, x: heads * head_dim; B, C: groups * state; dt: heads).
x | B | C pass a short causal convolution per channel and silu; dt = softplus(dt + dt_bias).  Per head h
(its B and C are those of group h // (heads / groups)) the state S [state, head_dim] moves token by token,
S = exp(-exp(A_log_h) dt) S + dt B x^T, and y = S^T C + D_h x.  y * silu(z) is RMS-normed in ``norm_groups``
equal parts, multiplied by a gain and projected out.

What a request keeps between steps is one float32 row per slot: the convolution's last taps-1 inputs, then
every head's state.  Everything behind the input projection is 32-bit (the projection leaves float32 rows
also where the model computes in bfloat16); the recurrence walks an entry's tokens in order whatever the
batch holds, so a token's result does not depend on how its prompt was cut.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import LayerCache, Mixer, PartEnv, StateNeed, StepContext, WeightDecl, register_part
from .linear import linear, linear_into_stream

DEFAULT_NAMES = {"in": "in_proj.weight", "conv": "conv1d.weight", "conv_bias": "conv1d.bias", "dt_bias": "dt_bias",
                 "a_log": "A_log", "d": "D", "norm": "norm.weight", "out": "out_proj.weight"}


@register_part("mixer", "mamba2")
class Mamba2(Mixer):
    def __init__(self, hidden_size: int, heads: int, head_dim: int, state: int, groups: int, conv: int,
                 norm_groups: int, norm_eps: float, prefix: str, names: Optional[Dict[str, str]] = None):
        if heads % groups:
            raise ValueError(f"{heads} heads are not a multiple of {groups} groups")
        if (heads * head_dim) % norm_groups:
            raise ValueError(f"{heads * head_dim} inner values do not cut into {norm_groups} equal parts")
        if not 1 <= conv <= ops.CONV_MAX_TAPS:
            raise ValueError(f"a convolution of {conv} taps: 1 to {ops.CONV_MAX_TAPS}")
        self.hidden_size, self.heads, self.head_dim, self.state, self.groups = hidden_size, heads, head_dim, state, groups
        self.taps, self.norm_groups, self.norm_eps, self.prefix = conv, norm_groups, float(norm_eps), prefix
        self.names = {**DEFAULT_NAMES, **(names or {})}
        self.inner = heads * head_dim
        self.channels = self.inner + 2 * groups * state              # x | B | C
        self.carry = (conv - 1) * self.channels                       # the convolution's part of the state row

    def _name(self, role: str) -> str:
        return f"{self.prefix}.{self.names[role]}"

    def cache_need(self):
        return StateNeed((self.carry + self.heads * self.state * self.head_dim,), torch.float32, graph_safe=True)

    def weights(self) -> List[WeightDecl]:
        H, small = self.hidden_size, dict(keep_fp32=True)
        return [WeightDecl(self._name("in"), (self.inner + self.channels + self.heads, H)),
                WeightDecl(self._name("conv"), (self.channels, self.taps), **small),
                WeightDecl(self._name("conv_bias"), (self.channels,), **small),
                WeightDecl(self._name("dt_bias"), (self.heads,), **small),
                WeightDecl(self._name("a_log"), (self.heads,), **small),
                WeightDecl(self._name("d"), (self.heads,), **small),
                WeightDecl(self._name("norm"), (self.inner,), init="gain", **small),
                WeightDecl(self._name("out"), (H, self.inner))]

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        get = lambda role: tensors[self._name(role)].contiguous()       # noqa: E731
        self.w_in, self.w_out = get("in"), get("out")
        self.conv_w, self.conv_b = get("conv"), get("conv_bias")
        self.dt_bias, self.a_log, self.d_skip, self.norm_gain = get("dt_bias"), get("a_log"), get("d"), get("norm")

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        proj = linear(x, self.w_in, out_dtype=torch.float32)             # z | x | B | C | dt
        rows = cache.state.view(cache.state.shape[0], -1)
        xbc = ops.conv_silu(proj, self.inner, self.channels, self.conv_w, self.conv_b, rows, ctx.token_entry,
                            ctx.q_start, ctx.entry_slot, ctx.num_entries, update_carry=cache.owner)
        y = ops.ssm_scan(xbc, proj, self.inner + self.channels, self.dt_bias, self.a_log, self.d_skip, rows, self.carry,
                         ctx.q_start, ctx.entry_slot, ctx.num_entries, self.heads, self.groups, self.state,
                         self.head_dim, write_state=cache.owner)
        gated = ops.gated_group_norm(y, proj, 0, self.norm_gain, self.norm_eps, self.norm_groups, ctx.dtype)
        return linear_into_stream(gated, self.w_out, ctx)
