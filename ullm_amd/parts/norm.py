"""RMS norm fused with the residual add (reference: ullm/layers/layernorm.py:15-34).

The reference carries the residual in the model dtype and rounds the 32-bit sum once per add
(layernorm.py:25-26); here the residual stream itself stays 32-bit, so the sum is never rounded.
The gain is held in 32-bit (the reference promotes it for the multiply, layernorm.py:30).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import Norm, NormedBranch, PartEnv, PendingNorm, WeightDecl, register_part


@register_part("norm", "rmsnorm")
class RMSNorm(Norm):
    adds_stacks = True

    def __init__(self, size: int, eps: float, weight_name: str):
        self.size = size
        self.eps = float(eps)
        self.weight_name = weight_name
        self.gain: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightDecl]:
        return [WeightDecl(self.weight_name, (self.size,), init="gain", keep_fp32=True)]

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        self.gain = tensors[self.weight_name].contiguous()

    def add_norm(self, branch, residual, rows=None, out_dtype=None):
        if isinstance(branch, NormedBranch):
            return add_normed_branch(branch, residual, self.kernel_form(), rows, out_dtype)
        if out_dtype is None:
            out_dtype = branch.dtype if branch is not None and branch.dim() == 2 else torch.float32
        return ops.add_rmsnorm(branch, residual, self.gain, self.eps, out_dtype, rows=rows)

    def kernel_form(self):
        return self.gain, self.eps, ops.NORM_RMS

    def pending(self, residual, out_dtype, scaled=None, squares=None):
        return PendingNorm(self, residual, self.gain, self.eps, out_dtype, scaled, squares)

    def ahead_gain(self):
        return self.gain


def add_normed_branch(branch: NormedBranch, residual, form, rows, out_dtype):
    """The stream takes ``mult * post(branch)`` and is normed by ``form`` = (gain, eps, kind), in one kernel."""
    gain, eps, kind = form
    if branch.post is None:                    # the branch joins the stream times the multiplier, unnormed
        post_gain, post_eps, post_kind = None, 0.0, ops.NORM_RMS
    else:
        post = branch.post.kernel_form()
        if post is None:
            raise TypeError(f"{type(branch.post).__name__} cannot stand behind a branch: it has no kernel form")
        post_gain, post_eps, post_kind = post
    return ops.add_norm_general(branch.branch, residual, gain, eps, kind, out_dtype or branch.branch.dtype, rows=rows,
                                post_gain=post_gain, post_eps=post_eps, post_kind=post_kind, mult=branch.mult)


@register_part("norm", "layernorm")
class LayerNorm(Norm):
    """(x - mean) / sqrt(mean of squared deviations + eps) * gain, no bias; computed in 32-bit."""

    def __init__(self, size: int, eps: float, weight_name: str):
        self.size = size
        self.eps = float(eps)
        self.weight_name = weight_name
        self.gain: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightDecl]:
        return [WeightDecl(self.weight_name, (self.size,), init="gain", keep_fp32=True)]

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        self.gain = tensors[self.weight_name].contiguous()

    def kernel_form(self):
        return self.gain, self.eps, ops.NORM_LAYER

    def add_norm(self, branch, residual, rows=None, out_dtype=None):
        if isinstance(branch, NormedBranch):
            return add_normed_branch(branch, residual, self.kernel_form(), rows, out_dtype)
        if branch is not None and branch.dim() == 3:
            branch = branch.sum(0)
        if out_dtype is None:
            out_dtype = branch.dtype if branch is not None else torch.float32
        return ops.add_norm_general(branch, residual, self.gain, self.eps, ops.NORM_LAYER, out_dtype, rows=rows)
