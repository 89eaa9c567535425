"""LayerNorm over the last dimension on the HIP kernel.

Mirrors protenix/model/layer_norm/layer_norm.py:190-233 (FusedLayerNorm) and
the factory protenix/model/triangular/layers.py:246-256: parameters `weight`
and `bias` (either may be absent), fp32 statistics, gamma/beta cast to the
input dtype, output in the input dtype.  Forward and backward
(FusedLayerNormAffineFunction, layer_norm.py:69-187) both run on HIP kernels.
"""
from __future__ import annotations

import numbers
from typing import Optional, Union

import torch
import torch.nn as nn

from . import ops


def _forward_only(*tensors: Optional[torch.Tensor], module: Optional[nn.Module] = None) -> None:
    """Refuses inputs (and, with `module`, parameters) that would need a backward pass.
    Under torch.no_grad() nothing is inspected: the parameter walk is not free."""
    if not torch.is_grad_enabled():
        return
    if module is not None:
        tensors = tensors + tuple(module.parameters())
    if any(t is not None and t.requires_grad for t in tensors):
        raise RuntimeError(
            "protenix_amd kernels are forward-only: call under torch.no_grad() "
            "(backward kernels are not part of this build)")


class FusedLayerNormAffineFunction(torch.autograd.Function):
    """layer_norm.py:69-187: forward keeps the fp32 row statistics for the backward kernel;
    weight / bias may be None."""

    @staticmethod
    def forward(ctx, input, weight, bias, normalized_shape, eps):  # noqa: A002
        ctx.normalized_shape = normalized_shape
        ctx.eps = eps
        input_ = input.contiguous()
        output, mean, invvar = ops.layer_norm(input_, weight, bias, eps, return_stats=True)
        ctx.save_for_backward(input_, weight, bias, mean, invvar)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        input_, weight_, bias_, mean, invvar = ctx.saved_tensors
        need = ctx.needs_input_grad
        grad_input, grad_weight, grad_bias = ops.layer_norm_backward(
            grad_output, input_, mean, invvar, weight_,
            need_weight=weight_ is not None and need[1], need_bias=bias_ is not None and need[2])
        return grad_input if need[0] else None, grad_weight, grad_bias, None, None


class FusedLayerNorm(nn.Module):
    def __init__(self, normalized_shape: Union[int, list, torch.Size], create_scale: bool = True,
                 create_offset: bool = True, eps: float = 1e-5) -> None:
        super().__init__()
        if isinstance(normalized_shape, numbers.Integral):
            normalized_shape = (normalized_shape,)
        self.normalized_shape = torch.Size(normalized_shape)
        if len(self.normalized_shape) != 1:
            raise ValueError("FusedLayerNorm normalises over the last dimension only")
        self.eps = eps
        if create_scale:
            self.weight = nn.Parameter(torch.ones(*normalized_shape))
        else:
            self.register_parameter("weight", None)
        if create_offset:
            self.bias = nn.Parameter(torch.zeros(*normalized_shape))
        else:
            self.register_parameter("bias", None)

    def reset_parameters(self) -> None:
        if self.weight is not None:
            nn.init.ones_(self.weight)
        if self.bias is not None:
            nn.init.zeros_(self.bias)

    def forward(self, input: torch.Tensor) -> torch.Tensor:  # noqa: A002
        if input.shape[-1] != self.normalized_shape[0]:
            raise RuntimeError(
                f"expected last dimension {self.normalized_shape[0]}, got {tuple(input.shape)}")
        if torch.is_grad_enabled() and any(
                t is not None and t.requires_grad for t in (input, self.weight, self.bias)):
            return FusedLayerNormAffineFunction.apply(input, self.weight, self.bias,
                                                      self.normalized_shape, self.eps)
        return ops.layer_norm(input, self.weight, self.bias, self.eps)

    def extra_repr(self) -> str:
        return f"{tuple(self.normalized_shape)}, eps={self.eps}"


def LayerNorm(c_in: int, create_scale: bool = True, create_offset: bool = True,
              eps: float = 1e-5) -> nn.Module:
    """Same call as the reference factory (layers.py:246-256)."""
    return FusedLayerNorm(c_in, create_scale=create_scale, create_offset=create_offset, eps=eps)
