"""Triangle multiplication and triangle attention on the gfx950 kernels.

Same classes, constructor arguments, parameter names and forward signatures as
protenix/model/triangular/triangular.py:93-197, 470-586 (TriangleMultiplicative
Update and its Outgoing/Incoming flavours) and :589-727 (TriangleAttention),
with the attention sub-module of protenix/model/triangular/layers.py:299-473
kept as the parameter container `mha`.  The kernel-selection strings of the
reference are accepted and validated; every valid value runs the HIP kernels.
Forward only; widths: c_z = 64 or 128 with c_hidden = 128 and 4 heads x 32, or (bf16, also
fp32 tensors under bf16 autocast) c_z = c_hidden = 256 with 8 heads x 32.  Anything else is
refused by the library with an "unsupported shape" error.
"""
from __future__ import annotations

from typing import List, Optional

import torch
import torch.nn as nn

from . import ops
from .layer_norm import LayerNorm, _forward_only
from .primitives import Linear, _cv, _WeightCache


def OpenfoldLinear(in_dim: int, out_dim: int, bias: bool = True, init: str = "default") -> Linear:
    """layers.py:104-197 by its `init` names."""
    if init not in ("default", "relu", "gating", "final"):
        raise ValueError("Invalid init string.")
    return Linear(in_dim, out_dim, bias=bias, initializer=init)


def _stream_and_compute_dtype(z: torch.Tensor, c_z: int):
    """(rows to hand to the kernels, arithmetic dtype, dtype to cast a returned update to).
    fp32 rows under torch.autocast(bfloat16): rows of 64 / 128 channels stay fp32 and the
    kernels run bf16 arithmetic on them (the fused fp32 residual stream); wider rows are
    rounded to the autocast dtype first."""
    ac = ops.autocast_compute_dtype(z)
    if ac is None:
        return z, z.dtype, None
    cd = ops.compute_dtype(z)
    if cd == z.dtype:          # no fused kernel for this width / autocast dtype
        return z.to(ac), ac, None
    return z, cd, cd


def _per_batch(z: torch.Tensor, mask: Optional[torch.Tensor]):
    """[*, N, N, C] -> list of ([N, N, C], [N, N] or None) sharing storage with z."""
    if z.dim() < 3:
        raise RuntimeError(f"expected [*, N, N, C], got {tuple(z.shape)}")
    n, c = z.shape[-2], z.shape[-1]
    if z.shape[-3] != n:
        raise RuntimeError(f"pair tensor must be square, got {tuple(z.shape)}")
    zb = z.reshape(-1, n, n, c)
    mb = None
    if mask is not None:
        if mask.shape != z.shape[:-1]:
            mask = mask.expand(z.shape[:-1])
        mb = mask.reshape(-1, n, n)
    return zb, mb


def kernel_triangular_mult(x: torch.Tensor, direction: str, mask: Optional[torch.Tensor],
                           norm_in_weight: Optional[torch.Tensor], norm_in_bias: Optional[torch.Tensor],
                           p_in_weight: torch.Tensor, g_in_weight: torch.Tensor,
                           norm_out_weight: Optional[torch.Tensor], norm_out_bias: Optional[torch.Tensor],
                           p_out_weight: torch.Tensor, g_out_weight: torch.Tensor,
                           eps: float = 1e-5) -> torch.Tensor:
    """The reference's fused triangle-multiplication operator (triangular.py:26-90 and its
    call site :497-514) on the HIP kernels: x [*, N, N, c_z], mask [*, N, N] or None,
    p_in_weight / g_in_weight the stacked a / b projections and gates [2 * c_hidden, c_z],
    p_out_weight = linear_z.weight, g_out_weight = linear_g.weight.  Returns the update."""
    if direction not in ("outgoing", "incoming"):
        raise ValueError(f"direction must be 'outgoing' or 'incoming', but got {direction}")
    _forward_only(x, p_in_weight, g_in_weight, p_out_weight, g_out_weight, norm_in_weight, norm_in_bias,
                  norm_out_weight, norm_out_bias)
    z, cd, cast_back = _stream_and_compute_dtype(x, x.shape[-1])
    ps = [_cv(p, cd, z.device) for p in (norm_in_weight, norm_in_bias, p_in_weight, g_in_weight,
                                         norm_out_weight, norm_out_bias, p_out_weight, g_out_weight)]
    src = z if z.is_contiguous() else z.contiguous()
    zb, mb = _per_batch(src, mask)
    out = torch.stack([ops.triangle_multiplicative_update(
        zb[i], direction == "incoming", None if mb is None else mb[i], *ps, eps=eps)
        for i in range(zb.shape[0])]).view(src.shape)
    return out.to(cast_back) if cast_back is not None else out


triangle_multiplicative_update = kernel_triangular_mult


class TriangleMultiplicativeUpdate(nn.Module):
    """Algorithms 11 and 12 of AF3 (triangular.py:172-570)."""

    def __init__(self, c_z: int, c_hidden: int, _outgoing: bool = True) -> None:
        super().__init__()
        self.c_z = c_z
        self.c_hidden = c_hidden
        self._outgoing = _outgoing
        self.linear_g = OpenfoldLinear(c_z, c_z, bias=False, init="gating")
        self.linear_z = OpenfoldLinear(c_hidden, c_z, bias=False, init="final")
        self.layer_norm_in = LayerNorm(c_z)
        self.layer_norm_out = LayerNorm(c_hidden)
        self.sigmoid = nn.Sigmoid()
        self.linear_a_p = OpenfoldLinear(c_z, c_hidden, bias=False)
        self.linear_a_g = OpenfoldLinear(c_z, c_hidden, bias=False, init="gating")
        self.linear_b_p = OpenfoldLinear(c_z, c_hidden, bias=False)
        self.linear_b_g = OpenfoldLinear(c_z, c_hidden, bias=False, init="gating")
        self._cache = _WeightCache()

    def _weights(self, dtype, device) -> dict:
        ps = (self.layer_norm_in.weight, self.layer_norm_in.bias, self.layer_norm_out.weight,
              self.layer_norm_out.bias, self.linear_a_p.weight, self.linear_a_g.weight,
              self.linear_b_p.weight, self.linear_b_g.weight, self.linear_z.weight,
              self.linear_g.weight)
        names = ("ln_in_w", "ln_in_b", "ln_out_w", "ln_out_b", "w_ap", "w_ag", "w_bp", "w_bg",
                 "w_z", "w_g")
        return self._cache.get(ps, dtype, device,
                               lambda: dict(zip(names, (_cv(p, dtype, device) for p in ps))))

    def forward(self, z: torch.Tensor, mask: Optional[torch.Tensor] = None,
                inplace_safe: bool = False, _add_with_inplace: bool = False,
                _inplace_chunk_size: Optional[int] = 256,
                triangle_multiplicative: str = "torch") -> torch.Tensor:
        """z [*, N, N, c_z], mask [*, N, N] -> update [*, N, N, c_z]; with
        `inplace_safe and _add_with_inplace` z is overwritten with z + update and
        returned (triangular.py:470-566)."""
        if triangle_multiplicative not in ("torch", "cuequivariance"):
            raise ValueError(
                "triangle_multiplicative must be 'cuequivariance' or 'torch', but got "
                f"{triangle_multiplicative}")
        _forward_only(z, module=self)
        add_inplace = bool(inplace_safe and _add_with_inplace)
        z_in = z
        z, cd, cast_back = _stream_and_compute_dtype(z, self.c_z)
        if z is not z_in and add_inplace:
            # rows rounded for the kernels: the update is added to the caller's own rows
            return z_in.add_(self.forward(z_in, mask=mask))
        w = self._weights(cd, z.device)
        src = z if z.is_contiguous() else z.contiguous()
        zb, mb = _per_batch(src, mask)
        out = src if add_inplace else torch.empty_like(src)
        ob = out.view(zb.shape)
        for bi in range(zb.shape[0]):
            ops.triangle_multiplication(zb[bi], None if mb is None else mb[bi], w,
                                        incoming=not self._outgoing, add_residual=add_inplace,
                                        out=ob[bi])
        if add_inplace and out is not z:
            z.copy_(out)
            return z
        # (an update computed on fp32 rows under autocast holds bf16 values: returned as the
        # autocast dtype, like the reference's linear_z output)
        return out.to(cast_back) if (cast_back is not None and not add_inplace) else out


class TriangleMultiplicationOutgoing(TriangleMultiplicativeUpdate):
    """Algorithm 11."""

    def __init__(self, c_z: int, c_hidden: int) -> None:
        super().__init__(c_z=c_z, c_hidden=c_hidden, _outgoing=True)


class TriangleMultiplicationIncoming(TriangleMultiplicativeUpdate):
    """Algorithm 12."""

    def __init__(self, c_z: int, c_hidden: int) -> None:
        super().__init__(c_z=c_z, c_hidden=c_hidden, _outgoing=False)


class Attention(nn.Module):
    """Parameter container with the names of layers.py:299-359; the arithmetic
    lives in TriangleAttention.forward (fused kernels)."""

    def __init__(self, c_q: int, c_k: int, c_v: int, c_hidden: int, no_heads: int,
                 gating: bool = True) -> None:
        super().__init__()
        self.c_q, self.c_k, self.c_v = c_q, c_k, c_v
        self.c_hidden = c_hidden
        self.no_heads = no_heads
        self.gating = gating
        self.linear_q = OpenfoldLinear(c_q, c_hidden * no_heads, bias=False)
        self.linear_k = OpenfoldLinear(c_k, c_hidden * no_heads, bias=False)
        self.linear_v = OpenfoldLinear(c_v, c_hidden * no_heads, bias=False)
        self.linear_o = OpenfoldLinear(c_hidden * no_heads, c_q, bias=False, init="final")
        self.linear_g = None
        if gating:
            self.linear_g = OpenfoldLinear(c_q, c_hidden * no_heads, bias=False, init="gating")
        self.sigmoid = nn.Sigmoid()

    def forward(self, *args, **kwargs):
        raise RuntimeError(
            "protenix_amd: the triangle-attention sub-module is fused into "
            "TriangleAttention.forward and cannot be called on its own")


class TriangleAttention(nn.Module):
    """Algorithms 13 / 14 of AF3 (triangular.py:589-715)."""

    def __init__(self, c_in: int, c_hidden: int, no_heads: int, starting: bool = True,
                 inf: float = 1e9) -> None:
        super().__init__()
        self.c_in = c_in
        self.c_hidden = c_hidden
        self.no_heads = no_heads
        self.starting = starting
        self.inf = inf
        self.layer_norm = LayerNorm(c_in)
        self.linear = OpenfoldLinear(c_in, no_heads, bias=False)
        self.mha = Attention(c_in, c_in, c_in, c_hidden, no_heads)
        self._cache = _WeightCache()

    def _weights(self, dtype, device) -> dict:
        m = self.mha
        ps = (self.layer_norm.weight, self.layer_norm.bias, m.linear_q.weight, m.linear_k.weight,
              m.linear_v.weight, m.linear_g.weight, self.linear.weight, m.linear_o.weight)
        names = ("ln_w", "ln_b", "w_q", "w_k", "w_v", "w_g", "w_b", "w_o")
        return self._cache.get(ps, dtype, device,
                               lambda: dict(zip(names, (_cv(p, dtype, device) for p in ps))))

    def _run(self, x: torch.Tensor, mask: Optional[torch.Tensor], transposed: bool,
             residual_inplace: bool, then_transition=None):
        """`then_transition`: a callable (arithmetic dtype, device) -> the dict of
        ops.triangle_attention(then_transition=...), for a contiguous x updated in place where
        ops.fuses_attention_transition() holds; the result is then (x, list of pair biases or
        Nones, one per pair tensor of the batch)."""
        _forward_only(x, module=self)
        x_in = x
        x, cd, cast_back = _stream_and_compute_dtype(x, self.c_in)
        if then_transition is not None:
            assert residual_inplace and x is x_in and x.is_contiguous()
            w = self._weights(cd, x.device)
            tt = then_transition(cd, x.device)
            xb, mb = _per_batch(x, mask)
            biases = [ops.triangle_attention(xb[bi], None if mb is None else mb[bi], w, self.no_heads,
                                             self.c_hidden, self.inf, transposed=transposed,
                                             add_residual=True, out=xb[bi], then_transition=tt)[1]
                      for bi in range(xb.shape[0])]
            return x, biases
        if residual_inplace and x is not x_in:
            # rows rounded for the kernels: the update is added to the caller's own rows
            return x_in.add_(self._run(x_in, mask, transposed, residual_inplace=False))
        w = self._weights(cd, x.device)
        src = x if x.is_contiguous() else x.contiguous()
        xb, mb = _per_batch(src, mask)
        out = src if residual_inplace else torch.empty_like(src)
        ob = out.view(xb.shape)
        for bi in range(xb.shape[0]):
            ops.triangle_attention(xb[bi], None if mb is None else mb[bi], w, self.no_heads,
                                   self.c_hidden, self.inf, transposed=transposed,
                                   add_residual=residual_inplace, out=ob[bi])
        if residual_inplace and out is not x:
            x.copy_(out)
            return x
        return out.to(cast_back) if (cast_back is not None and not residual_inplace) else out

    def forward(self, x: torch.Tensor, mask: Optional[torch.Tensor] = None,
                chunk_size: Optional[int] = None, triangle_attention: str = "torch",
                inplace_safe: bool = False) -> torch.Tensor:
        """x [*, I, J, c_in], mask [*, I, J] -> update [*, I, J, c_in].  Keys are
        masked per row with inf*(mask-1); `chunk_size` only bounds memory in the
        reference (rows are independent) and is not needed here, since the logits
        are never materialised."""
        assert triangle_attention in ("torch", "deepspeed", "triattention", "cuequivariance")
        return self._run(x, mask, transposed=not self.starting, residual_inplace=False)


TriangleAttentionStartingNode = TriangleAttention


class TriangleAttentionEndingNode(TriangleAttention):
    """Algorithm 14."""

    def __init__(self, c_in: int, c_hidden: int, no_heads: int, inf: float = 1e9) -> None:
        super().__init__(c_in, c_hidden, no_heads, starting=False, inf=inf)
