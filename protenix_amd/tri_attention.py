"""The fused triangle-attention operator on standard-layout tensors.

Mirrors protenix/model/tri_attention/op.py:37-77 (`TriAttentionFunction`: Q, K, V
[B, N, S, H, D], Bias1 [B, N, 1, 1, S], Bias2 [B, 1, H, S, S] -> O [B, N, S, H, D]) and its caller
protenix/model/triangular/layers.py:539-583 (`_tri_attention`: q, k, v [*, H, Q, C] and a list of
two biases).  Forward only (inference); the N^3 logits are never materialised.  Runs the same
attention core as `TriangleAttention`, behind a repack of the operands into the core's tile
order, so it costs one extra pass over Q, K, V compared with the fused module.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from . import _lib, ops
from .layer_norm import _forward_only


def tri_attention_forward(Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor,
                          Bias1: Optional[torch.Tensor], Bias2: torch.Tensor,
                          return_lse: bool = False):
    """O (and, with `return_lse`, M [B, N, S, H] fp32: log2 of the softmax denominator in
    base-2 logits, as the reference's kernel stores it, forward.py:185-188)."""
    _forward_only(Q, K, V, module=None)
    ops._dev(Q, "Q")
    if Q.dim() != 5:
        raise RuntimeError(f"expected Q of shape [B, N, S, H, D], got {tuple(Q.shape)}")
    B, N, S, H, D = Q.shape
    if K.shape != Q.shape or V.shape != Q.shape:
        raise RuntimeError("Q, K and V must have the same shape")
    dt = Q.dtype
    Q, K, V = (t.to(dt).contiguous() for t in (Q, K, V))
    b2 = Bias2.to(dt).expand(B, 1, H, S, S).contiguous()
    b1 = None if Bias1 is None else Bias1.to(dt).expand(B, N, 1, 1, S).contiguous()
    lib = _lib.load()
    O = torch.empty_like(Q)
    M = torch.empty((B, N, S, H), device=Q.device, dtype=torch.float32) if return_lse else None
    ws = ops._workspace((lib.ptx_triattn_core_workspace_elems(N, S, H),), dt, Q.device)
    with torch.cuda.device(Q.device):
        ops._call("triattn_core_fwd", lib.ptx_triattn_core_fwd, ops._ptr(Q), ops._ptr(K), ops._ptr(V),
                  ops._ptr(b1), ops._ptr(b2), ops._ptr(O), ops._ptr(M), ops._ptr(ws), B, N, S, H, D,
                  ops._dt(Q), ops._stream())
    return (O, M) if return_lse else O


class TriAttentionFunction:
    """Call-compatible with the reference's autograd function for inference:
    `TriAttentionFunction.apply(Q, K, V, Bias1, Bias2, deterministic=False) -> O`."""

    @staticmethod
    def apply(Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, Bias1: torch.Tensor,
              Bias2: torch.Tensor, deterministic: bool = False) -> torch.Tensor:
        return tri_attention_forward(Q, K, V, Bias1, Bias2)

    forward = apply


def tri_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                  biases: List[torch.Tensor]) -> torch.Tensor:
    """layers.py:539-583: q, k, v [*, H, Q, C_hidden] (q already scaled), biases = [mask bias
    broadcastable to [*, 1, 1, K], triangle bias broadcastable to [*, H, Q, K]] -> [*, Q, H, C]."""
    if len(biases) != 2:
        raise ValueError("tri_attention takes exactly two biases: the mask bias and the triangle bias")

    def five(x: torch.Tensor) -> torch.Tensor:
        nb = x.dim() - 3
        if nb < 2:
            return x.reshape(*((1,) * (2 - nb) + tuple(x.shape)))
        if nb > 2:
            return x.reshape(x.shape[0], -1, *x.shape[-3:])
        return x

    q, k, v = (t.transpose(-2, -3) for t in (q, k, v))      # [*, Q, H, C]
    shape = q.shape
    o = tri_attention_forward(five(q), five(k), five(v), five(biases[0]), five(biases[1]))
    return o.reshape(shape)
