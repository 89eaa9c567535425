"""The fused triangle-attention operator on standard-layout tensors.

Mirrors protenix/model/tri_attention/op.py:37-77 (`TriAttentionFunction`: Q, K, V
[B, N, S, H, D], Bias1 [B, N, 1, 1, S], Bias2 [B, 1, H, S, S] -> O [B, N, S, H, D]) and its caller
protenix/model/triangular/layers.py:539-583 (`_tri_attention`: q, k, v [*, H, Q, C] and a list of
two biases), with the backward of op.py:79-163.  The N^3 logits are never materialised.  Runs the same
attention core as `TriangleAttention`, behind a repack of the operands into the core's tile
order, so it costs one extra pass over Q, K, V compared with the fused module.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from . import _lib, ops
from .layer_norm import _forward_only


def _core_forward(Q, K, V, b1, b2, want_lse: bool):
    """Q, K, V [B, N, S, H, D], b1 [B, N, 1, 1, S] or None, b2 [B, 1, H, S, S], all contiguous and
    of Q's dtype -> O and (optionally) M."""
    B, N, S, H, D = Q.shape
    lib = _lib.load()
    O = torch.empty_like(Q)
    M = torch.empty((B, N, S, H), device=Q.device, dtype=torch.float32) if want_lse else None
    ws = ops._workspace((lib.ptx_triattn_core_workspace_elems(N, S, H),), Q.dtype, Q.device)
    with torch.cuda.device(Q.device):
        ops._call("triattn_core_fwd", lib.ptx_triattn_core_fwd, ops._ptr(Q), ops._ptr(K), ops._ptr(V),
                  ops._ptr(b1), ops._ptr(b2), ops._ptr(O), ops._ptr(M), ops._ptr(ws), B, N, S, H, D,
                  ops._dt(Q), ops._stream())
    return O, M


def _canonical(Q, K, V, Bias1, Bias2):
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
    return Q, K, V, b1, b2


class TriAttentionFunction(torch.autograd.Function):
    """Call-compatible with the reference's autograd function (tri_attention/op.py:37-163):
    `TriAttentionFunction.apply(Q, K, V, Bias1, Bias2, deterministic=False) -> O`, with
    gradients for Q, K, V and Bias2.  Bias1 gets none: the reference hands back an
    uninitialised tensor for it (op.py:120), its Bias1 being the mask bias, so a Bias1 that
    requires a gradient is refused here instead.  The kernels use no atomics: every call is
    deterministic whatever the flag says."""

    @staticmethod
    def forward(ctx, Q, K, V, Bias1, Bias2, deterministic=False):
        if ctx.needs_input_grad[3]:
            raise RuntimeError("TriAttentionFunction forms no gradient for Bias1 (the mask bias)")
        q, k, v, b1, b2 = _canonical(Q.detach(), K.detach(), V.detach(),
                                     None if Bias1 is None else Bias1.detach(), Bias2.detach())
        O, M = _core_forward(q, k, v, b1, b2, want_lse=True)
        ctx.save_for_backward(q, k, v, b1, b2, O, M)
        ctx.in_dtypes = (Q.dtype, K.dtype, V.dtype, Bias2.dtype)
        ctx.b2_shape = tuple(Bias2.shape)
        return O

    @staticmethod
    def backward(ctx, DO):
        q, k, v, b1, b2, O, M = ctx.saved_tensors
        B, N, S, H, D = q.shape
        DO = DO.to(q.dtype).contiguous()
        DQ, DK, DV = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        want_b2 = ctx.needs_input_grad[4]
        DB2 = torch.empty_like(b2) if want_b2 else None
        delta = ops._workspace((N * S * H,), torch.float32, q.device)
        lib = _lib.load()
        with torch.cuda.device(q.device):
            ops._call("triattn_core_bwd", lib.ptx_triattn_core_bwd, ops._ptr(q), ops._ptr(k),
                      ops._ptr(v), ops._ptr(b1), ops._ptr(b2), ops._ptr(O), ops._ptr(M), ops._ptr(DO),
                      ops._ptr(DQ), ops._ptr(DK), ops._ptr(DV), ops._ptr(DB2), ops._ptr(delta),
                      B, N, S, H, D, ops._dt(q), ops._stream())
        dq_t, dk_t, dv_t, db2_t = ctx.in_dtypes
        if want_b2:
            DB2 = DB2.sum_to_size(ctx.b2_shape) if tuple(DB2.shape) != ctx.b2_shape else DB2
            DB2 = DB2.to(db2_t)
        return DQ.to(dq_t), DK.to(dk_t), DV.to(dv_t), None, DB2, None


def tri_attention_forward(Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor,
                          Bias1: Optional[torch.Tensor], Bias2: torch.Tensor,
                          return_lse: bool = False):
    """O (and, with `return_lse`, M [B, N, S, H] fp32: log2 of the softmax denominator in
    base-2 logits, as the reference's kernel stores it, forward.py:185-188).  With
    `return_lse` the call is forward-only; without it, operands that require a gradient go
    through `TriAttentionFunction`."""
    if return_lse:
        _forward_only(Q, K, V, Bias2, module=None)
        return _core_forward(*_canonical(Q, K, V, Bias1, Bias2), want_lse=True)
    if torch.is_grad_enabled() and any(t.requires_grad for t in (Q, K, V, Bias2)):
        return TriAttentionFunction.apply(Q, K, V, Bias1, Bias2)
    return _core_forward(*_canonical(Q, K, V, Bias1, Bias2), want_lse=False)[0]


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
