"""Single-representation attention with pair bias, the has_s=False flavour the
Pairformer block uses (protenix/model/modules/transformer.py:40-254 with
pairformer.py:98-100; attention arithmetic of primitives.py:233-291, 636-879).

The only pass over the pair tensor - LayerNorm(z) followed by the c_z -> heads
projection - runs on the fused HIP kernel and never materialises LN(z).  The
rest lives on the [N, c_s] single track, on HIP kernels as well: LayerNorm, one
stacked projection, a flash-style attention that streams the pair bias and never
materialises the [heads, N, N] logits, and the output projection.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn

from . import ops
from .layer_norm import LayerNorm, _forward_only
from .primitives import Linear, LinearNoBias, _cv, _WeightCache


class Attention(nn.Module):
    """primitives.py:636-879 restricted to global attention with an additive
    bias: q carries a bias, output gated by sigmoid(linear_g(q_x))."""

    def __init__(self, c_q: int, c_k: int, c_v: int, c_hidden: int, num_heads: int,
                 gating: bool = True, q_linear_bias: bool = True,
                 local_attention_method: str = "global_attention_with_bias",
                 use_efficient_implementation: bool = True, zero_init: bool = True) -> None:
        super().__init__()
        self.c_q, self.c_k, self.c_v = c_q, c_k, c_v
        self.c_hidden = c_hidden
        self.num_heads = num_heads
        self.gating = gating
        self.linear_q = Linear(c_q, c_hidden * num_heads, bias=q_linear_bias)
        self.linear_k = LinearNoBias(c_k, c_hidden * num_heads)
        self.linear_v = LinearNoBias(c_v, c_hidden * num_heads)
        self.linear_o = LinearNoBias(c_hidden * num_heads, c_q)
        self.linear_g = None
        if gating:
            self.linear_g = LinearNoBias(c_q, c_hidden * num_heads, initializer="zeros")
            self.sigmoid = nn.Sigmoid()
        self.zero_init = zero_init
        if zero_init:
            nn.init.zeros_(self.linear_o.weight)
        self._cache_in = _WeightCache()
        self._cache_out = _WeightCache()

    def _fused_in(self, dtype, device):
        """q, k, gate and v projections of one input as a single GEMM: the four weights
        stacked in that order (v last: its columns leave the kernel transposed, which is how
        the attention kernel reads them) and the q bias, built once per weight set."""
        ps = (self.linear_q.weight, self.linear_q.bias, self.linear_k.weight, self.linear_g.weight,
              self.linear_v.weight)

        def make():
            wq, bq, wk, wg, wv = (_cv(p, dtype, device) for p in ps)
            return torch.cat([wq, wk, wg, wv], 0).contiguous(), bq
        return self._cache_in.get(ps, dtype, device, make)

    def _check_supported(self, q_x: torch.Tensor, kv_x: torch.Tensor) -> None:
        """The HIP kernels cover self-attention with a gate on float32 / bfloat16 GPU tensors,
        c_q a multiple of 16, head width 8, 16, 24 or 32 and 3 * heads * width a multiple of 32
        (the transposed tail of the stacked projection).  Anything else raises: no library
        GEMM or softmax stands in."""
        why = None
        if q_x is not kv_x:
            why = "q_x and kv_x must be the same tensor (self-attention)"
        elif any(l is None or l.precision is not None for l in
                 (self.linear_q, self.linear_k, self.linear_v, self.linear_g, self.linear_o)):
            why = "needs the gate and linear layers without a `precision` override"
        elif not (self.c_q == self.c_k == self.c_v and self.c_q % 16 == 0):
            why = f"c_q = c_k = c_v, a multiple of 16 (got {self.c_q}, {self.c_k}, {self.c_v})"
        elif not (self.c_hidden % 8 == 0 and self.c_hidden <= 32
                  and (3 * self.num_heads * self.c_hidden) % 32 == 0):
            why = (f"head width 8, 16, 24 or 32 with 3 * heads * width a multiple of 32 "
                   f"(got {self.num_heads} x {self.c_hidden})")
        elif q_x.dtype not in (torch.float32, torch.bfloat16):
            why = f"float32 or bfloat16 tensors (got {q_x.dtype})"
        if why is not None:
            raise RuntimeError(f"protenix_amd.Attention: unsupported configuration: {why}")

    def forward(self, q_x: torch.Tensor, kv_x: torch.Tensor,
                attn_bias: Optional[torch.Tensor] = None, residual: Optional[torch.Tensor] = None,
                **_unused) -> torch.Tensor:
        """Attention update of q_x; with `residual`, residual + update (added in the output
        projection's epilogue).  Three HIP kernels per batch element: stacked projection
        (q | k | gate row-major, v transposed), flash-style attention with the pair bias and
        the gate, output projection (+ residual).  Logits and softmax are fp32 and never
        materialised (the reference upcasts q, k and the bias and relies on autocast for v,
        primitives.py:255-270; here v is fp32 in the kernel as well)."""
        _forward_only(q_x, attn_bias, residual, module=self)
        ops._dev(q_x, "q_x")
        self._check_supported(q_x, kv_x)
        H, d = self.num_heads, self.c_hidden
        w, bq = self._fused_in(q_x.dtype, q_x.device)
        w_o = self._cache_out.get((self.linear_o.weight,), q_x.dtype, q_x.device,
                                  lambda: _cv(self.linear_o.weight, q_x.dtype, q_x.device))
        n, c = q_x.shape[-2], q_x.shape[-1]
        xb = q_x.reshape(-1, n, c)
        if not xb.is_contiguous():
            xb = xb.contiguous()
        bb = None
        if attn_bias is not None:
            bb = attn_bias.expand(*q_x.shape[:-2], H, n, n).reshape(-1, H, n, n)
        outs = []
        for i in range(xb.shape[0]):
            qkg, vt = ops.linear_split(xb[i], w, bq, H * d, 3 * H * d)
            outs.append(ops.single_attention(qkg, vt, None if bb is None else bb[i], H, d,
                                             1.0 / math.sqrt(d)))
        o = outs[0] if len(outs) == 1 else torch.stack(outs)
        return ops.linear(o.view(*q_x.shape[:-1], H * d), w_o, res=residual)


class AttentionPairBias(nn.Module):
    def __init__(self, has_s: bool = True, create_offset_ln_z: bool = False, n_heads: int = 16,
                 c_a: int = 768, c_s: int = 384, c_z: int = 128, biasinit: float = -2.0,
                 cross_attention_mode: bool = False) -> None:
        super().__init__()
        if has_s or cross_attention_mode:
            raise NotImplementedError(
                "protenix_amd.AttentionPairBias covers the Pairformer-block flavour "
                "(has_s=False, cross_attention_mode=False); the diffusion-module flavours "
                "are outside this package")
        assert c_a % n_heads == 0
        self.n_heads = n_heads
        self.has_s = has_s
        self.create_offset_ln_z = create_offset_ln_z
        self.cross_attention_mode = cross_attention_mode
        self.layernorm_a = LayerNorm(c_a)
        self.local_attention_method = "local_cross_attention"
        self.attention = Attention(c_q=c_a, c_k=c_a, c_v=c_a, c_hidden=c_a // n_heads,
                                   num_heads=n_heads, gating=True, q_linear_bias=True,
                                   local_attention_method=self.local_attention_method,
                                   zero_init=not has_s)
        self.layernorm_z = LayerNorm(c_z, create_offset=create_offset_ln_z)
        self.linear_nobias_z = LinearNoBias(in_features=c_z, out_features=n_heads)
        self._cache = _WeightCache()

    def pair_bias_weights(self, z: torch.Tensor) -> tuple:
        """(LayerNorm weight, bias, projection [heads, c_z]) in the arithmetic type of z's kernels."""
        ps = (self.layernorm_z.weight, self.layernorm_z.bias, self.linear_nobias_z.weight)
        cd = ops.compute_dtype(z)     # bf16 for fp32 rows of 128 channels under bf16 autocast
        return self._cache.get(ps, cd, z.device, lambda: tuple(_cv(p, cd, z.device) for p in ps))

    def pair_bias(self, z: torch.Tensor) -> torch.Tensor:
        """[*, N, N, c_z] -> fp32 [*, heads, N, N] = permute(linear(LN(z)))
        (transformer.py:191-194)."""
        ln_w, ln_b, w = self.pair_bias_weights(z)
        n, c = z.shape[-2], z.shape[-1]
        zb = z.contiguous().reshape(-1, n, n, c)
        out = torch.stack([ops.pair_bias(zb[i], ln_w, ln_b, w, out_f32=True)
                           for i in range(zb.shape[0])])
        return out.reshape(*z.shape[:-3], self.n_heads, n, n)

    def forward(self, a: torch.Tensor, s: Optional[torch.Tensor], z: torch.Tensor,
                n_queries: Optional[int] = None, n_keys: Optional[int] = None,
                inplace_safe: bool = False, chunk_size: Optional[int] = None,
                enable_efficient_fusion: bool = False) -> torch.Tensor:
        if n_queries or n_keys:
            raise NotImplementedError("local attention belongs to the diffusion module")
        return self.forward_with_bias(a, self.pair_bias(z))

    def forward_with_bias(self, a: torch.Tensor, bias: torch.Tensor,
                          residual: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The single-track part, given bias = pair_bias(z) (with `residual`: residual + update).
        Split off so that a caller can run it on another stream once the pass over z is done."""
        _forward_only(a, bias, module=self)
        a = self.layernorm_a(a)
        return self.attention(q_x=a, kv_x=a, attn_bias=bias, residual=residual)
