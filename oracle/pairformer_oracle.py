"""Plain-PyTorch restatement of the reference "torch" path of the Pairformer
pair stack.  TEST INFRASTRUCTURE: the checker for the HIP kernels and the CPU
baseline of ``bench.py``; the shipped package never imports it.

Every class keeps the reference's name, constructor arguments, parameter names
(state-dict keys) and ``forward`` signature, so a state dict moves between the
oracle, the HIP-backed modules and a reference checkpoint unchanged.

What pins each function (see tests/test_oracle_*.py):

* ``layer_norm``            -> ``torch.nn.LayerNorm`` + closed forms
                               (constant row -> beta, unit variance rows)
* ``layer_norm_backward``   -> autograd of ``F.layer_norm`` in fp64, central
                               differences, dx orthogonal to 1 and to x - mean
* ``linear``                -> ``torch.nn.functional.linear``
* triangle multiplication   -> ``torch.einsum`` + a triple-loop brute force on
                               tiny N, token-permutation equivariance,
                               outgoing/incoming transpose duality, mask-as-
                               token-deletion
* triangle attention        -> ``scaled_dot_product_attention`` per (row, head)
                               + brute-force softmax, fully masked row = mean
                               of V, masked keys are inert, chunked == unchunked
* ``Transition``            -> ``F.silu`` / explicit formula
* ``AttentionPairBias``     -> ``scaled_dot_product_attention`` with additive
                               mask, scale 1
* block / stack             -> composition; ``inplace_safe`` and ``chunk_size``
                               must not change the result

The reference holds no golden vectors for this path (its tests only check
shapes/contiguity of the block), so the pins above are the parity anchor.

dtype flow follows the reference: LayerNorm statistics in fp32 (torch does this
internally), gamma/beta and linear weights cast to the input dtype, every
intermediate stored in the input dtype.
"""

from __future__ import annotations

import math
from typing import List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F


# ----------------------------------------------------------------------------
# primitives
# ----------------------------------------------------------------------------
def layer_norm(
    x: torch.Tensor,
    weight: Optional[torch.Tensor],
    bias: Optional[torch.Tensor],
    eps: float = 1e-5,
) -> torch.Tensor:
    """y = (x - mean) * rsqrt(biased_var + eps) * gamma + beta over the last dim.

    Follows protenix/model/triangular/layers.py:224-243 (OpenFoldLayerNorm) and
    protenix/model/layer_norm/layer_norm.py:79-110 (gamma/beta cast to x.dtype).
    """
    d = x.dtype
    w = weight.to(d) if weight is not None else None
    b = bias.to(d) if bias is not None else None
    return F.layer_norm(x, (x.shape[-1],), w, b, eps)


def layer_norm_backward(
    dout: torch.Tensor,
    x: torch.Tensor,
    weight: Optional[torch.Tensor],
    eps: float = 1e-5,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dx, dgamma, dbeta) of layer_norm for upstream gradient dout, in the dtype of x.

    Follows the arithmetic of protenix/model/layer_norm/kernel/layer_norm_cuda_kernel.cu:672-716
    (grad_input = part1 - part2 - part3 in fp32) and :395-470 (parameter gradients: column
    sums of dout * (x - mean) * invvar and of dout); gamma cast to the gradient's dtype as
    layer_norm.py:114-176 does.  Arithmetic in fp32 (fp64 for fp64 inputs).
    """
    d = x.dtype
    f = torch.float64 if d == torch.float64 else torch.float32
    cols = x.shape[-1]
    xf, df = x.to(f), dout.to(d).to(f)
    g = weight.to(d).to(f) if weight is not None else torch.ones(cols, dtype=f)
    mean = xf.mean(-1, keepdim=True)
    invvar = torch.rsqrt(((xf - mean) ** 2).mean(-1, keepdim=True) + eps)
    xc = xf - mean
    gd = g * df
    part1 = gd * invvar
    part2 = gd.sum(-1, keepdim=True) * invvar / cols
    part3 = xc * ((gd * xc).sum(-1, keepdim=True) * invvar * invvar * invvar / cols)
    dx = part1 - part2 - part3
    red = tuple(range(x.dim() - 1))
    dgamma = (df * xc * invvar).sum(red) if red else df * xc * invvar
    dbeta = df.sum(red) if red else df
    return dx.to(d), dgamma.to(d), dbeta.to(d)


def linear(
    x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None
) -> torch.Tensor:
    """x @ W^T (+ b) with W cast to x.dtype.

    Follows protenix/model/triangular/layers.py:177-197 and
    protenix/model/modules/primitives.py:83-98.
    """
    b = bias.to(x.dtype) if bias is not None else None
    return F.linear(x, weight.to(x.dtype), b)


class LayerNorm(nn.Module):
    """Same constructor as the reference factory, layers.py:246-256."""

    def __init__(
        self,
        c_in: int,
        create_scale: bool = True,
        create_offset: bool = True,
        eps: float = 1e-5,
    ) -> None:
        super().__init__()
        self.c_in = (c_in,)
        self.eps = eps
        if create_scale:
            self.weight = nn.Parameter(torch.ones(c_in))
        else:
            self.register_parameter("weight", None)
        if create_offset:
            self.bias = nn.Parameter(torch.zeros(c_in))
        else:
            self.register_parameter("bias", None)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return layer_norm(x, self.weight, self.bias, self.eps)


class Linear(nn.Linear):
    """Bias handling of primitives.py:33-98 / layers.py:104-197, no init logic
    (the parity tests overwrite every parameter)."""

    def forward(self, input: torch.Tensor) -> torch.Tensor:  # noqa: A002
        return linear(input, self.weight, self.bias)


def LinearNoBias(in_features: int, out_features: int) -> Linear:
    return Linear(in_features, out_features, bias=False)


# ----------------------------------------------------------------------------
# triangle multiplication  (triangular.py:93-197, 470-586)
# ----------------------------------------------------------------------------
class TriangleMultiplicativeUpdate(nn.Module):
    def __init__(self, c_z: int, c_hidden: int, _outgoing: bool = True) -> None:
        super().__init__()
        self.c_z = c_z
        self.c_hidden = c_hidden
        self._outgoing = _outgoing
        self.linear_g = LinearNoBias(c_z, c_z)
        self.linear_z = LinearNoBias(c_hidden, c_z)
        self.layer_norm_in = LayerNorm(c_z)
        self.layer_norm_out = LayerNorm(c_hidden)
        self.linear_a_p = LinearNoBias(c_z, c_hidden)
        self.linear_a_g = LinearNoBias(c_z, c_hidden)
        self.linear_b_p = LinearNoBias(c_z, c_hidden)
        self.linear_b_g = LinearNoBias(c_z, c_hidden)

    def forward(
        self,
        z: torch.Tensor,
        mask: Optional[torch.Tensor] = None,
        inplace_safe: bool = False,
        _add_with_inplace: bool = False,
        _inplace_chunk_size: Optional[int] = 256,
        triangle_multiplicative: str = "torch",
    ) -> torch.Tensor:
        """triangular.py:519-566.  Returns the update, or z + update when
        ``inplace_safe and _add_with_inplace`` (the in-place variant at
        triangular.py:199-468 is a memory-only rewrite of the same values)."""
        if triangle_multiplicative not in ("torch", "cuequivariance"):
            raise ValueError(
                "triangle_multiplicative must be 'cuequivariance' or 'torch', "
                f"but got {triangle_multiplicative}"
            )
        if mask is None:
            mask = z.new_ones(z.shape[:-1])
        m = mask.unsqueeze(-1)
        zn = self.layer_norm_in(z)
        a = m * torch.sigmoid(self.linear_a_g(zn)) * self.linear_a_p(zn)
        b = m * torch.sigmoid(self.linear_b_g(zn)) * self.linear_b_p(zn)
        if self._outgoing:
            # x[i,j,c] = sum_k a[i,k,c] * b[j,k,c]      (triangular.py:129-131)
            x = torch.matmul(a.permute(*range(a.dim() - 3), -1, -3, -2),
                             b.permute(*range(b.dim() - 3), -1, -2, -3))
        else:
            # x[i,j,c] = sum_k a[k,i,c] * b[k,j,c]      (triangular.py:132-134)
            x = torch.matmul(a.permute(*range(a.dim() - 3), -1, -2, -3),
                             b.permute(*range(b.dim() - 3), -1, -3, -2))
        x = x.permute(*range(x.dim() - 3), -2, -1, -3)
        x = self.layer_norm_out(x)
        x = self.linear_z(x)
        x = x * torch.sigmoid(self.linear_g(zn))
        if inplace_safe and _add_with_inplace:
            x = x + z
        return x


class TriangleMultiplicationOutgoing(TriangleMultiplicativeUpdate):
    def __init__(self, c_z: int, c_hidden: int) -> None:
        super().__init__(c_z, c_hidden, _outgoing=True)


class TriangleMultiplicationIncoming(TriangleMultiplicativeUpdate):
    def __init__(self, c_z: int, c_hidden: int) -> None:
        super().__init__(c_z, c_hidden, _outgoing=False)


# ----------------------------------------------------------------------------
# triangle attention  (triangular.py:589-715; layers.py:276-296, 299-473)
# ----------------------------------------------------------------------------
def softmax_attention(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, biases: List[torch.Tensor]
) -> torch.Tensor:
    """softmax(q k^T + sum(biases)) v, biases added one by one in list order
    in the storage dtype (layers.py:276-296)."""
    a = torch.matmul(q, k.transpose(-1, -2))
    for b in biases:
        a = a + b
    a = torch.softmax(a, dim=-1)
    return torch.matmul(a, v)


class TriAttnMHA(nn.Module):
    """The gated multi-head attention of layers.py:299-473 (torch branch)."""

    def __init__(self, c_q: int, c_k: int, c_v: int, c_hidden: int, no_heads: int,
                 gating: bool = True) -> None:
        super().__init__()
        self.c_hidden = c_hidden
        self.no_heads = no_heads
        self.linear_q = LinearNoBias(c_q, c_hidden * no_heads)
        self.linear_k = LinearNoBias(c_k, c_hidden * no_heads)
        self.linear_v = LinearNoBias(c_v, c_hidden * no_heads)
        self.linear_o = LinearNoBias(c_hidden * no_heads, c_q)
        self.linear_g = LinearNoBias(c_q, c_hidden * no_heads) if gating else None

    def forward(self, q_x: torch.Tensor, kv_x: torch.Tensor,
                biases: Optional[List[torch.Tensor]] = None,
                triangle_attention: str = "torch") -> torch.Tensor:
        assert triangle_attention in ("torch", "deepspeed", "triattention",
                                      "cuequivariance")
        H = self.no_heads
        # [*, Q, H*D] -> [*, H, Q, D]
        q = self.linear_q(q_x).unflatten(-1, (H, -1)).transpose(-2, -3)
        k = self.linear_k(kv_x).unflatten(-1, (H, -1)).transpose(-2, -3)
        v = self.linear_v(kv_x).unflatten(-1, (H, -1)).transpose(-2, -3)
        q = q / math.sqrt(self.c_hidden)                     # layers.py:379-380
        o = softmax_attention(q, k, v, biases or [])         # [*, H, Q, D]
        o = o.transpose(-2, -3)                              # [*, Q, H, D]
        if self.linear_g is not None:
            g = torch.sigmoid(self.linear_g(q_x)).unflatten(-1, (H, -1))
            o = o * g
        return self.linear_o(o.flatten(-2))


class TriangleAttention(nn.Module):
    def __init__(self, c_in: int, c_hidden: int, no_heads: int,
                 starting: bool = True, inf: float = 1e9) -> None:
        super().__init__()
        self.c_in = c_in
        self.c_hidden = c_hidden
        self.no_heads = no_heads
        self.starting = starting
        self.inf = inf
        self.layer_norm = LayerNorm(c_in)
        self.linear = LinearNoBias(c_in, no_heads)
        self.mha = TriAttnMHA(c_in, c_in, c_in, c_hidden, no_heads)

    def forward(
        self,
        x: torch.Tensor,
        mask: Optional[torch.Tensor] = None,
        chunk_size: Optional[int] = None,
        triangle_attention: str = "torch",
        inplace_safe: bool = False,
    ) -> torch.Tensor:
        """triangular.py:657-715.  Keys are masked per row i with an additive
        inf*(mask-1); queries are never masked."""
        if mask is None:
            mask = x.new_ones(x.shape[:-1])
        if not self.starting:
            x = x.transpose(-2, -3)
            mask = mask.transpose(-1, -2)
        x = self.layer_norm(x)
        mask_bias = (self.inf * (mask - 1))[..., :, None, None, :]   # [*,I,1,1,J]
        tri_bias = self.linear(x)                                    # [*,I,J,H]
        tri_bias = tri_bias.permute(*range(tri_bias.dim() - 3), -1, -3, -2)
        tri_bias = tri_bias.unsqueeze(-4)                            # [*,1,H,I,J]
        if chunk_size is None:
            o = self.mha(x, x, [mask_bias, tri_bias], triangle_attention)
        else:
            # rows i are independent: chunking along I only bounds memory
            # (triangular.py:630-655, utils.py:693-815)
            outs = []
            I = x.shape[-3]
            for s in range(0, I, chunk_size):
                xs = x[..., s:s + chunk_size, :, :]
                outs.append(self.mha(xs, xs,
                                     [mask_bias[..., s:s + chunk_size, :, :, :],
                                      tri_bias], triangle_attention))
            o = torch.cat(outs, dim=-3)
        if not self.starting:
            o = o.transpose(-2, -3)
        return o


# ----------------------------------------------------------------------------
# transition  (primitives.py:166-230)
# ----------------------------------------------------------------------------
class Transition(nn.Module):
    def __init__(self, c_in: int, n: int) -> None:
        super().__init__()
        self.n = n
        self.c_in = c_in
        self.layernorm1 = LayerNorm(c_in)
        self.linear_no_bias_a = LinearNoBias(c_in, n * c_in)
        self.linear_no_bias_b = LinearNoBias(c_in, n * c_in)
        self.linear_no_bias = LinearNoBias(n * c_in, c_in)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """silu(W_a LN(x)) * (W_b LN(x)) -> W_o.  The reference's eval path
        splits rows into 8 chunks for long inputs (primitives.py:206-230):
        rows are independent, the values are the same."""
        y = self.layernorm1(x)
        rows = y.reshape(-1, y.shape[-1])
        n_chunk = 1 if x.shape[-2] < 3200 else 8
        outs = []
        for part in torch.chunk(rows, n_chunk, dim=0):
            h = F.silu(self.linear_no_bias_a(part)) * self.linear_no_bias_b(part)
            outs.append(self.linear_no_bias(h))
        return torch.cat(outs, dim=0).reshape(x.shape)


# ----------------------------------------------------------------------------
# single attention with pair bias, has_s=False
# (transformer.py:40-254, primitives.py:233-291, 636-879)
# ----------------------------------------------------------------------------
class SingleAttention(nn.Module):
    """primitives.py Attention as instantiated by AttentionPairBias: q has a
    bias, gating on, global attention with an additive bias."""

    def __init__(self, c_q: int, c_k: int, c_v: int, c_hidden: int,
                 num_heads: int) -> None:
        super().__init__()
        self.c_hidden = c_hidden
        self.num_heads = num_heads
        self.linear_q = Linear(c_q, c_hidden * num_heads, bias=True)
        self.linear_k = LinearNoBias(c_k, c_hidden * num_heads)
        self.linear_v = LinearNoBias(c_v, c_hidden * num_heads)
        self.linear_o = LinearNoBias(c_hidden * num_heads, c_q)
        self.linear_g = LinearNoBias(c_q, c_hidden * num_heads)

    def forward(self, q_x: torch.Tensor, kv_x: torch.Tensor,
                attn_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        H = self.num_heads
        q = self.linear_q(q_x).unflatten(-1, (H, -1)).transpose(-2, -3)
        k = self.linear_k(kv_x).unflatten(-1, (H, -1)).transpose(-2, -3)
        v = self.linear_v(kv_x).unflatten(-1, (H, -1)).transpose(-2, -3)
        q = q / math.sqrt(self.c_hidden)                     # primitives.py:750-751
        # q, k and the bias are upcast to fp32 (primitives.py:255-260).  The
        # reference leaves v in the storage dtype, which only works under
        # torch.autocast; here v is upcast too and the result cast back.
        d = q.dtype
        w = torch.matmul(q.float(), k.float().transpose(-1, -2))
        if attn_bias is not None:
            w = w + attn_bias.float()
        w = torch.softmax(w, dim=-1)
        o = torch.matmul(w, v.float()).to(d)                 # [*, H, Q, D]
        o = o.transpose(-2, -3)
        g = torch.sigmoid(self.linear_g(q_x)).unflatten(-1, (H, -1))
        return self.linear_o((o * g).flatten(-2))


class AttentionPairBias(nn.Module):
    """Only the has_s=False flavour used by PairformerBlock
    (pairformer.py:98-100)."""

    def __init__(self, has_s: bool = True, create_offset_ln_z: bool = False,
                 n_heads: int = 16, c_a: int = 768, c_s: int = 384,
                 c_z: int = 128, biasinit: float = -2.0,
                 cross_attention_mode: bool = False) -> None:
        super().__init__()
        if has_s or cross_attention_mode:
            raise NotImplementedError(
                "oracle covers AttentionPairBias(has_s=False) only")
        assert c_a % n_heads == 0
        self.n_heads = n_heads
        self.has_s = has_s
        self.layernorm_a = LayerNorm(c_a)
        self.attention = SingleAttention(c_a, c_a, c_a, c_a // n_heads, n_heads)
        self.layernorm_z = LayerNorm(c_z, create_offset=create_offset_ln_z)
        self.linear_nobias_z = LinearNoBias(c_z, n_heads)

    def forward(self, a: torch.Tensor, s: Optional[torch.Tensor],
                z: torch.Tensor, **_unused) -> torch.Tensor:
        a = self.layernorm_a(a)
        bias = self.linear_nobias_z(self.layernorm_z(z))      # [*, N, N, H]
        bias = bias.permute(*range(bias.dim() - 3), -1, -3, -2)
        return self.attention(a, a, attn_bias=bias)


# ----------------------------------------------------------------------------
# block and stack  (pairformer.py:42-340)
# ----------------------------------------------------------------------------
class PairformerBlock(nn.Module):
    def __init__(self, n_heads: int = 16, c_z: int = 128, c_s: int = 384,
                 c_hidden_mul: int = 128, c_hidden_pair_att: int = 32,
                 no_heads_pair: int = 4, num_intermediate_factor: int = 4,
                 dropout: float = 0.25, hidden_scale_up: bool = False) -> None:
        super().__init__()
        self.n_heads = n_heads
        if hidden_scale_up:
            no_heads_pair = c_z // c_hidden_pair_att
            c_hidden_mul = c_z
        self.tri_mul_out = TriangleMultiplicationOutgoing(c_z, c_hidden_mul)
        self.tri_mul_in = TriangleMultiplicationIncoming(c_z, c_hidden_mul)
        self.tri_att_start = TriangleAttention(c_z, c_hidden_pair_att, no_heads_pair)
        self.tri_att_end = TriangleAttention(c_z, c_hidden_pair_att, no_heads_pair)
        self.p_drop = dropout
        self.pair_transition = Transition(c_z, num_intermediate_factor)
        self.c_s = c_s
        if c_s > 0:
            self.attention_pair_bias = AttentionPairBias(
                has_s=False, create_offset_ln_z=True, n_heads=n_heads,
                c_a=c_s, c_z=c_z)
            self.single_transition = Transition(c_s, 4)

    def forward(self, s, z, pair_mask, triangle_multiplicative="torch",
                triangle_attention="torch", inplace_safe=False, chunk_size=None):
        """Eval path of pairformer.py:103-224 (dropout is the identity in
        eval: fused_ops.py:213-214)."""
        z = z + self.tri_mul_out(z, mask=pair_mask,
                                 triangle_multiplicative=triangle_multiplicative)
        z = z + self.tri_mul_in(z, mask=pair_mask,
                                triangle_multiplicative=triangle_multiplicative)
        z = z + self.tri_att_start(z, mask=pair_mask, chunk_size=chunk_size,
                                   triangle_attention=triangle_attention)
        z = z.transpose(-2, -3).contiguous()
        mask_t = pair_mask.transpose(-1, -2) if pair_mask is not None else None
        z = z + self.tri_att_end(z, mask=mask_t, chunk_size=chunk_size,
                                 triangle_attention=triangle_attention)
        z = z.transpose(-2, -3).contiguous()
        z = z + self.pair_transition(z)
        if self.c_s > 0:
            s = s + self.attention_pair_bias(a=s, s=None, z=z)
            s = s + self.single_transition(s)
        return s, z


class PairformerStack(nn.Module):
    def __init__(self, n_blocks: int = 48, n_heads: int = 16, c_z: int = 128,
                 c_s: int = 384, num_intermediate_factor: int = 4,
                 dropout: float = 0.25, blocks_per_ckpt: Optional[int] = None,
                 hidden_scale_up: bool = False) -> None:
        super().__init__()
        self.n_blocks = n_blocks
        self.n_heads = n_heads
        self.blocks_per_ckpt = blocks_per_ckpt
        self.blocks = nn.ModuleList(
            PairformerBlock(n_heads=n_heads, c_z=c_z, c_s=c_s,
                            num_intermediate_factor=num_intermediate_factor,
                            dropout=dropout, hidden_scale_up=hidden_scale_up)
            for _ in range(n_blocks))

    def forward(self, s, z, pair_mask, triangle_multiplicative="torch",
                triangle_attention="torch", inplace_safe=False, chunk_size=None
                ) -> Tuple[torch.Tensor, torch.Tensor]:
        for blk in self.blocks:
            s, z = blk(s, z, pair_mask,
                       triangle_multiplicative=triangle_multiplicative,
                       triangle_attention=triangle_attention,
                       inplace_safe=inplace_safe, chunk_size=chunk_size)
        return s, z


# ----------------------------------------------------------------------------
# seeded synthetic parameters and inputs (the measurement contract)
# ----------------------------------------------------------------------------
@torch.no_grad()
def seed_parameters_(module: nn.Module, seed: int = 4321) -> nn.Module:
    """Overwrite EVERY parameter (a default-initialised reference block is the
    identity because its gates and output projections start at zero):
    linear weights randn(out,in)/sqrt(in); 1-D ``*.weight`` (LayerNorm gamma)
    1 + 0.1*randn; LayerNorm beta 0.1*randn; linear biases 0.  Filled in
    named_parameters() order from one CPU generator, in fp32, then cast."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    linear_bias_names = {n + ".bias" for n, m in module.named_modules()
                         if isinstance(m, nn.Linear)}
    for name, p in module.named_parameters():
        if p.dim() == 2:
            v = torch.randn(p.shape, generator=g) / math.sqrt(p.shape[1])
        elif name.endswith("weight"):
            v = 1.0 + 0.1 * torch.randn(p.shape, generator=g)
        elif name in linear_bias_names:
            v = torch.zeros(p.shape)
        else:
            v = 0.1 * torch.randn(p.shape, generator=g)
        p.copy_(v.to(p.dtype))
    return module


def make_inputs(n_token: int, c_z: int = 128, c_s: int = 384, n_pad: int = 0,
                seed: int = 1234, dtype: torch.dtype = torch.float32):
    """z ~ N(0,1) [1,N,N,c_z], s ~ N(0,1) [1,N,c_s], pair_mask = m (x) m with the
    last ``n_pad`` tokens zero; generated in fp32 on the CPU, then cast."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    z = torch.randn(1, n_token, n_token, c_z, generator=g).to(dtype)
    s = torch.randn(1, n_token, c_s, generator=g).to(dtype)
    m = torch.ones(n_token)
    if n_pad > 0:
        m[n_token - n_pad:] = 0
    pair_mask = (m[:, None] * m[None, :])[None].to(dtype)
    return s, z, pair_mask
