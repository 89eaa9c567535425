"""PairformerBlock / PairformerStack on the gfx950 kernels.

Same constructor arguments, sub-module names (= state-dict keys) and forward
signatures as protenix/model/modules/pairformer.py:42-340.  Eval / no-grad
forward only.  The five pair updates of a block run as fused kernels that add
their result into the pair tensor on the way out; the ending-node attention
reads and writes the pair tensor through transposed addressing, so the two
`transpose(-2, -3).contiguous()` copies of the reference (pairformer.py:201,
214) do not exist here.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn as nn

from . import ops
from .primitives import Transition, _WeightCache, _cv
from .transformer import AttentionPairBias
from .triangular import (TriangleAttention, TriangleMultiplicationIncoming,
                         TriangleMultiplicationOutgoing)


# Pair tensors whose N_token is not a multiple of 8 are worked on as the next multiple with the
# extra tokens masked out (0: as they are).  Rows of a [N, N] plane then start at multiples of 16
# bytes, which the channel-major workspaces of the triangle updates (the contraction's result, V^T,
# the triangle bias) need for their 16-byte accesses: at N = 700 a block takes 2.91 ms as it is
# and 2.48 ms as 704 tokens of which 4 are masked, at 381 0.97 against 0.77 ms.  Masked tokens
# take no part in either triangle update and every other operation on the pair tensor is local to
# a pair, so the N x N corner of the result is what the unpadded tensor gives; the single
# representation is not padded (its attention has no mask), it reads the corner of the pair bias.
# Only without a pair mask (or with one of all ones): a token the caller masks is a row whose keys
# are all masked, the reference gives such a row the mean of V over all N keys, and with more keys
# that mean would be another.
# From pad_tokens_min_n tokens on: below, the extra launches (the padded rows' attention, the
# crop of the pair bias) cost a block more than the aligned rows save (N = 253: 0.48 -> 0.57 ms).
pad_tokens_to = 8
pad_tokens_min_n = 320


class _Padded:
    """z [*, N, N, c] (+ pair_mask) as [*, N', N', c] with N' the next multiple of `pad_tokens_to`."""

    def __init__(self, z: torch.Tensor) -> None:
        self.n = z.shape[-2]
        n2 = -(-self.n // pad_tokens_to) * pad_tokens_to
        self.z = z.new_zeros(*z.shape[:-3], n2, n2, z.shape[-1])
        self.z[..., :self.n, :self.n, :].copy_(z)
        self.mask = z.new_zeros(*z.shape[:-3], n2, n2)
        self.mask[..., :self.n, :self.n] = 1
        # (known without looking: padding at the end, N valid tokens)
        ops.declare_mask_class(self.mask, (False, self.n))

    def crop_bias(self, bias: torch.Tensor) -> torch.Tensor:
        return bias[..., :self.n, :self.n].contiguous()

    def result(self, z_out: Optional[torch.Tensor]) -> torch.Tensor:
        """The N x N corner, written into z_out if given (the caller's tensor, updated in place)."""
        ops.forget_mask(self.mask)
        corner = self.z[..., :self.n, :self.n, :]
        return corner.contiguous() if z_out is None else z_out.copy_(corner)


def _wants_padding(z: torch.Tensor, pair_mask: Optional[torch.Tensor]) -> bool:
    return (pad_tokens_to > 1 and z.is_cuda and z.dim() >= 3 and z.shape[-2] == z.shape[-3]
            and z.shape[-2] % pad_tokens_to != 0 and z.shape[-2] >= pad_tokens_min_n
            and (pair_mask is None or (pair_mask.is_cuda and ops.mask_class(pair_mask)[0])))


class PairformerBlock(nn.Module):
    def __init__(self, n_heads: int = 16, c_z: int = 128, c_s: int = 384, c_hidden_mul: int = 128,
                 c_hidden_pair_att: int = 32, no_heads_pair: int = 4,
                 num_intermediate_factor: int = 4, dropout: float = 0.25,
                 hidden_scale_up: bool = False) -> None:
        super().__init__()
        self.n_heads = n_heads
        if hidden_scale_up:
            no_heads_pair = c_z // c_hidden_pair_att
            c_hidden_mul = c_z
        self.tri_mul_out = TriangleMultiplicationOutgoing(c_z=c_z, c_hidden=c_hidden_mul)
        self.tri_mul_in = TriangleMultiplicationIncoming(c_z=c_z, c_hidden=c_hidden_mul)
        self.tri_att_start = TriangleAttention(c_in=c_z, c_hidden=c_hidden_pair_att,
                                               no_heads=no_heads_pair)
        self.tri_att_end = TriangleAttention(c_in=c_z, c_hidden=c_hidden_pair_att,
                                             no_heads=no_heads_pair)
        self.p_drop = dropout
        self.pair_transition = Transition(c_in=c_z, n=num_intermediate_factor)
        self._fused_cache = _WeightCache()
        self.c_s = c_s
        if self.c_s > 0:
            self.attention_pair_bias = AttentionPairBias(has_s=False, create_offset_ln_z=True,
                                                         n_heads=n_heads, c_a=c_s, c_z=c_z)
            self.single_transition = Transition(c_in=c_s, n=4)

    def forward(self, s: Optional[torch.Tensor], z: torch.Tensor, pair_mask: Optional[torch.Tensor],
                triangle_multiplicative: str = "torch", triangle_attention: str = "torch",
                inplace_safe: bool = False, chunk_size: Optional[int] = None
                ) -> Tuple[Optional[torch.Tensor], torch.Tensor]:
        """s [..., N, c_s] or None, z [..., N, N, c_z], pair_mask [..., N, N] or
        None -> (s, z).  With `inplace_safe` z is updated in place, as the
        reference's inference path does; otherwise the inputs are left untouched."""
        if self.training:
            raise RuntimeError("protenix_amd.PairformerBlock is inference-only: call .eval()")
        if triangle_multiplicative not in ("torch", "cuequivariance"):
            raise ValueError(
                "triangle_multiplicative must be 'cuequivariance' or 'torch', but got "
                f"{triangle_multiplicative}")
        assert triangle_attention in ("torch", "deepspeed", "triattention", "cuequivariance")
        if _wants_padding(z, pair_mask):
            pad = _Padded(z)
            s, _ = self._forward_unpadded(s, pad.z, pad.mask, pad)
            return s, pad.result(z if inplace_safe else None)
        if not inplace_safe or not z.is_contiguous():
            z = z.clone(memory_format=torch.contiguous_format)
        return self._forward_unpadded(s, z, pair_mask, None)

    def _forward_unpadded(self, s, z, pair_mask, pad):
        """z: contiguous, updated in place; pad: the _Padded that made it, or None."""
        ac = ops.autocast_compute_dtype(z)
        if ac is not None and ops.compute_dtype(z) == z.dtype:
            return self._forward_autocast_unfused(s, z, pair_mask, ac, pad)
        # (fp32 z under bf16 autocast: the same fused kernels, reading and updating the fp32
        # rows in place with bf16 arithmetic)
        bias = self._pair_track(z, pair_mask, want_bias=self.c_s > 0)
        if self.c_s > 0:
            s = self._single_track(s, bias if pad is None else pad.crop_bias(bias))
        return s, z

    def _pair_track(self, z: torch.Tensor, pair_mask: Optional[torch.Tensor],
                    want_bias: bool = False) -> Optional[torch.Tensor]:
        """The five pair updates, each "z += f(z)" fused into a kernel epilogue.  With
        `want_bias`, also the pair bias of the single attention, read off the finished z: in
        the transition's own epilogue where that kernel has one, by a kernel of its own
        otherwise."""
        self.tri_mul_out(z, mask=pair_mask, inplace_safe=True, _add_with_inplace=True)
        self.tri_mul_in(z, mask=pair_mask, inplace_safe=True, _add_with_inplace=True)
        self.tri_att_start._run(z, pair_mask, transposed=False, residual_inplace=True)
        # ending node: the starting-node module of the reference applied to z^T with
        # mask^T, expressed through transposed addressing of z and mask
        apb = self.attention_pair_bias if want_bias else None
        att, tr = self.tri_att_end, self.pair_transition
        if (z.is_contiguous() and tr.c_in == att.c_in
                and ops.fuses_attention_transition(z, att.no_heads, att.c_hidden, tr.n)
                and (apb is None or apb.n_heads <= 32)):
            # the ending node's last stage and the transition (and the pair bias) in one launch:
            # the tensor between the two never travels through memory
            def fused_weights(cd, device):
                ps = (att.mha.linear_g.weight, att.mha.linear_o.weight, tr.layernorm1.weight,
                      tr.layernorm1.bias, tr.linear_no_bias_a.weight, tr.linear_no_bias_b.weight,
                      tr.linear_no_bias.weight)
                def make():
                    w_g, w_o, ln_w, ln_b, w_a, w_b, w_to = (_cv(p, cd, device) for p in ps)
                    return {"packed": ops.attention_transition_pack(w_g, w_o, w_a, w_b, w_to),
                            "ln_w": ln_w, "ln_b": ln_b, "n_factor": tr.n}
                tt = dict(self._fused_cache.get(ps, cd, device, make))
                tt["pair_bias_w"] = None if apb is None else apb.pair_bias_weights(z)
                return tt
            _, biases = att._run(z, pair_mask, transposed=True, residual_inplace=True,
                                 then_transition=fused_weights)
            if apb is None:
                return None
            n = z.shape[-2]
            bias = biases[0] if len(biases) == 1 else torch.stack(biases)
            return bias.view(*z.shape[:-3], apb.n_heads, n, n)
        self.tri_att_end._run(z, pair_mask, transposed=True, residual_inplace=True)
        if not want_bias:
            self.pair_transition(z, _residual_out=z)
            return None
        apb = self.attention_pair_bias
        n = z.shape[-2]
        if z.is_contiguous() and self.pair_transition.fuses_pair_bias(z, apb.n_heads):
            # (one launch per pair tensor of a batch: the epilogue writes [heads][rows])
            pbw = apb.pair_bias_weights(z)
            zb = z.view(-1, n, n, z.shape[-1])
            bias = [self.pair_transition(zi, _residual_out=zi, _pair_bias_w=pbw)[1] for zi in zb]
            bias = bias[0] if len(bias) == 1 else torch.stack(bias)
            return bias.view(*z.shape[:-3], apb.n_heads, n, n)
        self.pair_transition(z, _residual_out=z)
        return apb.pair_bias(z)

    def _forward_autocast_unfused(self, s: Optional[torch.Tensor], z: torch.Tensor,
                                  pair_mask: Optional[torch.Tensor], ac: torch.dtype, pad=None
                                  ) -> Tuple[Optional[torch.Tensor], torch.Tensor]:
        """fp32 residual stream under torch.autocast where no fused fp32-row kernel applies (an
        autocast dtype other than bfloat16 - the kernels' 16-bit arithmetic is bf16 - or a row
        width outside 64 / 128 / 256): every update is computed by the kernels in the autocast
        dtype from a rounded copy of z and added to the fp32 z (in place; z is private here).
        Costs a cast and an add pass per update on top of the fused path; widths and dtypes the
        kernels do not take at all are refused by them."""
        m = None if pair_mask is None else pair_mask.to(ac)
        z.add_(self.tri_mul_out(z.to(ac), mask=m))
        z.add_(self.tri_mul_in(z.to(ac), mask=m))
        z.add_(self.tri_att_start._run(z.to(ac), m, transposed=False, residual_inplace=False))
        z.add_(self.tri_att_end._run(z.to(ac), m, transposed=True, residual_inplace=False))
        z.add_(self.pair_transition(z.to(ac)))
        if self.c_s > 0:
            bias = self.attention_pair_bias.pair_bias(z.to(ac))
            s = self._single_track(s, bias if pad is None else pad.crop_bias(bias))
        return s, z

    def _single_track(self, s: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
        """s += attention(s; bias from z); s += transition(s).  Needs nothing of z but
        `bias`, and z never depends on s.  Runs in the dtype of s, with autocast off: on an
        fp32 single representation the whole track is fp32 arithmetic (it is a thousandth of
        the block's work, and through 48 blocks its bf16 rounding, above all that of the
        transition, costs s a 2.4e-2 relative error against 5e-3 this way)."""
        with torch.autocast("cuda", enabled=False):
            s = self.attention_pair_bias.forward_with_bias(s, bias, residual=s)
            return self.single_transition(s, _residual_new=True)


class PairformerStack(nn.Module):
    def __init__(self, n_blocks: int = 48, n_heads: int = 16, c_z: int = 128, c_s: int = 384,
                 num_intermediate_factor: int = 4, dropout: float = 0.25,
                 blocks_per_ckpt: Optional[int] = None, hidden_scale_up: bool = False) -> None:
        super().__init__()
        self.n_blocks = n_blocks
        self.n_heads = n_heads
        self.blocks_per_ckpt = blocks_per_ckpt
        self.blocks = nn.ModuleList()
        for _ in range(n_blocks):
            self.blocks.append(PairformerBlock(n_heads=n_heads, c_z=c_z, c_s=c_s,
                                               num_intermediate_factor=num_intermediate_factor,
                                               dropout=dropout, hidden_scale_up=hidden_scale_up))

    def forward(self, s: torch.Tensor, z: torch.Tensor, pair_mask: Optional[torch.Tensor],
                triangle_multiplicative: str = "torch", triangle_attention: str = "torch",
                inplace_safe: bool = False, chunk_size: Optional[int] = None
                ) -> Tuple[torch.Tensor, torch.Tensor]:
        """Blocks in sequence (pairformer.py:291-340); activation checkpointing is
        a training device and does nothing under no-grad, as in the reference."""
        for blk in self.blocks:
            if blk.training:
                raise RuntimeError("protenix_amd.PairformerStack is inference-only: call .eval()")
        pad = None
        z_caller = z
        if _wants_padding(z, pair_mask) and len(self.blocks) > 0:
            # (one padded copy for the whole stack, see pad_tokens_to)
            pad = _Padded(z)
            z, pair_mask = pad.z, pad.mask
        elif not inplace_safe and len(self.blocks) > 0:
            # one private copy for the whole stack; the blocks then work in place
            z = z.clone(memory_format=torch.contiguous_format)
        if not z.is_contiguous():
            z = z.contiguous()
        if triangle_multiplicative not in ("torch", "cuequivariance"):
            raise ValueError(
                "triangle_multiplicative must be 'cuequivariance' or 'torch', but got "
                f"{triangle_multiplicative}")
        assert triangle_attention in ("torch", "deepspeed", "triattention", "cuequivariance")
        ac = ops.autocast_compute_dtype(z)
        if (not z.is_cuda or s is None or any(b.c_s == 0 for b in self.blocks)
                or (ac is not None and ops.compute_dtype(z) == z.dtype)):
            for blk in self.blocks:
                if pad is None:
                    s, z = blk(s, z, pair_mask, inplace_safe=True)
                else:
                    s, z = blk._forward_unpadded(s, z, pair_mask, pad)
            return s, (z if pad is None else pad.result(z_caller if inplace_safe else None))
        # The pair track never reads s, and the single track reads z only through the pair
        # bias: the small single-track kernels of block b run on a second stream (default
        # priority) underneath the pair kernels of block b + 1.
        main = torch.cuda.current_stream(z.device)
        side = self._side_stream(z.device)
        side.wait_stream(main)
        for blk in self.blocks:
            bias = blk._pair_track(z, pair_mask, want_bias=True)   # (bias: from z before the next block writes it)
            if pad is not None:
                bias = pad.crop_bias(bias)
            ready = main.record_event()
            with torch.cuda.stream(side):
                side.wait_event(ready)
                s = blk._single_track(s, bias)
            bias.record_stream(side)
        main.wait_stream(side)
        s.record_stream(main)
        return s, (z if pad is None else pad.result(z_caller if inplace_safe else None))

    def _side_stream(self, device: torch.device) -> "torch.cuda.Stream":
        streams = self.__dict__.setdefault("_streams", {})
        key = (device.type, device.index)
        if key not in streams:
            streams[key] = torch.cuda.Stream(device=device)
        return streams[key]
