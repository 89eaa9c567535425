"""Linear layers and the SwiGLU Transition of the Pairformer block.

Mirrors protenix/model/modules/primitives.py:33-101 (Linear / LinearNoBias),
:166-230 (Transition) and protenix/model/triangular/layers.py:104-197
(OpenfoldLinear, by its initialiser names).  The pair Transition (c_in = 64, 128, or 256 in bf16)
runs on the fused HIP kernel; other widths (the single track, c_in = 384) use
the HIP LayerNorm and the small-GEMM kernels of the single track.
"""
from __future__ import annotations

import math
from functools import partial
from typing import Optional

import torch
import torch.nn as nn

from . import ops
from .layer_norm import LayerNorm, _forward_only


def _trunc_normal_(w: torch.Tensor, scale: float) -> None:
    fan_in = w.shape[1]
    std = math.sqrt(scale / max(1, fan_in)) / 0.87962566103423978  # std of N(0,1) cut at +-2
    nn.init.trunc_normal_(w, mean=0.0, std=std, a=-2.0 * std, b=2.0 * std)


class Linear(nn.Linear):
    """nn.Linear with the reference's initialisers: "default" (LeCun truncated
    normal), "relu" (He), "zeros" / "final" / "gating" (weight 0; gating bias 1)."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None,
                 dtype=None, precision: Optional[torch.dtype] = None,
                 initializer: str = "default") -> None:
        self.use_bias = bias
        self.precision = precision
        self.initializer = initializer
        super().__init__(in_features, out_features, bias=bias, device=device, dtype=dtype)
        self._cache = _WeightCache()
        self._init_params()

    @torch.no_grad()
    def _init_params(self) -> None:
        if self.use_bias:
            nn.init.zeros_(self.bias)
        if self.initializer == "default":
            _trunc_normal_(self.weight, 1.0)
        elif self.initializer == "relu":
            _trunc_normal_(self.weight, 2.0)
        elif self.initializer in ("zeros", "final"):
            nn.init.zeros_(self.weight)
        elif self.initializer == "gating":
            nn.init.zeros_(self.weight)
            if self.use_bias:
                nn.init.ones_(self.bias)
        else:
            raise ValueError(f"Invalid initializer: {self.initializer}.")

    def forward(self, input: torch.Tensor) -> torch.Tensor:  # noqa: A002
        """primitives.py:83-98 on the HIP kernel of the single track: with `precision`, the
        product is formed in that dtype (autocast ignored) and returned in the input's dtype;
        without, in the input's dtype, or in the autocast dtype for an fp32 input under
        torch.autocast (as F.linear would).  GPU tensors, float32 / bfloat16, in_features a
        multiple of 16 and out_features of 8; anything else raises - no library GEMM stands in."""
        _forward_only(input, module=self)
        ops._dev(input, "input")
        if self.precision is not None:
            cd, od = self.precision, input.dtype
        else:
            cd = ops.autocast_compute_dtype(input) or input.dtype
            od = cd
        if cd not in (torch.float32, torch.bfloat16):
            raise RuntimeError(f"protenix_amd.Linear: unsupported arithmetic dtype {cd} "
                               "(float32 or bfloat16)")
        w, b = self._cache.get((self.weight, self.bias), cd, input.device, lambda: (
            _cv(self.weight, cd, input.device), _cv(self.bias, cd, input.device)))
        out = ops.linear(input.to(cd), w, b)
        return out if out.dtype == od else out.to(od)


LinearNoBias = partial(Linear, bias=False)


class _WeightCache:
    """Parameters converted once to the activation dtype/device; rebuilt when a
    parameter is modified in place or replaced."""

    def __init__(self) -> None:
        self._key = None
        self._val = None

    def get(self, params, dtype, device, build):
        key = (dtype, device) + tuple((id(p), p._version, p.data_ptr()) if p is not None else None
                                      for p in params)
        if key != self._key:
            self._val = build()
            self._key = key
        return self._val


def _cv(p: Optional[torch.Tensor], dtype, device) -> Optional[torch.Tensor]:
    return None if p is None else p.detach().to(device=device, dtype=dtype).contiguous()


class Transition(nn.Module):
    def __init__(self, c_in: int, n: int) -> None:
        super().__init__()
        self.n = n
        self.c_in = c_in
        self.layernorm1 = LayerNorm(c_in)
        self.linear_no_bias_a = LinearNoBias(c_in, n * c_in, initializer="relu")
        self.linear_no_bias_b = LinearNoBias(c_in, n * c_in, initializer="relu")
        self.linear_no_bias = LinearNoBias(n * c_in, c_in, initializer="zeros")
        self._cache = _WeightCache()
        self._cache_ab = _WeightCache()

    def _weights(self, dtype, device) -> dict:
        ps = (self.layernorm1.weight, self.layernorm1.bias, self.linear_no_bias_a.weight,
              self.linear_no_bias_b.weight, self.linear_no_bias.weight)
        def make():
            ln_w, ln_b, w_a, w_b, w_o = (_cv(p, dtype, device) for p in ps)
            return {"ln_w": ln_w, "ln_b": ln_b, "packed": ops.transition_pack(w_a, w_b, w_o)}
        return self._cache.get(ps, dtype, device, make)

    def fuses_pair_bias(self, x: torch.Tensor, heads: int) -> bool:
        """Whether forward(x, _pair_bias_w=...) is available: rows of 128 channels in bf16
        arithmetic (bf16 rows, or fp32 rows under bf16 autocast), at most 32 heads."""
        return (self.c_in == 128 and (self.n * self.c_in) % 64 == 0 and heads <= 32 and x.is_cuda
                and ops.compute_dtype(x) == torch.bfloat16)

    def forward(self, x: torch.Tensor, _residual_out: Optional[torch.Tensor] = None,
                _residual_new: bool = False, _pair_bias_w: Optional[tuple] = None):
        """Returns the update; with `_residual_out` (may be x itself) writes
        x + update there instead and returns it; with `_residual_new` returns x + update in a
        new tensor.  With `_pair_bias_w = (ln_w, ln_b, w)` (bf16; see fuses_pair_bias) and a
        residual output, returns (x + update, fp32 bias [heads, rows]) from one launch."""
        _forward_only(x, module=self)
        if _pair_bias_w is not None:
            assert _residual_out is not None and self.fuses_pair_bias(x, _pair_bias_w[2].shape[0])
            return ops.transition(x, self._weights(torch.bfloat16, x.device), self.n, add_residual=True,
                                  out=_residual_out, pair_bias_w=_pair_bias_w)
        cd = ops.compute_dtype(x)     # bf16 for fp32 rows of 64 / 128 / 256 channels under bf16 autocast
        fused = self.c_in in (64, 128) or (self.c_in == 256 and cd == torch.bfloat16)
        if _residual_new and _residual_out is None and fused:
            _residual_out = torch.empty_like(x)
        add = _residual_out is not None or _residual_new
        if fused and (self.n * self.c_in) % 64 == 0:
            out = ops.transition(x, self._weights(cd, x.device), self.n, add_residual=add,
                                 out=_residual_out)
            # (an update computed on fp32 rows under autocast holds bf16 values: returned in
            # the autocast dtype, like the reference's last linear)
            return out if (add or cd == x.dtype) else out.to(cd)
        # other widths (the single track, c_in = 384): HIP LayerNorm, SwiGLU and output kernels
        if any(l.precision is not None for l in (self.linear_no_bias_a, self.linear_no_bias_b,
                                                 self.linear_no_bias)):
            raise RuntimeError("protenix_amd.Transition: linear layers with a `precision` override "
                               "are not supported")
        if not (self.c_in % 16 == 0 and (self.n * self.c_in) % 16 == 0
                and x.dtype in (torch.float32, torch.bfloat16)):
            raise RuntimeError(
                f"protenix_amd.Transition: unsupported shape c_in={self.c_in} n={self.n} dtype={x.dtype} "
                "(c_in a multiple of 16, float32 or bfloat16)")
        y = self.layernorm1(x)
        ps = (self.linear_no_bias_a.weight, self.linear_no_bias_b.weight, self.linear_no_bias.weight)
        w_a, w_b, w_o = self._cache_ab.get(ps, y.dtype, y.device, lambda: tuple(
            _cv(p, y.dtype, y.device) for p in ps))
        h = ops.swiglu(y, w_a, w_b)
        u = ops.linear(h, w_o, res=x if add else None)
        return u if _residual_out is None else _residual_out.copy_(u)
