"""HIP-graph replay of a Pairformer block or stack for repeated calls at one shape.

Below a few hundred tokens the forward pass is bound by the host: a block issues about forty
kernel launches and the GPU finishes them faster than Python can enqueue them.  `Graphed`
records one forward pass of a `PairformerBlock` / `PairformerStack` into a HIP graph (through
`torch.cuda.CUDAGraph`, which also captures the second stream the stack uses for the single
track) and replays it for every later call with the same shapes and dtypes (and, for a single
pair mask, the same class of mask: padding at the end with the same number of valid tokens, or
any other mask - the class decides which attention kernels a forward pass launches).

    fast = protenix_amd.Graphed(stack)          # stack: eval mode, on the GPU
    s, z = fast(s, z, pair_mask)                # first call per shape: warm-up + capture

The reference has no counterpart (its trunk is launched eagerly, pairformer.py:291-340); this
is an optional wrapper and the modules themselves are unchanged.  Inputs are copied into the
graph's static buffers and the results are copied out, so the caller's tensors are never
aliased; parameters are baked in by address, so weights must not be replaced (in-place updates
of the same storage are picked up only by the kernels that read parameters directly: re-create
the wrapper after loading new weights).  Every captured shape keeps its workspaces alive.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch
import torch.nn as nn

from . import ops


class Graphed:
    def __init__(self, module: nn.Module, warmup: int = 2) -> None:
        if module.training:
            raise RuntimeError("protenix_amd.Graphed wraps inference modules: call .eval() first")
        self.module = module
        self.warmup = max(1, int(warmup))
        self._entries: Dict[tuple, tuple] = {}

    @staticmethod
    def _mask_class(z, pair_mask) -> tuple:
        """The class of the mask that decides which kernels run (ops.mask_class): a recording
        is made for one class and replayed for masks of that class only."""
        if pair_mask is None or not pair_mask.is_cuda:
            return (False, None)
        n = z.shape[-2]
        if pair_mask.numel() != n * n:
            return (False, None)      # a batch of masks: the general kernels
        return (False, ops.padded_tail(pair_mask.reshape(n, n), n))

    @classmethod
    def _key(cls, s, z, pair_mask) -> tuple:
        def sig(t):
            return None if t is None else (tuple(t.shape), t.dtype, t.device.index)
        return (sig(s), sig(z), sig(pair_mask), cls._mask_class(z, pair_mask))

    def _capture(self, s, z, pair_mask) -> tuple:
        if not z.is_cuda:
            raise RuntimeError("protenix_amd.Graphed needs GPU tensors")
        s_in = None if s is None else s.clone()
        z_io = z.clone(memory_format=torch.contiguous_format)
        m_in = None if pair_mask is None else pair_mask.clone()
        # Warm-up on a side stream, as graph capture requires: fills the weight caches and the
        # allocator, and loads every kernel, none of which may happen while capturing.
        side = torch.cuda.Stream(device=z.device)
        side.wait_stream(torch.cuda.current_stream(z.device))
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(self.warmup):
                z_io.copy_(z)
                self.module(s_in, z_io, m_in, inplace_safe=True)
        torch.cuda.current_stream(z.device).wait_stream(side)
        torch.cuda.synchronize(z.device)
        z_io.copy_(z)
        graph = torch.cuda.CUDAGraph()
        ops.capture_mask_class = self._mask_class(z, pair_mask)
        try:
            with torch.no_grad(), torch.cuda.graph(graph):
                s_out, z_out = self.module(s_in, z_io, m_in, inplace_safe=True)
        finally:
            ops.capture_mask_class = None
        return graph, s_in, z_io, m_in, s_out, z_out

    def __call__(self, s: Optional[torch.Tensor], z: torch.Tensor,
                 pair_mask: Optional[torch.Tensor] = None
                 ) -> Tuple[Optional[torch.Tensor], torch.Tensor]:
        """Same result as module(s, z, pair_mask) under torch.no_grad(); s, z, pair_mask are
        left untouched."""
        key = self._key(s, z, pair_mask)
        entry = self._entries.get(key)
        if entry is None:
            entry = self._capture(s, z, pair_mask)
            self._entries[key] = entry
        graph, s_in, z_io, m_in, s_out, z_out = entry
        z_io.copy_(z)
        if s_in is not None:
            s_in.copy_(s)
        if m_in is not None:
            m_in.copy_(pair_mask)
        graph.replay()
        return (None if s_out is None else s_out.clone()), z_out.clone()

    def shapes(self) -> list:
        """The (s, z, mask) signatures captured so far."""
        return list(self._entries)
