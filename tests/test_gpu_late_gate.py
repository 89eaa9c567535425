"""Triangle attention with the gate formed by the output kernel (ptx_triattn_gate_output, rows of
128 channels in bf16 arithmetic) against the same module with the gate stored by the projection
kernel and applied by the attention core, and against the oracle (layers.py:361-398)."""
import pytest
import torch

import protenix_amd as P
from protenix_amd import ops
from oracle import pairformer_oracle as O
from tests.util import oracle_and_product, pad_mask, rel_err, tol

pytestmark = pytest.mark.gpu


def _run(prod, z, mask, mixed, late):
    keep = ops.late_gate_enabled
    ops.late_gate_enabled = late
    try:
        with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16, enabled=mixed):
            return prod(z, mask)
    finally:
        ops.late_gate_enabled = keep


@pytest.mark.parametrize("mixed", [False, True])
@pytest.mark.parametrize("starting", [True, False])
@pytest.mark.parametrize("n,n_pad", [(1, 0), (2, 0), (33, 1), (37, 5), (64, 0), (100, 7), (256, 32)])
def test_late_gate_equals_stored_gate_and_oracle(mixed, starting, n, n_pad):
    dt = torch.float32 if mixed else torch.bfloat16
    ref, prod = oracle_and_product(O.TriangleAttention, P.TriangleAttention, 128, 32, 4,
                                   starting=starting, dtype=torch.bfloat16)
    prod = prod.to(dt)
    g = torch.Generator().manual_seed(n)
    z = (torch.randn(1, n, n, 128, generator=g) * 1.5).to(torch.bfloat16)
    mask = pad_mask(n, n_pad)
    if n_pad:
        mask[0, 3, :] = (torch.rand(n, generator=g) > 0.4).float()     # not symmetric
    with torch.no_grad():
        want = ref(z.float(), mask)
    zd, md = z.to("cuda", dt), mask.cuda()
    late = _run(prod, zd, md, mixed, True)
    stored = _run(prod, zd, md, mixed, False)
    assert late.shape == stored.shape and late.dtype == stored.dtype
    assert rel_err(late, want) <= tol(torch.bfloat16)
    # same operands in the same order through both paths: at most a rounding step apart
    assert rel_err(late, stored) <= 4e-3
    assert rel_err(late, want) <= 1.2 * rel_err(stored, want) + 1e-3


@pytest.mark.parametrize("mixed", [False, True])
def test_block_with_late_gate(mixed):
    """A whole block (in-place residual updates, transposed addressing for the ending node)."""
    dt = torch.float32 if mixed else torch.bfloat16
    ref, prod = oracle_and_product(O.PairformerBlock, P.PairformerBlock, dtype=torch.bfloat16)
    prod = prod.to(dt)
    s, z, pm = O.make_inputs(96, n_pad=9, dtype=torch.bfloat16)
    with torch.no_grad():
        s_ref, z_ref = ref(s.float(), z.float(), pm.float())
    outs = {}
    for late in (True, False):
        keep = ops.late_gate_enabled
        ops.late_gate_enabled = late
        try:
            with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16, enabled=mixed):
                outs[late] = prod(s.to("cuda", dt), z.to("cuda", dt), pm.cuda())
        finally:
            ops.late_gate_enabled = keep
    for late in (True, False):
        assert rel_err(outs[late][1], z_ref) <= tol(torch.bfloat16)
        assert rel_err(outs[late][0], s_ref) <= tol(torch.bfloat16)
    assert rel_err(outs[True][1], outs[False][1]) <= 4e-3


def test_gate_output_refusals():
    lib = P._lib.load()
    n = 32
    z = torch.randn(n, n, 128, device="cuda").bfloat16()
    o = torch.randn(4, n, n, 32, device="cuda").bfloat16()
    w = torch.randn(128, 128, device="cuda").bfloat16()
    out = torch.empty_like(z)
    args = [ops._ptr(o), ops._ptr(z), None, None, ops._ptr(w), ops._ptr(w), ops._ptr(out), n, 128, 4, 0, 1,
            1e-5, P._lib.PTX_BF16, None]
    assert lib.ptx_triattn_gate_output(*args) == 0
    for idx, bad in ((13, P._lib.PTX_F32), (8, 64), (9, 8), (0, None), (7, -1)):
        a = list(args)
        a[idx] = bad
        assert lib.ptx_triattn_gate_output(*a) != 0
    torch.cuda.synchronize()
