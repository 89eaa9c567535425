"""The ending-node attention's last stage and the pair transition in one launch
(ptx_triattn_output_transition_fwd) against the two launches it replaces
(ptx_triattn_gate_output, then ptx_transition_fwd / ptx_transition_pair_bias_fwd): the same
operations with the same roundings, so the results are compared bit for bit; and, through whole
blocks, against the oracle (pairformer.py:201-222 of the reference)."""
import pytest
import torch

import protenix_amd as P
from protenix_amd import ops
from oracle import pairformer_oracle as O
from tests.util import oracle_and_product, pad_mask, rel_err, tol

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _block(prod, s, z, pm, mixed, fused):
    keep = ops.fuse_attention_transition
    ops.fuse_attention_transition = fused
    try:
        ops.kernel_timer = {}
        with torch.no_grad(), torch.autocast("cuda", dtype=BF16, enabled=mixed):
            out = prod(s, z, pm)
        names = set(ops.kernel_timer)
        return out, names
    finally:
        ops.kernel_timer = None
        ops.fuse_attention_transition = keep


@pytest.mark.parametrize("mixed", [True, False])
@pytest.mark.parametrize("n,n_pad,c_s", [(1, 0, 384), (2, 0, 384), (33, 1, 384), (37, 5, 0), (64, 0, 384),
                                         (100, 7, 384), (130, 0, 0), (256, 32, 384)])
def test_block_fused_equals_two_launches_and_oracle(mixed, n, n_pad, c_s):
    dt = torch.float32 if mixed else BF16
    ref, prod = oracle_and_product(O.PairformerBlock, P.PairformerBlock, c_s=c_s, dtype=BF16)
    prod = prod.to(dt)
    s, z, pm = O.make_inputs(n, n_pad=n_pad, dtype=BF16)
    if n_pad:
        g = torch.Generator().manual_seed(n)
        pm[0, 3, :] = (torch.rand(n, generator=g) > 0.4).float()     # not symmetric
    if c_s == 0:
        s = None
    sd = None if s is None else s.to("cuda", dt)
    with torch.no_grad():
        s_ref, z_ref = ref(None if s is None else s.float(), z.float(), pm.float())
    (s_f, z_f), names_f = _block(prod, sd, z.to("cuda", dt), pm.cuda(), mixed, True)
    (s_u, z_u), names_u = _block(prod, sd, z.to("cuda", dt), pm.cuda(), mixed, False)
    assert "triattn_output_transition" in names_f and "transition" not in names_f
    assert "triattn_output_transition" not in names_u and "transition" in names_u
    assert torch.equal(z_f, z_u), rel_err(z_f, z_u)
    assert rel_err(z_f, z_ref) <= tol(BF16)
    if c_s:
        assert torch.equal(s_f, s_u), rel_err(s_f, s_u)     # the pair bias comes out of the same launch
        assert rel_err(s_f, s_ref) <= tol(BF16)


@pytest.mark.parametrize("mixed", [True, False])
def test_batched_stack_fused_equals_two_launches(mixed):
    dt = torch.float32 if mixed else BF16
    ref, prod = oracle_and_product(O.PairformerStack, P.PairformerStack, n_blocks=3, dtype=BF16)
    prod = prod.to(dt)
    n = 48
    g = torch.Generator().manual_seed(5)
    z = torch.randn(2, n, n, 128, generator=g).to(BF16)
    s = torch.randn(2, n, 384, generator=g).to(BF16)
    pm = torch.cat([pad_mask(n, 0), pad_mask(n, 5)])
    outs = {}
    for fused in (True, False):
        keep = ops.fuse_attention_transition
        ops.fuse_attention_transition = fused
        try:
            with torch.no_grad(), torch.autocast("cuda", dtype=BF16, enabled=mixed):
                outs[fused] = prod(s.to("cuda", dt), z.to("cuda", dt), pm.cuda())
        finally:
            ops.fuse_attention_transition = keep
    assert torch.equal(outs[True][1], outs[False][1])
    assert torch.equal(outs[True][0], outs[False][0])
    with torch.no_grad():
        s_ref, z_ref = ref(s.float(), z.float(), pm)
    assert rel_err(outs[True][1], z_ref) <= tol(BF16)
    assert rel_err(outs[True][0], s_ref) <= tol(BF16)


def test_fused_launch_refusals():
    lib = P._lib.load()
    n = 32
    z = torch.randn(n, n, 128, device="cuda").bfloat16()
    o = torch.randn(4, n, n, 32, device="cuda").bfloat16()
    packed = torch.zeros(lib.ptx_triattn_output_transition_packed_elems(4), device="cuda").bfloat16()
    out = torch.empty_like(z)
    args = [ops._ptr(o), ops._ptr(z), None, None, ops._ptr(packed), None, None, ops._ptr(out), n, 128, 4, 1,
            4, 1e-5, 1e-5, None, None, None, None, 0, 1, 1e-5, P._lib.PTX_BF16, None]
    assert lib.ptx_triattn_output_transition_fwd(*args) == 0
    for idx, bad in ((22, P._lib.PTX_F32), (9, 64), (10, 8), (0, None), (4, None), (8, -1), (12, 0)):
        a = list(args)
        a[idx] = bad
        assert lib.ptx_triattn_output_transition_fwd(*a) != 0
    torch.cuda.synchronize()
