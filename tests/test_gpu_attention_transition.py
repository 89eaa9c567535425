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


@pytest.mark.parametrize("mixed", [True, False])
@pytest.mark.parametrize("n,n_pad", [(61, 0), (101, 0), (203, 0), (629, 0)])
def test_sizes_padded_to_a_multiple_of_8(mixed, n, n_pad):
    """N_token that 8 does not divide runs as the next multiple with the extra tokens masked
    (protenix_amd.pairformer.pad_tokens_to): the same bits as the unpadded run, both
    within tolerance of the oracle, inputs untouched / updated in place as asked."""
    from protenix_amd import pairformer as pf
    dt = torch.float32 if mixed else BF16
    ref, prod = oracle_and_product(O.PairformerStack, P.PairformerStack, n_blocks=2, dtype=BF16)
    prod = prod.to(dt)
    s, z, pm = O.make_inputs(n, n_pad=n_pad, dtype=BF16)
    pmd = pm.cuda() if n == 101 else None       # (a mask of all ones, or none)
    with torch.no_grad():
        s_ref, z_ref = ref(s.float(), z.float(), pm.float(), chunk_size=128 if n > 256 else None)
    outs = {}
    for pad_to in (8, 0):
        keep = pf.pad_tokens_to, pf.pad_tokens_min_n
        pf.pad_tokens_to, pf.pad_tokens_min_n = pad_to, 0
        try:
            zd = z.to("cuda", dt)
            z_before = zd.clone()
            with torch.no_grad(), torch.autocast("cuda", dtype=BF16, enabled=mixed):
                s_o, z_o = prod(s.to("cuda", dt), zd, pmd)
                assert torch.equal(zd, z_before) and z_o.shape == zd.shape and z_o.is_contiguous()
                s_i, z_i = prod(s.to("cuda", dt), zd, pmd, inplace_safe=True)
                assert z_i is zd and torch.equal(z_i, z_o) and torch.equal(s_i, s_o)
            outs[pad_to] = (s_o, z_o)
        finally:
            pf.pad_tokens_to, pf.pad_tokens_min_n = keep
    for pad_to in (8, 0):
        assert rel_err(outs[pad_to][1], z_ref) <= tol(BF16)
        assert rel_err(outs[pad_to][0], s_ref) <= tol(BF16)
    print(f"padded vs unpadded: z {rel_err(outs[8][1], outs[0][1]):.2e} s {rel_err(outs[8][0], outs[0][0]):.2e}")
    # masked tokens contribute exact zeros in the same summation order: bit for bit
    assert torch.equal(outs[8][1], outs[0][1]) and torch.equal(outs[8][0], outs[0][0])


def test_padded_block_fp32_and_graph():
    """A single fp32 block at an odd size (padded internally) against the oracle, eager and
    through a recorded graph."""
    from protenix_amd import pairformer as pf
    ref, prod = oracle_and_product(O.PairformerBlock, P.PairformerBlock)
    s, z, pm = O.make_inputs(45, n_pad=0)
    keep = pf.pad_tokens_min_n
    pf.pad_tokens_min_n = 0
    try:
        with torch.no_grad():
            s_ref, z_ref = ref(s, z, pm)
            ops.kernel_timer = {}
            s_o, z_o = prod(s.cuda(), z.cuda(), None)
            assert "triattn_fwd_padded_rows" in ops.kernel_timer      # (ran as 48 tokens, 3 of them masked)
            ops.kernel_timer = None
            fast = P.Graphed(prod)
            for _ in range(3):
                s_g, z_g = fast(s.cuda(), z.cuda(), None)
                assert torch.equal(z_g, z_o) and torch.equal(s_g, s_o)
    finally:
        ops.kernel_timer = None
        pf.pad_tokens_min_n = keep
    assert rel_err(z_o, z_ref) <= tol(torch.float32) and rel_err(s_o, s_ref) <= tol(torch.float32)


@pytest.mark.parametrize("kw,n", [(dict(c_z=64, c_s=0), 327),
                                  (dict(c_z=256, hidden_scale_up=True), 323)])
def test_other_widths_padded_at_the_default_threshold(kw, n):
    """The template stack's width (no single track) and the scaled-up width at sizes just above
    the size from which odd sizes are padded: fp32 rows under bf16 autocast against the oracle,
    and the same bits as without the padding."""
    from protenix_amd import pairformer as pf
    assert n >= pf.pad_tokens_min_n and n % pf.pad_tokens_to
    ref, prod = oracle_and_product(O.PairformerStack, P.PairformerStack, n_blocks=1, dtype=BF16, **kw)
    prod = prod.float()
    c_s = kw.get("c_s", 384)
    s, z, pm = O.make_inputs(n, c_z=kw["c_z"], dtype=BF16)
    s_in = None if c_s == 0 else s.float()
    with torch.no_grad():
        s_ref, z_ref = ref(s_in, z.float(), pm.float(), chunk_size=64)
    outs = {}
    for pad_to in (8, 0):
        keep = pf.pad_tokens_to
        pf.pad_tokens_to = pad_to
        try:
            ops.kernel_timer = {}
            with torch.no_grad(), torch.autocast("cuda", dtype=BF16):
                outs[pad_to] = prod(None if s_in is None else s_in.cuda(), z.float().cuda(), None)
            assert ("triattn_fwd_padded_rows" in ops.kernel_timer) == (pad_to == 8)
        finally:
            ops.kernel_timer = None
            pf.pad_tokens_to = keep
    assert rel_err(outs[8][1], z_ref) <= tol(BF16)
    assert torch.equal(outs[8][1], outs[0][1])
    if c_s:
        assert rel_err(outs[8][0], s_ref) <= tol(BF16) and torch.equal(outs[8][0], outs[0][0])
