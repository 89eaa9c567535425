"""bf16 arithmetic on an fp32 residual stream (PTX_MIXED of the C ABI): what the modules run
when they are given fp32 tensors and fp32 parameters under torch.autocast(bfloat16), the
reference's inference mode (runner/inference.py:214-234).  Every operation against the fp32
oracle on the same fp32 inputs and parameters, bf16 tolerance (2e-2 of max |reference|)."""
import pytest
import torch

import protenix_amd as P
from oracle import pairformer_oracle as O
from protenix_amd import _lib, ops
from tests.util import TOL_BF16, pad_mask, rel_err

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _pair(oracle_cls, product_cls, *args, **kwargs):
    ref = O.seed_parameters_(oracle_cls(*args, **kwargs)).eval()
    prod = product_cls(*args, **kwargs)
    prod.load_state_dict(ref.state_dict())
    return ref, prod.to("cuda").eval()          # fp32 parameters on both sides


def _z(n, c=128, seed=1234):
    return torch.randn(1, n, n, c, generator=torch.Generator().manual_seed(seed))


def _amp():
    return torch.autocast("cuda", dtype=BF16)


@pytest.mark.parametrize("c_z", [128, 64])
@pytest.mark.parametrize("cls", ["TriangleMultiplicationOutgoing", "TriangleMultiplicationIncoming"])
@pytest.mark.parametrize("n,n_pad", [(64, 0), (100, 7), (37, 0), (200, 16)])
def test_trimul(c_z, cls, n, n_pad):
    ref, prod = _pair(getattr(O, cls), getattr(P, cls), c_z, 128)
    z = _z(n, c_z)
    mask = pad_mask(n, n_pad) if n_pad else None
    mc = None if mask is None else mask.cuda()
    with torch.no_grad():
        want = ref(z, mask)
        with _amp():
            got = prod(z.cuda(), mc)
            assert got.dtype == BF16          # like the reference's last linear under autocast
            zc = z.cuda().clone()
            got2 = prod(zc, mc, inplace_safe=True, _add_with_inplace=True)
    assert rel_err(got, want) <= TOL_BF16
    assert got2.data_ptr() == zc.data_ptr() and got2.dtype == torch.float32
    assert rel_err(got2, z + want) <= TOL_BF16
    # the fp32 rows took the bf16-rounded update and nothing else: z + update, exactly
    assert torch.equal(got2, z.cuda() + got.float())


@pytest.mark.parametrize("c_z", [128, 64])
@pytest.mark.parametrize("starting", [True, False])
@pytest.mark.parametrize("n,n_pad", [(64, 0), (100, 7), (37, 5), (256, 32)])
def test_triattn(c_z, starting, n, n_pad):
    ref, prod = _pair(O.TriangleAttention, P.TriangleAttention, c_z, 32, 4, starting=starting)
    z = _z(n, c_z)
    mask = pad_mask(n, n_pad) if n_pad else None
    with torch.no_grad():
        want = ref(z, mask, chunk_size=64)
        with _amp():
            got = prod(z.cuda(), None if mask is None else mask.cuda())
    assert got.dtype == BF16
    assert rel_err(got, want) <= TOL_BF16


@pytest.mark.parametrize("shape,factor", [((1, 50, 50, 128), 4), ((3001, 128), 4), ((77, 64), 2)])
def test_transition(shape, factor):
    ref, prod = _pair(O.Transition, P.Transition, shape[-1], factor)
    x = torch.randn(*shape, generator=torch.Generator().manual_seed(11))
    with torch.no_grad():
        want = ref(x)
        with _amp():
            got = prod(x.cuda())
            xc = x.cuda().clone()
            got2 = prod(xc, _residual_out=xc)
    assert got.dtype == BF16 and rel_err(got, want) <= TOL_BF16
    assert got2.dtype == torch.float32 and torch.equal(got2, x.cuda() + got.float())


def test_attention_pair_bias():
    ref, prod = _pair(O.AttentionPairBias, P.AttentionPairBias, has_s=False,
                      create_offset_ln_z=True, n_heads=16, c_a=384, c_z=128)
    n = 70
    g = torch.Generator().manual_seed(2)
    a, z = torch.randn(1, n, 384, generator=g), torch.randn(1, n, n, 128, generator=g)
    with torch.no_grad():
        want = ref(a, None, z)
        with _amp():
            bias = prod.pair_bias(z.cuda())
            got = prod(a.cuda(), None, z.cuda())
    assert bias.dtype == torch.float32
    assert rel_err(got, want) <= TOL_BF16


@pytest.mark.parametrize("n,n_pad", [(1, 0), (2, 1), (17, 1), (33, 0), (65, 1), (96, 9), (129, 1)])
def test_block(n, n_pad):
    ref, prod = _pair(O.PairformerBlock, P.PairformerBlock)
    s, z, pm = O.make_inputs(n, n_pad=n_pad)
    with torch.no_grad():
        want_s, want_z = ref(s, z, pm)
        sc, zc = s.cuda(), z.cuda()
        with _amp():
            got_s, got_z = prod(sc, zc, pm.cuda())
    assert got_z.dtype == torch.float32 and got_s.dtype == torch.float32
    assert torch.equal(zc.cpu(), z) and torch.equal(sc.cpu(), s)     # inputs untouched
    assert rel_err(got_z, want_z) <= TOL_BF16
    assert rel_err(got_s, want_s) <= TOL_BF16


def test_template_pair_stack_cz64_without_single_track():
    kw = dict(n_blocks=2, c_z=64, c_s=0, num_intermediate_factor=2)
    ref, prod = _pair(O.PairformerStack, P.PairformerStack, **kw)
    n = 90
    z, pm = _z(n, 64, seed=9), pad_mask(n, 6)
    with torch.no_grad():
        _, want = ref(None, z, pm)
        with _amp():
            _, got = prod(None, z.cuda(), pm.cuda())
    assert got.dtype == torch.float32 and rel_err(got, want) <= TOL_BF16


def test_results_do_not_depend_on_workspace_contents_and_are_deterministic():
    _, prod = _pair(O.PairformerBlock, P.PairformerBlock)
    s, z, pm = O.make_inputs(100, n_pad=7)
    outs = []
    try:
        for poison in (False, True, True):
            ops.poison_workspaces = poison
            with torch.no_grad(), _amp():
                outs.append(prod(s.cuda(), z.cuda(), pm.cuda()))
    finally:
        ops.poison_workspaces = False
    for s_o, z_o in outs[1:]:
        assert torch.equal(z_o, outs[0][1]) and torch.equal(s_o, outs[0][0])


def test_c_abi_refuses_mixed_where_no_kernel_is_built():
    lib = _lib.load()
    x = torch.randn(8, 128, device="cuda")
    y = torch.empty_like(x)
    st = torch.cuda.current_stream().cuda_stream
    # LayerNorm has no residual stream
    assert lib.ptx_layernorm_fwd(x.data_ptr(), None, None, y.data_ptr(), None, None, 8, 128, 1e-5,
                                 _lib.PTX_MIXED, st) == 1
    # rows of 256 channels: bf16 arithmetic only (PTX_BF16, PTX_MIXED), not fp32
    z = torch.randn(8, 8, 256, device="cuda")
    w = torch.randn(16, 256, device="cuda")
    out = torch.empty(16, 8, 8, device="cuda")
    assert lib.ptx_pair_bias_fwd(z.data_ptr(), None, None, w.data_ptr(), out.data_ptr(), 8, 256, 16,
                                 1, 1e-5, _lib.PTX_F32, st) == 2
    assert b"256" in lib.ptx_last_error_string()
    assert lib.ptx_pair_bias_fwd(z.data_ptr(), None, None, w.to(BF16).data_ptr(), out.data_ptr(), 8, 256, 16,
                                 1, 1e-5, _lib.PTX_MIXED, st) == 0


# ------------------------------------------------------------------ rows of 256 channels (hidden_scale_up)
@pytest.mark.parametrize("cls", ["TriangleMultiplicationOutgoing", "TriangleMultiplicationIncoming"])
@pytest.mark.parametrize("n,n_pad", [(64, 0), (100, 7), (37, 0)])
def test_trimul_cz256(cls, n, n_pad):
    ref, prod = _pair(getattr(O, cls), getattr(P, cls), 256, 256)
    z = _z(n, 256)
    mask = pad_mask(n, n_pad) if n_pad else None
    mc = None if mask is None else mask.cuda()
    with torch.no_grad():
        want = ref(z, mask)
        with _amp():
            got = prod(z.cuda(), mc)
            zc = z.cuda().clone()
            got2 = prod(zc, mc, inplace_safe=True, _add_with_inplace=True)
    assert got.dtype == BF16 and rel_err(got, want) <= TOL_BF16
    assert got2.data_ptr() == zc.data_ptr() and got2.dtype == torch.float32
    assert torch.equal(got2, z.cuda() + got.float())      # z + bf16(update), exactly


@pytest.mark.parametrize("starting", [True, False])
@pytest.mark.parametrize("n,n_pad", [(64, 0), (100, 7), (37, 5)])
def test_triattn_cz256(starting, n, n_pad):
    ref, prod = _pair(O.TriangleAttention, P.TriangleAttention, 256, 32, 8, starting=starting)
    z = _z(n, 256)
    mask = pad_mask(n, n_pad) if n_pad else None
    mc = None if mask is None else mask.cuda()
    with torch.no_grad():
        want = ref(z, mask, chunk_size=64)
        with _amp():
            got = prod(z.cuda(), mc)
            zc = z.cuda().clone()
            got2 = prod._run(zc, mc, transposed=not starting, residual_inplace=True)
    assert got.dtype == BF16 and rel_err(got, want) <= TOL_BF16
    assert got2.dtype == torch.float32 and torch.equal(got2, z.cuda() + got.float())


@pytest.mark.parametrize("shape,factor", [((1, 50, 50, 256), 4), ((3001, 256), 2)])
def test_transition_cz256(shape, factor):
    ref, prod = _pair(O.Transition, P.Transition, 256, factor)
    x = torch.randn(*shape, generator=torch.Generator().manual_seed(11))
    with torch.no_grad():
        want = ref(x)
        with _amp():
            got = prod(x.cuda())
            xc = x.cuda().clone()
            got2 = prod(xc, _residual_out=xc)
    assert got.dtype == BF16 and rel_err(got, want) <= TOL_BF16
    assert got2.dtype == torch.float32 and torch.equal(got2, x.cuda() + got.float())


@pytest.mark.parametrize("n_blocks", [1, 4])
def test_stack_cz256_scaled_up_runs_on_the_fused_fp32_row_kernels(n_blocks):
    """The scaled-up model (c_z = 256, hidden_scale_up: 8 pair heads, c_hidden_mul = 256;
    configs_model_type.py:52-85, pairformer.py:76-78) with fp32 tensors and parameters under
    bf16 autocast: against the oracle, with the kernel timer and a look at the allocator as
    witnesses that no rounded copy of z and no separate add pass exist any more."""
    kw = dict(n_blocks=n_blocks, c_z=256, hidden_scale_up=True)
    ref, prod = _pair(O.PairformerStack, P.PairformerStack, **kw)
    s, z, pm = O.make_inputs(72, c_z=256, n_pad=5)
    with torch.no_grad():
        want_s, want_z = ref(s, z, pm)
        sc, zc, pc = s.cuda(), z.cuda(), pm.cuda()
        ops.kernel_timer = {}
        try:
            with _amp():
                got_s, got_z = prod(sc, zc, pc)
            seen = {k: len(v) for k, v in ops.kernel_timer.items()}
        finally:
            ops.kernel_timer = None
    assert got_z.dtype == torch.float32 and got_s.dtype == torch.float32
    assert torch.equal(zc.cpu(), z)
    assert rel_err(got_z, want_z) <= TOL_BF16 and rel_err(got_s, want_s) <= TOL_BF16
    assert seen["trimul_project"] == 2 * n_blocks and seen["transition"] == n_blocks
    # the fused path hands the fp32 rows themselves to the kernels
    blk = prod.blocks[0]
    assert ops.compute_dtype(zc) == zc.dtype      # (outside autocast: fp32 arithmetic, refused for this width)
    with _amp():
        assert ops.compute_dtype(zc) == BF16
