"""Parity of the HIP path (through the C ABI) against the CPU oracle on the same
seeded inputs.  Reference for every comparison: the fp32 oracle evaluated on the
dtype-rounded inputs and parameters.  Tolerances (BASELINE): fp32 1e-4, bf16 2e-2,
both max-abs error relative to max |reference|."""
import pytest
import torch

import protenix_amd as P
from oracle import pairformer_oracle as O
from tests.util import TOL_BF16, oracle_and_product, pad_mask, rel_err, tol

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def _z(n, dtype, seed=1234, c=128):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(1, n, n, c, generator=g).to(dtype)


# ------------------------------------------------------------------ LayerNorm
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,cols", [(1000, 128), (4099, 128), (77, 384), (33, 64), (19, 100),
                                       (5, 7), (3, 4096), (2, 5000), (0, 128)])
@pytest.mark.parametrize("affine", ["both", "none", "scale", "offset"])
def test_layernorm(dtype, rows, cols, affine):
    g = torch.Generator().manual_seed(rows * 131 + cols)
    x = (torch.randn(rows, cols, generator=g) * 3 + 1.5).to(dtype)
    ln = P.LayerNorm(cols, create_scale=affine in ("both", "scale"),
                     create_offset=affine in ("both", "offset"))
    with torch.no_grad():
        if ln.weight is not None:
            ln.weight.copy_(1 + 0.1 * torch.randn(cols, generator=g))
        if ln.bias is not None:
            ln.bias.copy_(0.1 * torch.randn(cols, generator=g))
    ln = ln.to("cuda", dtype)
    with torch.no_grad():
        y = ln(x.cuda())
    assert y.dtype == dtype and y.shape == x.shape
    if rows == 0:
        return
    w = ln.weight.float().cpu() if ln.weight is not None else None
    b = ln.bias.float().cpu() if ln.bias is not None else None
    ref = O.layer_norm(x.float(), w, b)
    assert rel_err(y, ref) <= (1e-5 if dtype == torch.float32 else 2 ** -7)


@pytest.mark.parametrize("rows,cols", [(1000, 128), (4099, 128), (70001, 128), (77, 384), (19, 100), (5, 7),
                                       (3, 4096), (2, 5000), (0, 128)])
@pytest.mark.parametrize("affine", ["both", "none"])
def test_layernorm_float16(rows, cols, affine):
    """IEEE half, the third dtype the reference's kernel dispatches on
    (layer_norm_cuda_kernel.cu:304-330): forward and backward against the oracle."""
    dtype = torch.float16
    g = torch.Generator().manual_seed(rows * 17 + cols)
    x = (torch.randn(rows, cols, generator=g) * 3 + 1.5).to(dtype)
    dout = torch.randn(rows, cols, generator=g).to(dtype)
    ln = P.LayerNorm(cols, create_scale=affine == "both", create_offset=affine == "both")
    with torch.no_grad():
        if ln.weight is not None:
            ln.weight.copy_(1 + 0.1 * torch.randn(cols, generator=g))
            ln.bias.copy_(0.1 * torch.randn(cols, generator=g))
    ln = ln.to("cuda", dtype)
    xg = x.cuda().requires_grad_(True)
    y = ln(xg)
    assert y.dtype == dtype and y.shape == x.shape
    y.backward(dout.cuda())
    assert xg.grad.dtype == dtype and xg.grad.shape == x.shape
    if rows == 0:
        return
    w = ln.weight.detach().float().cpu() if ln.weight is not None else None
    b = ln.bias.detach().float().cpu() if ln.bias is not None else None
    assert rel_err(y, O.layer_norm(x.float(), w, b)) <= 2 ** -10      # half: 11 significant bits
    dx, dg, db = O.layer_norm_backward(dout.float(), x.float(), w)
    assert rel_err(xg.grad, dx) <= 2e-3
    if w is not None:
        assert rel_err(ln.weight.grad, dg) <= 2e-3 and rel_err(ln.bias.grad, db) <= 2e-3


def test_layernorm_stats_and_closed_forms():
    from protenix_amd import ops
    x = torch.randn(513, 128, device="cuda") * 2 + 3
    y, mean, rstd = ops.layer_norm(x, None, None, 1e-5, return_stats=True)
    assert torch.allclose(mean, x.mean(-1), atol=1e-5)
    assert torch.allclose(rstd, torch.rsqrt(x.var(-1, unbiased=False) + 1e-5), rtol=1e-4)
    beta = torch.randn(128, device="cuda")
    const = torch.full((9, 128), 4.25, device="cuda")
    assert torch.allclose(ops.layer_norm(const, torch.randn(128, device="cuda"), beta), beta.expand(9, 128), atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,cols", [(1000, 128), (4099, 128), (70001, 128), (77, 384), (300, 768),
                                       (33, 64), (64, 449), (19, 100), (5, 7), (3, 4096),
                                       (2, 5000), (0, 128)])
@pytest.mark.parametrize("affine", ["both", "none", "scale", "offset"])
def test_layernorm_backward(dtype, rows, cols, affine):
    """FusedLayerNorm under autograd: input and parameter gradients from the HIP backward
    kernels against the oracle's restatement of the reference's backward arithmetic."""
    g = torch.Generator().manual_seed(rows * 37 + cols)
    x = (torch.randn(rows, cols, generator=g) * 3 + 1.5).to(dtype)
    dout = torch.randn(rows, cols, generator=g).to(dtype)
    ln = P.LayerNorm(cols, create_scale=affine in ("both", "scale"),
                     create_offset=affine in ("both", "offset"))
    with torch.no_grad():
        if ln.weight is not None:
            ln.weight.copy_(1 + 0.1 * torch.randn(cols, generator=g))
        if ln.bias is not None:
            ln.bias.copy_(0.1 * torch.randn(cols, generator=g))
    ln = ln.to("cuda", dtype)
    xg = x.cuda().requires_grad_(True)
    y = ln(xg)
    y.backward(dout.cuda())
    assert xg.grad.shape == x.shape and xg.grad.dtype == dtype
    if rows == 0:
        for p_ in ln.parameters():
            assert torch.count_nonzero(p_.grad) == 0
        return
    w = ln.weight.detach().cpu() if ln.weight is not None else None
    dx, dg, db = O.layer_norm_backward(dout.float(), x.float(), None if w is None else w.float())
    tol = 1e-4 if dtype == torch.float32 else TOL_BF16
    assert rel_err(xg.grad, dx) <= tol
    if ln.weight is not None:
        assert rel_err(ln.weight.grad, dg) <= tol
    if ln.bias is not None:
        assert rel_err(ln.bias.grad, db) <= tol


def test_layernorm_backward_c_abi_options_and_determinism():
    """dgamma / dbeta are optional outputs; the partial sums are added in a fixed order."""
    from protenix_amd import ops
    x = torch.randn(5000, 128, device="cuda").bfloat16()
    dout = torch.randn(5000, 128, device="cuda").bfloat16()
    w = (1 + 0.1 * torch.randn(128, device="cuda")).bfloat16()
    _, mean, rstd = ops.layer_norm(x, w, None, 1e-5, return_stats=True)
    ops.poison_workspaces = True
    try:
        full = ops.layer_norm_backward(dout, x, mean, rstd, w, True, True)
        for need_w, need_b in ((False, False), (True, False), (False, True)):
            dx, dw, db = ops.layer_norm_backward(dout, x, mean, rstd, w, need_w, need_b)
            assert torch.equal(dx, full[0])
            assert (dw is None) == (not need_w) and (db is None) == (not need_b)
            assert dw is None or torch.equal(dw, full[1])
            assert db is None or torch.equal(db, full[2])
        again = ops.layer_norm_backward(dout, x, mean, rstd, w, True, True)
    finally:
        ops.poison_workspaces = False
    assert all(torch.equal(a, b) for a, b in zip(full, again))
    # no gamma: the same as a gamma of ones
    ones = ops.layer_norm_backward(dout, x, mean, rstd, torch.ones_like(w), True, True)
    none = ops.layer_norm_backward(dout, x, mean, rstd, None, True, True)
    assert all(torch.equal(a, b) for a, b in zip(ones, none))


# ------------------------------------------------------------------ TriMul
@pytest.mark.parametrize("mode", ["fp32", "bf16", "mixed"])
@pytest.mark.parametrize("direction", ["outgoing", "incoming"])
@pytest.mark.parametrize("n,n_pad,batch", [(64, 0, 1), (100, 7, 2), (37, 0, 1)])
def test_fused_trimul_operator(mode, direction, n, n_pad, batch):
    """The reference's one-call operator (triangular.py:26-90, call site :497-514): stacked
    input weights, one call; against the oracle module and, bit for bit, the three-stage module."""
    dtype = torch.float32 if mode == "fp32" else torch.bfloat16
    cls = "TriangleMultiplicationOutgoing" if direction == "outgoing" else "TriangleMultiplicationIncoming"
    ref, prod = oracle_and_product(getattr(O, cls), getattr(P, cls), 128, 128, dtype=dtype)
    g = torch.Generator().manual_seed(n + batch)
    z = torch.randn(batch, n, n, 128, generator=g).to(dtype)
    mask = pad_mask(n, n_pad).expand(batch, n, n).contiguous() if n_pad else None
    with torch.no_grad():
        want = ref(z.float(), None if mask is None else mask.float())
    m = prod if mode != "mixed" else prod.float()
    zd = z.cuda() if mode != "mixed" else z.float().cuda()
    md = None if mask is None else mask.to(zd.dtype).cuda()
    args = (m.layer_norm_in.weight, m.layer_norm_in.bias,
            torch.cat([m.linear_a_p.weight, m.linear_b_p.weight], 0),
            torch.cat([m.linear_a_g.weight, m.linear_b_g.weight], 0),
            m.layer_norm_out.weight, m.layer_norm_out.bias, m.linear_z.weight, m.linear_g.weight)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16, enabled=mode == "mixed"):
        got = P.kernel_triangular_mult(zd, direction, md, *args, eps=1e-5)
        staged = m(zd, mask=md)
    assert got.shape == z.shape and got.dtype == staged.dtype
    assert torch.equal(got, staged)
    assert rel_err(got, want) <= tol(dtype)
    with pytest.raises(ValueError):
        P.kernel_triangular_mult(zd, "sideways", md, *args)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cls", ["TriangleMultiplicationOutgoing", "TriangleMultiplicationIncoming"])
@pytest.mark.parametrize("n,n_pad", [(64, 0), (100, 7), (37, 0), (200, 16)])
def test_trimul(dtype, cls, n, n_pad):
    ref, prod = oracle_and_product(getattr(O, cls), getattr(P, cls), 128, 128, dtype=dtype)
    z = _z(n, dtype)
    mask = pad_mask(n, n_pad, dtype) if n_pad else None
    with torch.no_grad():
        want = ref(z.float(), None if mask is None else mask.float())
        got = prod(z.cuda(), None if mask is None else mask.cuda())
        assert rel_err(got, want) <= tol(dtype)
        # z + update, in place
        zc = z.cuda().clone()
        got2 = prod(zc, None if mask is None else mask.cuda(), inplace_safe=True, _add_with_inplace=True)
        assert got2.data_ptr() == zc.data_ptr()
        assert rel_err(got2, z.float() + want) <= tol(dtype)


def test_trimul_random_mask_and_errors():
    ref, prod = oracle_and_product(O.TriangleMultiplicationOutgoing, P.TriangleMultiplicationOutgoing, 128, 128)
    n = 48
    z = _z(n, torch.float32)
    mask = (torch.rand(1, n, n, generator=torch.Generator().manual_seed(3)) > 0.3).float()
    with torch.no_grad():
        assert rel_err(prod(z.cuda(), mask.cuda()), ref(z, mask)) <= 1e-4
        with pytest.raises(ValueError):
            prod(z.cuda(), triangle_multiplicative="bogus")
        with pytest.raises(RuntimeError):
            prod(z)                      # CPU tensor: no silent fallback
    bad = P.TriangleMultiplicationOutgoing(64, 64).cuda()
    with torch.no_grad(), pytest.raises(RuntimeError, match="unsupported"):
        bad(torch.randn(1, 8, 8, 64, device="cuda"))


# ------------------------------------------------------------------ TriAttn
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("starting", [True, False])
@pytest.mark.parametrize("n,n_pad", [(64, 0), (100, 7), (37, 5), (256, 32), (320, 0)])
def test_triattn(dtype, starting, n, n_pad):
    ref, prod = oracle_and_product(O.TriangleAttention, P.TriangleAttention, 128, 32, 4,
                                   starting=starting, dtype=dtype)
    z = _z(n, dtype)
    mask = pad_mask(n, n_pad, dtype) if n_pad else None
    with torch.no_grad():
        want = ref(z.float(), None if mask is None else mask.float(), chunk_size=64)
        got = prod(z.cuda(), None if mask is None else mask.cuda())
    # padded query rows (fully masked keys) are included: they must equal the
    # reference's mean-of-v behaviour too
    assert rel_err(got, want) <= tol(dtype)


def test_triattn_random_mask_large_logits():
    """Random key masks, rows with every key masked, and logits big enough that
    the -1e9 absorption and the order of the two bias adds matter."""
    ref, prod = oracle_and_product(O.TriangleAttention, P.TriangleAttention, 128, 32, 4)
    n = 72
    z = _z(n, torch.float32) * 4
    g = torch.Generator().manual_seed(5)
    mask = (torch.rand(1, n, n, generator=g) > 0.4).float()
    mask[0, 3] = 0
    mask[0, 70] = 0
    with torch.no_grad():
        for p_ref, p_prod in ((ref.linear, prod.linear), (ref.mha.linear_q, prod.mha.linear_q)):
            p_ref.weight.mul_(3)
            p_prod.weight.mul_(3)
        want = ref(z, mask)
        got = prod(z.cuda(), mask.cuda())
    assert rel_err(got, want) <= 1e-4


@pytest.mark.parametrize("starting", [True, False])
def test_triattn_mask_changed_in_place_and_replaced(starting):
    """The converted (and, for the ending node, transposed) copy of a mask is kept between
    calls: a mask edited in place, and a new mask tensor of the same shape, must each be seen.
    Non-symmetric masks, so that a missed transpose shows as well."""
    ref, prod = oracle_and_product(O.TriangleAttention, P.TriangleAttention, 128, 32, 4, starting=starting)
    n = 80
    z = _z(n, torch.float32)
    g = torch.Generator().manual_seed(11)
    mask = (torch.rand(1, n, n, generator=g) > 0.3).float()
    mask_dev = mask.cuda()
    with torch.no_grad():
        assert rel_err(prod(z.cuda(), mask_dev), ref(z, mask)) <= 1e-4
        assert rel_err(prod(z.cuda(), mask_dev), ref(z, mask)) <= 1e-4      # served from the kept copy
        mask[0, :, 5] = 0
        mask[0, 7, :] = 1
        mask_dev[0, :, 5] = 0                                               # in place: same tensor
        mask_dev[0, 7, :] = 1
        assert rel_err(prod(z.cuda(), mask_dev), ref(z, mask)) <= 1e-4
        other = (torch.rand(1, n, n, generator=g) > 0.5).float()
        del mask_dev
        assert rel_err(prod(z.cuda(), other.cuda()), ref(z, other)) <= 1e-4  # a new tensor, maybe the old address
        assert rel_err(prod(z.cuda(), other.bool().cuda()), ref(z, other)) <= 1e-4


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_all_ones_mask_is_no_mask(dtype):
    """A mask of all ones is handed to the kernels as "no mask" (decided once per mask): the same
    bits as with the mask loaded and applied, which is what a capturing stream still does."""
    ref, prod = oracle_and_product(O.PairformerBlock, P.PairformerBlock, dtype=dtype)
    s, z, pm = (t.cuda() for t in O.make_inputs(70, dtype=dtype))
    with torch.no_grad():
        s0, z0 = prod(s, z, None)
        s1, z1 = prod(s, z, pm)
        P.ops._mask_cache.clear()
        keep = torch.cuda.is_current_stream_capturing
        torch.cuda.is_current_stream_capturing = lambda: True      # the mask is then used unexamined
        try:
            s2, z2 = prod(s, z, pm.clone())
        finally:
            torch.cuda.is_current_stream_capturing = keep
            P.ops._mask_cache.clear()
    assert torch.equal(z0, z1) and torch.equal(s0, s1)
    assert torch.equal(z0, z2) and torch.equal(s0, s2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_triattn_nan_stays_where_the_reference_puts_it(dtype):
    """A NaN at z[i0, j0] reaches, in the reference, row i0 (a poisoned key of that row) and the
    queries at position i0 of every row (their triangle bias).  The fast softmax paths of the
    attention core must not spread it any further, and everything else must still be right."""
    ref, prod = oracle_and_product(O.TriangleAttention, P.TriangleAttention, 128, 32, 4, dtype=dtype)
    n, i0, j0 = 160, 37, 101
    z = _z(n, dtype)
    z[0, i0, j0, 5] = float("nan")
    with torch.no_grad():
        want = ref(z.float(), None)
        got = prod(z.cuda(), None).float().cpu()
    bad = torch.isnan(want).any(-1)[0]
    expect = torch.zeros(n, n, dtype=torch.bool)
    expect[i0, :] = True
    expect[:, i0] = True
    assert torch.equal(bad, expect)                       # the oracle's own spread, as derived
    assert torch.isnan(got[0][expect]).any(-1).all()      # poisoned where the reference is
    clean = ~expect
    assert torch.isfinite(got[0][clean]).all()
    err = (got[0][clean] - want[0][clean]).abs().max() / want[0][clean].abs().max()
    assert err <= tol(dtype)


# ------------------------------------------------------------------ Transition / pair bias
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(1, 50, 50, 128), (3001, 128), (1, 64, 384)])
def test_transition(dtype, shape):
    ref, prod = oracle_and_product(O.Transition, P.Transition, shape[-1], 4, dtype=dtype)
    x = torch.randn(*shape, generator=torch.Generator().manual_seed(11)).to(dtype)
    with torch.no_grad():
        assert rel_err(prod(x.cuda()), ref(x.float())) <= tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_pair_bias(dtype):
    kw = dict(has_s=False, create_offset_ln_z=True, n_heads=16, c_a=384, c_z=128)
    ref, prod = oracle_and_product(O.AttentionPairBias, P.AttentionPairBias, dtype=dtype, **kw)
    n = 70
    z = _z(n, dtype)
    s = torch.randn(1, n, 384, generator=torch.Generator().manual_seed(2)).to(dtype)
    with torch.no_grad():
        bias = prod.pair_bias(z.cuda())
        want_bias = ref.linear_nobias_z(ref.layernorm_z(z.float())).permute(0, 3, 1, 2)
        assert bias.dtype == torch.float32
        assert rel_err(bias, want_bias) <= tol(dtype)
        assert rel_err(prod(a=s.cuda(), s=None, z=z.cuda()), ref(a=s.float(), s=None, z=z.float())) <= tol(dtype)


# ------------------------------------------------------------------ block / stack
def test_block_c1_fp32_n64():
    """BASELINE config 1: one PairformerBlock, fp32, N=64, mask of ones."""
    ref, prod = oracle_and_product(O.PairformerBlock, P.PairformerBlock)
    s, z, pm = O.make_inputs(64)
    with torch.no_grad():
        s_ref, z_ref = ref(s, z, pm)
        zc = z.cuda()
        s_got, z_got = prod(s.cuda(), zc, pm.cuda())
        assert torch.equal(zc.cpu(), z), "inputs must stay untouched without inplace_safe"
        assert rel_err(z_got, z_ref) <= 1e-4 and rel_err(s_got, s_ref) <= 1e-4
        s2, z2 = prod(s.cuda(), zc, None, inplace_safe=True)
        assert z2.data_ptr() == zc.data_ptr()
        assert rel_err(z2, z_ref) <= 1e-4 and rel_err(s2, s_ref) <= 1e-4


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,n_pad", [(96, 9), (130, 0)])
def test_block_masked(dtype, n, n_pad):
    ref, prod = oracle_and_product(O.PairformerBlock, P.PairformerBlock, dtype=dtype)
    s, z, pm = O.make_inputs(n, n_pad=n_pad, dtype=dtype)
    with torch.no_grad():
        s_ref, z_ref = ref(s.float(), z.float(), pm.float())
        s_got, z_got = prod(s.cuda(), z.cuda(), pm.cuda())
    assert rel_err(z_got, z_ref) <= tol(dtype) and rel_err(s_got, s_ref) <= tol(dtype)


def test_block_without_single_track():
    ref, prod = oracle_and_product(O.PairformerBlock, P.PairformerBlock, c_s=0)
    _, z, pm = O.make_inputs(40, n_pad=3)
    with torch.no_grad():
        s_got, z_got = prod(None, z.cuda(), pm.cuda())
        assert s_got is None and rel_err(z_got, ref(None, z, pm)[1]) <= 1e-4


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_batched_and_noncontiguous_inputs(dtype):
    """Leading batch dimensions, a non-contiguous pair tensor (a transposed view, as
    pairformer.py:201 produces it), a boolean-valued mask in another dtype: the caller's
    tensors are left untouched unless inplace_safe is set."""
    ref, prod = oracle_and_product(O.PairformerBlock, P.PairformerBlock, dtype=dtype)
    n = 48
    g = torch.Generator().manual_seed(99)
    z = torch.randn(2, n, n, 128, generator=g).to(dtype)
    s = torch.randn(2, n, 384, generator=g).to(dtype)
    pm = torch.stack([pad_mask(n, 5)[0], pad_mask(n, 0)[0]])           # fp32, per-sample padding
    with torch.no_grad():
        s_ref, z_ref = ref(s.float(), z.float(), pm)
        z_dev = z.cuda().transpose(1, 2).contiguous().transpose(1, 2)   # same values, strided
        assert not z_dev.is_contiguous()
        z_keep = z_dev.clone()
        s_got, z_got = prod(s.cuda(), z_dev, pm.cuda())
    assert torch.equal(z_dev, z_keep)
    assert rel_err(z_got, z_ref) <= tol(dtype) and rel_err(s_got, s_ref) <= tol(dtype)
    # each sample on its own gives the same answer as inside the batch
    with torch.no_grad():
        s1, z1 = prod(s[1:].cuda(), z[1:].cuda(), pm[1:].cuda())
    assert torch.equal(z1, z_got[1:]) and torch.equal(s1, s_got[1:])


@pytest.mark.parametrize("dtype", DTYPES)
def test_stack_4_blocks(dtype):
    ref, prod = oracle_and_product(O.PairformerStack, P.PairformerStack, n_blocks=4, dtype=dtype)
    s, z, pm = O.make_inputs(80, n_pad=6, dtype=dtype)
    with torch.no_grad():
        s_ref, z_ref = ref(s.float(), z.float(), pm.float())
        s_got, z_got = prod(s.cuda(), z.cuda(), pm.cuda())
    assert rel_err(z_got, z_ref) <= tol(dtype) and rel_err(s_got, s_ref) <= tol(dtype)


# ------------------------------------------------------------------ c_z = 64 (the template embedder's pair stack)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cls", ["TriangleMultiplicationOutgoing", "TriangleMultiplicationIncoming"])
@pytest.mark.parametrize("n,n_pad", [(64, 0), (100, 7), (37, 0)])
def test_trimul_cz64(dtype, cls, n, n_pad):
    """c_z = 64 with the default c_hidden_mul = 128 (pairformer.py:969-977 of the reference)."""
    ref, prod = oracle_and_product(getattr(O, cls), getattr(P, cls), 64, 128, dtype=dtype)
    z = _z(n, dtype, c=64)
    mask = pad_mask(n, n_pad, dtype) if n_pad else None
    with torch.no_grad():
        want = ref(z.float(), None if mask is None else mask.float())
        got = prod(z.cuda(), None if mask is None else mask.cuda())
        assert got.shape == want.shape and rel_err(got, want) <= tol(dtype)
        zc = z.cuda().clone()
        got2 = prod(zc, None if mask is None else mask.cuda(), inplace_safe=True, _add_with_inplace=True)
        assert got2.data_ptr() == zc.data_ptr()
        assert rel_err(got2, z.float() + want) <= tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("starting", [True, False])
@pytest.mark.parametrize("n,n_pad", [(64, 0), (100, 7), (37, 5)])
def test_triattn_cz64(dtype, starting, n, n_pad):
    ref, prod = oracle_and_product(O.TriangleAttention, P.TriangleAttention, 64, 32, 4,
                                   starting=starting, dtype=dtype)
    z = _z(n, dtype, c=64)
    mask = pad_mask(n, n_pad, dtype) if n_pad else None
    with torch.no_grad():
        want = ref(z.float(), None if mask is None else mask.float(), chunk_size=64)
        got = prod(z.cuda(), None if mask is None else mask.cuda())
    assert got.shape == want.shape and rel_err(got, want) <= tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,factor", [((1, 50, 50, 64), 2), ((3001, 64), 4), ((77, 64), 1)])
def test_transition_cz64(dtype, shape, factor):
    ref, prod = oracle_and_product(O.Transition, P.Transition, 64, factor, dtype=dtype)
    x = torch.randn(*shape, generator=torch.Generator().manual_seed(11)).to(dtype)
    with torch.no_grad():
        assert rel_err(prod(x.cuda()), ref(x.float())) <= tol(dtype)
        xc = x.cuda().clone()
        got = prod(xc, _residual_out=xc)
        assert got.data_ptr() == xc.data_ptr()
        assert rel_err(got, x.float() + ref(x.float())) <= tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_template_pair_stack_cz64(dtype):
    """The stack as the template embedder builds it: c_z = 64, no single track, two blocks,
    transition factor 2 (pairformer.py:969-977 of the reference)."""
    kw = dict(n_blocks=2, c_z=64, c_s=0, num_intermediate_factor=2)
    ref, prod = oracle_and_product(O.PairformerStack, P.PairformerStack, dtype=dtype, **kw)
    _, z, pm = O.make_inputs(90, c_z=64, n_pad=6, dtype=dtype)
    with torch.no_grad():
        _, z_ref = ref(None, z.float(), pm.float())
        s_got, z_got = prod(None, z.cuda(), pm.cuda())
    assert s_got is None and rel_err(z_got, z_ref) <= tol(dtype)


# ------------------------------------------------------------------ c_z = 256 (scaled-up hidden widths, bf16)
BF16 = torch.bfloat16


@pytest.mark.parametrize("cls", ["TriangleMultiplicationOutgoing", "TriangleMultiplicationIncoming"])
@pytest.mark.parametrize("n,n_pad", [(64, 0), (100, 7), (37, 0)])
def test_trimul_cz256(cls, n, n_pad):
    """c_z = c_hidden = 256, as `hidden_scale_up` gives (pairformer.py:76-78 of the reference)."""
    ref, prod = oracle_and_product(getattr(O, cls), getattr(P, cls), 256, 256, dtype=BF16)
    z = _z(n, BF16, c=256)
    mask = pad_mask(n, n_pad, BF16) if n_pad else None
    with torch.no_grad():
        want = ref(z.float(), None if mask is None else mask.float())
        got = prod(z.cuda(), None if mask is None else mask.cuda())
        assert got.shape == want.shape and rel_err(got, want) <= tol(BF16)
        zc = z.cuda().clone()
        got2 = prod(zc, None if mask is None else mask.cuda(), inplace_safe=True, _add_with_inplace=True)
        assert rel_err(got2, z.float() + want) <= tol(BF16)


@pytest.mark.parametrize("starting", [True, False])
@pytest.mark.parametrize("n,n_pad", [(64, 0), (100, 7), (37, 5)])
def test_triattn_cz256(starting, n, n_pad):
    ref, prod = oracle_and_product(O.TriangleAttention, P.TriangleAttention, 256, 32, 8,
                                   starting=starting, dtype=BF16)
    z = _z(n, BF16, c=256)
    mask = pad_mask(n, n_pad, BF16) if n_pad else None
    with torch.no_grad():
        want = ref(z.float(), None if mask is None else mask.float(), chunk_size=64)
        got = prod(z.cuda(), None if mask is None else mask.cuda())
    assert got.shape == want.shape and rel_err(got, want) <= tol(BF16)


@pytest.mark.parametrize("shape,factor", [((1, 50, 50, 256), 4), ((3001, 256), 2)])
def test_transition_cz256(shape, factor):
    ref, prod = oracle_and_product(O.Transition, P.Transition, 256, factor, dtype=BF16)
    x = torch.randn(*shape, generator=torch.Generator().manual_seed(11)).to(BF16)
    with torch.no_grad():
        assert rel_err(prod(x.cuda()), ref(x.float())) <= tol(BF16)
        xc = x.cuda().clone()
        got = prod(xc, _residual_out=xc)
        assert rel_err(got, x.float() + ref(x.float())) <= tol(BF16)


def test_block_cz256_scaled_up():
    """A block as the scaled-up model builds it: c_z = 256, hidden_scale_up (8 pair heads,
    c_hidden_mul = 256), with the single track."""
    kw = dict(c_z=256, hidden_scale_up=True)
    ref, prod = oracle_and_product(O.PairformerBlock, P.PairformerBlock, dtype=BF16, **kw)
    s, z, pm = O.make_inputs(72, c_z=256, n_pad=5, dtype=BF16)
    with torch.no_grad():
        s_ref, z_ref = ref(s.float(), z.float(), pm.float())
        s_got, z_got = prod(s.cuda(), z.cuda(), pm.cuda())
    assert rel_err(z_got, z_ref) <= tol(BF16) and rel_err(s_got, s_ref) <= tol(BF16)


def test_cz256_fp32_is_refused():
    """fp32 arithmetic on rows of 256 channels has no kernels (fp32 rows under bf16 autocast
    have: tests/test_gpu_mixed.py)."""
    blk = P.TriangleMultiplicationOutgoing(256, 256).cuda()
    with torch.no_grad(), pytest.raises(RuntimeError, match="unsupported"):
        blk(torch.randn(1, 8, 8, 256, device="cuda"))


# ------------------------------------------------------------------ workspaces
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,n_pad", [(100, 7), (72, 0), (37, 5)])
def test_results_do_not_depend_on_workspace_contents(dtype, n, n_pad):
    """The kernels get their workspaces uninitialised; filled with NaN instead, every module
    must return bit-identical results (tails beyond N are never read into a result, nor into
    a decision that changes the rounding of one)."""
    from protenix_amd import ops
    z = _z(n, dtype).cuda()
    mask = pad_mask(n, n_pad, dtype).cuda() if n_pad else None
    mods = [P.TriangleMultiplicationOutgoing(128, 128), P.TriangleMultiplicationIncoming(128, 128),
            P.TriangleAttention(128, 32, 4, starting=True), P.TriangleAttention(128, 32, 4, starting=False)]
    for mod in mods:
        O.seed_parameters_(mod)
        mod = mod.to("cuda", dtype).eval()
        with torch.no_grad():
            want = mod(z, mask)
            ops.poison_workspaces = True
            try:
                got = mod(z, mask)
            finally:
                ops.poison_workspaces = False
        assert torch.equal(got, want), type(mod).__name__


# ------------------------------------------------------------------ smallest and odd sizes
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,n_pad", [(1, 0), (2, 1), (5, 0), (17, 1), (33, 0), (65, 1), (127, 0), (129, 1)])
def test_block_edge_sizes(dtype, n, n_pad):
    """One block at sizes around the 32-row / 64-key tile edges, down to a single token."""
    ref, prod = oracle_and_product(O.PairformerBlock, P.PairformerBlock, dtype=dtype)
    s, z, pm = O.make_inputs(n, n_pad=n_pad, seed=9 + n, dtype=dtype)
    pm = pm if n_pad else None
    with torch.no_grad():
        s_ref, z_ref = ref(s.float(), z.float(), None if pm is None else pm.float())
        s_got, z_got = prod(s.cuda(), z.cuda(), None if pm is None else pm.cuda())
    assert rel_err(z_got, z_ref) <= tol(dtype) and rel_err(s_got, s_ref) <= tol(dtype)
