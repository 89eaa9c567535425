"""Backward of the fused attention operator (ptx_triattn_core_bwd behind
TriAttentionFunction): dQ, dK, dV and dBias2 against torch autograd through the oracle's
softmax_attention (the reference's torch-path _attention, layers.py:276-296) on the same
operands; the contract is the reference's TriAttentionFunction.backward
(tri_attention/op.py:79-163).  Rows whose every key is masked are left out of the operands: their
log-sum-exp is about -1.4e9, where fp32 no longer resolves log2 of the key count, so the
reference's M format itself carries no usable gradient for them."""
import math

import pytest
import torch

import protenix_amd as P
from oracle import pairformer_oracle as O
from tests.util import rel_err, tol

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def _operands(B, N, S, H, dtype, seed, n_masked=0, b2_batch=None):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, N, S, H, 32, generator=g) / math.sqrt(32)).to(dtype)
    k = torch.randn(B, N, S, H, 32, generator=g).to(dtype)
    v = torch.randn(B, N, S, H, 32, generator=g).to(dtype)
    do = torch.randn(B, N, S, H, 32, generator=g).to(dtype)
    mask = torch.ones(B, N, S)
    if n_masked:
        mask[..., S - n_masked:] = 0
        mask[:, 1] = (torch.rand(B, S, generator=g) > 0.5).float()
        mask[:, 1, 0] = 1                          # never a row with every key masked
    b1 = (1e9 * (mask - 1)).reshape(B, N, 1, 1, S).to(dtype)
    b2 = torch.randn(B if b2_batch is None else b2_batch, 1, H, S, S, generator=g).to(dtype)
    return q, k, v, b1, b2, do


def _autograd_reference(q, k, v, b1, b2, do):
    q, k, v, b2 = (t.float().clone().requires_grad_(True) for t in (q, k, v, b2))
    o = O.softmax_attention(q.transpose(-2, -3), k.transpose(-2, -3), v.transpose(-2, -3),
                            [b1.float(), b2]).transpose(-2, -3)
    o.backward(do.float())
    return o.detach(), q.grad, k.grad, v.grad, b2.grad


def _product(q, k, v, b1, b2, do, grad_b2=True):
    q, k, v, b2 = (t.cuda().requires_grad_(r) for t, r in ((q, True), (k, True), (v, True), (b2, grad_b2)))
    o = P.TriAttentionFunction.apply(q, k, v, b1.cuda(), b2)
    o.backward(do.cuda())
    return o.detach(), q.grad, k.grad, v.grad, b2.grad


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,N,S,H,n_masked", [(1, 32, 32, 4, 0), (1, 64, 64, 4, 0), (2, 37, 37, 4, 5),
                                              (1, 8, 100, 2, 7), (1, 130, 130, 2, 0), (1, 3, 200, 8, 16)])
def test_gradients_against_autograd_of_the_torch_path(dtype, B, N, S, H, n_masked):
    ops = _operands(B, N, S, H, dtype, seed=N * 11 + S, n_masked=n_masked)
    want = _autograd_reference(*ops)
    got = _product(*ops)
    for name, g, w in zip(("O", "dQ", "dK", "dV", "dBias2"), got, want):
        assert g.shape == w.shape and g.dtype == dtype, name
        # dBias2 sums N rows of bf16-rounded products: allow the rounding of the sum itself
        assert rel_err(g, w) <= tol(dtype), name


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,S", [(5, 96), (3, 50)])
def test_no_bias1_is_a_bias1_of_zeros(dtype, N, S):
    """Without a mask bias the kernels read a row of Bias2 in its place and weigh it with zero:
    same gradients as with a Bias1 of zeros, and as the torch path's."""
    q, k, v, b1, b2, do = _operands(1, N, S, 2, dtype, seed=S)
    want = _autograd_reference(q, k, v, b1, b2, do)
    with_zeros = _product(q, k, v, b1, b2, do)
    qc, kc, vc, b2c = (t.cuda().requires_grad_(True) for t in (q, k, v, b2))
    P.TriAttentionFunction.apply(qc, kc, vc, None, b2c).backward(do.cuda())
    for name, g, z, w in zip(("dQ", "dK", "dV", "dBias2"), (qc.grad, kc.grad, vc.grad, b2c.grad),
                             with_zeros[1:], want[1:]):
        assert torch.equal(g, z), name
        assert rel_err(g, w) <= tol(dtype), name


@pytest.mark.parametrize("dtype", DTYPES)
def test_bias2_broadcast_over_the_batch_and_not_requiring_grad(dtype):
    ops = _operands(2, 16, 40, 4, dtype, seed=9, n_masked=3, b2_batch=1)
    want = _autograd_reference(*ops)
    got = _product(*ops)
    assert got[4].shape == ops[4].shape
    for g, w in zip(got, want):
        assert rel_err(g, w) <= tol(dtype)
    skipped = _product(*ops, grad_b2=False)
    assert skipped[4] is None
    for a, b in zip(skipped[:4], got[:4]):
        assert torch.equal(a, b)


def test_caller_level_function_differentiates():
    """layers.py:539-583 spelling: q, k, v [*, H, Q, C], the result [*, Q, H, C]."""
    g = torch.Generator().manual_seed(2)
    S, H = 48, 4
    q = (torch.randn(S, H, S, 32, generator=g) / math.sqrt(32))
    k, v = torch.randn(S, H, S, 32, generator=g), torch.randn(S, H, S, 32, generator=g)
    b1 = torch.zeros(S, 1, 1, S)
    b2 = torch.randn(1, H, S, S, generator=g)
    do = torch.randn(S, S, H, 32, generator=g)
    ref = [t.clone().requires_grad_(True) for t in (q, k, v, b2)]
    O.softmax_attention(ref[0], ref[1], ref[2], [b1, ref[3]]).transpose(-2, -3).backward(do)
    dev = [t.cuda().requires_grad_(True) for t in (q, k, v, b2)]
    P.tri_attention(dev[0], dev[1], dev[2], [b1.cuda(), dev[3]]).backward(do.cuda())
    for a, b in zip(dev, ref):
        assert a.grad.shape == b.grad.shape
        assert rel_err(a.grad, b.grad) <= 1e-4


def test_bias1_requiring_grad_is_refused():
    q, k, v, b1, b2, _ = _operands(1, 4, 32, 2, torch.float32, seed=1)
    with pytest.raises(RuntimeError, match="Bias1"):
        P.TriAttentionFunction.apply(q.cuda(), k.cuda(), v.cuda(), b1.cuda().requires_grad_(True), b2.cuda())


@pytest.mark.parametrize("dtype", DTYPES)
def test_full_size_invariants(dtype):
    """N = S = 768, 4 heads (the benchmark's attention shape), where autograd on the CPU is out
    of reach: (1) dS sums to zero over the keys of every (row, query, head), so dBias2 summed
    over keys is the rounding noise of 768 rows; (2) the operator is linear in dO; (3) a
    64-row slice agrees with autograd on the CPU."""
    N = S = 768
    q, k, v, b1, b2, do = _operands(1, N, S, 4, dtype, seed=77, n_masked=40)
    _, dq, dk, dv, db2 = _product(q, k, v, b1, b2, do)
    scale = db2.float().abs().max().item()
    assert db2.float().sum(-1).abs().max().item() <= (5e-4 if dtype == torch.float32 else 1.0) * scale
    _, dq2, dk2, dv2, db22 = _product(q, k, v, b1, b2, (2 * do.float()).to(dtype))
    for a, b in ((dq, dq2), (dk, dk2), (dv, dv2), (db2, db22)):
        assert rel_err(2 * a.float(), b.float()) <= (1e-5 if dtype == torch.float32 else 1e-2)
    sl = slice(100, 164)
    want = _autograd_reference(q[:, sl], k[:, sl], v[:, sl], b1[:, sl], b2, do[:, sl])
    for g, w in zip((dq, dk, dv), want[1:4]):
        assert rel_err(g[:, sl], w) <= tol(dtype)
