"""The single-representation track on HIP kernels, through the C ABI: ptx_linear_fwd (plain,
with bias, with residual, with a transposed tail), ptx_swiglu_fwd and ptx_single_attention_fwd,
against torch's own linear / silu / softmax on the same operands (the calls the reference
makes: primitives.py:83-98, 206-230, 233-291) and the oracle's AttentionPairBias."""
import math

import pytest
import torch
import torch.nn.functional as F

import protenix_amd as P
from oracle import pairformer_oracle as O
from protenix_amd import ops
from tests.util import TOL_BF16, oracle_and_product, rel_err, tol

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def _rand(*shape, dtype, seed, scale=1.0):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,k,n_out", [(768, 384, 384), (37, 384, 1536), (1, 16, 8), (100, 1536, 384),
                                          (65, 48, 40)])
def test_linear(dtype, rows, k, n_out):
    x = _rand(rows, k, dtype=dtype, seed=1)
    w = _rand(n_out, k, dtype=dtype, seed=2, scale=1 / math.sqrt(k))
    b = _rand(n_out, dtype=dtype, seed=3)
    r = _rand(rows, n_out, dtype=dtype, seed=4)
    want = F.linear(x.float(), w.float())
    assert rel_err(ops.linear(x.cuda(), w.cuda()), want) <= tol(dtype)
    assert rel_err(ops.linear(x.cuda(), w.cuda(), bias=b.cuda()), want + b.float()) <= tol(dtype)
    assert rel_err(ops.linear(x.cuda(), w.cuda(), res=r.cuda()), want + r.float()) <= tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [768, 100, 33, 1])
def test_linear_with_transposed_tail(dtype, rows):
    k, n_out, split = 384, 1536, 1152
    x = _rand(rows, k, dtype=dtype, seed=5)
    w = _rand(n_out, k, dtype=dtype, seed=6, scale=1 / math.sqrt(k))
    b = _rand(384, dtype=dtype, seed=7)
    want = F.linear(x.float(), w.float())
    want[:, :384] += b.float()
    head, tail = ops.linear_split(x.cuda(), w.cuda(), b.cuda(), 384, split)
    assert head.shape == (rows, split) and tail.shape == (n_out - split, ((rows + 31) // 32) * 32)
    assert rel_err(head, want[:, :split]) <= tol(dtype)
    assert rel_err(tail[:, :rows], want[:, split:].T) <= tol(dtype)
    assert (tail[:, rows:] == 0).all()          # the padding the attention kernel multiplies by 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,k,hidden", [(768, 384, 1536), (50, 64, 128), (1, 16, 8)])
def test_swiglu(dtype, rows, k, hidden):
    x = _rand(rows, k, dtype=dtype, seed=8)
    wa = _rand(hidden, k, dtype=dtype, seed=9, scale=1 / math.sqrt(k))
    wb = _rand(hidden, k, dtype=dtype, seed=10, scale=1 / math.sqrt(k))
    want = F.silu(F.linear(x.float(), wa.float())) * F.linear(x.float(), wb.float())
    assert rel_err(ops.swiglu(x.cuda(), wa.cuda(), wb.cuda()), want) <= tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bias_dtype", ["fp32", "same", "none"])
@pytest.mark.parametrize("n,heads,d", [(768, 16, 24), (100, 16, 24), (37, 4, 32), (64, 2, 8), (1, 3, 16)])
def test_single_attention(dtype, bias_dtype, n, heads, d):
    hd = heads * d
    qkg = _rand(n, 3 * hd, dtype=dtype, seed=11)
    v = _rand(n, hd, dtype=dtype, seed=12)
    ldt = ((n + 31) // 32) * 32
    vt = torch.zeros(hd, ldt, dtype=dtype)
    vt[:, :n] = v.T
    bias = None if bias_dtype == "none" else _rand(heads, n, n, dtype=torch.float32, seed=13, scale=2.0)
    if bias is not None and bias_dtype == "same":
        bias = bias.to(dtype)
    scale = 1.0 / math.sqrt(d)
    q, k, g = (qkg[:, i * hd:(i + 1) * hd].float().view(n, heads, d).transpose(0, 1) for i in range(3))
    logits = torch.matmul(q, k.transpose(-1, -2)) * scale
    if bias is not None:
        logits = logits + bias.float()
    o = torch.matmul(torch.softmax(logits, -1), v.float().view(n, heads, d).transpose(0, 1))
    want = (o * torch.sigmoid(g)).transpose(0, 1).reshape(n, hd)
    got = ops.single_attention(qkg.cuda(), vt.cuda(), None if bias is None else bias.cuda(), heads, d, scale)
    assert rel_err(got, want) <= tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [768, 130])
def test_attention_pair_bias_module_runs_on_the_hip_kernels(dtype, n):
    """AttentionPairBias (has_s=False) and the c_s = 384 Transition against the oracle, with the
    kernel timer as witness that every step went through the C ABI (no library GEMM, no
    materialised logits)."""
    ref, prod = oracle_and_product(O.AttentionPairBias, P.AttentionPairBias, has_s=False,
                                   create_offset_ln_z=True, n_heads=16, c_a=384, c_z=128, dtype=dtype)
    g = torch.Generator().manual_seed(2)
    a, z = torch.randn(1, n, 384, generator=g).to(dtype), torch.randn(1, n, n, 128, generator=g).to(dtype)
    ops.kernel_timer = {}
    try:
        with torch.no_grad():
            want = ref(a.float(), None, z.float())
            got = prod(a.cuda(), None, z.cuda())
        seen = set(ops.kernel_timer)
    finally:
        ops.kernel_timer = None
    assert {"pair_bias", "layernorm", "linear", "single_attention"} <= seen
    assert rel_err(got, want) <= tol(dtype)
    reft, prodt = oracle_and_product(O.Transition, P.Transition, 384, 4, dtype=dtype)
    ops.kernel_timer = {}
    try:
        with torch.no_grad():
            want = reft(a.float())
            got = prodt(a.cuda())
            got_res = prodt(a.cuda(), _residual_new=True)
        seen = set(ops.kernel_timer)
    finally:
        ops.kernel_timer = None
    assert {"layernorm", "swiglu", "linear"} <= seen
    assert rel_err(got, want) <= tol(dtype)
    assert rel_err(got_res, a.float() + want) <= tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_linear_module_runs_on_the_hip_kernel(dtype):
    """primitives.Linear called on its own (primitives.py:83-98): the HIP kernel, with and
    without bias, with a `precision` override, on batched input, under autocast."""
    x = _rand(3, 50, 384, dtype=dtype, seed=21)
    for bias in (True, False):
        lin = P.primitives.Linear(384, 136, bias=bias)
        with torch.no_grad():
            lin.weight.copy_(_rand(136, 384, dtype=dtype, seed=22, scale=1 / math.sqrt(384)).float())
            if bias:
                lin.bias.copy_(_rand(136, dtype=dtype, seed=23).float())
        want = F.linear(x.float(), lin.weight.float(), lin.bias.float() if bias else None)
        lin = lin.to("cuda", dtype).eval()
        ops.kernel_timer = {}
        try:
            with torch.no_grad():
                got = lin(x.cuda())
            # frozen parameters, grad mode on: still the HIP kernel
            lin.requires_grad_(False)
            got2 = lin(x.cuda())
            assert len(ops.kernel_timer.get("linear", ())) == 2
        finally:
            ops.kernel_timer = None
        assert got.dtype == dtype and got.shape == (3, 50, 136)
        assert rel_err(got, want) <= tol(dtype) and torch.equal(got, got2)
    # precision override: fp32 product of a bf16 input, result in the input's dtype
    lin = P.primitives.Linear(384, 136, bias=False, precision=torch.float32).to("cuda").eval()
    with torch.no_grad():
        y = lin(x.to(torch.bfloat16).cuda())
        want = F.linear(x.to(torch.bfloat16).float(), lin.weight.float().cpu())
    assert y.dtype == torch.bfloat16 and rel_err(y, want) <= TOL_BF16
    # fp32 input and parameters under autocast: bf16 arithmetic and result, as F.linear gives
    lin = P.primitives.Linear(384, 136).to("cuda").eval()
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        y = lin(x.float().cuda())
    assert y.dtype == torch.bfloat16
    want = F.linear(x.float(), lin.weight.float().cpu(), lin.bias.float().cpu())
    assert rel_err(y, want) <= TOL_BF16
    with pytest.raises(RuntimeError, match="forward-only"):
        P.primitives.Linear(384, 136).to("cuda")(x.float().cuda())


@pytest.mark.parametrize("dtype", DTYPES)
def test_single_track_with_frozen_parameters_and_grad_mode_on(dtype):
    """Eval mode with frozen parameters outside torch.no_grad(): the same HIP kernels and the
    same bits as under no_grad (there is no second implementation to fall into)."""
    n = 100
    ref, prod = oracle_and_product(O.AttentionPairBias, P.AttentionPairBias, has_s=False,
                                   create_offset_ln_z=True, n_heads=16, c_a=384, c_z=128, dtype=dtype)
    reft, prodt = oracle_and_product(O.Transition, P.Transition, 384, 4, dtype=dtype)
    g = torch.Generator().manual_seed(3)
    a, z = torch.randn(1, n, 384, generator=g).to(dtype), torch.randn(1, n, n, 128, generator=g).to(dtype)
    with torch.no_grad():
        want, want_t = prod(a.cuda(), None, z.cuda()), prodt(a.cuda())
    prod.requires_grad_(False)
    prodt.requires_grad_(False)
    assert torch.is_grad_enabled()
    ops.kernel_timer = {}
    try:
        got, got_t = prod(a.cuda(), None, z.cuda()), prodt(a.cuda())
        seen = set(ops.kernel_timer)
    finally:
        ops.kernel_timer = None
    assert {"pair_bias", "layernorm", "linear", "single_attention", "swiglu"} <= seen
    assert torch.equal(got, want) and torch.equal(got_t, want_t)


def test_refusals():
    from protenix_amd import _lib
    lib = _lib.load()
    x = torch.zeros(4, 20, device="cuda")
    w = torch.zeros(8, 20, device="cuda")
    with pytest.raises(RuntimeError, match="multiple of 16"):
        ops.linear(x, w)
    qkg = torch.zeros(4, 3 * 40, device="cuda")
    vt = torch.zeros(40, 32, device="cuda")
    with pytest.raises(RuntimeError, match="head dim"):
        ops.single_attention(qkg, vt, None, 1, 40, 1.0)
    assert lib.ptx_linear_fwd(None, None, None, 0, None, None, None, 8, 0, 0, 16, 8, 0, None) == 0   # no rows
