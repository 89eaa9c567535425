"""The fused attention operator on standard-layout tensors (ptx_triattn_core_fwd): the I/O
contract of the reference's TriAttentionFunction (tri_attention/op.py:37-77) and of its caller
_tri_attention (layers.py:539-583), against the oracle's softmax_attention (the reference's
torch-path _attention, layers.py:276-296) on the same operands."""
import math

import pytest
import torch

import protenix_amd as P
from oracle import pairformer_oracle as O
from tests.util import rel_err, tol

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def _operands(B, N, S, H, D, dtype, seed, n_masked=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, N, S, H, D, generator=g) * scale / math.sqrt(D)).to(dtype)
    k = (torch.randn(B, N, S, H, D, generator=g) * scale).to(dtype)
    v = torch.randn(B, N, S, H, D, generator=g).to(dtype)
    mask = torch.ones(B, N, S)
    if n_masked:
        mask[..., S - n_masked:] = 0          # trailing keys padded, in every row
        mask[:, 1] = (torch.rand(B, S, generator=g) > 0.5).float()   # one row with a random key mask
        mask[:, min(2, N - 1)] = 0            # one row with every key masked
    bias1 = (1e9 * (mask - 1)).reshape(B, N, 1, 1, S).to(dtype)
    bias2 = torch.randn(B, 1, H, S, S, generator=g).to(dtype)
    return q, k, v, bias1, bias2


def _reference(q, k, v, bias1, bias2):
    # [B, N, S, H, D] -> the torch path's [B, N, H, S, D]
    qh, kh, vh = (t.float().transpose(-2, -3) for t in (q, k, v))
    o = O.softmax_attention(qh, kh, vh, [bias1.float(), bias2.float()])
    logits = torch.matmul(qh, kh.transpose(-1, -2)) + bias1.float() + bias2.float()
    lse2 = torch.logsumexp(logits, dim=-1) / math.log(2.0)           # [B, N, H, S]
    return o.transpose(-2, -3), lse2.transpose(-1, -2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,N,S,H,n_masked", [(1, 64, 64, 4, 0), (2, 37, 37, 4, 5), (1, 8, 100, 4, 7),
                                              (1, 130, 130, 2, 0), (1, 3, 200, 8, 16)])
def test_against_torch_path_attention(dtype, B, N, S, H, n_masked):
    q, k, v, b1, b2 = _operands(B, N, S, H, 32, dtype, seed=N * 7 + S, n_masked=n_masked)
    want_o, want_m = _reference(q, k, v, b1, b2)
    got_o, got_m = P.tri_attention_forward(q.cuda(), k.cuda(), v.cuda(), b1.cuda(), b2.cuda(),
                                           return_lse=True)
    assert got_o.shape == q.shape and got_o.dtype == dtype
    assert got_m.shape == (B, N, S, H) and got_m.dtype == torch.float32
    assert rel_err(got_o, want_o) <= tol(dtype)
    # LSE: rows whose keys are all masked hold -1e9-sized values; compare where it is informative
    ok = want_m > -1e8
    assert torch.allclose(got_m.cpu()[ok], want_m[ok], atol=2e-5 * (1 if dtype == torch.float32 else 2000),
                          rtol=1e-5 if dtype == torch.float32 else 1e-2)
    # the function-object spelling of the reference
    again = P.TriAttentionFunction.apply(q.cuda(), k.cuda(), v.cuda(), b1.cuda(), b2.cuda())
    assert torch.equal(again, got_o)


def test_large_logits_keep_the_reference_add_order():
    """Logits big enough that (q.k + mask_bias) + tri_bias differs from any other order, rows
    with every key masked (-> mean of v), fp32."""
    q, k, v, b1, b2 = _operands(1, 16, 72, 4, 32, torch.float32, seed=5, n_masked=9, scale=3.0)
    b2 = b2 * 3
    want_o, _ = _reference(q, k, v, b1, b2)
    got = P.tri_attention_forward(q.cuda(), k.cuda(), v.cuda(), b1.cuda(), b2.cuda())
    assert rel_err(got, want_o) <= 1e-4


@pytest.mark.parametrize("dtype", DTYPES)
def test_caller_level_signature_of_layers_tri_attention(dtype):
    """layers.py:539-583: q, k, v arrive as [*, H, Q, C] with one leading batch dim or three,
    the biases broadcastable; the result is [*, Q, H, C]."""
    g = torch.Generator().manual_seed(3)
    for lead in ((50,), (2, 1, 20)):
        S, H, D = 50, 4, 32
        q = (torch.randn(*lead, H, S, D, generator=g) / math.sqrt(D)).to(dtype)
        k = torch.randn(*lead, H, S, D, generator=g).to(dtype)
        v = torch.randn(*lead, H, S, D, generator=g).to(dtype)
        mask = (torch.rand(*lead, S, generator=g) > 0.2).float()
        b1 = (1e9 * (mask - 1))[..., None, None, :].to(dtype)                  # [*, 1, 1, S]
        b2 = torch.randn(*lead[:-1], 1, H, S, S, generator=g).to(dtype)         # [*', 1, H, S, S]
        want = O.softmax_attention(q.float(), k.float(), v.float(), [b1.float(), b2.float()]).transpose(-2, -3)
        got = P.tri_attention(q.cuda(), k.cuda(), v.cuda(), [b1.cuda(), b2.cuda()])
        assert got.shape == want.shape
        assert rel_err(got, want) <= tol(dtype)


def test_equals_the_fused_module_core():
    """The same kernel serves TriangleAttention: feeding the module's own q, k, v and biases
    (computed here with torch from the module's parameters) through the standard-layout entry
    reproduces the module's attention output before gating and output projection."""
    n, H, D = 96, 4, 32
    ref = O.seed_parameters_(O.TriangleAttention(128, D, H)).eval()
    g = torch.Generator().manual_seed(1)
    x = torch.randn(1, n, n, 128, generator=g)
    mask = (torch.rand(1, n, n, generator=g) > 0.1).float()
    with torch.no_grad():
        xn = O.layer_norm(x, ref.layer_norm.weight, ref.layer_norm.bias)
        q = (xn @ ref.mha.linear_q.weight.T).view(1, n, n, H, D) / math.sqrt(D)
        k = (xn @ ref.mha.linear_k.weight.T).view(1, n, n, H, D)
        v = (xn @ ref.mha.linear_v.weight.T).view(1, n, n, H, D)
        b1 = (1e9 * (mask - 1))[:, :, None, None, :]
        b2 = (xn @ ref.linear.weight.T).permute(0, 3, 1, 2)[:, None]
        gate = torch.sigmoid(xn @ ref.mha.linear_g.weight.T)
        o = P.tri_attention_forward(q.cuda(), k.cuda(), v.cuda(), b1.cuda(), b2.cuda()).cpu()
        got = (o.reshape(1, n, n, H * D) * gate) @ ref.mha.linear_o.weight.T
        want = ref(x, mask)
    assert rel_err(got, want) <= 1e-4


def test_refusals():
    from protenix_amd import _lib
    lib = _lib.load()
    t = torch.zeros(1, 4, 4, 2, 16, device="cuda")
    b2 = torch.zeros(1, 1, 2, 4, 4, device="cuda")
    with pytest.raises(RuntimeError, match="head dim 32"):
        P.tri_attention_forward(t, t, t, None, b2)
    with pytest.raises(RuntimeError):
        P.tri_attention_forward(t.cpu(), t.cpu(), t.cpu(), None, b2.cpu())
    assert lib.ptx_triattn_core_workspace_elems(0, 4, 2) == 0
