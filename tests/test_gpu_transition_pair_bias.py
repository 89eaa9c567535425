"""The pair transition with the pair bias of the following single attention formed in its
epilogue (ptx_transition_pair_bias_fwd) against the two separate kernels it replaces
(ptx_transition_fwd, then ptx_pair_bias_fwd on the stored result) and against torch's own
layer_norm + linear on the stored result; reference: pairformer.py:215-222, transformer.py:191-194."""
import pytest
import torch
import torch.nn.functional as F

import protenix_amd as P
from protenix_amd import ops
from oracle import pairformer_oracle as O
from tests.util import rel_err

pytestmark = pytest.mark.gpu


def _setup(n, mixed, seed):
    g = torch.Generator().manual_seed(seed)
    tr = O.seed_parameters_(O.Transition(128, 4), seed=seed)
    prod = P.Transition(128, 4)
    prod.load_state_dict(tr.state_dict())
    z = torch.randn(n, n, 128, generator=g) * 2
    ln_w = 1 + 0.3 * torch.randn(128, generator=g)
    ln_b = 0.2 * torch.randn(128, generator=g)
    w = torch.randn(16, 128, generator=g) / 11
    dt = torch.float32 if mixed else torch.bfloat16
    prod = prod.to("cuda", dt).eval()
    pbw = tuple(t.to("cuda", torch.bfloat16) for t in (ln_w, ln_b, w))
    return prod, z.to("cuda", dt), pbw


@pytest.mark.parametrize("mixed", [False, True])
@pytest.mark.parametrize("n", [37, 64, 100, 256])
def test_fused_equals_the_two_kernels(mixed, n):
    prod, z, pbw = _setup(n, mixed, seed=n)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16, enabled=mixed):
        assert prod.fuses_pair_bias(z, 16)
        z_sep = prod(z, _residual_new=True)
        bias_sep = ops.pair_bias(z_sep, *pbw, out_f32=True)
        z_fused = z.clone()
        out, bias = prod(z_fused, _residual_out=z_fused, _pair_bias_w=pbw)
    assert out.data_ptr() == z_fused.data_ptr()
    assert torch.equal(z_fused, z_sep)                      # the transition itself: same bits
    bias = bias.view(16, n, n)
    assert bias.dtype == torch.float32 and torch.isfinite(bias).all()
    # same LayerNorm of the same stored rows, other summation order: a bf16 rounding of a
    # normalised value may flip here and there
    assert rel_err(bias, bias_sep) <= 4e-3
    want = F.linear(F.layer_norm(z_sep.float(), (128,), pbw[0].float(), pbw[1].float(), 1e-5),
                    pbw[2].float()).permute(2, 0, 1)
    assert rel_err(bias, want) <= 2e-2
    assert rel_err(bias, want) <= 1.5 * max(rel_err(bias_sep, want), 1e-3)


@pytest.mark.parametrize("mixed", [False, True])
def test_block_with_fused_bias_equals_block_without(mixed, monkeypatch):
    """A Pairformer block end to end: the single representation that comes out with the bias
    from the transition's epilogue against the one with the stand-alone pair-bias kernel."""
    ref = O.seed_parameters_(O.PairformerBlock(), seed=5)
    blk = P.PairformerBlock()
    blk.load_state_dict(ref.state_dict())
    dt = torch.float32 if mixed else torch.bfloat16
    blk = blk.to("cuda", dt).eval()
    s, z, pm = (t.to("cuda", dt) for t in O.make_inputs(96, n_pad=7, dtype=torch.bfloat16))
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16, enabled=mixed):
        s1, z1 = blk(s, z.clone(), pm, inplace_safe=True)
        monkeypatch.setattr(P.primitives.Transition, "fuses_pair_bias", lambda self, x, heads: False)
        s2, z2 = blk(s, z.clone(), pm, inplace_safe=True)
    assert torch.equal(z1, z2)
    # (a bf16 single representation moves by whole bf16 steps: 2^-8 of the value)
    assert rel_err(s1, s2) <= (2e-3 if mixed else 8e-3)


def test_refusals():
    prod, z, pbw = _setup(32, False, seed=1)
    lib = P._lib.load()
    out = torch.empty_like(z)
    bias = torch.empty(16, 32 * 32, device="cuda")
    w = prod._weights(torch.bfloat16, z.device)
    args = [ops._ptr(z), ops._ptr(w["ln_w"]), ops._ptr(w["ln_b"]), ops._ptr(w["packed"]), ops._ptr(out),
            32 * 32, 128, 4, 1, 1e-5, ops._ptr(pbw[0]), ops._ptr(pbw[1]), ops._ptr(pbw[2]), ops._ptr(bias),
            16, 1, 1e-5, P._lib.PTX_BF16, None]
    assert lib.ptx_transition_pair_bias_fwd(*args) == 0
    for idx, bad in ((17, P._lib.PTX_F32), (6, 64), (14, 33), (14, 0)):
        a = list(args)
        a[idx] = bad
        assert lib.ptx_transition_pair_bias_fwd(*a) != 0
    torch.cuda.synchronize()
