"""Pins the CPU oracle (oracle/pairformer_oracle.py) against independent
formulations: float64 brute-force loops written from the AF3 algorithm
statements, library routines (nn.LayerNorm, einsum, SDPA) and invariants chosen
so that a dropped term, a wrong sign/index or a transposed operand fails."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import pairformer_oracle as O

torch.manual_seed(0)
D64 = torch.float64


def _mod(cls, *a, **k):
    m = cls(*a, **k).to(D64)
    O.seed_parameters_(m, seed=7)
    return m.eval()


# ------------------------------------------------------------------ LayerNorm
def test_layer_norm_matches_library_and_closed_forms():
    x = torch.randn(5, 7, 128, dtype=D64)
    w = torch.randn(128, dtype=D64)
    b = torch.randn(128, dtype=D64)
    ref = torch.nn.LayerNorm(128, eps=1e-5).to(D64)
    with torch.no_grad():
        ref.weight.copy_(w)
        ref.bias.copy_(b)
    assert torch.allclose(O.layer_norm(x, w, b), ref(x), atol=1e-12)
    # explicit formula: biased variance, eps inside the sqrt
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    assert torch.allclose(O.layer_norm(x, w, b), (x - mu) / torch.sqrt(var + 1e-5) * w + b, atol=1e-12)
    # constant row -> beta exactly
    c = torch.full((3, 128), 4.25, dtype=D64)
    assert torch.allclose(O.layer_norm(c, w, b), b.expand(3, 128), atol=1e-12)
    # no affine: zero mean, unit (biased) variance up to eps
    y = O.layer_norm(x * 50, None, None)
    assert y.mean(-1).abs().max() < 1e-12
    assert (y.var(-1, unbiased=False) - 1).abs().max() < 1e-6
    # optional scale / offset (create_scale/create_offset = False)
    assert torch.allclose(O.layer_norm(x, w, None), O.layer_norm(x, None, None) * w, atol=1e-12)
    assert torch.allclose(O.layer_norm(x, None, b), O.layer_norm(x, None, None) + b, atol=1e-12)


@pytest.mark.parametrize("affine", [True, False])
def test_layer_norm_backward_matches_autograd_and_finite_differences(affine):
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(2, 9, 24, generator=g, dtype=D64) * 2 + 0.7).requires_grad_(True)
    w = (1 + 0.3 * torch.randn(24, generator=g, dtype=D64)).requires_grad_(True) if affine else None
    b = (0.3 * torch.randn(24, generator=g, dtype=D64)).requires_grad_(True) if affine else None
    dout = torch.randn(2, 9, 24, generator=g, dtype=D64)
    y = F.layer_norm(x, (24,), w, b, 1e-5)
    y.backward(dout)
    dx, dg, db = O.layer_norm_backward(dout, x.detach(), None if w is None else w.detach())
    assert torch.allclose(dx, x.grad, atol=1e-12)
    if affine:
        assert torch.allclose(dg, w.grad, atol=1e-12) and torch.allclose(db, b.grad, atol=1e-12)
    else:
        # without gamma the "parameter gradients" are those of an all-ones gamma / zero beta
        xn = O.layer_norm(x.detach(), None, None)
        assert torch.allclose(dg, (dout * xn).sum((0, 1)), atol=1e-12)
        assert torch.allclose(db, dout.sum((0, 1)), atol=1e-12)
    # central differences on a few coordinates of the scalar <dout, LN(x)>
    f = lambda t: (dout * O.layer_norm(t, None if w is None else w.detach(),
                                       None if b is None else b.detach())).sum()
    x0 = x.detach()
    for idx in [(0, 0, 0), (1, 4, 7), (1, 8, 23)]:
        e = torch.zeros_like(x0)
        e[idx] = 1e-6
        assert abs((f(x0 + e) - f(x0 - e)).item() / 2e-6 - dx[idx].item()) < 1e-6
    # the Jacobian of the normalisation annihilates shifts and (up to eps) rescalings of a row
    assert dx.sum(-1).abs().max() < 1e-12
    xc = x0 - x0.mean(-1, keepdim=True)
    var = (xc ** 2).mean(-1)
    gd = dout * (w.detach() if affine else 1.0)
    expect = (gd * xc).sum(-1) * 1e-5 * torch.rsqrt(var + 1e-5) ** 3   # vanishes with eps
    assert torch.allclose((dx * xc).sum(-1), expect, atol=1e-12)


def test_layer_norm_backward_bf16_arithmetic_in_fp32():
    g = torch.Generator().manual_seed(4)
    x = (torch.randn(50, 128, generator=g) * 3 + 1).bfloat16()
    dout = torch.randn(50, 128, generator=g).bfloat16()
    w = 1 + 0.2 * torch.randn(128, generator=g)
    dx, dg, db = O.layer_norm_backward(dout, x, w)
    assert dx.dtype == dg.dtype == db.dtype == torch.bfloat16
    rx, rg, rb = O.layer_norm_backward(dout.double(), x.double(), w.bfloat16().double())
    for got, ref in ((dx, rx), (dg, rg), (db, rb)):
        assert (got.double() - ref).abs().max() <= 2 ** -8 * ref.abs().max()


def test_layer_norm_bf16_statistics_in_fp32():
    x = (torch.randn(64, 128) * 3 + 10).bfloat16()
    w = torch.randn(128)
    b = torch.randn(128)
    y = O.layer_norm(x, w, b)
    assert y.dtype == torch.bfloat16
    ref = O.layer_norm(x.double(), w.bfloat16().double(), b.bfloat16().double())
    assert (y.double() - ref).abs().max() <= 2 ** -8 * ref.abs().max()


# ------------------------------------------------------------- TriMul
def _trimul_brute(m, z, mask):
    """Algorithms 11/12 of AF3 as written, with python loops."""
    N, c = z.shape[0], m.c_hidden
    zn = F.layer_norm(z, (z.shape[-1],), m.layer_norm_in.weight, m.layer_norm_in.bias, 1e-5)
    a = torch.zeros(N, N, c, dtype=D64)
    b = torch.zeros(N, N, c, dtype=D64)
    for i in range(N):
        for j in range(N):
            v = zn[i, j]
            a[i, j] = mask[i, j] * torch.sigmoid(m.linear_a_g.weight @ v) * (m.linear_a_p.weight @ v)
            b[i, j] = mask[i, j] * torch.sigmoid(m.linear_b_g.weight @ v) * (m.linear_b_p.weight @ v)
    out = torch.zeros_like(z)
    for i in range(N):
        for j in range(N):
            acc = torch.zeros(c, dtype=D64)
            for k in range(N):
                acc += a[i, k] * b[j, k] if m._outgoing else a[k, i] * b[k, j]
            x = F.layer_norm(acc, (c,), m.layer_norm_out.weight, m.layer_norm_out.bias, 1e-5)
            out[i, j] = torch.sigmoid(m.linear_g.weight @ zn[i, j]) * (m.linear_z.weight @ x)
    return out


@pytest.mark.parametrize("cls", [O.TriangleMultiplicationOutgoing, O.TriangleMultiplicationIncoming])
def test_trimul_brute_force(cls):
    N, cz, c = 5, 6, 4
    m = _mod(cls, cz, c)
    z = torch.randn(N, N, cz, dtype=D64)
    mask = (torch.rand(N, N) > 0.3).to(D64)
    got = m(z[None], mask[None])[0]
    assert torch.allclose(got, _trimul_brute(m, z, mask), atol=1e-10)
    # mask=None == ones
    assert torch.allclose(m(z[None]), m(z[None], torch.ones(1, N, N, dtype=D64)), atol=1e-12)


def test_trimul_einsum_duality_equivariance_and_mask():
    N, cz = 7, 8
    out = _mod(O.TriangleMultiplicationOutgoing, cz, cz)
    inc = _mod(O.TriangleMultiplicationIncoming, cz, cz)
    inc.load_state_dict(out.state_dict())
    z = torch.randn(1, N, N, cz, dtype=D64)
    # contraction alone against einsum
    zn = out.layer_norm_in(z)
    a = torch.sigmoid(out.linear_a_g(zn)) * out.linear_a_p(zn)
    b = torch.sigmoid(out.linear_b_g(zn)) * out.linear_b_p(zn)
    x_out = torch.einsum("...ikc,...jkc->...ijc", a, b)
    x_in = torch.einsum("...kic,...kjc->...ijc", a, b)
    fin = lambda mod, x: mod.linear_z(mod.layer_norm_out(x)) * torch.sigmoid(mod.linear_g(zn))
    assert torch.allclose(out(z), fin(out, x_out), atol=1e-11)
    assert torch.allclose(inc(z), fin(inc, x_in), atol=1e-11)
    # duality: the incoming contraction over rows of (a, b) is the outgoing
    # contraction over columns of (a^T, b^T)
    x_dual = torch.einsum("...ikc,...jkc->...ijc", a.transpose(1, 2), b.transpose(1, 2))
    assert torch.allclose(inc(z), fin(out, x_dual), atol=1e-11)
    assert not torch.allclose(inc(z), out(z), atol=1e-3)
    # token-permutation equivariance
    p = torch.randperm(N)
    zp = z[:, p][:, :, p]
    for mod in (out, inc):
        assert torch.allclose(mod(zp), mod(z)[:, p][:, :, p], atol=1e-11)
    # masking token t (row and column) == deleting token t from the sum
    t = 2
    mask = torch.ones(1, N, N, dtype=D64)
    mask[:, t, :] = 0
    mask[:, :, t] = 0
    keep = [i for i in range(N) if i != t]
    zk = z[:, keep][:, :, keep]
    for mod in (out, inc):
        full = mod(z, mask)[:, keep][:, :, keep]
        assert torch.allclose(full, mod(zk), atol=1e-11)
    # zero output projection -> zero update; z + update when asked
    assert torch.allclose(out(z, inplace_safe=True, _add_with_inplace=True), z + out(z), atol=1e-12)
    with pytest.raises(ValueError):
        out(z, triangle_multiplicative="bogus")


# ------------------------------------------------------------- TriAttn
def _triattn_brute(m, x, mask):
    """Algorithm 13 (starting node) with loops, float64."""
    I, J, _ = x.shape
    H, D = m.no_heads, m.c_hidden
    xn = F.layer_norm(x, (x.shape[-1],), m.layer_norm.weight, m.layer_norm.bias, 1e-5)
    q = (xn @ m.mha.linear_q.weight.T).view(I, J, H, D)
    k = (xn @ m.mha.linear_k.weight.T).view(I, J, H, D)
    v = (xn @ m.mha.linear_v.weight.T).view(I, J, H, D)
    g = torch.sigmoid(xn @ m.mha.linear_g.weight.T).view(I, J, H, D)
    tb = xn @ m.linear.weight.T                                      # [I, J, H]
    o = torch.zeros(I, J, H, D, dtype=D64)
    for i in range(I):
        for h in range(H):
            for j in range(J):
                logit = torch.zeros(J, dtype=D64)
                for kk in range(J):
                    logit[kk] = (q[i, j, h] @ k[i, kk, h]) / math.sqrt(D) \
                        + m.inf * (mask[i, kk] - 1) + tb[j, kk, h]
                w = torch.softmax(logit, 0)
                o[i, j, h] = (w[:, None] * v[i, :, h]).sum(0)
    return (o * g).reshape(I, J, H * D) @ m.mha.linear_o.weight.T


def test_triattn_brute_force_and_sdpa():
    I, cz, H, D = 6, 8, 2, 4
    m = _mod(O.TriangleAttention, cz, D, H)
    x = torch.randn(I, I, cz, dtype=D64)
    mask = (torch.rand(I, I) > 0.3).to(D64)
    mask[:, 0] = 1                       # every row keeps one key
    got = m(x[None], mask[None])[0]
    assert torch.allclose(got, _triattn_brute(m, x, mask), atol=1e-9)
    # library routine: SDPA with an additive mask, per (row, head)
    xn = m.layer_norm(x)
    q = m.mha.linear_q(xn).view(I, I, H, D).transpose(1, 2)
    k = m.mha.linear_k(xn).view(I, I, H, D).transpose(1, 2)
    v = m.mha.linear_v(xn).view(I, I, H, D).transpose(1, 2)
    bias = (m.inf * (mask - 1))[:, None, None, :] + m.linear(xn).permute(2, 0, 1)[None]
    o = F.scaled_dot_product_attention(q, k, v, attn_mask=bias, scale=1 / math.sqrt(D))
    o = o.transpose(1, 2) * torch.sigmoid(m.mha.linear_g(xn)).view(I, I, H, D)
    assert torch.allclose(got, m.mha.linear_o(o.reshape(I, I, H * D)), atol=1e-9)


def test_triattn_mask_semantics_chunking_and_ending_node():
    I, cz, H, D = 8, 16, 4, 4
    m = _mod(O.TriangleAttention, cz, D, H).float()
    x = torch.randn(1, I, I, cz)
    tok = torch.ones(I)
    tok[-2:] = 0
    mask = (tok[:, None] * tok[None, :])[None]
    out = m(x, mask)
    # masked keys are inert for rows that keep at least one key
    x2 = x.clone()
    x2[:, :, -2:, :] += 5 * torch.randn(1, I, 2, cz)       # perturb padded keys of every row
    out2 = m(x2, mask)
    assert torch.allclose(out[:, :-2, :-2], out2[:, :-2, :-2], atol=1e-6)
    # fully masked rows: -1e9 absorbs the logits in fp32 -> uniform mean of V over ALL keys
    xn = m.layer_norm(x)
    v = m.mha.linear_v(xn)
    g = torch.sigmoid(m.mha.linear_g(xn))
    expect = m.mha.linear_o(v[:, -2:].mean(2, keepdim=True) * g[:, -2:])
    assert torch.allclose(out[:, -2:], expect, atol=1e-5)
    # chunked == unchunked, any chunk size
    for cs in (1, 3, 8, 64):
        assert torch.allclose(m(x, mask, chunk_size=cs), out, atol=1e-6)
    assert torch.allclose(m(x), m(x, torch.ones(1, I, I)), atol=0)
    # ending node == starting node on the transposed pair tensor
    e = O.TriangleAttention(cz, D, H, starting=False).float()
    e.load_state_dict(m.state_dict())
    mk = (torch.rand(1, I, I) > 0.2).float()
    mk[..., 0, :] = 1
    assert torch.allclose(e(x, mk), m(x.transpose(1, 2), mk.transpose(1, 2)).transpose(1, 2), atol=1e-6)


def test_attention_biases_are_added_to_the_logits():
    """softmax_attention: the biases enter the logits additively, with a plus sign.  With v = I
    the output IS the probability matrix: a per-query constant on every key changes nothing,
    and raising one key's bias by d multiplies its odds by exp(d) exactly."""
    g = torch.Generator().manual_seed(8)
    S, d = 7, 4
    q, k = torch.randn(2, 3, S, d, generator=g, dtype=D64), torch.randn(2, 3, S, d, generator=g, dtype=D64)
    v = torch.eye(S, dtype=D64).expand(2, 3, S, S)
    mb = torch.zeros(2, 1, 1, S, dtype=D64)
    mb[..., 5] = -1e9                                        # a masked key
    tb = torch.randn(1, 3, S, S, generator=g, dtype=D64)
    p0 = O.softmax_attention(q, k, v, [mb, tb])
    assert torch.allclose(p0.sum(-1), torch.ones(2, 3, S, dtype=D64), atol=1e-12)
    assert (p0[..., 5] == 0).all()
    shift = torch.randn(1, 3, S, 1, generator=g, dtype=D64)
    assert torch.allclose(O.softmax_attention(q, k, v, [mb, tb + shift]), p0, atol=1e-12)
    bump = torch.zeros(S, dtype=D64)
    bump[2] = 0.75
    p1 = O.softmax_attention(q, k, v, [mb, tb + bump])
    want = p0 * torch.exp(bump)
    want = want / want.sum(-1, keepdim=True)
    assert torch.allclose(p1, want, atol=1e-12)
    # the logits themselves: q.k with no hidden scale
    a = torch.einsum("bhqd,bhkd->bhqk", q, k) + mb + tb
    assert torch.allclose(p0, torch.softmax(a, -1), atol=1e-12)


# ------------------------------------------------------------- Transition / APB
def test_transition_formula():
    t = _mod(O.Transition, 6, 4)
    x = torch.randn(3, 5, 6, dtype=D64)
    y = F.layer_norm(x, (6,), t.layernorm1.weight, t.layernorm1.bias, 1e-5)
    a = y @ t.linear_no_bias_a.weight.T
    b = y @ t.linear_no_bias_b.weight.T
    ref = ((a / (1 + torch.exp(-a))) * b) @ t.linear_no_bias.weight.T
    assert torch.allclose(t(x), ref, atol=1e-11)
    # long-input path (8 chunks) gives the same values
    xl = torch.randn(3300, 6, dtype=D64)
    assert torch.allclose(t(xl), torch.cat([t(c) for c in xl.split(100)]), atol=1e-11)


def test_attention_pair_bias_against_sdpa():
    N, cs, cz, H = 7, 12, 6, 3
    m = _mod(O.AttentionPairBias, has_s=False, create_offset_ln_z=True, n_heads=H, c_a=cs, c_z=cz)
    with torch.no_grad():
        m.attention.linear_q.bias.copy_(torch.randn(cs, dtype=D64))
    s = torch.randn(1, N, cs, dtype=D64)
    z = torch.randn(1, N, N, cz, dtype=D64)
    a = F.layer_norm(s, (cs,), m.layernorm_a.weight, m.layernorm_a.bias, 1e-5)
    bias = (F.layer_norm(z, (cz,), m.layernorm_z.weight, m.layernorm_z.bias, 1e-5)
            @ m.linear_nobias_z.weight.T).permute(0, 3, 1, 2)
    A = m.attention
    d = cs // H
    q = (a @ A.linear_q.weight.T + A.linear_q.bias).view(1, N, H, d).transpose(1, 2) / math.sqrt(d)
    k = (a @ A.linear_k.weight.T).view(1, N, H, d).transpose(1, 2)
    v = (a @ A.linear_v.weight.T).view(1, N, H, d).transpose(1, 2)
    o = F.scaled_dot_product_attention(q, k, v, attn_mask=bias, scale=1.0).transpose(1, 2).reshape(1, N, cs)
    ref = (o * torch.sigmoid(a @ A.linear_g.weight.T)) @ A.linear_o.weight.T
    # the oracle, like the reference (primitives.py:233-291), forms logits and softmax in fp32
    # whatever the input dtype: fp32 rounding is the floor here, a wrong term gives O(1)
    assert torch.allclose(m(a=s, s=None, z=z), ref, atol=2e-6, rtol=0)


# ------------------------------------------------------------- block / stack
def test_block_composition_and_identity_default():
    N, cz, cs = 6, 8, 12
    blk = _mod(O.PairformerBlock, n_heads=3, c_z=cz, c_s=cs, c_hidden_mul=8, c_hidden_pair_att=4, no_heads_pair=2)
    s = torch.randn(1, N, cs, dtype=D64)
    z = torch.randn(1, N, N, cz, dtype=D64)
    tok = torch.ones(N, dtype=D64)
    tok[-1] = 0
    pm = (tok[:, None] * tok[None, :])[None]
    s1, z1 = blk(s, z, pm)
    # manual composition, ending node expressed with starting=False on the untransposed tensor
    zz = z + blk.tri_mul_out(z, pm)
    zz = zz + blk.tri_mul_in(zz, pm)
    zz = zz + blk.tri_att_start(zz, pm)
    end = O.TriangleAttention(cz, 4, 2, starting=False).to(D64)
    end.load_state_dict(blk.tri_att_end.state_dict())
    zz = zz + end(zz, pm)
    zz = zz + blk.pair_transition(zz)
    ss = s + blk.attention_pair_bias(a=s, s=None, z=zz)
    ss = ss + blk.single_transition(ss)
    assert torch.allclose(z1, zz, atol=1e-10) and torch.allclose(s1, ss, atol=1e-10)
    # flags that must not change values
    s2, z2 = blk(s, z, pm, inplace_safe=True, chunk_size=2)
    assert torch.allclose(z1, z2, atol=1e-10) and torch.allclose(s1, s2, atol=1e-10)
    # zeroed output projections (the reference's default init) -> identity block
    with torch.no_grad():
        for name, p in blk.named_parameters():
            if name.endswith(("linear_z.weight", "linear_o.weight", "linear_no_bias.weight")):
                p.zero_()
    s3, z3 = blk(s, z, pm)
    assert torch.equal(s3, s) and torch.equal(z3, z)
    # c_s = 0 flavour (MSA pair stack) has no single track
    b0 = _mod(O.PairformerBlock, c_z=cz, c_s=0, c_hidden_mul=8, c_hidden_pair_att=4, no_heads_pair=2)
    assert b0(None, z, pm)[0] is None


def test_stack_is_sequential_blocks_and_state_dict_keys():
    st = _mod(O.PairformerStack, n_blocks=2, n_heads=3, c_z=8, c_s=12)
    # PairformerStack does not expose the per-block hidden sizes; the default 128/32x4 are used
    keys = set(st.state_dict().keys())
    for k in ("blocks.0.tri_mul_out.linear_a_p.weight", "blocks.0.tri_mul_in.layer_norm_out.bias",
              "blocks.1.tri_att_start.mha.linear_q.weight", "blocks.1.tri_att_end.linear.weight",
              "blocks.0.pair_transition.linear_no_bias_a.weight",
              "blocks.0.attention_pair_bias.attention.linear_q.bias",
              "blocks.0.attention_pair_bias.layernorm_z.bias",
              "blocks.1.single_transition.layernorm1.weight"):
        assert k in keys, k
    n = sum(p.numel() for p in O.PairformerBlock().parameters())
    assert n == 2 * 98816 + 2 * 82688 + 196864 + 740736 + 1770240
    # the stack is its blocks applied in order, each to the previous one's (s, z)
    O.seed_parameters_(st)
    g = torch.Generator().manual_seed(3)
    s = torch.randn(1, 9, 12, generator=g, dtype=D64)
    z = torch.randn(1, 9, 9, 8, generator=g, dtype=D64)
    pm = (torch.rand(1, 9, 9, generator=g) > 0.2).to(D64)
    s1, z1 = st(s, z, pm)
    s2, z2 = s, z
    for blk in st.blocks:
        s2, z2 = blk(s2, z2, pm)
    assert torch.equal(s1, s2) and torch.equal(z1, z2)
    assert not torch.equal(z1, z)


def test_seeded_inputs_are_deterministic():
    s, z, pm = O.make_inputs(16, n_pad=4)
    s2, z2, pm2 = O.make_inputs(16, n_pad=4)
    assert torch.equal(z, z2) and torch.equal(s, s2)
    assert pm.shape == (1, 16, 16) and pm[0, :12, :12].all() and pm[0, 12:].sum() == 0 and pm[0, :, 12:].sum() == 0
    a = O.seed_parameters_(O.PairformerBlock(c_z=8, c_s=16, n_heads=2, c_hidden_mul=8, c_hidden_pair_att=4, no_heads_pair=2))
    b = O.seed_parameters_(O.PairformerBlock(c_z=8, c_s=16, n_heads=2, c_hidden_mul=8, c_hidden_pair_att=4, no_heads_pair=2))
    for (n1, p1), (_, p2) in zip(a.named_parameters(), b.named_parameters()):
        assert torch.equal(p1, p2), n1
    assert a.attention_pair_bias.attention.linear_q.bias.abs().sum() == 0
    assert (a.tri_mul_out.linear_z.weight.std() * math.sqrt(8) - 1).abs() < 0.3
