"""HIP-graph replay of the stack (protenix_amd.Graphed) against the eager path: every replay is
checked, with eager work and synchronisations between the replays."""
import pytest
import torch

import protenix_amd as P
from oracle import pairformer_oracle as O
from tests.util import rel_err

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _stack(dtype, **kw):
    ref = O.seed_parameters_(O.PairformerStack(**kw))
    st = P.PairformerStack(**kw)
    st.load_state_dict(ref.state_dict())
    return st.to("cuda", dtype).eval()


@pytest.mark.parametrize("dtype", [torch.float32, BF16])
def test_graphed_stack_replays_match_eager(dtype):
    st = _stack(dtype, n_blocks=3)
    fast = P.Graphed(st)
    for n, n_pad in ((64, 0), (100, 7)):
        for rep in range(3):
            s, z, pm = O.make_inputs(n, n_pad=n_pad, seed=100 + 7 * rep + n, dtype=dtype)
            s, z, pm = s.cuda(), z.cuda(), (pm.cuda() if n_pad else None)
            z0, s0 = z.clone(), s.clone()
            with torch.no_grad():
                s_ref, z_ref = st(s, z, pm)           # eager, between replays
                torch.cuda.synchronize()
                s_got, z_got = fast(s, z, pm)
                torch.cuda.synchronize()
            assert torch.equal(z, z0) and torch.equal(s, s0)          # inputs untouched
            # the same kernels on the same values: bit-identical
            assert torch.equal(z_got, z_ref), (n, rep, rel_err(z_got, z_ref))
            assert torch.equal(s_got, s_ref), (n, rep, rel_err(s_got, s_ref))
    assert len(fast.shapes()) == 2


def test_graphed_block_without_single_track():
    blk = P.PairformerBlock(c_s=0)
    O.seed_parameters_(blk)
    blk = blk.to("cuda", BF16).eval()
    fast = P.Graphed(blk)
    for rep in range(3):
        _, z, _ = O.make_inputs(80, seed=5 + rep, dtype=BF16)
        z = z.cuda()
        with torch.no_grad():
            _, z_ref = blk(None, z, None)
            s_got, z_got = fast(None, z, None)
        assert s_got is None and torch.equal(z_got, z_ref)


def test_graphed_replays_convert_the_mask_they_are_given():
    """The pair mask's converted copy is kept between eager calls; a graph must not bake in the
    copy (or the "all ones: no mask" decision) of the mask it was captured with."""
    st = _stack(BF16, n_blocks=2)
    fast = P.Graphed(st)
    n = 72
    s, z, _ = O.make_inputs(n, seed=3, dtype=BF16)
    s, z = s.cuda(), z.cuda()
    masks = [torch.ones(1, n, n), O.make_inputs(n, n_pad=9)[2], torch.ones(1, n, n),
             (torch.rand(1, n, n, generator=torch.Generator().manual_seed(1)) > 0.3).float()]
    for m in masks:
        m = m.cuda()
        with torch.no_grad():
            s_ref, z_ref = st(s, z, m)
            s_got, z_got = fast(s, z, m)
        assert torch.equal(z_got, z_ref) and torch.equal(s_got, s_ref)
    assert len(fast.shapes()) == 1


def test_graphed_padded_tail_has_its_own_recording():
    """Where the eager call runs a padded-tail mask as two attention launches, so does a recording
    (same bits), and masks of another class get another recording."""
    keep = P.ops.prefix_mask_min_n
    P.ops.prefix_mask_min_n = 0
    try:
        st = _stack(BF16, n_blocks=2)
        fast = P.Graphed(st)
        n = 72
        s, z, _ = O.make_inputs(n, seed=3, dtype=BF16)
        s, z = s.cuda(), z.cuda()
        masks = [O.make_inputs(n, n_pad=9)[2], torch.ones(1, n, n), O.make_inputs(n, n_pad=9)[2],
                 O.make_inputs(n, n_pad=20)[2],
                 (torch.rand(1, n, n, generator=torch.Generator().manual_seed(1)) > 0.3).float()]
        for m in masks:
            m = m.cuda()
            with torch.no_grad():
                s_ref, z_ref = st(s, z, m)
                s_got, z_got = fast(s, z, m)
            assert torch.equal(z_got, z_ref) and torch.equal(s_got, s_ref)
        # 63 valid tokens, 52 valid tokens, everything else
        assert len(fast.shapes()) == 3
    finally:
        P.ops.prefix_mask_min_n = keep

