"""Triangle attention under a pair mask m (x) m with the padding at the end (the reference's
pair_mask of a padded batch, loss.py:589): the valid rows run over the valid keys with no mask
(ptx_triattn_fwd_rows), the padded rows through the masked path.  Compared with the same module
handing the mask to the kernels as it is, and with the oracle (layers.py:276-296: a masked key
of a row with unmasked keys has weight exactly zero, a fully masked row averages v)."""
import pytest
import torch

import protenix_amd as P
from protenix_amd import ops
from oracle import pairformer_oracle as O
from tests.util import oracle_and_product, pad_mask, rel_err, tol

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _every_size():
    """The two-range path at every N (the host side takes it from some 480 tokens on)."""
    keep = ops.prefix_mask_min_n
    ops.prefix_mask_min_n = 0
    yield
    ops.prefix_mask_min_n = keep


def _run(prod, z, mask, mixed, prefix):
    keep = ops.prefix_mask_enabled
    ops.prefix_mask_enabled = prefix
    ops._mask_cache.clear()
    try:
        with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16, enabled=mixed):
            return prod(z, mask)
    finally:
        ops.prefix_mask_enabled = keep
        ops._mask_cache.clear()


def test_short_rows_keep_one_launch():
    ops.prefix_mask_min_n = 480
    _, prod = oracle_and_product(O.TriangleAttention, P.TriangleAttention, 128, 32, 4, dtype=torch.bfloat16)
    z = torch.randn(1, 96, 96, 128).to(torch.bfloat16).cuda()
    ops.kernel_timer = {}
    try:
        with torch.no_grad():
            prod(z, pad_mask(96, 10).cuda())
        assert len(ops.kernel_timer["triattn_fwd"]) == 1 and "triattn_fwd_padded_rows" not in ops.kernel_timer
    finally:
        ops.kernel_timer = None


@pytest.mark.parametrize("mode", ["bf16", "mixed", "fp32"])
@pytest.mark.parametrize("starting", [True, False])
@pytest.mark.parametrize("n,n_pad", [(2, 1), (33, 1), (37, 5), (64, 63), (100, 36), (128, 64), (130, 2),
                                     (256, 32), (300, 45), (512, 40), (512, 64), (768, 48)])
def test_padded_tail_equals_given_mask_and_oracle(mode, starting, n, n_pad):
    mixed = mode == "mixed"
    dt = torch.bfloat16 if mode == "bf16" else torch.float32
    wdt = torch.float32 if mode == "fp32" else torch.bfloat16
    ref, prod = oracle_and_product(O.TriangleAttention, P.TriangleAttention, 128, 32, 4,
                                   starting=starting, dtype=wdt)
    prod = prod.to(dt)
    g = torch.Generator().manual_seed(1000 * n + n_pad)
    z = (torch.randn(1, n, n, 128, generator=g) * 1.5).to(wdt)
    mask = pad_mask(n, n_pad)
    with torch.no_grad():
        want = ref(z.float(), mask)
    zd, md = z.to("cuda", dt), mask.cuda()
    calls = {}
    ops.kernel_timer = {}
    try:
        fast = _run(prod, zd, md, mixed, True)
        calls = {k: len(v) for k, v in ops.kernel_timer.items()}
    finally:
        ops.kernel_timer = None
    plain = _run(prod, zd, md, mixed, False)
    assert calls.get("triattn_fwd") == 1 and calls.get("triattn_fwd_padded_rows") == 1   # valid rows, padded rows
    assert fast.shape == plain.shape and fast.dtype == plain.dtype
    assert torch.isfinite(fast.float()).all()
    t = tol(torch.float32 if mode == "fp32" else torch.bfloat16)
    assert rel_err(fast, want) <= t
    # the same keys with the same weights; the tile that holds the boundary forms its logits on
    # the matrix pipe in one case and on the vector ALU in the other, so the probabilities and
    # the outputs may each land on a neighbouring 16-bit value
    assert rel_err(fast, plain) <= (1e-5 if mode == "fp32" else 1e-2)
    assert rel_err(fast, want) <= 1.2 * rel_err(plain, want) + (1e-6 if mode == "fp32" else 2e-3)


@pytest.mark.parametrize("mask_kind", ["ones", "holes", "asymmetric", "middle", "all_zero"])
def test_other_masks_take_the_general_path(mask_kind):
    n = 96
    ref, prod = oracle_and_product(O.TriangleAttention, P.TriangleAttention, 128, 32, 4,
                                   starting=True, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(7)
    z = torch.randn(1, n, n, 128, generator=g).to(torch.bfloat16)
    if mask_kind == "ones":
        mask = torch.ones(1, n, n)
    elif mask_kind == "holes":
        mask = (torch.rand(1, n, n, generator=g) > 0.3).float()
    elif mask_kind == "asymmetric":
        mask = pad_mask(n, 10)
        mask[0, :, n - 20:] = 0           # rows keep 76 keys, 86 rows are valid: not m (x) m
    elif mask_kind == "middle":
        m = torch.ones(n)
        m[40:50] = 0                      # m (x) m, but the padding is not at the end
        mask = (m[:, None] * m[None, :])[None]
    else:
        mask = torch.zeros(1, n, n)
    with torch.no_grad():
        want = ref(z.float(), mask)
    ops._mask_cache.clear()
    ops.kernel_timer = {}
    try:
        with torch.no_grad():
            got = prod(z.cuda(), mask.cuda())
        calls = len(ops.kernel_timer["triattn_fwd"]) + len(ops.kernel_timer.get("triattn_fwd_padded_rows", ()))
    finally:
        ops.kernel_timer = None
        ops._mask_cache.clear()
    assert calls == 1
    assert rel_err(got, want) <= tol(torch.bfloat16)


def test_block_and_stack_with_padded_tail():
    """Both attention nodes (the ending node reads the mask transposed) inside a block, in place."""
    ref, prod = oracle_and_product(O.PairformerBlock, P.PairformerBlock, dtype=torch.bfloat16)
    s, z, pm = O.make_inputs(150, n_pad=22, dtype=torch.bfloat16)
    with torch.no_grad():
        s_ref, z_ref = ref(s.float(), z.float(), pm.float())
    outs = {}
    for prefix in (True, False):
        keep = ops.prefix_mask_enabled
        ops.prefix_mask_enabled = prefix
        ops._mask_cache.clear()
        try:
            with torch.no_grad():
                outs[prefix] = prod(s.cuda(), z.cuda(), pm.cuda())
        finally:
            ops.prefix_mask_enabled = keep
            ops._mask_cache.clear()
    for prefix in (True, False):
        assert rel_err(outs[prefix][1], z_ref) <= tol(torch.bfloat16)
        assert rel_err(outs[prefix][0], s_ref) <= tol(torch.bfloat16)
    assert rel_err(outs[True][1], outs[False][1]) <= 1e-2


def test_rows_entry_refusals():
    lib = P._lib.load()
    args = [None] * 7
    # rows beyond n, n_keys beyond n, n_keys = 0
    assert lib.ptx_triattn_fwd_rows(*args, 64, 4, 32, 64, 0, 1e9, 60, 8, 64, 1, None) == 1
    assert lib.ptx_triattn_fwd_rows(*args, 64, 4, 32, 64, 0, 1e9, 0, 64, 65, 1, None) == 1
    assert lib.ptx_triattn_fwd_rows(*args, 64, 4, 32, 64, 0, 1e9, 0, 64, 0, 1, None) == 1
    # an empty range is no work
    assert lib.ptx_triattn_fwd_rows(*args, 64, 4, 32, 64, 0, 1e9, 10, 0, 64, 1, None) == 0


@pytest.mark.parametrize("n", [512, 130])
@pytest.mark.parametrize("rows", [(0, 512), (3, 5), (7, 1), (100, 33), (509, 3)])
def test_rows_entry_writes_its_rows_only(n, rows):
    """ptx_triattn_fwd_rows on a range of rows (odd counts, odd starts: at n = 512 the core takes
    two rows per wave) gives those rows of ptx_triattn_fwd's result bit for bit and leaves every
    other row of o alone."""
    r0, cnt = rows
    r0, cnt = min(r0, n - 1), min(cnt, n - min(r0, n - 1))
    lib = P._lib.load()
    bf = torch.bfloat16
    g = torch.Generator().manual_seed(n)
    z = torch.randn(n, n, 128, generator=g).to(bf).cuda()

    def w(*s):
        return (torch.randn(*s, generator=g) / s[-1] ** 0.5).to(bf).cuda()

    ln_w, ln_b = torch.ones(128, dtype=bf).cuda(), torch.zeros(128, dtype=bf).cuda()
    wq, wk, wv, wg, wb = w(128, 128), w(128, 128), w(128, 128), w(128, 128), w(4, 128)
    pitch = lib.ptx_key_pitch(n)
    q = torch.empty(4, n, n, 32, dtype=bf, device="cuda")
    gate = torch.empty_like(q)
    k = torch.empty(lib.ptx_triattn_kv_elems(n, 4), dtype=bf, device="cuda")
    vt = torch.empty_like(k)
    tb = torch.empty(lib.ptx_triattn_bias_elems(n, 4), dtype=bf, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    p = lambda t: t.data_ptr()
    assert lib.ptx_triattn_project(p(z), p(ln_w), p(ln_b), p(wq), p(wk), p(wv), p(wg), p(wb), p(q), p(k), p(vt),
                                   p(gate), p(tb), n, 128, 4, 32, pitch, 0, 1e-5, 1, st) == 0
    full = torch.empty_like(q)
    assert lib.ptx_triattn_fwd(p(q), p(k), p(vt), p(gate), p(tb), None, p(full), n, 4, 32, pitch, 0, 1e9, 1, st) == 0
    part = torch.full_like(q, 7.0)
    assert lib.ptx_triattn_fwd_rows(p(q), p(k), p(vt), p(gate), p(tb), None, p(part), n, 4, 32, pitch, 0, 1e9,
                                    r0, cnt, n, 1, st) == 0
    torch.cuda.synchronize()
    assert torch.equal(part[:, r0:r0 + cnt], full[:, r0:r0 + cnt])
    assert (part[:, :r0] == 7.0).all() and (part[:, r0 + cnt:] == 7.0).all()
