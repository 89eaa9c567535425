"""Parity at depth and at the full benchmark sizes.

The 48-block stack is compared with the fp32 CPU oracle where the oracle finishes in seconds
(N_token = 128, 256), in the three modes the package runs in: fp32; bf16 arithmetic on an fp32
residual stream (fp32 tensors under torch.autocast(bfloat16), the reference's inference mode,
runner/inference.py:214-234); bf16 throughout.  At N_token = 768 and 2048 the oracle is out of
reach for 48 blocks (about five CPU minutes at 768), so one block is compared with it there
and the full workloads are checked against the fp32 HIP path - itself within 1e-5 of the oracle
at depth - and through the padding-is-token-deletion property.

Tolerances are the benchmark's: fp32 1e-4, bf16 2e-2, max-abs error over max |reference|.
bf16 *throughout* does not meet 2e-2 at depth: rounding the residual stream after each of the
240 updates (|z| grows to ~37, half an ulp there is 0.06-0.12) accumulates to 5e-2 - 6.5e-2
after 48 blocks; that mode is held to the tolerance only over the first blocks, and the
mode with the fp32 residual stream is the one the benchmark runs.
"""
import pytest
import torch

import protenix_amd as P
from oracle import pairformer_oracle as O
from tests.util import TOL_BF16, TOL_F32, pad_mask, rel_err

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _oracle_stack(n_blocks, seed=4321):
    ref = O.seed_parameters_(O.PairformerStack(n_blocks=n_blocks), seed=seed).eval()
    with torch.no_grad():
        for p in ref.parameters():
            p.copy_(p.to(BF16).float())     # the same bf16-representable weights in every mode
    return ref


def _product_stack(ref, mode):
    st = P.PairformerStack(n_blocks=len(ref.blocks))
    st.load_state_dict(ref.state_dict())
    return st.to("cuda", BF16 if mode == "bf16" else torch.float32).eval()


def _run(st, mode, s, z, pm, upto=None):
    """(s, z) after every block in `upto` (1-based), on the GPU; inputs are left untouched."""
    dt = BF16 if mode == "bf16" else torch.float32
    sc, zc, pc = s.to(dt).cuda(), z.to(dt).cuda(), pm.to(dt).cuda()
    outs = {}
    with torch.no_grad():
        for i, blk in enumerate(st.blocks):
            if mode == "autocast":
                with torch.autocast("cuda", dtype=BF16):
                    sc, zc = blk(sc, zc, pc)
            else:
                sc, zc = blk(sc, zc, pc)
            if upto is None or i + 1 in upto:
                outs[i + 1] = (sc.float().cpu(), zc.float().cpu())
    return outs


@pytest.mark.parametrize("n", [128, 256])
def test_stack_48_blocks_against_oracle(n):
    ref = _oracle_stack(48)
    s, z, pm = O.make_inputs(n, n_pad=8, dtype=BF16)
    want = {}
    with torch.no_grad():
        so, zo = s.float(), z.float()
        for i, blk in enumerate(ref.blocks):
            so, zo = blk(so, zo, pm.float())
            if i + 1 in (2, 48):
                want[i + 1] = (so.clone(), zo.clone())
    checks = {"fp32": (TOL_F32, (2, 48)), "autocast": (TOL_BF16, (2, 48)), "bf16": (TOL_BF16, (2,))}
    report = []
    for mode, (tol, depths) in checks.items():
        got = _run(_product_stack(ref, mode), mode, s, z, pm, upto=(2, 48))
        for d in (2, 48):
            es, ez = rel_err(got[d][0], want[d][0]), rel_err(got[d][1], want[d][1])
            known = "" if d in depths else " (KNOWN OUT OF TOLERANCE, not asserted: bf16 storage of the residual stream drifts)"
            report.append(f"{mode}@{d}: z {ez:.2e} s {es:.2e}{known}")
            if d in depths:
                assert ez <= tol and es <= tol, report
    print("; ".join(report))


def test_scaled_up_stack_cz256_at_depth():
    """The scaled-up model's pair stack (c_z = 256, hidden_scale_up: 8 pair heads, c_hidden_mul =
    256; configs_model_type.py:52-85, pairformer.py:76-78 of the reference) through 24 blocks
    at N_token = 96: bf16 arithmetic on the fp32 residual stream (the fused fp32-row kernels
    of this width) against the fp32 oracle."""
    kw = dict(n_blocks=24, c_z=256, hidden_scale_up=True)
    ref = O.seed_parameters_(O.PairformerStack(**kw)).eval()
    with torch.no_grad():
        for p in ref.parameters():
            p.copy_(p.to(BF16).float())
    st = P.PairformerStack(**kw)
    st.load_state_dict(ref.state_dict())
    st = st.to("cuda").eval()
    s, z, pm = O.make_inputs(96, c_z=256, n_pad=6, dtype=BF16)
    s, z, pm = s.float(), z.float(), pm.float()
    with torch.no_grad():
        want_s, want_z = ref(s, z, pm)
        with torch.autocast("cuda", dtype=BF16):
            got_s, got_z = st(s.cuda(), z.cuda(), pm.cuda())
    ez, es = rel_err(got_z, want_z), rel_err(got_s, want_s)
    print(f"c_z = 256, 24 blocks, N = 96, fp32 residual stream: z {ez:.2e} s {es:.2e}")
    assert got_z.dtype == torch.float32 and ez <= TOL_BF16 and es <= TOL_BF16


def test_block_n768_against_oracle():
    """One full PairformerBlock at the benchmark's N_token = 768 with 48 padded tokens, bf16
    throughout and bf16 on fp32 rows, against the fp32 oracle."""
    n = 768
    ref = _oracle_stack(1)
    s, z, pm = O.make_inputs(n, n_pad=48, dtype=BF16)
    torch.set_num_threads(min(16, torch.get_num_threads() or 16))
    with torch.no_grad():
        want_s, want_z = ref.blocks[0](s.float(), z.float(), pm.float(), chunk_size=128)
    for mode in ("bf16", "autocast"):
        got_s, got_z = _run(_product_stack(ref, mode), mode, s, z, pm)[1]
        assert rel_err(got_z, want_z) <= TOL_BF16, mode
        assert rel_err(got_s, want_s) <= TOL_BF16, mode


def test_config4_stack_48_blocks_n768():
    """The benchmark workload itself: 48 blocks at N_token = 768, mask of ones, bf16
    arithmetic on the fp32 residual stream, against the fp32 HIP path (within 1e-5 of the
    oracle through 48 blocks, see test_stack_48_blocks_against_oracle)."""
    n = 768
    ref = _oracle_stack(48)
    s, z, pm = O.make_inputs(n, dtype=BF16)
    outs = {}
    for mode in ("fp32", "autocast"):
        st = _product_stack(ref, mode)
        with torch.no_grad():
            sc, zc, pc = s.float().cuda(), z.float().cuda(), pm.float().cuda()
            if mode == "autocast":
                with torch.autocast("cuda", dtype=BF16):
                    outs[mode] = st(sc, zc, pc)
            else:
                outs[mode] = st(sc, zc, pc)
        outs[mode] = tuple(t.float().cpu() for t in outs[mode])
        del st
        torch.cuda.empty_cache()
    es = rel_err(outs["autocast"][0], outs["fp32"][0])
    ez = rel_err(outs["autocast"][1], outs["fp32"][1])
    print(f"48 blocks, N = 768: z {ez:.2e} s {es:.2e}")
    assert ez <= TOL_BF16 and es <= TOL_BF16


def test_config5_stack_48_blocks_n2048_pad64():
    """48 blocks at N_token = 2048 with 64 padded tokens, bf16 arithmetic on the fp32 residual
    stream: the N^3 logits are never materialised (peak HBM stays a small multiple of the pair
    tensor), and the valid corner of the pair tensor equals the stack run on the cropped
    inputs - padded keys are inert in both triangle updates, every other operation on the
    pair tensor is local to a pair."""
    n, n_pad = 2048, 64
    nv = n - n_pad
    ref = _oracle_stack(48)
    st = _product_stack(ref, "autocast")
    del ref
    g = torch.Generator().manual_seed(7)
    z = torch.randn(1, n, n, 128, generator=g)
    s = torch.randn(1, n, 384, generator=g)
    mask = pad_mask(n, n_pad)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    with torch.no_grad(), torch.autocast("cuda", dtype=BF16):
        zc = z.cuda()
        s_full, z_full = st(s.cuda(), zc, mask.cuda(), inplace_safe=True)
        torch.cuda.synchronize()
        peak = torch.cuda.max_memory_allocated() - base
        z_bytes = n * n * 128 * 4
        print(f"peak HBM over the resident weights: {peak / 1e9:.2f} GB ({peak / z_bytes:.1f} fp32 pair tensors)")
        assert peak <= 6 * z_bytes, f"peak {peak / 1e9:.2f} GB"     # N^3 logits would be 69 GB
        z_full = z_full[:, :nv, :nv].float().cpu()
        del zc
        torch.cuda.empty_cache()
        _, z_crop = st(s[:, :nv].contiguous().cuda(), z[:, :nv, :nv].contiguous().cuda(),
                       pad_mask(nv, 0).cuda(), inplace_safe=True)
    assert torch.isfinite(z_full).all() and torch.isfinite(s_full.float()).all()
    e = rel_err(z_crop, z_full)
    print(f"48 blocks, N = 2048, 64 padded: full vs cropped z {e:.2e}")
    # masked keys contribute exact zeros in the same summation order: bit for bit
    assert torch.equal(z_crop.float().cpu(), z_full), f"padded keys leak: {e:.2e}"
