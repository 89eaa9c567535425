"""CPU-side checks: the C-ABI library builds/loads and exports every symbol the
header declares, argument validation answers without touching a GPU, and the
drop-in modules keep the reference's state-dict layout."""
import ctypes
import os
import re

import pytest
import torch

import protenix_amd as P
from oracle import pairformer_oracle as O
from protenix_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "protenix_amd.h")).read()
    return re.findall(r"PTX_API\s+[\w\s\*]+?\b(ptx_\w+)\s*\(", text)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), n
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert set(_lib.SIGNATURES) == set(names)
    assert lib.ptx_version() == _lib.ABI_VERSION
    assert lib.ptx_last_error_string() is not None


def test_key_pitch():
    lib = _lib.load()
    assert [lib.ptx_key_pitch(n) for n in (0, 1, 64, 65, 768, 2048)] == [0, 64, 64, 128, 768, 2048]


def test_argument_validation_without_gpu():
    lib = _lib.load()
    # unknown dtype, bad sizes, unsupported widths: rejected before any launch
    assert lib.ptx_layernorm_fwd(None, None, None, None, None, None, 4, 128, 1e-5, 7, None) == 1
    assert b"dtype" in lib.ptx_last_error_string()
    assert lib.ptx_layernorm_fwd(None, None, None, None, None, None, 4, 128, 1e-5, 0, None) == 1
    assert lib.ptx_layernorm_fwd(None, None, None, None, None, None, 0, 128, 1e-5, 0, None) == 0
    assert lib.ptx_layernorm_bwd(*([None] * 9), 4, 128, 7, None) == 1
    assert lib.ptx_layernorm_bwd(*([None] * 9), 4, 128, 0, None) == 1      # null pointers
    assert lib.ptx_layernorm_bwd(*([None] * 9), 0, 128, 0, None) == 0      # nothing to do
    assert lib.ptx_layernorm_bwd_workspace_elems(1000, 128) >= 2 * 128
    assert lib.ptx_layernorm_bwd_workspace_elems(0, 128) == 0
    assert lib.ptx_trimul_contract(None, None, None, 8, 128, 63, 1, None) == 1
    assert b"k_pitch" in lib.ptx_last_error_string()
    assert lib.ptx_trimul_project(*([None] * 10), 8, 64, 64, 64, 0, 1e-5, 1, None) == 2
    assert b"128" in lib.ptx_last_error_string()
    assert lib.ptx_triattn_fwd(*([None] * 7), 8, 4, 16, 64, 0, 1e9, 1, None) == 2
    assert lib.ptx_triattn_project(*([None] * 13), 8, 128, 8, 16, 64, 0, 1e-5, 1, None) == 2
    assert lib.ptx_transition_fwd(*([None] * 5), 10, 384, 4, 0, 1e-5, 0, None) == 2
    assert lib.ptx_transition_pack(None, None, None, None, 384, 4, 0, None) == 2
    assert lib.ptx_transition_packed_elems(128, 4) == 3 * 4 * 128 * 128
    assert lib.ptx_pair_bias_fwd(*([None] * 5), 8, 128, 33, 1, 1e-5, 0, None) == 2
    assert lib.ptx_triattn_output(None, None, None, None, 8, 128, 0, 1, 0, None) == 1
    with pytest.raises(RuntimeError, match="unsupported shape"):
        _lib.check(2, "x")


def test_modules_refuse_cpu_tensors_and_grad():
    ln = P.LayerNorm(128)
    with torch.no_grad(), pytest.raises(RuntimeError, match="GPU tensor"):
        ln(torch.randn(4, 128))
    with pytest.raises(RuntimeError, match="GPU tensor"):
        ln(torch.randn(4, 128))          # LayerNorm has a backward; it still needs the GPU
    tm = P.TriangleMultiplicationOutgoing(128, 128)
    with pytest.raises(RuntimeError, match="forward-only"):
        tm(torch.randn(1, 4, 4, 128))
    blk = P.PairformerBlock()
    with pytest.raises(RuntimeError, match="inference-only"):
        blk(torch.randn(1, 8, 384), torch.randn(1, 8, 8, 128), None)
    with torch.no_grad(), pytest.raises(ValueError):
        blk.eval()(torch.randn(1, 8, 384), torch.randn(1, 8, 8, 128), None, triangle_multiplicative="x")


def test_state_dict_layout_matches_oracle_and_default_init_is_identity_shaped():
    a, b = P.PairformerStack(n_blocks=2), O.PairformerStack(n_blocks=2)
    sa, sb = a.state_dict(), b.state_dict()
    assert list(sa.keys()) == list(sb.keys())
    for k in sa:
        assert sa[k].shape == sb[k].shape, k
    a.load_state_dict(sb)
    blk = P.PairformerBlock()
    # the reference zero-initialises gates and output projections
    for name in ("tri_mul_out.linear_z", "tri_mul_in.linear_g", "tri_att_start.mha.linear_o",
                 "tri_att_end.mha.linear_g", "pair_transition.linear_no_bias",
                 "attention_pair_bias.attention.linear_o", "attention_pair_bias.attention.linear_g"):
        assert blk.get_submodule(name).weight.abs().sum() == 0, name
    assert blk.tri_mul_out.linear_a_p.weight.std() > 0
    assert P.TriangleAttentionEndingNode(128, 32, 4).starting is False
    with pytest.raises(NotImplementedError):
        P.AttentionPairBias(has_s=True)


# state-dict keys of one Pairformer block, as the reference's modules declare them
# (triangular.py:113-119, 190-197, 622-628; layers.py:340-357; primitives.py:175-188, 695-716;
# transformer.py:79-98) - written out literally, not derived from any of this repository's code
_BLOCK_KEYS = {
    **{f"{m}.{k}": shape for m in ("tri_mul_out", "tri_mul_in") for k, shape in {
        "linear_g.weight": (128, 128), "linear_z.weight": (128, 128),
        "layer_norm_in.weight": (128,), "layer_norm_in.bias": (128,),
        "layer_norm_out.weight": (128,), "layer_norm_out.bias": (128,),
        "linear_a_p.weight": (128, 128), "linear_a_g.weight": (128, 128),
        "linear_b_p.weight": (128, 128), "linear_b_g.weight": (128, 128)}.items()},
    **{f"{m}.{k}": shape for m in ("tri_att_start", "tri_att_end") for k, shape in {
        "layer_norm.weight": (128,), "layer_norm.bias": (128,), "linear.weight": (4, 128),
        "mha.linear_q.weight": (128, 128), "mha.linear_k.weight": (128, 128),
        "mha.linear_v.weight": (128, 128), "mha.linear_o.weight": (128, 128),
        "mha.linear_g.weight": (128, 128)}.items()},
    "pair_transition.layernorm1.weight": (128,), "pair_transition.layernorm1.bias": (128,),
    "pair_transition.linear_no_bias_a.weight": (512, 128),
    "pair_transition.linear_no_bias_b.weight": (512, 128),
    "pair_transition.linear_no_bias.weight": (128, 512),
    "attention_pair_bias.layernorm_a.weight": (384,), "attention_pair_bias.layernorm_a.bias": (384,),
    "attention_pair_bias.attention.linear_q.weight": (384, 384),
    "attention_pair_bias.attention.linear_q.bias": (384,),
    "attention_pair_bias.attention.linear_k.weight": (384, 384),
    "attention_pair_bias.attention.linear_v.weight": (384, 384),
    "attention_pair_bias.attention.linear_o.weight": (384, 384),
    "attention_pair_bias.attention.linear_g.weight": (384, 384),
    "attention_pair_bias.layernorm_z.weight": (128,), "attention_pair_bias.layernorm_z.bias": (128,),
    "attention_pair_bias.linear_nobias_z.weight": (16, 128),
    "single_transition.layernorm1.weight": (384,), "single_transition.layernorm1.bias": (384,),
    "single_transition.linear_no_bias_a.weight": (1536, 384),
    "single_transition.linear_no_bias_b.weight": (1536, 384),
    "single_transition.linear_no_bias.weight": (384, 1536),
}


def test_product_state_dict_is_the_reference_checkpoint_layout():
    """A reference checkpoint loads unchanged: the product's PairformerStack has exactly the
    reference's keys and shapes under blocks.{i}. (and so has the oracle)."""
    import protenix_amd as P
    from oracle import pairformer_oracle as O

    for mod in (P, O):
        sd = mod.PairformerStack(n_blocks=2).state_dict()
        want = {f"blocks.{i}.{k}": v for i in range(2) for k, v in _BLOCK_KEYS.items()}
        assert set(sd.keys()) == set(want.keys()), set(sd.keys()) ^ set(want.keys())
        for k, shape in want.items():
            assert tuple(sd[k].shape) == shape, (k, tuple(sd[k].shape))
    # the MSA module's pair stack has no single track (pairformer.py:622-624)
    sd = P.PairformerBlock(c_s=0).state_dict()
    assert not any(k.startswith(("attention_pair_bias", "single_transition")) for k in sd)
    assert len(sd) == len(_BLOCK_KEYS) - 16


def test_mask_class_finds_a_padded_tail_and_nothing_else():
    """ops.mask_class: (all ones, n_valid); n_valid only for m (x) m with the zeros of m at the
    end (the reference's pair_mask of a padded batch, loss.py:589)."""
    import torch
    from protenix_amd import ops

    def outer(v):
        return v[:, None] * v[None, :]

    v = torch.ones(8)
    assert ops.mask_class(None) == (True, None)
    assert ops.mask_class(outer(v)) == (True, None)
    v[5:] = 0
    tail = outer(v)
    assert ops.mask_class(tail) == (False, 5)
    assert ops.mask_class(tail.to(torch.bfloat16)) == (False, 5)
    hole = torch.ones(8)
    hole[2:4] = 0
    assert ops.mask_class(outer(hole)) == (False, None)            # padding not at the end
    head = torch.ones(8)
    head[:3] = 0
    assert ops.mask_class(outer(head)) == (False, None)            # padding at the front
    spoilt = tail.clone()
    spoilt[0, 7] = 1
    assert ops.mask_class(spoilt) == (False, None)                 # not m (x) m
    spoilt = tail.clone()
    spoilt[6, 6] = 1
    assert ops.mask_class(spoilt) == (False, None)
    assert ops.mask_class(tail * 0.5) == (False, None)             # not 0 / 1
    assert ops.mask_class(torch.zeros(4, 4)) == (False, None)      # no valid token
    assert ops.mask_class(torch.ones(1, 4, 4)) == (True, None)     # batched: all-ones check only
    # an entry follows the version counter of the tensor it was made for
    m = outer(torch.ones(6))
    assert ops.mask_class(m) == (True, None)
    m[:, 4:] = 0
    m[4:, :] = 0
    assert ops.mask_class(m) == (False, 4)
    # the attention takes the two-launch path from prefix_mask_min_n tokens on
    assert ops.padded_tail(tail, 8) is None
    keep = ops.prefix_mask_min_n
    ops.prefix_mask_min_n = 0
    try:
        assert ops.padded_tail(tail, 8) == 5
        assert ops.padded_tail(outer(hole), 8) is None
    finally:
        ops.prefix_mask_min_n = keep


def test_mask_class_takes_inference_mode_masks_and_large_batches():
    """A mask made under torch.inference_mode() has no version counter: it is classified on
    every call instead of being cached (an in-place change of it could not be noticed), and
    the caches hold every element of a batch of masks larger than eight."""
    import torch
    from protenix_amd import ops

    with torch.inference_mode():
        v = torch.ones(8)
        v[6:] = 0
        m = v[:, None] * v[None, :]
        assert m.is_inference()
        assert ops.mask_class(m) == (False, 6)
        m[:, 5:] = 0
        m[5:, :] = 0
        assert ops.mask_class(m) == (False, 5)
        z = torch.zeros(8, 8, 4)
        out = ops._mask_for(m, z, torch.float32, transpose=True)
        assert out.dtype == torch.float32 and torch.equal(out, m.t())
    # a batch of 12 masks, looked at twice: the second look finds every entry
    batch = torch.ones(12, 8, 8)
    for i in range(12):
        batch[i, :, 8 - i % 4 - 1:] = 0
        batch[i, 8 - i % 4 - 1:, :] = 0
    first = [ops.mask_class(batch[i]) for i in range(12)]
    assert first == [(False, 8 - i % 4 - 1) for i in range(12)]
    keys = {ops._mask_key(batch[i]) for i in range(12)}
    assert keys <= {k for k, _, _ in ops._class_cache}


def test_modules_refuse_what_the_kernels_do_not_cover_instead_of_falling_back():
    """No library GEMM or softmax stands in for a HIP kernel: CPU tensors, a `precision`
    override inside the fused modules, unsupported head shapes and cross-attention raise."""
    import pytest
    import torch
    import protenix_amd as P
    from protenix_amd.primitives import Linear, Transition
    from protenix_amd.transformer import Attention

    with torch.no_grad():
        with pytest.raises(RuntimeError, match="no CPU fallback"):
            Linear(16, 8)(torch.zeros(4, 16))
        with pytest.raises(RuntimeError, match="no CPU fallback"):
            Attention(32, 32, 32, 8, 4).eval()(torch.zeros(4, 32), torch.zeros(4, 32))
        att = Attention(48, 48, 48, 24, 2).eval()       # 3 * 2 * 24 = 144: not a multiple of 32
        x = torch.zeros(4, 48)
        with pytest.raises(RuntimeError, match="unsupported configuration"):
            att._check_supported(x, x)
        with pytest.raises(RuntimeError, match="self-attention"):
            Attention(32, 32, 32, 8, 4)._check_supported(x, x.clone())
        Attention(384, 384, 384, 24, 16)._check_supported(x, x)      # the block's own shape
        tr = Transition(384, 4).eval()
        tr.linear_no_bias_a.precision = torch.float32
        with pytest.raises(RuntimeError, match="precision"):
            tr(torch.zeros(4, 384))
    import inspect
    from protenix_amd import primitives, transformer
    for mod in (primitives, transformer):
        src = inspect.getsource(mod)
        assert "torch.nn.functional" not in src and "torch.softmax(" not in src and "torch.matmul(" not in src
