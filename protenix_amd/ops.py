"""Tensor-level wrappers over the C ABI: validate, allocate outputs and
workspaces with torch, pass raw device pointers and the current HIP stream."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib

_DTYPES = {torch.float32: _lib.PTX_F32, torch.bfloat16: _lib.PTX_BF16}


def _dt(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise RuntimeError(f"protenix_amd kernels take float32 or bfloat16 tensors, got {t.dtype}")


def _dt_stream(z: torch.Tensor, compute: torch.dtype) -> int:
    """dtype code of a call whose residual-stream tensors (z, x, out) are `z` and whose
    weights and workspaces are `compute`: PTX_MIXED for fp32 rows with bf16 arithmetic."""
    if z.dtype == compute:
        return _dt(z)
    if z.dtype == torch.float32 and compute == torch.bfloat16:
        return _lib.PTX_MIXED
    raise RuntimeError(f"protenix_amd: rows in {z.dtype} with weights in {compute} are not supported "
                       "(same dtype, or float32 rows with bfloat16 weights)")


def _dev(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"protenix_amd: `{name}` is on {t.device}; the HIP kernels need a GPU tensor "
            "(there is no CPU fallback)")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


# Optional per-kernel timing: while `kernel_timer` is a dict, every C-ABI call
# is bracketed by HIP events on the stream it is launched on and the pairs are
# appended under the entry point's name; read them with kernel_times().
kernel_timer: Optional[dict] = None


def _call(name: str, fn, *args) -> None:
    if kernel_timer is None:
        _lib.check(fn(*args), name)
        return
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    _lib.check(fn(*args), name)
    e1.record()
    kernel_timer.setdefault(name, []).append((e0, e1))


def kernel_times(timer: dict) -> dict:
    """name -> list of launch-to-completion durations in ms (synchronises)."""
    torch.cuda.synchronize()
    return {k: [a.elapsed_time(b) for a, b in v] for k, v in timer.items()}


def _same(t: Optional[torch.Tensor], like: torch.Tensor, name: str) -> Optional[torch.Tensor]:
    """Parameter tensor in the activation dtype/device, contiguous."""
    if t is None:
        return None
    if t.dtype != like.dtype or t.device != like.device:
        t = t.to(device=like.device, dtype=like.dtype)
    return t.contiguous()


def compute_dtype(x: torch.Tensor) -> torch.dtype:
    """dtype the kernels' arithmetic, weights and workspaces take for rows `x`: x's own, or
    bfloat16 for float32 rows of 64, 128 or 256 channels under torch.autocast(bfloat16) - the
    fused fp32-residual-stream mode (PTX_MIXED of the C ABI)."""
    ac = autocast_compute_dtype(x)
    if ac == torch.bfloat16 and x.shape[-1] in (64, 128, 256):
        return ac
    return x.dtype


def autocast_compute_dtype(x: torch.Tensor) -> Optional[torch.dtype]:
    """The dtype torch.autocast would run this fp32 CUDA tensor's matmuls in, else None.
    Production inference keeps fp32 parameters and an fp32 pair tensor under
    torch.autocast("cuda", bfloat16) (inference.py:220-224 of the reference)."""
    if not (x.is_cuda and x.dtype == torch.float32):
        return None
    try:
        enabled = torch.is_autocast_enabled("cuda")
    except TypeError:   # older signature
        enabled = torch.is_autocast_enabled()
    if not enabled:
        return None
    try:
        return torch.get_autocast_dtype("cuda")
    except AttributeError:
        return torch.get_autocast_gpu_dtype()


def key_pitch(n: int) -> int:
    return _lib.load().ptx_key_pitch(n)


_LN_DTYPES = dict(_DTYPES)
_LN_DTYPES[torch.float16] = _lib.PTX_F16


def _dt_ln(t: torch.Tensor) -> int:
    """dtype code of the stand-alone LayerNorm, which also takes float16."""
    try:
        return _LN_DTYPES[t.dtype]
    except KeyError:
        raise RuntimeError(f"protenix_amd LayerNorm takes float32, bfloat16 or float16 tensors, got {t.dtype}")


def layer_norm(x: torch.Tensor, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor],
               eps: float = 1e-5, return_stats: bool = False):
    """LayerNorm over the last dim (reference: layer_norm.py:70-112)."""
    _dev(x, "input")
    lib = _lib.load()
    x = x.contiguous()
    cols = x.shape[-1]
    rows = x.numel() // cols if cols else 0
    w = _same(weight, x, "weight")
    b = _same(bias, x, "bias")
    y = torch.empty_like(x)
    mean = rstd = None
    if return_stats:
        mean = torch.empty(rows, dtype=torch.float32, device=x.device)
        rstd = torch.empty(rows, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _call("layernorm", lib.ptx_layernorm_fwd, _ptr(x), _ptr(w), _ptr(b), _ptr(y), _ptr(mean), _ptr(rstd),
                                         rows, cols, eps, _dt_ln(x), _stream())
    return (y, mean, rstd) if return_stats else y


def layer_norm_backward(dout: torch.Tensor, x: torch.Tensor, mean: torch.Tensor, rstd: torch.Tensor,
                        weight: Optional[torch.Tensor], need_weight: bool, need_bias: bool):
    """Gradients of layer_norm (reference: layer_norm.py:114-187): dx in x's dtype and, when
    asked for, dweight / dbias [cols] in x's dtype; mean, rstd as returned by
    layer_norm(..., return_stats=True)."""
    _dev(x, "input")
    lib = _lib.load()
    x = x.contiguous()
    dout = dout.to(dtype=x.dtype).contiguous()
    cols = x.shape[-1]
    rows = x.numel() // cols if cols else 0
    w = _same(weight, x, "weight")
    dx = torch.empty_like(x)
    dw = torch.empty(cols, dtype=x.dtype, device=x.device) if need_weight else None
    db = torch.empty(cols, dtype=x.dtype, device=x.device) if need_bias else None
    ws = None
    if need_weight or need_bias:
        ws = _workspace((lib.ptx_layernorm_bwd_workspace_elems(max(rows, 1), cols),), torch.float32,
                        x.device)
    with torch.cuda.device(x.device):
        _call("layernorm_bwd", lib.ptx_layernorm_bwd, _ptr(dout), _ptr(x), _ptr(mean), _ptr(rstd),
              _ptr(w), _ptr(dx), _ptr(dw), _ptr(db), _ptr(ws), rows, cols, _dt_ln(x), _stream())
    return dx, dw, db


# Workspaces are handed to the kernels uninitialised.  With `poison_workspaces` set (tests),
# they are filled with NaN first: no result may depend on what a workspace held before.
poison_workspaces = False


def _workspace(shape, dtype, device) -> torch.Tensor:
    if poison_workspaces:
        return torch.full(shape, float("nan"), dtype=dtype, device=device)
    return torch.empty(shape, dtype=dtype, device=device)


# The same pair mask comes back for every update of every block: its copy in the kernels' dtype
# (and, for the ending node, its transpose: the attention core then reads a row's key mask as
# one run of memory instead of a strided gather per key tile) is made once and kept.  An entry
# holds the caller's tensor, so its storage cannot be freed and handed out again while the entry
# lives, and is valid for that storage, view geometry and version counter only.
_mask_cache: list = []


# Pair masks of padded batches are m (x) m with the padding at the end: the triangle attention
# then runs its valid rows over the valid keys without a mask (see triangle_attention).  False
# hands every mask to the kernels as it is (tests compare the two).  Below some 480 tokens the
# second launch costs what the first one saves (measured per update, two launches against the
# masked kernel: 170 against 157 us at N = 384 with 32 padded tokens, 237 = 237 at 448, 293
# against 305 at 512, 390 against 411 at 576, 1.42 against 1.59 ms at 1024).
prefix_mask_enabled = True
prefix_mask_min_n = 480


_CACHE_ENTRIES = 64      # masks kept per cache: a batch of pair masks has one entry per element


def _mask_key(mask: torch.Tensor) -> Optional[tuple]:
    """Identity of a mask's contents for the caches below, or None for a mask that cannot be
    cached: a tensor made under torch.inference_mode() has no version counter, so an in-place
    change of it would go unseen; such masks are converted and classified on every call."""
    if mask.is_inference():
        return None
    return (mask.untyped_storage().data_ptr(), mask.storage_offset(), tuple(mask.shape), tuple(mask.stride()),
            mask.dtype, mask.device, mask._version)


_class_cache: list = []     # (key, mask, (all ones, n_valid or None)), most recent first
# While a HIP graph is being recorded nothing can be looked at: the class the recording is made
# for, set by its owner (graph.py), who replays it only for masks of that class.
capture_mask_class: Optional[tuple] = None


# A mask whose class its maker knows (the pair stack's own padding of odd sizes): (mask, class),
# looked up by identity, also while a graph is being recorded.
_declared_mask: Optional[tuple] = None


def declare_mask_class(mask: torch.Tensor, cls: tuple) -> None:
    """Tells mask_class() the class of `mask` (a tensor built by the caller, who must not change
    it afterwards and calls forget_mask() when done with it) so that nothing has to be looked at."""
    global _declared_mask
    _declared_mask = (mask, cls)


def _is_declared(mask: torch.Tensor) -> bool:
    # (the declared tensor itself, or the [n, n] view of it that the per-tensor loops of a batch of one make)
    d = _declared_mask
    return d is not None and (mask is d[0] or (
        mask.dim() == 2 and mask.data_ptr() == d[0].data_ptr() and mask.numel() == d[0].numel()
        and mask.is_contiguous()))


def forget_mask(mask: torch.Tensor) -> None:
    """Drops what is kept for a mask its maker is done with: a declared class, the cached class
    and the cached converted copies (which hold the mask alive)."""
    global _declared_mask
    if _declared_mask is not None and _declared_mask[0] is mask:
        _declared_mask = None
    ptr = mask.untyped_storage().data_ptr()    # (entries may be views of it, one per pair tensor of a batch)
    _class_cache[:] = [e for e in _class_cache if e[1].untyped_storage().data_ptr() != ptr]
    _mask_cache[:] = [e for e in _mask_cache if e[1].untyped_storage().data_ptr() != ptr]


def mask_class(mask: Optional[torch.Tensor]) -> tuple:
    """(all ones, n_valid) of a pair mask: n_valid is the number of valid tokens if the mask is
    [n, n] = m (x) m with m = n_valid ones followed by zeros (0 < n_valid < n), else None.
    Computed where the mask lives, fetched with one synchronisation per mask (not per call) and
    kept with the mask's storage, view geometry and version counter."""
    if mask is None:
        return (True, None)
    if _is_declared(mask):
        return _declared_mask[1]
    if mask.is_cuda and torch.cuda.is_current_stream_capturing():
        return capture_mask_class or (False, None)
    key = _mask_key(mask)
    for i, (k, _, cls) in enumerate(_class_cache if key is not None else ()):
        if k == key:
            if i:
                _class_cache.insert(0, _class_cache.pop(i))
            return cls
    if mask.dim() != 2 or mask.shape[0] != mask.shape[1] or mask.shape[0] == 0:
        cls = (bool((mask == 1).all()), None)
    else:
        row, col = mask[0, :], mask[:, 0]
        nv = row.float().sum()
        steps = (row[1:] > row[:-1]).any() if row.numel() > 1 else torch.zeros((), dtype=torch.bool, device=mask.device)
        prefix = ((mask == col[:, None] * row[None, :]).all() & (row == col).all()
                  & ((row == 0) | (row == 1)).all() & ~steps)
        ones, prefix, nv = torch.stack([(mask == 1).all().float(), prefix.float(), nv]).tolist()
        cls = (bool(ones), int(nv) if prefix and 0 < int(nv) < mask.shape[0] else None)
    if key is not None:
        _class_cache.insert(0, (key, mask, cls))
        del _class_cache[_CACHE_ENTRIES:]
    return cls


def padded_tail(mask: Optional[torch.Tensor], n: int) -> Optional[int]:
    """n_valid if the triangle attention treats this [n, n] mask as a padded tail (two launches:
    valid rows over valid keys without a mask, padded rows with it), else None."""
    if mask is None or not prefix_mask_enabled:
        return None
    # (a declared mask - the pair stack's own padding of an odd size, a handful of rows - takes the
    # two launches at any size: the valid rows then run exactly what the unpadded tensor would)
    if n < prefix_mask_min_n and not _is_declared(mask):
        return None
    return mask_class(mask)[1]


def _mask_for(mask: Optional[torch.Tensor], z: torch.Tensor, dtype: Optional[torch.dtype] = None,
              transpose: bool = False) -> Optional[torch.Tensor]:
    """The mask in the kernels' dtype, or None for a mask of all ones."""
    if mask is None:
        return None
    dtype = dtype or z.dtype

    def convert() -> torch.Tensor:
        out = mask.to(device=z.device, dtype=dtype)
        return out.transpose(-1, -2).contiguous() if transpose else out.contiguous()

    # Under stream capture the conversion is part of what is recorded: a replay must convert the
    # mask it is given then, so nothing is looked up, examined or kept (a mask of all ones is
    # then still loaded and applied, which changes no bit).
    if not z.is_cuda or torch.cuda.is_current_stream_capturing():
        return convert()
    # A mask of all ones changes no bit of any result (x * 1, logit + 0): it is handed on as
    # "no mask", which spares the kernels its loads.
    if mask_class(mask)[0]:
        return None
    key = _mask_key(mask)
    if key is None:
        return convert()
    key = key + (dtype, z.device, transpose)
    for i, (k, _, out) in enumerate(_mask_cache):
        if k == key:
            if i:
                _mask_cache.insert(0, _mask_cache.pop(i))
            return out
    out = convert()
    _mask_cache.insert(0, (key, mask, out))
    del _mask_cache[2 * _CACHE_ENTRIES:]
    return out


def triangle_multiplication(z: torch.Tensor, mask: Optional[torch.Tensor], w: dict, incoming: bool,
                            add_residual: bool, out: Optional[torch.Tensor] = None,
                            eps: float = 1e-5) -> torch.Tensor:
    """One [N, N, c_z] pair tensor through project -> contract -> output.
    `w` holds the parameters already in z's dtype (see triangular.py)."""
    _dev(z, "z")
    lib = _lib.load()
    n, c_z = z.shape[0], z.shape[-1]
    c_h = w["w_ap"].shape[0]
    cd = w["w_ap"].dtype            # arithmetic / workspace dtype; z may be fp32 beside bf16 weights
    dt, st = _dt_stream(z, cd), _stream()
    pitch = key_pitch(n)
    mask = _mask_for(mask, z, cd)
    # contraction operands in the library's fragment order (see include/protenix_amd.h)
    n_op = lib.ptx_trimul_operand_elems(n, c_h)
    a = _workspace((n_op,), cd, z.device)
    b = _workspace((n_op,), cd, z.device)
    with torch.cuda.device(z.device):
        _call("trimul_project", lib.ptx_trimul_project, _ptr(z), _ptr(mask), _ptr(w["ln_in_w"]), _ptr(w["ln_in_b"]), _ptr(w["w_ap"]),
            _ptr(w["w_ag"]), _ptr(w["w_bp"]), _ptr(w["w_bg"]), _ptr(a), _ptr(b), n, c_z, c_h, pitch,
            int(incoming), eps, dt, st)
        x = _workspace((c_h, n, n), cd, z.device)
        _call("trimul_contract", lib.ptx_trimul_contract, _ptr(a), _ptr(b), _ptr(x), n, c_h, pitch, dt, st)
        del a, b
        if out is None:
            out = torch.empty_like(z)
        _call("trimul_output", lib.ptx_trimul_output, _ptr(x), _ptr(z), _ptr(w["ln_in_w"]), _ptr(w["ln_in_b"]), _ptr(w["ln_out_w"]),
            _ptr(w["ln_out_b"]), _ptr(w["w_z"]), _ptr(w["w_g"]), _ptr(out), n, c_z, c_h,
            int(add_residual), eps, dt, st)
    return out


def triangle_multiplicative_update(x: torch.Tensor, incoming: bool, mask: Optional[torch.Tensor],
                                   norm_in_weight, norm_in_bias, p_in_weight: torch.Tensor,
                                   g_in_weight: torch.Tensor, norm_out_weight, norm_out_bias,
                                   p_out_weight: torch.Tensor, g_out_weight: torch.Tensor,
                                   eps: float = 1e-5) -> torch.Tensor:
    """One [N, N, c_z] pair tensor through the one-call operator of the C ABI
    (ptx_triangle_multiplicative_update: stacked input weights, one workspace); returns the
    update.  Parameters in x's dtype, or bfloat16 beside float32 rows (PTX_MIXED)."""
    _dev(x, "x")
    lib = _lib.load()
    n, c_z = x.shape[0], x.shape[-1]
    c_h = p_in_weight.shape[0] // 2
    cd = p_in_weight.dtype
    mask = _mask_for(mask, x, cd)
    ws = _workspace((lib.ptx_triangle_multiplicative_update_workspace_elems(n, c_h),), cd, x.device)
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        _call("triangle_multiplicative_update", lib.ptx_triangle_multiplicative_update, _ptr(x),
              int(incoming), _ptr(mask), _ptr(norm_in_weight), _ptr(norm_in_bias), _ptr(p_in_weight),
              _ptr(g_in_weight), _ptr(norm_out_weight), _ptr(norm_out_bias), _ptr(p_out_weight),
              _ptr(g_out_weight), _ptr(out), _ptr(ws), n, c_z, c_h, 0, eps, _dt_stream(x, cd), _stream())
    return out


# Triangle attention on rows of 128 channels in bf16 arithmetic: the gate is formed by the output
# kernel (ptx_triattn_gate_output) instead of travelling through memory.  False restores the
# three stages with a stored gate (tests compare the two).
late_gate_enabled = True


# The ending node's last stage and the pair transition behind it as one launch where the
# late-gate kernels apply (see triangle_attention(then_transition=...)).  False: two launches
# (tests compare the two, bit for bit).
fuse_attention_transition = True


def attention_transition_pack(w_g: torch.Tensor, w_o: torch.Tensor, w_a: torch.Tensor,
                              w_b: torch.Tensor, w_to: torch.Tensor) -> torch.Tensor:
    """Packs the attention's gate and output weights [128, 128] and the three Transition weights
    (c = 128, bf16) into the streaming order of the fused launch."""
    _dev(w_g, "w_g")
    lib = _lib.load()
    n_factor = w_a.shape[0] // w_a.shape[1]
    packed = torch.empty((lib.ptx_triattn_output_transition_packed_elems(n_factor),), dtype=w_g.dtype,
                         device=w_g.device)
    with torch.cuda.device(w_g.device):
        _call("transition_pack", lib.ptx_triattn_output_transition_pack, _ptr(w_g.contiguous()),
              _ptr(w_o.contiguous()), _ptr(w_a.contiguous()), _ptr(w_b.contiguous()),
              _ptr(w_to.contiguous()), _ptr(packed), n_factor, _dt(w_g), _stream())
    return packed


def fuses_attention_transition(z: torch.Tensor, heads: int, d: int, n_factor: int) -> bool:
    """Whether triangle_attention(then_transition=...) is available for rows `z`."""
    return (fuse_attention_transition and late_gate_enabled and z.is_cuda and z.shape[-1] == 128
            and heads == 4 and d == 32 and compute_dtype(z) == torch.bfloat16
            and (n_factor * 128) % 64 == 0 and n_factor <= 64)


def triangle_attention(z: torch.Tensor, mask: Optional[torch.Tensor], w: dict, heads: int, d: int,
                       inf: float, transposed: bool, add_residual: bool,
                       out: Optional[torch.Tensor] = None, eps: float = 1e-5,
                       then_transition: Optional[dict] = None):
    """Starting-node attention over z (transposed=False) or over z^T with the
    result written back transposed (transposed=True), i.e. the ending node as
    the Pairformer block uses it, without materialising z^T.  `mask` is indexed
    like z: the key mask of logical row i is mask[i, :] (or mask[:, i]).
    `then_transition` (with add_residual, where fuses_attention_transition() holds): the pair
    transition that follows, {"packed": attention_transition_pack(...), "ln_w", "ln_b",
    "n_factor", "pair_bias_w": (ln_w, ln_b, w [heads, 128]) or None}; the result is then
    out = z' + transition(z') with z' = z + attention(z), from the launch that forms z', and
    the return value (out, fp32 pair bias [heads, n*n] of out or None)."""
    _dev(z, "z")
    lib = _lib.load()
    n, c = z.shape[0], z.shape[-1]
    cd = w["w_q"].dtype
    dt, st = _dt_stream(z, cd), _stream()
    pitch = key_pitch(n)
    # (ending node: the key mask of logical row i is mask[:, i]; a transposed copy makes it a row)
    n_valid = padded_tail(mask, n)
    mask = _mask_for(mask, z, cd, transpose=transposed)
    dev = z.device
    # attention-core layouts (see include/protenix_amd.h): q, gate, output head-major; K, V^T
    # and the triangle bias in fragment-ordered key tiles
    n_kv, n_tb = lib.ptx_triattn_kv_elems(n, heads), lib.ptx_triattn_bias_elems(n, heads)
    # rows of 128 channels in bf16 arithmetic: no gate tensor, the output kernel forms the gate
    late_gate = late_gate_enabled and c == 128 and heads == 4 and d == 32 and cd == torch.bfloat16
    q = _workspace((heads, n, n, d), cd, dev)
    g = _workspace((heads, n, n, d), cd, dev)     # the gate, then (or only) the attention output
    k = _workspace((n_kv,), cd, dev)
    vt = _workspace((n_kv,), cd, dev)
    tb = _workspace((n_tb,), cd, dev)
    with torch.cuda.device(dev):
        _call("triattn_project", lib.ptx_triattn_project, _ptr(z), _ptr(w["ln_w"]),
              _ptr(w["ln_b"]), _ptr(w["w_q"]), _ptr(w["w_k"]), _ptr(w["w_v"]), _ptr(w["w_g"]),
              _ptr(w["w_b"]), _ptr(q), _ptr(k), _ptr(vt), None if late_gate else _ptr(g), _ptr(tb),
              n, c, heads, d, pitch, int(transposed), eps, dt, st)
        # o overwrites g: each element of g is read once, by the thread that then writes o there
        if mask is not None and n_valid is not None:
            # mask = m (x) m, padding at the end: the valid rows attend the valid keys with no
            # mask at all (a masked key of such a row has weight exactly zero in the reference);
            # the padded rows, all of whose keys are masked, go through the masked path
            for name, rows, mk, nk in (("triattn_fwd", (0, n_valid), None, n_valid),
                                       ("triattn_fwd_padded_rows", (n_valid, n - n_valid), mask, n)):
                _call(name, lib.ptx_triattn_fwd_rows, _ptr(q), _ptr(k), _ptr(vt),
                      None if late_gate else _ptr(g), _ptr(tb), _ptr(mk), _ptr(g), n, heads, d, pitch,
                      0, float(inf), rows[0], rows[1], nk, dt, st)
        else:
            _call("triattn_fwd", lib.ptx_triattn_fwd, _ptr(q), _ptr(k), _ptr(vt),
                  None if late_gate else _ptr(g), _ptr(tb), _ptr(mask), _ptr(g), n, heads, d, pitch, 0,
                  float(inf), dt, st)
        del q, k, vt, tb
        if out is None:
            out = torch.empty_like(z)
        if then_transition is not None:
            assert late_gate and add_residual
            tt = then_transition
            pbw = tt.get("pair_bias_w")
            bias = None
            if pbw is not None:
                bias = torch.empty((pbw[2].shape[0], n * n), dtype=torch.float32, device=dev)
            _call("triattn_output_transition", lib.ptx_triattn_output_transition_fwd, _ptr(g), _ptr(z),
                  _ptr(w["ln_w"]), _ptr(w["ln_b"]), _ptr(tt["packed"]), _ptr(tt["ln_w"]), _ptr(tt["ln_b"]),
                  _ptr(out), n, c, heads, int(transposed), tt["n_factor"], eps, eps,
                  _ptr(pbw[0]) if pbw else None, _ptr(pbw[1]) if pbw else None,
                  _ptr(pbw[2].contiguous()) if pbw else None, _ptr(bias), 0 if pbw is None else pbw[2].shape[0],
                  1, eps, dt, st)
            return out, bias
        if late_gate:
            _call("triattn_output", lib.ptx_triattn_gate_output, _ptr(g), _ptr(z), _ptr(w["ln_w"]),
                  _ptr(w["ln_b"]), _ptr(w["w_g"]), _ptr(w["w_o"]), _ptr(out), n, c, heads,
                  int(transposed), int(add_residual), eps, dt, st)
        else:
            _call("triattn_output", lib.ptx_triattn_output, _ptr(g), _ptr(w["w_o"]), _ptr(z), _ptr(out),
                  n, c, int(transposed), int(add_residual), dt, st)
    return out


def transition_pack(w_a: torch.Tensor, w_b: torch.Tensor, w_o: torch.Tensor) -> torch.Tensor:
    """Packs the three Transition weights (c = 64 or 128) into the fused kernel's streaming order."""
    _dev(w_a, "w_a")
    lib = _lib.load()
    c = w_a.shape[1]
    n_factor = w_a.shape[0] // c
    packed = torch.empty((lib.ptx_transition_packed_elems(c, n_factor),), dtype=w_a.dtype,
                         device=w_a.device)
    with torch.cuda.device(w_a.device):
        _call("transition_pack", lib.ptx_transition_pack, _ptr(w_a.contiguous()),
              _ptr(w_b.contiguous()), _ptr(w_o.contiguous()), _ptr(packed), c, n_factor, _dt(w_a),
              _stream())
    return packed


def transition(x: torch.Tensor, w: dict, n_factor: int, add_residual: bool,
               out: Optional[torch.Tensor] = None, eps: float = 1e-5,
               pair_bias_w: Optional[tuple] = None):
    """x [..., c] -> [x +] W_o(silu(W_a LN x) * W_b LN x), c = 64 or 128; `w["packed"]` comes from
    transition_pack.  With `pair_bias_w = (ln_w, ln_b, w [heads, c])` (c = 128, bf16 arithmetic)
    the same launch also forms the pair bias of the finished rows and the result is
    (out, bias fp32 [heads, rows]) - what pair_bias() would compute from `out`."""
    _dev(x, "x")
    lib = _lib.load()
    c = x.shape[-1]
    x2 = x.reshape(-1, c)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    rows = x2.shape[0]
    dt, st = _dt_stream(x, w["packed"].dtype), _stream()
    if out is None:
        out = torch.empty_like(x2)
    o2 = out.view(-1, c)
    with torch.cuda.device(x.device):
        if pair_bias_w is None:
            _call("transition", lib.ptx_transition_fwd, _ptr(x2), _ptr(w["ln_w"]), _ptr(w["ln_b"]),
                  _ptr(w["packed"]), _ptr(o2), rows, c, n_factor, int(add_residual), eps, dt, st)
            return out.view(x.shape)
        pln_w, pln_b, pw = pair_bias_w
        bias = torch.empty((pw.shape[0], rows), dtype=torch.float32, device=x.device)
        _call("transition", lib.ptx_transition_pair_bias_fwd, _ptr(x2), _ptr(w["ln_w"]), _ptr(w["ln_b"]),
              _ptr(w["packed"]), _ptr(o2), rows, c, n_factor, int(add_residual), eps, _ptr(pln_w),
              _ptr(pln_b), _ptr(pw.contiguous()), _ptr(bias), pw.shape[0], 1, eps, dt, st)
    return out.view(x.shape), bias


def pair_bias(z: torch.Tensor, ln_w: Optional[torch.Tensor], ln_b: Optional[torch.Tensor],
              w: torch.Tensor, out_f32: bool = True, eps: float = 1e-5) -> torch.Tensor:
    """bias[h, i, j] = (W LN(z[i, j]))[h] for one [N, N, 128] pair tensor."""
    _dev(z, "z")
    lib = _lib.load()
    n, c = z.shape[0], z.shape[-1]
    heads = w.shape[0]
    out = torch.empty((heads, n, n), dtype=torch.float32 if out_f32 else w.dtype, device=z.device)
    with torch.cuda.device(z.device):
        _call("pair_bias", lib.ptx_pair_bias_fwd, _ptr(z), _ptr(ln_w), _ptr(ln_b), _ptr(w), _ptr(out), n, c,
                                         heads, int(out_f32), eps, _dt_stream(z, w.dtype), _stream())
    return out


# ---------------------------------------------------------------- single-representation track
def linear(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
           res: Optional[torch.Tensor] = None) -> torch.Tensor:
    """[res +] x w^T [+ bias] for x [..., k], w [n_out, k] in x's dtype (k % 16 == 0,
    n_out % 8 == 0), on the HIP kernel of the single track."""
    _dev(x, "x")
    lib = _lib.load()
    k, n_out = x.shape[-1], w.shape[0]
    x2 = x.reshape(-1, k)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    rows = x2.shape[0]
    out = torch.empty((rows, n_out), dtype=x.dtype, device=x.device)
    r2 = None
    if res is not None:
        r2 = res.reshape(-1, n_out)
        if not r2.is_contiguous():
            r2 = r2.contiguous()
    with torch.cuda.device(x.device):
        _call("linear", lib.ptx_linear_fwd, _ptr(x2), _ptr(w), _ptr(bias), n_out if bias is not None else 0,
              _ptr(r2), _ptr(out), None, n_out, 0, rows, k, n_out, _dt(x), _stream())
    return out.view(*x.shape[:-1], n_out)


def linear_split(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], bias_cols: int,
                 split_col: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """x [rows, k] -> (y[:, :split_col] row-major, y[:, split_col:] transposed with the row axis
    padded with zeros to a multiple of 32), y = x w^T (+ bias on the first bias_cols columns)."""
    _dev(x, "x")
    lib = _lib.load()
    rows, k = x.shape
    n_out = w.shape[0]
    ldt = ((rows + 31) // 32) * 32
    out = torch.empty((rows, split_col), dtype=x.dtype, device=x.device)
    out_t = torch.empty((n_out - split_col, ldt), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        _call("linear", lib.ptx_linear_fwd, _ptr(x), _ptr(w), _ptr(bias), bias_cols, None, _ptr(out),
              _ptr(out_t), split_col, ldt, rows, k, n_out, _dt(x), _stream())
    return out, out_t


def swiglu(x: torch.Tensor, w_a: torch.Tensor, w_b: torch.Tensor) -> torch.Tensor:
    """silu(x w_a^T) * (x w_b^T) for x [..., k]."""
    _dev(x, "x")
    lib = _lib.load()
    k, hidden = x.shape[-1], w_a.shape[0]
    x2 = x.reshape(-1, k)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    out = torch.empty((x2.shape[0], hidden), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        _call("swiglu", lib.ptx_swiglu_fwd, _ptr(x2), _ptr(w_a), _ptr(w_b), _ptr(out), x2.shape[0], k,
              hidden, _dt(x), _stream())
    return out.view(*x.shape[:-1], hidden)


def single_attention(qkg: torch.Tensor, vt: torch.Tensor, bias: Optional[torch.Tensor], heads: int,
                     d: int, scale: float, gated: bool = True) -> torch.Tensor:
    """qkg [n, 3 * heads * d] (q | k | gate logits, head-major), vt [heads * d, ldt], bias
    [heads, n, n] fp32 or qkg's dtype -> gated attention output [n, heads * d]."""
    _dev(qkg, "qkg")
    lib = _lib.load()
    n, hd = qkg.shape[0], heads * d
    es = qkg.element_size()
    out = torch.empty((n, hd), dtype=qkg.dtype, device=qkg.device)
    base = qkg.data_ptr()
    if bias is not None:
        if bias.dtype not in (torch.float32, qkg.dtype):
            bias = bias.to(qkg.dtype)
        bias = bias.contiguous()
    with torch.cuda.device(qkg.device):
        _call("single_attention", lib.ptx_single_attention_fwd, base, base + hd * es, _ptr(vt),
              base + 2 * hd * es if gated else None, _ptr(bias),
              int(bias is not None and bias.dtype == torch.float32),
              _ptr(out), n, heads, d, qkg.shape[1], vt.shape[1], hd, float(scale), _dt(qkg), _stream())
    return out


# ---------------------------------------------------------------- measurement aid
def hbm_stream(src: Optional[torch.Tensor], dst: Optional[torch.Tensor], nontemporal: bool = False) -> None:
    """One streaming pass with plain 16-byte accesses: copy src -> dst, read src only (dst None) or
    write dst only (src None); the rate of such a pass is the ceiling an HBM-bound kernel of the
    same size is reported against."""
    t = src if src is not None else dst
    _dev(t, "src" if src is not None else "dst")
    if src is not None and dst is not None and src.numel() * src.element_size() != dst.numel() * dst.element_size():
        raise RuntimeError("hbm_stream: src and dst differ in size")
    if not all(x is None or x.is_contiguous() for x in (src, dst)):
        raise RuntimeError("hbm_stream: tensors must be contiguous")
    with torch.cuda.device(t.device):
        _call("hbm_stream", _lib.load().ptx_hbm_stream, _ptr(src), _ptr(dst), t.numel() * t.element_size(),
              int(nontemporal), _stream())
