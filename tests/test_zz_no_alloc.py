"""ptx_layernorm_bwd_static, the entry point that allocates nothing: its built-in scratch
must give the same bits as ptx_layernorm_bwd with a caller-provided workspace, on two calls
in a row, the second on a smaller input (the scratch keeps the first call's contents)."""
import pytest
import torch

from protenix_amd import _lib, ops

pytestmark = pytest.mark.gpu


def _case(rows, cols, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(rows, cols, generator=g) * 2 + 0.5).to(dtype).cuda()
    dout = torch.randn(rows, cols, generator=g).to(dtype).cuda()
    w = (1 + 0.1 * torch.randn(cols, generator=g)).to(dtype).cuda()
    return x, dout, w


def _static(lib, x, dout, mean, rstd, w):
    rows, cols = x.shape
    dx = torch.full_like(x, float("nan"))
    dw = torch.full((cols,), float("nan"), dtype=x.dtype, device=x.device)
    db = torch.full((cols,), float("nan"), dtype=x.dtype, device=x.device)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = lib.ptx_layernorm_bwd_static(dout.data_ptr(), x.data_ptr(), mean.data_ptr(),
                                      rstd.data_ptr(), w.data_ptr(), dx.data_ptr(), dw.data_ptr(),
                                      db.data_ptr(), rows, cols, ops._dt(x),
                                      torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "layernorm_bwd_static")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return dx, dw, db


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_static_scratch_matches_workspace_entry_point(dtype):
    lib = _lib.load()
    # the second call is smaller in rows and in columns: fewer, shorter partial rows than the
    # scratch still holds from the first
    for rows, cols, seed in ((40000, 384, 1), (1500, 128, 2), (3, 1024, 3)):
        x, dout, w = _case(rows, cols, dtype, seed)
        _, mean, rstd = ops.layer_norm(x, w, None, return_stats=True)
        want = ops.layer_norm_backward(dout, x, mean, rstd, w, True, True)
        got = _static(lib, x, dout, mean, rstd, w)
        for a, b in zip(got, want):
            assert torch.equal(a, b)


def test_static_scratch_rejects_rows_longer_than_its_limit():
    lib = _lib.load()
    x, dout, w = _case(8, 1032, torch.float32, 4)
    _, mean, rstd = ops.layer_norm(x, w, None, return_stats=True)
    dx = torch.empty_like(x)
    dw = torch.empty(1032, device="cuda")
    rc = lib.ptx_layernorm_bwd_static(dout.data_ptr(), x.data_ptr(), mean.data_ptr(),
                                      rstd.data_ptr(), w.data_ptr(), dx.data_ptr(), dw.data_ptr(),
                                      dw.data_ptr(), 8, 1032, 0,
                                      torch.cuda.current_stream().cuda_stream)
    assert rc == 2
    assert b"1024" in lib.ptx_last_error_string()
