"""Shared helpers of the parity tests."""
import torch

from oracle import pairformer_oracle as O

# BASELINE tolerances: max-abs error relative to max |reference|
TOL_F32 = 1e-4
TOL_BF16 = 2e-2


def rel_err(y: torch.Tensor, ref: torch.Tensor) -> float:
    y = y.detach().double().cpu()
    ref = ref.detach().double().cpu()
    assert y.shape == ref.shape, (y.shape, ref.shape)
    assert torch.isfinite(y).all(), "non-finite values in the kernel output"
    return ((y - ref).abs().max() / ref.abs().max().clamp_min(1e-30)).item()


def tol(dtype: torch.dtype) -> float:
    return TOL_F32 if dtype == torch.float32 else TOL_BF16


def oracle_and_product(oracle_cls, product_cls, *args, dtype=torch.float32, seed=4321, **kwargs):
    """The oracle module in fp32 on the CPU, holding `dtype`-rounded parameters,
    and the HIP-backed module on cuda:0 in `dtype` with the same parameters."""
    ref = O.seed_parameters_(oracle_cls(*args, **kwargs), seed=seed).eval()
    with torch.no_grad():
        for p in ref.parameters():
            p.copy_(p.to(dtype).float())
    prod = product_cls(*args, **kwargs)
    prod.load_state_dict(ref.state_dict())
    prod = prod.to(device="cuda", dtype=dtype).eval()
    return ref, prod


def pad_mask(n: int, n_pad: int, dtype=torch.float32) -> torch.Tensor:
    m = torch.ones(n)
    if n_pad:
        m[n - n_pad:] = 0
    return (m[:, None] * m[None, :])[None].to(dtype)
