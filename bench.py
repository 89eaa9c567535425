#!/usr/bin/env python3
"""Headline benchmark: forward of the 48-block PairformerStack at N_token = 768
in bf16 on one MI355X (BASELINE config 4), synthetic seeded inputs and weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  `value` is the wall time of one trunk forward (ms) with
inputs resident in HBM.  `roofline` describes the dominant kernel (the triangle-
attention core) from HIP-event timings taken in place, on the launch stream,
during one extra instrumented pass over the same workload; `kernels` lists every
kernel the same way.  `cpu_baseline` times the CPU oracle (a PyTorch restatement
of the reference's torch path) on a bounded sample of the same workload on this
box's host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

N_TOKEN = 768
N_BLOCKS = 48
C_Z, C_S = 128, 384
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E
# HBM bytes per launch of the triangle-attention core at N_token = 768, bf16, measured with
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on this benchmark and calibrated against a plain
# elementwise kernel of known size (profiles/trunk_n768_bf16_hbm_traffic.txt):
# 603780 KiB fetched + 147456 KiB written.  Algorithmic: 594432 + 147456 KiB.
TRIATTN_FWD_TRAFFIC_BYTES_N768 = (604154 + 147460) * 1024

# Algorithmic work per launch at N tokens, c = 128, bf16 (2 bytes):
#   flops for the MFMA-bound kernels, bytes for the HBM-bound ones.
def _work(n: int) -> dict:
    e = n * n * 128 * 2   # bytes of one [N, N, 128] bf16 tensor
    return {
        "triattn_fwd":     ("mfma", 512.0 * n ** 3),              # QK^T + PV, 4*N^3*H*D
        "trimul_contract": ("mfma", 256.0 * n ** 3),              # 2*N^3*c
        "transition":      ("mfma", 393216.0 * n * n),            # 3 GEMMs 128<->512, fused
        "trimul_project":  ("hbm", 3.0 * e),                      # read z, write a and b
        "trimul_output":   ("hbm", 3.0 * e),                      # read x and z, write z
        "triattn_project": ("hbm", 5.0 * e),                      # read z, write q k v g (+ bias)
        "triattn_output":  ("hbm", 3.0 * e),                      # read o and z, write z
        "pair_bias":       ("hbm", 1.0 * e + 16 * n * n * 4),     # read z, write fp32 [16,N,N]
        "layernorm":       ("hbm", None),                         # single track only, tiny
    }


def _cpu_baseline(n_token: int, budget_note: str) -> dict:
    """One PairformerBlock of the oracle on the host cores, fp32, row-chunked
    triangle attention so the logits fit in RAM; reported x48."""
    import torch

    from oracle import pairformer_oracle as O

    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    blk = O.seed_parameters_(O.PairformerBlock()).eval()
    s, z, pm = O.make_inputs(n_token)
    with torch.no_grad():
        t0 = time.perf_counter()
        blk(s, z, pm, chunk_size=128)
        dt = time.perf_counter() - t0
    return {
        "value": round(dt * 1e3 * N_BLOCKS, 1),
        "unit": "ms",
        "cores": cores,
        "kind": "port",
        "sample": f"1 of {N_BLOCKS} blocks at N_token={n_token}, fp32, chunk_size=128, "
                  f"{dt:.2f} s measured, x{N_BLOCKS} extrapolated{budget_note}",
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--n-token", type=int, default=N_TOKEN)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported "
              "(the pair stack is not sharded in this build).", file=sys.stderr)
        return 2

    import torch

    import protenix_amd as P
    from oracle import pairformer_oracle as O
    from protenix_amd import ops

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    n = args.n_token
    dtype = torch.bfloat16

    # seeded weights (oracle's rule) loaded into the HIP-backed stack
    ref = O.seed_parameters_(O.PairformerStack(n_blocks=N_BLOCKS))
    stack = P.PairformerStack(n_blocks=N_BLOCKS)
    stack.load_state_dict(ref.state_dict())
    del ref
    stack = stack.to(dev, dtype).eval()
    s0, z0, pm = O.make_inputs(n, dtype=dtype)
    s0, z0, pm = s0.to(dev), z0.to(dev), pm.to(dev)
    z = torch.empty_like(z0)

    def step():
        z.copy_(z0)
        return stack(s0, z, pm, inplace_safe=True)

    with torch.no_grad():
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            s_out, z_out = step()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / max(1, args.steps)
        finite = bool(torch.isfinite(z_out.float()).all() and torch.isfinite(s_out.float()).all())
        peak_gb = torch.cuda.max_memory_allocated() / 1e9

        # instrumented pass: HIP events around every kernel launch, in place
        ops.kernel_timer = {}
        step()
        times = ops.kernel_times(ops.kernel_timer)
        ops.kernel_timer = None

    work = _work(n)
    kernels = []
    for name, durs in sorted(times.items(), key=lambda kv: -sum(kv[1])):
        avg = sum(durs) / len(durs)
        bound, amount = work.get(name, ("hbm", None))
        ent = {"kernel": name, "launches": len(durs), "avg_ms": round(avg, 4),
               "total_ms": round(sum(durs), 2), "bound": bound}
        if amount:
            if bound == "mfma":
                ach, peak, unit = amount / (avg * 1e-3) / 1e12, PEAK_BF16_TFLOPS, "TFLOP/s"
            else:
                ach, peak, unit = amount / (avg * 1e-3) / 1e9, PEAK_HBM_GBS, "GB/s"
            ent.update(achieved=round(ach, 1), peak=peak, unit=unit, frac=round(ach / peak, 4))
        kernels.append(ent)
    dom = next(k for k in kernels if k["kernel"] == "triattn_fwd")
    roofline = {"kernel": "triattn_fwd_kernel", "bound": "mfma", "achieved": dom["achieved"],
                "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": dom["frac"],
                "traffic": TRIATTN_FWD_TRAFFIC_BYTES_N768 if n == N_TOKEN else None,
                "avg_ms": dom["avg_ms"], "launches": dom["launches"],
                "algorithmic": "512*N^3 flop per launch (QK^T + PV over 4 heads x 32)"}

    out = {
        "metric": "Pairformer 48-block trunk fwd ms at N_token=768 bf16",
        "value": round(ms, 2),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 2),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"PairformerStack {N_BLOCKS} blocks forward, N_token={n}, c_z=128, "
                               "c_s=384, bf16, no grad, pair mask all ones, inplace_safe",
                   "n_token": n, "n_blocks": N_BLOCKS},
        "blocks_per_s": round(N_BLOCKS / (ms * 1e-3), 1),
        "ms_per_block": round(ms / N_BLOCKS, 3),
        "trunk_tflops": round(N_BLOCKS * 1.36e12 * (n / 768.0) ** 3 / (ms * 1e-3) / 1e12, 1),
        "output_finite": finite,
        "peak_hbm_gb": round(peak_gb, 2),
        "roofline": roofline,
        "kernels": kernels,
    }
    if not args.no_cpu_baseline:
        del stack, z, z0
        torch.cuda.empty_cache()
        out["cpu_baseline"] = _cpu_baseline(n, "")
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
