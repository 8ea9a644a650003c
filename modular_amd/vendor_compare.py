"""Times the per-token / per-channel scaled FP8 matmul of this library beside the vendor library's
(hipBLASLt, reached through `torch._scaled_mm` with row-wise scales) on one GPU, and reports how far the two
results are apart.

    python -m modular_amd.vendor_compare [--shapes M,N,K ...] [--reps 100]

The reference made the same comparison on MI355X before it dropped its hipBLASLt route for FP8
(max/kernels/src/linalg/matmul/gpu/__init__.mojo:820-838: nine (N, K) cells, among them N = 2304, K = 16384).
Only the row-wise form can be compared: the vendor library has no 128 x 128 block-scaled FP8 matmul.
Weights rotate through copies totalling more than the 256 MB last-level cache, so both sides read them from HBM.
"""
from __future__ import annotations

import argparse
import time

import torch

import modular_amd as mx
from modular_amd import synth

DEFAULT_SHAPES = [
    (2048, 28672, 4096), (2048, 4096, 14336), (4096, 7168, 16384), (4096, 24576, 1536), (4096, 32768, 512),
    (4096, 1536, 7168), (4096, 576, 7168), (8192, 8192, 8192), (2048, 2304, 16384), (256, 2304, 16384),
    (16, 2304, 16384), (256, 8192, 28672), (128, 8192, 28672), (64, 28672, 4096), (48, 8192, 28672),
    (32, 8192, 28672), (16, 57344, 8192), (8, 57344, 8192), (1, 57344, 8192),
]


def _time_us(fn, reps: int) -> float:
    # half a second of back-to-back launches first: an idle GPU needs that long to settle its clock
    t_end = time.perf_counter() + 0.4
    while time.perf_counter() < t_end:
        for _ in range(16):
            fn()
        torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps * 1e3


def compare(M: int, N: int, K: int, reps: int, dev: torch.device) -> dict:
    row = mx.rowwise_fp8_config()
    copies = max(2, int(600e6 // (N * K)))
    a = synth.random_fp8((M, K), 1, device=dev)
    sa = synth.random_scales((1, M), 3, device=dev)
    ws = [synth.random_fp8((N, K), 10 + i, device=dev) for i in range(copies)]
    sb = synth.random_scales((N, 1), 4, device=dev)
    sa_v, sb_v = sa.reshape(M, 1).contiguous(), sb.reshape(1, N).contiguous()
    turn = [0]

    def ours():
        turn[0] = (turn[0] + 1) % copies
        return mx.dynamic_scaled_matmul(a, ws[turn[0]], sa, sb, row.input_scale, row.weight_scale)

    def vendor():
        turn[0] = (turn[0] + 1) % copies
        return torch._scaled_mm(a, ws[turn[0]].t(), scale_a=sa_v, scale_b=sb_v, out_dtype=torch.bfloat16)

    out = {"M": M, "N": N, "K": K, "ours_us": round(_time_us(ours, reps), 1)}
    try:
        turn[0] = 0
        c_v = vendor().float()
        turn[0] = 0
        c_o = ours().float()
        out["max_abs_diff_over_max_abs"] = float((c_v - c_o).abs().max() / c_o.abs().max())
        out["vendor_us"] = round(_time_us(vendor, reps), 1)
        out["vendor_over_ours"] = round(out["vendor_us"] / out["ours_us"], 2)
    except (RuntimeError, NotImplementedError) as e:  # a torch build without the row-wise FP8 route
        out["vendor_error"] = f"{type(e).__name__}: {str(e)[:160]}"
    return out


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--shapes", nargs="*", default=None, help="M,N,K triples (default: Llama / DeepSeek-V3 cells)")
    ap.add_argument("--reps", type=int, default=100)
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("vendor_compare needs a GPU")
    shapes = [tuple(int(v) for v in s.split(",")) for s in args.shapes] if args.shapes else DEFAULT_SHAPES
    dev = torch.device("cuda:0")
    print(f"{'M':>6} {'N':>6} {'K':>6} {'ours us':>9} {'vendor us':>10} {'vendor/ours':>12} {'max|d|/max|c|':>14}")
    for (M, N, K) in shapes:
        r = compare(M, N, K, args.reps, dev)
        if "vendor_error" in r:
            print(f"{M:>6} {N:>6} {K:>6} {r['ours_us']:>9.1f}   {r['vendor_error']}", flush=True)
        else:
            print(f"{M:>6} {N:>6} {K:>6} {r['ours_us']:>9.1f} {r['vendor_us']:>10.1f} {r['vendor_over_ours']:>12.2f} "
                  f"{r['max_abs_diff_over_max_abs']:>14.2e}", flush=True)


if __name__ == "__main__":
    main()
