"""Command-line timing of the 2D x 3D (MoE expert projection) path on one MI355X.

    python -m grouped_mm_bf16_amd.bench_2d3d --experts 8 --batch-size 8192 \
        --active-experts-per-token 2 --embedding-size 4096 --output-features 14336

Takes the flags of the reference's bench/bench_2d3d.py:73-113 that describe the
workload (experts, routing or uniform load, K, N, dtype, seed, iterations, mode,
which gradients) and reports the same two figures per line, milliseconds per call
and TFLOP/s of useful work (2 * routed tokens * K * N per product,
bench/bench_2d3d.py:183-186).  The reference's Triton tile knobs (--block-m ...,
--impl prologue|rowwise) have no meaning here; --impl selects the kernel family of
this library instead.  Timing is with events on the launch stream.
"""
from __future__ import annotations

import argparse

import torch

from . import kernels


def _routed_sizes(args, dev) -> torch.Tensor:
    if (args.batch_size is None) != (args.active_experts_per_token is None):
        raise SystemExit("--batch-size and --active-experts-per-token go together")
    if args.batch_size is None:
        return torch.full((args.experts,), args.tokens_per_expert, dtype=torch.int64, device=dev)
    if args.active_experts_per_token > args.experts:
        raise SystemExit("--active-experts-per-token cannot exceed --experts")
    # uniform random routing: every (token, slot) picks an expert
    picks = torch.randint(0, args.experts, (args.batch_size * args.active_experts_per_token,), device=dev)
    return torch.bincount(picks, minlength=args.experts)


def _time(fn, iters: int, warmup: int) -> float:
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--experts", type=int, default=64)
    ap.add_argument("--batch-size", type=int, default=None)
    ap.add_argument("--active-experts-per-token", type=int, default=None)
    ap.add_argument("--tokens-per-expert", type=int, default=2048)
    ap.add_argument("--embedding-size", type=int, default=32, help="K")
    ap.add_argument("--output-features", type=int, default=64, help="N")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp16", "fp32"])
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--iters", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--mode", default="forward", choices=["forward", "backward", "both"])
    ap.add_argument("--backward", default="both", choices=["da", "db", "both"])
    ap.add_argument("--impl", default="auto", choices=["auto", "mfma", "generic", "both"],
                    help="kernel family (both = mfma then generic)")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("needs a GPU")
    dev = torch.device("cuda")
    dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[args.dtype]
    torch.manual_seed(args.seed)

    sizes = _routed_sizes(args, dev)
    offs = sizes.cumsum(0).to(torch.int32)
    rows = int(offs[-1].item())
    k, n, g = args.embedding_size, args.output_features, args.experts
    a = torch.randn(rows, k, device=dev, dtype=dtype)
    b = torch.randn(g, k, n, device=dev, dtype=dtype)
    grad_out = torch.randn(rows, n, device=dev, dtype=dtype)
    out = torch.empty(rows, n, device=dev, dtype=dtype)
    grad_a, grad_b = torch.empty_like(a), torch.empty_like(b)
    # gradients of the 2D x 3D product as forward variants on transposed views
    b_t, a_t = b.transpose(1, 2), a.transpose(0, 1)

    def forward():
        kernels.grouped_mm_2d3d(a, b, offs, out)

    want_da, want_db = args.backward in ("da", "both"), args.backward in ("db", "both")

    def backward():
        if want_da:
            kernels.grouped_mm_2d3d(grad_out, b_t, offs, grad_a)
        if want_db:
            kernels.grouped_mm_2d2d(a_t, grad_out, offs, grad_b)

    load = (f"batch_size={args.batch_size}, active_experts_per_token={args.active_experts_per_token}"
            if args.batch_size is not None else f"tokens_per_expert={args.tokens_per_expert}")
    desc = (f"(experts={g}, total_routed_tokens={rows}, {load}, embedding_size={k}, "
            f"output_features={n}, dtype={args.dtype}, seed={args.seed})")
    product = 2.0 * rows * k * n
    for impl in (["mfma", "generic"] if args.impl == "both" else [args.impl]):
        with kernels.forced_path(impl):
            try:
                if args.mode in ("forward", "both"):
                    ms = _time(forward, args.iters, args.warmup)
                    print(f"{impl:7s}  forward  {ms:9.4f} ms  {product / ms / 1e9:8.3f} TFLOPs   {desc}  family={kernels.last_path()}")
                if args.mode in ("backward", "both"):
                    ms = _time(backward, args.iters, args.warmup)
                    flops = product * (int(want_da) + int(want_db))
                    print(f"{impl:7s}  backward {ms:9.4f} ms  {flops / ms / 1e9:8.3f} TFLOPs   {desc}  backward={args.backward}")
            except RuntimeError as ex:
                print(f"{impl:7s}  not applicable to these shapes: {ex}")


if __name__ == "__main__":
    main()
