"""Run one kernel a few times on synthetic operands, for a profiler to look at.

    python -m dlgo_amd.kernels.probe gemm --n 16384 --k 2048 --t 2048 --epilogue swiglu --kind 20
    python -m dlgo_amd.kernels.probe prefill-attention --tokens 2048 --heads 32 --kv-heads 8 --head-dim 64
    python -m dlgo_amd.kernels.probe mfma-peak         # MFMAs on registers alone: the rate the chip sustains

Prints the mean wall time of a call, the host's share included (for short kernels that share is most of it).  Under
`rocprofv3 --pmc ...` or `--kernel-trace --stats` the kernel's own counters and durations are what one reads; this
program only provides the launches: one to warm up and --calls more.
"""
from __future__ import annotations

import argparse
import time

import torch

from . import ops

EPILOGUES = {"store": ops.EPI_STORE, "accumulate": ops.EPI_ACCUM_F32, "swiglu": ops.EPI_SWIGLU, "store-f32": ops.EPI_STORE_F32}


def _timed(fn, calls: int) -> float:
    fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(calls):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / calls


def gemm(args) -> None:
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    g = torch.Generator(device="cuda").manual_seed(0)
    w = (0.05 * torch.randn(args.n, args.k, device="cuda", generator=g)).to(dtype)
    x = torch.randn(args.t, args.k, device="cuda", generator=g).to(dtype)
    epi = EPILOGUES[args.epilogue]
    cols = args.n // 2 if epi == ops.EPI_SWIGLU else args.n
    out = torch.zeros(args.t, cols, device="cuda", dtype=torch.float32 if epi in (ops.EPI_ACCUM_F32, ops.EPI_STORE_F32) else dtype)
    scratch = torch.empty(ops.GEMM_SPLIT_FLOATS, device="cuda") if args.splits != 1 else None
    sec = _timed(lambda: ops.gemm(w, x, out, epi, args.kind, scratch=scratch, splits=args.splits), args.calls)
    print(f"gemm N={args.n} K={args.k} T={args.t} {args.dtype} {args.epilogue} kind {args.kind}: {sec * 1e6:.1f} us a call (with the host's share), "
          f"{2.0 * args.n * args.k * args.t / sec / 1e12:.0f} TFLOP/s, {args.n * args.k * w.element_size() / sec / 1e12:.2f} TB/s of weights")


def prefill_attention(args) -> None:
    from ..cache import PAGE
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    h, kv, hd, t = args.heads, args.kv_heads, args.head_dim, args.tokens
    pages = (t + PAGE - 1) // PAGE
    g = torch.Generator(device="cuda").manual_seed(0)
    cache = torch.randn(pages * 2 * kv * PAGE * hd, device="cuda", generator=g).to(dtype)
    q = torch.randn(t, h * hd, device="cuda", generator=g).to(dtype)
    out = torch.empty_like(q)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
    table = i32([list(range(pages))])
    positions, tok_seq, slots = i32(list(range(t))), i32([0] * t), i32([0])
    call = lambda: ops.attention(q, out, h, kv, hd, positions, tok_seq, slots, table, cache, 2 * kv * PAGE * hd, kv * PAGE * hd,
                                 q_lens=[t], start_pos=[0])
    sec = _timed(call, args.calls)
    flops = h * 2.0 * 2.0 * hd * t * (t + 1) / 2.0
    print(f"prefill attention T={t} H={h} KV={kv} hd={hd} {args.dtype}: {sec * 1e6:.1f} us a call (with the host's share), "
          f"{flops / sec / 1e12:.0f} TFLOP/s")


def mfma_peak(args) -> None:
    import ctypes

    from . import build
    lib = build.load("probe")
    lib.dlgo_probe_mfma.restype = ctypes.c_char_p
    out = torch.empty(args.blocks * 256, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def call():
        err = lib.dlgo_probe_mfma(ctypes.c_void_p(out.data_ptr()), args.blocks, args.iters, stream)
        if err:
            raise RuntimeError(err.decode())
    sec = _timed(call, args.calls)
    flops = args.blocks * 4 * args.iters * 16 * 32768.0
    print(f"MFMA 32x32x16 bf16 on registers alone, {args.blocks} blocks of 4 waves: {sec * 1e3:.2f} ms a call, "
          f"{flops / sec / 1e12:.0f} TFLOP/s")


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="what", required=True)
    a = sub.add_parser("gemm", help="out (epilogue)= x @ weight.T")
    a.add_argument("--n", type=int, required=True)
    a.add_argument("--k", type=int, required=True)
    a.add_argument("--t", type=int, required=True)
    a.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    a.add_argument("--epilogue", default="store", choices=sorted(EPILOGUES))
    a.add_argument("--kind", type=int, default=0, help="0 = the library's own choice")
    a.add_argument("--splits", type=int, default=1, help="runs of the inner size (0 = the library's own choice)")
    a.add_argument("--calls", type=int, default=3)
    a.set_defaults(run=gemm)
    b = sub.add_parser("prefill-attention", help="causal attention of one sequence's rows over its cache pages")
    b.add_argument("--tokens", type=int, default=2048)
    b.add_argument("--heads", type=int, default=32)
    b.add_argument("--kv-heads", type=int, default=8)
    b.add_argument("--head-dim", type=int, default=64)
    b.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    b.add_argument("--calls", type=int, default=3)
    b.set_defaults(run=prefill_attention)
    c = sub.add_parser("mfma-peak", help="matrix instructions on registers alone")
    c.add_argument("--blocks", type=int, default=256 * 8, help="blocks of four waves (256 compute units take 8 each at a time)")
    c.add_argument("--iters", type=int, default=20000)
    c.add_argument("--calls", type=int, default=3)
    c.set_defaults(run=mfma_peak)
    args = ap.parse_args()
    args.run(args)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
