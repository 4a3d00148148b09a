"""One kernel at one size, launched a few times and timed with HIP events: the program to put
behind `rocprofv3 ... --` when a single kernel's counters are wanted.

    python -m longbow_quarrel_amd.kernels.probe linear --m 2048 --n 28672 --k 4096 [--tile 2x4] [--swiglu]
    python -m longbow_quarrel_amd.kernels.probe rmsnorm --m 2048 --n 4096

`--tile WMxWN` forces the tiled matrix-core kernel with that wave tile (float32 out, no epilogue)
whatever the dispatcher would choose.  Inputs are random; nothing is checked here (the tests do that).
"""
from __future__ import annotations

import argparse
import ctypes
import json
import sys

import torch

from .hip import HipKernels


def _time(fn, reps: int) -> float:
    fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e3 / reps  # microseconds


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="probe", description=__doc__, formatter_class=argparse.RawTextHelpFormatter)
    ap.add_argument("op", choices=["linear", "rmsnorm"])
    ap.add_argument("--m", type=int, default=8, help="rows")
    ap.add_argument("--n", type=int, default=4096, help="columns of the output (width for rmsnorm)")
    ap.add_argument("--k", type=int, default=4096, help="inner size of the product")
    ap.add_argument("--reps", type=int, default=3)
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--tile", default="", help="WMxWN: force the tiled kernel with this wave tile")
    ap.add_argument("--swiglu", action="store_true", help="the product with the fused SwiGLU epilogue (n = 2 I)")
    args = ap.parse_args(argv)

    kn = HipKernels()
    dev = "cuda:0"
    dtype = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    g = torch.Generator(device=dev).manual_seed(0)
    info = {"op": args.op, "m": args.m, "n": args.n, "k": args.k, "dtype": args.dtype}
    if args.op == "rmsnorm":
        x = torch.randn((args.m, args.n), generator=g, device=dev)
        w = torch.randn((args.n,), generator=g, device=dev)
        out = torch.empty((args.m, args.n), dtype=dtype, device=dev)
        us = _time(lambda: kn.rmsnorm(x, w, 1e-5, out), args.reps)
        info["GB/s"] = round((x.numel() * 4 + out.numel() * out.element_size()) / us / 1e3, 1)
    else:
        x = torch.randn((args.m, args.k), generator=g, device=dev).to(dtype)
        w = (torch.randn((args.n, args.k), generator=g, device=dev) * 0.02).to(dtype)
        if args.tile:
            wm, wn = (int(v) for v in args.tile.lower().split("x"))
            out = torch.empty((args.m, args.n), dtype=torch.float32, device=dev)
            p = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731

            def fn():
                kn._check(kn.lib.lq_debug_gemm_tiled(p(x), p(w), p(out), args.m, args.n, args.k, wm, wn, kn.stream))
            info["tile"] = args.tile
        elif args.swiglu:
            out = torch.empty((args.m, args.n // 2), dtype=dtype, device=dev)
            fn = lambda: kn.linear_swiglu(x, w, out)  # noqa: E731
        else:
            pieces = kn.linear_pieces(dtype, args.m, args.n, args.k)
            out = torch.empty((pieces, args.m, args.n) if pieces > 1 else (args.m, args.n),
                              dtype=torch.float32, device=dev)
            info["pieces"] = pieces
            fn = lambda: kn.linear(x, w, out)  # noqa: E731
        us = _time(fn, args.reps)
        info["TFLOP/s"] = round(2.0 * args.m * args.n * args.k / us / 1e6, 1)
        info["weight GB/s"] = round(w.numel() * w.element_size() / us / 1e3, 1)
    info["us"] = round(us, 2)
    print(json.dumps(info))
    return 0


if __name__ == "__main__":
    sys.exit(main())
