"""Re-measure the alternatives behind the library's dispatch thresholds on the GPU at hand.

    python -m lego_amd.tune transpose --dtype f16 --shapes 9999x10001,8200x8192
    python -m lego_amd.tune rows --shapes 8192x6144,8192x7168
    python -m lego_amd.tune gemm --shapes 8192x8192x1024,4096x4096x4096
    python -m lego_amd.tune grouped

Every alternative is launched through a tuning entry point of ``include/lego_hip.h`` (a tiling, a team size, a
kernel variant or a split chosen by hand) in ONE process, on buffers that rotate through more than the 256 MB
last-level cache holds, after enough back-to-back launches for the part's clocks to settle.  Boxes differ by a few
per cent, so only figures of one run compare.  Prints one line per shape; changes nothing: the thresholds are
constants in ``lego_amd/build.py`` and ``lego_amd/csrc/lego_hip_abi.hip``.
"""
from __future__ import annotations

import argparse
import ctypes
import math
import sys


def _timed(torch, fn, steps=100, settle_ms=40.0):
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(5):
        fn()
    stop.record()
    torch.cuda.synchronize()
    per_call = max(start.elapsed_time(stop) / 5, 1e-3)
    for _ in range(min(5000, int(settle_ms / per_call) + 1)):
        fn()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def _rotating(torch, make, each_bytes, pool_bytes=1 << 30):
    return [make() for _ in range(max(2, math.ceil(pool_bytes / each_bytes)))]


def _shapes(text, rank):
    out = [tuple(int(v) for v in s.split("x")) for s in text.split(",") if s]
    assert all(len(s) == rank for s in out), f"shapes must be {'x'.join('N' * rank)}"
    return out


def tune_transpose(torch, lib, ns):
    """Every tiling of ``build.TRANSPOSE[dtype]`` that takes the shape, by its number in that list."""
    from .build import TRANSPOSE
    tdt, es = (torch.half, 2) if ns.dtype == "f16" else (torch.float32, 4)
    entry = getattr(lib, f"lego_hip_transpose_{ns.dtype}_tiling")
    auto = getattr(lib, f"lego_hip_transpose_{ns.dtype}")
    stream, p = _stream(torch), _ptr
    for R, C in _shapes(ns.shapes or "9999x10001,8200x8192,10000x10000,16384x16384", 2):
        sets = _rotating(torch, lambda: (torch.randn(R, C, device="cuda").to(tdt), torch.empty(C, R, device="cuda", dtype=tdt)),
                         2 * es * R * C)
        turn = [0]
        out = []
        for n, cfg in [(-1, None)] + list(enumerate(TRANSPOSE[ns.dtype])):
            def fn():
                s = sets[turn[0] % len(sets)]
                turn[0] += 1
                return auto(p(s[0]), p(s[1]), R, C, stream) if n < 0 else entry(p(s[0]), p(s[1]), R, C, n, stream)
            if fn() != 0:
                continue          # this tiling does not take the shape
            torch.cuda.synchronize()
            label = "dispatch" if n < 0 else f"#{n} {cfg['tile'][0] * cfg['group'][0]}x{cfg['tile'][1] * cfg['group'][1]} " \
                f"{cfg['order'] if isinstance(cfg['order'], str) else '-'.join(str(v) for v in cfg['order'])}" \
                f"{' ragged' if cfg.get('ragged') else ' edge' if cfg.get('edge') else ''}"
            out.append(f"{label}: {2 * es * R * C / _timed(torch, fn) / 1e6:.0f}")
        print(f"transpose {ns.dtype} {R}x{C} [GB/s]  " + " | ".join(out), flush=True)
        del sets


def tune_rows(torch, lib, ns):
    """fp16 softmax and LayerNorm forward with 1, 2, 4, 8 and 16 waves per row against the dispatch."""
    stream, p = _stream(torch), _ptr
    for M, N in _shapes(ns.shapes or "8192x8192,8192x6144,16384x4096,4096x4096", 2):
        sets = _rotating(torch, lambda: ((2 * torch.randn(M, N, device="cuda")).half(), torch.empty(M, N, device="cuda", dtype=torch.half)),
                         4 * M * N)
        w = (1 + 0.1 * torch.randn(N, device="cuda")).half()
        b = (0.1 * torch.randn(N, device="cuda")).half()
        mean, rstd = torch.empty(M, device="cuda"), torch.empty(M, device="cuda")
        eps = ctypes.c_float(1e-5)
        turn = [0]
        for kind in ("softmax", "layernorm_fwd"):
            out = []
            for wpr in (0, 1, 2, 4, 8, 16):
                def fn():
                    s = sets[turn[0] % len(sets)]
                    turn[0] += 1
                    if kind == "softmax":
                        return lib.lego_hip_softmax_f16(p(s[0]), p(s[1]), M, N, stream) if wpr == 0 else \
                            lib.lego_hip_softmax_f16_wpr(p(s[0]), p(s[1]), M, N, wpr, stream)
                    return lib.lego_hip_layernorm_fwd_f16(p(s[0]), p(s[1]), p(w), p(b), p(mean), p(rstd), M, N, eps, stream) if wpr == 0 else \
                        lib.lego_hip_layernorm_fwd_f16_wpr(p(s[0]), p(s[1]), p(w), p(b), p(mean), p(rstd), M, N, eps, wpr, stream)
                if fn() != 0:
                    continue      # the row does not fit a team of this size
                torch.cuda.synchronize()
                out.append(f"{'dispatch' if wpr == 0 else f'{wpr} waves'}: {4 * M * N / _timed(torch, fn) / 1e6:.0f}")
            print(f"{kind} f16 {M}x{N} [GB/s]  " + " | ".join(out), flush=True)
        del sets


def tune_gemm(torch, lib, ns):
    """The fp16 256 x 256-tile kernel variants (MFMA shape, waves per SIMD) and the entry point's own choice."""
    stream, p = _stream(torch), _ptr
    names = {-1: "dispatch", 0: "16x16x32, 4 waves", 1: "32x32x16, 4 waves", 2: "32x32x16, 8 waves"}
    for M, N, K in _shapes(ns.shapes or "8192x8192x8192,8192x8192x1024,4096x4096x4096,2048x2048x2048", 3):
        a = (torch.randn(M, K, device="cuda") / math.sqrt(K)).half()
        b = (torch.randn(K, N, device="cuda") / math.sqrt(K)).half()
        c = torch.empty(M, N, device="cuda", dtype=torch.half)
        plan = (ctypes.c_int * 2)()
        assert lib.lego_hip_gemm_plan(M, N, K, plan) == 0
        out = [f"plan: {plan[0]} x {plan[0]} tiles, {plan[1]} x {plan[1]} MFMA blocks"]
        for v, label in names.items():
            def fn():
                return lib.lego_hip_gemm_f16(p(a), p(b), p(c), M, N, K, stream) if v < 0 else \
                    lib.lego_hip_gemm_f16_variant(p(a), p(b), p(c), M, N, K, v, stream)
            if fn() != 0:
                continue
            torch.cuda.synchronize()
            out.append(f"{label}: {2.0 * M * N * K / _timed(torch, fn, steps=30 if K >= 4096 else 100) / 1e9:.0f}")
        print(f"gemm f16 {M}x{N}x{K} [TFLOP/s]  " + " | ".join(out), flush=True)


def tune_grouped(torch, lib, ns):
    """The benchmark's grouped problem set with the tail of the launch split by hand (-1: 128 x 128 tiles)."""
    stream = _stream(torch)
    g = torch.Generator().manual_seed(5)
    idx = torch.randint(0, 3, (8, 3), generator=g)
    dims = [[(1024, 2048, 4096)[int(v)] for v in row] for row in idx]
    A = [(torch.randn(m, k, generator=g) / math.sqrt(k)).half().cuda() for m, n, k in dims]
    B = [(torch.randn(k, n, generator=g) / math.sqrt(k)).half().cuda() for m, n, k in dims]
    C = [torch.empty(m, n, dtype=torch.half, device="cuda") for m, n, k in dims]
    arr = ctypes.c_void_p * 8
    pa, pb, pc = arr(*[t.data_ptr() for t in A]), arr(*[t.data_ptr() for t in B]), arr(*[t.data_ptr() for t in C])
    sz = (ctypes.c_int * 24)(*[v for d in dims for v in d])
    plan = (ctypes.c_int * 3)()
    assert lib.lego_hip_grouped_gemm_f16_plan(sz, 8, plan) == 0
    flop = sum(2.0 * m * n * k for m, n, k in dims)
    out = [f"plan: tile {plan[0]}, {plan[1]} tiles, last {plan[2]} in halves"]
    for split in (None, -1, 0, 64, 96, 128, 160, 192, 224, 256, 320):
        def fn():
            return lib.lego_hip_grouped_gemm_f16(pa, pb, pc, sz, 8, stream) if split is None else \
                lib.lego_hip_grouped_gemm_f16_split(pa, pb, pc, sz, 8, split, stream)
        assert fn() == 0
        torch.cuda.synchronize()
        label = "dispatch" if split is None else "128x128 tiles" if split < 0 else f"split {split}"
        out.append(f"{label}: {flop / _timed(torch, fn) / 1e9:.0f}")
    print("grouped gemm f16, benchmark problem set [TFLOP/s]  " + " | ".join(out), flush=True)


def _stream(torch):
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("what", choices=("transpose", "rows", "gemm", "grouped"))
    ap.add_argument("--dtype", choices=("f16", "f32"), default="f16", help="transposes only")
    ap.add_argument("--shapes", default="", help="comma list, RxC (transpose, rows) or MxNxK (gemm); default: a few per kernel")
    ns = ap.parse_args(argv)
    import torch
    from . import runtime
    if not torch.cuda.is_available():
        print("lego_amd.tune: no GPU visible", file=sys.stderr)
        return 1
    lib = runtime.load_library()
    {"transpose": tune_transpose, "rows": tune_rows, "gemm": tune_gemm, "grouped": tune_grouped}[ns.what](torch, lib, ns)
    return 0


if __name__ == "__main__":
    sys.exit(main())
