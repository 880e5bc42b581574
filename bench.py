#!/usr/bin/env python3
"""Benchmark of the lego_hip hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  A "step" is one launch of the headline workload, the fp16
16384x16384 transpose through the LEGO tiled + XOR-swizzled staging layout (the configuration
the headline metric is quoted on); ``value`` is its effective HBM bandwidth with the input
already resident in device memory.  The other four configurations are timed in the same
run with the same K and W and reported under ``kernels`` with their own roofline
fractions.  ``cpu_baseline`` times the reference's CPU path for the headline workload -- the source and
destination offsets as LEGO's Python/Triton printer emits them, evaluated with ``torch.arange`` for
``tl.arange``, then one gather/scatter -- on a bounded panel of the same matrix, on this host's
cores; the other configurations carry their own ``cpu_baseline`` (PyTorch CPU operators, as the
reference's CPU path has them) under ``kernels``.

Timing uses HIP events recorded on the stream the kernels are launched on (torch's
current stream).  Working sets that fit the 256 MB Infinity Cache are timed twice: "hot"
(same buffers every launch) and "rotating" (a pool of buffers larger than the cache).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16/bf16 MFMA, published
MFMA_FP8_PEAK_TFLOPS = 5000.0  # MI355X dense fp8 MFMA, published

SETTLE_MS = 40.0               # untimed device time before every timed region, see timed()

HEADLINE_KERNEL = "lego_transpose_f16_64x256_w128x8"
TRAFFIC_PROFILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "hbm_traffic_pmc.txt")


def headline_traffic_bytes():
    """HBM bytes per launch of the headline kernel, read from the committed counter summary (rocprofv3
    --pmc FETCH_SIZE / WRITE_SIZE, scaled by what the same counters read for a plain copy of known
    size): the "scaled bytes" column of the kernel's row.  None when the summary has no such row."""
    try:
        with open(TRAFFIC_PROFILE) as fh:
            for line in fh:
                if line.startswith((HEADLINE_KERNEL + " ", HEADLINE_KERNEL + "<")):
                    numbers = [int(tok) for tok in line.split(")", 1)[1].split() if tok.isdigit()]
                    return numbers[2]          # fetch KiB, write KiB, scaled bytes, algorithmic
    except (OSError, IndexError, ValueError):
        pass
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--skip-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--settle-ms", type=float, default=SETTLE_MS,
                    help="untimed device time of back-to-back launches before every timed region (0 for counter runs, "
                         "whose values do not depend on the clocks)")
    ap.add_argument("--sustain", type=float, default=0.0, metavar="SECONDS",
                    help="after timing the 8192^3 GEMM, keep launching it back to back for this long (for sampling "
                         "socket power and clocks with amd-smi from another process) and report the sustained rate")
    ap.add_argument("--only", default="", help="comma list of configs to time (c1,c2,c3,c4,c5,extra,apps,energy,timeline); "
                    "c2 is always timed; 'extra' adds LayerNorm backward and the other GEMM layouts and element "
                    "types, 'apps' the stencil, Needleman-Wunsch and LUD programs, 'energy' (with c4) the sustained "
                    "comparison of GEMM variants and MFMA-only streams for power sampling, 'timeline' (when named) the "
                    "per-phase times of the tiles of the fp16 GEMM and grouped GEMM from their measurement build")
    ns = ap.parse_args()
    if ns.gpus != 1:
        print("bench.py: this build measures one MI355X; every configuration of the hot path is a "
              "single-GPU kernel and --gpus above 1 is not supported", file=sys.stderr)
        sys.exit(2)

    import torch
    from lego_amd import ops, runtime
    runtime.load_library()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    K, W = ns.steps, ns.warmup
    only = set(filter(None, ns.only.split(",")))

    def want(name):
        return not only or name in only

    def timed(fn, steps=K, warmup=W, settle_ms=None):
        """Average milliseconds per call over exactly ``steps`` calls timed with events on the launch
        stream.  Untimed before them: ``warmup`` calls, then as many more as fill SETTLE_MS of device
        time, queued back to back with the timed ones -- after an idle gap the part needs about 20 ms
        of continuous work to return to its steady clocks (a launch of the row softmax reads 4.3 TB/s
        in the first 2 ms after a gap, 5.8 after 10 ms and 6.15 from 25 ms on)."""
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        for _ in range(max(1, warmup)):
            fn()
        stop.record()
        torch.cuda.synchronize()
        per_call = start.elapsed_time(stop) / max(1, warmup)
        settle = ns.settle_ms if settle_ms is None else settle_ms
        for _ in range(min(5000, int(settle / max(per_call, 1e-3)) + 1) if settle > 0 else 0):
            fn()
        start.record()
        for _ in range(steps):
            fn()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / steps

    def rotating(make, call, pool_bytes, each_bytes):
        """Time ``call(buffers)`` cycling through enough buffer sets to exceed the cache."""
        n = max(2, math.ceil(pool_bytes / each_bytes))
        sets = [make() for _ in range(n)]
        state = {"i": 0}

        def fn():
            call(sets[state["i"] % n])
            state["i"] += 1
        return timed(fn)

    cpu_threads = torch.get_num_threads()

    def cpu_timed(fn, unit_count, unit, sample):
        """One timed run of a CPU-path function: a ``cpu_baseline`` entry (None with --skip-cpu)."""
        if ns.skip_cpu:
            return None
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        return dict(value=unit_count / dt / 1e9, unit=unit, cores=cpu_threads, kind="port",
                    sample=f"{sample}; {dt:.2f} s, one run, {cpu_threads} threads of {os.cpu_count()} visible cores")

    kernels = {}
    gen = lambda seed: torch.Generator().manual_seed(seed)  # noqa: E731

    # ---- C2 (headline): fp16 16384^2 transpose ------------------------------------------
    n2 = 16384
    x2 = torch.randn(n2, n2, generator=gen(1)).half().to(dev)
    out2 = ops.transpose(x2)
    assert torch.equal(out2, x2.t()), "transpose parity failed"
    bytes2 = 2 * n2 * n2 * 2
    y2 = torch.empty_like(x2)
    # the timed region calls the C ABI directly on preallocated buffers
    import ctypes
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731

    def c2():
        runtime.call("lego_hip_transpose_f16", p(x2), p(y2), n2, n2, stream)
    ms2 = timed(c2)
    gbs2 = bytes2 / ms2 / 1e6
    copy_ms = timed(lambda: y2.copy_(x2))
    copy_gbs = bytes2 / copy_ms / 1e6
    copy16_ms = timed(lambda: runtime.call("lego_hip_copy16", p(x2), p(y2), ctypes.c_ulonglong(bytes2 // 2), stream))
    kernels["c2_transpose_f16_16384"] = dict(ms=ms2, gbs=gbs2, frac_hbm=gbs2 / HBM_PEAK_GBS,
                                             bytes=bytes2, parity="bit-exact")
    kernels["device_copy_512MiB"] = dict(ms=copy_ms, gbs=copy_gbs, frac_hbm=copy_gbs / HBM_PEAK_GBS,
                                         note="torch copy_ of the same buffers")
    stream_ms = timed(lambda: runtime.call("lego_hip_copy16_stream", p(x2), p(y2), ctypes.c_ulonglong(bytes2 // 2), stream))
    kernels["device_copy_stream_512MiB"] = dict(
        ms=stream_ms, gbs=bytes2 / stream_ms / 1e6, frac_hbm=bytes2 / stream_ms / 1e6 / HBM_PEAK_GBS,
        note="non-temporal copy of the same buffers, one contiguous 16 KiB chunk per workgroup: what a kernel that "
             "reads and writes every byte once reaches here")
    kernels["device_copy16_512MiB"] = dict(ms=copy16_ms, gbs=bytes2 / copy16_ms / 1e6,
                                           note="plain 16-byte-per-lane copy kernel of this library (counter calibration)")

    # ---- what the memory delivers here: one-directional streams and copies on rotating 512 MiB buffers ----------
    # (three pairs in turn, so that nothing is served by the 256 MB last-level cache).  A kernel that reads and writes
    # every byte once spends half its bytes in each direction: it cannot pass 1 / (0.5 / read + 0.5 / write).
    probe_bytes = 512 << 20
    pin = [x2.view(-1)[:probe_bytes // 2]] + [torch.randn(probe_bytes // 2, device=dev).half() for _ in range(2)]
    pout = [y2.view(-1)[:probe_bytes // 2]] + [torch.empty(probe_bytes // 2, dtype=torch.half, device=dev) for _ in range(2)]
    turn_p = [0]

    def probe(mode, vectors):
        def fn():
            turn_p[0] = (turn_p[0] + 1) % 3
            runtime.call("lego_hip_hbm_probe", p(pin[turn_p[0]]), p(pout[turn_p[0]]), ctypes.c_ulonglong(probe_bytes),
                         mode, vectors, stream)
        return fn
    ceiling = {}
    for label, mode, vectors, moved in (("read_only_16KiB_per_wg", 0, 4, 1), ("write_only_16KiB_per_wg", 1, 4, 1),
                                        ("read_only_4KiB_per_wg", 0, 1, 1), ("write_only_4KiB_per_wg", 1, 1, 1),
                                        ("copy_16KiB_per_wg", 2, 4, 2), ("copy_4KiB_per_wg", 2, 1, 2)):
        ms_p = timed(probe(mode, vectors))
        ceiling[label] = dict(ms=ms_p, gbs=moved * probe_bytes / ms_p / 1e6)
    read_gbs = max(ceiling["read_only_16KiB_per_wg"]["gbs"], ceiling["read_only_4KiB_per_wg"]["gbs"])
    write_gbs = max(ceiling["write_only_16KiB_per_wg"]["gbs"], ceiling["write_only_4KiB_per_wg"]["gbs"])
    achievable = 1.0 / (0.5 / read_gbs + 0.5 / write_gbs)
    ceiling["read_plus_write_bound_gbs"] = achievable
    ceiling["note"] = ("non-temporal 16-byte accesses, 256 lanes per workgroup, 1 or 4 vectors per lane; three rotating pairs "
                       "of 512 MiB buffers; read_plus_write_bound = 1 / (0.5 / best read-only + 0.5 / best write-only): the "
                       "rate a kernel that reads and writes every byte once cannot pass on this part")
    kernels["hbm_ceiling"] = ceiling
    kernels["c2_transpose_f16_16384"].update(achievable_gbs=achievable, frac_of_achievable=gbs2 / achievable)
    c2()      # y2 holds the transpose again (the probes wrote into it)
    del pin, pout

    # ---- C1: fp32 4096^2 transpose ---------------------------------------------------------
    if want("c1"):
        n1 = 4096
        x1 = (torch.rand(n1, n1, generator=gen(0), dtype=torch.float32) * 2 - 1).to(dev)
        assert torch.equal(ops.transpose(x1), x1.t())
        y1 = torch.empty_like(x1)
        b1 = 2 * n1 * n1 * 4
        hot = timed(lambda: runtime.call("lego_hip_transpose_f32", p(x1), p(y1), n1, n1, stream))
        rot = rotating(lambda: (torch.rand(n1, n1, device=dev), torch.empty(n1, n1, device=dev)),
                       lambda s: runtime.call("lego_hip_transpose_f32", p(s[0]), p(s[1]), n1, n1, stream),
                       1 << 30, b1)
        # a launch this short pays its ramp: the same bytes through a plain copy (one 16-byte vector per lane), same pool
        rot_copy = rotating(lambda: (torch.rand(n1, n1, device=dev), torch.empty(n1, n1, device=dev)),
                            lambda s: runtime.call("lego_hip_hbm_probe", p(s[0]), p(s[1]), n1 * n1 * 4, 2, 1, stream),
                            1 << 30, b1)
        kernels["c1_transpose_f32_4096"] = dict(ms_hot=hot, gbs_hot=b1 / hot / 1e6, ms=rot, gbs=b1 / rot / 1e6,
                                                frac_hbm=b1 / rot / 1e6 / HBM_PEAK_GBS, bytes=b1,
                                                achievable_gbs=achievable, frac_of_achievable=b1 / rot / 1e6 / achievable,
                                                plain_copy_same_bytes_gbs=b1 / rot_copy / 1e6,
                                                frac_of_plain_copy=rot_copy / rot,
                                                parity="bit-exact",
                                                note="gbs = rotating buffers (1 GiB pool); gbs_hot = cache resident; "
                                                     "plain_copy_same_bytes = a copy kernel over the same 2 x 64 MiB")
        if not ns.skip_cpu:
            from lego_amd.kernels.transpose import python_offsets
            from oracle import cpu_path
            s1, d1 = python_offsets(32, 32)
            x1c = x1.cpu()
            got1 = {}
            kernels["c1_transpose_f32_4096"]["cpu_baseline"] = cpu_timed(
                lambda: got1.update(y=cpu_path.transpose_printed(x1c, s1, d1, 32, 32)), b1, "GB/s",
                "the whole 4096x4096 fp32 matrix: printed offsets of both TileBy([128,128],[32,32]) layouts "
                "evaluated with torch.arange, then one gather/scatter")
            assert torch.equal(got1["y"], ops.transpose(x1).cpu()), "GPU result differs from the CPU path"
            del x1c, got1
        del x1, y1

    # ---- C3: softmax and LayerNorm forward, fp16 8192x8192 -------------------------------------
    if want("c3"):
        m3 = n3 = 8192
        x3c = (2.0 * torch.randn(m3, n3, generator=gen(2))).half()
        g3 = gen(3)
        w3c = (1 + 0.1 * torch.randn(n3, generator=g3)).half()
        b3c = (0.1 * torch.randn(n3, generator=g3)).half()
        x3, w3, b3 = x3c.to(dev), w3c.to(dev), b3c.to(dev)
        y3 = torch.empty_like(x3)
        mean3 = torch.empty(m3, device=dev)
        rstd3 = torch.empty(m3, device=dev)
        by3 = 2 * m3 * n3 * 2
        ref_s = torch.softmax(x3.float(), -1)
        err_s = (ops.softmax(x3).float() - ref_s).abs().max().item()
        ref_l = torch.nn.functional.layer_norm(x3.float(), (n3,), w3.float(), b3.float(), 1e-5)
        err_l = (ops.layer_norm_fwd(x3, w3, b3, 1e-5)[0].float() - ref_l).abs().max().item()
        del ref_s, ref_l

        def sm(s=None):
            xx, yy = (x3, y3) if s is None else s
            runtime.call("lego_hip_softmax_f16", p(xx), p(yy), m3, n3, stream)

        def ln(s=None):
            xx, yy = (x3, y3) if s is None else s
            runtime.call("lego_hip_layernorm_fwd_f16", p(xx), p(yy), p(w3), p(b3), p(mean3), p(rstd3),
                         m3, n3, ctypes.c_float(1e-5), stream)
        mk = lambda: (x3.clone(), torch.empty_like(x3))  # noqa: E731
        for name, fn, err in (("c3_softmax_f16_8192", sm, err_s), ("c3_layernorm_fwd_f16_8192", ln, err_l)):
            hot = timed(fn)
            rot = rotating(mk, fn, 1 << 30, by3)
            kernels[name] = dict(ms_hot=hot, gbs_hot=by3 / hot / 1e6, ms=rot, gbs=by3 / rot / 1e6,
                                 frac_hbm=by3 / rot / 1e6 / HBM_PEAK_GBS, bytes=by3, max_abs_err_vs_fp32=err,
                                 achievable_gbs=achievable, frac_of_achievable=by3 / rot / 1e6 / achievable,
                                 note="gbs = rotating buffers (1 GiB pool); gbs_hot = cache resident; "
                                      "x ~ N(0, sigma=2)")
        if not ns.skip_cpu:
            from oracle import kernels as ok3
            kernels["c3_softmax_f16_8192"]["cpu_baseline"] = cpu_timed(
                lambda: ok3.softmax(x3c), by3, "GB/s", "the whole 8192x8192 matrix: torch.softmax(x.float(), -1).half()")
            kernels["c3_layernorm_fwd_f16_8192"]["cpu_baseline"] = cpu_timed(
                lambda: ok3.layernorm_fwd(x3c, w3c, b3c, 1e-5), by3, "GB/s",
                "the whole 8192x8192 matrix: F.layer_norm(x.float(), ...).half() plus mean and rstd")
        # next row: LayerNorm backward (reference formula: 3 * numel * element size, layernorm.py:555)
        if want("extra"):
            dy3 = (0.1 * torch.randn(m3, n3, generator=gen(6))).half().to(dev)
            ln()
            torch.cuda.synchronize()
            need = ctypes.c_ulonglong(0)
            runtime.call("lego_hip_layernorm_bwd_workspace_bytes", m3, n3, ctypes.byref(need))
            ws = torch.empty(need.value // 4, device=dev)
            dx3, dw3, db3 = torch.empty_like(x3), torch.empty_like(w3), torch.empty_like(b3)

            def lnb():
                runtime.call("lego_hip_layernorm_bwd_f16", p(dy3), p(x3), p(w3), p(mean3), p(rstd3), p(dx3), p(dw3),
                             p(db3), p(ws), need, m3, n3, stream)
            ms_b = timed(lnb)
            kernels["next_layernorm_bwd_f16_8192"] = dict(ms=ms_b, gbs=3 * m3 * n3 * 2 / ms_b / 1e6,
                                                         frac_hbm=3 * m3 * n3 * 2 / ms_b / 1e6 / HBM_PEAK_GBS,
                                                         bytes=3 * m3 * n3 * 2, note="cache-resident buffers")
            del dy3, dx3, ws
            # rows of any length: 8191 elements (the rows of a workgroup start alike and split at the same columns) and
            # a transpose of odd sides (16-byte accesses at any element); rotating inputs
            mr, nr = 16386, 8191
            gr = gen(7)
            xr = [(2.0 * torch.randn(mr, nr, generator=gr)).half().to(dev) for _ in range(3)]
            dyr = (0.1 * torch.randn(mr, nr, generator=gr)).half().to(dev)
            wr = (1 + 0.1 * torch.randn(nr, generator=gr)).half().to(dev)
            br = (0.1 * torch.randn(nr, generator=gr)).half().to(dev)
            yr, dxr = [torch.empty_like(xr[0]) for _ in range(3)], torch.empty_like(xr[0])     # results rotate too
            dwr, dbr = torch.empty_like(wr), torch.empty_like(br)
            meanr, rstdr = torch.empty(mr, device=dev), torch.empty(mr, device=dev)
            runtime.call("lego_hip_layernorm_bwd_workspace_bytes", mr, nr, ctypes.byref(need))
            wsr = torch.empty(need.value // 4, device=dev)
            turn = [0]

            def lnr():
                turn[0] = (turn[0] + 1) % 3
                runtime.call("lego_hip_layernorm_fwd_f16", p(xr[turn[0]]), p(yr[turn[0]]), p(wr), p(br), p(meanr), p(rstdr), mr, nr, 1e-5, stream)

            def smr():
                turn[0] = (turn[0] + 1) % 3
                runtime.call("lego_hip_softmax_f16", p(xr[turn[0]]), p(yr[turn[0]]), mr, nr, stream)

            def lnbr():
                turn[0] = (turn[0] + 1) % 3
                runtime.call("lego_hip_layernorm_bwd_f16", p(dyr), p(xr[turn[0]]), p(wr), p(meanr), p(rstdr), p(dxr), p(dwr),
                             p(dbr), p(wsr), need, mr, nr, stream)
            for name, fn, passes in (("next_softmax_f16_16386x8191_any_length", smr, 2),
                                     ("next_layernorm_fwd_f16_16386x8191_any_length", lnr, 2),
                                     ("next_layernorm_bwd_f16_16386x8191_any_length", lnbr, 3)):
                ms_r = timed(fn)
                kernels[name] = dict(ms=ms_r, gbs=passes * mr * nr * 2 / ms_r / 1e6,
                                     frac_hbm=passes * mr * nr * 2 / ms_r / 1e6 / HBM_PEAK_GBS)
            del xr, dyr, yr, dxr, wsr
            for rows_t, cols_t in ((9999, 10001),):
                xt = [torch.randn(rows_t, cols_t, generator=gr).half().to(dev) for _ in range(3)]
                # the results rotate as well: written to one buffer that the last-level cache holds, call after call, plain
                # stores never reach memory (4.6 instead of 3.5 TB/s)
                ot = [torch.empty(cols_t, rows_t, dtype=torch.half, device=dev) for _ in range(3)]

                def trr():
                    turn[0] = (turn[0] + 1) % 3
                    runtime.call("lego_hip_transpose_f16", p(xt[turn[0]]), p(ot[turn[0]]), rows_t, cols_t, stream)
                trr()
                assert torch.equal(ot[turn[0]], xt[turn[0]].t())
                ms_t = timed(trr)
                kernels[f"next_transpose_f16_{rows_t}x{cols_t}_any_shape"] = dict(
                    ms=ms_t, gbs=2 * rows_t * cols_t * 2 / ms_t / 1e6, frac_hbm=2 * rows_t * cols_t * 2 / ms_t / 1e6 / HBM_PEAK_GBS)
                del xt, ot
        del x3, y3

    # ---- C4: fp16 GEMM 8192^3 ----------------------------------------------------------------------
    if want("c4"):
        n4 = 8192
        g4 = gen(4)
        a4 = (torch.randn(n4, n4, generator=g4) / math.sqrt(n4)).half().to(dev)
        b4 = (torch.randn(n4, n4, generator=g4) / math.sqrt(n4)).half().to(dev)
        c4 = torch.empty(n4, n4, dtype=torch.half, device=dev)
        fl4 = 2 * n4 ** 3

        def gm():
            runtime.call("lego_hip_gemm_f16", p(a4), p(b4), p(c4), n4, n4, n4, stream)
        gm()
        # parity on a 512-row panel against fp32 accumulation
        ref = a4[:512].float() @ b4.float()
        rel = ((c4[:512].float() - ref).norm() / ref.norm()).item()
        ms = timed(gm, steps=max(5, K // 5), warmup=max(2, W // 5))
        lib_ms = timed(lambda: torch.matmul(a4, b4, out=c4), steps=max(5, K // 5), warmup=max(2, W // 5))
        # Two consecutive 128 MiB allocations put B exactly 2^27 bytes after A, and with K = 8192 the A and
        # B request streams then meet in the same memory channels; the same operands with B moved by one
        # 128-byte line show what the kernel does without that coincidence.
        b4s_buf = torch.empty(n4 * n4 + 64, dtype=torch.half, device=dev)
        b4s = b4s_buf[64:].view(n4, n4)
        b4s.copy_(b4)

        def gms():
            runtime.call("lego_hip_gemm_f16", p(a4), p(b4s), p(c4), n4, n4, n4, stream)
        ms_s = timed(gms, steps=max(5, K // 5), warmup=max(2, W // 5))
        lib_ms_s = timed(lambda: torch.matmul(a4, b4s, out=c4), steps=max(5, K // 5), warmup=max(2, W // 5))
        # What the matrix cores sustain on operands of this distribution when a kernel issues nothing but MFMAs (one wave
        # per SIMD, 256 accumulator registers, fragments loaded once): the rate that the part's power management
        # leaves to an fp16 GEMM whose data movement costs nothing.
        probe_wgs, probe_iters = 256, 2048
        probe_ops = (torch.randn(probe_wgs * 32768, generator=g4) / math.sqrt(n4)).half().to(dev)
        probe_sink = torch.empty(probe_wgs * 512, device=dev)
        # flop per launch: one MFMA per accumulator block and round, 32 k-values deep for 16x16x32, 16 for 32x32x16
        probe_flop = {shape: probe_wgs * probe_iters * (4194304.0 if shape in (1, 3) else 2097152.0) for shape in range(5)}

        def mfma_only(shape):
            return lambda: runtime.call("lego_hip_mfma_probe", p(probe_ops), p(probe_sink), shape, probe_iters, probe_wgs, stream)
        ms_probe = timed(mfma_only(1), steps=max(5, K // 5), warmup=max(2, W // 5))
        ms_probe32 = timed(mfma_only(0), steps=max(5, K // 5), warmup=max(2, W // 5))
        mfma_achievable = probe_flop[1] / ms_probe / 1e9
        kernels["mfma_ceiling_f16"] = dict(
            ms=ms_probe, tflops=mfma_achievable, frac_mfma=mfma_achievable / MFMA_F16_PEAK_TFLOPS,
            tflops_32x32x16=probe_flop[0] / ms_probe32 / 1e9,
            note="v_mfma_f32_16x16x32_f16 only (the GEMM kernels' instruction), 256 workgroups of four waves, operands "
                 "N(0,1)/sqrt(8192) held in registers: what the part sustains at its power and current limits with the "
                 "pipe full; tflops_32x32x16 = the same with v_mfma_f32_32x32x16_f16")
        kernels["c4_gemm_f16_8192"] = dict(ms=ms, tflops=fl4 / ms / 1e9, frac_mfma=fl4 / ms / 1e9 / MFMA_F16_PEAK_TFLOPS,
                                           achievable_tflops=mfma_achievable, frac_of_achievable=fl4 / ms / 1e9 / mfma_achievable,
                                           flop=fl4, rel_err_vs_fp32=rel,
                                           vendor_library_tflops=fl4 / lib_ms / 1e9,
                                           b_address=f"a + {b4.data_ptr() - a4.data_ptr()} bytes",
                                           tflops_b_moved_128_bytes=fl4 / ms_s / 1e9,
                                           vendor_library_tflops_b_moved_128_bytes=fl4 / lib_ms_s / 1e9,
                                           note="vendor_library = torch.matmul (hipBLASLt) on the same buffers")
        del b4s, b4s_buf
        if ns.sustain > 0 and "energy" not in only:
            for name, fn in (("sustained", gm), ("vendor_library_sustained", lambda: torch.matmul(a4, b4, out=c4))):
                per = []
                t_end = time.perf_counter() + ns.sustain
                while time.perf_counter() < t_end:
                    per.append(timed(fn, steps=100, warmup=1))
                kernels["c4_gemm_f16_8192"][name + "_tflops"] = fl4 / (sum(per) / len(per)) / 1e9
                kernels["c4_gemm_f16_8192"][name + "_seconds"] = ns.sustain
                time.sleep(1.0)      # an idle second between the two, visible in the power samples
        if "energy" in only:
            # Energy-per-flop comparison: every variant back to back for --sustain seconds (default 3) with an idle second
            # between, wall-clock times recorded so that socket power and clocks sampled by another process (amd-smi in a
            # loop) can be laid beside them; counters for the same kernels come from a rocprofv3 --pmc run of this leg.
            seconds = ns.sustain if ns.sustain > 0 else 3.0
            c4w = torch.empty_like(c4)
            def variant(v, out):
                return lambda: runtime.call("lego_hip_gemm_f16_variant", p(a4), p(b4), p(out), n4, n4, n4, v, stream)
            for v in (1, 2):
                variant(v, c4w)()
                torch.cuda.synchronize()
                assert ((c4w[:512].float() - ref).norm() / ref.norm()).item() <= 1e-2
            phases = [("gemm 8192^3: 4 waves of 128x128, one per SIMD, 16x16x32 MFMA (built)", fl4, variant(0, c4)),
                      ("gemm 8192^3: 4 waves of 128x128, one per SIMD, 32x32x16 MFMA", fl4, variant(1, c4w)),
                      ("gemm 8192^3: 8 waves of 128x64, two per SIMD, 32x32x16 MFMA", fl4, variant(2, c4w)),
                      ("gemm 8192^3: vendor library (torch.matmul)", fl4, lambda: torch.matmul(a4, b4, out=c4)),
                      ("MFMA only: 32x32x16 f16, one wave per SIMD", probe_flop[0], mfma_only(0)),
                      ("MFMA only: 16x16x32 f16, one wave per SIMD", probe_flop[1], mfma_only(1)),
                      ("MFMA only: 32x32x16 f16, two waves per SIMD", probe_flop[4], mfma_only(4)),
                      ("MFMA only: 16x16x32 f16, two waves per SIMD", probe_flop[3], mfma_only(3)),
                      ("MFMA only: 32x32x16 bf16 (the same bits), one wave per SIMD", probe_flop[2], mfma_only(2))]
            table = []
            for label, flop, fn in phases:
                per = []
                t_begin = time.time()
                t_end = time.perf_counter() + seconds
                while time.perf_counter() < t_end:
                    per.append(timed(fn, steps=20, warmup=1, settle_ms=0.0))
                steady = per[len(per) // 3:]
                table.append(dict(variant=label, tflops=flop / (sum(steady) / len(steady)) / 1e9, wall_clock_begin=t_begin,
                                  wall_clock_end=time.time()))
                print(f"{t_begin:.2f} .. {time.time():.2f}  {label}: {table[-1]['tflops']:.1f} TFLOP/s", file=sys.stderr, flush=True)
                time.sleep(1.0)
            kernels["c4_energy_per_flop"] = table
            del c4w
        if not ns.skip_cpu:
            from oracle import kernels as ok4
            a4c, b4c = a4[:1024].cpu(), b4.cpu()
            kernels["c4_gemm_f16_8192"]["cpu_baseline"] = cpu_timed(
                lambda: ok4.gemm(a4c, b4c), 2 * 1024 * n4 * n4 / 1e3, "TFLOP/s",
                "rows 0..1023 of A (an eighth of the workload): (A.float() @ B.float()).half()")
            del a4c, b4c
        if want("extra"):
            for ta, tb in ((0, 1), (1, 0), (1, 1)):
                def gv(ta=ta, tb=tb):
                    runtime.call("lego_hip_gemm_f16_ex", p(a4), p(b4), p(c4), n4, n4, n4, ta, tb, 0, stream)
                msv = timed(gv, steps=max(5, K // 5), warmup=max(2, W // 5))
                kernels[f"next_gemm_f16_8192_{'t' if ta else 'n'}{'t' if tb else 'n'}"] = dict(
                    ms=msv, tflops=fl4 / msv / 1e9, frac_mfma=fl4 / msv / 1e9 / MFMA_F16_PEAK_TFLOPS)
            ab, bb = a4.bfloat16(), b4.bfloat16()
            cb = torch.empty_like(ab)

            def gb():
                runtime.call("lego_hip_gemm_bf16_ex", p(ab), p(bb), p(cb), n4, n4, n4, 0, 0, 0, stream)
            msb = timed(gb, steps=max(5, K // 5), warmup=max(2, W // 5))
            lib_msb = timed(lambda: torch.matmul(ab, bb, out=cb), steps=max(5, K // 5), warmup=max(2, W // 5))
            kernels["next_gemm_bf16_8192"] = dict(ms=msb, tflops=fl4 / msb / 1e9,
                                                  frac_mfma=fl4 / msb / 1e9 / MFMA_F16_PEAK_TFLOPS,
                                                  vendor_library_tflops=fl4 / lib_msb / 1e9)
            del ab, bb, cb
            # 8-bit operands as the reference makes them: randn fp16 cast to float8_e5m2 (matmul_sympy.py:346-364)
            g8 = gen(6)
            a8 = torch.randn(n4, n4, generator=g8, dtype=torch.float16).to(torch.float8_e5m2).cuda()
            b8 = torch.randn(n4, n4, generator=g8, dtype=torch.float16).to(torch.float8_e5m2).cuda()
            c8 = torch.empty(n4, n4, dtype=torch.float16, device="cuda")

            def g8f():
                runtime.call("lego_hip_gemm_fp8_ex", p(a8), p(b8), p(c8), n4, n4, n4, 0, 0, 0, 1, stream)
            g8f()
            ref8 = a8[:256].float() @ b8.float()
            rel8 = ((c8[:256].float() - ref8).norm() / ref8.norm()).item()
            ms8 = timed(g8f, steps=max(5, K // 5), warmup=max(2, W // 5))
            # the same instruction with nothing around it, on operands of the same distribution
            ops8 = a8.view(-1)[:probe_wgs * 65536]
            ms_probe8 = timed(lambda: runtime.call("lego_hip_mfma_probe", p(ops8), p(probe_sink), 5, probe_iters // 2, probe_wgs, stream),
                              steps=max(5, K // 5), warmup=max(2, W // 5))
            ceiling8 = probe_wgs * (probe_iters // 2) * 8388608.0 / ms_probe8 / 1e9
            ms_probe8s = timed(lambda: runtime.call("lego_hip_mfma_probe", p(ops8), p(probe_sink), 7, probe_iters // 4, probe_wgs, stream),
                               steps=max(5, K // 5), warmup=max(2, W // 5))
            kernels["mfma_ceiling_fp8_e5m2"] = dict(
                ms=ms_probe8, tflops=ceiling8, frac_mfma=ceiling8 / MFMA_FP8_PEAK_TFLOPS,
                tflops_16x16x128=probe_wgs * (probe_iters // 4) * 16777216.0 / ms_probe8s / 1e9,
                note="v_mfma_f32_32x32x64_f8f6f4 only (the 8-bit GEMM kernels' instruction), operands randn cast to e5m2 "
                     "held in registers, 256 workgroups of four waves: what the part sustains with the pipe full; "
                     "tflops_16x16x128 = the same with v_mfma_f32_16x16x128_f8f6f4")
            kernels["next_gemm_fp8_e5m2_8192"] = dict(ms=ms8, tflops=fl4 / ms8 / 1e9,
                                                      frac_mfma=fl4 / ms8 / 1e9 / MFMA_FP8_PEAK_TFLOPS,
                                                      achievable_tflops=ceiling8, frac_of_achievable=fl4 / ms8 / 1e9 / ceiling8,
                                                      rel_err_vs_fp32=rel8, note="peak = 5.0 PFLOP/s dense fp8")
            del a8, b8, c8, ref8, ops8
            # shapes off the tile grid: ragged in M and N (lane masks in scalar registers instead of edge tests), and
            # a skinny product split along K with a workspace (bound by reading B once: GB/s of operand bytes)
            mr = nr = 8184
            cr = torch.empty(mr, nr, dtype=torch.float16, device="cuda")

            br = b4[:, :nr].contiguous()      # rows 0..8183 of A are its first rows as they lie; B's columns need their own buffer

            def gr2():
                runtime.call("lego_hip_gemm_f16_ex", p(a4), p(br), p(cr), mr, nr, n4, 0, 0, 0, stream)
            msr = timed(gr2, steps=max(5, K // 5), warmup=max(2, W // 5))
            flr = 2.0 * mr * nr * n4
            kernels["next_gemm_f16_8184x8184x8192_ragged"] = dict(ms=msr, tflops=flr / msr / 1e9,
                                                                  frac_mfma=flr / msr / 1e9 / MFMA_F16_PEAK_TFLOPS)
            del br, cr
            ms_k = 16
            a_s = a4[:ms_k].contiguous()
            c_s = torch.empty(ms_k, n4, dtype=torch.float16, device="cuda")
            need_s = ctypes.c_ulonglong(0)
            runtime.call("lego_hip_gemm_workspace_bytes", ms_k, n4, n4, ctypes.byref(need_s))
            ws_s = torch.empty(max(need_s.value, 16) // 4, device="cuda")

            def gs():
                runtime.call("lego_hip_gemm_ex_ws", 0, p(a_s), p(b4), p(c_s), ms_k, n4, n4, 0, 0, 0, p(ws_s), need_s, stream)
            mss = timed(gs, steps=K, warmup=W)
            lib_mss = timed(lambda: torch.matmul(a_s, b4, out=c_s), steps=K, warmup=W)
            bytes_s = 2.0 * (ms_k * n4 + n4 * n4 + ms_k * n4)
            kernels["next_gemm_f16_16x8192x8192_split_k"] = dict(ms=mss, gbs=bytes_s / mss / 1e6,
                                                                 frac_hbm=bytes_s / mss / 1e6 / HBM_PEAK_GBS,
                                                                 workspace_bytes=need_s.value, vendor_library_ms=lib_mss)
            del a_s, c_s, ws_s
            # N and K that are no multiples of 8: the tiled kernels on zero-padded copies in the caller's workspace
            mo = n4 - 1
            a_o = a4[:mo, :mo].contiguous()
            b_o = b4[:mo, :mo].contiguous()
            c_o = torch.empty(mo, mo, dtype=torch.float16, device="cuda")
            need_o = ctypes.c_ulonglong(0)
            runtime.call("lego_hip_gemm_workspace_bytes", mo, mo, mo, ctypes.byref(need_o))
            ws_o = torch.empty(max(need_o.value, 16) // 4, device="cuda")

            def go():
                runtime.call("lego_hip_gemm_ex_ws", 0, p(a_o), p(b_o), p(c_o), mo, mo, mo, 0, 0, 0, p(ws_o), need_o, stream)
            mso = timed(go, steps=max(5, K // 5), warmup=max(2, W // 5))
            lib_mso = timed(lambda: torch.matmul(a_o, b_o, out=c_o), steps=max(5, K // 5), warmup=max(2, W // 5))
            flo = 2.0 * mo * mo * mo
            kernels["next_gemm_f16_8191x8191x8191_zero_padded"] = dict(ms=mso, tflops=flo / mso / 1e9,
                                                                       frac_mfma=flo / mso / 1e9 / MFMA_F16_PEAK_TFLOPS,
                                                                       workspace_bytes=need_o.value, vendor_library_ms=lib_mso)
            del a_o, b_o, c_o, ws_o
        del a4, b4, c4, ref

    # ---- C5: grouped fp16 GEMM, 8 problems -------------------------------------------------------------
    if want("c5"):
        g5 = gen(5)
        idx = torch.randint(0, 3, (8, 3), generator=g5)
        dims = [[(1024, 2048, 4096)[int(v)] for v in row] for row in idx]
        A = [(torch.randn(m, k, generator=g5) / math.sqrt(k)).half().to(dev) for m, n, k in dims]
        B = [(torch.randn(k, n, generator=g5) / math.sqrt(k)).half().to(dev) for m, n, k in dims]
        C = [torch.empty(m, n, dtype=torch.half, device=dev) for m, n, k in dims]
        arr = ctypes.c_void_p * 8
        pa, pb, pc = arr(*[t.data_ptr() for t in A]), arr(*[t.data_ptr() for t in B]), arr(*[t.data_ptr() for t in C])
        sz = (ctypes.c_int * 24)(*[v for d in dims for v in d])

        def gg():
            runtime.call("lego_hip_grouped_gemm_f16", pa, pb, pc, sz, 8, stream)
        gg()
        rel = max(((c.float() - a.float() @ b.float()).norm() / (a.float() @ b.float()).norm()).item()
                  for a, b, c in zip(A, B, C))
        fl5 = sum(2 * m * n * k for m, n, k in dims)
        ms = timed(gg, steps=max(5, K // 5), warmup=max(2, W // 5))
        kernels["c5_grouped_gemm_f16"] = dict(ms=ms, tflops=fl5 / ms / 1e9, frac_mfma=fl5 / ms / 1e9 / MFMA_F16_PEAK_TFLOPS,
                                              **({"achievable_tflops": kernels["mfma_ceiling_f16"]["tflops"],
                                                  "frac_of_achievable": fl5 / ms / 1e9 / kernels["mfma_ceiling_f16"]["tflops"]}
                                                 if "mfma_ceiling_f16" in kernels else {}),
                                              flop=fl5, problems=dims, rel_err_vs_fp32=rel)
        plan5 = (ctypes.c_int * 3)()
        runtime.call("lego_hip_grouped_gemm_f16_plan", sz, 8, plan5)
        kernels["c5_grouped_gemm_f16"]["launch"] = dict(tile=plan5[0], tiles=plan5[1], tiles_split_in_halves=plan5[2])
        if ns.sustain > 0:
            # The grouped launch back to back for --sustain seconds, then one GEMM of four exactly full rounds of the same
            # 16-k-tile tiles (8192 x 8192 x 1024), with wall-clock times for power and clock samples taken by another process.
            a1k = (torch.randn(8192, 1024, generator=g5) / 32).half().to(dev)
            b1k = (torch.randn(1024, 8192, generator=g5) / 32).half().to(dev)
            c1k = torch.empty(8192, 8192, dtype=torch.half, device=dev)
            table = []
            for label, flop, fn in (("grouped GEMM, config 5", fl5, gg),
                                    ("gemm 8192 x 8192 x 1024 (1024 tiles of 16 k-tiles: four full rounds)", 2.0 * 8192 * 8192 * 1024,
                                     lambda: runtime.call("lego_hip_gemm_f16", p(a1k), p(b1k), p(c1k), 8192, 8192, 1024, stream))):
                per = []
                t_begin = time.time()
                t_end = time.perf_counter() + ns.sustain
                while time.perf_counter() < t_end:
                    per.append(timed(fn, steps=200, warmup=1, settle_ms=0.0))
                steady = per[len(per) // 3:]
                table.append(dict(variant=label, tflops=flop / (sum(steady) / len(steady)) / 1e9, wall_clock_begin=t_begin,
                                  wall_clock_end=time.time()))
                print(f"{t_begin:.2f} .. {time.time():.2f}  {label}: {table[-1]['tflops']:.1f} TFLOP/s", file=sys.stderr, flush=True)
                time.sleep(1.0)
            kernels["c5_sustained"] = table
            del a1k, b1k, c1k
        if not ns.skip_cpu:
            from oracle import kernels as ok5
            Ac, Bc = [t.cpu() for t in A], [t.cpu() for t in B]
            kernels["c5_grouped_gemm_f16"]["cpu_baseline"] = cpu_timed(
                lambda: ok5.grouped_gemm(Ac, Bc), fl5 / 1e3, "TFLOP/s",
                "all 8 problems: (A.float() @ B.float()).half() each")
            del Ac, Bc
        del A, B, C

    # ---- where the time of a GEMM tile goes: the measurement build of the fp16 kernels (same tiles and schedules) ------
    if "timeline" in only:
        import numpy as np
        g5 = gen(5)
        idx = torch.randint(0, 3, (8, 3), generator=g5)
        dims = [[(1024, 2048, 4096)[int(v)] for v in row] for row in idx]
        A = [(torch.randn(m, k, generator=g5) / math.sqrt(k)).half().to(dev) for m, n, k in dims]
        B = [(torch.randn(k, n, generator=g5) / math.sqrt(k)).half().to(dev) for m, n, k in dims]
        C = [torch.empty(m, n, dtype=torch.half, device=dev) for m, n, k in dims]
        arr = ctypes.c_void_p * 8
        pa, pb, pc = arr(*[t.data_ptr() for t in A]), arr(*[t.data_ptr() for t in B]), arr(*[t.data_ptr() for t in C])
        sz = (ctypes.c_int * 24)(*[v for d in dims for v in d])
        plan5 = (ctypes.c_int * 3)()
        runtime.call("lego_hip_grouped_gemm_f16_plan", sz, 8, plan5)
        at = (torch.randn(8192, 8192, generator=g5) / 90.5).half().to(dev)
        bt = (torch.randn(8192, 8192, generator=g5) / 90.5).half().to(dev)
        ct = torch.empty(8192, 8192, dtype=torch.half, device=dev)

        def plain(k):
            return lambda: runtime.call("lego_hip_gemm_f16_variant", p(at), p(bt), p(ct), 8192, 8192, k, 3, stream)
        runtime.call("lego_hip_grouped_gemm_f16_stamps", pa, pb, pc, sz, 8, stream)
        torch.cuda.synchronize()
        assert max(((c.float() - a.float() @ b.float()).norm() / (a.float() @ b.float()).norm()).item()
                   for a, b, c in zip(A, B, C)) <= 1e-2
        names = ("entry -> first k-tile in LDS", "-> first fragments read", "main loop and the k-tile before the last",
                 "slots of the last k-tile (results leave under them)", "tail: last staging and stores issued",
                 "last stores leave")
        table = []
        for label, wgs, flop, fn in (
                ("grouped GEMM, config 5", plan5[1] + plan5[2], sum(2.0 * m * n * k for m, n, k in dims),
                 lambda: runtime.call("lego_hip_grouped_gemm_f16_stamps", pa, pb, pc, sz, 8, stream)),
                ("gemm 8192 x 8192 x 1024", 1024, 2.0 * 8192 * 8192 * 1024, plain(1024)),
                ("gemm 8192 x 8192 x 8192", 1024, 2.0 * 8192 ** 3, plain(8192))):
            ms_t = timed(fn, steps=20, warmup=3)          # the stamps of the last launch of a steady run stay
            rows = np.zeros(8 * wgs, dtype=np.uint64)
            runtime.call("lego_hip_gemm_stamps_read", rows.ctypes.data_as(ctypes.c_void_p), wgs)
            st = rows.reshape(wgs, 8)
            tus = (st[:, :7].astype(np.int64) - int(st[:, 0].min())) * 0.01          # 100 MHz counter -> microseconds
            where = ((st[:, 7] >> np.uint64(8)) & np.uint64(0xff)) | ((st[:, 7] >> np.uint64(16)) << np.uint64(8))
            span = float(tus[:, 6].max())
            phases = {nm: dict(mean=float(d.mean()), p10=float(np.percentile(d, 10)), p90=float(np.percentile(d, 90)))
                      for nm, d in zip(names, (tus[:, i + 1] - tus[:, i] for i in range(6)))}
            busy, gaps, first, last_idle = [], [], [], []
            for cu in np.unique(where):
                own = tus[where == cu]
                own = own[np.argsort(own[:, 0])]
                busy.append(float((own[:, 6] - own[:, 0]).sum()))
                first.append(float(own[0, 0]))
                last_idle.append(span - float(own[-1, 6]))
                gaps += [float(own[i + 1, 0] - own[i, 6]) for i in range(len(own) - 1)]
            entry = dict(workload=label, workgroups=wgs, ms=ms_t, tflops=flop / ms_t / 1e9, span_us=span,
                         workgroup_us_mean=float((tus[:, 6] - tus[:, 0]).mean()), phases_us=phases,
                         cus_seen=int(len(busy)), cu_busy_fraction=float(np.mean(busy)) / span,
                         cu_first_start_us_mean=float(np.mean(first)), cu_idle_after_last_us_mean=float(np.mean(last_idle)),
                         gap_between_workgroups_on_a_cu_us=dict(mean=float(np.mean(gaps)) if gaps else 0.0,
                                                                p90=float(np.percentile(gaps, 90)) if gaps else 0.0,
                                                                per_cu_total_mean=float(np.sum(gaps)) / len(busy)),
                         start_us_deciles=[float(v) for v in np.percentile(tus[:, 0], range(0, 101, 10))],
                         end_us_deciles=[float(v) for v in np.percentile(tus[:, 6], range(0, 101, 10))])
            table.append(entry)
        kernels["gemm_tile_timeline"] = dict(
            note="measurement build (lane 0 of each workgroup stores the 100 MHz real-time counter at seven points and "
                 "the CU it ran on); last launch of 20 back-to-back ones after the settle phase; cu_busy_fraction = "
                 "time between a workgroup's entry and its last store leaving, summed per CU, over the kernel's span",
            workloads=table)
        del A, B, C, at, bt, ct

    # ---- next rows: the reference's lego_c benchmark programs (stencils on bricks, Needleman-Wunsch, LUD) ----
    if want("apps"):
        n = 384
        # three fields and three results in turn: one pair of 216 MiB each would partly live in the 256 MB last-level cache
        xs = [(torch.rand(n, n, n, generator=gen(7)) * 2 - 1).to(dev) for _ in range(3)]
        ys = [torch.zeros_like(xs[0]) for _ in range(3)]
        cs = torch.rand(8, 8, 8, generator=gen(8)).to(dev)
        cl = torch.tensor([-6.0, 1.0], device=dev)
        which = [0]
        for name, entry, cc in (("f3d", "lego_hip_stencil_f3d_f32", cs), ("laplacian", "lego_hip_stencil_laplacian_f32", cl)):
            for bricks in (0, 1):
                def st(entry=entry, cc=cc, bricks=bricks):
                    which[0] = (which[0] + 1) % 3
                    runtime.call(entry, p(xs[which[0]]), p(ys[which[0]]), p(cc), n, 1, bricks, stream)
                ms = timed(st, steps=max(5, K // 5), warmup=max(2, W // 5))
                kernels[f"next_stencil_{name}_384_r1_{'bricks' if bricks else 'rowmajor'}"] = dict(
                    ms=ms, gbs=2 * n ** 3 * 4 / ms / 1e6, bytes=2 * n ** 3 * 4)
        del xs, ys
        nn = 8192
        refm = torch.randint(-4, 12, (nn + 1, nn + 1), generator=gen(9), dtype=torch.int32).to(dev)
        mat = torch.zeros((nn + 1, nn + 1), dtype=torch.int32, device=dev)
        border = -torch.arange(nn + 1, dtype=torch.int32, device=dev) * 10
        mat[:, 0] = border
        mat[0, :] = border

        def nwf():
            runtime.call("lego_hip_nw_i32", p(refm), p(mat), nn, 10, stream)
        ms = timed(nwf, steps=3, warmup=1)
        kernels["next_needleman_wunsch_8192"] = dict(ms=ms, gcells_per_s=nn * nn / ms / 1e6,
                                                     note="255 launches, one per anti-diagonal of 64x64 tiles")
        del refm, mat
        # the three sizes the reference publishes (29.7, 111.2 and 653.5 ms for its LEGO kernel on an A100,
        # benchmarks/cuda/lud/PerformanceSummary.txt:24-36)
        for nl, ref_ms, seed in ((4096, 29.746, 10), (8192, 111.202, 12), (16384, 653.476, 11)):
            a0 = torch.rand(nl, nl, generator=gen(seed)).to(dev)
            a0.diagonal().add_(float(nl))
            wk = torch.empty_like(a0)

            def luf():
                wk.copy_(a0)
                runtime.call("lego_hip_lud_f32", p(wk), nl, stream)
            reps = 3 if nl < 16384 else 2
            ms = timed(luf, steps=reps, warmup=1) - timed(lambda: wk.copy_(a0), steps=reps, warmup=1)
            kernels[f"next_lud_f32_{nl}"] = dict(ms=ms, tflops=(2 / 3) * nl ** 3 / ms / 1e9, reference_ms_a100=ref_ms,
                                                 note="time of a matrix copy subtracted; block steps of 64 in pairs")
            del a0, wk

    # ---- CPU baseline: the reference's CPU path on a bounded panel of the headline matrix -----------------
    cpu = None
    if not ns.skip_cpu:
        from lego_amd.kernels.transpose import python_offsets
        from oracle import cpu_path
        rows = 8192
        c2()                      # y2 was last written by the copy ceiling measurement
        torch.cuda.synchronize()
        panel = x2[:rows].cpu()
        src_text, dst_text = python_offsets(64, 64)
        t0 = time.perf_counter()
        got = cpu_path.transpose_printed(panel, src_text, dst_text, 64, 64, total_rows=n2)
        dt = time.perf_counter() - t0
        assert torch.equal(got, y2[:, :rows].cpu()), "GPU result differs from the CPU path"
        cpu = dict(value=2 * panel.numel() * 2 / dt / 1e9, unit="GB/s", cores=cpu_threads, kind="port",
                   sample=f"rows 0..{rows - 1} of the 16384x16384 fp16 matrix ({rows}/16384 of the workload): the "
                          f"offsets of both LEGO layouts as the Python/Triton printer emits them, evaluated with "
                          f"torch.arange for tl.arange, then one gather/scatter; {dt:.2f} s, one run, "
                          f"{cpu_threads} threads of {os.cpu_count()} visible cores")

    line = {
        "metric": "HBM GB/s (transpose/softmax/LN) + fp16 GEMM TFLOPS, % of roofline, 1 GPU",
        "value": gbs2, "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": ms2,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "2-D fp16 transpose 16384x16384, LEGO TileBy([256,256],[64,64]) row-major -> "
                               "column-major, 1x4 tiles per workgroup, workgroups in windows of 128x8 macro tiles, XOR-swizzled LDS "
                               "staging, inputs N(0,1) seed 1"},
        "roofline": {"bound": "hbm", "achieved": gbs2, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": gbs2 / HBM_PEAK_GBS, "traffic": headline_traffic_bytes(),
                     "achievable": achievable, "frac_of_achievable": gbs2 / achievable,
                     "achievable_note": "1 / (0.5 / read-only + 0.5 / write-only) of this run's one-directional "
                                        "streams (kernels.hbm_ceiling)",
                     "kernel": HEADLINE_KERNEL, "algorithmic_bytes_per_launch": bytes2},
        "cpu_baseline": cpu,
        "kernels": kernels,
        "peaks": {"hbm_gbs": HBM_PEAK_GBS, "mfma_f16_tflops": MFMA_F16_PEAK_TFLOPS,
                  "mfma_fp8_tflops": MFMA_FP8_PEAK_TFLOPS},
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
