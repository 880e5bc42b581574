"""Generates the HIP sources from the LEGO layouts and builds liblego_hip.so for gfx950.

    python -m lego_amd.build            # generate + compile
    python -m lego_amd.build --emit     # generate only

Generated text goes to lego_amd/csrc/generated/, the library to lego_amd/lib/.  hipcc
cross-compiles without a GPU.
"""
from __future__ import annotations

import argparse
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

from .kernels import gemm, layernorm_bwd, lud, nw, rowwise, stencil, transpose
from .kernels.common import BANNER, CSRC, GENERATED
from .lego_hip import HIPCC_FLAGS, hipcc_path

ROOT = Path(__file__).resolve().parents[1]
LIB_DIR = Path(__file__).resolve().parent / "lib"
LIB_PATH = LIB_DIR / "liblego_hip.so"
OBJ_DIR = LIB_DIR / "obj"

# the tilings the library is built with
# Per element type, in order of preference: the fastest tiling for shapes that its windows
# divide (then the same in smaller windows), a wide macro tile in skewed ("diag") order, a 64x64 one for shapes the wide tile
# does not divide, and the wide tile with edge tests for shapes in whole 16-byte vectors.
# The tilings with edge tests run their tiles in strips eight tile columns wide and load with plain (cached) loads:
# when a row is not a whole number of 128-byte lines the row segments of neighbouring tiles share lines, and a
# tile's neighbours on all four sides then run on the same XCD at about the same time (measured in one process
# against column order with non-temporal loads: fp16 9999 x 10001 3.52 -> 4.10 TB/s, 16386 x 8191 2.95 -> 3.92,
# 10000^2 3.78 -> 4.28; fp32 9999 x 10001 3.79 -> 4.48, 8200 x 8192 3.94 -> 4.89; fp16 10000 x 10240 4.72 -> 4.51).
# Their macro tiles are 128 bytes of a source row by 512 bytes of a destination row (fp16 256 x 64, fp32 128 x 32): a read
# segment is one line when it is not cut, a write segment four (five lines touched for four written when it is cut, where
# the 256-byte segments of the square tiles built before touched three for two).  Against those square tiles, TB/s with
# rotating results, fp16 any shape 9999 x 10001 4.09 -> 4.23, 8191 x 16386 4.32 -> 4.80, 12345 x 6789 4.14 -> 4.30, 24600 x 24576
# 4.78 -> 4.95, 16386 x 8191 3.91 -> 3.89; whole vectors 8200 x 8192 4.16 -> 4.47, 10000^2 4.27 -> 4.38, 24600 x 24576 4.86 -> 5.02,
# 8192 x 8200 4.5 -> 4.44; fp32 any shape 9999 x 10001 4.48 -> 4.60, 16386 x 8191 4.66 -> 4.86, 4099 x 4101 4.18 -> 4.47; whole
# vectors 10000^2 4.80 -> 5.04, 10000 x 10240 4.91 -> 5.21, 6152^2 4.32 -> 4.65, 8200 x 8192 4.90 -> 4.76, and 24600 x 24576 4.81 ->
# 4.39, which is why the fp32 tiling with edge tests stops at 384 Mi elements.  Taller or wider tiles lose (fp16 512 x 64:
# 3.75 at 9999 x 10001; 256 x 128 4.01; 128 x 256 3.68).
# What remains is the count of 128-byte lines an access touches: the same kernel on fp16 10048^2 (rows of whole lines)
# moves 5.3 TB/s, on 10016^2 (whole 64-byte halves) 4.5, on 10000^2 3.8 (a 256-byte row segment touches three lines).
# fp32 4096^2 (2048 workgroups of 32 KiB, five resident per CU: 1.6 rounds) against tilings whose workgroups make whole
# rounds: 64x64 tiles in the same windows (4096 workgroups, eight per CU: two rounds) 26.2 us, 32x128 tiles 25.6 us,
# 64x64 tiles in 32x16 windows 26.8 us, the 64x128 tiles built 24.6 us; a plain copy of the same 2 x 64 MiB takes 22.4 us.
TRANSPOSE = {
    "f32": [dict(dtype="f32", tile=(32, 32), group=(2, 4), order=("window", 64, 8), max_bytes=1536 << 20),
            dict(dtype="f32", tile=(32, 32), group=(2, 4), order=("window", 32, 8), max_bytes=1536 << 20),
            dict(dtype="f32", tile=(32, 32), group=(1, 8), order="diag", min_elements=2 << 20),   # smaller: 64x64 tiles
            dict(dtype="f32", tile=(32, 32), group=(2, 2), order="diag"),
            dict(dtype="f32", tile=(32, 32), group=(4, 1), order=("strip", 8), edge=True, xcd=True, max_elements=384 << 20),
            dict(dtype="f32", tile=(32, 32), group=(2, 4), order=("strip", 8), edge=True, xcd=True),
            dict(dtype="f32", tile=(32, 32), group=(4, 1), order=("strip", 8), edge=True, ragged=True, xcd=True, min_elements=3 << 20),
            dict(dtype="f32", tile=(32, 32), group=(2, 2), order="col", edge=True, ragged=True, xcd=True),
            dict(dtype="f32", tile=(32, 32), group=(4, 2), order=("strip", 8), edge=True, ragged=True, xcd=True, tuning_only=True)],
    "f16": [dict(dtype="f16", tile=(64, 64), group=(1, 4), order=("window", 128, 8)),
            dict(dtype="f16", tile=(64, 64), group=(1, 4), order=("window", 64, 8)),
            dict(dtype="f16", tile=(64, 64), group=(1, 4), order=("window", 32, 8)),
            dict(dtype="f16", tile=(64, 64), group=(1, 4), order="diag", min_elements=2 << 20),   # smaller: 64x64 tiles
            dict(dtype="f16", tile=(64, 64), group=(1, 1), order="diag"),
            dict(dtype="f16", tile=(64, 64), group=(4, 1), order=("strip", 8), edge=True, xcd=True),
            dict(dtype="f16", tile=(64, 64), group=(4, 1), order=("strip", 8), edge=True, ragged=True, xcd=True, min_elements=40 << 20),
            dict(dtype="f16", tile=(64, 64), group=(1, 1), order="col", edge=True, ragged=True, xcd=True),
            dict(dtype="f16", tile=(64, 64), group=(2, 2), order=("strip", 8), edge=True, xcd=True, tuning_only=True),
            dict(dtype="f16", tile=(64, 64), group=(2, 2), order=("strip", 8), edge=True, ragged=True, xcd=True, tuning_only=True)],
}
# (element type, vectorised, waves per row): 16-byte accesses need N % (16/size) == 0; the
# element-per-access kernels ("s") take any N
ROWWISE = [("f16", True, 1), ("f16", True, 2), ("f16", True, 4), ("f16", True, 8), ("f32", True, 1), ("f32", True, 4), ("f32", True, 8),
           ("f16", False, 1), ("f32", False, 1), ("f16", False, 4), ("f32", False, 4), ("f16", False, 8), ("bf16", False, 8), ("f32", False, 8),
           ("f16", True, 16), ("f32", True, 16), ("f16", False, 16), ("f32", False, 16),
           ("bf16", True, 1), ("bf16", True, 4), ("bf16", True, 8), ("bf16", True, 16), ("bf16", False, 1), ("bf16", False, 4),
           ("bf16", False, 16)]
# (element type, lanes per row): teams of a part of a wave for rows of at most that many 16-byte vectors
ROWWISE_SHORT = [(d, lanes, vec) for d in ("f16", "bf16", "f32") for lanes in (16, 32) for vec in (True, False)]
# LayerNorm launches of many rows: this many workgroups that stage gamma and beta in LDS and walk the rows
ROWWISE_STREAM_WGS = {("f16", True, 4): 1024, ("bf16", True, 4): 1024, ("f16", True, 8): 512, ("bf16", True, 8): 512, ("f32", True, 8): 512, ("f16", True, 16): 256, ("bf16", True, 16): 256,
                      # rows of any length: a team's rows must start alike, so the count times the teams per workgroup is a multiple of 8
                      ("f16", False, 1): 1024, ("f16", False, 4): 1024, ("f16", False, 16): 256,
                      ("f16", False, 8): 512, ("bf16", False, 8): 512, ("f32", False, 8): 512,
                      ("bf16", False, 1): 1024, ("bf16", False, 4): 1024, ("bf16", False, 16): 256,
                      ("f32", False, 1): 1024, ("f32", False, 4): 1024, ("f32", False, 16): 256}
# ... of teams of four waves only with four vectors per lane (16-bit rows of 4097-8192 elements); measured with and without
# the walking launch, fp16 TB/s: 8192 x 5120 5.22 / 5.47, 8192 x 6144 5.48 / 5.57, 2048 x 8192 5.01 / 5.39, but
# 8192 x 3072 5.13 / 4.96, 16384 x 4096 5.89 / 5.81, 65536 x 2560 6.07 / 5.47
ROWWISE_STREAM_MIN_VECTORS = {("f16", True, 4): 4, ("bf16", True, 4): 4}
ROWWISE_DEFAULT_WAVES = 4
ROWWISE_WIDE_TEAM_ABOVE_N, ROWWISE_WIDE_TEAM_FROM_M = 6144, 4096
ROWWISE_TWO_WAVES_ABOVE_N, ROWWISE_TWO_WAVES_FROM_M = 1536, 16384
ROWWISE_MAX_N = rowwise.MAX_N
GEMM = dict(bm=256, bn=256, bk=64, waves=(2, 2), max_group_m=8)
GEMM_SMALL_TILE = 128
GEMM_WAVES_TWO_PER_SIMD = (2, 4)
GEMM_SMALL_DTYPES = ("f16", "bf16", "bf16h")     # a 128-byte row of 8-bit elements is too short for their [k][n] rotation
GEMM_SMALL_NT_ONLY = ("e4m3", "e5m2")             # ... so 8-bit operands get the small tile where both are k-major (A as given, B transposed)
GEMM_DTYPES = ("f16", "bf16", "bf16h", "e4m3", "e5m2")     # bf16h: bfloat16 operands, fp16 result
GEMM_SPARSE_ROUND_DTYPES = ("f16", "bf16", "bf16h")   # 16-bit operands: also built on the 32x32x16 MFMA (see collect())
# The MFMA of the 256 x 256 tiles: v_mfma_f32_16x16x32 for 16-bit operands (the same matrix-core cycles per flop as
# 32x32x16, but the socket's power limit leaves it a higher clock: a stream of nothing but MFMAs runs 1.95 against
# 1.68 PFLOP/s, and the GEMM gains 3 to 7 %: 8192^3 1.29 -> 1.36, 4096^3 1.22 -> 1.31, 8192 x 8192 x 1024 1.12 -> 1.17
# PFLOP/s); 32x32x64 for 8-bit operands.  The 128 x 128 tiles keep 32 x 32 blocks: their sums along K are laid out for them.
GEMM_MFMA_BLOCK = {"f16": 16, "bf16": 16, "bf16h": 16, "e4m3": 32, "e5m2": 32}
GEMM_BK = {"f16": 64, "bf16": 64, "bf16h": 64, "e4m3": 128, "e5m2": 128}   # 128 bytes of k per operand row in every case


def collect():
    """Run every generator: ``(units, text of launchers.h)``, nothing written."""
    units = []
    tmeta = {}
    for dtype, configs in TRANSPOSE.items():
        for cfg in configs:
            cfg = dict(cfg)
            max_bytes = cfg.pop("max_bytes", None)   # only for matrices that fit the last-level cache
            tuning_only = cfg.pop("tuning_only", False)      # built for comparison, never picked
            min_elements = cfg.pop("min_elements", None)
            max_elements = cfg.pop("max_elements", None)
            unit, meta = transpose.emit(**cfg)
            meta["max_bytes"] = max_bytes
            meta["tuning_only"] = tuning_only
            if min_elements:
                meta["min_elements"] = min_elements
            if cfg.get("edge"):
                vec = 4 if dtype == "f32" else 8
                meta["row_multiple"] = meta["col_multiple"] = vec
                # smaller matrices have too few of these macro tiles: the 64x64 ones of the any-shape kernels are ahead up
                # to about 32 Mi elements (fp16 2056^2 3.2 against 2.3 TB/s, 4104^2 4.2 / 3.8; 6152^2 3.7 / 4.0)
                meta["min_elements"] = 32 << 20
            meta["max_elements"] = max_elements
            meta["any_element"] = bool(cfg.get("ragged"))
            if cfg.get("ragged"):     # any shape with at least one whole vector per row of both matrices
                meta["row_multiple"] = meta["col_multiple"] = 1
                meta["min_side"] = vec
                # 64x64 tiles for the smaller matrices, which have too few of the larger macro tiles: fp16 up to 40 Mi
                # elements (64x64 / 256x64, TB/s: 4099 x 4101 3.69 / 3.45, 6001 x 6003 3.94 / 3.81, 7001 x 7003 3.94 / 4.02),
                # fp32 up to 3 Mi (64x64 / 128x32: 1449 x 1451 2.49 / 2.40, 2049 x 2051 3.29 / 3.41, 4099 x 4101 4.15 / 4.47);
                # matrices of under 16 Ki elements go one element per access
                meta["min_elements"] = (min_elements or (64 << 20)) if (meta["SR"], meta["SC"]) != (64, 64) else (16 << 10)
            unit.filename = meta["kernel"].replace("lego_", "", 1) + ".hip"
            units.append(unit)
            tmeta.setdefault(dtype, []).append(meta)
    units.append(transpose.emit_any())
    units += [rowwise.emit(w, dtype, vec, stream_wgs=ROWWISE_STREAM_WGS.get((dtype, vec, w), 0),
                           stream_min_vectors=ROWWISE_STREAM_MIN_VECTORS.get((dtype, vec, w), 1)) for dtype, vec, w in ROWWISE]
    units += [rowwise.emit(1, dtype, vec, team_lanes=lanes) for dtype, lanes, vec in ROWWISE_SHORT]
    units.append(rowwise.emit_long())
    for dtype in GEMM_DTYPES:
        for ta in (False, True):
            for tb in (False, True):
                g, m_ = gemm.emit(**dict(GEMM, bk=GEMM_BK[dtype]), trans_a=ta, trans_b=tb, dtype=dtype,
                                  block=GEMM_MFMA_BLOCK[dtype], with_grouped=dtype == "f16" and not (ta or tb),
                                  with_split=dtype == "f16" and not (ta or tb))
                units.append(g)
                if dtype == "f16":
                    mg = m_
                # the same kernel on 128x128 tiles, two workgroups per CU: for problems with too few
                # 256x256 tiles to fill the chip
                if dtype in GEMM_SMALL_DTYPES:
                    gs, _ = gemm.emit(**dict(GEMM, bk=GEMM_BK[dtype], bm=GEMM_SMALL_TILE, bn=GEMM_SMALL_TILE),
                                      trans_a=ta, trans_b=tb, dtype=dtype,
                                      with_grouped=dtype == "f16" and not (ta or tb), with_splitk=True)
                    units.append(gs)
                elif dtype in GEMM_SMALL_NT_ONLY and tb and not ta:
                    gs, _ = gemm.emit(**dict(GEMM, bk=GEMM_BK[dtype], bm=GEMM_SMALL_TILE, bn=GEMM_SMALL_TILE),
                                      trans_a=ta, trans_b=tb, dtype=dtype, with_grouped=False)
                    units.append(gs)
    # The 256 x 256 tile on 32 x 32 accumulator blocks (v_mfma_f32_32x32x16), four waves of 128 x 128: behind at the
    # socket's power limit (8192^3: 1.29 against 1.36 PFLOP/s) and ahead away from it, so launches of one round that
    # leaves a third of the CUs idle take it (kSparseRoundBelow in lego_hip_abi.hip); the fp16 build for operands as
    # given is also behind the tuning entry point, beside a second alternative kept for the comparison: eight waves of
    # 128 x 64 per workgroup, two per SIMD with 128 accumulator registers each (a second wave to issue from while one
    # waits; 8192^3 1.28).
    g32 = [gemm.emit(**dict(GEMM, bk=GEMM_BK[dtype]), trans_a=ta, trans_b=tb, dtype=dtype, with_grouped=False, suffix="_m32")[0]
           for dtype in GEMM_SPARSE_ROUND_DTYPES for ta in (False, True) for tb in (False, True)]
    g8, _ = gemm.emit(**dict(GEMM, bk=GEMM_BK["f16"], waves=GEMM_WAVES_TWO_PER_SIMD), dtype="f16", with_grouped=False)
    # A measurement build of the fp16 kernels as launched (same tiles, same schedules): lane 0 of every workgroup
    # records the real-time counter at seven points of its tile and the CU it ran on, for the per-phase tables of
    # bench.py --only timeline.
    gst, _ = gemm.emit(**dict(GEMM, bk=GEMM_BK["f16"]), dtype="f16", block=GEMM_MFMA_BLOCK["f16"], with_grouped=True,
                       with_split=True, suffix="_stamps", stamps=True)
    units += g32 + [g8, gst]
    units.append(gemm.emit_any())
    lbs, mlb = layernorm_bwd.emit()
    units += lbs
    nwu, mnw = nw.emit()
    units.append(nwu)
    stu, mst = stencil.emit()
    units.append(stu)
    luu, mlu = lud.emit()
    units.append(luu)

    h = [f"// {BANNER}", "#pragma once", "#include <hip/hip_runtime.h>", "",
         "hipError_t lego_transpose_any_launch(const void*, void*, int, int, int, hipStream_t);"]
    for dtype, metas in tmeta.items():
        for m in metas:
            h.append(f"hipError_t {m['kernel']}_launch(const void*, void*, int, int, hipStream_t);")
        h += [f"// picks the first tiling that divides the shape; any other shape takes the tiling with vectors at any element and edge tests, a tiny matrix the one-element-per-access kernel",
              f"inline hipError_t lego_transpose_{dtype}_dispatch(const void* in, void* out, int rows, int cols, "
              "hipStream_t stream) {"]
        for m in metas:
            if m["tuning_only"]:
                continue
            fits = "" if m["max_bytes"] is None else \
                f" && 2ull * rows * cols * {4 if dtype == 'f32' else 2} <= {m['max_bytes']}ull"
            if m.get("min_side"):
                fits += f" && rows >= {m['min_side']} && cols >= {m['min_side']}"
            if m.get("min_elements"):
                fits += f" && 1ull * rows * cols >= {m['min_elements']}ull"
            if m.get("max_elements"):
                fits += f" && 1ull * rows * cols <= {m['max_elements']}ull"
            h.append(f"  if (rows % {m['row_multiple']} == 0 && cols % {m['col_multiple']} == 0{fits}) "
                     f"return {m['kernel']}_launch(in, out, rows, cols, stream);")
        h += [f"  return lego_transpose_any_launch(in, out, rows, cols, {4 if dtype == 'f32' else 2}, stream);", "}",
              "// matrices whose base is only element aligned (a sliced view): the tilings whose vectors sit at any element",
              f"inline hipError_t lego_transpose_{dtype}_dispatch_any_base(const void* in, void* out, int rows, int cols, "
              "hipStream_t stream) {"]
        for m in metas:
            if m["any_element"] and not m["tuning_only"]:
                h.append(f"  if (rows >= {m['min_side']} && cols >= {m['min_side']} && 1ull * rows * cols >= {m['min_elements']}ull) "
                         f"return {m['kernel']}_launch(in, out, rows, cols, stream);")
        h += [f"  return lego_transpose_any_launch(in, out, rows, cols, {4 if dtype == 'f32' else 2}, stream);", "}",
              "// tiling number `tiling` of the list above, for a shape it takes (16-byte aligned bases); the caller compares tilings with it",
              f"inline hipError_t lego_transpose_{dtype}_tiling(int tiling, const void* in, void* out, int rows, int cols, "
              "hipStream_t stream) {"]
        for n_, m in enumerate(metas):
            fits = f" && rows >= {m['min_side']} && cols >= {m['min_side']}" if m.get("min_side") else ""
            h.append(f"  if (tiling == {n_} && rows % {m['row_multiple']} == 0 && cols % {m['col_multiple']} == 0{fits}) "
                     f"return {m['kernel']}_launch(in, out, rows, cols, stream);      // {m['SR']} x {m['SC']}")
        h += ["  return hipErrorInvalidValue;", "}", ""]
    for dtype, vec, w in ROWWISE:
        tag = dtype if vec else dtype + "s"
        h += [f"hipError_t lego_softmax_{tag}_w{w}_launch(const void*, void*, int, int, hipStream_t);",
              f"hipError_t lego_layernorm_fwd_{tag}_w{w}_launch(const void*, void*, const void*, const void*, "
              "float*, float*, int, int, float, hipStream_t);"]
    for dtype, lanes, vec in ROWWISE_SHORT:
        tag = dtype if vec else dtype + "s"
        h += [f"hipError_t lego_softmax_{tag}_l{lanes}_launch(const void*, void*, int, int, hipStream_t);",
              f"hipError_t lego_layernorm_fwd_{tag}_l{lanes}_launch(const void*, void*, const void*, const void*, "
              "float*, float*, int, int, float, hipStream_t);"]
    h += [f"hipError_t lego_softmax_long_{d}_launch(const void*, void*, int, int, hipStream_t);" for d in rowwise.ELEMENTS]
    h += [
          f"#define LEGO_ROWWISE_MAX_N {ROWWISE_MAX_N}",
          f"#define LEGO_ROWWISE_MAX_N_SMALL_TEAMS {rowwise.MAX_N_SMALL_TEAMS}",
          "// waves per row: one wave keeps short rows free of barriers, four waves keep the",
          "// register footprint of long rows small enough for full occupancy, sixteen (a whole",
          "// workgroup of 1024 lanes) hold the rows that four cannot",
          f"inline int lego_rowwise_default_wpr(int n) {{ return n <= 2048 ? 1 : n <= {rowwise.MAX_N_SMALL_TEAMS} ? "
          f"{ROWWISE_DEFAULT_WAVES} : {rowwise.LONG_ROW_WAVES}; }}",
          "// 16-bit rows of whole vectors: eight waves (a workgroup of 512 lanes, two to four vectors per lane) for long",
          "// rows of tall matrices, where they measure 3-5 % above four waves; fewer rows leave too few workgroups",
          "// ... and two waves (two rows per workgroup) for 2049-4096 rows of 2049-4096 elements: one round of workgroups on",
          "// the 256 CUs instead of two (4096 x 4096: softmax 4.9 -> 5.4 TB/s, LayerNorm 4.4 -> 5.0; no gain from 8192 rows on)",
          "// ... and for rows of 1537-2048 elements, which one wave holds as four vectors per lane, of matrices of 16384 rows",
          "// and more (2-5 % above one wave there, 1-11 % below it at 8192 rows)",
          f"inline int lego_rowwise_f16_wpr(int m, int n) {{ return n > {ROWWISE_WIDE_TEAM_ABOVE_N} && n <= "
          f"{rowwise.MAX_N_SMALL_TEAMS} && m >= {ROWWISE_WIDE_TEAM_FROM_M} ? 8 : n > 2048 && n <= 4096 && m > 2048 && m <= 4096 ? 2 "
          f": n > {ROWWISE_TWO_WAVES_ABOVE_N} && n <= 2048 && m >= {ROWWISE_TWO_WAVES_FROM_M} ? 2 : lego_rowwise_default_wpr(n); }}", ""]
    h += ["unsigned lego_layernorm_bwd_groups(int M, int N);", "unsigned lego_layernorm_bwd_f32_groups(int M, int N);",
          "unsigned lego_layernorm_bwd_bf16_groups(int M, int N);",
          "hipError_t lego_layernorm_bwd_f32_launch(const void*, const void*, const void*, const float*, const float*, "
          "void*, void*, void*, float*, int, int, int, hipStream_t);",
          "hipError_t lego_layernorm_bwd_bf16_launch(const void*, const void*, const void*, const float*, const float*, "
          "void*, void*, void*, float*, int, int, int, hipStream_t);",
          "hipError_t lego_layernorm_bwd_f16_launch(const void*, const void*, const void*, const float*, const float*, "
          "void*, void*, void*, float*, int, int, int, hipStream_t);",
          f"#define LEGO_LAYERNORM_BWD_MAX_N {mlb['MAX_N']}", ""]
    h += [f"hipError_t lego_gemm_{d}_{v}{t}_launch(const void*, const void*, void*, int, int, int, int, hipStream_t);"
          for d in GEMM_DTYPES for v in ("nn", "nt", "tn", "tt")
          for t in ("", f"_t{GEMM_SMALL_TILE}x{GEMM_SMALL_TILE}") if not t or d in GEMM_SMALL_DTYPES or (d in GEMM_SMALL_NT_ONLY and v == "nt")]
    h += [f"hipError_t lego_gemm_{d}_{v}_t{GEMM_SMALL_TILE}x{GEMM_SMALL_TILE}_splitk_launch(const void*, const void*, void*, int, int, int, int, "
          "int, float*, hipStream_t);" for d in GEMM_SMALL_DTYPES for v in ("nn", "nt", "tn", "tt")]
    h += [
          "hipError_t lego_grouped_gemm_f16_launch(const void* const*, const void* const*, void* const*, "
          "const int*, int, hipStream_t);",
          f"hipError_t lego_grouped_gemm_f16_t{GEMM_SMALL_TILE}x{GEMM_SMALL_TILE}_launch(const void* const*, "
          "const void* const*, void* const*, const int*, int, hipStream_t);",
          "hipError_t lego_gemm_f16_nn_w2x4_launch(const void*, const void*, void*, int, int, int, int, hipStream_t);",
          *[f"hipError_t lego_gemm_{d}_{v}_m32_launch(const void*, const void*, void*, int, int, int, int, hipStream_t);"
            for d in GEMM_SPARSE_ROUND_DTYPES for v in ("nn", "nt", "tn", "tt")],
          "hipError_t lego_gemm_f16_nn_stamps_launch(const void*, const void*, void*, int, int, int, int, hipStream_t);",
          "hipError_t lego_grouped_gemm_f16_stamps_launch(const void* const*, const void* const*, void* const*, "
          "const int*, int, hipStream_t);",
          "hipError_t lego_grouped_gemm_f16_stamps_split_launch(const void* const*, const void* const*, void* const*, "
          "const int*, int, int, hipStream_t);",
          "hipError_t lego_gemm_stamps_read(unsigned long long*, int);",
          "hipError_t lego_gemm_any_launch(const void*, const void*, void*, int, int, int, int, int, int, int, hipStream_t);",
          "hipError_t lego_grouped_gemm_f16_split_launch(const void* const*, const void* const*, void* const*, "
          "const int*, int, int, hipStream_t);",
          f"#define LEGO_GEMM_BM {mg['BM']}", f"#define LEGO_GEMM_BN {mg['BN']}", f"#define LEGO_GEMM_BK {mg['BK']}",
          f"#define LEGO_GEMM_BK_8BIT {GEMM_BK['e5m2']}",
          f"#define LEGO_GROUPED_MAX_GROUPS {mg['MAX_GROUPS']}", ""]
    h += ["hipError_t lego_nw_i32_launch(const int*, int*, int, int, hipStream_t);",
          f"#define LEGO_NW_TILE {mnw['B']}", "",
          "hipError_t lego_stencil_f32_launch(const float*, float*, const float*, int, int, int, int, hipStream_t);",
          f"#define LEGO_STENCIL_BRICK {mst['B']}", f"#define LEGO_STENCIL_MAX_RADIUS {mst['MAX_RADIUS']}",
          f"#define LEGO_STENCIL_STAR_MAX_RADIUS {mst['STAR_MAX_RADIUS']}", "",
          "hipError_t lego_lud_f32_launch(float*, int, hipStream_t);", "hipError_t lego_lud_f32_plan(int, int*, int, int*);", f"#define LEGO_LUD_BLOCK {mlu['B']}", ""]
    return units, "\n".join(h)


def generate():
    """Write every generated source; returns the list of .hip paths to compile."""
    units, text = collect()
    GENERATED.mkdir(parents=True, exist_ok=True)
    header = GENERATED / "launchers.h"
    if not header.exists() or header.read_text() != text:
        header.write_text(text)
    paths = [u.write() for u in units]
    # sources of translation units that are no longer generated would still be found by a glob: remove them
    for stale in set(GENERATED.glob("*.hip")) - set(paths):
        stale.unlink()
    return paths


# Instructions that must lie between an MFMA written as inline assembly and the first other instruction that reads
# its result: the compiler inserts the wait states of MFMAs it knows (at most 19, for the sixteen-pass ones) but does
# not look into inline assembly.  The 16x16x32 MFMA takes four passes; the kernels built keep 23 and more.
ASM_MFMA_MIN_DISTANCE = 16


def asm_mfma_read_distance(assembly: str):
    """Smallest number of issue slots, per function of a gfx950 assembly listing, between an MFMA and the next
    instruction other than an MFMA that names one of the accumulation registers it writes (``a7`` or a range
    ``a[4:7]``), counted along the listing: ``{function: (distance, register, instruction)}``.  An instruction
    counts one slot, an MFMA in between four (it issues no sooner than the matrix core is free of the one before,
    four passes at least).  Functions in which no MFMA result is read back are left out."""
    import re
    out, name, last, count = {}, None, {}, 0
    for line in assembly.split("\n"):
        text = line.strip()
        m = re.match(r"^([A-Za-z_][\w$.]*):", line)
        if m and not text.startswith("."):
            name, last, count = m.group(1), {}, 0
            continue
        if not text or text[0] in ";." or text.endswith(":"):
            continue
        m = re.match(r"v_mfma\S+\s+a\[(\d+):(\d+)\]", text)
        count += 4 if m else 1
        if m:
            for r in range(int(m.group(1)), int(m.group(2)) + 1):
                last[r] = count
            continue
        regs = [int(r) for r in re.findall(r"\ba(\d+)\b", text)]
        for lo, hi in re.findall(r"\ba\[(\d+):(\d+)\]", text):
            regs += range(int(lo), int(hi) + 1)
        for r in regs:
            if r in last and text.split()[0] not in ("v_accvgpr_write_b32", "v_accvgpr_mov_b32"):
                found = (count - last[r], r, text.split()[0])
                if name not in out or found < out[name]:
                    out[name] = found
    return out


def _compile(src: Path, incremental: bool = False) -> Path:
    obj = OBJ_DIR / (src.stem + ".o")
    if incremental and obj.exists():
        # the generated text is only rewritten when it changes, so modification times tell
        # (only the hand-written ABI file includes the two headers)
        deps = [src] + ([GENERATED / "launchers.h", ROOT / "include" / "lego_hip.h"] if src.parent == CSRC else [])
        newest = max(p.stat().st_mtime for p in deps)
        if obj.stat().st_mtime > newest:
            return obj
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-I", str(ROOT / "include"), "-I", str(CSRC), "-c", str(src), "-o", str(obj)]
    asm_mfma = "asm volatile(\"v_mfma" in src.read_text()
    if asm_mfma:       # keep the device assembly beside the object and check what the compiler cannot
        cmd.insert(1, "-save-temps=obj")
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{res.stderr}")
    if asm_mfma:
        listing = OBJ_DIR / f"{src.stem}-hip-amdgcn-amd-amdhsa-gfx950.s"
        close = {f: d for f, d in asm_mfma_read_distance(listing.read_text()).items() if d[0] < ASM_MFMA_MIN_DISTANCE}
        for temp in [*OBJ_DIR.glob(f"{src.stem}-h*"), *OBJ_DIR.glob(f"{src.stem}.hip-*")]:
            temp.unlink()
        if close:
            obj.unlink()
            raise RuntimeError(f"{src.name}: an accumulator is read within {ASM_MFMA_MIN_DISTANCE} instructions of "
                               f"the inline-assembly MFMA that writes it: {close}")
    return obj


def build(verbose=True, incremental=False):
    """Generate, compile every translation unit for gfx950 and link liblego_hip.so.  With
    ``incremental`` a translation unit whose object file is newer than its source is kept."""
    sources = generate() + [CSRC / "lego_hip_abi.hip"]
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    with ThreadPoolExecutor(max_workers=8) as pool:
        objs = list(pool.map(lambda s: _compile(s, incremental), sources))
    cmd = [hipcc_path(), f"--offload-arch=gfx950", "-shared", "-fPIC", *[str(o) for o in objs], "-o", str(LIB_PATH)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    if verbose:
        print(f"built {LIB_PATH} from {len(sources)} translation units")
    return LIB_PATH


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--emit", action="store_true", help="generate sources only")
    ap.add_argument("--incremental", action="store_true", help="recompile only the sources that changed")
    ns = ap.parse_args()
    if ns.emit:
        for p in generate():
            print(p)
    else:
        build(incremental=ns.incremental)
    sys.exit(0)
