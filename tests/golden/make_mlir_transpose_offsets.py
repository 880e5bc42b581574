"""Writes tests/golden/mlir_transpose_offsets.npz and mlir_transpose_digests.json.

Run in the build container only (it reads the reference's committed generated programs
under /root/reference/mlir_generated/transpose/, which are data produced by the
reference's MLIR lowering, and executes nothing from the reference).  A small
interpreter for the ``arith`` subset those programs use evaluates, for every
(block, thread, loop step), the offset of each ``memref.load`` / ``memref.store`` in the
kernel body.  The N=256 offsets are stored whole; larger sizes are stored as SHA-256
digests of the same int32 arrays.

    python tests/golden/make_mlir_transpose_offsets.py
"""
import hashlib
import json
import re
import sys
from pathlib import Path

import numpy as np

REF = Path("/root/reference/mlir_generated/transpose")
OUT = Path(__file__).resolve().parent


def interpret(path):
    """Returns {"grid": g, "block": b, "accesses": [(kind, space, offsets[g, b, steps])...]}."""
    text = path.read_text().splitlines()
    env = {}
    grid = block = None
    accesses = []
    in_kernel = False
    loop_var = None
    loop_range = None
    body = []          # buffered loop body
    blocks = threads = None

    def val(tok):
        return env[tok]

    def run(line, env, record):
        line = line.strip()
        m = re.match(r"(%\w+) = arith\.constant (-?\d+) : (i32|index)", line)
        if m:
            env[m.group(1)] = np.int64(int(m.group(2)))
            return
        m = re.match(r"(%\w+) = arith\.index_cast (%\w+) :", line)
        if m:
            env[m.group(1)] = env[m.group(2)]
            return
        m = re.match(r"(%\w+) = arith\.(remui|divui|muli|addi) (%\w+), (%\w+) : i32", line)
        if m:
            a, b = env[m.group(3)], env[m.group(4)]
            op = m.group(2)
            r = {"remui": lambda: a % b, "divui": lambda: a // b,
                 "muli": lambda: a * b, "addi": lambda: a + b}[op]()
            env[m.group(1)] = r & 0xFFFFFFFF  # i32 wrap-around (never triggers in range)
            return
        m = re.match(r"(%\w+) = memref\.load (%\w+)\[(%\w+)\] : memref<\d+xf32(, 3)?>", line)
        if m:
            env[m.group(1)] = ("value",)
            record("load", "lds" if m.group(4) else "global", env[m.group(3)])
            return
        m = re.match(r"memref\.store (%\w+), (%\w+)\[(%\w+)\] : memref<\d+xf32(, 3)?>", line)
        if m:
            record("store", "lds" if m.group(4) else "global", env[m.group(3)])
            return
        if line.startswith(("memref.assume_alignment", "gpu.barrier", "gpu.terminator")):
            return
        m = re.match(r"(%\w+) = gpu\.(block_id|thread_id)\s+x", line)
        if m:
            env[m.group(1)] = blocks if m.group(2) == "block_id" else threads
            return
        raise ValueError(f"{path.name}: cannot interpret: {line}")

    it = iter(text)
    for line in it:
        s = line.strip()
        if not in_kernel:
            m = re.match(r"(%\w+) = arith\.constant (-?\d+) : (i32|index)", s)
            if m:
                env[m.group(1)] = np.int64(int(m.group(2)))
            m = re.match(r"gpu\.launch blocks\(.*\) in \(%\w+ = (%\w+),.*threads\(.*\) in \(%\w+ = (%\w+),", s)
            if m:
                grid, block = int(env[m.group(1)]), int(env[m.group(2)])
                blocks = np.arange(grid, dtype=np.int64)[:, None, None]
                threads = np.arange(block, dtype=np.int64)[None, :, None]
                in_kernel = True
            continue
        if s.startswith("gpu.terminator"):
            break
        m = re.match(r"affine\.for (%\w+) = (\d+) to (\d+) \{", s)
        if m:
            steps = np.arange(int(m.group(2)), int(m.group(3)), dtype=np.int64)[None, None, :]
            scope = dict(env)
            scope[m.group(1)] = steps

            def record(kind, space, off, n=steps.shape[2]):
                accesses.append((kind, space, np.broadcast_to(off, (grid, block, n)).astype(np.int32)))
            for inner in it:
                if inner.strip() == "}":
                    break
                run(inner, scope, record)
            continue
        run(s, env, lambda *a: (_ for _ in ()).throw(ValueError("access outside a loop")))
    return {"grid": grid, "block": block, "accesses": accesses}


def main():
    if not REF.exists():
        sys.exit("reference not mounted; fixtures are committed, nothing to do")
    arrays, digests = {}, {}
    for path in sorted(REF.glob("transpose_*.mlir")):
        kind, n = re.match(r"transpose_(naive|smem)_(\d+)\.mlir", path.name).groups()
        res = interpret(path)
        names = []
        for i, (op, space, off) in enumerate(res["accesses"]):
            key = f"{kind}_{n}_{i}_{space}_{op}"
            names.append(key)
            digests[key] = {"sha256": hashlib.sha256(np.ascontiguousarray(off).tobytes()).hexdigest(),
                            "shape": list(off.shape), "source": f"mlir_generated/transpose/{path.name}"}
            if n == "256":
                arrays[key] = off
        print(path.name, res["grid"], res["block"], names)
    np.savez_compressed(OUT / "mlir_transpose_offsets.npz", **arrays)
    (OUT / "mlir_transpose_digests.json").write_text(json.dumps(digests, indent=1, sort_keys=True) + "\n")


if __name__ == "__main__":
    main()
