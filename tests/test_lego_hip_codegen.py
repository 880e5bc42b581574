"""The HIP lowering on the CPU: printer output, the builder DSL, the kernel generators, and
(with hipcc, which cross-compiles gfx950 without a GPU) that the emitted text compiles."""
import shutil
import subprocess

import pytest
import sympy as sp

from lego_amd.lego_hip import (HIPCC_FLAGS, HipTensor, LEGOHipCodePrinter, hipcc_path, printer)
from lego_amd.lego import Col, OrderBy, Row, BitXor
from lego_amd.kernels import dsl_transpose, gemm, rowwise, transpose


def test_printer_integer_forms():
    a, b, n = sp.symbols("a b n", integer=True, positive=True)
    pr = LEGOHipCodePrinter()
    assert pr.doprint(sp.floor(a / b)) == "((a)/(b))"
    assert pr.doprint(sp.Mod(a, b)) == "a % b"
    assert pr.doprint(sp.Min(a, b)) == "((a) < (b) ? (a) : (b))"      # not fmin: indices are integers
    assert pr.doprint(sp.Max(a - 5, 1)) == "((1) > (a - 5) ? (1) : (a - 5))"
    assert pr.doprint(BitXor(a, 4 * b)) == "((a) ^ (4*b))"
    assert pr.doprint(a ** 2) == "a*a"
    lay = OrderBy(Row(n, n)).TileBy([n / 32, n / 32], [32, 32])
    text = LEGOHipCodePrinter(lane_vectors={0: "row", 1: "col"}).doprint(lay["bi", "bj", :, :])
    assert text == "32*bj + n*(32*bi + row) + col"


def test_builder_emits_the_reference_transpose_offsets():
    mod = dsl_transpose.transpose_smem(256)
    src = mod.source
    assert "__shared__ float lds0[1024];" in src and "__syncthreads();" in src
    # the same offsets the reference's MLIR holds (transpose_smem_256.mlir:33-69), up to term order
    assert "2048*it3 + 32*(bX1 % 8) + tX2 % 32 + 8192*((bX1)/(8)) + 256*((tX2)/(32))" in src
    assert "8*it5 + 32*(tX2 % 32) + ((tX2)/(32))" in src
    assert mod.launchers == ["lego_dsl_transpose_smem_f32_256_k0_launch"]
    naive = dsl_transpose.transpose_naive(256).source
    assert "8*it3 + 8192*(bX1 % 8) + 256*(tX2 % 32) + 32*((bX1)/(8)) + ((tX2)/(32))" in naive


def test_builder_offsets_match_golden_mlir_offsets(golden_dir):
    """Evaluate the emitted C expressions for every block, thread and step against the offsets
    interpreted from the reference's generated program."""
    import re

    import numpy as np
    gold = np.load(golden_dir / "mlir_transpose_offsets.npz")
    src = dsl_transpose.transpose_smem(256).source
    exprs = re.findall(r"\[\(size_t\)\((.*?)\)\]", src)
    assert len(exprs) == 4
    bX = np.arange(64, dtype=np.int64)[:, None, None]
    tX = np.arange(256, dtype=np.int64)[None, :, None]
    it = np.arange(4, dtype=np.int64)[None, None, :]
    keys = ["smem_256_0_global_load", "smem_256_1_lds_store", "smem_256_2_lds_load", "smem_256_3_global_store"]
    for text, key in zip(exprs, keys):
        py = re.sub(r"\(\((\w+)\)/\((\d+)\)\)", r"(\1//\2)", text)
        val = eval(py, {"__builtins__": {}}, {"bX1": bX, "tX2": tX, "it3": it, "it5": it})
        assert np.array_equal(np.broadcast_to(val, gold[key].shape), gold[key]), key


def test_generators_emit_layout_derived_text():
    t, meta = transpose.emit("f16", (64, 64), (1, 4), "diag")
    assert "const size_t Bj = (wg + ((wg)/(nBj))) % nBj;" in t.text
    assert "64*Bi + R*(256*Bj + 2*k) + 8*rv" in t.text            # column-major destination
    r = rowwise.emit(4)
    assert "const unsigned row = team + wg;" in r.text or "const unsigned row = wg" in r.text
    g, _ = gemm.emit()
    # the reference's grouped launch order, printed with integer min/max
    assert "pid % ((GM) < (num_pid_m) ? (GM) : (num_pid_m))" in g.text
    assert "ds_read_tr16_b64" in g.text and "mfma_f32_32x32x16_f16" in g.text


@pytest.mark.skipif(shutil.which(hipcc_path()) is None and not __import__("os").path.exists(hipcc_path()),
                    reason="hipcc not available")
def test_builder_module_compiles_for_gfx950(tmp_path):
    src = tmp_path / "k.hip"
    src.write_text(dsl_transpose.transpose_naive(512).source)
    res = subprocess.run([hipcc_path(), *HIPCC_FLAGS, "--cuda-device-only", "-c", str(src), "-o", str(tmp_path / "k.o")],
                         capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


def test_negative_products_keep_their_parentheses():
    """sympy prints x - 4*Mod(r, 2) as 'x - 4*r % 2'; C and Python read that as x - (4*r) % 2."""
    from lego_amd.lego_python import LEGOPythonCodePrinter
    r, x = sp.symbols("r x", integer=True, nonnegative=True)
    for pr in (LEGOHipCodePrinter(), LEGOPythonCodePrinter()):
        for expr in (x - 4 * sp.Mod(r, 2), x - sp.Mod(r, 2), 7 - x * sp.Mod(r, 3), -sp.Mod(r, 2) + 9):
            text = pr.doprint(expr).replace("/", "//")
            for rv in range(6):
                for xv in range(4):
                    assert eval(text, {}, {"r": rv, "x": xv}) == expr.subs({r: rv, x: xv}), (expr, text)


def test_sympy_mod_product_defect_is_guarded():
    """Mod(8*Mod(y, 2048), 256) must stay a function that equals (8*(y % 2048)) % 256."""
    y = sp.Symbol("y", integer=True, nonnegative=True)
    for c, n, q in [(8, 2048, 256), (3, 5, 7), (6, 10, 4), (4, 3, 8), (12, 7, 18)]:
        e = sp.Mod(c * sp.Mod(y, n), q)
        for v in range(0, 80, 3):
            assert int(e.subs(y, v)) == (c * (v % n)) % q


def test_mod_by_a_power_is_parenthesised():
    """Small integer powers are printed as products (as the reference does); as an operand of
    ``%`` such a product needs parentheses that sympy's precedence table does not ask for."""
    from lego_amd.lego_c import LEGOCCodePrinter
    w, n = sp.symbols("w n", integer=True, positive=True)
    for printer in (LEGOHipCodePrinter(), LEGOCCodePrinter()):
        text = printer.doprint(sp.floor(sp.Mod(w, n**2) / n))
        assert text == "((w % (n*n))/(n))"
        for wv in range(0, 60, 7):
            for nv in (2, 3, 5):
                assert eval(text.replace("/", "//"), {}, {"w": wv, "n": nv}) == (wv % (nv * nv)) // nv
        assert printer.doprint(sp.Mod(n**2, 7)) == "(n*n) % 7"


def test_loops_carry_values():
    """``generate_loop(iter_args=...)``: carried values become named temporaries, the body's return
    values are assigned after all of them are formed, and the decorated name is a callable that
    returns the temporaries (the reference binds it to a function as well, lego/lego_mlir.py:105-107)."""
    mod = dsl_transpose.row_sums(128, 48)
    text = mod.source
    assert "float carry" in text and "= 0.0;" in text
    body = text[text.index("for (unsigned"):]
    assert body.index("const float next") < body.index("carry", body.index("const float next") + 20)
    assert "+= 1" in body and "< 48" in body
    # two carried values swap through temporaries, not through each other
    from lego_amd.lego_hip import HipTensor, printer
    from lego_amd.lego import OrderBy, Row

    @printer.generate_hip(name="swap")
    def module():
        T = HipTensor(OrderBy(Row(64)).TileBy([64]), "f32")

        @printer.generate_gpu_kernel([T], [T], (1, 1, 1), (64, 1, 1))
        def kernel(_):
            tX = printer.get_thread_linear_index()

            @printer.generate_loop(OrderBy(Row(3)).TileBy([3]), iter_args=[1.0, 2.0])
            def swap(pargs, _, carried):
                return carried[1], carried[0]
            a, b = swap()
            T[tX] = a - b
    lines = [ln.strip() for ln in module.source.splitlines()]
    first = next(i for i, ln in enumerate(lines) if ln.startswith("const float next"))
    assert lines[first + 1].startswith("const float next") and lines[first + 2].startswith("carry")
    with pytest.raises(ValueError):
        @printer.generate_hip(name="bad")
        def bad():
            T = HipTensor(OrderBy(Row(64)).TileBy([64]), "f32")

            @printer.generate_gpu_kernel([T], [T], (1, 1, 1), (64, 1, 1))
            def kernel(_):
                @printer.generate_loop(OrderBy(Row(3)).TileBy([3]), iter_args=[1.0, 2.0])
                def loop(pargs, _, carried):
                    return carried[0]
                loop()


def _launch_order_exprs():
    npm, npn, gm, pid = sp.symbols("num_pid_m num_pid_n GM pid", integer=True, positive=True)
    return gemm.launch_order(npm, npn, gm, pid)      # benchmarks/triton/matmul_sympy.py:57-65


class _ReferenceShapedCPrinter(sp.printing.c.C99CodePrinter):
    """What the HIP printer finds beside it when its file is dropped into the reference's package: a C99
    printer that takes its settings as keywords and overrides ``floor`` only, so ``Min``/``Max`` fall
    through to ``fmin``/``fmax`` (the behaviour of lego/lego_c.py:5-38, restated here in five lines)."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, kwargs)

    def _print_floor(self, expr):
        num, den = expr.args[0].as_numer_denom()
        return f"(({self._print(num)})/({self._print(den)}))"


@pytest.mark.parametrize("parent", [sp.printing.c.C99CodePrinter, _ReferenceShapedCPrinter])
def test_hip_rules_print_integers_over_a_stock_c_printer(parent, tmp_path):
    """The HIP printer's rules do not lean on the C printer they sit on: over sympy's own C99 printer and over
    one shaped like the reference's (both print Min/Max as fmin/fmax), the grouped launch order still comes out
    as integer ternaries, character for character what LEGOHipCodePrinter prints, and its value is the
    reference's generated pid_m / pid_n (triton_generated/matmul/matmul_NTA_NTB.py:108-109)."""
    from lego_amd.lego_hip import HipIntegerRules
    from oracle.kernels import grouped_pid

    pm, pn = _launch_order_exprs()
    assert "fmin" in parent().doprint(pm) or "fmin" in _ReferenceShapedCPrinter().doprint(pm)      # what is being avoided
    over = type("HipOver" + parent.__name__, (HipIntegerRules, parent), {})
    pr = over(allow_unknown_functions=True)
    text_m, text_n = pr.doprint(pm), pr.doprint(pn)
    ours = LEGOHipCodePrinter(allow_unknown_functions=True)
    assert (text_m, text_n) == (ours.doprint(pm), ours.doprint(pn))
    for text in (text_m, text_n):
        assert "fmin" not in text and "fmax" not in text and "?" in text
    a, b = sp.symbols("a b", integer=True, positive=True)
    assert pr.doprint(BitXor(a, 4 * b)) == "((a) ^ (4*b))"
    assert pr.doprint(a - 4 * sp.Mod(b, 2)) == "a - 4*(b % 2)"
    assert pr.doprint(sp.Mod(a, b ** 2)) == "a % (b*b)"

    # the printed text is C: compile it with the host compiler and run it over whole launch grids
    cases = ((32, 32, 8), (16, 8, 8), (8, 16, 4), (4, 4, 8), (6, 5, 3))
    src = tmp_path / "order.c"
    src.write_text(
        "#include <stdio.h>\n"
        f"static int pm(int pid, int num_pid_m, int num_pid_n, int GM) {{ return {text_m}; }}\n"
        f"static int pn(int pid, int num_pid_m, int num_pid_n, int GM) {{ return {text_n}; }}\n"
        "int main(void) {\n"
        + "".join(f"  for (int pid = 0; pid < {npm * npn}; ++pid) printf(\"%d %d\\n\", pm(pid, {npm}, {npn}, {gm}), pn(pid, {npm}, {npn}, {gm}));\n"
                  for npm, npn, gm in cases)
        + "  return 0;\n}\n")
    exe = tmp_path / "order"
    subprocess.run(["gcc", "-O1", "-Wall", "-Werror", str(src), "-o", str(exe)], check=True, capture_output=True)
    got = [tuple(int(v) for v in line.split()) for line in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines()]
    want = [tuple(int(v) for v in grouped_pid(pid, npm, npn, gm)) for npm, npn, gm in cases for pid in range(npm * npn)]
    assert got == want
