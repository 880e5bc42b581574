"""lego_hip: the HIP (gfx950 / MI355X) lowering of LEGO layouts.

Two faces, like the reference's backends (reference: lego/lego_c.py:5-38 is a printer
backend, lego/lego_mlir.py:26-393 is a builder backend):

``LEGOHipCodePrinter``
    a sympy code printer.  Generators print LEGO offset expressions with it and paste
    them into HIP kernel templates, the way the reference's generators paste
    ``LEGOPythonCodePrinter`` output into Triton templates
    (benchmarks/triton/matmul_sympy.py:453-460).

``printer`` / ``HipTensor``
    a kernel-builder with the names of the reference's MLIR builder -- ``generate_gpu_kernel``,
    ``generate_loop``, ``get_block_linear_index``, ``get_thread_linear_index``,
    ``insert_barrier``, ``translate`` -- that emits HIP C++ text instead of MLIR, so a
    program such as benchmarks/mlir/transpose_smem.py:28-80 runs against it by changing
    the import.  As in the reference, the decorators run their body at once.

Text becomes code through ``HipModule``: ``hipcc --offload-arch=gfx950 -shared`` and
``ctypes``.  Importing this module needs neither the compiler nor a GPU.
"""
from __future__ import annotations

import ctypes
import functools
import hashlib
import os
import subprocess
from enum import Enum
from pathlib import Path

from .lego import *  # noqa: F401,F403
from .lego import GroupBy, TritonRange, product, sp
from .lego_c import LEGOCCodePrinter
from sympy.printing.precedence import precedence as _precedence

GFX_ARCH = "gfx950"
HIPCC_FLAGS = [
    f"--offload-arch={GFX_ARCH}", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 arithmetic is kept off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
]
_PKG_DIR = Path(__file__).resolve().parent
JIT_DIR = _PKG_DIR / "lib" / "jit"


# ---------------------------------------------------------------------------
# expression printer
# ---------------------------------------------------------------------------

class HipIntegerRules:
    """Every printing rule an index expression needs to come out as C++ integer arithmetic, as a mixin
    that goes IN FRONT of any sympy C printer.

    ``LEGOHipCodePrinter`` carries these rules itself instead of inheriting them from the C printer
    it sits beside: the reference's ``LEGOCCodePrinter`` (lego/lego_c.py:5-38) overrides ``floor`` and
    ``Pow`` only, so ``Min``/``Max`` -- which the grouped launch order uses
    (benchmarks/triton/matmul_sympy.py:57-65) -- would print as the C99 printer's ``fmin``/``fmax``, a
    ``BitXor`` swizzle as an unknown function call, and ``x - 4*Mod(r, 2)`` as ``x - 4*r % 2``.  With
    the mixin first in the method resolution order the text is the same over either parent, or over
    ``sympy.printing.c.C99CodePrinter`` directly."""

    def _print_floor(self, expr):
        num, den = expr.args[0].as_numer_denom()
        return f"(({self._print(num)})/({self._print(den)}))"

    @staticmethod
    def _small_power(expr):
        return expr.is_Pow and expr.exp.is_Integer and 2 <= int(expr.exp) <= 4

    def _print_Pow(self, expr):
        if self._small_power(expr):      # i*i, as the reference prints it (benchmarks/cuda/nw/needle_kernel.cu:10)
            return "*".join([self.parenthesize(expr.base, _precedence(expr))] * int(expr.exp))
        return super()._print_Pow(expr)

    def _print_Mod(self, expr):
        # an operand printed as a product needs parentheses that sympy's ranking of Pow above % does not ask for
        parts = []
        for arg in expr.args:
            text = self.parenthesize(arg, _precedence(expr))
            parts.append(f"({text})" if self._small_power(arg) else text)
        return " % ".join(parts)

    def _print_Mul(self, expr):
        # sympy picks the parenthesisation level of a product before it strips the sign, so a negative
        # product's factors would print at the level of a sum: print the positive product on its own
        coeff, _ = expr.as_coeff_Mul()
        if coeff.is_negative:
            positive = -expr
            text = self._print(positive)
            return "-(" + text + ")" if isinstance(positive, sp.Mod) else "-" + text
        return super()._print_Mul(expr)

    def _integer_select(self, args, op):
        out = self._print(args[0])
        for a in args[1:]:
            b = self._print(a)
            out = f"(({out}) {op} ({b}) ? ({out}) : ({b}))"
        return out

    def _print_Min(self, expr):
        return self._integer_select(expr.args, "<")

    def _print_Max(self, expr):
        return self._integer_select(expr.args, ">")

    def _print_BitXor(self, expr):      # dispatched by the function's name: any integer-valued Function called BitXor
        a, b = expr.args
        return f"(({self._print(a)}) ^ ({self._print(b)}))"


    # ``lane_vectors`` maps the axis of a ``TritonRange`` to the name of the per-lane scalar that plays the
    # role of that index vector in the kernel (a lane holds one element of a Triton block, so
    # ``tl.arange(0, BM)[:, None]`` becomes, say, ``row``).  Without a mapping the vector prints as ``lane<axis>``.
    def __init__(self, settings=None, lane_vectors=None, **kwargs):
        self.lane_vectors = dict(lane_vectors or {})
        merged = dict(settings or {})
        merged.update(kwargs)
        # The parents disagree on how settings arrive: this package's C printer and the reference's
        # (lego/lego_c.py:6-7) take them as keywords, sympy's own C printers as one positional dict.
        try:
            super().__init__(**merged)
        except TypeError:
            super().__init__(merged)


    def _print_TritonRange(self, expr):
        axis = int(expr.args[1]) if expr.args[1].is_Integer else expr.args[1]
        name = self.lane_vectors.get(axis, f"lane{axis}")
        vec = expr.args[0]
        lo = vec.args[0] if getattr(vec, "args", None) else 0
        return name if lo == 0 else f"({self._print(lo)} + {name})"

    def _print_Relational(self, expr):
        return f"{self._print(expr.lhs)} {expr.rel_op} {self._print(expr.rhs)}"


class LEGOHipCodePrinter(HipIntegerRules, LEGOCCodePrinter):
    """Prints index expressions as HIP/C++ integer arithmetic: ``HipIntegerRules`` over the C printer of the
    package it is part of (``LEGOHipCodePrinter(lane_vectors={0: "row", 1: "col"}).doprint(expr)``)."""


# ---------------------------------------------------------------------------
# modules: text -> shared object -> ctypes
# ---------------------------------------------------------------------------

def hipcc_path():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    return "hipcc"


def compile_shared(sources, out_path, extra_flags=(), include_dirs=()):
    """``hipcc -shared`` the given source files into ``out_path`` for gfx950."""
    out_path = Path(out_path)
    out_path.parent.mkdir(parents=True, exist_ok=True)
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-shared", *extra_flags]
    for inc in include_dirs:
        cmd += ["-I", str(inc)]
    cmd += [str(s) for s in sources] + ["-o", str(out_path)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{' '.join(cmd)}\n{res.stderr}")
    return out_path


class HipModule:
    """HIP source text plus the C-ABI launchers it exports."""

    def __init__(self, name, source, launchers=()):
        self.name = name
        self.source = source
        self.launchers = list(launchers)
        self._lib = None

    @property
    def digest(self):
        return hashlib.sha256(self.source.encode()).hexdigest()[:16]

    @property
    def so_path(self):
        return JIT_DIR / f"{self.name}-{self.digest}.so"

    def build(self, force=False):
        """Compile (unless an object for this exact text is already there)."""
        if force or not self.so_path.exists():
            JIT_DIR.mkdir(parents=True, exist_ok=True)
            src = JIT_DIR / f"{self.name}-{self.digest}.hip"
            src.write_text(self.source)
            compile_shared([src], self.so_path)
        return self.so_path

    def load(self):
        if self._lib is None:
            self._lib = ctypes.CDLL(str(self.build()))
        return self._lib

    def launch(self, launcher, *tensors, stream=0):
        """Call ``int launcher(void* ..., hipStream_t)`` with device pointers of torch
        tensors (or raw ints).  Raises on a non-zero ``hipError_t``."""
        fn = getattr(self.load(), launcher)
        fn.restype = ctypes.c_int
        args = [ctypes.c_void_p(t.data_ptr() if hasattr(t, "data_ptr") else int(t)) for t in tensors]
        err = fn(*args, ctypes.c_void_p(stream))
        if err != 0:
            raise RuntimeError(f"{launcher}: hipError_t {err}")

    def __str__(self):
        return self.source


# ---------------------------------------------------------------------------
# kernel builder
# ---------------------------------------------------------------------------

class MemorySpace(Enum):
    HOST_MEMORY = 0
    GLOBAL_MEMORY = 1
    SHARED_MEMORY = 3
    PRIVATE_MEMORY = 5


_CTYPES = {"f32": "float", "f16": "_Float16", "i32": "int", "u32": "unsigned"}


class HipValue:
    """A named temporary of the kernel being emitted (the SSA value of the MLIR builder)."""

    def __init__(self, name, ctype):
        self.name, self.ctype = name, ctype

    def __str__(self):
        return self.name

    # arithmetic on temporaries prints as C++ expressions (the MLIR builder's arith ops on SSA values)
    def _binary(self, op, other, swap=False):
        a, b = (other, self) if swap else (self, other)
        return HipValue(f"({a} {op} {b})", self.ctype)

    def __add__(self, other):
        return self._binary("+", other)

    def __radd__(self, other):
        return self._binary("+", other, swap=True)

    def __sub__(self, other):
        return self._binary("-", other)

    def __rsub__(self, other):
        return self._binary("-", other, swap=True)

    def __mul__(self, other):
        return self._binary("*", other)

    def __rmul__(self, other):
        return self._binary("*", other, swap=True)


class _Emitter:
    def __init__(self):
        self.lines = []
        self.depth = 1
        self.counter = 0

    def emit(self, text):
        self.lines.append("  " * self.depth + text)

    def fresh(self, stem):
        self.counter += 1
        return f"{stem}{self.counter}"


class HipKernelBuilder:
    """HIP counterpart of the reference's ``SympyMLIRPrinter`` (lego/lego_mlir.py:26-272).

    Index arithmetic is unsigned 32-bit, as in the reference's lowering
    (``divui``/``remui``, lego/lego_mlir.py:231-249); the final pointer add is 64-bit.
    """

    def __init__(self):
        self._code = LEGOHipCodePrinter()
        self._em = None           # emitter of the kernel under construction
        self._kernels = []        # finished (name, text, launcher text, launcher name)
        self._module_name = None
        self._sym_i = 0

    # ---- module --------------------------------------------------------------------
    def generate_hip(self, name="lego_module"):
        """Run ``body`` and return the ``HipModule`` holding every kernel it generated
        (counterpart of ``generate_mlir``, lego/lego_mlir.py:53-70, which prints)."""
        def decorator(body):
            self._kernels, self._module_name = [], name
            body()
            parts = ["// generated by lego_amd.lego_hip -- do not edit",
                     "#include <hip/hip_runtime.h>", ""]
            launchers = []
            for kname, ktext, ltext, lname in self._kernels:
                parts += [ktext, "", ltext, ""]
                launchers.append(lname)
            self._module_name = None
            return HipModule(name, "\n".join(parts), launchers)
        return decorator

    # ---- kernels ---------------------------------------------------------------------
    def generate_gpu_kernel(self, ins, outs, gridSize, blockSize, workgroup_memory=(),
                            private_memory=(), name=None):
        """Emit one ``__global__`` kernel and its launcher.  ``ins``/``outs`` become pointer
        parameters in that order, ``workgroup_memory`` tensors become ``__shared__`` arrays,
        ``private_memory`` tensors per-lane arrays (lego/lego_mlir.py:115-165)."""
        def decorator(body):
            tensors = []
            for t in list(ins) + list(outs):
                if t not in tensors:
                    tensors.append(t)
            kname = name or f"{self._module_name or 'lego'}_k{len(self._kernels)}"
            em = self._em = _Emitter()
            for i, t in enumerate(tensors):
                t.set_memory_space(MemorySpace.GLOBAL_MEMORY)
                t.ref = f"g{i}"
            for i, t in enumerate(workgroup_memory):
                t.set_memory_space(MemorySpace.SHARED_MEMORY)
                t.ref = f"lds{i}"
                em.emit(f"__shared__ {t.ctype} {t.ref}[{int(t.get_flattend_shape())}];")
            for i, t in enumerate(private_memory):
                t.set_memory_space(MemorySpace.PRIVATE_MEMORY)
                t.ref = f"priv{i}"
                em.emit(f"{t.ctype} {t.ref}[{int(t.get_flattend_shape())}];")
            body(tuple(t.ref for t in tensors))
            self._em = None
            threads = int(product(list(blockSize)))
            params = ", ".join(
                f"{'const ' if t not in outs else ''}{t.ctype}* __restrict__ {t.ref}" for t in tensors)
            ktext = (f"extern \"C\" __global__ void __launch_bounds__({threads}) {kname}({params}) {{\n"
                     + "\n".join(em.lines) + "\n}")
            lname = f"{kname}_launch"
            largs = ", ".join(f"{'const ' if t not in outs else ''}void* p{i}" for i, t in enumerate(tensors))
            casts = ", ".join(
                f"static_cast<{'const ' if t not in outs else ''}{t.ctype}*>(p{i})" for i, t in enumerate(tensors))
            g, b = [int(v) for v in gridSize], [int(v) for v in blockSize]
            ltext = (f"extern \"C\" int {lname}({largs}, hipStream_t stream) {{\n"
                     f"  hipLaunchKernelGGL({kname}, dim3({g[0]}, {g[1]}, {g[2]}), dim3({b[0]}, {b[1]}, {b[2]}),"
                     f" 0, stream, {casts});\n"
                     f"  return static_cast<int>(hipGetLastError());\n}}")
            self._kernels.append((kname, ktext, ltext, lname))
        return decorator

    def generate_loop(self, l: GroupBy, step=1, iter_args=()):
        """``for`` over ``prod(l.dims())`` steps; the body receives the logical index
        ``l.inv(i)`` and the flat counter (lego/lego_mlir.py:85-108).  The loop is emitted
        with ``#pragma unroll`` because its trip count is a generation-time constant.

        With ``iter_args`` (initial values: temporaries or literals) the loop carries values, as the
        reference's ``affine.for ... iter_args``: each becomes a named C++ temporary, the body
        receives them as a third argument and returns their next values, and -- as in the
        reference, where the decorated name is then bound to a function -- the decorator returns a
        callable that emits the loop when called and returns the carried temporaries as they stand
        after the last step.  ``ctype`` of a carried value: that of its initial temporary, ``float``
        for a literal."""
        carried = tuple(iter_args)

        def emit_loop(body):
            em = self._em
            carries = []
            for init in carried:
                ctype = init.ctype if isinstance(init, HipValue) else ("float" if isinstance(init, float) else "unsigned")
                carry = HipValue(em.fresh("carry"), ctype)
                em.emit(f"{ctype} {carry} = {init};")
                carries.append(carry)
            var = em.fresh("it")
            trip = self._code.doprint(sp.sympify(product(l.dims())))
            em.emit("#pragma unroll")
            em.emit(f"for (unsigned {var} = 0; {var} < {trip}; {var} += {int(step)}) {{")
            em.depth += 1
            idx = sp.Symbol(var, integer=True, nonnegative=True)
            if carries:
                nxt = body(l.inv(idx), idx, tuple(carries))
                nxt = tuple(nxt) if isinstance(nxt, (tuple, list)) else (nxt,)
                if len(nxt) != len(carries):
                    raise ValueError("the loop body must return one value per iter_arg")
                # all next values are formed before any carried temporary changes, as a yield does
                tmps = []
                for carry, value in zip(carries, nxt):
                    tmp = em.fresh("next")
                    em.emit(f"const {carry.ctype} {tmp} = {value};")
                    tmps.append(tmp)
                for carry, tmp in zip(carries, tmps):
                    em.emit(f"{carry} = {tmp};")
            else:
                body(l.inv(idx), idx)
            em.depth -= 1
            em.emit("}")
            return tuple(carries)

        def decorator(body):
            if carried:
                return lambda: emit_loop(body)
            emit_loop(body)
        return decorator

    def get_block_linear_index(self):
        return self._named("bX", "blockIdx.x")

    def get_thread_linear_index(self):
        return self._named("tX", "threadIdx.x")

    def _named(self, stem, value):
        name = self._em.fresh(stem)
        self._em.emit(f"const unsigned {name} = {value};")
        return sp.Symbol(name, integer=True, nonnegative=True)

    def insert_barrier(self):
        self._em.emit("__syncthreads();")

    def translate(self, expr):
        """C++ text of an index expression over the symbols handed out by this builder."""
        return self._code.doprint(sp.sympify(expr))

    # ---- used by HipTensor ------------------------------------------------------------
    def _load(self, tensor, offset):
        name = self._em.fresh("v")
        self._em.emit(f"const {tensor.ctype} {name} = {tensor.ref}[(size_t)({self.translate(offset)})];")
        return HipValue(name, tensor.ctype)

    def _store(self, tensor, offset, value):
        self._em.emit(f"{tensor.ref}[(size_t)({self.translate(offset)})] = {value};")


class HipTensor:
    """A buffer addressed by *logical* LEGO indices (reference: ``MLIRTensor``,
    lego/lego_mlir.py:274-390).  ``tensor.layout`` may be re-assigned between phases of
    a kernel, which is how the reference re-reads a staging tile in another order
    (benchmarks/mlir/transpose_smem.py:61,74)."""

    def __init__(self, layout: GroupBy, dtype="f32", is_dim_shape=False):
        if dtype not in _CTYPES:
            raise ValueError(f"unsupported dtype {dtype!r}")
        self.layout = layout
        self.dtype = dtype
        self.ctype = _CTYPES[dtype]
        self.dimension = layout.d
        self.memory_space = MemorySpace.HOST_MEMORY
        self.ref = None

    def get_flattend_shape(self):
        return product(self.layout.dims())

    def set_memory_space(self, memory_space: MemorySpace):
        self.memory_space = memory_space
        return self

    def offset(self, key):
        """Simplified flat offset of logical index ``key`` (expressions allowed)."""
        if not isinstance(key, tuple):
            key = (key,)
        dummies = {sp.Symbol(f"_tr{i}", integer=True): sp.sympify(k) for i, k in enumerate(key)}
        return self.layout[tuple(dummies)].xreplace(dummies)

    def __getitem__(self, key):
        return printer._load(self, self.offset(key))

    def __setitem__(self, key, value):
        printer._store(self, self.offset(key), value)


printer = HipKernelBuilder()
