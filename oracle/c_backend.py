"""Compile-and-run side of the CPU oracle (test infrastructure; see package
docstring): what `CCompiler`, `CKernel`, `CBuffer` and `CBackendRegistry` do in
`crates/backend-c/src/{compiler,kernel,buffer,lib}.rs`.

`openmp=True` adds what `backend-openmp` adds: `#pragma omp parallel for` on the
outermost loop of each kernel (`src/backend/compile.rs:400-480`) and `-fopenmp`
(`crates/backend-openmp/src/compiler.rs:153-166`).  It is a second CPU
baseline, never the parity reference.
"""

from __future__ import annotations

import ctypes
import os
import re
import subprocess
import tempfile
from typing import List, Optional, Sequence

import numpy as np

from .c_renderer import render_program
from .sexpr import parse

_ITEMSIZE = {"bool": 1, "i8": 1, "u8": 1, "i16": 2, "u16": 2, "f16": 2, "bf16": 2,
             "i32": 4, "u32": 4, "f32": 4, "i64": 8, "u64": 8, "f64": 8, "int": 8}

GCC_ARGS = ["-O3", "-ffast-math", "-shared", "-fPIC"]     # compiler.rs:153-165


def _dtype_name(dt) -> str:
    return dt if isinstance(dt, str) else getattr(dt, "name", str(dt))


class CBuffer:
    """Host memory, zero-initialised (buffer.rs:84-93)."""

    def __init__(self, shape: Sequence[int], dtype):
        self.shape = list(shape)
        self.dtype = dtype
        n = 1
        for s in self.shape:
            n *= int(s)
        self._nbytes = n * _ITEMSIZE[_dtype_name(dtype)]
        self.data = np.zeros(max(self._nbytes, 1), dtype=np.uint8)

    def byte_len(self) -> int:
        return self._nbytes

    def read_to_host(self) -> bytes:
        return self.data[:self._nbytes].tobytes()

    def write_from_host(self, raw: bytes) -> None:
        if len(raw) != self._nbytes:                       # buffer.rs:107-113
            raise ValueError(f"Buffer size mismatch: expected {self._nbytes}, got {len(raw)}")
        self.data[:self._nbytes] = np.frombuffer(raw, dtype=np.uint8)

    def clone_buffer(self) -> "CBuffer":
        b = CBuffer(self.shape, self.dtype)
        b.data[:] = self.data
        return b

    def ptr(self) -> ctypes.c_void_p:
        return ctypes.c_void_p(self.data.ctypes.data)


def _add_openmp_pragmas(src: str) -> str:
    """Mark each kernel's outermost `for` (the first loop at one indent level
    inside a function body) as parallel."""
    out = []
    for line in src.split("\n"):
        if re.match(r"^    for \(", line):
            out.append("    #pragma omp parallel for")
        out.append(line)
    return "\n".join(out)


class CKernel:
    def __init__(self, source: str, entry_point: str, n_ptr_args: int, openmp: bool = False,
                 gcc_args: Optional[Sequence[str]] = None):
        """`gcc_args` replaces the reference's flags; tests that compare two forms of one
        kernel for equal evaluation order use it to compile without -ffast-math."""
        self.source = source
        self.entry_point = entry_point
        self.n_ptr_args = n_ptr_args
        self._tmp = tempfile.TemporaryDirectory(prefix="eclat_c_")
        src_path = os.path.join(self._tmp.name, "kernel.c")
        lib_path = os.path.join(self._tmp.name, f"lib{entry_point}.so")
        with open(src_path, "w") as f:
            f.write(source)
        args = ["gcc"] + list(GCC_ARGS if gcc_args is None else gcc_args) + (["-fopenmp"] if openmp else []) + \
               ["-o", lib_path, src_path, "-lm"]
        r = subprocess.run(args, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"CompilationFailed: stderr: {r.stderr}\nstdout: {r.stdout}")
        self._lib = ctypes.CDLL(lib_path)
        self._fn = getattr(self._lib, entry_point)
        self._fn.restype = None

    def execute(self, inputs: Sequence[CBuffer], outputs: Sequence[CBuffer]) -> None:
        args = [b.ptr() for b in inputs] + [b.ptr() for b in outputs]
        if not 1 <= len(args) <= 6:                        # kernel.rs:161-167
            raise RuntimeError(f"Unsupported number of kernel arguments: {len(args)}. "
                               f"Maximum supported is 6.")
        self._fn(*args)

    def call_raw(self, *ptrs) -> None:
        self._fn(*ptrs)


def compile_program_text(ast_text: str, openmp: bool = False, gcc_args: Optional[Sequence[str]] = None) -> CKernel:
    """One Program holding one kernel -> a callable (lib.rs:50-112)."""
    tree = parse(ast_text)
    kernels = [x for x in tree[1:] if isinstance(x, list) and x[0] == "kernel"]
    if len(kernels) != 1:
        raise ValueError("the C backend compiles one kernel per program")
    k = kernels[0]
    nptr = sum(1 for p in k[2][1:] if isinstance(p[1], list) and p[1][0] == "ptr")
    src = render_program(ast_text)
    if openmp:
        src = _add_openmp_pragmas(src)
    return CKernel(src, str(k[1]), nptr, openmp=openmp, gcc_args=gcc_args)


class CBackend:
    """Plugs into `harp_amd.frontend.device.register_backend` from tests."""

    def __init__(self, openmp: bool = False, exact_division: bool = False):
        """`exact_division`: the reference's flags (-O3 -ffast-math, compiler.rs:153-165) plus
        -mno-recip, device kind "c-exactdiv".  Under -ffast-math gcc divides floats in a vectorised
        loop with rcpps and one Newton-Raphson step, in a scalar loop with divss: the same
        `1.0f / x` then differs in its last bit between two kernels of one program, and a test for
        equality between a value and its recomputation (the gradient of max / min goes to the
        elements equal to it) fails where it should hold.  Tests of such gradients use this kind."""
        self.kind = "c-exactdiv" if exact_division else "openmp" if openmp else "c"
        self.openmp = openmp
        self.gcc_args = list(GCC_ARGS) + ["-mno-recip"] if exact_division else None
        self._devices = {}

    def name(self) -> str:
        return "OpenMP (oracle)" if self.openmp else "C (oracle)"

    def is_available(self) -> bool:
        return True

    def create_device(self, index: int):
        return self._devices.setdefault(index, ("cpu", index))

    def list_devices(self) -> List[str]:
        return ["cpu"]

    def allocate_buffer(self, device, shape, dtype) -> CBuffer:
        return CBuffer(shape, dtype)

    def compile_ast(self, device, program, signature=None) -> CKernel:
        return compile_program_text(program.to_sexpr(), openmp=self.openmp, gcc_args=self.gcc_args)
