"""Python face of the HIP backend: the objects the front end's registry drives.

Mirrors what a reference backend crate exports (`crates/backend-c/src/lib.rs`):
a registry object (`BackendRegistry`, `src/backend/device.rs:83-171`), a device,
buffers (`Buffer`, `src/backend/traits.rs:455-482`) and compiled kernels
(`Kernel`, `:531-587`).  Everything goes through the C ABI of
`include/eclat_hip.h`; nothing here computes on the host.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import byref, c_char_p, c_float, c_int, c_size_t, c_void_p
from typing import Dict, List, Optional, Sequence

from . import _lib
from ._lib import DeviceProps, EhError, LaunchInfo, check, lib


def _sexpr(ast) -> bytes:
    return (ast if isinstance(ast, str) else ast.to_sexpr()).encode()


def _opts(options) -> Optional[bytes]:
    if not options:
        return None
    if isinstance(options, dict):
        options = ",".join(f"{k}={int(v) if isinstance(v, bool) else v}" for k, v in options.items())
    return options.encode()


def _launch_dict(info: LaunchInfo) -> dict:
    return {"entry": info.entry.decode(), "source": info.source.decode(),
            "schedule": info.schedule.decode(), "grid": list(info.grid),
            "block": list(info.block), "lds_bytes": info.lds_bytes, "n_args": info.n_args,
            "n_kernels": info.n_kernels, "algo_bytes": info.algo_bytes, "flops": info.flops,
            "lane": info.lane, "n_waits": info.n_waits, "tune_key": "%016x" % info.tune_key}


# ---------------------------------------------------------------------------
# rendering / compiling without a device
# ---------------------------------------------------------------------------

class Plan:
    """Result of `eh_render_program`: HIP sources and dispatch per launch."""

    def __init__(self, ast, options=None):
        self._h = c_void_p()
        check(lib.eh_render_program(_sexpr(ast), _opts(options), byref(self._h)))
        n = c_int()
        check(lib.eh_plan_num_launches(self._h, byref(n)))
        self.launches: List[dict] = []
        for i in range(n.value):
            info = LaunchInfo()
            check(lib.eh_plan_launch(self._h, i, byref(info)))
            d = _launch_dict(info)
            d["args"], d["kernels"], d["written"], d["overwrites"], d["waits"] = [], [], [], [], []
            s, v = c_char_p(), c_int()
            for a in range(info.n_args):
                check(lib.eh_plan_launch_arg(self._h, i, a, byref(s)))
                d["args"].append(s.value.decode())
                check(lib.eh_plan_launch_arg_written(self._h, i, a, byref(v)))
                d["written"].append(bool(v.value))
                d["overwrites"].append(v.value == 2)      # every element of an exactly-sized buffer
            for w in range(info.n_waits):
                check(lib.eh_plan_launch_wait(self._h, i, w, byref(v)))
                d["waits"].append(v.value)
            for k in range(info.n_kernels):
                check(lib.eh_plan_launch_kernel(self._h, i, k, byref(s)))
                d["kernels"].append(s.value.decode())
            self.launches.append(d)
        check(lib.eh_plan_num_buffers(self._h, byref(n)))
        self.buffers: List[dict] = []
        for i in range(n.value):
            name, role, nb, el = c_char_p(), c_char_p(), c_size_t(), c_int()
            check(lib.eh_plan_buffer(self._h, i, byref(name), byref(role), byref(nb), byref(el)))
            self.buffers.append({"name": name.value.decode(), "role": role.value.decode(),
                                 "bytes": nb.value, "elided": bool(el.value)})
        check(lib.eh_plan_release(self._h))
        self._h = None


def render_program(ast, options=None) -> Plan:
    return Plan(ast, options)


def normalize_ast(ast) -> str:
    """AST text of `ast` with the reference optimiser's rewrites undone (`eh_normalize_ast`)."""
    out = c_void_p()
    check(lib.eh_normalize_ast(_sexpr(ast), byref(out)))
    try:
        return ctypes.string_at(out).decode()
    finally:
        lib.eh_free(out)


def tune_key(ast) -> str:
    """The 16 hex digits under which the file named by ECLAT_HIP_TUNE holds this program's options."""
    k = ctypes.c_ulonglong()
    check(lib.eh_tune_key(_sexpr(ast), byref(k)))
    return f"{k.value:016x}"


def compile_source(source: str, arch: str = "gfx950") -> bytes:
    """hiprtc: HIP C -> code object.  Works without a GPU."""
    blob, n = c_void_p(), c_size_t()
    check(lib.eh_compile_source(source.encode(), arch.encode(), byref(blob), byref(n)))
    try:
        return ctypes.string_at(blob, n.value)
    finally:
        lib.eh_free(blob)


def device_count() -> int:
    n = c_int()
    check(lib.eh_device_count(byref(n)))
    return n.value


# ---------------------------------------------------------------------------
# device objects
# ---------------------------------------------------------------------------

class HipDevice:
    def __init__(self, index: int = 0):
        self._h = c_void_p()
        check(lib.eh_device_open(index, byref(self._h)))
        self.index = index
        p = DeviceProps()
        check(lib.eh_device_get_props(self._h, byref(p)))
        self.props = {f: (getattr(p, f).decode() if isinstance(getattr(p, f), bytes)
                          else getattr(p, f)) for f, _ in DeviceProps._fields_}

    def profile(self) -> dict:
        """DeviceProfile (traits.rs:163-182) for gfx950."""
        return dict(self.props)

    def sync(self) -> None:
        check(lib.eh_device_sync(self._h))

    def trim(self) -> int:
        """Returns the memory of released buffers to the driver; gives the bytes that were kept."""
        kept = c_size_t(0)
        check(lib.eh_device_trim(self._h, byref(kept)))
        return kept.value

    def alloc(self, nbytes: int) -> "HipBuffer":
        return HipBuffer(self, [nbytes], None, nbytes=nbytes)


class HipBuffer:
    """Device memory, zero-filled on allocation."""

    def __init__(self, device: HipDevice, shape: Sequence[int], dtype, nbytes: Optional[int] = None):
        self.device = device
        self.shape = list(shape)
        self.dtype = dtype
        if nbytes is None:
            n = 1
            for s in self.shape:
                n *= int(s)
            nbytes = n * dtype.itemsize()
        self._nbytes = int(nbytes)
        self._h = c_void_p()
        check(lib.eh_buffer_alloc(device._h, self._nbytes, byref(self._h)))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            lib.eh_buffer_release(h)

    def byte_len(self) -> int:
        return self._nbytes

    def device_ptr(self) -> int:
        p = c_void_p()
        check(lib.eh_buffer_device_ptr(self._h, byref(p)))
        return p.value or 0

    def write_from_host(self, raw) -> None:
        raw = raw if isinstance(raw, bytes) else bytes(raw)
        check(lib.eh_buffer_write(self._h, raw if raw else None, len(raw)))     # read in place

    def write_array(self, arr) -> None:
        """Zero-copy upload of a C-contiguous numpy array."""
        check(lib.eh_buffer_write(self._h, c_void_p(arr.ctypes.data), arr.nbytes))

    def read_to_host(self) -> bytes:
        out = ctypes.create_string_buffer(max(self._nbytes, 1))
        check(lib.eh_buffer_read(self._h, out, self._nbytes))
        return out.raw[:self._nbytes]

    def read_array(self, np_dtype, shape=None):
        import numpy as np
        out = np.empty(self._nbytes // np.dtype(np_dtype).itemsize, dtype=np_dtype)
        check(lib.eh_buffer_read(self._h, c_void_p(out.ctypes.data), self._nbytes))
        return out.reshape(shape) if shape is not None else out

    def clone_buffer(self) -> "HipBuffer":
        b = HipBuffer(self.device, self.shape, self.dtype, nbytes=self._nbytes)
        check(lib.eh_buffer_copy(b._h, self._h))
        return b


class HipGraph:
    """The launches of one program run on fixed buffers, replayed as a whole (eh_program_record)."""

    def __init__(self, program, binding):
        self._h = c_void_p()
        self._keep = (program, binding)
        check(lib.eh_program_record(program._h, binding[0], len(program.buffers), byref(self._h)))

    def replay(self, sync: bool = True) -> None:
        check(lib.eh_graph_replay(self._h, 1 if sync else 0))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            lib.eh_graph_release(h)


class HipProgram:
    """A Program AST compiled for a device (`eh_program_*`)."""

    def __init__(self, device: HipDevice, ast, options=None):
        self.device = device
        self._h = c_void_p()
        check(lib.eh_program_compile(device._h, _sexpr(ast), _opts(options), byref(self._h)))
        n = c_int()
        check(lib.eh_program_num_buffers(self._h, byref(n)))
        self.buffers: List[dict] = []
        for i in range(n.value):
            name, role, nb, el = c_char_p(), c_char_p(), c_size_t(), c_int()
            check(lib.eh_program_buffer(self._h, i, byref(name), byref(role), byref(nb), byref(el)))
            self.buffers.append({"name": name.value.decode(), "role": role.value.decode(),
                                 "bytes": nb.value, "elided": bool(el.value)})
        check(lib.eh_program_num_launches(self._h, byref(n)))
        self.launches: List[dict] = []
        for i in range(n.value):
            info = LaunchInfo()
            check(lib.eh_program_launch(self._h, i, byref(info)))
            self.launches.append(_launch_dict(info))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            lib.eh_program_release(h)

    def bind(self, named: Dict[str, HipBuffer]):
        """Handle array for `run` (buffers by table name); keeps the buffers alive."""
        arr = (c_void_p * len(self.buffers))()
        keep = []
        for i, b in enumerate(self.buffers):
            hb = named.get(b["name"])
            arr[i] = hb._h if hb is not None else None
            keep.append(hb)
        return (arr, keep)

    def run(self, binding, sync: bool = True) -> None:
        check(lib.eh_program_execute(self._h, binding[0], len(self.buffers), 1 if sync else 0))

    def record(self, binding) -> "HipGraph":
        """One `run` on this binding captured as a HIP graph; `replay` queues it with one call."""
        return HipGraph(self, binding)

    def execute(self, inputs: Dict[str, HipBuffer]) -> Dict[str, HipBuffer]:
        """Binds inputs by name, allocates the outputs, queues the launches, returns the
        outputs.  Nothing waits here: reads, later programs and the reuse of released memory
        are all ordered behind these launches on the device's stream, so the host can build the
        next step meanwhile.  ECLAT_HIP_SYNC=1 in the environment waits after every program."""
        named = dict(inputs)
        outs = {}
        for b in self.buffers:
            if b["role"] == "output" and b["name"] not in named:
                hb = HipBuffer(self.device, [b["bytes"]], None, nbytes=b["bytes"])
                named[b["name"]] = hb
                outs[b["name"]] = hb
        self.run(self.bind(named), sync=os.environ.get("ECLAT_HIP_SYNC", "0") == "1")
        return outs

    def binary(self, launch: int = 0) -> bytes:
        blob, n = c_void_p(), c_size_t()
        check(lib.eh_program_binary(self._h, launch, byref(blob), byref(n)))
        return ctypes.string_at(blob, n.value)


class HipKernel:
    """One compiled kernel: `Kernel::execute(inputs, outputs)`.  The reference's kernels return when
    the work is done; `sync=False` only queues the launch on the device's stream, which every read
    of a buffer and every reuse of its memory is ordered behind (what the Rust binding does unless
    ECLAT_HIP_SYNC=1)."""

    def __init__(self, device: HipDevice, program_ast, options=None):
        self._prog = HipProgram(device, program_ast, options)

    def execute(self, inputs: Sequence[HipBuffer], outputs: Sequence[HipBuffer], sync: bool = True) -> None:
        ins = (c_void_p * max(len(inputs), 1))(*[b._h for b in inputs])
        outs = (c_void_p * max(len(outputs), 1))(*[b._h for b in outputs])
        check(lib.eh_program_execute_positional(self._prog._h, ins, len(inputs), outs,
                                                len(outputs), 1 if sync else 0))

    def get_binary(self) -> bytes:
        return self._prog.binary(0)

    @property
    def launches(self):
        return self._prog.launches


class HipModule:
    """One entry point of a code object (`compile_from_binary` + `execute_with_sizes`)."""

    def __init__(self, device: HipDevice, blob: bytes, entry: str):
        self.device = device
        self._h = c_void_p()
        buf = (ctypes.c_char * len(blob)).from_buffer_copy(blob)
        check(lib.eh_module_load(device._h, buf, len(blob), entry.encode(), byref(self._h)))

    def launch(self, grid, block, args: Sequence[HipBuffer], lds_bytes: int = 0, sync: bool = True):
        g = (ctypes.c_uint * 3)(*grid)
        b = (ctypes.c_uint * 3)(*block)
        a = (c_void_p * max(len(args), 1))(*[x._h for x in args])
        check(lib.eh_module_launch(self._h, g, b, lds_bytes, a, len(args), 1 if sync else 0))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            lib.eh_module_release(h)


class Event:
    def __init__(self, device: HipDevice):
        self.device = device           # an event must not outlive its device
        self._h = c_void_p()
        check(lib.eh_event_create(device._h, byref(self._h)))

    def record(self) -> None:
        check(lib.eh_event_record(self._h))

    def sync(self) -> None:
        check(lib.eh_event_sync(self._h))

    def elapsed_ms(self, stop: "Event") -> float:
        ms = c_float()
        check(lib.eh_event_elapsed_ms(self._h, stop._h, byref(ms)))
        return ms.value

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            lib.eh_event_release(h)


class HipBackendRegistry:
    """Registered with the front end as kind "hip"."""

    kind = "hip"

    def __init__(self, options=None):
        self.options = options
        self._devices: Dict[int, HipDevice] = {}

    def name(self) -> str:
        return "HIP (gfx950)"

    def is_available(self) -> bool:
        return device_count() > 0

    def supports_runtime(self) -> bool:
        return True

    def list_devices(self) -> List[str]:
        return [f"hip:{i}" for i in range(device_count())]

    def create_device(self, index: int) -> HipDevice:
        if index not in self._devices:
            self._devices[index] = HipDevice(index)
        return self._devices[index]

    def allocate_buffer(self, device: HipDevice, shape, dtype) -> HipBuffer:
        return HipBuffer(device, shape, dtype)

    def compile_ast(self, device: HipDevice, program, signature=None) -> HipKernel:
        return HipKernel(device, program, self.options)

    def compile_program(self, device: HipDevice, program) -> HipProgram:
        return HipProgram(device, program, self.options)


def init(options=None) -> None:
    """Registers the backend with the front end (the reference crates do this
    from a constructor function, `crates/backend-c/src/lib.rs:125-134`)."""
    from .frontend.device import register_backend
    register_backend(HipBackendRegistry(options))
