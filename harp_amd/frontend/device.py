"""Backend registry and default-device selection.

Host-side mirror of the reference's `src/backend/device.rs` (`BackendRegistry`
`:83-171`, `register_backend` `:180-190`, device-string parsing `:357-366`,
`:504-528`) and `src/backend/global.rs` (default device `:76-148`,
`allocate_buffer_on_default_device` `:182`, `compile_ast_with_cache`
`:243-360`).  A backend object provides:

    kind -> str                      name() -> str        is_available() -> bool
    create_device(index) -> device   list_devices() -> [str]
    allocate_buffer(device, shape, dtype) -> Buffer      (zero-filled)
    compile_ast(device, program_ast, signature) -> Kernel

Buffer: shape, dtype, byte_len(), read_to_host() -> bytes,
write_from_host(bytes), clone_buffer().  Kernel: execute(inputs, outputs).
A backend may additionally provide compile_program(device, program_ast) for
whole-program compilation (cross-kernel fusion); the executor uses it when
present.
"""

from __future__ import annotations

import threading
from collections import OrderedDict
from typing import Dict, List, Optional, Tuple


class DeviceError(Exception):
    pass


_BACKENDS: "OrderedDict[str, object]" = OrderedDict()
_lock = threading.RLock()
_tls = threading.local()

# kernel cache (cache/store.rs:116-168): LRU of 1024 compiled kernels
_CACHE_CAPACITY = 1024
_kernel_cache: "OrderedDict[Tuple[str, str, int], object]" = OrderedDict()
_program_cache: "OrderedDict[tuple, object]" = OrderedDict()
_cache_stats = {"hits": 0, "misses": 0, "entries": 0, "evictions": 0}


def register_backend(backend) -> None:
    """Later registrations of the same kind are ignored (device.rs:180-190)."""
    with _lock:
        if backend.kind not in _BACKENDS:
            _BACKENDS[backend.kind] = backend


def registered_backends() -> List[str]:
    return list(_BACKENDS.keys())


def parse_device_str(s: str) -> Tuple[str, int]:
    """'hip', 'hip:0', 'c' ... (device.rs:504-528)."""
    s = s.strip().lower()
    if ":" in s:
        name, idx = s.split(":", 1)
        try:
            index = int(idx)
        except ValueError:
            raise DeviceError(f"Invalid device index: {idx}")
    else:
        name, index = s, 0
    if not name:
        raise DeviceError("Empty device string")
    return name, index


class EclatDevice:
    def __init__(self, device_str: str):
        kind, index = parse_device_str(device_str)
        with _lock:
            backend = _BACKENDS.get(kind)
        if backend is None:
            raise DeviceError(f"Backend '{kind}' is not registered "
                              f"(registered: {registered_backends()})")
        if not backend.is_available():
            raise DeviceError(f"Backend '{kind}' is not available on this system")
        self.kind = kind
        self.index = index
        self.backend = backend
        self.device = backend.create_device(index)

    def allocate_buffer(self, shape, dtype):
        return self.backend.allocate_buffer(self.device, list(shape), dtype)

    def compile_ast(self, program, signature=None):
        return self.backend.compile_ast(self.device, program, signature)

    def supports_program(self) -> bool:
        return hasattr(self.backend, "compile_program")

    def compile_program(self, program):
        return self.backend.compile_program(self.device, program)

    def set_as_default(self) -> None:
        _tls.device = self


def set_device_str(device_str: str) -> None:
    EclatDevice(device_str).set_as_default()


def set_device(device: EclatDevice) -> None:
    device.set_as_default()


def clear_default_device() -> None:
    _tls.device = None


def get_default_device() -> Optional[EclatDevice]:
    return getattr(_tls, "device", None)


def has_default_device() -> bool:
    return get_default_device() is not None


def get_default_device_kind() -> str:
    d = get_default_device()
    return d.kind if d is not None else "none"


def allocate_buffer_on_default_device(shape, dtype):
    d = get_default_device()
    if d is None:
        raise DeviceError("No default device set")
    return d.allocate_buffer(shape, dtype)


def compile_ast_with_cache(program, signature=None):
    """Key = AST text + device kind + device identity (cache/mod.rs:24-31)."""
    d = get_default_device()
    if d is None:
        raise DeviceError("No default device set")
    key = (program.to_sexpr(), d.kind, id(d.device))
    with _lock:
        hit = _kernel_cache.get(key)
        if hit is not None:
            _kernel_cache.move_to_end(key)
            _cache_stats["hits"] += 1
            return hit
        _cache_stats["misses"] += 1
    kernel = d.compile_ast(program, signature)
    with _lock:
        _kernel_cache[key] = kernel
        while len(_kernel_cache) > _CACHE_CAPACITY:
            _kernel_cache.popitem(last=False)
            _cache_stats["evictions"] += 1
        _cache_stats["entries"] = len(_kernel_cache)
    return kernel


_PROGRAM_CACHE_CAPACITY = 64          # whole programs keep their temporaries resident,
_PROGRAM_CACHE_BYTES = 32 << 30       # so the cache is also bounded by what they hold on the device


def _resident_bytes(compiled) -> int:
    """Device memory a cached program keeps between runs (its temporaries)."""
    return sum(b["bytes"] for b in getattr(compiled, "buffers", ())
               if b.get("role") == "temp" and not b.get("elided"))


def compile_program_with_cache(program):
    """Whole-program counterpart of `compile_ast_with_cache`, same key.  A training loop
    realizes the same Program every step: a hit skips rendering, module loading and the
    allocation of the program's temporaries.  Hits and misses count in the same statistics."""
    d = get_default_device()
    if d is None:
        raise DeviceError("No default device set")
    key = ("program", program.to_sexpr(), d.kind, id(d.device))
    with _lock:
        hit = _program_cache.get(key)
        if hit is not None:
            _program_cache.move_to_end(key)
            _cache_stats["hits"] += 1
            return hit
        _cache_stats["misses"] += 1
    compiled = d.compile_program(program)
    with _lock:
        _program_cache[key] = compiled
        while len(_program_cache) > 1 and (len(_program_cache) > _PROGRAM_CACHE_CAPACITY or
                                           sum(_resident_bytes(p) for p in _program_cache.values())
                                           > _PROGRAM_CACHE_BYTES):
            _program_cache.popitem(last=False)
            _cache_stats["evictions"] += 1
    return compiled


def cache_stats() -> Dict[str, int]:
    with _lock:
        return dict(_cache_stats)


def clear_cache() -> None:
    with _lock:
        _kernel_cache.clear()
        _program_cache.clear()
        for k in _cache_stats:
            _cache_stats[k] = 0
