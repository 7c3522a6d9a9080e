"""`HIP` device for the jsgrad Device API: registry, Buffer, Allocator, Program, Compiler.

Mirrors the contracts of the reference so that code written against them reads the same:
  Device.get / canonicalize            /root/reference/jsgrad/device.ts:9-44
  Buffer                               /root/reference/jsgrad/device.ts:66-172
  Allocator / Program / Compiler / Compiled   /root/reference/jsgrad/runtime/allocator.ts:28-47,99-139,166-191
The template for an FFI-backed device is /root/reference/jsgrad/runtime/ops_dawn.ts:234-307.
Everything below calls libjsgrad_hip.so; there is no CPU implementation behind it.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
import tempfile

import numpy as np

from . import diskcache, ffi
from .ffi import HipError, check

DTYPES = {"float32": (np.float32, ffi.F32), "float16": (np.float16, ffi.F16), "int8": (np.int8, None), "uint8": (np.uint8, None),
          "int32": (np.int32, None), "int16": (np.int16, None),
          # bfloat16 has no numpy type: the 16 bits travel as uint16 and only jsgrad_hip_cast ever interprets them
          "bfloat16": (np.uint16, ffi.BF16)}


def itemsize(dtype: str) -> int:
    return np.dtype(DTYPES[dtype][0]).itemsize


class HIPAllocator:
    """Allocator<bigint>: buffers are raw device addresses (allocator.ts:28-47)."""

    def __init__(self, lib):
        self.lib = lib

    def alloc(self, size: int, options=None) -> int:
        if size <= 0:
            raise ValueError(f"alloc size must be positve, getting {size}")
        return self._alloc(size, options)

    def free(self, opaque: int, size: int = 0, options=None) -> None:
        self._free(opaque, options)

    def _alloc(self, size: int, options=None) -> int:
        out = C.c_void_p()
        check(self.lib.jsgrad_hip_malloc(size, C.byref(out)))
        return out.value

    def _free(self, opaque: int, options=None) -> None:
        check(self.lib.jsgrad_hip_free(opaque))

    def free_cache(self) -> None:
        """LRUAllocator.free_cache (allocator.ts:65-70).  The cache itself lives in the library, behind _alloc/_free: a freed
        block waits there for the next request of its size class, and `free` (called from Buffer finalisers) never waits."""
        check(self.lib.jsgrad_hip_free_cache())

    def mem_info(self) -> tuple[int, int]:
        """(bytes handed out, bytes lying idle in the cache)."""
        live, idle = C.c_size_t(0), C.c_size_t(0)
        check(self.lib.jsgrad_hip_mem_info(C.byref(live), C.byref(idle)))
        return live.value, idle.value

    def _copyin(self, dest: int, src) -> None:
        mv = np.ascontiguousarray(src)
        check(self.lib.jsgrad_hip_copyin(dest, mv.ctypes.data_as(C.c_void_p), mv.nbytes))

    def _copyout(self, dest: np.ndarray, src: int) -> None:
        assert dest.flags["C_CONTIGUOUS"]
        check(self.lib.jsgrad_hip_copyout(dest.ctypes.data_as(C.c_void_p), src, dest.nbytes))

    def _offset(self, buf: int, size: int, offset: int) -> int:
        return buf + offset

    def _transfer(self, dest: int, src: int, sz: int, src_dev=None, dest_dev=None) -> None:
        check(self.lib.jsgrad_hip_copy(dest, src, sz))


class HIPProgram:
    """Program (allocator.ts:99-107): `lib` is a gfx950 code object, `call` launches one kernel."""

    def __init__(self, lib, name: str, image: bytes):
        if not image:
            raise ValueError("Lib is empty")
        if not name:
            raise ValueError("Name can't be undefined")
        self.lib, self.name, self.image = lib, name, image
        mod, fn = C.c_void_p(), C.c_void_p()
        self._keep = C.create_string_buffer(image, len(image))
        check(lib.jsgrad_hip_module_load(self._keep, len(image), C.byref(mod)))
        self._mod = mod
        check(lib.jsgrad_hip_module_get(mod, name.encode(), C.byref(fn)))
        self._fn = fn

    def call(self, bufs: list[int], global_size=(1, 1, 1), local_size=(1, 1, 1), vals=(), wait: bool = False):
        """Returns seconds when wait is set (the contract engine/realize.ts:62-80 relies on)."""
        g = (C.c_uint32 * 3)(*[int(v) for v in global_size])
        l = (C.c_uint32 * 3)(*[int(v) for v in local_size])
        pb = (C.c_void_p * max(1, len(bufs)))(*bufs)
        pv = (C.c_int32 * max(1, len(vals)))(*[int(v) for v in vals])
        secs = C.c_double(0.0)
        check(self.lib.jsgrad_hip_launch(self._fn, g, l, pb, len(bufs), pv, len(vals), int(wait), C.byref(secs)))
        return secs.value if wait else None

    def __del__(self):
        try:
            if getattr(self, "_mod", None):
                self.lib.jsgrad_hip_module_unload(self._mod)
        except Exception:
            pass


class HIPCompiler:
    """Compiler (allocator.ts:123-139) for generic (non-Llama) kernels: HIP source -> gfx950 code object.
    The CPU counterpart shells out to clang (ops_clang.ts:12-25); this one shells out to hipcc --genco."""

    FLAGS = ["-O3", "-include", "hip/hip_runtime.h", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

    def __init__(self, arch: str = "gfx950", hipcc: str = "/opt/rocm/bin/hipcc", cachekey: str | None = "auto"):
        self.arch, self.hipcc = arch, hipcc
        if cachekey == "auto":
            # one table per (architecture, flags, compiler): a code object made for another of these must never be loaded
            cachekey = f"compile_hip_{arch}_{self._toolchain_id()}"
        # Compiler's constructor (allocator.ts:125-127): no key, no cache
        self.cachekey = None if os.environ.get("DISABLE_COMPILER_CACHE") else cachekey
        self.cache: dict[str, bytes] = {}
        self.compiles = 0       # hipcc runs of this object (tests and DEBUG output)

    def _toolchain_id(self) -> str:
        """Eight hex digits over the flags and the compiler's own version line (empty where hipcc cannot be run: the
        compile itself will say so)."""
        import hashlib
        try:
            ver = subprocess.run([self.hipcc, "--version"], capture_output=True, text=True, timeout=60).stdout
        except (OSError, subprocess.SubprocessError):
            ver = ""
        return hashlib.sha256((" ".join(self.FLAGS) + "\n" + ver).encode()).hexdigest()[:8]

    def compile(self, src: str) -> bytes:
        self.compiles += 1
        with tempfile.TemporaryDirectory() as d:
            code, out = os.path.join(d, "k.hip"), os.path.join(d, "k.co")
            with open(code, "w") as f:
                f.write(src)
            r = subprocess.run([self.hipcc, "--genco", f"--offload-arch={self.arch}", *self.FLAGS, code, "-o", out], capture_output=True, text=True)
            if r.returncode != 0:
                raise CompileError(r.stderr)
            with open(out, "rb") as f:
                return f.read()

    def compile_cached(self, src: str) -> bytes:
        """Compiler.compile_cached (allocator.ts:129-137): the code object comes from the disk cache when this source was
        compiled before, by this process or an earlier one; in front of it, a dictionary for this process."""
        if src in self.cache:
            return self.cache[src]
        lib = diskcache.disk_get(self.cachekey, src) if self.cachekey else None
        if lib is None:
            if os.environ.get("ASSERT_COMPILE"):
                raise RuntimeError(f"tried to compile with ASSERT_COMPILE set\n{src}")
            lib = self.compile(src)
            if self.cachekey is not None:
                diskcache.disk_put(self.cachekey, src, lib)
        self.cache[src] = bytes(lib)
        return self.cache[src]


class CompileError(Exception):
    pass


class HIP:
    """Compiled('HIP') (allocator.ts:166-191): allocator + compiler + runtime; `init` is idempotent and lazy."""

    def __init__(self, device: str = "HIP"):
        self.device = device
        self.index = int(device.split(":")[1]) if ":" in device else 0
        self.lib = ffi.load()
        self.allocator = HIPAllocator(self.lib)
        self.compiler = HIPCompiler()
        self._ready = False

    def init(self) -> "HIP":
        if not self._ready:
            check(self.lib.jsgrad_hip_init(self.index))
            self._ready = True
        return self

    def runtime(self, name: str, image: bytes) -> HIPProgram:
        self.init()
        return HIPProgram(self.lib, name, image)

    def synchronize(self) -> None:
        check(self.lib.jsgrad_hip_sync())

    @property
    def name(self) -> str:
        buf = C.create_string_buffer(256)
        check(self.lib.jsgrad_hip_device_name(buf, 256))
        return buf.value.decode()

    @property
    def cu_count(self) -> int:
        n = C.c_int(0)
        check(self.lib.jsgrad_hip_cu_count(C.byref(n)))
        return n.value


class _Device:
    """Device registry (device.ts:9-44).  `HIP` is the only entry: one backend, no dispatch."""
    DEVICES = {"HIP": HIP}

    def __init__(self):
        self.opened: dict[str, HIP] = {}

    @property
    def DEFAULT(self) -> str:
        return os.environ.get("DEVICE") or os.environ.get("D") or "HIP"

    def canonicalize(self, device: str | None = None) -> str:
        if device is None:
            return self.DEFAULT
        d = device.split(":", 1)[0].upper()
        return d + device[len(d):].replace(":0", "")

    def get(self, device: str) -> HIP:
        if device in self.opened:
            return self.opened[device]
        ix = self.canonicalize(device)
        cls = self.DEVICES.get(ix.split(":")[0].upper())
        if cls is None:
            raise ValueError(f"No device for {ix}")
        dev = cls(ix)
        self.opened[device] = dev
        return dev

    def default(self) -> HIP:
        return self.get(self.DEFAULT)


Device = _Device()


class Buffer:
    """Buffer (device.ts:66-172): a typed, lazily allocated span of device memory, or a view into one."""

    def __init__(self, device: str, size: int, dtype: str, base: "Buffer | None" = None, offset: int = 0, initial_value=None, preallocate: bool = False):
        self.device, self.size, self.dtype, self._base, self.offset = device, int(size), dtype, base, offset
        self._buf: int | None = None
        self.allocator: HIPAllocator | None = None
        if base is None and offset != 0:
            raise ValueError("base buffers can't have offset")
        if base is not None and base._base is not None:
            raise ValueError("base can't have a base")
        if initial_value is not None:
            self.allocate()
            self.copyin(initial_value)
        if preallocate:
            self.ensure_allocated()

    @property
    def base(self) -> "Buffer":
        return self._base if self._base is not None else self

    @property
    def nbytes(self) -> int:
        return self.size * itemsize(self.dtype)

    def is_allocated(self) -> bool:
        return self._buf is not None

    def ensure_allocated(self) -> "Buffer":
        return self if self.is_allocated() else self.allocate()

    def allocate(self) -> "Buffer":
        if self.is_allocated():
            raise RuntimeError("can't allocate already allocated buffer")
        dev = Device.get(self.device).init()
        self.allocator = dev.allocator
        if self._base is not None:
            self._base.ensure_allocated()
            self._buf = self.allocator._offset(self._base._buf, self.nbytes, self.offset)
        else:
            self._buf = self.allocator.alloc(self.nbytes)
        return self

    def deallocate(self) -> None:
        if not self.is_allocated():
            raise RuntimeError("buffer must be allocated to deallocate")
        if self._base is None:
            self.allocator.free(self._buf, self.nbytes)
        self._buf = None

    def __del__(self):
        try:
            if self._buf is not None and self._base is None:
                self.allocator.free(self._buf, self.nbytes)
        except Exception:
            pass

    @property
    def ptr(self) -> int:
        return self.ensure_allocated()._buf

    def copyin(self, mv) -> "Buffer":
        mv = np.ascontiguousarray(mv)
        if mv.nbytes != self.nbytes:
            raise ValueError(f"size mismatch, {mv.nbytes} != {self.dtype} {self.size}")
        if not self.is_allocated():
            raise RuntimeError("can't copyin to unallocated buffer")
        self.allocator._copyin(self._buf, mv)
        return self

    def copyout(self, mv: np.ndarray) -> np.ndarray:
        if mv.nbytes != self.nbytes:
            raise ValueError(f"size mismatch, {mv.nbytes} != {self.dtype} {self.size}")
        if not self.is_allocated():
            raise RuntimeError("can't copyout unallocated buffer")
        self.allocator._copyout(mv, self._buf)
        return mv

    def as_buffer(self) -> np.ndarray:
        """Host copy as a flat numpy array of the buffer's dtype."""
        return self.copyout(np.empty(self.size, DTYPES[self.dtype][0]))

    def view(self, size: int, dtype: str, offset: int) -> "Buffer":
        if offset >= self.nbytes:
            raise ValueError("offset must be less than nbytes")
        if self._base is not None:
            return Buffer(self.device, size, dtype, base=self._base, offset=self.offset + offset)
        return Buffer(self.device, size, dtype, base=self, offset=offset)
