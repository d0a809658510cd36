"""ctypes binding of libroller_hip.so -- the only way this package reaches the GPU.

It plays the part that CuPy plays in the reference (``cp.cuda.Module``, ``cp.cuda.Event``,
``cp.zeros`` ..., /root/reference/src/roller.py:498-534): device buffers, events, module load and
kernel launch, plus the JIT of the GEMM kernel template.  Every call goes through the C ABI in
``include/roller_hip.h``; a non-zero status becomes a ``HipError`` carrying the library's text,
so the per-hint ``try/except Exception`` of the benchmark sweep (benchmark.py:43-58) keeps
working unchanged.

There is no CPU fallback: if the shared library is missing, ``lib()`` raises.
"""

from __future__ import annotations

import ctypes as C
import os
import subprocess
import sys
from dataclasses import dataclass, fields
from pathlib import Path
from typing import Optional, Sequence

import numpy as np

PKG_DIR = Path(__file__).resolve().parent
CSRC_DIR = PKG_DIR / "csrc"
REPO_ROOT = PKG_DIR.parent
LIB_PATH = PKG_DIR / "libroller_hip.so"
DEFAULT_CACHE_DIR = PKG_DIR / "_cache"
ROCM = Path(os.environ.get("ROCM_PATH", "/opt/rocm"))

RL_ERR_INVALID_ARG = -1001
RL_ERR_COMPILE = -1002
RL_ERR_IO = -1003
RL_ERR_NO_DEVICE = -1004


class HipError(RuntimeError):
    """A call into libroller_hip.so failed; ``status`` is its return value."""

    def __init__(self, status: int, text: str):
        super().__init__(f"[{status}] {text}")
        self.status = status


class DeviceProps(C.Structure):
    _fields_ = [
        ("name", C.c_char * 128),
        ("arch", C.c_char * 64),
        ("compute_units", C.c_int),
        ("wavefront_size", C.c_int),
        ("lds_bytes_per_block", C.c_int),
        ("regs_per_block", C.c_int),
        ("l2_bytes", C.c_int),
        ("clock_khz", C.c_int),
        ("mem_clock_khz", C.c_int),
        ("mem_bus_bits", C.c_int),
        ("total_mem_bytes", C.c_size_t),
    ]


class _GemmConfigC(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "bm", "bn", "bk", "wm", "wn", "mi", "stages", "pad_a", "pad_b", "vec", "edge", "swz",
        "group", "accum", "direct", "trans_b", "streamk")]


class StreamKSchedule(C.Structure):
    """``rl_streamk_schedule``: how a stream-K configuration splits one problem."""
    _fields_ = [("grid", C.c_int), ("k_steps", C.c_int), ("tiles", C.c_int), ("tile_rows", C.c_int), ("tile_cols", C.c_int),
                ("units", C.c_long), ("workspace_bytes", C.c_size_t), ("counter_bytes", C.c_size_t), ("whole_tiles", C.c_int)]


class StreamKSegment(C.Structure):
    """``rl_streamk_segment``: one run of K steps of one tile."""
    _fields_ = [(n, C.c_int) for n in ("tile", "tile_m", "tile_n", "k_begin", "k_end", "pieces",
                                       "first_workgroup", "slot")]


@dataclass(frozen=True)
class GemmConfig:
    """Parameters of one instance of the kernel template (``rl_gemm_config``)."""

    bm: int = 128
    bn: int = 128
    bk: int = 16
    wm: int = 64
    wn: int = 64
    mi: int = 32
    stages: int = 2
    pad_a: int = 4
    pad_b: int = 0
    vec: int = 4
    edge: int = 1
    swz: int = 3
    group: int = 8
    accum: int = 0
    direct: int = 0
    trans_b: int = 0
    streamk: int = 0

    def to_c(self) -> _GemmConfigC:
        return _GemmConfigC(*(getattr(self, f.name) for f in fields(self)))

    @property
    def threads(self) -> int:
        return 64 * (self.bm // self.wm) * (self.bn // self.wn)

    @property
    def lds_bytes(self) -> int:
        b_tile = self.bn * (self.bk + self.pad_b) if self.trans_b else self.bk * (self.bn + self.pad_b)
        return self.lds_buffers * (self.bm * (self.bk + self.pad_a) + b_tile) * 4

    @property
    def lds_buffers(self) -> int:
        """LDS buffers per pipeline depth: 1, 2, 2 (plus a register stage), 3, 4."""
        return self.stages - 1 if self.stages >= 3 else self.stages

    def tag(self) -> str:
        return (f"b{self.bm}x{self.bn}x{self.bk}_w{self.wm}x{self.wn}_mi{self.mi}_s{self.stages}"
                f"_p{self.pad_a}.{self.pad_b}_v{self.vec}_e{self.edge}_z{self.swz}.{self.group}"
                f"_a{self.accum}" + ("_d1" if self.direct else "") + ("_tb" if self.trans_b else "")
                + (f"_sk{self.streamk}" if self.streamk else ""))

    MAX_STAGES = 5


# --------------------------------------------------------------------------------------------
# building and loading the shared library
# --------------------------------------------------------------------------------------------

def build_library(verbose: bool = False) -> Path:
    """Builds libroller_hip.so: csrc/roller_hip.cpp (host code; the kernel template is embedded as text
    and compiled for gfx950 by hiprtc at run time or by ``precompile``) and csrc/roller_scratch.hip
    (hipcc, gfx950: the static scratch array of the launch entry point that allocates nothing)."""
    template = CSRC_DIR / "gemm_f32_mfma.hip"
    obj_dir = REPO_ROOT / "build"
    obj_dir.mkdir(exist_ok=True)
    scratch_obj = obj_dir / "roller_scratch.o"
    cmds = [
        ["hipcc", "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         f"-I{CSRC_DIR}", "-c", str(CSRC_DIR / "roller_scratch.hip"), "-o", str(scratch_obj)],
        ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra",
         "-D__HIP_PLATFORM_AMD__", f"-I{ROCM / 'include'}", f"-I{REPO_ROOT / 'include'}",
         f'-DRL_TEMPLATE_PATH="{template}"', f'-DRL_SK_DECODE_PATH="{CSRC_DIR / "gemm_sk_decode.inc"}"',
         f"-I{CSRC_DIR}", str(CSRC_DIR / "roller_hip.cpp"), str(scratch_obj),
         "-o", str(LIB_PATH), f"-L{ROCM / 'lib'}", "-lamdhip64", "-lhiprtc",
         f"-Wl,-rpath,{ROCM / 'lib'}"],
    ]
    for cmd in cmds:
        if verbose:
            print(" ".join(cmd))
        subprocess.run(cmd, check=True)
    global _lib
    _lib = None
    return LIB_PATH


_lib: Optional[C.CDLL] = None

_SIGNATURES = {
    "rl_init": ([C.c_int], C.c_int),
    "rl_device_info": ([C.POINTER(DeviceProps)], C.c_int),
    "rl_last_error": ([], C.c_char_p),
    "rl_compile": ([C.c_char_p, C.c_char_p, C.POINTER(C.c_char_p), C.c_int, C.POINTER(C.c_void_p),
                    C.POINTER(C.c_size_t), C.POINTER(C.c_void_p)], C.c_int),
    "rl_free_host": ([C.c_void_p], None),
    "rl_module_load": ([C.c_void_p, C.POINTER(C.c_void_p)], C.c_int),
    "rl_module_get_function": ([C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p)], C.c_int),
    "rl_module_unload": ([C.c_void_p], C.c_int),
    "rl_func_set_max_dynamic_lds": ([C.c_void_p, C.c_int], C.c_int),
    "rl_launch": ([C.c_void_p] + [C.c_uint] * 7 + [C.c_void_p, C.POINTER(C.c_void_p), C.c_int], C.c_int),
    "rl_malloc": ([C.POINTER(C.c_void_p), C.c_size_t], C.c_int),
    "rl_free": ([C.c_void_p], C.c_int),
    "rl_memcpy_h2d": ([C.c_void_p, C.c_void_p, C.c_size_t], C.c_int),
    "rl_memcpy_d2h": ([C.c_void_p, C.c_void_p, C.c_size_t], C.c_int),
    "rl_memset": ([C.c_void_p, C.c_int, C.c_size_t], C.c_int),
    "rl_stream_create": ([C.POINTER(C.c_void_p)], C.c_int),
    "rl_stream_destroy": ([C.c_void_p], C.c_int),
    "rl_event_create": ([C.POINTER(C.c_void_p)], C.c_int),
    "rl_event_record": ([C.c_void_p, C.c_void_p], C.c_int),
    "rl_event_sync": ([C.c_void_p], C.c_int),
    "rl_event_elapsed_ms": ([C.c_void_p, C.c_void_p, C.POINTER(C.c_float)], C.c_int),
    "rl_event_destroy": ([C.c_void_p], C.c_int),
    "rl_sync": ([], C.c_int),
    "rl_gemm_template_source": ([], C.c_char_p),
    "rl_gemm_config_check": ([C.POINTER(_GemmConfigC), C.POINTER(C.c_int), C.POINTER(C.c_int)], C.c_int),
    "rl_set_cache_dir": ([C.c_char_p], C.c_int),
    "rl_gemm_precompile": ([C.POINTER(_GemmConfigC), C.POINTER(C.c_size_t)], C.c_int),
    "rl_gemm_plan_create": ([C.POINTER(_GemmConfigC), C.POINTER(C.c_void_p), C.POINTER(C.c_float)], C.c_int),
    "rl_gemm_plan_function": ([C.c_void_p, C.POINTER(C.c_void_p)], C.c_int),
    "rl_gemm_plan_lds_bytes": ([C.c_void_p], C.c_int),
    "rl_gemm_plan_lds_limit": ([C.c_void_p], C.c_int),
    "rl_gemm_plan_threads": ([C.c_void_p], C.c_int),
    "rl_gemm_plan_build_log": ([C.c_void_p], C.c_char_p),
    "rl_gemm_plan_resources": ([C.c_void_p] + [C.POINTER(C.c_int)] * 5, C.c_int),
    "rl_gemm_plans_clear": ([], C.c_int),
    "rl_gemm_plan_launch": ([C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p] + [C.c_int] * 6 + [C.c_void_p], C.c_int),
    "rl_gemm_plan_workspace_bytes": ([C.c_void_p, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)], C.c_int),
    "rl_gemm_plan_launch_ws": ([C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p] + [C.c_int] * 6 + [C.c_void_p, C.c_size_t, C.c_void_p], C.c_int),
    "rl_gemm_plan_launch_static": ([C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p] + [C.c_int] * 6 + [C.c_void_p], C.c_int),
    "rl_gemm_streamk_schedule": ([C.POINTER(_GemmConfigC)] + [C.c_int] * 4 + [C.POINTER(StreamKSchedule)], C.c_int),
    "rl_gemm_streamk_segments": ([C.POINTER(_GemmConfigC)] + [C.c_int] * 5 + [C.POINTER(StreamKSegment), C.c_int, C.POINTER(C.c_int)], C.c_int),
    "rl_gemm_f32": ([C.POINTER(_GemmConfigC), C.c_void_p, C.c_void_p, C.c_void_p] + [C.c_int] * 6 + [C.c_void_p], C.c_int),
}

EXPORTS = tuple(_SIGNATURES)


def lib() -> C.CDLL:
    """The loaded library.  Raises if it has not been built: there is no other GEMM path."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise HipError(RL_ERR_IO, f"{LIB_PATH} is missing; run __graft_entry__.build() "
                                      "(or mlir_roller_amd.hip.build_library()) first")
        handle = C.CDLL(str(LIB_PATH))
        for name, (argtypes, restype) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = handle
        cache = os.environ.get("ROLLER_HIP_CACHE", str(DEFAULT_CACHE_DIR))
        if cache:
            check(handle.rl_set_cache_dir(cache.encode()))
    return _lib


def check(status: int) -> None:
    if status != 0:
        raise HipError(status, lib().rl_last_error().decode(errors="replace"))


_initialised = False


def init(device: int = 0) -> None:
    """Creates the HIP context on ``device`` (once)."""
    global _initialised
    if not _initialised:
        check(lib().rl_init(device))
        _initialised = True


def device_info() -> DeviceProps:
    init()
    props = DeviceProps()
    check(lib().rl_device_info(C.byref(props)))
    return props


def set_cache_dir(path: Optional[os.PathLike]) -> None:
    global _cache_dir_override
    check(lib().rl_set_cache_dir(str(path).encode() if path else None))
    _cache_dir_override = str(path) if path else None


def synchronize() -> None:
    check(lib().rl_sync())


_roctx = None


def _roctx_lib():
    """libroctx64 (ROCm's marker API), or False if it cannot be loaded."""
    global _roctx
    if _roctx is None:
        _roctx = False
        for name in ("libroctx64.so", "libroctx64.so.4", str(ROCM / "lib" / "libroctx64.so")):
            try:
                handle = C.CDLL(name)
                handle.roctxRangePushA.argtypes = [C.c_char_p]
                handle.roctxRangePushA.restype = C.c_int
                handle.roctxRangePop.restype = C.c_int
                _roctx = handle
                break
            except (OSError, AttributeError):
                continue
    return _roctx


class profiler_range:
    """``with profiler_range("name"):`` -- a roctx range that ``rocprofv3 --marker-trace`` shows, the
    counterpart of ``cupyx.profiler.time_range`` (roller.py:556).  Does nothing when the marker
    library is not installed."""

    def __init__(self, name: str):
        self.name = name.encode()
        self.pushed = False

    def __enter__(self):
        lib_ = _roctx_lib()
        if lib_:
            lib_.roctxRangePushA(self.name)
            self.pushed = True
        return self

    def __exit__(self, *exc):
        if self.pushed:
            _roctx_lib().roctxRangePop()
        return False


# --------------------------------------------------------------------------------------------
# device memory, streams, events
# --------------------------------------------------------------------------------------------

class DevicePtr(int):
    """A device address.  An ``int`` in every respect (arithmetic, formatting, ctypes pointer
    arguments) that kernel launches recognise as an address: it is passed as an 8-byte pointer
    whatever its value, where a plain ``int`` is a 4-byte kernel parameter."""

    __slots__ = ()

    def __repr__(self) -> str:
        return f"DevicePtr({int(self):#x})"


class _DataView:
    """``array.data.ptr``, the spelling of CuPy that the reference's launch uses (roller.py:548)."""

    __slots__ = ("ptr",)

    def __init__(self, ptr: int):
        self.ptr = DevicePtr(ptr)


class DeviceArray:
    """A row-major fp32 (or any dtype) array in HBM; frees its allocation when collected.
    ``ptr`` (and ``data.ptr``, as in CuPy) is its device address as a ``DevicePtr``."""

    def __init__(self, shape: Sequence[int], dtype=np.float32):
        init()
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = C.c_void_p()
        check(lib().rl_malloc(C.byref(p), self.nbytes))
        self.ptr = DevicePtr(p.value or 0)

    @property
    def data(self) -> _DataView:
        return _DataView(self.ptr)

    @classmethod
    def from_host(cls, host: np.ndarray) -> "DeviceArray":
        host = np.ascontiguousarray(host)
        out = cls(host.shape, host.dtype)
        out.set(host)
        return out

    @classmethod
    def zeros(cls, shape: Sequence[int], dtype=np.float32) -> "DeviceArray":
        out = cls(shape, dtype)
        out.fill_bytes(0)
        return out

    def set(self, host: np.ndarray) -> None:
        host = np.ascontiguousarray(host, dtype=self.dtype)
        if host.nbytes != self.nbytes:
            raise ValueError(f"host array has {host.nbytes} bytes, device array {self.nbytes}")
        check(lib().rl_memcpy_h2d(self.ptr, host.ctypes.data, self.nbytes))

    def get(self) -> np.ndarray:
        out = np.empty(self.shape, dtype=self.dtype)
        check(lib().rl_memcpy_d2h(out.ctypes.data, self.ptr, self.nbytes))
        return out

    def fill_bytes(self, value: int) -> None:
        check(lib().rl_memset(self.ptr, value, self.nbytes))

    def free(self) -> None:
        if getattr(self, "ptr", 0):
            lib().rl_free(self.ptr)
            self.ptr = DevicePtr(0)

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Stream:
    """A HIP stream of default priority."""

    def __init__(self):
        init()
        p = C.c_void_p()
        check(lib().rl_stream_create(C.byref(p)))
        self.handle = p.value

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                lib().rl_stream_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


def _stream_handle(stream) -> Optional[int]:
    if stream is None:
        return None
    return stream.handle if isinstance(stream, Stream) else int(stream)


class Event:
    """Counterpart of ``cp.cuda.Event`` (roller.py:516-522)."""

    def __init__(self):
        init()
        p = C.c_void_p()
        check(lib().rl_event_create(C.byref(p)))
        self.handle = p.value

    def record(self, stream=None) -> None:
        check(lib().rl_event_record(self.handle, _stream_handle(stream)))

    def synchronize(self) -> None:
        check(lib().rl_event_sync(self.handle))

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                lib().rl_event_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


def get_elapsed_time(start: Event, stop: Event) -> float:
    """Milliseconds between two recorded events (``cp.cuda.get_elapsed_time``, roller.py:580)."""
    ms = C.c_float()
    check(lib().rl_event_elapsed_ms(start.handle, stop.handle, C.byref(ms)))
    return float(ms.value)


# --------------------------------------------------------------------------------------------
# JIT and launch
# --------------------------------------------------------------------------------------------

def template_source() -> str:
    return lib().rl_gemm_template_source().decode()


def compile_source(source: str, name: str = "kernel.hip", options: Sequence[str] = ()) -> tuple[bytes, str]:
    """hiprtc: HIP source -> gfx950 code object.  Returns (code, build log); needs no GPU."""
    opts = (C.c_char_p * max(len(options), 1))(*[o.encode() for o in options])
    code, size, log = C.c_void_p(), C.c_size_t(), C.c_void_p()
    status = lib().rl_compile(source.encode(), name.encode(), opts, len(options), C.byref(code),
                              C.byref(size), C.byref(log))
    text = C.string_at(log.value).decode(errors="replace") if log.value else ""
    if log.value:
        lib().rl_free_host(log)
    if status != 0:
        raise HipError(status, lib().rl_last_error().decode(errors="replace"))
    blob = C.string_at(code.value, size.value)
    lib().rl_free_host(code)
    return blob, text


def code_object_resources(code: bytes) -> dict:
    """Register, spill and scratch figures from the metadata note of a gfx950 code object (the same
    msgpack keys ``rl_gemm_plan_resources`` reads); -1 where a key is missing.  Needs no GPU."""
    def value_after(key: bytes) -> int:
        i = code.find(key)
        if i < 0 or i + len(key) >= len(code):
            return -1
        p = code[i + len(key):i + len(key) + 5]
        if p[0] <= 0x7F:
            return p[0]
        if p[0] == 0xCC and len(p) >= 2:
            return p[1]
        if p[0] == 0xCD and len(p) >= 3:
            return (p[1] << 8) | p[2]
        if p[0] == 0xCE and len(p) >= 5:
            return int.from_bytes(p[1:5], "big")
        return -1
    names = {"vgprs": b".vgpr_count", "agprs": b".agpr_count", "sgprs": b".sgpr_count",
             "vgpr_spills": b".vgpr_spill_count", "sgpr_spills": b".sgpr_spill_count",
             "scratch_bytes": b".private_segment_fixed_size"}
    return {k: value_after(v) for k, v in names.items()}


def compile_config(cfg: "GemmConfig") -> bytes:
    """The kernel template compiled for ``cfg`` through hiprtc, without cache or GPU."""
    options = [f"-D{f.name.upper()}={getattr(cfg, f.name)}" for f in fields(cfg)]
    return compile_source(template_source(), "gemm_f32_mfma.hip", options)[0]


class Module:
    """Counterpart of ``cp.cuda.Module`` (roller.py:504-506)."""

    def __init__(self, code: bytes):
        init()
        self._code = C.create_string_buffer(code, len(code))
        p = C.c_void_p()
        check(lib().rl_module_load(self._code, C.byref(p)))
        self.handle = p.value

    def get_function(self, name: str) -> "Function":
        p = C.c_void_p()
        check(lib().rl_module_get_function(self.handle, name.encode(), C.byref(p)))
        return Function(p.value, owner=self)

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                lib().rl_module_unload(self.handle)
                self.handle = None
        except Exception:
            pass


class Ptr:
    """A raw device address as a kernel argument (``dA.data.ptr`` in the reference,
    roller.py:548): always passed as an 8-byte pointer, whatever its value (NULL included)."""

    __slots__ = ("address",)

    def __init__(self, address: int):
        address = int(address)
        if not 0 <= address < 2**64:
            raise ValueError(f"device address {address:#x} does not fit 64 bits")
        self.address = address

    def __repr__(self) -> str:
        return f"Ptr({self.address:#x})"


def _pack_arg(a):
    """One kernel argument as the ctypes object whose storage ``hipModuleLaunchKernel`` reads.
    The width is decided by the argument's type, never by its value: ``DeviceArray``, ``Ptr``,
    ``DevicePtr`` (what ``array.ptr`` and ``array.data.ptr`` are) and ``c_void_p`` are 8-byte pointers; a Python or numpy integer is a 4-byte ``int``
    (``OverflowError`` if it does not fit -- use ``ctypes.c_long`` for a 64-bit parameter and
    ``Ptr`` for an address); a float is a 4-byte ``float``; ctypes scalars pass through."""
    if isinstance(a, DeviceArray):
        return C.c_void_p(a.ptr)
    if isinstance(a, Ptr):
        return C.c_void_p(a.address)
    if isinstance(a, DevicePtr):
        return C.c_void_p(int(a))
    if isinstance(a, (C._SimpleCData,)):
        return a
    if isinstance(a, (bool, np.bool_)):
        raise TypeError("cannot pass a bool to a kernel; use an int")
    if isinstance(a, (int, np.integer)):
        v = int(a)
        if not -2**31 <= v < 2**31:
            raise OverflowError(f"{v} does not fit a 32-bit int kernel parameter; pass ctypes.c_long(...) for a "
                                "64-bit integer or hip.Ptr(...) for a device address")
        return C.c_int(v)
    if isinstance(a, (float, np.floating)):
        return C.c_float(float(a))
    raise TypeError(f"cannot pass {type(a).__name__} to a kernel")


class Function:
    """A loaded kernel: ``f(grid, block, args, shared_mem=0, stream=None)`` like
    ``cp.cuda.Function.__call__`` (roller.py:545-550)."""

    def __init__(self, handle: int, owner=None):
        self.handle = handle
        self._owner = owner

    def set_max_dynamic_lds(self, nbytes: int) -> None:
        check(lib().rl_func_set_max_dynamic_lds(self.handle, int(nbytes)))

    def __call__(self, grid, block, args, shared_mem: int = 0, stream=None) -> None:
        g = tuple(grid) + (1,) * (3 - len(grid))
        b = tuple(block) + (1,) * (3 - len(block))
        packed = [_pack_arg(a) for a in args]
        argv = (C.c_void_p * max(len(packed), 1))(*[C.cast(C.pointer(p), C.c_void_p) for p in packed])
        check(lib().rl_launch(self.handle, g[0], g[1], g[2], b[0], b[1], b[2], int(shared_mem),
                              _stream_handle(stream), argv, len(packed)))


def config_check(cfg: GemmConfig) -> tuple[int, int]:
    """(dynamic LDS bytes, threads per workgroup) of ``cfg``; raises if the template rejects it."""
    lds, threads = C.c_int(), C.c_int()
    c = cfg.to_c()
    check(lib().rl_gemm_config_check(C.byref(c), C.byref(lds), C.byref(threads)))
    return lds.value, threads.value


def precompile(cfg: GemmConfig) -> int:
    """Compiles ``cfg`` into the on-disk cache without a GPU; returns the code-object size."""
    size = C.c_size_t()
    c = cfg.to_c()
    check(lib().rl_gemm_precompile(C.byref(c), C.byref(size)))
    return size.value


def _address(x) -> int:
    """Device address of a matrix argument of the typed GEMM entry points (their ctypes
    signatures declare pointers, so an int is never mistaken for anything else)."""
    if isinstance(x, DeviceArray):
        return x.ptr
    if isinstance(x, Ptr):
        return x.address
    return int(x)


def _precompile_worker(job: tuple) -> tuple:
    cache_dir, cfg_values = job
    cfg = GemmConfig(*cfg_values)
    try:
        if cache_dir:
            set_cache_dir(cache_dir)
        return cfg_values, precompile(cfg), ""
    except HipError as e:
        return cfg_values, 0, str(e)


_cache_dir_override: Optional[str] = None


def precompile_many(configs: Sequence[GemmConfig], jobs: Optional[int] = None) -> dict:
    """Fills the on-disk cache for ``configs`` with ``jobs`` worker processes (hiprtc is
    single-threaded and needs no GPU; default: the CPUs this process may run on, at most 16).
    The workers are fresh interpreters (``spawn``): a fork of a process that has initialised the
    GPU would inherit its runtime's threads and queues.  They get the parent's cache directory
    explicitly.  Returns ``{config: error text}`` for the ones that failed; the rest are in the cache."""
    import concurrent.futures as cf
    import multiprocessing as mp

    todo = list(dict.fromkeys(configs))
    if jobs is None:
        jobs = min(16, len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1))
    lib()
    cache_dir = _cache_dir_override or os.environ.get("ROLLER_HIP_CACHE", str(DEFAULT_CACHE_DIR))
    work = [(cache_dir, tuple(getattr(c, f.name) for f in fields(c))) for c in todo]
    failed = {}
    # a spawned worker re-imports the parent's main module by path; a parent that was fed from a pipe or
    # typed at the prompt has none, and its workers would die on start
    main_file = getattr(sys.modules.get("__main__"), "__file__", None)
    spawnable = main_file is None or os.path.exists(main_file)
    if jobs <= 1 or len(todo) <= 1 or not spawnable:
        results = list(map(_precompile_worker, work))
    else:
        with cf.ProcessPoolExecutor(max_workers=min(jobs, len(todo)), mp_context=mp.get_context("spawn")) as pool:
            results = list(pool.map(_precompile_worker, work, chunksize=4))
    for vals, _, err in results:
        if err:
            failed[GemmConfig(*vals)] = err
    return failed


class GemmPlan:
    """One compiled and loaded instance of the kernel template (``rl_gemm_plan``)."""

    def __init__(self, cfg: GemmConfig):
        init()
        self.cfg = cfg
        p, ms = C.c_void_p(), C.c_float()
        c = cfg.to_c()
        check(lib().rl_gemm_plan_create(C.byref(c), C.byref(p), C.byref(ms)))
        self.handle = p.value
        self.compile_ms = float(ms.value)
        self.lds_bytes = lib().rl_gemm_plan_lds_bytes(self.handle)
        self.lds_limit = lib().rl_gemm_plan_lds_limit(self.handle)
        self.threads = lib().rl_gemm_plan_threads(self.handle)

    @property
    def function(self) -> Function:
        p = C.c_void_p()
        check(lib().rl_gemm_plan_function(self.handle, C.byref(p)))
        return Function(p.value, owner=self)

    def resources(self) -> dict:
        vals = [C.c_int() for _ in range(5)]
        check(lib().rl_gemm_plan_resources(self.handle, *[C.byref(v) for v in vals]))
        return dict(zip(("vgprs", "agprs", "sgprs", "spilled", "scratch_bytes"), (v.value for v in vals)))

    def build_log(self) -> str:
        """What hiprtc printed for this kernel ("" if nothing, or if it came from the disk cache)."""
        return (lib().rl_gemm_plan_build_log(self.handle) or b"").decode(errors="replace")

    def workspace_bytes(self, M: int, N: int, K: int) -> tuple[int, int]:
        """(workspace bytes, of which arrival counters that must start at zero) that a launch of this
        plan on an M x N x K problem needs; (0, 0) unless the plan is a stream-K one."""
        total, counters = C.c_size_t(), C.c_size_t()
        check(lib().rl_gemm_plan_workspace_bytes(self.handle, M, N, K, C.byref(total), C.byref(counters)))
        return total.value, counters.value

    def launch(self, A, B, Cm, M: int, N: int, K: int, lda: Optional[int] = None,
               ldb: Optional[int] = None, ldc: Optional[int] = None, stream=None, workspace=None) -> None:
        """Enqueues the GEMM.  ``workspace`` (stream-K plans only) replaces the workspace that the
        library keeps per stream: a ``DeviceArray``, or ``"static"`` for the library's fixed scratch
        array (``rl_gemm_plan_launch_static``: no allocation on any path, a limited size)."""
        ptr = _address
        width_b = K if self.cfg.trans_b else N
        dims = (M, N, K, K if lda is None else lda, width_b if ldb is None else ldb, N if ldc is None else ldc)
        if workspace == "static":
            check(lib().rl_gemm_plan_launch_static(self.handle, ptr(A), ptr(B), ptr(Cm), *dims, _stream_handle(stream)))
        elif workspace is None:
            check(lib().rl_gemm_plan_launch(self.handle, ptr(A), ptr(B), ptr(Cm), *dims, _stream_handle(stream)))
        else:
            check(lib().rl_gemm_plan_launch_ws(self.handle, ptr(A), ptr(B), ptr(Cm), *dims, ptr(workspace),
                                               workspace.nbytes, _stream_handle(stream)))


def streamk_schedule(cfg: GemmConfig, M: int, N: int, K: int, compute_units: int = 256) -> StreamKSchedule:
    """How ``cfg`` (a stream-K configuration) splits an M x N x K problem; host arithmetic, no GPU."""
    out, c = StreamKSchedule(), cfg.to_c()
    check(lib().rl_gemm_streamk_schedule(C.byref(c), M, N, K, compute_units, C.byref(out)))
    return out


def streamk_segments(cfg: GemmConfig, M: int, N: int, K: int, workgroup: int, compute_units: int = 256) -> list:
    """The segments that (logical) workgroup ``workgroup`` of a stream-K launch works, in order."""
    c, count = cfg.to_c(), C.c_int()
    buf = (StreamKSegment * 64)()
    check(lib().rl_gemm_streamk_segments(C.byref(c), M, N, K, compute_units, workgroup, buf, 64, C.byref(count)))
    if count.value > 64:
        buf = (StreamKSegment * count.value)()
        check(lib().rl_gemm_streamk_segments(C.byref(c), M, N, K, compute_units, workgroup, buf, count.value, C.byref(count)))
    return [buf[i] for i in range(count.value)]


def gemm_f32(cfg: GemmConfig, A, B, Cm, M: int, N: int, K: int, lda=None, ldb=None, ldc=None,
             stream=None) -> None:
    """``rl_gemm_f32``: plan lookup (JIT on first use) + launch in one call."""
    init()
    ptr = _address
    c = cfg.to_c()
    width_b = K if cfg.trans_b else N
    check(lib().rl_gemm_f32(C.byref(c), ptr(A), ptr(B), ptr(Cm), M, N, K,
                            K if lda is None else lda, width_b if ldb is None else ldb,
                            N if ldc is None else ldc, _stream_handle(stream)))
