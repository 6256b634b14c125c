"""ctypes binding of ``libcleave_hip.so`` (the C ABI declared in ``include/cleave_hip.h``).

This is the only place the Python side touches the HIP runtime: everything above it passes
source text, raw device pointers and sizes.  There is no fallback: if the library is not
built the loader raises ``BackendUnavailable``.
"""

from __future__ import annotations

import ctypes
import os
import threading
from pathlib import Path

from ..core.errors import BackendUnavailable, CompileError, LdsExceeded

LIB_NAME = "libcleave_hip.so"
CSRC_DIR = Path(__file__).resolve().parent.parent / "csrc"
ABI_VERSION = 1

CHIP_OK, CHIP_ERR_INVALID, CHIP_ERR_COMPILE, CHIP_ERR_RUNTIME, CHIP_ERR_LDS = range(5)

# Names every build of the library must export; checked at load and by the CPU test-suite.
EXPORTS = (
    "chip_abi_version", "chip_last_error", "chip_device_count", "chip_device_info_get",
    "chip_compile", "chip_free", "chip_module_load", "chip_module_unload", "chip_get_function",
    "chip_function_attributes", "chip_launch", "chip_launch_seq", "chip_launch_seq_fixed_scratch",
    "chip_time_launches", "chip_time_graph",
)
FIXED_SCRATCH_BYTES = 64 << 20      # CHIP_FIXED_SCRATCH_BYTES of the header

# Options every kernel is compiled with.  Packed-fp32 instruction selection is switched off:
# some of its forms have produced silently wrong results on this hardware generation.
BASE_OPTIONS = ("-O3", "-std=c++17", "-fno-math-errno", "-ffp-contract=fast",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops")


class DeviceInfo(ctypes.Structure):
    _fields_ = [
        ("abi_version", ctypes.c_int32), ("device", ctypes.c_int32),
        ("compute_units", ctypes.c_int32), ("wavefront_size", ctypes.c_int32),
        ("max_threads_per_block", ctypes.c_int32), ("lds_bytes_per_block", ctypes.c_int32),
        ("regs_per_block", ctypes.c_int32), ("clock_khz", ctypes.c_int32),
        ("memory_clock_khz", ctypes.c_int32), ("memory_bus_bits", ctypes.c_int32),
        ("l2_bytes", ctypes.c_int32), ("reserved0", ctypes.c_int32),
        ("total_memory_bytes", ctypes.c_uint64),
        ("arch_name", ctypes.c_char * 64), ("name", ctypes.c_char * 128), ("uuid", ctypes.c_char * 40),
    ]


class FuncAttr(ctypes.Structure):
    _fields_ = [("num_regs", ctypes.c_int32), ("static_lds_bytes", ctypes.c_int32),
                ("scratch_bytes", ctypes.c_int32), ("max_threads_per_block", ctypes.c_int32)]


class LaunchDesc(ctypes.Structure):
    _fields_ = [("fn", ctypes.c_void_p), ("grid", ctypes.c_uint32 * 3), ("block", ctypes.c_uint32 * 3),
                ("lds_bytes", ctypes.c_uint32), ("nargs", ctypes.c_int32),
                ("args", ctypes.POINTER(ctypes.c_void_p))]


class ScratchArg(ctypes.Structure):
    _fields_ = [("launch", ctypes.c_int32), ("arg", ctypes.c_int32), ("offset", ctypes.c_uint64)]


_lock = threading.Lock()
_lib = None


def library_path() -> Path:
    override = os.environ.get("CLEAVE_HIP_LIBRARY")
    return Path(override) if override else CSRC_DIR / LIB_NAME


def available() -> bool:
    return library_path().is_file()


def load():
    """The loaded library (cached).  Raises ``BackendUnavailable`` when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = library_path()
        if not path.is_file():
            raise BackendUnavailable(
                f"{path} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C cleave_amd/csrc`; there is no fallback path")
        # PyTorch bundles its own HIP runtime under the same sonames as the system one.  A
        # process must end up with exactly one of them: importing torch first makes the
        # dynamic loader resolve this library's libamdhip64 / libhiprtc to the copies torch
        # already mapped (the other order leaves torch unable to see the GPU).
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        try:
            lib = ctypes.CDLL(str(path))
        except OSError as e:
            raise BackendUnavailable(f"cannot load {path}: {e}") from e
        missing = [n for n in EXPORTS if not hasattr(lib, n)]
        if missing:
            raise BackendUnavailable(f"{path} does not export {missing}")
        _declare(lib)
        if lib.chip_abi_version() != ABI_VERSION:
            raise BackendUnavailable(f"{path} has ABI {lib.chip_abi_version()}, expected {ABI_VERSION}")
        _lib = lib
    return _lib


def _declare(lib):
    c = ctypes
    lib.chip_abi_version.restype = c.c_int
    lib.chip_last_error.restype = c.c_char_p
    lib.chip_device_count.restype = c.c_int
    lib.chip_device_info_get.argtypes = [c.c_int, c.POINTER(DeviceInfo)]
    lib.chip_compile.argtypes = [c.c_char_p, c.c_char_p, c.c_char_p, c.POINTER(c.c_char_p), c.c_int,
                                 c.POINTER(c.c_void_p), c.POINTER(c.c_size_t), c.POINTER(c.c_void_p)]
    lib.chip_free.argtypes = [c.c_void_p]
    lib.chip_free.restype = None
    lib.chip_module_load.argtypes = [c.c_void_p, c.c_size_t, c.POINTER(c.c_void_p)]
    lib.chip_module_unload.argtypes = [c.c_void_p]
    lib.chip_get_function.argtypes = [c.c_void_p, c.c_char_p, c.POINTER(c.c_void_p)]
    lib.chip_function_attributes.argtypes = [c.c_void_p, c.POINTER(FuncAttr)]
    lib.chip_launch.argtypes = [c.c_void_p, c.POINTER(c.c_uint32), c.POINTER(c.c_uint32), c.c_uint32,
                                c.c_void_p, c.POINTER(c.c_void_p), c.c_int]
    lib.chip_launch_seq.argtypes = [c.POINTER(LaunchDesc), c.c_int, c.c_void_p]
    lib.chip_launch_seq_fixed_scratch.argtypes = [c.POINTER(LaunchDesc), c.c_int, c.c_void_p, c.POINTER(ScratchArg),
                                                  c.c_int, c.c_uint64, c.c_int]
    lib.chip_time_launches.argtypes = [c.POINTER(LaunchDesc), c.c_int, c.c_void_p, c.c_int, c.c_int, c.c_int,
                                       c.POINTER(c.POINTER(c.c_void_p)), c.POINTER(c.c_float)]
    lib.chip_time_graph.argtypes = [c.POINTER(LaunchDesc), c.c_int, c.c_void_p, c.c_int, c.c_int, c.c_int, c.c_int,
                                    c.POINTER(c.POINTER(c.c_void_p)), c.POINTER(c.c_float)]


def last_error() -> str:
    return (load().chip_last_error() or b"").decode("utf-8", "replace")


class HipError(RuntimeError):
    def __init__(self, status: int, text: str):
        super().__init__(text)
        self.status = status


def _check(status: int, what: str):
    if status == CHIP_OK:
        return
    text = f"{what}: {last_error()}"
    if status == CHIP_ERR_LDS:
        raise LdsExceeded(text)
    if status == CHIP_ERR_COMPILE:
        raise CompileError(text)
    raise HipError(status, text)


def device_count() -> int:
    n = load().chip_device_count()
    return max(0, n)


def device_info(dev: int = 0) -> dict:
    info = DeviceInfo()
    _check(load().chip_device_info_get(dev, ctypes.byref(info)), "chip_device_info_get")
    out = {}
    for name, _ in DeviceInfo._fields_:
        v = getattr(info, name)
        out[name] = v.decode("utf-8", "replace") if isinstance(v, bytes) else v
    return out


def compile_source(source: str, name: str = "kernel.hip", arch: str = "gfx950", options=()) -> tuple[bytes, str]:
    """``(code object bytes, compiler log)``.  Needs no GPU."""
    lib = load()
    opts = [o.encode() for o in (*BASE_OPTIONS, *options)]
    arr = (ctypes.c_char_p * len(opts))(*opts)
    code, size, log = ctypes.c_void_p(), ctypes.c_size_t(), ctypes.c_void_p()
    status = lib.chip_compile(source.encode(), name.encode(), arch.encode(), arr, len(opts),
                              ctypes.byref(code), ctypes.byref(size), ctypes.byref(log))
    text = ""
    if log.value:
        text = ctypes.string_at(log.value).decode("utf-8", "replace")
        lib.chip_free(log)
    if status != CHIP_OK:
        if code.value:
            lib.chip_free(code)
        _check(status, "chip_compile")
    blob = ctypes.string_at(code.value, size.value)
    lib.chip_free(code)
    return blob, text


class Module:
    """A loaded code object; function handles die with it."""

    def __init__(self, code: bytes):
        self._code = code  # keep the bytes alive as long as the module
        self._handle = ctypes.c_void_p()
        buf = ctypes.create_string_buffer(code, len(code))
        _check(load().chip_module_load(buf, len(code), ctypes.byref(self._handle)), "chip_module_load")
        self._functions = {}

    def function(self, name: str) -> int:
        if name not in self._functions:
            fn = ctypes.c_void_p()
            _check(load().chip_get_function(self._handle, name.encode(), ctypes.byref(fn)),
                   f"chip_get_function({name})")
            self._functions[name] = fn.value
        return self._functions[name]

    def attributes(self, name: str) -> dict:
        attr = FuncAttr()
        _check(load().chip_function_attributes(self.function(name), ctypes.byref(attr)), "chip_function_attributes")
        return {n: getattr(attr, n) for n, _ in FuncAttr._fields_}

    def unload(self):
        if self._handle:
            h, self._handle = self._handle, None
            self._functions.clear()
            try:
                load().chip_module_unload(h)
            except Exception:  # noqa: BLE001 - interpreter shutdown
                pass

    def __del__(self):
        try:
            self.unload()
        except Exception:  # noqa: BLE001
            pass


class PackedArgs:
    """Kernel arguments marshalled once: a ``void*[]`` of pointers to the argument values."""

    _CTYPES = {"ptr": ctypes.c_void_p, "i32": ctypes.c_int32, "u32": ctypes.c_uint32,
               "i64": ctypes.c_int64, "u64": ctypes.c_uint64, "f32": ctypes.c_float}

    def __init__(self, values):
        """``values``: ``[(kind, value)]`` with kind in ptr/i32/u32/i64/u64/f32."""
        self.storage = []
        for kind, value in values:
            if kind not in self._CTYPES:
                raise ValueError(f"unknown kernel argument kind {kind!r}")
            self.storage.append(self._CTYPES[kind](value))
        self.array = (ctypes.c_void_p * max(1, len(self.storage)))(
            *[ctypes.cast(ctypes.pointer(s), ctypes.c_void_p) for s in self.storage])
        self.n = len(self.storage)

    @property
    def pointer(self):
        return ctypes.cast(self.array, ctypes.POINTER(ctypes.c_void_p))


def _dim3(values):
    v = list(values) + [1] * (3 - len(values))
    return (ctypes.c_uint32 * 3)(*[int(x) for x in v[:3]])


def make_desc(fn: int, grid, block, lds_bytes: int, args: PackedArgs) -> LaunchDesc:
    d = LaunchDesc()
    d.fn = fn
    d.grid = _dim3(grid)
    d.block = _dim3(block)
    d.lds_bytes = int(lds_bytes)
    d.nargs = args.n
    d.args = args.pointer
    return d


def launch(fn: int, grid, block, lds_bytes: int, stream: int, args: PackedArgs):
    _check(load().chip_launch(fn, _dim3(grid), _dim3(block), int(lds_bytes), ctypes.c_void_p(stream or 0),
                              args.pointer, args.n), "chip_launch")


def launch_seq(descs, stream: int):
    arr = (LaunchDesc * len(descs))(*descs)
    _check(load().chip_launch_seq(arr, len(descs), ctypes.c_void_p(stream or 0)), "chip_launch_seq")


def launch_seq_fixed_scratch(descs, stream: int, refs, scratch_bytes: int, clear: bool = False):
    """``launch_seq`` with the sequence's scratch buffers inside the library's fixed per-GPU array:
    ``refs`` is ``[(launch index, argument index, byte offset)]``.  Allocates no device memory."""
    arr = (LaunchDesc * len(descs))(*descs)
    ref_arr = (ScratchArg * max(1, len(refs)))(*[ScratchArg(int(l), int(a), int(o)) for l, a, o in refs])
    _check(load().chip_launch_seq_fixed_scratch(arr, len(descs), ctypes.c_void_p(stream or 0), ref_arr, len(refs),
                                                int(scratch_bytes), int(bool(clear))),
           "chip_launch_seq_fixed_scratch")


def time_launches(descs, stream: int, warmup: int, iters: int, arg_sets=None, graph_batch: int = 0) -> float:
    """Milliseconds per pass of the launch sequence, measured with HIP events on ``stream``.
    ``arg_sets``: optional list (one entry per rotation set) of lists of ``PackedArgs`` (one
    per launch in ``descs``).  ``graph_batch`` > 0: capture that many passes into one HIP graph
    and time replays of it (at least ``iters`` passes in total) instead of an eager launch loop."""
    arr = (LaunchDesc * len(descs))(*descs)
    ms = ctypes.c_float()
    nsets, sets_ptr = 0, None
    if arg_sets and len(arg_sets) > 1:
        nsets = len(arg_sets)
        flat = [a.pointer for s in arg_sets for a in s]
        if len(flat) != nsets * len(descs):
            raise ValueError("each argument set needs one PackedArgs per launch")
        sets_arr = (ctypes.POINTER(ctypes.c_void_p) * len(flat))(*flat)
        sets_ptr = ctypes.cast(sets_arr, ctypes.POINTER(ctypes.POINTER(ctypes.c_void_p)))
    if graph_batch:
        rounds = max(1, -(-int(iters) // int(graph_batch)))
        _check(load().chip_time_graph(arr, len(descs), ctypes.c_void_p(stream or 0), int(warmup), int(graph_batch),
                                      rounds, nsets, sets_ptr, ctypes.byref(ms)), "chip_time_graph")
        return float(ms.value)
    _check(load().chip_time_launches(arr, len(descs), ctypes.c_void_p(stream or 0), int(warmup), int(iters),
                                     nsets, sets_ptr, ctypes.byref(ms)), "chip_time_launches")
    return float(ms.value)
