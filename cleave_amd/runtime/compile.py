"""Source text in, callable out: compile generated HIP with hiprtc and wrap the launches.

Keeps the two names every caller in the reference goes through,
``_load_main_kernel_from_code(source)`` and ``_compile(loaded, out_idx)``
(``python/cleave/runtime/compile.py:30-58``), plus ``build_candidate_code`` and ``check_code``
(``:133-173``).  The object ``_compile`` returns is a ``CompiledKernel``: ``kernel(*inputs)``
returns the outputs when ``out_idx`` lists trailing parameter indices, ``kernel(*inputs,
*outputs)`` writes caller-owned outputs when ``out_idx`` is None, ``get_kernel_source()``
returns the HIP text, and ``params`` is the plain ``[(name, dtype, shape, role)]`` list that
replaces the TVM adapter objects the reference's helpers poke at.
"""

from __future__ import annotations

import ast
import hashlib
import threading
from dataclasses import dataclass

from ..codegen import HipCodeGen, parse_manifest
from ..core.errors import BackendUnavailable, CompileError
from ..schedule.plan import ParamSpec
from . import shim
from .validate import DEFAULT_TOLERANCE, BenchOptions, Tolerance, _check_kernel, _stage

_TORCH_DTYPES = {"float16": "float16", "bfloat16": "bfloat16", "float32": "float32", "int32": "int32"}
_DTYPE_BYTES = {"float16": 2, "bfloat16": 2, "float32": 4, "int32": 4}


@dataclass(frozen=True)
class CompilerPassOptions:
    """Kept for signature compatibility (``python/cleave/runtime/compile.py:24-27``); the HIP
    templates have no optional layout passes, so neither flag changes the emitted source."""

    tc_awareness_pass: bool = True
    mla_decode_pass: bool = False


@dataclass
class LoadedKernel:
    """A generated source and the manifest parsed out of it."""

    source: str
    manifest: dict

    @property
    def params(self) -> list:
        return [ParamSpec.from_json(p) for p in self.manifest["params"]]


def _load_main_kernel_from_code(code_str: str) -> LoadedKernel:
    return LoadedKernel(code_str, parse_manifest(code_str))


# ----------------------------------------------------------------------------- grid expressions
_ALLOWED_NODES = (ast.Expression, ast.BinOp, ast.UnaryOp, ast.Constant, ast.Name, ast.Load, ast.Call,
                  ast.Add, ast.Sub, ast.Mult, ast.FloorDiv, ast.Mod, ast.USub)


def _ceildiv(a, b):
    return -(-int(a) // int(b))


def eval_extent(expr, dims: dict) -> int:
    """Evaluate a grid extent: integers, dim names, ``+ - * // %`` and ``ceildiv/min/max``."""
    if isinstance(expr, int):
        return expr
    tree = ast.parse(str(expr), mode="eval")
    for node in ast.walk(tree):
        if not isinstance(node, _ALLOWED_NODES):
            raise CompileError(f"grid expression {expr!r} uses {type(node).__name__}")
        if isinstance(node, ast.Call) and not (isinstance(node.func, ast.Name) and node.func.id in ("ceildiv", "min", "max")):
            raise CompileError(f"grid expression {expr!r} calls something other than ceildiv/min/max")
    env = {"ceildiv": _ceildiv, "min": min, "max": max, **dims}
    try:
        return int(eval(compile(tree, "<grid>", "eval"), {"__builtins__": {}}, env))  # noqa: S307 - AST checked above
    except NameError as e:
        raise CompileError(f"grid expression {expr!r}: {e}") from e


# ----------------------------------------------------------------------------- code object cache
_code_cache: dict = {}
_code_lock = threading.Lock()


def compile_code_object(source: str, arch: str = "gfx950") -> bytes:
    """hiprtc-compile ``source`` (memoised per process by content)."""
    key = hashlib.sha256((arch + "\0" + source).encode()).hexdigest()
    with _code_lock:
        hit = _code_cache.get(key)
    if hit is not None:
        return hit
    code, _log = shim.compile_source(source, "cleave_kernel.hip", arch)
    with _code_lock:
        _code_cache[key] = code
    return code


def code_object_stats(code: bytes) -> list[dict]:
    """Per kernel of a gfx950 code object, what the compiler's metadata note says of it: ``name``,
    ``vgprs``, ``agprs``, ``sgprs``, ``spilled_vgprs``, ``spilled_sgprs``, ``scratch_bytes`` (per lane)
    and ``lds_bytes``.  A kernel with scratch traffic in its loop pays for it twice here (the reload
    waits for every tile load in flight), so searches and tests read this rather than guess."""
    import struct

    import msgpack

    if code[:4] != b"\x7fELF":
        raise CompileError("not an ELF code object")
    shoff, = struct.unpack_from("<Q", code, 0x28)
    shentsize, shnum = struct.unpack_from("<HH", code, 0x3A)
    out = []
    for i in range(shnum):
        _, kind, _, _, off, size = struct.unpack_from("<IIQQQQ", code, shoff + i * shentsize)
        pos = off
        while kind == 7 and pos + 12 <= off + size:                     # SHT_NOTE
            namesz, descsz, ntype = struct.unpack_from("<III", code, pos)
            at = pos + 12 + ((namesz + 3) & ~3)
            if ntype == 32:                                              # NT_AMDGPU_METADATA
                for k in msgpack.unpackb(code[at:at + descsz], raw=False).get("amdhsa.kernels", ()):
                    out.append({"name": k.get(".name"), "vgprs": k.get(".vgpr_count", 0), "agprs": k.get(".agpr_count", 0),
                                "sgprs": k.get(".sgpr_count", 0), "spilled_vgprs": k.get(".vgpr_spill_count", 0),
                                "spilled_sgprs": k.get(".sgpr_spill_count", 0),
                                "scratch_bytes": k.get(".private_segment_fixed_size", 0),
                                "lds_bytes": k.get(".group_segment_fixed_size", 0)})
            pos = at + ((descsz + 3) & ~3)
    return out


class CompiledKernel:
    def __init__(self, loaded: LoadedKernel, out_idx, code: bytes):
        self.loaded = loaded
        self.manifest = loaded.manifest
        self.params = loaded.params
        self.dyn_dims = list(self.manifest.get("dyn_dims", ()))
        self.out_idx = None if out_idx is None else [int(i) for i in out_idx]
        self._code = code
        self._module = None
        self._scratch = {}
        self._caller_params = [p for p in self.params if p.role != "scratch"]
        self._n_out = sum(p.role == "output" for p in self.params)
        if self.out_idx is not None:
            want = list(range(-self._n_out, 0))
            norm = sorted(i if i < 0 else i - len(self._caller_params) for i in self.out_idx)
            if norm != want:
                raise CompileError(f"out_idx {self.out_idx} does not name the kernel's {self._n_out} trailing outputs")

    @property
    def stats(self) -> list[dict]:
        """Registers, spills, scratch and LDS of every entry point (``code_object_stats``)."""
        return code_object_stats(self._code)

    # the reference's callers read these two
    def get_kernel_source(self) -> str:
        return self.loaded.source

    @property
    def result_idx(self):
        return self.out_idx

    @property
    def module(self) -> shim.Module:
        if self._module is None:
            if shim.device_count() < 1:
                raise BackendUnavailable("no HIP device is visible: kernels can be compiled but not loaded or run")
            self._module = shim.Module(self._code)
        return self._module

    def attributes(self) -> dict:
        return {l["entry"]: self.module.attributes(l["entry"]) for l in self.manifest["launches"]}

    # ------------------------------------------------------------------ binding
    def _bind(self, args):
        import torch

        expect = self._caller_params if self.out_idx is None else [p for p in self._caller_params if p.role != "output"]
        if len(args) != len(expect):
            names = ", ".join(p.name for p in expect)
            raise TypeError(f"kernel expects {len(expect)} arguments ({names}), got {len(args)}")
        bound, dims, device = {}, {}, None
        for p, a in zip(expect, args):
            if p.role == "scalar":
                bound[p.name] = float(a) if p.dtype.startswith("float") else int(a)
                continue
            if not isinstance(a, torch.Tensor):
                raise TypeError(f"{p.name}: expected a torch tensor, got {type(a).__name__}")
            if not a.is_cuda:
                raise ValueError(f"{p.name}: tensor lives on {a.device}; kernels only run on the GPU")
            if str(a.dtype).replace("torch.", "") != _TORCH_DTYPES[p.dtype]:
                raise TypeError(f"{p.name}: dtype {a.dtype} != {p.dtype}")
            if not a.is_contiguous():
                raise ValueError(f"{p.name}: tensor must be contiguous")
            if len(a.shape) != len(p.shape):
                raise ValueError(f"{p.name}: shape {tuple(a.shape)} has rank {len(a.shape)}, expected {p.shape}")
            for want, got in zip(p.shape, a.shape):
                if isinstance(want, int):
                    if int(got) != want:
                        raise ValueError(f"{p.name}: shape {tuple(a.shape)} != {p.shape}")
                elif str(want).isidentifier():
                    if dims.setdefault(str(want), int(got)) != int(got):
                        raise ValueError(f"{p.name}: extent {want}={got} conflicts with {dims[str(want)]}")
            device = device or a.device
            bound[p.name] = a
        # derived extents such as "batch+1" are checked once every plain name is known
        for p, a in zip(expect, args):
            if p.role == "scalar":
                continue
            for want, got in zip(p.shape, a.shape):
                if not isinstance(want, int) and not str(want).isidentifier():
                    if eval_extent(want, dims) != int(got):
                        raise ValueError(f"{p.name}: extent {want} should be {eval_extent(want, dims)}, got {got}")
        # extents the generator derives from the inferred ones (a work-item size chosen from the
        # table length, say): evaluated in order, passed to the kernels like any other extent
        for name, expr in self.manifest.get("derived_dims", ()):
            dims[name] = eval_extent(expr, dims)
        missing = [d for d in self.dyn_dims if d not in dims]
        if missing:
            raise ValueError(f"run-time dims {missing} could not be inferred from the arguments")
        return bound, dims, device

    def _shape(self, p: ParamSpec, dims) -> tuple:
        return tuple(s if isinstance(s, int) else eval_extent(s, dims) for s in p.shape)

    def _materialise(self, bound, dims, device):
        import os

        import torch

        # CLEAVE_POISON_BUFFERS=1: fresh outputs and scratch start as NaN instead of whatever the
        # allocator hands back, so that a kernel which leaves part of a buffer unwritten (or reads
        # scratch it has not written) fails its comparison every time instead of now and then.
        poison = bool(os.environ.get("CLEAVE_POISON_BUFFERS"))

        def fresh(shape, dtype):
            t = torch.empty(shape, dtype=dtype, device=device)
            if poison and t.is_floating_point():
                t.fill_(float("nan"))
            return t

        outs = []
        for p in self.params:
            if p.role == "output" and p.name not in bound:
                t = fresh(self._shape(p, dims), getattr(torch, p.dtype))
                bound[p.name] = t
                outs.append(t)
            elif p.role == "output":
                outs.append(bound[p.name])
        for p in self.params:
            if p.role != "scratch":
                continue
            owner = p.alias or p.name
            shape = self._shape(p, dims)
            key = (owner, shape, str(device))
            if key not in self._scratch:
                self._scratch[key] = fresh(shape, getattr(torch, p.dtype))
            bound[p.name] = self._scratch[key]
        return outs

    def _descs(self, bound, dims, fixed=None, refs=None):
        """Launch descriptors.  ``fixed``: ``{scratch parameter: byte offset}``; those arguments are
        left null here and listed in ``refs`` as (launch, argument, offset) for the library to point
        into its fixed scratch array."""
        keep, descs = [], []
        for l in self.manifest["launches"]:
            values = []
            for name in l["args"]:
                if name in dims and name not in bound:
                    values.append(("i32", dims[name]))
                    continue
                if fixed is not None and name in fixed:
                    refs.append((len(descs), len(values), fixed[name]))
                    values.append(("ptr", 0))
                    continue
                v = bound[name]
                if isinstance(v, float):
                    values.append(("f32", v))
                elif isinstance(v, int):
                    values.append(("i32", v))
                else:
                    values.append(("ptr", v.data_ptr()))
            packed = shim.PackedArgs(values)
            grid = [eval_extent(g, dims) for g in l["grid"]]
            if min(grid) < 1:
                return None, None  # an empty problem (e.g. batch == 0): nothing to launch
            if grid[1] > 65535 or grid[2] > 65535 or grid[0] > 2 ** 31 - 1:
                raise CompileError(f"grid {grid} exceeds the launch limits")
            keep.append(packed)
            descs.append(shim.make_desc(self.module.function(l["entry"]), grid, l["block"], l["lds"], packed))
        return descs, keep

    # ------------------------------------------------------------------ run
    def __call__(self, *args):
        import torch

        bound, dims, device = self._bind(args)
        outs = self._materialise(bound, dims, device)
        with torch.cuda.device(device):
            descs, keep = self._descs(bound, dims)
            if descs:
                shim.launch_seq(descs, torch.cuda.current_stream(device).cuda_stream)
        del keep
        if self.out_idx is None:
            return None
        return outs[0] if len(outs) == 1 else outs

    def fixed_scratch_layout(self, dims) -> tuple:
        """``({scratch parameter: byte offset}, bytes)``: the kernel's scratch buffers laid out
        one after the other at multiples of 256 bytes (two names of one buffer share an offset)."""
        offsets, owners, end = {}, {}, 0
        for p in self.params:
            if p.role != "scratch":
                continue
            owner = p.alias or p.name
            if owner not in owners:
                owners[owner] = end
                n = _DTYPE_BYTES[p.dtype]
                for extent in self._shape(p, dims):
                    n *= extent
                end += -(-n // 256) * 256
            offsets[p.name] = owners[owner]
        return offsets, end

    def call_fixed_scratch(self, *args, clear: bool = False) -> None:
        """Run with caller-owned outputs and no allocation of device memory: the scratch buffers
        (split partials) live in the native library's fixed per-GPU array instead of tensors.  The
        kernel must have been made with ``out_idx=None``; ``args`` are the inputs, scalars and
        outputs in parameter order.  A layout beyond the array's size is refused by the library.
        Calls that overlap on one GPU share the array and race."""
        import torch

        if self.out_idx is not None:
            raise TypeError("call_fixed_scratch needs caller-owned outputs: compile with out_idx=None")
        bound, dims, device = self._bind(args)
        fixed, nbytes = self.fixed_scratch_layout(dims)
        refs = []
        with torch.cuda.device(device):
            descs, keep = self._descs(bound, dims, fixed, refs)
            if descs:
                shim.launch_seq_fixed_scratch(descs, torch.cuda.current_stream(device).cuda_stream, refs, nbytes, clear)
        del keep

    def time(self, *args, warmup: int = 4, iters: int = 100, rotate=None, only=None, graph_batch: int = 0) -> float:
        """Milliseconds per call measured with HIP events inside the native library.  ``rotate``:
        further argument tuples (same signature) cycled through call by call, so a working set
        larger than the 256 MB last-level cache keeps every call reading HBM.  ``only``: indices
        of the launches to time (e.g. ``[0]`` for the partial kernel of a fused pair alone).
        ``graph_batch`` > 0: time replays of a HIP graph holding that many calls (the reference's
        way of timing) instead of an eager launch loop."""
        import torch

        sets = [args] + list(rotate or [])
        all_descs, all_keep, held = [], [], []
        device = None
        for a in sets:
            bound, dims, device = self._bind(a)
            held.append(self._materialise(bound, dims, device))
            if self.out_idx is not None:
                for t in held[-1]:
                    t.zero_()      # the outputs are this call's own: whatever they hold afterwards, the timed launches wrote
            with torch.cuda.device(device):
                descs, keep = self._descs(bound, dims)
            if not descs:
                raise ValueError("cannot time an empty launch")
            if only is not None:
                descs, keep = [descs[i] for i in only], [keep[i] for i in only]
            all_descs.append(descs)
            all_keep.append(keep)
        with torch.cuda.device(device):
            stream = torch.cuda.current_stream(device).cuda_stream
            ms = shim.time_launches(all_descs[0], stream, warmup, iters, all_keep if len(sets) > 1 else None,
                                    graph_batch=graph_batch)
        self.last_timed_outputs = held[0]      # what the timed launches of the first argument set wrote
        return ms


def _compile(loaded, out_idx):
    """hiprtc-compile a loaded source; the code object is loaded on first launch."""
    if isinstance(loaded, str):
        loaded = _load_main_kernel_from_code(loaded)
    with _stage("compile"):
        code = compile_code_object(loaded.source, loaded.manifest.get("arch", "gfx950"))
        return CompiledKernel(loaded, out_idx, code)


def build_candidate_code(cand, options: CompilerPassOptions | None = None) -> str:
    """HIP source of one tiling candidate: the default ``build_fn`` of ``run_candidates``
    (``python/cleave/runtime/compile.py:133-148``)."""
    from ..schedule import apply_tiling

    return HipCodeGen().gen(apply_tiling(cand))


def check_code(code_str, *, graph=None, dtype=None, out_idx=None, reference_cache_dir=None,
               tolerance: Tolerance | None = None, benchmark: BenchOptions | None = None):
    """``(device source, latency_ms | None)``: compile, validate against the published
    reference and optionally time one kernel (``python/cleave/runtime/compile.py:151-173``)."""
    loaded = _load_main_kernel_from_code(code_str)
    if out_idx is None:
        out_idx = loaded.manifest["out_idx"]
    kernel = _compile(loaded, out_idx)
    latency_ms = _check_kernel(kernel, graph=graph, dtype=dtype, reference_cache_dir=reference_cache_dir,
                               tolerance=tolerance or DEFAULT_TOLERANCE, benchmark=benchmark)
    return kernel.get_kernel_source(), latency_ms
