"""Code generation: a scheduled ``KernelPlan`` becomes HIP source text for gfx950.

Takes the place of the reference's TileLang emitter
(``python/cleave/codegen/__init__.py:24-60`` and ``kernel.py``/``split.py``/``macros.py``):
``HipCodeGen().gen(plan)`` returns one self-contained translation unit, and
``gen([partial, combine])`` the fused two-kernel form of a split pair
(``python/cleave/codegen/split.py:13-123``) whose partial buffers are scratch parameters named
``Partial_<X>_split`` / ``Partial_<X>_combine`` (one allocation, two names).

A generated source is: a manifest comment (JSON: parameters in call order, launches with grid
expressions, LDS bytes), a block of ``#define``s instantiating the template, the shared
helpers, and the hand-written template body.  The kernel entry is ``main_kernel``; parameter
names follow the reference's contract (``PlaceHolder_<NAME>``, run-time scalars between inputs
and outputs, then ``OutputNode_<i>``; ``python/cleave/codegen/kernel.py:576-612``).
"""

from __future__ import annotations

import json
import math
from pathlib import Path

from ..core.errors import CodegenError
from ..schedule.plan import KernelPlan, ParamSpec

TEMPLATE_DIR = Path(__file__).resolve().parent / "templates"
ENTRY = "main_kernel"
COMBINE_ENTRY = "main_kernel_combine"
MANIFEST_BEGIN = "// CLEAVE-HIP-MANIFEST-BEGIN"
MANIFEST_END = "// CLEAVE-HIP-MANIFEST-END"
LOG2E = 1.4426950408889634

_C_TYPES = {"float16": "elem_t", "bfloat16": "elem_t", "float32": "float", "int32": "int"}


def _template(name: str) -> str:
    return (TEMPLATE_DIR / name).read_text()


def _f(x: float) -> str:
    """A C float literal that round-trips."""
    text = repr(float(x))
    if "e" not in text and "." not in text and "inf" not in text and "nan" not in text:
        text += ".0"
    return text + "f"


def tail_requested(tile) -> bool:
    return bool(int(tile.get("TAIL", 0)))


def _c_param(p: ParamSpec) -> str:
    if p.role == "scalar":
        return f"{_C_TYPES[p.dtype]} {p.name}"
    const = "const " if p.role == "input" else ""
    return f"{const}{_C_TYPES[p.dtype]}* __restrict__ {p.name}"


class _Unit:
    """Accumulates one translation unit: defines, launches, parameters."""

    def __init__(self, plan: KernelPlan):
        self.plan = plan
        self.defines: list = []
        self.launches: list = []
        self.templates: list = ["common.hip"]

    def define(self, name, value):
        if isinstance(value, bool):
            value = int(value)
        self.defines.append(f"#define {name} {value}")

    def signature(self, macro, entry_macro, entry, params, dyn_dims, dyn_c_names=None):
        """Define the C parameter list of one kernel; returns the manifest's argument names.
        ``dyn_c_names``: the identifiers the template uses for the run-time extents, when the
        operator spec renamed them."""
        parts = [_c_param(p) for p in params] + [f"int {d}" for d in (dyn_c_names or dyn_dims)]
        self.define(entry_macro, entry)
        self.define(macro, ", ".join(parts))
        return [p.name for p in params] + list(dyn_dims)

    def launch(self, entry, grid, block, lds, args):
        self.launches.append({"entry": entry, "grid": [str(g) for g in grid], "block": [int(block), 1, 1],
                              "lds": int(lds), "args": list(args)})


class HipCodeGen:
    def gen(self, plan_or_pair, *, params=None) -> str:
        """Source text for one plan, or for ``[partial, combine]`` fused into one unit."""
        try:
            if isinstance(plan_or_pair, (list, tuple)):
                if len(plan_or_pair) == 1:
                    return self._gen_one(plan_or_pair[0])
                if len(plan_or_pair) != 2:
                    raise CodegenError(f"expected one plan or a [partial, combine] pair, got {len(plan_or_pair)}")
                return self._gen_fused(*plan_or_pair)
            return self._gen_one(plan_or_pair)
        except CodegenError:
            raise
        except (KeyError, ValueError, TypeError, ZeroDivisionError) as e:
            raise CodegenError(f"{type(e).__name__} while instantiating a template: {e}") from e

    # ------------------------------------------------------------------ drivers
    def _gen_one(self, plan: KernelPlan) -> str:
        unit = _Unit(plan)
        emit = getattr(self, f"_emit_{plan.template}", None)
        if emit is None:
            raise CodegenError(f"no template named {plan.template!r}")
        probes = sorted(k for k in (plan.tiling or {}) if str(k).startswith("DBG_"))
        if probes:
            # (the shipped templates hold no measurement switches: a key that asks for one would be ignored)
            raise CodegenError(f"tiling keys {probes} name measurement switches, which the templates do not have")
        splits = plan.split_factor or 1
        if plan.role == "main" and splits != 1:
            raise CodegenError("a main kernel cannot carry a split factor")
        params = list(plan.params)
        emit(unit, plan, params, partial=plan.role in ("main", "partial", "fused"),
             combine=plan.role in ("combine", "fused") and splits > 1, fused=plan.role == "fused")
        return self._finish(unit, plan, params)

    def _gen_fused(self, partial: KernelPlan, combine: KernelPlan) -> str:
        """Partial and combine in one unit: the partial's outputs become scratch parameters."""
        if partial.role != "partial" or combine.role != "combine":
            raise CodegenError("a fused pair is [partial, combine]")
        pair = {partial.template, combine.template}
        if len(pair) > 1 and not pair <= {"gemm", "gemm_dma", "skinny"} and pair != {"attn_prefill", "attn_decode"}:
            raise CodegenError(f"partial ({partial.template}) and combine ({combine.template}) templates differ")
        params = [p for p in partial.params if p.role in ("input", "scalar")]
        operands = dict(partial.operands)
        for p in partial.params:
            if p.role == "output":
                role = next(r for r, n in partial.operands.items() if n == p.name)
                split_name, comb_name = f"Partial_{role}_split", f"Partial_{role}_combine"
                params.append(ParamSpec(split_name, p.dtype, p.shape, "scratch"))
                params.append(ParamSpec(comb_name, p.dtype, p.shape, "scratch", alias=split_name))
                operands[role] = split_name
                operands[f"{role}_COMBINE"] = comb_name
        for p in combine.params:
            if p.role == "output":
                params.append(p)
        operands.update({r: n for r, n in combine.operands.items() if r.startswith("OUT")})
        fused = KernelPlan(template=partial.template, role="fused", family=partial.family, dtype=partial.dtype,
                           problem=partial.problem, tiling=partial.tiling, params=params, operands=operands,
                           split_factor=partial.split_factor, dyn_dims=partial.dyn_dims, n_threads=partial.n_threads,
                           lds_bytes=partial.lds_bytes, label=f"{partial.label} + combine", extra=dict(partial.extra))
        return self._gen_one(fused)

    def _finish(self, unit: _Unit, plan: KernelPlan, params) -> str:
        n_out = sum(p.role == "output" for p in params)
        manifest = {
            "format": 1, "generator": "cleave_amd", "arch": "gfx950", "template": plan.template,
            "role": plan.role, "family": plan.family, "dtype": plan.dtype, "label": plan.label,
            "split": plan.split_factor, "tiling": plan.tiling,
            "params": [p.to_json() for p in params], "dyn_dims": list(plan.dyn_dims),
            "derived_dims": [list(d) for d in plan.extra.get("derived_dims", ())],
            "out_idx": list(range(-n_out, 0)), "launches": unit.launches,
        }
        head = [MANIFEST_BEGIN] + ["// " + line for line in json.dumps(manifest, indent=1).splitlines()] + [MANIFEST_END]
        body = [f"// ---- template: {plan.template}  role: {plan.role}  {plan.label}"]
        body += unit.defines
        for name in unit.templates:
            body.append(_template(name))
        return "\n".join(head + body) + "\n"

    # ------------------------------------------------------------------ shared pieces
    @staticmethod
    def _common(unit: _Unit, plan: KernelPlan, partial: bool, combine: bool):
        unit.define("CL_BF16", plan.dtype == "bfloat16")
        unit.define("CL_SPLITS", plan.split_factor or 1)
        unit.define("CL_EMIT_PARTIAL", partial)
        unit.define("CL_EMIT_COMBINE", combine)

    @staticmethod
    def _by_name(params):
        return {p.name: p for p in params}

    # ------------------------------------------------------------------ matmul families
    def _matmul_common(self, unit, plan, params, partial, combine, fused):
        p, op = plan.problem, plan.operands
        self._common(unit, plan, partial, combine)
        norm = plan.family == "rmsnorm_matmul"
        lora = plan.family == "lora"
        for k in ("M", "N", "K"):
            unit.define(f"CL_{k}", p[k])
        if lora:
            unit.define("CL_LORA", 1)
            unit.define("CL_R", p["R"])
        unit.define("CL_NORM", norm)
        unit.define("CL_GAMMA", bool(norm and p.get("gamma")))
        unit.define("CL_EPS", _f(p.get("eps", 0.0)))
        unit.define("CL_BATCH_A", p["batch_A"])
        unit.define("CL_BATCH_B", p["batch_B"])
        unit.define("CL_TRANS_A", p["trans_A"])
        unit.define("CL_TRANS_B", p["trans_B"])
        splits = plan.split_factor or 1
        names = self._by_name(params)
        ins = [q for q in params if q.role in ("input", "scalar")]
        outs = [q for q in params if q.role == "output"]
        batch = max(p["batch_A"], p["batch_B"])
        if partial:
            if plan.role in ("main",):
                sig = ins + outs
                unit.define("CL_ARG_OUT", op["OUT"])
            elif plan.role == "partial":
                sig = ins + outs
            else:  # fused
                sig = ins + [names[op["PACC"]]] + ([names[op["PSS"]]] if norm else []) + ([names[op["PD"]]] if lora else [])
            if splits > 1:
                unit.define("CL_ARG_PACC", op["PACC"])
                if norm:
                    unit.define("CL_ARG_PSS", op["PSS"])
                if lora:
                    unit.define("CL_ARG_PD", op["PD"])
            for role, macro in (("A", "CL_ARG_A"), ("B", "CL_ARG_B"), ("C", "CL_ARG_C"), ("GAMMA", "CL_ARG_GAMMA"),
                                ("LA", "CL_ARG_LA"), ("LB", "CL_ARG_LB")):
                if role in op:
                    unit.define(macro, op[role])
            unit.define("CL_ARG_X", op["A"])
            unit.define("CL_ARG_W", op["B"])
            args = unit.signature("CL_PARTIAL_PARAMS", "CL_PARTIAL_NAME", ENTRY, sig, ())
            self._partial_args = args
        if combine:
            if plan.role == "combine":
                sig, entry, suffix = ins + outs, ENTRY, ""
            else:
                # the combine reads the same allocation under its `_combine` name
                sig = [names[op["PACC_COMBINE"]]] + ([names[op["PSS_COMBINE"]]] if norm else []) \
                    + ([names[op["PD_COMBINE"]], names[op["LB"]]] if lora else []) + outs
                entry, suffix = COMBINE_ENTRY, "_COMBINE"
            unit.define("CL_CARG_PACC", op["PACC" + suffix])
            if norm:
                unit.define("CL_CARG_PSS", op["PSS" + suffix])
            if lora:
                unit.define("CL_CARG_PD", op["PD" + suffix])
                unit.define("CL_CARG_LB", op["LB"])
            unit.define("CL_CARG_OUT", op["OUT"])
            args = unit.signature("CL_COMBINE_PARAMS", "CL_COMBINE_NAME", entry, sig, ())
            # columns per thread: the most that still leaves the chip a few hundred workgroups
            total = batch * p["M"] * p["N"]
            cols = next((c for c in (4, 2, 1) if p["N"] % c == 0 and total // c // 256 >= 256), 1)
            if lora:
                # a workgroup of the LoRA combine works on one row (it sums that row's rank-R partials once, in LDS)
                cols = next((c for c in (4, 2, 1) if p["N"] % (256 * c) == 0), None)
                if cols is None:
                    raise CodegenError("the LoRA combine needs N to be a multiple of 256")
            unit.define("CL_COMBINE_ROWS", batch * p["M"])
            unit.define("CL_COMBINE_COLS", cols)
            self._combine_args = (entry, args, -(-(total // cols) // 256))

    def _emit_gemm(self, unit, plan, params, partial, combine, fused):
        p, t = plan.problem, plan.tiling
        self._matmul_common(unit, plan, params, partial, combine, fused)
        tile = dict(BM=64, BN=64, BK=64, WM=1, WN=1)
        tile.update(t)
        for k, v in tile.items():
            unit.define(f"CL_{k}", v)
        splits = plan.split_factor or 1
        batch = max(p["batch_A"], p["batch_B"])
        unit.templates.append("gemm.hip")
        if partial:
            from ..schedule.policy import gemm_lds_bytes

            if p["K"] % (splits * tile["BK"]) and (splits > 1 or p["K"] % 8):
                raise CodegenError(f"K={p['K']} is neither a multiple of splits*BK={splits * tile['BK']} nor, unsplit, of 8")
            grid = (-(-p["N"] // tile["BN"]), -(-p["M"] // tile["BM"]), batch * splits)
            lds = gemm_lds_bytes(tile["BM"], tile["BN"], tile["BK"], plan.family == "rmsnorm_matmul")
            unit.launch(ENTRY, grid, tile["WM"] * tile["WN"] * 64, lds, self._partial_args)
        if combine:
            entry, args, blocks = self._combine_args
            unit.templates.append("matmul_combine.hip")
            unit.launch(entry, (blocks, 1, 1), 256, 0, args)

    def _emit_gemm_dma(self, unit, plan, params, partial, combine, fused):
        p, t = plan.problem, plan.tiling
        if plan.family == "rmsnorm_matmul":
            # the norm is applied to the product's rows, which needs a norm without a learned weight
            if p.get("gamma") or p["trans_A"] or (plan.split_factor or 1) > 1 or combine:
                raise CodegenError("the direct-to-LDS matmul fuses an RMSNorm only without a learned weight, for "
                                   "row-major A, unsplit")
        elif plan.family not in ("matmul", "swiglu", "matmul_rowsum"):
            raise CodegenError(f"the direct-to-LDS matmul template has no {plan.family} form")
        self._matmul_common(unit, plan, params, partial, combine, fused)
        tile = dict(BM=128, BN=128, BK=64, WM=2, WN=2)
        tile.update(t)
        for k, v in tile.items():
            unit.define(f"CL_{k}", v)
        splits = plan.split_factor or 1
        swiglu = plan.family == "swiglu"
        if swiglu != bool(tile.get("SWIGLU")) or (swiglu and (splits > 1 or combine)):
            raise CodegenError("SwiGLU is the SWIGLU tiling of the direct-to-LDS matmul, unsplit")
        rowsum = plan.family == "matmul_rowsum"
        if rowsum != bool(tile.get("ROWSUM")) or (rowsum and (splits > 1 or combine or p["N"] % tile["BN"])):
            raise CodegenError("matmul + row sum is the ROWSUM tiling of the direct-to-LDS matmul, unsplit, over whole column tiles")
        # (SwiGLU: the B tile holds BN / 2 columns of each weight, so a tile covers BN / 2 columns of the output)
        out_bn = tile["BN"] // 2 if swiglu else tile["BN"]
        if swiglu and (tile["BN"] // tile["WN"] // 16) % 2:
            raise CodegenError("a SwiGLU wave owns an even number of column fragments")
        batch = max(p["batch_A"], p["batch_B"])
        unit.templates.append("gemm_dma.hip")
        if partial:
            if tile["BK"] != 64 or p["K"] % (splits * 64):
                raise CodegenError(f"K={p['K']} is not a multiple of splits*64={splits * 64}")
            if (not p["trans_B"] and p["N"] % 8) or (p["trans_A"] and p["M"] % 8) or p["K"] % 8:
                raise CodegenError("16-byte global chunks need the minor extent of each operand to be a multiple of 8")
            grid = (1 if rowsum else -(-p["N"] // out_bn), -(-p["M"] // tile["BM"]), batch * splits)
            stages = int(tile.get("STAGES", 2))
            if stages != 2:
                waves = tile["WM"] * tile["WN"]
                if (stages != 3 or rowsum or not int(tile.get("ASM_LOADS", 1)) or 3 * (tile["BM"] + tile["BN"]) * 128 > 160 * 1024
                        or (tile["BM"] // 8) % waves or (tile["BN"] // 8) % waves
                        or (tail_requested(tile) and (tile["BM"] // 16) % waves)):
                    raise CodegenError("three LDS stages: tiles of which three images fit 160 KiB, every wave loading the same "
                                       "number of 1 KiB units of each (of a tail's half-height A tile as well), assembly tile "
                                       "loads, no row-sum walk")
            tail = int(tile.get("TAIL", 0))
            if tail:
                # the last `tail` tiles run as two half-height workgroups each, on a one-dimensional grid
                if (rowsum or p["trans_A"] or batch * splits != 1 or not 0 < tail <= grid[0] * grid[1]
                        or tile["BM"] % (32 * tile["WM"]) or p["M"] % tile["BM"]):
                    raise CodegenError("the tail split needs row-major A, whole row tiles that halve, one batch and one split")
                grid = (grid[0] * grid[1] + tail, 1, 1)
            # the tile images are static LDS arrays of the kernel: no dynamic LDS at launch
            unit.launch(ENTRY, grid, tile["WM"] * tile["WN"] * 64, 0, self._partial_args)
        if combine:
            entry, args, blocks = self._combine_args
            unit.templates.append("matmul_combine.hip")
            unit.launch(entry, (blocks, 1, 1), 256, 0, args)

    def _emit_rowsum(self, unit, plan, params, partial, combine, fused):
        p, op = plan.problem, plan.operands
        if combine or (plan.split_factor or 1) > 1:
            raise CodegenError("row reductions have no split form")
        if p["N"] % 8:
            raise CodegenError("row reductions read 16-byte chunks: the row length must be a multiple of 8")
        rows = int(plan.tiling.get("ROWS_PER_BLOCK", 4))
        if rows not in (1, 2, 4):
            raise CodegenError("1, 2 or 4 rows per workgroup")
        self._common(unit, plan, partial, combine)
        for k, v in (("CL_M", p["M"]), ("CL_N", p["N"]), ("CL_DIV", bool(p["div"])), ("CL_ROWS_PER_BLOCK", rows)):
            unit.define(k, v)
        unit.define("CL_ARG_X", op["X"])
        unit.define("CL_ARG_OUT", op["OUT"])
        ins = [q for q in params if q.role in ("input", "scalar")]
        outs = [q for q in params if q.role == "output"]
        args = unit.signature("CL_PARTIAL_PARAMS", "CL_PARTIAL_NAME", ENTRY, ins + outs, ())
        unit.templates.append("rowsum.hip")
        unit.launch(ENTRY, (-(-p["M"] // rows), 1, 1), 64 * rows, 0, args)

    def _emit_skinny(self, unit, plan, params, partial, combine, fused):
        p, t = plan.problem, plan.tiling
        self._matmul_common(unit, plan, params, partial, combine, fused)
        tile = dict(WAVES_N=1, WAVES_K=1, PREFETCH=2)
        tile.update(t)
        for k, v in tile.items():
            unit.define(f"CL_{k}", v)
        unit.templates.append("skinny_matmul.hip")
        splits = plan.split_factor or 1
        lora = plan.family == "lora"
        if lora != bool(tile.get("LORA")):
            raise CodegenError("LoRA is the LORA tiling of the few-row matmul")
        if lora and (p["R"] % 8 or p["R"] > 64):
            raise CodegenError("LoRA rank must be a multiple of 8 up to 64")
        if partial:
            from ..schedule.policy import lora_lds_bytes, skinny_lds_bytes

            if p["M"] > 64 or p["K"] % 32 or p["N"] % 8:
                raise CodegenError("the few-row matmul template needs M <= 64, K % 32 == 0, N % 8 == 0")
            grid = (-(-p["N"] // (128 * tile["WAVES_N"])), splits, 1)
            lds = skinny_lds_bytes(-(-p["M"] // 16), tile["WAVES_N"], tile["WAVES_K"])
            if lora:
                lds = lora_lds_bytes(-(-p["M"] // 16), tile["WAVES_N"], tile["WAVES_K"], p["R"])
            if lds > 160 * 1024:
                raise CodegenError(f"the few-row matmul's cross-wave reduction would need {lds} bytes of LDS at "
                                   f"WAVES_N={tile['WAVES_N']} WAVES_K={tile['WAVES_K']} and {p['M']} rows (160 KiB per workgroup)")
            unit.launch(ENTRY, grid, tile["WAVES_N"] * tile["WAVES_K"] * 64, lds, self._partial_args)
        if combine:
            entry, args, blocks = self._combine_args
            unit.templates.append("matmul_combine.hip")
            unit.launch(entry, (blocks, 1, 1), 256, 0, args)

    # ------------------------------------------------------------------ attention families
    def _attn_common(self, unit, plan, params, partial, combine, fused, vdim, total_rows, emit_lse):
        op = plan.operands
        self._common(unit, plan, partial, combine)
        unit.define("CL_VDIM", vdim)
        unit.define("CL_TOTAL_ROWS", total_rows)
        unit.define("CL_EMIT_LSE", emit_lse)
        names = self._by_name(params)
        # (a `Scratch_*` parameter is written by a launch of this unit ahead of the attention kernel, which reads it)
        ins = [q for q in params if q.role in ("input", "scalar") or q.name.startswith("Scratch_")]
        outs = [q for q in params if q.role == "output"]
        derived = tuple(name for name, _ in plan.extra.get("derived_dims", ()))
        dyn = tuple(plan.dyn_dims) + derived
        dyn_c = tuple((plan.problem.get("dim_names") or {}).keys()) or None
        if dyn_c is not None:
            dyn_c += derived
        splits = plan.split_factor or 1
        part_roles = ("PM", "PL", "PO")
        if partial:
            if plan.role == "fused":
                sig = ins + [names[op[r]] for r in part_roles]
            else:
                sig = ins + outs
            if splits > 1:
                for r in part_roles:
                    unit.define(f"CL_ARG_{r}", op[r])
            else:
                unit.define("CL_ARG_OUT", op["OUT"])
                if emit_lse:
                    unit.define("CL_ARG_LSE", op["OUT1"])
            self._partial_args = unit.signature("CL_PARTIAL_PARAMS", "CL_PARTIAL_NAME", ENTRY, sig, dyn, dyn_c)
        if combine:
            if plan.role == "combine":
                sig, entry, suffix = ins + outs, ENTRY, ""
            else:
                sig, entry, suffix = [names[op[f"{r}_COMBINE"]] for r in part_roles] + outs, COMBINE_ENTRY, "_COMBINE"
                if plan.tiling.get("CHUNK_PAGES"):
                    sig = [names[op["INDPTR"]]] + sig
            if plan.tiling.get("CHUNK_PAGES"):
                unit.define("CL_CARG_INDPTR", op["INDPTR"])
            for r in part_roles:
                unit.define(f"CL_CARG_{r}", op[r + suffix])
            unit.define("CL_CARG_OUT", op["OUT"])
            if emit_lse:
                unit.define("CL_CARG_LSE", op["OUT1"])
            args = unit.signature("CL_COMBINE_PARAMS", "CL_COMBINE_NAME", entry, sig, dyn, dyn_c)
            self._combine_args = (entry, args)

    def _emit_attn_decode(self, unit, plan, params, partial, combine, fused):
        p, t, op = plan.problem, plan.tiling, plan.operands
        if partial and (p.get("norm_eps") or p.get("linear")):
            raise CodegenError("the streaming attention kernel has no QK-norm form and no softmax-free form")
        paged = bool(p.get("paged"))
        rows = p["group"] * p["sq"]
        emit_lse = bool(p.get("emit_lse"))
        if paged:
            batch_name = p["dim_names"]["batch"]
            total_rows = f"(batch * {p['q_heads']})"          # C expression inside the kernels
            units = f"{batch_name} * {p['kv_heads']}"          # grid expression over manifest dims
            grid_rows = f"({batch_name} * {p['q_heads']})"
        else:
            total_rows = p["units"] * rows
            units = str(p["units"])
            grid_rows = str(total_rows)
        self._attn_common(unit, plan, params, partial, combine, fused, p["vdim"], total_rows, emit_lse)
        waves = int(t.get("WAVES", 4))
        unit.define("CL_HEAD_DIM", p["head_dim"])
        unit.define("CL_ROWS", rows)
        unit.define("CL_WAVES", waves)
        unit.define("CL_PREFETCH", int(t.get("PREFETCH", 1)))
        chunk_pages = bool(t.get("CHUNK_PAGES", 0)) and paged and (plan.split_factor or 1) > 1
        unit.define("CL_CHUNK_PAGES", chunk_pages)
        if int(t.get("LOCKSTEP", 0)):
            if not chunk_pages:
                raise CodegenError("LOCKSTEP (a barrier per step between the waves of a workgroup) exists for chunked items only")
            unit.define("CL_LOCKSTEP", 1)
        skew = int(t.get("SKEW", 0))
        if skew:
            # the rotation of units over the XCDs assumes that launch index % 8 is blockIdx.x % 8
            per_x = (p["kv_heads"] if paged else p["units"]) * (-(-rows // 16))
            if (plan.split_factor or 1) % 2 or chunk_pages or per_x % 8 or not 0 < skew <= 500 or not partial:
                raise CodegenError("SKEW (split ranges skewed between even and odd XCDs, in thousandths of a pair's steps, "
                                   "1..500) needs an even split count, a grid of whole groups of eight unit tiles and no chunked items")
            unit.define("CL_SKEW", skew)
        unit.define("CL_PAGED", paged)
        unit.define("CL_PAGE_SIZE", p.get("page_size", 1))
        unit.define("CL_KV_HEADS", p.get("kv_heads", 1))
        unit.define("CL_Q_HEADS", p.get("q_heads", 1))
        unit.define("CL_SKV", p.get("skv", 0))
        unit.define("CL_SCALE_LOG2E", _f(float(p.get("scale", 1.0)) * LOG2E))
        for role, macro in (("Q", "CL_ARG_Q"), ("K", "CL_ARG_K"), ("V", "CL_ARG_V"), ("INDPTR", "CL_ARG_INDPTR"),
                            ("INDICES", "CL_ARG_INDICES"), ("LAST", "CL_ARG_LAST")):
            if role in op:
                unit.define(macro, op[role])
        if p["head_dim"] % 32 or not (p["vdim"] % 128 == 0 or p["vdim"] == 64):
            raise CodegenError("decode attention needs head_dim % 32 == 0 and value width 64 or k*128")
        splits = plan.split_factor or 1
        row_tiles = -(-rows // 16)
        unit.templates += ["attn_decode.hip", "attn_combine.hip"]
        if partial:
            from ..schedule.policy import attn_lds_bytes

            if chunk_pages:
                items = f"ceildiv({p['dim_names']['n_idx']}, chunk_pages) + {batch_name}"
                grid = (items, 1, 1)
            else:
                grid = (f"({units}) * {row_tiles}", splits, 1)
            # (a wave that shares its rows with no other stores straight from its accumulators: no LDS)
            lds = 0 if waves == 1 or chunk_pages else attn_lds_bytes(waves, p["vdim"])
            unit.launch(ENTRY, grid, waves * 64, lds, self._partial_args)
        if combine:
            entry, args = self._combine_args
            unit.launch(entry, (f"ceildiv({grid_rows} * {p['vdim'] // 4}, 256)", 1, 1), 256, 0, args)

    def _emit_attn_dense_prefill(self, unit, plan, params, partial, combine):
        """The LDS-shared prefill kernel over the dense attention family's operands: every unit
        (batch entry x kv head) has ``group * sq`` query rows that all see all keys."""
        p, op = plan.problem, plan.operands
        splits = plan.split_factor or 1
        d, rows = p["head_dim"], p["group"] * p["sq"]
        if splits > 1 and p.get("emit_lse"):
            raise CodegenError("the split form of the many-row attention kernel has no lse output")
        if d % 64 or d > 256 or p["vdim"] % 64 or p["vdim"] > 256:
            raise CodegenError("the many-row attention kernel needs key and value widths in whole 64-feature panels (<= 256)")
        norm = p.get("norm_eps") or {}
        # KPRE: the keys of a QK-norm attention are normalised once by a launch of their own into a
        # scratch copy, which the attention kernel then reads as plain keys
        kpre = bool(plan.tiling.get("KPRE"))
        if kpre:
            if "k" not in norm or not partial or p.get("k_major") or d not in (64, 128, 256):
                raise CodegenError("KPRE normalises row-major keys of a QK-norm attention, 64, 128 or 256 wide, ahead of the kernel that reads them")
            key = self._by_name(params)[op["K"]]
            at = next(i for i, q in enumerate(params) if q.role in ("scratch", "output"))
            params.insert(at, ParamSpec("Scratch_kn", key.dtype, key.shape, "scratch"))
        self._attn_common(unit, plan, params, partial, combine, False, p["vdim"], p["units"] * rows, False)
        for k, v in (("CL_DENSE", 1), ("CL_RAGGED", 1), ("CL_HEAD_DIM", d), ("CL_KV_HEADS", 1), ("CL_Q_HEADS", 1),
                     ("CL_ROWS", rows), ("CL_SKV", p["skv"])):
            unit.define(k, v)
        unit.define("CL_SCALE", _f(float(p.get("scale", 1.0))))
        unit.define("CL_LINEAR", bool(p.get("linear")))
        if p.get("k_major") and p["skv"] % 32:
            raise CodegenError("feature-major keys need a key count in whole 32-key steps")
        unit.define("CL_KT", bool(p.get("k_major")))
        unit.define("CL_QNORM", "q" in norm)
        unit.define("CL_KNORM", "k" in norm and not kpre)
        unit.define("CL_QNORM_EPS", _f(float(norm.get("q", 0.0))))
        unit.define("CL_KNORM_EPS", _f(float(norm.get("k", 0.0))))
        for role, macro in (("Q", "CL_ARG_Q"), ("K", "CL_ARG_K"), ("V", "CL_ARG_V")):
            unit.define(macro, "Scratch_kn" if kpre and role == "K" else op[role])
        for k, v in plan.tiling.items():
            if k not in ("SHARED", "KPRE"):
                unit.define(f"CL_PF_{k}", int(v))
        unit.define("CL_EMIT_KPRE", kpre)
        unit.templates += ["attn_prefill_lds.hip", "attn_combine.hip"]
        if kpre:
            by_name = self._by_name(params)
            key_rows = p["units"] * p["skv"]
            unit.define("CL_KPRE_ROWS", key_rows)
            unit.define("CL_KPRE_SRC", op["K"])
            unit.define("CL_KPRE_DST", "Scratch_kn")
            args = unit.signature("CL_KPRE_PARAMS", "CL_KPRE_NAME", ENTRY + "_keys", [by_name[op["K"]], by_name["Scratch_kn"]], ())
            unit.templates.append("rows_norm.hip")
            unit.launch(ENTRY + "_keys", (-(-(key_rows * (d // 8)) // 256), 1, 1), 256, 0, args)
        if partial:
            items = -(-(-(-rows // 128)) // 8) * 8              # padded to a multiple of 8 (one eighth of the space per XCD)
            unit.launch(ENTRY, (items, p["units"], splits), 256, 0, self._partial_args)
        if combine:
            entry, args = self._combine_args
            unit.launch(entry, (-(-(p["units"] * rows * (p["vdim"] // 4)) // 256), 1, 1), 256, 0, args)

    def _emit_attn_prefill(self, unit, plan, params, partial, combine, fused):
        if not plan.problem.get("paged"):
            return self._emit_attn_dense_prefill(unit, plan, params, partial, combine)
        """Causal prefill over ragged queries (token-table or packed keys): one item per 16-row tile
        (tokens x head group of one kv head), one wave per kv head."""
        p, op = plan.problem, plan.operands
        if combine or (plan.split_factor or 1) > 1:
            raise CodegenError("prefill has no split-KV form")
        emit_lse = bool(p.get("emit_lse"))
        self._attn_common(unit, plan, params, partial, combine, fused, p["vdim"], f"(total_q * {p['q_heads']})", emit_lse)
        d, group = p["head_dim"], p["group"]
        if d % 32 or not (d % 128 == 0 or d == 64) or 16 % group or p["kv_heads"] > 16:
            raise CodegenError("prefill needs head_dim 64 or k*128, a head group dividing 16 and at most 16 kv heads")
        for k, v in (("CL_HEAD_DIM", d), ("CL_KV_HEADS", p["kv_heads"]), ("CL_Q_HEADS", p["q_heads"]),
                     ("CL_RAGGED", bool(p["ragged"]))):
            unit.define(k, v)
        for role, macro in (("Q", "CL_ARG_Q"), ("K", "CL_ARG_K"), ("V", "CL_ARG_V"), ("QINDPTR", "CL_ARG_QINDPTR"),
                            ("INDPTR", "CL_ARG_INDPTR"), ("INDICES", "CL_ARG_INDICES")):
            if role in op:
                unit.define(macro, op[role])
        if int(plan.tiling.get("SHARED", 0)):
            # four waves share every key tile through LDS: 128 query rows per workgroup and kv head
            if d % 64 or d > 256:
                raise CodegenError("the LDS-shared prefill kernel needs a head dim of whole 64-feature panels (<= 256)")
            unit.templates.append("attn_prefill_lds.hip")
            for k, v in plan.tiling.items():
                if k != "SHARED":
                    unit.define(f"CL_PF_{k}", int(v))
            # the item axis is padded to a multiple of 8 so that the kernel can hand every XCD one
            # contiguous eighth of the (kv head, item) space
            items = f"ceildiv(ceildiv({p['dim_names']['total_q']}, {128 // group}) + batch, 8) * 8"
            unit.launch(ENTRY, (items, p["kv_heads"], 1), 256, 0, self._partial_args)
            return
        unit.templates.append("attn_prefill.hip")
        items = f"ceildiv({p['dim_names']['total_q']}, {16 // group}) + batch"
        unit.launch(ENTRY, (items, 1, 1), p["kv_heads"] * 64, 0, self._partial_args)

    def _emit_mla_decode(self, unit, plan, params, partial, combine, fused):
        p, t, op = plan.problem, plan.tiling, plan.operands
        if p.get("paged"):
            return self._emit_mla_paged(unit, plan, params, partial, combine, fused)
        total_rows = p["batch"] * p["heads"]
        emit_lse = bool(p.get("emit_lse"))
        self._attn_common(unit, plan, params, partial, combine, fused, p["ckv"], total_rows, emit_lse)
        if int(t.get("XW", 0)):
            # The cross-wave form (64 heads per workgroup, weights exchanged through LDS) was
            # withdrawn: it measured level with this kernel and its split form once returned a
            # wrong result whose cause was never found.
            raise CodegenError("tiling XW=1 (cross-wave MLA decode) is withdrawn; use WAVES/HG/VSPLIT/STAGES")
        if int(t.get("DUO", 0)):
            return self._emit_mla_duo(unit, plan, partial, combine, total_rows)
        waves, hg, stages = int(t.get("WAVES", 4)), int(t.get("HG", 1)), int(t.get("STAGES", 3))
        vsplit = int(t.get("VSPLIT", 1))
        if waves not in (1, 2, 4, 8):
            raise CodegenError("the MLA template runs 1, 2, 4 or 8 waves per workgroup")
        if waves % vsplit or p["heads"] % (16 * hg * waves // vsplit) or (p["ckv"] // 16) % (4 * vsplit):
            raise CodegenError(f"{p['heads']} heads / {p['ckv']} features do not divide into {waves} waves of "
                               f"{16 * hg} heads sharing a head set by {vsplit}")
        if p["ckv"] % 64 or p["kpe"] % 64:
            raise CodegenError("the MLA template loads 64-feature panels: latent and rope widths must be multiples of 64")
        for k, v in (("CL_HEADS", p["heads"]), ("CL_CKV", p["ckv"]), ("CL_KPE", p["kpe"]), ("CL_SKV", p["skv"]),
                     ("CL_WAVES", waves), ("CL_HG", hg), ("CL_STAGES", stages), ("CL_VSPLIT", vsplit),
                     ("CL_BATCH", p["batch"])):
            unit.define(k, v)
        if "LDS_AHEAD" in t:
            unit.define("CL_LDS_AHEAD", int(t["LDS_AHEAD"]))
        if "OCC" in t:
            unit.define("CL_OCC", int(t["OCC"]))
        # split partials of this family are stored in the element type (normalised per split)
        unit.define("CL_PO_ELEM", 1)
        unit.define("CL_SCALE_LOG2E", _f(float(p["scale"]) * LOG2E))
        for role, macro in (("Q", "CL_ARG_Q"), ("QPE", "CL_ARG_QPE"), ("KV", "CL_ARG_KV"), ("KPE", "CL_ARG_KPE")):
            if role in op:
                unit.define(macro, op[role])
        splits = plan.split_factor or 1
        unit.templates += ["mla_decode.hip", "attn_combine.hip"]
        if partial:
            grid = (p["batch"] * (p["heads"] // (16 * hg * waves // vsplit)), splits, 1)
            # the LDS images are a static array of the kernel: no dynamic LDS at launch
            unit.launch(ENTRY, grid, waves * 64, 0, self._partial_args)
        if combine:
            entry, args = self._combine_args
            unit.launch(entry, (-(-(total_rows * (p["ckv"] // 8)) // 256), 1, 1), 256, 0, args)


    def _emit_mla_duo(self, unit, plan, partial, combine, total_rows):
        """The score-wave / value-wave form of MLA decode: eight waves own 64 heads, four making the
        scores of 32 heads x half of each step's tokens, four the value products of 32 heads x half
        the latent features."""
        p, t, op = plan.problem, plan.tiling, plan.operands
        if p["heads"] % 64 or p["ckv"] % 128 or p["kpe"] % 64:
            raise CodegenError("the score-wave / value-wave MLA kernel needs heads % 64 == 0, a latent width in "
                               "multiples of 128 and a rope width in multiples of 64")
        from ..schedule.policy import mla_lds_bytes

        if mla_lds_bytes(p["ckv"], p["kpe"], 4) + 9 * 1024 > 160 * 1024:
            raise CodegenError("four images of the paired-wave MLA kernel do not fit LDS at these widths")
        for k, v in (("CL_HEADS", p["heads"]), ("CL_CKV", p["ckv"]), ("CL_KPE", p["kpe"]), ("CL_SKV", p["skv"]),
                     ("CL_BATCH", p["batch"]), ("CL_PO_ELEM", 1)):
            unit.define(k, v)
        if "LDS_AHEAD" in t:
            ahead = int(t["LDS_AHEAD"])
            if ahead < 2 or ahead % 2 or (p["ckv"] // 32) % (ahead // 2):
                raise CodegenError("LDS_AHEAD of the score-wave / value-wave MLA kernel: an even number of reads whose "
                                   "half divides the feature blocks of a value wave")
            unit.define("CL_LDS_AHEAD", ahead)
        if "S_AHEAD" in t:
            if not 1 <= int(t["S_AHEAD"]) <= (p["ckv"] + p["kpe"]) // 32:
                raise CodegenError("S_AHEAD: between 1 and the key fragments of a step")
            unit.define("CL_S_AHEAD", int(t["S_AHEAD"]))
        if "S_PANELS" in t:
            if not 0 <= int(t["S_PANELS"]) < (p["ckv"] + p["kpe"]) // 64:
                raise CodegenError("S_PANELS: the score waves can load between none and all but one of a step's 64-feature panels")
            unit.define("CL_S_PANELS", int(t["S_PANELS"]))
        unit.define("CL_SCALE_LOG2E", _f(float(p["scale"]) * LOG2E))
        for role, macro in (("Q", "CL_ARG_Q"), ("QPE", "CL_ARG_QPE"), ("KV", "CL_ARG_KV"), ("KPE", "CL_ARG_KPE")):
            if role in op:
                unit.define(macro, op[role])
        unit.templates += ["mla_decode_duo.hip", "attn_combine.hip"]
        if partial:
            unit.launch(ENTRY, (p["batch"] * (p["heads"] // 64), plan.split_factor or 1, 1), 512, 0, self._partial_args)
        if combine:
            entry, args = self._combine_args
            unit.launch(entry, (-(-(total_rows * (p["ckv"] // 8)) // 256), 1, 1), 256, 0, args)

    def _emit_mla_paged(self, unit, plan, params, partial, combine, fused):
        """Paged MLA decode (token table, page size 1): one wave per (work item, 16 heads); work
        items are requests (single kernel) or table slices of at most ``chunk_pages`` entries
        (split form, folded by the chunked combine)."""
        p, t, op = plan.problem, plan.tiling, plan.operands
        prefill = bool(p.get("prefill"))
        batch_name = "batch" if prefill else p["dim_names"]["batch"]
        emit_lse = bool(p.get("emit_lse"))
        rows = f"(total_q * {p['heads']})" if prefill else f"(batch * {p['heads']})"
        self._attn_common(unit, plan, params, partial, combine, fused, p["ckv"], rows, emit_lse)
        if prefill and (plan.split_factor or 1) > 1:
            raise CodegenError("prefill has no split-KV form")
        if p["heads"] % 16 or p["ckv"] % 64 or p["kpe"] % 64:
            raise CodegenError("paged MLA decode needs heads % 16 == 0 and latent / rope widths that are multiples of 64")
        chunked = (plan.split_factor or 1) > 1
        if chunked and not t.get("CHUNK_PAGES"):
            raise CodegenError("the split form of paged MLA decode is the chunked one (CHUNK_PAGES)")
        for k, v in (("CL_HEADS", p["heads"]), ("CL_CKV", p["ckv"]), ("CL_KPE", p["kpe"]), ("CL_CHUNKED", chunked),
                     ("CL_CHUNK_PAGES", chunked), ("CL_Q_HEADS", p["heads"]), ("CL_PREFILL", prefill)):
            unit.define(k, v)
        tok = int(t.get("TOK", 1)) if prefill else 1
        if tok not in (1, 2, 4):
            raise CodegenError("a paged MLA prefill item holds 1, 2 or 4 query tokens")
        if prefill:
            unit.define("CL_ARG_QINDPTR", op["QINDPTR"])
            unit.define("CL_MP_TOK", tok)
        if "LDS_AHEAD" in t:
            unit.define("CL_LDS_AHEAD", int(t["LDS_AHEAD"]))
        stages, ksplit = int(t.get("STAGES", 2)), int(t.get("KSPLIT", 1))
        panels = (p["ckv"] + p["kpe"]) // 64
        if ksplit not in (1, 2) or (ksplit > 1 and (chunked or tok != 1)):
            raise CodegenError("KSPLIT (two waves dealing an item's steps out between them) is 1 or 2, for the single kernel "
                               "with one query token per item")
        share = 1 if ksplit > 1 else tok
        if stages not in (2, 3, 4) or ksplit * stages * panels * 4096 > 160 * 1024 or (stages - 2) * (4 // share) * panels > 63:
            raise CodegenError(f"STAGES={stages} KSPLIT={ksplit}: two to four images of {panels * 4096} bytes per key-sharing "
                               "wave within 160 KiB of LDS, and at most 63 loads in flight behind the awaited step")
        unit.define("CL_MP_STAGES", stages)
        unit.define("CL_MP_KSPLIT", ksplit)
        for role, macro in (("Q", "CL_ARG_Q"), ("QPE", "CL_ARG_QPE"), ("KV", "CL_ARG_KV"), ("KPE", "CL_ARG_KPE"),
                            ("INDPTR", "CL_ARG_INDPTR"), ("INDICES", "CL_ARG_INDICES")):
            unit.define(macro, op[role])
        unit.templates += ["mla_paged_decode.hip", "attn_combine.hip"]
        if partial:
            items = f"ceildiv({p['dim_names']['n_idx']}, chunk_pages) + {batch_name}" if chunked else batch_name
            if prefill:
                items = f"ceildiv({p['dim_names']['total_q']}, {tok}) + batch"
            unit.launch(ENTRY, (items, p["heads"] // 16, 1), 64 * max(tok, ksplit), 0, self._partial_args)
        if combine:
            entry, args = self._combine_args
            unit.launch(entry, (f"ceildiv(({batch_name} * {p['heads']}) * {p['ckv'] // 4}, 256)", 1, 1), 256, 0, args)


def parse_manifest(source: str) -> dict:
    """The manifest a generated source carries (raises ``CodegenError`` when it has none)."""
    try:
        start = source.index(MANIFEST_BEGIN) + len(MANIFEST_BEGIN)
        end = source.index(MANIFEST_END)
    except ValueError:
        raise CodegenError("source has no kernel manifest: not produced by HipCodeGen") from None
    lines = [line[3:] if line.startswith("// ") else line.lstrip("/") for line in source[start:end].strip().splitlines()]
    try:
        return json.loads("\n".join(lines))
    except json.JSONDecodeError as e:
        raise CodegenError(f"kernel manifest is not valid JSON: {e}") from e


__all__ = ["HipCodeGen", "parse_manifest", "ENTRY", "COMBINE_ENTRY", "TEMPLATE_DIR"]
