"""``KernelPlan``: a tiling applied to its stage graph, i.e. everything codegen needs.

The reference's ``apply_tiling`` (``python/cleave/schedule/tiling.py:593-882``) rewrites the
flat graph into a grid tier plus loop tiers with per-node iterators.  Templates own their
loop structure here, so a scheduled plan is flat: template, role, problem, tiling, and the
kernel's parameter list in call order (inputs in graph order, run-time scalars, partial
buffers, outputs: the order of ``python/cleave/codegen/kernel.py:576-612``).
"""

from __future__ import annotations

from dataclasses import dataclass, field


@dataclass(frozen=True)
class ParamSpec:
    name: str
    dtype: str
    shape: tuple            # ints, or names of run-time dims
    role: str               # input | scalar | scratch | output
    alias: str | None = None  # scratch: the parameter whose allocation this one shares

    def to_json(self):
        d = {"name": self.name, "dtype": self.dtype, "shape": list(self.shape), "role": self.role}
        if self.alias:
            d["alias"] = self.alias
        return d

    @classmethod
    def from_json(cls, d):
        return cls(d["name"], d["dtype"], tuple(d["shape"]), d["role"], d.get("alias"))


@dataclass
class KernelPlan:
    template: str
    role: str               # main | partial | combine | fused
    family: str
    dtype: str
    problem: dict
    tiling: dict
    params: list            # list[ParamSpec] in call order
    operands: dict          # template operand role (A, B, Q, ...) -> parameter name
    split_factor: int | None = None
    dyn_dims: tuple = ()
    n_threads: int = 64
    lds_bytes: int = 0
    label: str = ""
    extra: dict = field(default_factory=dict)

    @property
    def inputs(self):
        return [p for p in self.params if p.role == "input"]

    @property
    def outputs(self):
        return [p for p in self.params if p.role == "output"]
