"""``TileDict``: one tiling candidate (``python/cleave/schedule/policy/hint.py:7-38``)."""

from __future__ import annotations

from dataclasses import dataclass, field


@dataclass(eq=False)
class TileDict:
    template: str                 # gemm | gemm_dma | skinny | attn_decode | mla_decode
    role: str                     # main | partial | combine
    tiling: dict                  # template parameters (BM/BN/BK/WM/WN, WAVES, ...)
    output_tile: list = field(default_factory=list)
    rstep_map: dict = field(default_factory=dict)
    n_threads: int = 64
    split_factor: int | None = None
    score: float = 0.0            # modelled cost, lower is better
    lds_bytes: int = 0
    est_vgprs: int = 0
    flat_graph: object = field(default=None, repr=False)   # the StageGraph this tiles

    @property
    def label(self) -> str:
        knobs = " ".join(f"{k}={v}" for k, v in self.tiling.items())
        return f"{self.template}[{knobs}]" if knobs else self.template

    def key(self) -> tuple:
        return (self.template, self.role, self.split_factor, tuple(sorted(self.tiling.items())))
