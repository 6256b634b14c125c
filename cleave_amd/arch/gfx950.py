"""Limits of one MI355X (gfx950, CDNA4) as the schedule search sees them.

Takes the place of the reference's CUDA description (``python/cleave/arch/cuda.py:121-183``:
164 KB shared memory, 65 536 registers, warp 32, 128-byte transactions, 132 SMs offline).
Nothing is inherited from it: wavefronts are 64 lanes, a compute unit has four SIMDs with
512 vector registers per lane each, a workgroup may own up to 160 KiB of LDS, the widest
global access is 16 bytes per lane (dwordx4), and the matrix cores take 16x16x32 and
32x32x16 f16/bf16 tiles with f32 accumulators.
"""

from __future__ import annotations

import dataclasses
import functools


@dataclasses.dataclass(frozen=True)
class Arch:
    name: str = "gfx950"
    compute_units: int = 256
    xcds: int = 8                       # accelerator dies, each with its own L2
    simds_per_cu: int = 4
    wavefront: int = 64
    max_threads_per_block: int = 1024
    vgprs_per_lane: int = 512           # arch + accumulation registers of one SIMD lane
    lds_bytes: int = 160 * 1024         # per workgroup (and per compute unit)
    lds_banks: int = 64
    max_vector_bytes: int = 16          # dwordx4 per lane
    l2_bytes: int = 4 * 1024 * 1024     # per XCD
    infinity_cache_bytes: int = 256 * 1024 * 1024
    hbm_bytes: int = 288 * 1024 ** 3
    hbm_gbps: float = 8000.0            # published peak, GB/s
    mfma_dense_tflops: float = 2516.6   # f16 / bf16 dense, published peak
    clock_ghz: float = 2.4
    # (M, N, K) of the f16/bf16 matrix-core tiles the templates are written for
    mfma_tiles: tuple = ((16, 16, 32), (32, 32, 16))

    @property
    def waves_per_simd_limit(self) -> int:
        return 8

    def waves_per_simd(self, vgprs: int) -> int:
        """Resident wavefronts per SIMD for a kernel using ``vgprs`` registers per lane."""
        vgprs = max(1, int(vgprs))
        granule = 8
        need = -(-vgprs // granule) * granule
        return max(0, min(self.waves_per_simd_limit, self.vgprs_per_lane // need))

    def blocks_per_cu(self, threads: int, lds_bytes: int, vgprs: int = 128) -> int:
        waves = -(-threads // self.wavefront)
        by_regs = (self.waves_per_simd(vgprs) * self.simds_per_cu) // max(1, waves)
        by_lds = self.lds_bytes // lds_bytes if lds_bytes else 32
        return max(0, min(by_regs, by_lds, 32))

    def describe(self) -> dict:
        return dataclasses.asdict(self)


GFX950 = Arch()


@functools.lru_cache(maxsize=None)
def get_arch(name: str = "gfx950") -> Arch:
    """The static description, with the CU count / LDS limit refined from the device when
    the native library and a GPU are both present."""
    base = name.split(":")[0]
    if base != "gfx950":
        raise ValueError(f"no description for {name!r}: this back end is written for gfx950 only")
    try:
        from ..runtime import shim

        if shim.available() and shim.device_count() > 0:
            info = shim.device_info(0)
            if info["arch_name"].startswith("gfx950"):
                return dataclasses.replace(GFX950, compute_units=info["compute_units"] or 256,
                                           lds_bytes=info["lds_bytes_per_block"] or GFX950.lds_bytes)
    except Exception:  # noqa: BLE001 - a probe failure leaves the published numbers in place
        pass
    return GFX950
