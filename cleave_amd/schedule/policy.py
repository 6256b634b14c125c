"""Launch-plan search space for gfx950 and the model that ranks it.

Stands where the reference's roller-style policy stands
(``python/cleave/schedule/policy/default.py:23-1110``): enumerate tilings, discard the ones
the hardware cannot hold, rank by a traffic x waves model, keep ``topk``.  Nothing of its
CUDA-shaped space is kept (warp 32, 64x32x32 wmma base tile, 164 KB shared memory, 128/256
threads).  The space here is written for one MI355X:

* 64-lane wavefronts, four SIMDs and 512 vector registers per lane per SIMD, up to 160 KiB of
  LDS per workgroup, 256 compute units;
* matrix-core tiles of 16x16x32 (f16/bf16, f32 accumulate), so every tile extent is a
  multiple of 16 and every contraction step a multiple of 32;
* 16-byte (dwordx4) global accesses: eight elements per lane, rows walked so that sixteen
  lanes cover 256 contiguous bytes;
* bandwidth-bound families (few-row matmul, decode attention) stream operands HBM -> registers
  and are tiled by *waves in flight*, not by LDS tiles; the split factor is what fills the
  256 compute units.
"""

from __future__ import annotations

import itertools
import math

from ..arch import Arch
from .hint import TileDict

ELEM_BYTES = {"float16": 2, "bfloat16": 2}


def _ceil(a, b):
    return -(-a // b)


def _waves_time(blocks, per_cu, arch: Arch):
    """Number of full passes the grid makes over the machine."""
    return _ceil(blocks, max(1, per_cu * arch.compute_units))


# ----------------------------------------------------------------------------- GEMM
def gemm_lds_bytes(bm, bn, bk, norm=False):
    return 2 * (bm + bn) * bk * 2 + (bm * 4 if norm else 0)


def gemm_candidates(low, role, factor, arch: Arch):
    p = low.problem
    splits = factor or 1
    M, N, K = p["M"], p["N"], p["K"]
    if K % splits:
        return []
    kps = K // splits
    batch = max(p["batch_A"], p["batch_B"])
    norm = low.family == "rmsnorm_matmul"
    out = []
    shapes = (16, 32, 64, 128, 256)
    for bm, bn, bk, (wm, wn), depth in itertools.product(
            shapes, shapes, (64,), ((1, 1), (1, 2), (2, 1), (2, 2), (1, 4), (4, 1), (2, 4), (4, 2)), (1, 2)):
        if bm % (16 * wm) or bn % (16 * wn):
            continue
        if kps % bk and (splits > 1 or K % 8):       # a ragged last step: unsplit, rows of whole 16-byte chunks
            continue
        if bm > max(16, 2 * M) or bn > max(16, 2 * N):
            continue
        threads = wm * wn * 64
        tm, tn = bm // wm // 16, bn // wn // 16
        acc_regs = tm * tn * 4
        if acc_regs > 256:
            continue
        if p["trans_A"] and (bm % 8 or M % 8):
            continue
        if not p["trans_B"] and (bn % 8 or N % 8):
            continue
        # staging registers per thread and step in flight: K-minor tiles move 16-byte chunks (4
        # registers), K-major ones 8x8 blocks (32) or, when those would idle threads, 4x8 halves (16)
        def stage(rows, k_major):
            if not k_major:
                return _ceil(rows * (bk // 8), threads) * 4
            blocks = (rows // 8) * (bk // 8)
            if rows % 64 == 0 and blocks < threads:
                return _ceil(2 * blocks, threads) * 16
            return _ceil(blocks, threads) * 32
        stage_regs = depth * (stage(bm, p["trans_A"]) + stage(bn, not p["trans_B"]))
        frag_regs = (min(tm, 3) + 2 * tn) * 4
        vgprs = acc_regs + stage_regs + frag_regs + 40
        if vgprs > arch.vgprs_per_lane:
            continue
        lds = gemm_lds_bytes(bm, bn, bk, norm)
        if lds > arch.lds_bytes:
            continue
        blocks = _ceil(M, bm) * _ceil(N, bn) * batch * splits
        per_cu = arch.blocks_per_cu(threads, lds, vgprs)
        if per_cu < 1:
            continue
        if depth == 2 and (_ceil(kps, bk) < 4 or per_cu * threads > 512 and vgprs > 128):
            continue
        passes = _waves_time(blocks, per_cu, arch)
        live = min(per_cu, _ceil(blocks, arch.compute_units))         # blocks a CU really holds
        # one pass over the machine: the CU's matrix cores, its L1 path (about 24 B/clk sustained
        # for these access shapes) and its LDS are shared by the blocks it holds
        mfma_clk = live * (bm * bn * kps * 2) / 4096.0 / min(1.0, live * wm * wn / 8.0)
        l1_clk = live * ((bm + bn) * kps * 2) / (24.0 * (1.6 if depth == 2 else 1.0))
        lds_clk = live * (tm + tn) * 16 * wm * wn * kps * 2 / 256.0
        pass_clk = max(mfma_clk, l1_clk, lds_clk) + 2500 + 1200 * _ceil(kps, bk) / max(1, min(live, 2))
        score = passes * pass_clk
        # (where the direct-to-LDS kernel offers the same tile it has measured a quarter to two thirds
        # faster -- 2048 x 4096 x 4096 on 128 x 128 tiles: 67 against 91 us; 512 x 512 x 4096 on 16 x 32 tiles:
        # 14 against 42 -- while this model ranked the register-staged one ahead: its candidates go behind)
        if low.family == "matmul":
            score *= 2.0
        tiling = dict(BM=bm, BN=bn, BK=bk, WM=wm, WN=wn, GDEPTH=depth)
        out.append(TileDict("gemm", role, tiling, output_tile=[bm, bn], rstep_map={"k": bk}, n_threads=threads,
                            split_factor=factor, score=score, lds_bytes=lds, est_vgprs=vgprs))
    return out


def gemm_dma_candidates(low, role, factor, arch: Arch):
    """Tilings of the direct-to-LDS matmul: the plain matmul, and the RMSNorm -> matmul without a
    learned weight, unsplit (the norm then scales the product's rows; with a weight the operand
    would have to pass through registers on its way to LDS).  No staging registers, so the budget is accumulators plus two
    k blocks of operand fragments; tiles whose accumulators would fill a whole register class
    (256) are left out: the compiler then shuffles them on every step."""
    p = low.problem
    splits = factor or 1
    post_norm = low.family == "rmsnorm_matmul" and not p.get("gamma") and not p["trans_A"] and splits == 1 \
        and role == "main"
    if low.family != "matmul" and not post_norm:
        return []
    M, N, K = p["M"], p["N"], p["K"]
    if K % (splits * 64) or (not p["trans_B"] and N % 8) or (p["trans_A"] and M % 8):
        return []
    kps = K // splits
    batch = max(p["batch_A"], p["batch_B"])
    out = []
    shapes = (16, 32, 64, 128, 256)
    for bm, bn, (wm, wn) in itertools.product(
            shapes, shapes, ((1, 1), (1, 2), (2, 1), (2, 2), (1, 4), (4, 1), (2, 4), (4, 2))):
        if bm % (16 * wm) or bn % (16 * wn):
            continue
        if bm > max(16, 2 * M) or bn > max(16, 2 * N):
            continue
        threads = wm * wn * 64
        tm, tn = bm // wm // 16, bn // wn // 16
        if tm & (tm - 1) or tn & (tn - 1) or tm * tn * 4 > 128:
            continue
        if post_norm and low.dtype == "bfloat16" and tm * tn * 4 > 64 and wm > wn:
            continue      # bf16 squares go through float conversions: beside a 128-register, 4-row-fragment tile they spill
        # every wave must own whole 1 KiB load units of both tiles or none
        units_a, units_b = bm // 8, bn // 8
        vgprs = tm * tn * 4 + (tm + tn) * 6 + -(-units_a // (wm * wn)) + -(-units_b // (wm * wn)) + 24
        if vgprs > arch.vgprs_per_lane:
            continue
        lds = gemm_lds_bytes(bm, bn, 64)
        if lds > arch.lds_bytes:
            continue
        blocks = _ceil(M, bm) * _ceil(N, bn) * batch * splits
        per_cu = arch.blocks_per_cu(threads, lds, vgprs)
        if per_cu < 1:
            continue
        passes = _waves_time(blocks, per_cu, arch)
        live = min(per_cu, _ceil(blocks, arch.compute_units))
        mfma_clk = live * (bm * bn * kps * 2) / 4096.0 / min(1.0, live * wm * wn / 8.0)
        # LDS -> register traffic: about 32 B/clk per SIMD for 16-byte reads, two thirds of that for
        # the transposing reads of a K-major operand
        a_rate = 21.0 if p["trans_A"] else 32.0
        b_rate = 32.0 if p["trans_B"] else 21.0
        waves_per_simd = max(1.0, live * wm * wn / 4.0)
        lds_clk = waves_per_simd * kps * 2 * 16 * (tm / a_rate + tn / b_rate)
        fetch_clk = live * ((bm + bn) * kps * 2) / 24.0
        pass_clk = max(mfma_clk, lds_clk, fetch_clk) + 2500 + 1500 * (kps // 64) / max(1, min(live, 2))
        # (equal tiles: the wave grids with more waves have measured a few per cent faster -- more loads in flight)
        score = passes * pass_clk * (1.0 + 0.03 / (wm * wn))
        tiling = dict(BM=bm, BN=bn, BK=64, WM=wm, WN=wn)
        out.append(TileDict("gemm_dma", role, tiling, output_tile=[bm, bn], rstep_map={"k": 64}, n_threads=threads,
                            split_factor=factor, score=score, lds_bytes=lds, est_vgprs=vgprs))
        # Three LDS stages where three images fit beside as many workgroups per compute unit as two
        # allow: the loads of a step asked for two steps ahead and spread over the whole step
        # (256 x 128 tiles on 4096 x 14336 x 4096: 426 us against 526).
        if (3 * (bm + bn) * 128 * per_cu <= arch.lds_bytes and units_a % (wm * wn) == 0 and units_b % (wm * wn) == 0
                and not post_norm):
            out.append(TileDict("gemm_dma", role, dict(tiling, STAGES=3), output_tile=[bm, bn], rstep_map={"k": 64},
                                n_threads=threads, split_factor=factor, score=0.85 * score, lds_bytes=3 * lds // 2,
                                est_vgprs=vgprs))
        # A last round that fills at most half of the machine: its tiles as two half-height
        # workgroups each (row-major A, one workgroup per compute unit, unsplit, unbatched).
        tail = blocks % arch.compute_units
        if (blocks > arch.compute_units and 0 < tail <= arch.compute_units // 2 and per_cu == 1 and splits == 1
                and batch == 1 and not p["trans_A"] and tm >= 2 and M % bm == 0):
            out.append(TileDict("gemm_dma", role, dict(tiling, TAIL=tail), output_tile=[bm, bn], rstep_map={"k": 64},
                                n_threads=threads, split_factor=factor, score=(passes - 0.45) * pass_clk,
                                lds_bytes=lds, est_vgprs=vgprs))
    return out


def swiglu_candidates(low, role, factor, arch: Arch):
    """SwiGLU runs on the direct-to-LDS matmul with a B tile made of two halves, the same
    columns of the bare weight and of the gate weight: the tilings of a matmul twice as wide in
    which every wave owns an even number of column fragments (half of them per weight)."""
    import copy

    if factor and factor > 1:
        return []
    twin = copy.copy(low)
    twin.family, twin.problem = "matmul", dict(low.problem, N=2 * low.problem["N"])
    out = []
    for c in gemm_dma_candidates(twin, role, None, arch):
        t = c.tiling
        tn = t["BN"] // t["WN"] // 16
        if tn % 2 or low.problem["N"] % (t["BN"] // 2):
            continue
        c.tiling = dict(t, SWIGLU=1)
        c.output_tile = [t["BM"], t["BN"] // 2]
        out.append(c)
    return out


def rowsum_candidates(low, role, factor, arch: Arch):
    """Matmul + row sum: tilings of the direct-to-LDS matmul in which one workgroup owns BM rows and
    walks all of N (whole column tiles), so the grid is the row tiles alone: ranked by how many
    step sequences of ``(N / BN) * (K / 64)`` steps the machine runs one after another."""
    import copy

    if factor and factor > 1:
        return []
    p = low.problem
    twin = copy.copy(low)
    twin.family = "matmul"
    out = []
    for c in gemm_dma_candidates(twin, role, None, arch):
        t = c.tiling
        if p["N"] % t["BN"]:
            continue
        blocks = _ceil(p["M"], t["BM"])
        steps = (p["N"] // t["BN"]) * (p["K"] // 64)
        waves = t["WM"] * t["WN"]
        mfma_clk = (t["BM"] // t["WM"] // 16) * (t["BN"] // t["WN"] // 16) * 2 * 16.4 * max(1.0, waves / 4.0)
        c.score = _waves_time(blocks, 1, arch) * steps * (mfma_clk + 700)
        c.tiling = dict(t, ROWSUM=1)
        c.output_tile = [t["BM"], 1]
        out.append(c)
    return out


def lora_lds_bytes(mt, waves_n, waves_k, rank):
    """The few-row kernel's reduction buffers twice (main and rank-R accumulators) plus the D tile."""
    return 2 * skinny_lds_bytes(mt, waves_n, waves_k) + waves_n * 16 * mt * rank * 4 + 16


def lora_candidates(low, role, factor, arch: Arch):
    """LoRA: the few-row matmul with the rank-R product ``x @ a`` riding along.  Unsplit, the epilogue
    applies the rank update; split over K, the partial kernel writes partial sums of both products
    and the combine applies it (it needs the whole of ``x @ a``)."""
    import copy

    p = low.problem
    if p["R"] % 8 or p["R"] > 64 or ((factor or 1) > 1 and p["N"] % 256):
        return []
    twin = copy.copy(low)
    twin.family = "matmul"
    if not skinny_ok(twin):
        return []
    out = []
    for c in skinny_candidates(twin, role, factor, arch):
        t = c.tiling
        lds = lora_lds_bytes(_ceil(p["M"], 16), t["WAVES_N"], t["WAVES_K"], p["R"])
        if lds > arch.lds_bytes:
            continue
        c.tiling, c.lds_bytes = dict(t, LORA=1), lds
        if t["WAVES_N"] * t["WAVES_K"] > 4:
            # more than four waves have 256 registers each: the ring of tiles (each now carries a block
            # of the rank-R factor too) is one tile shallower so that nothing spills
            c.tiling["PREFETCH"] = 1
        out.append(c)
    return out


def rowsum_only_candidates(low, role, factor, arch: Arch):
    """Row reductions: one wave per row, 1, 2 or 4 rows per workgroup; the cost is the stream."""
    p = low.problem
    if (factor or 1) > 1 or p["N"] % 8:
        return []
    out = []
    for rows in (4, 2, 1):
        blocks = _ceil(p["M"], rows)
        nbytes = p["M"] * p["N"] * 2 * (3 if p["div"] else 1)
        score = nbytes / (arch.hbm_gbps * 1e3 * 0.6) * 2400 + 3000 + 200 * _waves_time(blocks, 8, arch) + rows
        out.append(TileDict("rowsum", role, dict(ROWS_PER_BLOCK=rows), output_tile=[rows, p["N"] if p["div"] else 1],
                            rstep_map={"n": 512}, n_threads=64 * rows, split_factor=factor, score=score, lds_bytes=0,
                            est_vgprs=40))
    return out


# ----------------------------------------------------------------------------- few-row matmul
def skinny_ok(low) -> bool:
    p = low.problem
    return (p["M"] <= 64 and not p["trans_A"] and not p["trans_B"] and p["batch_A"] == 1 and p["batch_B"] == 1
            and p["K"] % 32 == 0 and p["N"] % 8 == 0 and p["N"] >= 8)


def skinny_lds_bytes(mt, waves_n, waves_k):
    return ((waves_k - 1) * waves_n * mt * 32 * 64 + waves_k * mt * 16) * 4 + 16


def skinny_candidates(low, role, factor, arch: Arch):
    p = low.problem
    splits = factor or 1
    M, N, K = p["M"], p["N"], p["K"]
    mt = _ceil(M, 16)
    steps = K // 32
    if steps % splits:
        return []
    out = []
    for waves_n, waves_k in itertools.product((1, 2, 4), (1, 2, 4, 8)):
        threads = waves_n * waves_k * 64
        if threads > 1024:
            continue
        per_split = steps // splits
        if per_split < waves_k:
            continue
        lds = skinny_lds_bytes(mt, waves_n, waves_k)
        if lds > arch.lds_bytes:
            continue
        vgprs = mt * 32 + 3 * 32 + 32 + mt * 4 + 40
        blocks = _ceil(N, 128 * waves_n) * splits
        per_cu = arch.blocks_per_cu(threads, max(lds, 1), vgprs)
        if per_cu < 1:
            continue
        passes = _waves_time(blocks, per_cu, arch)
        waves_live = min(blocks, per_cu * arch.compute_units) * waves_n * waves_k
        # a wave keeps ~3 steps of 8 KiB in flight; HBM wants ~16 MiB outstanding machine-wide
        inflight = waves_live * 24 * 1024
        bw_frac = min(1.0, inflight / (12 * 1024 * 1024))
        stream_us = (K * N * 2) / (arch.hbm_gbps * 1e3 * bw_frac)
        partial_us = (2 * splits * M * N * 4) / (arch.hbm_gbps * 1e3) if splits > 1 else 0.0
        tail = 1.0 + 0.25 * (passes - 1) + 0.02 * waves_k
        score = (stream_us * tail + partial_us) * 2400
        tiling = dict(WAVES_N=waves_n, WAVES_K=waves_k)
        out.append(TileDict("skinny", role, tiling, output_tile=[M, 128 * waves_n], rstep_map={"k": 32},
                            n_threads=threads, split_factor=factor, score=score, lds_bytes=lds, est_vgprs=vgprs))
    return out


# ----------------------------------------------------------------------------- decode attention
def attn_lds_bytes(waves, vdim):
    """LDS of the streaming decode kernel: every wave but the first parks its accumulators (a 16-byte piece per
    lane and accumulator, eight accumulators per 128 value features) and its 16 reference points and sums."""
    return (waves - 1) * (-(-vdim // 128) * 8 * 64 * 16 + 128)


def attn_ok(low) -> bool:
    p = low.problem
    return p["head_dim"] % 32 == 0 and (p["vdim"] % 128 == 0 or p["vdim"] == 64)


def attn_candidates(low, role, factor, arch: Arch, waves_options=(1, 2, 4, 8)):
    p = low.problem
    splits = factor or 1
    rows = p["group"] * p["sq"]
    row_tiles = _ceil(rows, 16)
    d, vd = p["head_dim"], p["vdim"]
    steps = _ceil(p["skv"], 32)
    out = []
    for waves in waves_options:
        lds = attn_lds_bytes(waves, vd)
        if lds > arch.lds_bytes:
            continue
        kv_regs = (2 * (d // 32) + 8 * _ceil(vd, 128)) * 4
        vgprs = 2 * kv_regs + 32 * _ceil(vd, 128) + 4 * (d // 32) + 32 + 48
        if vgprs > arch.vgprs_per_lane:
            continue
        blocks = p["units"] * row_tiles * splits
        per_cu = arch.blocks_per_cu(waves * 64, lds, vgprs)
        if per_cu < 1:
            continue
        passes = _waves_time(blocks, per_cu, arch)
        steps_per_wave = _ceil(_ceil(steps, splits), waves)
        waves_live = min(blocks, per_cu * arch.compute_units) * min(waves, _ceil(steps, splits))
        inflight = waves_live * 2 * kv_regs * 64 * 4 / 2
        # (measured on the 8192-key decode: 512 one-wave workgroups with one 16 KB step in flight each stream at
        # the rate of the box; two and four waves per workgroup take 7 % and 20 % longer)
        bw_frac = min(1.0, inflight / (8 * 1024 * 1024))
        bytes_total = p["units"] * row_tiles * p["skv"] * (d + vd) * 2
        stream_us = bytes_total / (arch.hbm_gbps * 1e3 * bw_frac) * (1.0 + 0.07 * math.log2(waves) ** 1.5)
        ramp_us = 1.5                                    # fixed launch + drain cost
        partial_us = (2 * splits * p["units"] * rows * (vd + 2) * 4) / (arch.hbm_gbps * 1e3) if splits > 1 else 0.0
        score = (stream_us * (1.0 + 0.2 * (passes - 1)) + ramp_us + partial_us + 0.05 * waves) * 2400
        tiling = dict(WAVES=waves)
        out.append(TileDict("attn_decode", role, tiling, output_tile=[16, vd], rstep_map={"kv": 32},
                            n_threads=waves * 64, split_factor=factor, score=score, lds_bytes=lds, est_vgprs=vgprs))
        # split ranges spread over the XCDs and skewed between even and odd ones (measured on the 8192-key
        # decode: with all splits of a unit on one XCD the kernel ends with its slowest XCD, 4-5 % later)
        if splits > 1 and splits % 2 == 0 and waves <= 2 and (p["units"] * row_tiles) % 8 == 0 and steps >= 4 * splits:
            for skew in (30, 60):
                out.append(TileDict("attn_decode", role, dict(WAVES=waves, SKEW=skew), output_tile=[16, vd],
                                    rstep_map={"kv": 32}, n_threads=waves * 64, split_factor=factor,
                                    score=score * (0.96 if skew == 30 else 0.965), lds_bytes=lds, est_vgprs=vgprs))
        # a second step of loads in flight (measured on the 8192-key decode: with about two waves per CU
        # streaming, the deeper ring is worth a few percent; with many waves it is not)
        if waves <= 2 and vgprs + kv_regs <= arch.vgprs_per_lane and steps_per_wave >= 8:
            out.append(TileDict("attn_decode", role, dict(WAVES=waves, PREFETCH=2), output_tile=[16, vd],
                                rstep_map={"kv": 32}, n_threads=waves * 64, split_factor=factor, score=score * 1.001,
                                lds_bytes=lds, est_vgprs=vgprs + kv_regs))
    return out


def attn_many_rows_candidates(low, role, factor, arch: Arch):
    """Units with many query rows (prefill-shaped dense attention): the kernel whose four waves
    share every key tile through LDS, 128 query rows per workgroup, instead of one 16-row tile per
    workgroup streaming all keys.  Key and value widths in 64-feature panels; split over the keys
    (ranges of whole 32-key steps, f32 partials) when there are too few units and rows to fill the chip."""
    p = low.problem
    rows, d = p["group"] * p["sq"], p["head_dim"]
    vd = p["vdim"]
    splits = factor or 1
    # plain softmax attention with few rows per unit belongs to the streaming decode kernel; QK-norm, the
    # chained matmul and widths the streaming kernel has no form for (a 192-wide value) exist in this
    # kernel only, so there it takes units of any height (one workgroup per unit, most of its 128 rows masked)
    only_here = bool(p.get("norm_eps") or p.get("linear")) or not attn_ok(low)
    if (rows < 64 and not only_here) or d % 64 or d > 256 or vd % 64 or vd > 256 or p["skv"] < 1:
        return []
    if splits > 1 and p.get("emit_lse"):
        return []
    if p.get("k_major") and p["skv"] % 32:       # feature-major keys are loaded in whole 32-key steps
        return []
    items = p["units"] * _ceil(rows, 128) * splits
    steps = _ceil(_ceil(p["skv"], 32), splits)
    # a workgroup-step is 32 matrix ops per wave beside as many vector ops; two workgroups per CU
    score = _waves_time(items, 2, arch) * (steps * 2200 + 9000)
    out = [TileDict("attn_prefill", role, dict(SHARED=1), output_tile=[128, vd], rstep_map={"kv": 32}, n_threads=256,
                    split_factor=factor, score=score, lds_bytes=4 * 32 * (d + vd) * 2, est_vgprs=230)]
    # normalised keys: every workgroup of a unit normalises all of its keys again (a quarter more
    # matrix ops per step and the scaling of the scores); with many row blocks per unit a launch
    # that normalises them once into a scratch copy is cheaper
    if "k" in (p.get("norm_eps") or {}) and not p.get("k_major") and d in (64, 128, 256) and rows >= 512:
        out.append(TileDict("attn_prefill", role, dict(SHARED=1, KPRE=1), output_tile=[128, vd], rstep_map={"kv": 32},
                            n_threads=256, split_factor=factor, score=0.8 * score, lds_bytes=4 * 32 * (d + vd) * 2,
                            est_vgprs=230))
    return out


# ----------------------------------------------------------------------------- MLA decode
def mla_lds_bytes(ckv, kpe, stages=3):
    """`stages` token-major images of a 32-token step: (ckv + kpe) / 64 panels of 32 x 64 elements."""
    return stages * ((ckv + kpe) // 64) * 32 * 64 * 2


def mla_ok(low) -> bool:
    p = low.problem
    return p["heads"] % 16 == 0 and p["ckv"] % 64 == 0 and p["kpe"] % 64 == 0


def mla_candidates(low, role, factor, arch: Arch):
    p = low.problem
    splits = factor or 1
    out = []
    d = p["ckv"] + p["kpe"]
    for waves, (hg, vsplit), stages in itertools.product((1, 2, 4, 8), ((1, 1), (2, 2)), (2, 3, 4)):
        # 32 heads per wave only with the value features shared out over a wave pair: the
        # accumulators of 32 heads x all features would fill a whole register class
        if waves % vsplit or (p["ckv"] // 16) % (4 * vsplit):
            continue
        heads_per_block = 16 * hg * waves // vsplit
        if p["heads"] % heads_per_block:
            continue
        lds = mla_lds_bytes(p["ckv"], p["kpe"], stages)
        if lds > arch.lds_bytes:
            continue
        units_per = (d // 64) * 4 // min(waves, 4)
        if (stages - 2) * units_per >= 64:        # the wait for a step's loads counts the younger ones
            continue
        # Q fragments and accumulators of a wave's heads stay in registers for the whole split
        # (plus the ring of LDS operand reads and the softmax state); loads use no registers
        vgprs = hg * (d // 32 * 4 + p["ckv"] // 16 * 4 // vsplit + 4) + 32 + 24
        if vgprs > arch.vgprs_per_lane:
            continue
        blocks = p["batch"] * (p["heads"] // heads_per_block) * splits
        per_cu = arch.blocks_per_cu(waves * 64, lds, vgprs)
        if per_cu < 1:
            continue
        passes = _waves_time(blocks, per_cu, arch)
        steps = _ceil(_ceil(p["skv"], 32), splits)
        # per step and wave: the score operands are 1 KiB reads at about 32 B/clk and SIMD, the
        # value operands transposing reads at about two thirds of that; each feeds hg matrix ops
        score_reads, value_reads = 2 * (d // 32), p["ckv"] // 16 // vsplit
        mfma_clk = (score_reads + value_reads + 1) * hg * 18
        lds_clk = (score_reads * 32 + value_reads * 48) * 0.45     # measured: LDS reads hide under the matrix ops
        simd_share = max(1.0, per_cu * waves / 4.0)
        # measured: the matrix ops of a step plus about 1500 clocks that nothing overlaps (barrier,
        # load issue, the softmax between the two products); per workgroup of heads_per_block heads
        step_clk = (max(mfma_clk, lds_clk) * simd_share / per_cu + 1500) * (64.0 / heads_per_block)
        util = min(1.0, blocks / (per_cu * arch.compute_units))
        # a step's loads have (stages - 1) steps of matrix work to arrive in
        latency_clk = 4000.0 / (stages - 1)
        step_clk = max(step_clk, latency_clk)
        # split partials go out and come back once (element type): 2 * splits * rows * ckv * 2 bytes
        partial_clk = (4 * splits * p["batch"] * p["heads"] * p["ckv"]) / (arch.hbm_gbps * 1e3 * 0.6) * 2400 \
            if splits > 1 else 0.0
        score = passes * steps * step_clk * (1.0 + 0.3 * (1 - util)) + 8000 + partial_clk
        out.append(TileDict("mla_decode", role, dict(WAVES=waves, HG=hg, VSPLIT=vsplit, STAGES=stages),
                            output_tile=[heads_per_block, p["ckv"]], rstep_map={"kv": 32}, n_threads=waves * 64,
                            split_factor=factor, score=score, lds_bytes=lds, est_vgprs=vgprs))
    # The score-wave / value-wave form: eight waves own 64 heads, every LDS operand feeds two matrix
    # ops.  Measured 25-30 % ahead of the best form above wherever both run, so it is ranked first
    # (with the shorter read-ahead of its value operands as a second candidate).
    duo_lds = mla_lds_bytes(p["ckv"], p["kpe"], 4) + 9 * 1024
    if out and p["heads"] % 64 == 0 and p["ckv"] % 128 == 0 and duo_lds <= arch.lds_bytes:
        best = min(c.score for c in out)
        # (third: the score waves ask for about half of every image's panels -- a wave that waits for the
        # path into the compute unit does not hold up the other wave of its SIMD, and the value
        # waves are the longer chain of a step; measured 1-2 % ahead)
        shared = max(1, (p["ckv"] + p["kpe"]) // 64 // 2)
        for tiling, rel in ((dict(DUO=1), 0.75), (dict(DUO=1, LDS_AHEAD=4), 0.76),
                            (dict(DUO=1, LDS_AHEAD=4, S_PANELS=shared), 0.755)):
            out.append(TileDict("mla_decode", role, tiling, output_tile=[64, p["ckv"]], rstep_map={"kv": 32},
                                n_threads=512, split_factor=factor, score=rel * best, lds_bytes=duo_lds, est_vgprs=208))
    return out


# ----------------------------------------------------------------------------- combine kernels
def combine_candidates(low, factor, arch: Arch):
    """The combine of a split has one shape: one thread per 4 (attention) or 4/8 (matmul)
    output columns, 256 threads; it is memory-trivial next to its partial."""
    family = {"matmul": "gemm", "rmsnorm_matmul": "gemm", "lora": "gemm", "attention": "attn_decode",
              "mla": "mla_decode"}[low.family]
    return [TileDict(family, "combine", {}, output_tile=[1, 256], rstep_map={"split": factor}, n_threads=256,
                     split_factor=factor, score=1.0, lds_bytes=0, est_vgprs=32)]
