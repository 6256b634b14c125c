"""Workload axes of the shipped paged operators and the request lengths derived from them.

The reference ships axes captured from SOL-ExecBench runs as ``wl_<batch>_<num_pages>_<n_idx>``
(``python/cleave/dynamic/workloads.py:15-326``) and synthesises per-request lengths from them
deterministically (``:329-361``).  The four axes of each operator below are the ones its
checked-in H100 baseline names (``tests/perf/baselines/h100-80gb-hbm3.json``); length
synthesis follows the same scheme: ``n_idx`` split into ``batch`` positive page counts by a
generator seeded with ``crc32(repr((operator, axes)))``, every page full but the last.
"""

from __future__ import annotations

import random
import zlib

WORKLOADS = {
    "gqa_paged_decode_h32_kv8_d128_ps1": ((1, 11, 10), (16, 1069, 1034), (16, 81390, 12942), (64, 68237, 58966)),
    "gqa_paged_decode_h32_kv4_d128_ps1": ((1, 8, 7), (16, 1070, 1020), (16, 32348, 23079), (64, 61535, 61519)),
    "gqa_paged_decode_h32_kv8_d128_ps64": ((4, 349, 212), (16, 1686, 1033), (32, 15178, 14103), (128, 52033, 47438)),
    "mla_paged_decode_h16_ckv512_kpe64_ps1": ((1, 989669, 8), (16, 989669, 457), (64, 989669, 9945),
                                              (64, 989669, 75145)),
    # causal prefill: (batch, total_q, n_idx, num_pages) with a token table, (batch, total_q, total_kv) packed
    "gqa_paged_prefill_causal_h32_kv8_d128_ps1": ((1, 1, 34, 51), (12, 7009, 30, 70149), (1, 10447, 1, 2),
                                                  (52, 10749, 99, 20585)),
    "gqa_paged_prefill_causal_h32_kv4_d128_ps1": ((1, 1, 33, 50), (1, 1210, 1, 176707), (27, 15344, 48, 556622),
                                                  (63, 14263, 142, 626709)),
    "gqa_ragged_prefill_causal_h32_kv8_d128": ((1, 1, 1), (1, 35, 35), (36, 12845, 12845), (10, 12571, 12571)),
    "gqa_ragged_prefill_causal_h32_kv4_d128": ((1, 1, 1), (1, 34, 34), (15, 969, 969), (33, 16294, 16294)),
    "mla_paged_prefill_causal_h16_ckv512_kpe64_ps1": ((1, 1, 34, 989669), (4, 4, 121, 989669), (1, 96, 98, 989669),
                                                      (56, 8987, 14390, 989669)),
}

# The softmax scale the reference's MLA operators are run at (``python/cleave/dynamic/workloads.py:12-13``).
MLA_SM_SCALE = 0.1352337747812271

# Geomean latency over exactly those axes on the reference's own back end, as recorded in its
# checked-in baseline (``tests/perf/baselines/h100-80gb-hbm3.json``, NVIDIA H100 80GB HBM3, bf16):
# microseconds per axis in the order above.  Quoted beside this back end's numbers, never a target.
REFERENCE_H100_US = {
    "gqa_paged_decode_h32_kv8_d128_ps1": (2.4898, 5.2114, 59.4166, 137.0866),
    "gqa_paged_decode_h32_kv4_d128_ps1": (2.4530, 5.0890, 80.3984, 131.4043),
    "gqa_paged_decode_h32_kv8_d128_ps64": (74.0303, 149.6087, 1667.6903, 4817.6807),
    "mla_paged_decode_h16_ckv512_kpe64_ps1": (5.8886, 8.6802, 35.6304, 258.9872),
    "gqa_paged_prefill_causal_h32_kv8_d128_ps1": (3.9, 24.7, 31.4, 39.9),
    "gqa_paged_prefill_causal_h32_kv4_d128_ps1": (3.8, 5.7, 49.0, 50.2),
    "gqa_ragged_prefill_causal_h32_kv8_d128": (3.6, 4.0, 444.9, 663.6),
    "gqa_ragged_prefill_causal_h32_kv4_d128": (3.6, 4.0, 25.8, 548.5),
    "mla_paged_prefill_causal_h16_ckv512_kpe64_ps1": (5.6, 5.7, 8.8, 795.4),
}


def _rng(operator, axes):
    return random.Random(zlib.crc32(repr((operator, axes)).encode()))


def _positive(total, parts, rng):
    """``total`` split into exactly ``parts`` positive integers."""
    cuts = sorted(rng.sample(range(1, total), parts - 1)) if parts > 1 else []
    bounds = [0, *cuts, total]
    return [b - a for a, b in zip(bounds, bounds[1:])]


def _tokens(pages, page_size, rng):
    return [(n - 1) * page_size + (page_size if page_size == 1 else rng.randint(1, page_size)) for n in pages]


def decode_lengths(operator, axes, page_size):
    """``(batch, num_pages, n_idx, kv_lens)`` of one captured decode workload."""
    batch, pool, n_idx = axes
    rng = _rng(operator, axes)
    batch = min(batch, n_idx)
    kv_lens = _tokens(_positive(n_idx, batch, rng), page_size, rng)
    return batch, max(pool, n_idx), n_idx, kv_lens


def _nonnegative(total, parts, rng):
    cuts = sorted(rng.randrange(total + 1) for _ in range(parts - 1))
    bounds = [0, *cuts, total]
    return [b - a for a, b in zip(bounds, bounds[1:])]


def prefill_lengths(operator, axes):
    """``(batch, q_lens, kv_lens)`` of one captured prefill workload
    (``python/cleave/dynamic/workloads.py:362-378``): the query run is cut into positive lengths;
    with at least as many keys as queries every request gets its own tokens plus a share of the
    surplus (its cached prefix), otherwise the keys are cut independently (windows shorter than
    the query run occur in the captures and leave fully masked rows)."""
    batch, total_q, n_idx = axes[0], axes[1], axes[2]
    rng = _rng(operator, axes)
    batch = min(batch, total_q, n_idx)
    q_lens = _positive(total_q, batch, rng)
    if n_idx >= total_q:
        extra = _nonnegative(n_idx - total_q, batch, rng)
        kv_lens = [q + e for q, e in zip(q_lens, extra)]
    else:
        kv_lens = _positive(n_idx, batch, rng)
    return batch, q_lens, kv_lens


def case(operator, axes, dims, page_size=1, scale=None, dtype=None, device="cuda"):
    """``(inputs, expected outputs)`` of one workload of an operator."""
    from . import reference

    if "prefill" in operator:
        batch, q_lens, kv_lens = prefill_lengths(operator, axes)
        total_q, n_idx = sum(q_lens), sum(kv_lens)
        if operator.startswith("mla_paged_prefill"):
            wl = (*dims[:3], max(axes[3], n_idx), n_idx, total_q)
            inputs = reference.mla_paged_prefill_inputs(wl, q_lens, kv_lens, scale=scale, dtype=dtype, device=device)
            expected = reference.mla_paged_prefill_reference(wl, q_lens, kv_lens, dtype=dtype)
        elif operator.startswith("gqa_ragged"):
            wl = (*dims[:3], total_q, n_idx)
            inputs = reference.gqa_ragged_prefill_inputs(wl, q_lens, kv_lens, scale=scale, dtype=dtype, device=device)
            expected = reference.gqa_ragged_prefill_reference(wl, q_lens, kv_lens, dtype=dtype)
        else:
            wl = (*dims[:3], max(axes[3], n_idx), n_idx, total_q)
            inputs = reference.gqa_paged_prefill_inputs(wl, q_lens, kv_lens, scale=scale, dtype=dtype, device=device)
            expected = reference.gqa_paged_prefill_reference(wl, q_lens, kv_lens, dtype=dtype)
        return inputs, expected(*inputs)
    batch, pool, n_idx, kv_lens = decode_lengths(operator, axes, page_size)
    if operator.startswith("mla_paged_decode"):
        wl = (batch, *dims[:3], pool, n_idx)
        inputs = reference.mla_paged_decode_inputs(wl, kv_lens, scale=scale, dtype=dtype, device=device)
        expected = reference.mla_paged_decode_reference(wl, kv_lens, dtype=dtype)
        return inputs, expected(*inputs)
    wl = (batch, *dims[:3], pool, n_idx)
    inputs = reference.gqa_paged_decode_inputs(wl, kv_lens, page_size=page_size, scale=scale, dtype=dtype, device=device)
    expected = reference.gqa_paged_decode_reference(wl, kv_lens, page_size=page_size, dtype=dtype)
    return inputs, expected(*inputs)
