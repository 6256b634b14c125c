"""Torch evaluation of a stage graph: the reference every candidate is validated against.

Counterpart of the reference's graph executor (``python/cleave/runtime/reference.py:63-479``):
seeded inputs per placeholder (``make_inputs``), evaluation with operands kept in their
storage dtype and arithmetic in fp32 (``execute``), and the helpers that line tensors up with
a compiled kernel's parameters.  Tensors live on ``device`` ("cuda" by default, as there);
nothing here is on a kernel's launch path.

Stage roles: ``main`` evaluates the operator; ``partial`` evaluates what the split kernel
writes (per-split f32 partials); ``combine`` evaluates the reduction of given partials.
Attention partials carry (m, l, O) with m the split's row maximum of the scaled scores in
the log2 domain, l the sum of 2^(s - m) and O the matching weighted values.
"""

from __future__ import annotations

import hashlib
import math

LOG2E = 1.4426950408889634


def placeholder_order(graph) -> list:
    return list(graph.placeholders)


def output_order(graph) -> list:
    return list(graph.outputs)


def graph_out_indices(graph) -> list:
    """Trailing parameter indices of the outputs: ``range(-n_out, 0)``."""
    return list(range(-len(graph.outputs), 0))


def torch_dtype(name: str):
    import torch

    return getattr(torch, str(name).replace("torch.", ""))


def fingerprint_seed(graph) -> int:
    """A seed that depends only on placeholder names, shapes and dtypes."""
    h = hashlib.sha256()
    for ph in graph.placeholders:
        h.update(f"{ph.name}:{tuple(ph.shape)}:{ph.dtype};".encode())
    h.update(f"{getattr(graph, 'role', 'main')}:{getattr(graph, 'split_factor', None)}".encode())
    return int.from_bytes(h.digest()[:4], "little")


def _positive_placeholders(graph) -> set:
    """Inputs that must be sampled strictly positive: running sums of a combine stage."""
    if getattr(graph, "role", "main") != "combine":
        return set()
    return {ph.name for ph in graph.placeholders if ph.name.endswith(("_PL", "_PSS"))}


def make_inputs(graph, dtype=None, device: str = "cuda", seed: int | None = None) -> list:
    import torch

    gen = torch.Generator(device="cpu").manual_seed(fingerprint_seed(graph) if seed is None else int(seed))
    positive = _positive_placeholders(graph)
    made = []
    for ph in graph.placeholders:
        if ph.dtype == "int32":
            x = torch.randint(0, 16, tuple(ph.shape), generator=gen, dtype=torch.int32)
        elif ph.name in positive:
            x = torch.rand(tuple(ph.shape), generator=gen) + 0.5
        else:
            x = torch.randn(tuple(ph.shape), generator=gen)
            low = getattr(graph, "lowered", None)
            if low is not None and low.family in ("matmul", "rmsnorm_matmul", "swiglu", "matmul_rowsum", "lora") and getattr(graph, "role", "main") != "combine":
                role = next((r for r, n in low.operands.items() if n is ph), None)
                if role in ("B", "C", "LA"):
                    x = x / math.sqrt(low.problem["K"])  # keep products O(1) so tolerances mean something
        made.append(x.to(dtype=torch_dtype(ph.dtype), device=device))
    return made


# ----------------------------------------------------------------------------- evaluators
def _mm_operands(low, feed):
    p = low.problem
    a = feed[low.operands["A"].name].float()
    b = feed[low.operands["B"].name].float()
    a = a.reshape(p["batch_A"], *a.shape[-2:])
    b = b.reshape(p["batch_B"], *b.shape[-2:])
    if p["trans_A"]:
        a = a.mT
    if p["trans_B"]:
        b = b.mT
    batch = max(p["batch_A"], p["batch_B"])
    if a.shape[0] != batch:
        a = a.repeat_interleave(batch // a.shape[0], dim=0)
    if b.shape[0] != batch:
        b = b.repeat_interleave(batch // b.shape[0], dim=0)
    return a, b  # (batch, M, K), (batch, K, N)


def _eval_matmul(low, feed, role, factor, out_dtype):
    import torch

    p = low.problem
    a, b = _mm_operands(low, feed)
    norm = low.family == "rmsnorm_matmul"
    raw = a
    if norm and p.get("gamma"):
        gamma = feed[low.operands["GAMMA"].name].float().reshape(1, 1, -1)
        a = (a * gamma).to(out_dtype).float()  # the kernel rounds x*gamma to the storage dtype
    if role == "partial":
        kc = p["K"] // factor
        acc = torch.stack([a[:, :, s * kc:(s + 1) * kc] @ b[:, s * kc:(s + 1) * kc, :] for s in range(factor)])
        outs = [acc.reshape(factor, -1, p["N"])]
        if norm:
            outs.append(torch.stack([(raw[:, :, s * kc:(s + 1) * kc] ** 2).sum(-1) for s in range(factor)])
                        .reshape(factor, -1))
        return outs
    y = a @ b
    if norm:
        y = y * torch.rsqrt((raw ** 2).mean(-1, keepdim=True) + p["eps"])
    return [y.to(out_dtype)]


def _eval_swiglu(low, feed, out_dtype):
    """``(a @ b) * silu(a @ c)``: products, gate and product of the two in fp32
    (``tests/_graphs.py:403-436`` of the reference: every node of the graph is fp32 up to the output)."""
    import torch

    a, b = _mm_operands(low, feed)
    c = feed[low.operands["C"].name].float()
    c = (c.mT if low.problem["trans_B"] else c).unsqueeze(0)
    return [((a @ b) * torch.nn.functional.silu(a @ c)).to(out_dtype)]


def _eval_matmul_combine(low, feed, out_dtype, out_shape):
    import torch

    p = low.problem
    acc = feed["PlaceHolder_PACC"].float().sum(0)
    if low.family == "rmsnorm_matmul":
        ss = feed["PlaceHolder_PSS"].float().sum(0)
        acc = acc * torch.rsqrt(ss / p["K"] + p["eps"]).unsqueeze(-1)
    return [acc.to(out_dtype).reshape(out_shape)]


def _attn_scores(low, feed):
    """``(scores (units, rows, skv) scaled to the log2 domain, values (units, skv, vdim))``."""
    import torch

    p = low.problem
    if low.family == "mla":
        q, qpe = feed[low.operands["Q"].name].float(), feed[low.operands["QPE"].name].float()
        kv, kpe = feed[low.operands["KV"].name].float(), feed[low.operands["KPE"].name].float()
        s = q @ kv.mT + qpe @ kpe.mT
        return s * (p["scale"] * LOG2E), kv
    q = feed[low.operands["Q"].name].float()
    k = feed[low.operands["K"].name].float()
    v = feed[low.operands["V"].name].float()
    norm = p.get("norm_eps") or {}
    if "q" in norm:
        q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + norm["q"])
    if "k" in norm:
        k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + norm["k"])
    units, rows = p["units"], p["group"] * p["sq"]
    q = q.reshape(units, rows, p["head_dim"])
    k = k.reshape(units, p["head_dim"], p["skv"]).mT if p.get("k_major") else k.reshape(units, p["skv"], p["head_dim"])
    v = v.reshape(units, p["skv"], p["vdim"])
    return (q @ k.mT) * (p["scale"] * LOG2E), v


def _eval_attention(low, feed, role, factor, out_dtype, out_shapes):
    import torch

    s, v = _attn_scores(low, feed)
    linear = bool(low.problem.get("linear"))    # (q k^T) v: the scores themselves, in the storage type, weigh the values
    if linear and role != "partial":
        return [((s / LOG2E).to(out_dtype).float() @ v).to(out_dtype).reshape(out_shapes[0])]
    if role == "partial":
        n = s.shape[-1]
        steps = -(-n // 32)
        per = -(-steps // factor)
        pm, pl, po = [], [], []
        for i in range(factor):
            lo, hi = min(n, i * per * 32), min(n, (i + 1) * per * 32)
            if hi <= lo:
                pm.append(torch.full(s.shape[:-1], 0.0 if linear else -1.0e30, device=s.device))
                pl.append(torch.full(s.shape[:-1], 1.0 / factor if linear else 0.0, device=s.device))
                po.append(torch.zeros(*s.shape[:-1], v.shape[-1], device=s.device))
                continue
            blk = s[..., lo:hi]
            if linear:       # plain partial sums: m = 0 and l = 1 / factor make the softmax combine add them up
                pm.append(torch.zeros(s.shape[:-1], device=s.device))
                pl.append(torch.full(s.shape[:-1], 1.0 / factor, device=s.device))
                po.append((blk / LOG2E).to(out_dtype).float() @ v[..., lo:hi, :])
                continue
            m = blk.amax(-1)
            w = torch.exp2(blk - m.unsqueeze(-1)).to(out_dtype).float()
            pm.append(m)
            pl.append(w.sum(-1))
            po.append(w @ v[..., lo:hi, :])
        return [torch.stack(t).reshape(shape) for t, shape in zip((pm, pl, po), out_shapes)]
    w = torch.softmax(s / LOG2E, dim=-1)
    return [(w @ v).to(out_dtype).reshape(out_shapes[0])]


def _eval_attention_combine(feed, out_dtype, out_shape):
    import torch

    pm, pl, po = (feed[f"PlaceHolder_{n}"].float() for n in ("PM", "PL", "PO"))
    m = pm.amax(0)
    f = torch.exp2(pm - m)
    l = (pl * f).sum(0)
    o = (po * f.unsqueeze(-1)).sum(0) / l.clamp_min(1e-30).unsqueeze(-1)
    return [o.to(out_dtype).reshape(out_shape)]


def execute(graph, inputs, device=None) -> list:
    """Evaluate a stage graph on ``inputs`` (in placeholder order); one tensor per output."""
    low = graph.lowered
    role, factor = getattr(graph, "role", "main"), getattr(graph, "split_factor", None)
    feed = {ph.name: x for ph, x in zip(graph.placeholders, inputs)}
    outs = graph.outputs
    out_dtype = torch_dtype(outs[0].dtype)
    shapes = [tuple(o.shape) for o in outs]
    if low.family in ("matmul", "rmsnorm_matmul"):
        if role == "combine":
            return _eval_matmul_combine(low, feed, out_dtype, shapes[0])
        res = _eval_matmul(low, feed, role, factor, torch_dtype(graph.dtype))
        return [r.reshape(s) for r, s in zip(res, shapes)]
    if low.family == "rowsum":
        x = feed[low.operands["X"].name].float()
        total = x.sum(-1, keepdim=True)
        return [((x / total) if low.problem["div"] else total).to(out_dtype).reshape(shapes[0])]
    if low.family == "swiglu":
        return [r.reshape(s) for r, s in zip(_eval_swiglu(low, feed, out_dtype), shapes)]
    if low.family == "lora":
        # x @ w + (x @ a) @ b, the down product rounded to the storage type before the up product;
        # split over K: partial sums of x @ w and of x @ a, and a combine that applies the rank update
        import torch

        if role == "combine":
            down = feed["PlaceHolder_PD"].float().sum(0).to(torch_dtype(graph.dtype)).float()
            lb = feed[low.operands["LB"].name].float()
            return [(feed["PlaceHolder_PACC"].float().sum(0) + down @ lb).to(out_dtype).reshape(shapes[0])]
        a, b = _mm_operands(low, feed)
        la = feed[low.operands["LA"].name].float()
        if role == "partial":
            kc = low.problem["K"] // factor
            pacc = torch.stack([a[0, :, s * kc:(s + 1) * kc] @ b[0, s * kc:(s + 1) * kc] for s in range(factor)])
            pd = torch.stack([a[0, :, s * kc:(s + 1) * kc] @ la[s * kc:(s + 1) * kc] for s in range(factor)])
            return [pacc.reshape(shapes[0]), pd.reshape(shapes[1])]
        lb = feed[low.operands["LB"].name].float()
        down = (a @ la).to(torch_dtype(graph.dtype)).float()
        return [(a @ b + down @ lb).to(out_dtype).reshape(shapes[0])]
    if low.family == "matmul_rowsum":
        a, b = _mm_operands(low, feed)
        return [(a @ b).sum(-1).to(out_dtype).reshape(shapes[0])]
    if low.family in ("attention", "mla"):
        if role == "combine":
            return _eval_attention_combine(feed, out_dtype, shapes[0])
        return _eval_attention(low, feed, role, factor, torch_dtype(graph.dtype), shapes)
    raise NotImplementedError(f"no evaluator for family {low.family!r}")


def build_inputs_and_reference(graph, dtype=None, device: str = "cuda"):
    """``(inputs_by_name, [reference outputs], out_idx)``."""
    inputs = make_inputs(graph, dtype, device)
    by_name = {ph.name: x for ph, x in zip(graph.placeholders, inputs)}
    return by_name, execute(graph, inputs), graph_out_indices(graph)


def reconcile_output_layout(reference, shape):
    """``reference`` viewed as ``shape`` when they hold the same elements in the same order."""
    shape = tuple(shape)
    if tuple(reference.shape) == shape or reference.numel() != math.prod(shape):
        return reference
    return reference.reshape(shape)


def order_inputs_for_kernel(inputs_by_name: dict, kernel) -> list:
    """The kernel's caller-supplied non-output arguments, in its parameter order."""
    ordered = []
    for p in kernel.params:
        if p.role in ("input", "scalar"):
            if p.name not in inputs_by_name:
                raise KeyError(f"kernel parameter {p.name!r} has no bound input (have {sorted(inputs_by_name)})")
            ordered.append(inputs_by_name[p.name])
    return ordered
