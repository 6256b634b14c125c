"""numpy restatement of ``Program.reference`` (reference
``python/cleave/frontend/program.py:296-321``) and ``grouped_matmul`` (``:352-363``).

TEST INFRASTRUCTURE: see the package docstring.  Semantics restated, not imported:
  * every input is upcast to float32 before any arithmetic (``:303``);
  * every op computes in float32: matmul with grouped batch broadcast == repeat-interleave of
    the smaller batch extent (``:352-363``), keepdim sum / max reductions (``:308-311``), silu,
    exp, sqrt, and add / sub / mul / div with either a tensor or a Python scalar on either side
    (``:312-316``);
  * each output is cast to its declared dtype once, at the end (``:317``).
The program is consumed through its public records (``kind``, ``args``, ``attr``, ``out``), so
this file does not depend on how the frontend evaluates anything.
"""

from __future__ import annotations

import numpy as np


def to_f32(x) -> np.ndarray:
    """torch tensor (any float dtype, any device) or array -> float32 numpy array."""
    if hasattr(x, "detach"):
        x = x.detach().cpu()
        if "int" in str(x.dtype):
            return x.numpy().astype(np.float32)
        return x.float().numpy()
    return np.asarray(x, dtype=np.float32)


def round_to_dtype(x: np.ndarray, dtype: str) -> np.ndarray:
    """float32 values rounded (nearest even) to ``dtype``'s grid, returned as float32."""
    x = np.asarray(x, dtype=np.float32)
    if dtype == "float32":
        return x
    if dtype == "float16":
        with np.errstate(over="ignore"):
            return x.astype(np.float16).astype(np.float32)
    if dtype == "bfloat16":
        bits = x.view(np.uint32).astype(np.uint64)
        nan = np.isnan(x)
        rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) << 16
        out = (rounded & 0xFFFFFFFF).astype(np.uint32).view(np.float32)
        return np.where(nan, x, out)
    raise ValueError(f"unsupported dtype {dtype!r}")


def grouped_matmul(a, b, trans_a=False, trans_b=False):
    if trans_a:
        a = np.swapaxes(a, -1, -2)
    if trans_b:
        b = np.swapaxes(b, -1, -2)
    for axis in range(a.ndim - 2):
        na, nb = a.shape[axis], b.shape[axis]
        if na > nb:
            b = np.repeat(b, na // nb, axis=axis)
        elif nb > na:
            a = np.repeat(a, nb // na, axis=axis)
    return np.matmul(a, b, dtype=np.float32)


def _silu(x):
    return x / (1.0 + np.exp(-x, dtype=np.float32))


def evaluate(program, inputs, round_outputs=True) -> list:
    """One float32 array per program output (rounded to the output dtype's grid unless
    ``round_outputs`` is False)."""
    feed = iter([to_f32(x) for x in inputs])
    env = {}
    records = list(program.ops)

    def val(a):
        return env[a] if isinstance(a, int) else np.float32(a)

    for r in records:
        k = r.kind
        if k == "output":
            continue
        if k == "input":
            env[r.out] = next(feed)
        elif k == "matmul":
            env[r.out] = grouped_matmul(env[r.args[0]], env[r.args[1]], r.attr("trans_A"), r.attr("trans_B"))
        elif k == "reduce_sum":
            env[r.out] = env[r.args[0]].sum(axis=r.attr("dim"), keepdims=True, dtype=np.float32)
        elif k == "reduce_max":
            env[r.out] = env[r.args[0]].max(axis=r.attr("dim"), keepdims=True)
        elif k == "exp":
            env[r.out] = np.exp(env[r.args[0]], dtype=np.float32)
        elif k == "sqrt":
            env[r.out] = np.sqrt(env[r.args[0]], dtype=np.float32)
        elif k == "silu":
            env[r.out] = _silu(env[r.args[0]])
        elif k in ("add", "sub", "mul", "div"):
            x, y = val(r.args[0]), val(r.args[1])
            env[r.out] = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide}[k](
                x, y, dtype=np.float32)
        else:
            raise NotImplementedError(f"oracle: unknown record kind {k!r}")
    outs = []
    for o in program.outputs:
        y = env[o.tensor.id]
        outs.append(round_to_dtype(y, o.tensor.dtype.name) if round_outputs else y)
    return outs
