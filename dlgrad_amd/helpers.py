"""Op enums and the shape/stride rules kernels are launched with.

The enum members and the function names are the ones the reference's Buffer and
runtimes use (dlgrad/helpers.py:18-58, :114-212, :276-334) so a runtime written
against one works against the other.  The bodies are this package's own.
Two extra enum members exist only here: `BufferOps.CREATE` is given a meaning
(host array -> device buffer) and `CustomOps.TO_HOST` is new (device buffer ->
host array); the reference needs neither because its pointers are host memory.
"""
from __future__ import annotations

import itertools
import os
from collections.abc import Iterable
from enum import Enum, auto
from functools import lru_cache
from math import prod


class _Op(Enum):
    """Members are singletons compared by identity, so the identity hash serves; Enum's own
    __hash__ is a Python-level function and these objects key a dict on every op."""
    __hash__ = object.__hash__


class UnaryOps(_Op):
    SUM = auto()
    MAX = auto()
    NEG = auto()
    EXP = auto()
    LOG = auto()
    POW = auto()
    SQRT = auto()
    RSQRT = auto()
    TRANSPOSE = auto()
    RELU = auto()
    ARGMAX = auto()
    WHERE = auto()
    MEAN = auto()
    CLAMP = auto()
    MASKED_FILL = auto()
    PERMUTE = auto()


class BufferOps(_Op):
    CREATE = auto()
    UNIFORM = auto()
    ARANGE = auto()
    FULL = auto()


class BinaryOps(_Op):
    ADD = auto()
    SUB = auto()
    MUL = auto()
    DIV = auto()
    MATMUL = auto()
    GT = auto()
    GTE = auto()
    EQT = auto()
    CMP = auto()


class CustomOps(_Op):
    INDEX = auto()
    CE_FORWARD = auto()
    CE_BACKWARD = auto()
    PRINT = auto()
    EMBEDDING = auto()
    TO_HOST = auto()
    # fused row kernels (no counterpart in the reference, which composes them
    # from max/sub/exp/sum/div: tensor.py:634-669, ops.py:337-370)
    SOFTMAX = auto()
    SOFTMAX_BWD = auto()            # y * (g - sum(g * y)) over the last axis, one kernel
    MASKED_SOFTMAX = auto()         # softmax(masked_fill(x * scale, mask, -inf)) over the last axis, one kernel
    MASKED_SOFTMAX_BWD = auto()     # its backward, one kernel
    CAUSAL_ATTENTION = auto()       # softmax(mask(q k^T * scale)) v on (B, T, heads*d) projections, heads read in place
    CAUSAL_ATTENTION_BWD = auto()
    CAUSAL_ATTENTION_QKV = auto()   # the same for q, k, v interleaved as one (B, T, 3C) projection
    CAUSAL_ATTENTION_QKV_BWD = auto()
    CACHED_ATTENTION = auto()       # one new position attending to the rows of a (block, B, heads*d) key/value cache in place
    LOG_SOFTMAX = auto()
    LOG_SOFTMAX_GATHER = auto()     # log-softmax rows + the ce_forward gather, one kernel
    CE_GRAD = auto()                # ((exp(lsm) - onehot) * upstream) / N, one kernel
    CE_STATS = auto()               # per row of the logits: max, log(sum(exp(x - max))) and the target's log-prob, one read-only kernel
    CE_GRAD_LOGITS = auto()         # ((exp((x - max) - logsum) - onehot) * upstream) / N from the logits and the two row statistics
    ADAM_STEP = auto()              # the 14 element-wise kernels of one Adam update, one kernel
    ADAM_STEP_INPLACE = auto()      # the same, in place, constants from device memory (graph replay)
    MATMUL_NT = auto()              # x @ y^T with y read in place (no materialised transpose)
    MATMUL_TN = auto()              # x^T @ y with x read in place
    MATMUL_PAIR = auto()            # two independent products (the dX and dW of a linear layer) as one launch
    FROM_U8 = auto()                # host uint8 array -> device fp32 buffer, cast on the device
    ROW_STORE = auto()              # dst[(int)idx, :] = src with idx read on the device (KV cache inside a graph)
    COPY_INTO = auto()              # device-to-device copy into an existing buffer (a KV-cache row)
    ADAM_MULTI_INPLACE = auto()     # one launch for a whole parameter list (addresses in a device table)
    SGD_STEP_INPLACE = auto()       # p -= (momentum-filtered) g * lr where p is (graph replay)
    SET_VALUES = auto()             # a few floats given by value written into an existing buffer by a kernel (no transfer, no wait)
    EMBEDDING_SUM = auto()          # token rows + position rows of a transformer's input: two gathers and their sum, one kernel
    DECODE_QKV_ROW = auto()         # q, k, v of one new position from the stacked projection, k and v stored into their cache rows
    DECODE_EMBED = auto()           # the input of a decoding step (token + position embedding, cache-row mask) from device-resident state
    DECODE_NEXT = auto()            # argmax of the logits, appended to the token buffer, made the next token; the index advanced
    DECODE_SAMPLE = auto()          # the same with the token drawn from softmax(logits / temperature) by a given uniform number
    RMSNORM = auto()                # (x * rsqrt(mean(x^2) + eps)) * w over the last axis, one kernel
    RMSNORM_BWD = auto()            # its backward: dx in one kernel, dw by partial rows + a column sum


def prod_(x: Iterable) -> int:
    return prod(x) if x else 1


@lru_cache(maxsize=4096)
def _stride_of(shape: tuple) -> tuple:
    out, acc = [], 1
    for d in reversed(shape):
        out.append(acc)
        acc *= d
    return tuple(reversed(out))


def calculate_stride(shape: tuple | list) -> tuple:
    """Row-major element strides; () for a 0-d shape (helpers.py:176-187)."""
    return _stride_of(tuple(shape))


@lru_cache(maxsize=4096)
def check_broadcast(x_shape: tuple, y_shape: tuple) -> bool:
    """True, or AssertionError when a trailing-aligned pair of dims is neither
    equal nor 1 (helpers.py:64-82)."""
    for a, b in itertools.zip_longest(reversed(x_shape), reversed(y_shape), fillvalue=1):
        if a != b and a != 1 and b != 1:
            raise AssertionError(
                f"Cannot broadcast {y_shape} to {x_shape}, the dimensions {a} and {b} dont match")
    return True


@lru_cache(maxsize=4096)
def broadcast_shapes_2(s1: tuple, s2: tuple) -> tuple:
    """numpy-style broadcast of two shapes (helpers.py:311-334)."""
    n = max(len(s1), len(s2))
    a = (1,) * (n - len(s1)) + tuple(s1)
    b = (1,) * (n - len(s2)) + tuple(s2)
    out = []
    for d1, d2 in zip(a, b):
        if d1 != d2 and d1 != 1 and d2 != 1:
            raise ValueError(f"Operands could not be broadcast together with shapes {s1} {s2}")
        out.append(d2 if d1 == 1 else d1)
    return tuple(out)


get_broadcast_shape = broadcast_shapes_2   # helpers.py:135-155 computes the same thing


def get_broadcast_strides_2(out_shape: tuple, in_shape: tuple, in_stride: tuple) -> tuple:
    """Strides of `in` viewed at `out_shape`: 0 wherever a size-1 (or missing
    leading) dim is stretched (helpers.py:276-309)."""
    pad = len(out_shape) - len(in_shape)
    shape = (1,) * pad + tuple(in_shape)
    stride = (0,) * pad + tuple(in_stride)
    res = []
    for o, i, s in zip(out_shape, shape, stride):
        if i == o:
            res.append(s)
        elif i == 1:
            res.append(0)
        else:
            raise ValueError(f"Shape mismatch: cannot broadcast {in_shape} to {out_shape}")
    return tuple(res)


@lru_cache(maxsize=4096)
def broadcast_shapes(s1: tuple, s2: tuple) -> tuple[tuple, tuple, tuple]:
    """Matmul operand alignment: left-pad both to equal rank, broadcast the batch
    dims, check the inner dims; returns (padded1, padded2, out) (helpers.py:114-133)."""
    n = max(len(s1), len(s2))
    p1 = (1,) * (n - len(s1)) + tuple(s1)
    p2 = (1,) * (n - len(s2)) + tuple(s2)
    batch = []
    for d1, d2 in zip(p1[:-2], p2[:-2]):
        if d1 != d2 and 1 not in (d1, d2):
            raise ValueError(f"Cannot broadcast batch dims: {s1} and {s2}")
        batch.append(max(d1, d2))
    if p1[-1] != p2[-2]:
        raise ValueError(f"Matrix inner dims must match: {s1} and {s2}")
    return p1, p2, tuple(batch) + (p1[-2], p2[-1])


def cal_sum_max_out_shape(ndim: int, dim: int, inp_shape: tuple, keepdim: bool = False) -> tuple:
    """Output shape of sum/max/mean; dim == -1 means "all elements" (helpers.py:204-212)."""
    if dim == -1:
        return tuple(inp_shape) if keepdim else ()
    t = list(inp_shape)
    if keepdim:
        t[dim] = 1
    else:
        del t[dim]
    return tuple(t)


def collapse_dims(shape: tuple, *strides: tuple) -> tuple[tuple, list[tuple]]:
    """Merge adjacent dims that every operand walks contiguously.

    `shape` is the iteration space, each `strides[k]` one operand's element strides
    over it (0 = broadcast).  Dims of extent 1 vanish; dims d, d+1 merge when
    stride[d] == stride[d+1] * shape[d+1] for every operand.  Returns the reduced
    shape and strides (at least one dim).  This is what lets a 4-D broadcast such
    as (16,4,128,128) * (16,4,128,1) run as a 2-D rows-by-columns kernel.
    """
    dims = [(n, tuple(s[i] for s in strides)) for i, n in enumerate(shape) if n != 1]
    if not dims:
        return (1,), [(0,) for _ in strides]
    merged = [dims[0]]
    for n, st in dims[1:]:
        pn, pst = merged[-1]
        if all(ps == s * n for ps, s in zip(pst, st)):
            merged[-1] = (pn * n, st)
        else:
            merged.append((n, st))
    out_shape = tuple(n for n, _ in merged)
    out_strides = [tuple(st[k] for _, st in merged) for k in range(len(strides))]
    return out_shape, out_strides


CACHE_DIR = os.environ.get(
    "DLGRAD_HIP_CACHE_DIR",
    os.path.join(os.path.dirname(os.path.abspath(__file__)), "_kcache"))

# Reference quirks that live inside a kernel's contract (int-truncated `full` and
# `pow` arguments, dlgrad/runtime/cpu.py:252 and :500) are reproduced when this is
# on, which is the default because parity is judged against that behaviour.
STRICT_REFERENCE = os.environ.get("DLGRAD_STRICT_REFERENCE", "1") != "0"


def sample_from_logits(logits, u: float, temperature: float = 1.0) -> int:
    """The token np.random.choice(V, p=softmax(logits / temperature)) returns when its uniform draw is u:
    the host-side sampling of examples/gpt.py:209-221 and :258-266 (numpy on the downloaded logits) with
    the random number made explicit.  choice() inverts the cumulative sum of p, taken in float64 and
    divided by its last entry: the first index whose entry exceeds u."""
    import numpy as np
    x = np.asarray(logits, dtype=np.float32).reshape(-1) / np.float32(temperature)
    x = x - np.max(x)
    e = np.exp(x)
    p = e / e.sum()
    cdf = np.cumsum(p.astype(np.float64))
    cdf /= cdf[-1]
    return min(int(np.searchsorted(cdf, float(u), side="right")), x.size - 1)
