"""numpy restatement of the reference's remaining nodes around the product path:
arithmetic (ginn/node/common.h), selection (select.h, compare.h), picking
(pick.h), reductions (reduce.h), layout (layout.h: Stack, Chip, broadcasts,
Permute) and the in-place nodes (inplace.h), forward and backward.

TEST INFRASTRUCTURE ONLY: see the package docstring.

Conventions as in oracle/nodes.py: Fortran-ordered arrays whose ``shape`` is
the reference's Shape; everything in the dtype of the inputs.  Every function
returns the value, and every ``*_backward`` returns the list of input
gradients for an output gradient ``dy`` (None for inputs without one).

Pinned by tests/test_oracle_nodes_more.py against the reference's known
answers (test/nodes.cu.cpp:66-125, 286-325, 382-421, 443-657, 755-911,
942-1021, re-typed in tests/golden/reference_nodes_more.json) and by central
finite differences with the protocol of test/testutil.h:93-171.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np

from . import nodes as N


def _f(x):
    x = np.asarray(x)
    return x if x.ndim == 0 else np.asfortranarray(x)  # asfortranarray would make a rank-0 value rank 1


# ---------------------------------------------------------------------------
# Arithmetic  (ginn/node/common.h)
# ---------------------------------------------------------------------------

def add_scalar(x, s):                       # :26-52
    return _f(x + s)


def subtract_scalar(s, x):                  # :55-95: s - x; dx -= dy
    return _f(s - x)


def prod_scalar(x, s):                      # :187-231
    return _f(x * s)


def subtract(a, b):                         # :162-187
    return _f(a - b)


def subtract_backward(dy):
    return [_f(dy), _f(-dy)]


def cwise_max(ins: Sequence[np.ndarray]):   # :319-330: running maximum
    out = np.array(ins[0], copy=True)
    for x in ins[1:]:
        out = np.maximum(out, x)
    return _f(out)


def cwise_max_backward(ins, value, dy):     # :332-341: every input equal to the maximum receives dy
    return [_f(dy * (x == value)) for x in ins]


def dropout_apply(x, mask, p):              # :374-394 with the mask given
    if p == 1.0:
        return _f(np.zeros_like(x))
    return _f(x * mask * (1.0 / (1.0 - p)))


# ---------------------------------------------------------------------------
# Selection and comparison  (ginn/node/select.h, compare.h)
# ---------------------------------------------------------------------------

def select(cond, a, b):                     # select.h:31-58; a / b may be scalars (shape ())
    cond = np.asarray(cond, dtype=bool)
    return _f(np.where(cond, a, b))


def select_backward(cond, a, b, dy):        # :60-80: a scalar branch receives the sum
    cond = np.asarray(cond, dtype=bool)
    da = dy * cond
    db = dy * (~cond)
    if np.ndim(a) == 0:
        da = np.asarray(da.sum())
    if np.ndim(b) == 0:
        db = np.asarray(db.sum())
    return [_f(da), _f(db)]


def _mask_view(x, mask):
    ms, xs = mask.shape, x.shape
    assert len(ms) == len(xs)
    i = 0
    while i < len(xs) and ms[i] == xs[i]:
        i += 1
    assert all(d == 1 for d in ms[i:]), "Unexpected mask shape!"
    m = mask.reshape((mask.size, 1), order="F")
    return m, x.reshape((mask.size, x.size // mask.size), order="F")


def mask(x, msk, val):                      # select.h:121-146
    m, xm = _mask_view(x, msk)
    return _f(np.where(m != 0, xm, val).reshape(x.shape, order="F"))


def mask_backward(x, msk, dy):              # :148-160
    m, dm = _mask_view(dy, msk)
    return [_f(np.where(m != 0, dm, 0.0).reshape(x.shape, order="F"))]


def less_than(a, b):                        # compare.h:33-36
    return _f(a < b)


# ---------------------------------------------------------------------------
# Picking  (ginn/node/pick.h)
# ---------------------------------------------------------------------------

def pick(x, index):                         # :54-82: one entry per column -> [1 x cols]
    m = N.mat(x)
    index = np.asarray(index, dtype=np.int64).reshape(-1)
    assert index.size == m.shape[1], "Index size does not match input columns!"
    return _f(m[index, np.arange(m.shape[1])].reshape(1, -1))


def pick_backward(x, index, dy, sign=1.0):  # :84-132
    m = N.mat(x)
    index = np.asarray(index, dtype=np.int64).reshape(-1)
    d = np.zeros(m.shape, dtype=m.dtype, order="F")
    d[index, np.arange(m.shape[1])] += sign * np.asarray(dy).reshape(-1)
    return [_f(d.reshape(np.shape(x), order="F"))]


def pick_softmax(x, index):                 # :171-201
    sm = N.softmax_cols(N.mat(x))
    return pick(sm, index), sm


def pick_softmax_backward(x, index, sm, dy):
    dsm = pick_backward(sm, index, dy)[0]
    return [_f(N.nonlin_backward(N.SOFTMAX, dsm, N.mat(x), sm).reshape(np.shape(x), order="F"))]


def pick_neg_log_softmax(x, index):         # :203-248
    p, sm = pick_softmax(x, index)
    return _f(-np.log(p)), sm


def pick_neg_log_softmax_backward(x, index, sm, dy):
    index = np.asarray(index, dtype=np.int64).reshape(-1)
    g = np.asarray(dy).reshape(1, -1)
    d = sm * g
    d[index, np.arange(sm.shape[1])] -= g.reshape(-1)
    return [_f(d.reshape(np.shape(x), order="F"))]


def pick_neg_log_sigmoid(x, index):         # :250-272
    s = N.nonlin_forward(N.SIGMOID, x)
    idx = np.asarray(index).reshape(np.shape(x), order="F").astype(bool)
    return _f(-np.where(idx, np.log(s), np.log(1.0 - s))), s


def pick_neg_log_sigmoid_backward(index, s, dy):   # :274-280
    idx = np.asarray(index).reshape(s.shape, order="F").astype(s.dtype)
    return [_f((s - idx) * dy)]


# ---------------------------------------------------------------------------
# Reductions  (ginn/node/reduce.h)
# ---------------------------------------------------------------------------

def axis_sum(x, axes: Sequence[int]):       # :53-136
    axes = list(axes)
    assert axes == sorted(axes), "Axes need to be specified in sorted order in AxisSum!"
    assert len(set(axes)) == len(axes), "Axes need to be uniquely specified in AxisSum!"
    return _f(np.asarray(x).sum(axis=tuple(axes)))


def axis_sum_backward(x, axes, dy):
    g = np.asarray(dy)
    for a in axes:
        g = np.expand_dims(g, a)
    return [_f(np.broadcast_to(g, np.shape(x)).copy())]


def mean(x):                                # :138-159
    return _f(np.asarray(np.mean(x)))


def mean_backward(x, dy):
    return [_f(np.full(np.shape(x), float(dy) / np.size(x)))]


def variance(x):                            # :164-177: biased
    m = np.mean(x)
    return _f(np.asarray(np.mean((x - m) ** 2))), m


def variance_backward(x, m, dy):            # :178-187
    return [_f((x - m) * float(dy) * (2.0 / np.size(x)))]


def argmax_axis(x, dim):                    # ginn/util/amax.h:54-66: first maximum wins
    return _f(np.argmax(x, axis=dim))


# ---------------------------------------------------------------------------
# Layout  (ginn/node/layout.h)
# ---------------------------------------------------------------------------

def stack(grid: Sequence[Sequence[np.ndarray]]):   # :350-397: shape = inner shape + {m, n}
    m, n = len(grid), len(grid[0])
    s = np.shape(grid[0][0])
    out = np.zeros(s + (m, n), dtype=np.asarray(grid[0][0]).dtype, order="F")
    for i in range(m):
        assert len(grid[i]) == n, "Inner container sizes mismatch!"
        for j in range(n):
            assert np.shape(grid[i][j]) == s, "Input shapes mismatch!"
            out[..., i, j] = grid[i][j]
    return out


def stack_backward(grid_ids: Sequence[Sequence[int]], n_inputs: int, dy):
    """grid_ids[i][j] = which input sits at (i, j); an input that appears
    several times receives the sum (:399-444)."""
    grads: List[Optional[np.ndarray]] = [None] * n_inputs
    for i, row in enumerate(grid_ids):
        for j, k in enumerate(row):
            g = dy[..., i, j]
            grads[k] = g.copy() if grads[k] is None else grads[k] + g
    return [_f(g) for g in grads]


def chip(x, offset, dim):                   # :631-697
    return _f(np.take(x, offset, axis=dim))


def chip_backward(x, offset, dim, dy):
    d = np.zeros(np.shape(x), dtype=np.asarray(dy).dtype, order="F")
    idx = [slice(None)] * d.ndim
    idx[dim] = offset
    d[tuple(idx)] += dy
    return [d]


def row_broadcast(x, rows):                 # :831-862
    assert x.ndim == 2 and x.shape[0] == 1
    return _f(np.repeat(x, rows, axis=0))


def row_broadcast_backward(dy):
    return [_f(dy.sum(axis=0, keepdims=True))]


def transpose(x, i, j):                     # :822-828
    perm = list(range(np.ndim(x)))
    perm[i], perm[j] = perm[j], perm[i]
    return N.permute(x, perm), perm


# ---------------------------------------------------------------------------
# In-place nodes  (ginn/node/inplace.h): same values as their plain twins; the
# backward of InPlaceCwiseProd divides the product by b (:88-93).
# ---------------------------------------------------------------------------

def inplace_cwise_prod_backward(value, b, dy):
    return [_f(dy * b), _f(dy * (value / b))]


def layernorm_backward_assign(dy, y, std):  # :222-238: what the accumulating form adds, assigned
    return N.layernorm_backward(dy, y, std)
