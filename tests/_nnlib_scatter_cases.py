"""Known answers of NNlib.scatter! / NNlib.scatter held by the reference's tests
(test/nn/scatter_gather.jl:254-428): destination, source and one-based index arrays, and the expected
result per operation.  `keep` cases scatter into the given destination, the others into a destination
filled with the operation's neutral element (what NNlib.scatter builds before it calls scatter!,
reference ext/ReactantNNlibExt/Implementations.jl:463-474).  For "divide" the source is doubled first,
as the reference test does."""
import numpy as np

F = np.float32
INF = np.inf
NEUTRAL = {"add": 0.0, "subtract": 0.0, "maximum": -INF, "minimum": INF, "multiply": 1.0, "divide": 1.0, "mean": 0.0}

_D1 = F([3, 4, 5, 6, 7])
_D2 = F([[3, 3, 4, 4, 5], [5, 5, 6, 6, 7]])
_I1 = np.array([4, 2, 1, 5, 3], dtype=np.int64)
_I2 = np.array([[1, 2, 3, 4], [4, 2, 1, 3], [3, 5, 5, 3]], dtype=np.int64)
_R15 = np.arange(1, 6, dtype=F)
_S34 = np.ones((3, 1), F) * np.arange(1, 5, dtype=F)[None, :]


def _rows(*rows):
    return F(rows)


def _frac(*den):
    return F([1.0 / d for d in den])


# (name, dst, src_keep, src_fresh, idx, {op: (res_keep, res_fresh)})
SETS = [
    ("1d src, 1d index => 1d output", _D1, np.ones(5, F), _R15, _I1, {
        "add": (F([4, 5, 6, 7, 8]), F([3, 2, 5, 1, 4])),
        "subtract": (F([2, 3, 4, 5, 6]), F([-3, -2, -5, -1, -4])),
        "maximum": (F([3, 4, 5, 6, 7]), F([3, 2, 5, 1, 4])),
        "minimum": (F([1, 1, 1, 1, 1]), F([3, 2, 5, 1, 4])),
        "multiply": (F([3, 4, 5, 6, 7]), F([3, 2, 5, 1, 4])),
        "divide": (F([1.5, 2.0, 2.5, 3.0, 3.5]), _frac(6, 4, 10, 2, 8)),
        "mean": (F([4, 5, 6, 7, 8]), F([3, 2, 5, 1, 4])),
    }),
    ("2d src, 1d index => 2d output", _D2, np.ones((2, 5), F), np.ones((2, 1), F) * _R15[None, :], _I1, {
        "add": (_rows([4, 4, 5, 5, 6], [6, 6, 7, 7, 8]), _rows([3, 2, 5, 1, 4], [3, 2, 5, 1, 4])),
        "subtract": (_rows([2, 2, 3, 3, 4], [4, 4, 5, 5, 6]), _rows([-3, -2, -5, -1, -4], [-3, -2, -5, -1, -4])),
        "maximum": (_rows([3, 3, 4, 4, 5], [5, 5, 6, 6, 7]), _rows([3, 2, 5, 1, 4], [3, 2, 5, 1, 4])),
        "minimum": (_rows([1, 1, 1, 1, 1], [1, 1, 1, 1, 1]), _rows([3, 2, 5, 1, 4], [3, 2, 5, 1, 4])),
        "multiply": (_rows([3, 3, 4, 4, 5], [5, 5, 6, 6, 7]), _rows([3, 2, 5, 1, 4], [3, 2, 5, 1, 4])),
        "divide": (_rows([1.5, 1.5, 2.0, 2.0, 2.5], [2.5, 2.5, 3.0, 3.0, 3.5]), np.stack([_frac(6, 4, 10, 2, 8)] * 2)),
        "mean": (_rows([4, 4, 5, 5, 6], [6, 6, 7, 7, 8]), _rows([3, 2, 5, 1, 4], [3, 2, 5, 1, 4])),
    }),
    ("2d src, 2d index => 1d output", _D1, np.ones((3, 4), F), _S34, _I2, {
        "add": (F([5, 6, 9, 8, 9]), F([4, 4, 12, 5, 5])),
        "subtract": (F([1, 2, 1, 4, 5]), F([-4, -4, -12, -5, -5])),
        "maximum": (F([3, 4, 5, 6, 7]), F([3, 2, 4, 4, 3])),
        "minimum": (F([1, 1, 1, 1, 1]), F([1, 2, 1, 1, 2])),
        "multiply": (F([3, 4, 5, 6, 7]), F([3, 4, 48, 4, 6])),
        "divide": (F([0.75, 1.0, 0.3125, 1.5, 1.75]), _frac(12, 16, 768, 16, 24)),
        "mean": (F([4, 5, 6, 7, 8]), F([2, 2, 3, 2.5, 2.5])),
    }),
    ("3d src, 2d index => 2d output", _D2, np.ones((2, 3, 4), F), F([1, 2])[:, None, None] * _S34[None], _I2, {
        "add": (_rows([5, 5, 8, 6, 7], [7, 7, 10, 8, 9]), _rows([4, 4, 12, 5, 5], [8, 8, 24, 10, 10])),
        "subtract": (_rows([1, 1, 0, 2, 3], [3, 3, 2, 4, 5]), _rows([-4, -4, -12, -5, -5], [-8, -8, -24, -10, -10])),
        "maximum": (_rows([3, 3, 4, 4, 5], [5, 5, 6, 6, 7]), _rows([3, 2, 4, 4, 3], [6, 4, 8, 8, 6])),
        "minimum": (_rows([1, 1, 1, 1, 1], [1, 1, 1, 1, 1]), _rows([1, 2, 1, 1, 2], [2, 4, 2, 2, 4])),
        "multiply": (_rows([3, 3, 4, 4, 5], [5, 5, 6, 6, 7]), _rows([3, 4, 48, 4, 6], [12, 16, 768, 16, 24])),
        "divide": (_rows([0.75, 0.75, 0.25, 1.0, 1.25], [1.25, 1.25, 0.375, 1.5, 1.75]),
                   np.stack([_frac(12, 16, 768, 16, 24), _frac(48, 64, 12288, 64, 96)])),
        "mean": (_rows([4, 4, 5, 5, 6], [6, 6, 7, 7, 8]), _rows([2, 2, 3, 2.5, 2.5], [4, 4, 6, 5, 5])),
    }),
]


def cases():
    """(id, op, dst, src, idx, expected)"""
    out = []
    for name, dst, src_keep, src_fresh, idx, res in SETS:
        for op, (r_keep, r_fresh) in res.items():
            scale = F(2.0) if op == "divide" else F(1.0)
            out.append(("%s/%s/into-dst" % (name, op), op, dst.copy(), src_keep * scale, idx, r_keep))
            fresh = np.full(dst.shape, NEUTRAL[op], F)
            out.append(("%s/%s/fresh" % (name, op), op, fresh, src_fresh * scale, idx, r_fresh))
    return out
