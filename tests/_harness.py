"""Shared helpers: run one StableHLO module on the GPU through the C ABI and in
the oracle on identical bytes."""
import numpy as np

from oracle import stablehlo_interp as I


def gpu_run(rx, client, text, args, exe=None):
    """args: list of oracle Tensors.  Returns (list of oracle Tensors from the GPU, executable)."""
    exe = exe or rx.xla_compile(client, text)
    bufs = []
    for a in args:
        raw = np.frombuffer(a.to_bytes(), dtype=rx._STORAGE[a.dt]).reshape(a.shape)
        bufs.append(rx.Buffer.from_host(client, raw, a.dt))
    outs = exe.execute_sharded(bufs)
    res = []
    for ab in outs:
        b = ab.synced_buffer()
        raw = b.to_host()
        res.append(I.Tensor.from_bytes(raw.tobytes(), b.dtype(), b.shape()))
    return res, exe


def oracle_run(text, args, hifi=True, excess=False):
    return I.run_text(text, args, hifi=hifi, excess=excess)


def rel_err(got, ref):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    den = np.maximum(np.abs(ref), 1e-30)
    return float(np.max(np.abs(got - ref) / den)) if got.size else 0.0


def max_rel_to_scale(got, ref):
    """max |got-ref| / max|ref|: error relative to the magnitude of the result."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    scale = max(float(np.max(np.abs(ref))), 1e-30) if ref.size else 1.0
    return float(np.max(np.abs(got - ref))) / scale if got.size else 0.0


def abs_args(args):
    """The operands with every element replaced by its magnitude (exact in the operand's own type)."""
    return [I.Tensor(np.abs(a.a), a.dt) for a in args]


def contraction_err(got, ref, bound):
    """max over the entries of |got - ref|_ij / bound_ij, where bound_ij = (|A| . |B|)_ij plus the magnitudes the
    epilogue adds: the componentwise error of a contraction.  One large entry cannot set the scale for the others,
    so a wrong small entry (a dropped K tail in one tile, a bad bias lane) shows."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    bound = np.asarray(bound, dtype=np.float64)
    assert got.shape == ref.shape == bound.shape, (got.shape, ref.shape, bound.shape)
    if not got.size:
        return 0.0
    assert np.all(bound >= 0)
    return float(np.max(np.abs(got - ref) / np.maximum(bound, 1e-300)))


def dot_bound(text, args):
    """(|A| . |B|) of a module that is one dot_general (any dimension numbers), by running the oracle on the magnitudes."""
    return np.asarray(I.run_text(text, abs_args(args), hifi=True)[0].a, dtype=np.float64)
