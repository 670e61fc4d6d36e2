"""The reference's polybench stencil suite (benchmark/polybench/stencil.jl, vectorized forms as
`@trace for` loops) on the GPU against the oracle, bit for bit: time loops over small arrays run as
chain kernels (several update steps per launch, the arrays held in LDS tiles), which must give
exactly what one launch per step gives."""
import numpy as np
import pytest

from _harness import gpu_run, oracle_run
from oracle import stablehlo_interp as I
import _polybench_cases as C

pytestmark = pytest.mark.gpu
P = C.P


def _fields(shapes, dt="f32", seed=0):
    rng = np.random.default_rng(seed)
    if dt[0] == "i":
        return [I.Tensor(rng.integers(-1000, 1000, size=s).astype(I.NP_OF[dt]), dt) for s in shapes]
    return [I.tensor(rng.random(s), dt) for s in shapes]


def _kinds(exe):
    return [l["kind"] for l in exe.launches()]


SMALL = [
    ("jacobi_1d", dict(n=2048, tsteps=40), [(2048,)] * 2),
    ("jacobi_1d", dict(n=777, tsteps=70), [(777,)] * 2),          # not a multiple of the tile; more steps than one kernel takes
    ("jacobi_1d", dict(n=5, tsteps=3), [(5,)] * 2),
    ("jacobi_2d", dict(n=512, tsteps=12), [(512, 512)] * 2),
    ("jacobi_2d", dict(n=101, tsteps=9), [(101, 101)] * 2),
    ("heat_3d", dict(n=40, tsteps=5), [(40, 40, 40)] * 2),
    ("fdtd_2d", dict(nx=200, ny=150, tmax=11), [(150, 200)] * 3 + [(11,)]),
    ("fdtd_2d", dict(nx=1024, ny=2048, tmax=7), [(2048, 1024)] * 3 + [(7,)]),
]


@pytest.mark.parametrize("dt", ["f32", "f64"])
@pytest.mark.parametrize("name,kw,shapes", SMALL)
def test_polybench_stencils_match_the_oracle_bit_for_bit(rx, client, name, kw, shapes, dt):
    text = P.build(name, dt=dt, **kw)
    args = _fields(shapes, dt, seed=len(shapes) + kw.get("tsteps", 0))
    got, exe = gpu_run(rx, client, text, args)
    if name != "heat_3d" and shapes[0][0] > 8:
        assert "map_chain" in _kinds(exe)
    ref = oracle_run(text, args)
    for g_, r_ in zip(got, ref):
        assert np.array_equal(g_.a, r_.a)


@pytest.mark.parametrize("name", ["jacobi_1d", "jacobi_2d", "fdtd_2d"])
def test_polybench_reference_sizes(rx, client, name):
    """benchmark/polybench/stencil.jl:71,229,301: the sizes the reference benchmarks."""
    sz = P.POLYBENCH_SIZES[name]
    shapes = {"jacobi_1d": [(sz.get("n"),)] * 2, "jacobi_2d": [(sz.get("n"),) * 2] * 2,
              "fdtd_2d": [(sz.get("ny"), sz.get("nx"))] * 3 + [(sz.get("tmax"),)]}[name]
    text = P.build(name)
    args = _fields(shapes, "f32", seed=3)
    got, exe = gpu_run(rx, client, text, args)
    kinds = _kinds(exe)
    assert kinds.count("map_chain") >= len(kinds) - 1 and len(kinds) <= 140
    for g_, r_ in zip(got, oracle_run(text, args)):
        assert np.array_equal(g_.a, r_.a)


def test_heat_3d_reference_size(rx, client):
    """benchmark/polybench/stencil.jl:170 (128^3), a quarter of its 256 time steps: one map launch
    per half step (rank-3 steps are not chained), in place once the arrays are temporaries."""
    text = P.build("heat_3d", tsteps=64)
    args = _fields([(128, 128, 128)] * 2, "f32", seed=4)
    got, exe = gpu_run(rx, client, text, args)
    assert _kinds(exe) == ["map"] * 2 + ["map_in_place"] * 126
    for g_, r_ in zip(got, oracle_run(text, args)):
        assert np.array_equal(g_.a, r_.a)


def test_chained_and_unchained_plans_agree(rx, client, monkeypatch):
    text = P.build("fdtd_2d", nx=300, ny=170, tmax=9)
    args = _fields([(170, 300)] * 3 + [(9,)], "f32", seed=8)
    chained, exe = gpu_run(rx, client, text, args)
    assert "map_chain" in _kinds(exe)
    monkeypatch.setenv("RX_CHAIN_STEPS", "1")
    plain, exe1 = gpu_run(rx, client, text, args)
    assert "map_chain" not in _kinds(exe1) and "map_in_place" in _kinds(exe1) and len(exe1.launches()) > len(exe.launches())
    assert np.array_equal(chained[0].a, plain[0].a)
    monkeypatch.setenv("RX_IN_PLACE", "0")
    copied, exe2 = gpu_run(rx, client, text, args)
    assert set(_kinds(exe2)) == {"map"}
    assert np.array_equal(chained[0].a, copied[0].a)


@pytest.mark.parametrize("tile,steps,threads", [("7,13", "5", "64"), ("64,64", "16", "1024"), ("3,200", "2", "256"), ("16,16", "9", "128")])
def test_chain_tilings(rx, client, monkeypatch, tile, steps, threads):
    """Tile sizes that do not divide the array, chains cut at odd lengths, every workgroup size."""
    monkeypatch.setenv("RX_CHAIN_TILE", tile)
    monkeypatch.setenv("RX_CHAIN_STEPS", steps)
    monkeypatch.setenv("RX_CHAIN_THREADS", threads)
    monkeypatch.setenv("RX_CHAIN_REDUNDANCY", "50")
    text = P.build("jacobi_2d", n=75, tsteps=7)
    args = _fields([(75, 75)] * 2, "f32", seed=9)
    got, exe = gpu_run(rx, client, text, args)
    assert "map_chain" in _kinds(exe)
    for g_, r_ in zip(got, oracle_run(text, args)):
        assert np.array_equal(g_.a, r_.a)


RANDOM = [
    # shape, fields, steps, dtype, results
    ((300,), 2, 12, "f32", None),
    ((300,), 3, 30, "f64", [1]),
    ((64, 90), 3, 10, "f32", None),
    ((64, 90), 2, 17, "f32", [0]),
    ((33, 47), 4, 12, "i32", None),
    ((1500,), 1, 9, "i64", None),
    ((20, 24, 28), 2, 6, "f32", None),
]


@pytest.mark.parametrize("seed", [0, 1, 2])
@pytest.mark.parametrize("shape,nfields,nsteps,dt,results", RANDOM)
def test_random_update_step_programs(rx, client, monkeypatch, shape, nfields, nsteps, dt, results, seed):
    """Random in-place update steps over a few arrays (random boxes, reaches of up to two cells, a
    field returned or dropped): whatever the planner chains must equal the oracle's step-by-step
    evaluation."""
    monkeypatch.setenv("RX_CHAIN_MAX_RANK", "3")
    monkeypatch.setenv("RX_CHAIN_REDUNDANCY", "8")
    rng = np.random.default_rng(100 * seed + nsteps)
    text = C.random_update_program(rng, shape, nfields, nsteps, dt, results)
    args = _fields([shape] * nfields, dt, seed=seed)
    got, exe = gpu_run(rx, client, text, args)      # most of these plans hold chain kernels, some only maps
    for g_, r_ in zip(got, oracle_run(text, args)):
        assert np.array_equal(g_.a, r_.a)


def test_steps_that_read_their_own_field_at_an_offset_are_not_chained_in_place(rx, client):
    rng = np.random.default_rng(77)
    text = C.random_update_program(rng, (400,), 2, 10, "f32", None, self_offsets=True)
    args = _fields([(400,)] * 2, "f32", seed=5)
    got, exe = gpu_run(rx, client, text, args)
    for g_, r_ in zip(got, oracle_run(text, args)):
        assert np.array_equal(g_.a, r_.a)


def test_intermediate_version_that_is_returned_ends_the_chain(rx, client):
    """B after the first half step is a result of its own: it must reach memory."""
    b = P._Loop()
    t = P._tt([500], "f32")
    b.types["%arg0"] = b.types["%arg1"] = t
    A, B = "%arg0", "%arg1"
    outs = []
    for i in range(6):
        B = b.update(B, P._star(b, A, [498], [1], [[-1], [0], [1]], 0.25, "f32"), [1])
        if i == 2:
            outs.append(B)
        A = b.update(A, P._star(b, B, [498], [1], [[-1], [0], [1]], 0.25, "f32"), [1])
    outs += [A, B]
    text = (P._HDR.format(name="tap") + "  func.func @main(%%arg0: %s, %%arg1: %s) -> (%s, %s, %s) {\n" % (t, t, t, t, t) + b.text()
            + "    return %s : %s, %s, %s\n  }\n}\n" % (", ".join(outs), t, t, t))
    args = _fields([(500,)] * 2, "f32", seed=6)
    got, exe = gpu_run(rx, client, text, args)
    assert "map_chain" in _kinds(exe)
    for g_, r_ in zip(got, oracle_run(text, args)):
        assert np.array_equal(g_.a, r_.a)


IN_PLACE = [
    # array, box start, box shape, dtype
    ((1000,), (3,), (900,), "f32"),
    ((1000,), (0,), (1000,), "f32"),             # the whole array
    ((64, 130), (5, 1), (50, 127), "f32"),       # rows whose vectors straddle both edges of the box
    ((64, 130), (63, 129), (1, 1), "f64"),       # one element
    ((20, 30, 44), (1, 2, 3), (18, 20, 37), "i32"),
    ((7, 9, 11, 16), (1, 0, 2, 5), (5, 9, 8, 6), "f32"),
    ((300, 300), (100, 0), (17, 300), "i8"),     # 16 elements per vector
]


@pytest.mark.parametrize("shape,start,box,dt", IN_PLACE)
def test_range_setindex_writes_in_place(rx, client, shape, start, box, dt):
    """y = f(x), a temporary that is worth storing; s = sum(y); y[range] = z + y[range]; return y and y + s:
    the update takes over the temporary's buffer and writes only the box (the sum reads it before)."""
    t, tb = P._tt(shape, dt), P._tt(box, dt)
    lim = ", ".join("%d:%d" % (s, s + n) for s, n in zip(start, box))
    idx = "".join("    %%s%d = stablehlo.constant dense<%d> : tensor<i64>\n" % (d, s) for d, s in enumerate(start))
    text = ("module {\n  func.func @main(%%arg0: %s, %%arg1: %s) -> (%s, %s) {\n" % (t, tb, t, t)
            + "    %%y0 = stablehlo.add %%arg0, %%arg0 : %s\n" % t
            + "".join("    %%a%d = stablehlo.add %%y%d, %%arg0 : %s\n    %%y%d = stablehlo.multiply %%a%d, %%a%d : %s\n" % (k, k, t, k + 1, k, k, t) for k in range(4))
            + "    %%y = stablehlo.subtract %%y4, %%arg0 : %s\n" % t
            + "    %%sum = stablehlo.reduce(%%y init: %%z0) applies stablehlo.add across dimensions = [%s] : (%s, %s) -> %s\n"
            % (", ".join(str(d) for d in range(len(shape))), t, P._tt([], dt), P._tt([], dt))
            + "    %%old = stablehlo.slice %%y [%s] : (%s) -> %s\n" % (lim, t, tb)
            + "    %%new = stablehlo.add %%arg1, %%old : %s\n" % tb + idx
            + "    %%r = stablehlo.dynamic_update_slice %%y, %%new, %s : (%s, %s, %s) -> %s\n"
            % (", ".join("%%s%d" % d for d in range(len(shape))), t, tb, ", ".join(["tensor<i64>"] * len(shape)), t)
            + "    %%sb = stablehlo.broadcast_in_dim %%sum, dims = [] : (%s) -> %s\n" % (P._tt([], dt), t)
            + "    %%w = stablehlo.add %%r, %%sb : %s\n" % t
            + "    return %%r, %%w : %s, %s\n  }\n}\n" % (t, t))
    text = text.replace("    %y0 = ", "    %%z0 = stablehlo.constant dense<%s> : %s\n    %%y0 = " % ("0.0" if dt[0] == "f" else "0", P._tt([], dt)), 1).replace("%%", "%")
    if dt[0] == "f":
        args = _fields([shape, box], dt, seed=1)
    else:
        rng = np.random.default_rng(1)
        args = [I.Tensor(rng.integers(-20, 20, size=s).astype(I.NP_OF[dt]), dt) for s in (shape, box)]
    got, exe = gpu_run(rx, client, text, args)
    assert "map_in_place" in _kinds(exe), _kinds(exe)
    ref = oracle_run(text, args)
    assert np.array_equal(got[0].a, ref[0].a)
    if dt[0] == "f":
        np.testing.assert_allclose(got[1].a, ref[1].a, rtol=1e-4)
    else:
        assert np.array_equal(got[1].a, ref[1].a)


LINALG_MEDIUM = {
    "gemm": dict(n=512, m=1024), "gemver": dict(n=1024), "gesummv": dict(n=1024), "syr2k": dict(n=512), "syrk": dict(n=512),
    "2mm": dict(n=512), "3mm": dict(p=128, q=256, r=512, s=1024), "atax": dict(n=1024), "bicg": dict(n=512, m=1024),
    "doitgen": dict(r=32, q=64, p=128), "mvt": dict(n=1024), "correlation": dict(n=512), "covariance": dict(n=512),
}


@pytest.mark.parametrize("size", ["small", "medium"])
@pytest.mark.parametrize("name", sorted(C.LINALG_SMALL))
def test_polybench_linalg_programs(rx, client, name, size):
    """The BLAS / linear-algebra / data-mining programs of benchmark/polybench (matrix products with
    scaled and transposed operands, two products feeding one sum, matrix-vector products as reductions,
    column statistics) against the oracle with f64 accumulation; f32 tolerance 1e-5 sqrt(k) of the result's scale."""
    kw = C.LINALG_SMALL[name] if size == "small" else LINALG_MEDIUM[name]
    text, shapes = P.linalg(name, **kw)
    args = [C.to_tensor(I, a) for a in C.linalg_args(shapes, seed=len(name) + len(size))]
    got, exe = gpu_run(rx, client, text, args)
    ref = oracle_run(text, args, hifi=True)
    k = max(max(s) if s else 1 for s in shapes)
    for g_, r_ in zip(got, ref):
        assert g_.a.shape == r_.a.shape
        scale = max(1.0, float(np.max(np.abs(r_.a))))
        assert float(np.max(np.abs(g_.a.astype(np.float64) - r_.a.astype(np.float64)))) <= 1e-5 * np.sqrt(k) * scale


@pytest.mark.parametrize("shape,nfields,nsteps,dt", [((500,), 1, 20, "f32"), ((300,), 2, 25, "f64"), ((48, 70), 2, 12, "f32"), ((40, 40), 1, 9, "i32"),
                                                     ((12, 20, 24), 2, 5, "f32")])
def test_steps_that_read_the_array_they_supersede_use_two_tiles(rx, client, monkeypatch, shape, nfields, nsteps, dt):
    """u = f(u shifted): the new version cannot overwrite the old one in place; the chain kernel keeps two
    LDS tiles for such an array and writes them in turns."""
    monkeypatch.setenv("RX_CHAIN_MAX_RANK", "3")
    monkeypatch.setenv("RX_CHAIN_REDUNDANCY", "8")
    for seed in (0, 1):
        rng = np.random.default_rng(10 * seed + nsteps)
        text = C.random_update_program(rng, shape, nfields, nsteps, dt, None, self_offsets=True)
        args = _fields([shape] * nfields, dt, seed=seed)
        got, exe = gpu_run(rx, client, text, args)
        for g_, r_ in zip(got, oracle_run(text, args)):
            assert np.array_equal(g_.a, r_.a)
    assert "map_chain" in _kinds(exe)


def test_pad_form_time_loop_of_one_array(rx, client, monkeypatch):
    """u = pad(f(u interior neighbours)) repeated (a heat equation written out of place, the form of the
    3-d diffusion / advection program): chained at small sizes, same bits as one launch per step."""
    import importlib
    PR = importlib.import_module("reactant_jl_amd.programs")
    monkeypatch.setenv("RX_CHAIN_MAX_RANK", "3")
    monkeypatch.setenv("RX_CHAIN_REDUNDANCY", "20")
    monkeypatch.setenv("RX_CHAIN_TILE", "4,8,16")
    nx, ny, nz = 30, 17, 8
    text = PR.stencil(nx, ny, nz, steps=6, embed="pad")
    full = (nz + 6, ny + 6, nx + 6)
    rng = np.random.default_rng(4)
    c = np.zeros(full)
    c[3:-3, 3:-3, 3:-3] = rng.random((nz, ny, nx))
    args = [I.Tensor(c, "f64")] + [I.Tensor(rng.uniform(-1, 1, full), "f64") for _ in range(3)]
    got, exe = gpu_run(rx, client, text, args)
    assert "map_chain" in _kinds(exe), _kinds(exe)
    ref = oracle_run(text, args)
    assert np.array_equal(got[0].a, ref[0].a)
    monkeypatch.setenv("RX_CHAIN_STEPS", "1")
    plain, exe1 = gpu_run(rx, client, text, args)
    assert "map_chain" not in _kinds(exe1) and np.array_equal(plain[0].a, got[0].a)
