"""Minor-to-major orders other than the descending one (ir_parser_fused.cc:132-152) and column-major GEMM results
(gemm_impl.cc:345-351, :408-469).

The oracle's reading of a layout is pinned first, against element offsets computed from strides by brute force and
against np.transpose / np.einsum; then the compiler is checked against the oracle (program structure and buffer
bounds on the CPU, values on the GPU).
"""
import itertools
import re

import numpy as np
import pytest

import test_gpu_parity as parity
from cpu_bounds import check_module
from mononn_amd import MonoNNError, MonoNNModule
from mononn_amd.hlo.builder import HloModuleBuilder
from oracle import hlo_interp


def relayout(text, layouts):
    """Replace the layout printed on the defining line of each named instruction."""
    for name, lay in layouts.items():
        pat = re.compile(r"(%" + re.escape(name) + r" = [a-z0-9]+\[[0-9,]*\])\{[0-9,]*\}")
        text, n = pat.subn(lambda m: m.group(1) + "{" + ",".join(map(str, lay)) + "}", text)
        assert n == 1, name
    return text


def offsets_by_strides(dims, layout):
    """Flat element offset of every logical index when minor_to_major[0] is the fastest-varying dimension."""
    stride, s = {}, 1
    for d in layout:
        stride[d] = s
        s *= dims[d]
    off = np.zeros(dims, dtype=np.int64)
    for idx in itertools.product(*[range(d) for d in dims]):
        off[idx] = sum(i * stride[d] for d, i in enumerate(idx))
    return off


def to_memory(a, layout):
    """Memory image of a logical array: flat buffer filled by stride arithmetic, shaped slowest dimension first."""
    flat = np.zeros(a.size, dtype=a.dtype)
    flat[offsets_by_strides(a.shape, layout).ravel()] = a.ravel()
    return flat.reshape([a.shape[d] for d in reversed(layout)])


def from_memory(buf, dims, layout):
    return buf.ravel()[offsets_by_strides(dims, layout)]


def elementwise_module(dims, in_layout, out_layout, dtype="f32"):
    mb = HloModuleBuilder("cluster_9__layouts.1")
    e = mb.entry
    x = e.parameter(dtype, dims, "x")
    y = e.parameter(dtype, dims, "y")

    def body(f, px, py):
        return f.add(f.mul(px, f.splat(dtype, 2.0, dims)), py)
    z = e.fusion("kLoop", [x, y], body)
    e.set_tuple_root([z])
    return relayout(mb.text(), {x.name: in_layout, z.name: out_layout}), z.name


def bitcast_module(in_dims, in_layout, out_dims, out_layout, dtype="f32"):
    mb = HloModuleBuilder("cluster_9__bitcast_layouts.1")
    e = mb.entry
    x = e.parameter(dtype, in_dims, "x")
    h = e.unary("negate", x)              # a computed value, so that the bitcast's operand is not a buffer itself
    b = e.bitcast(h, out_dims)
    z = e.unary("negate", b)
    e.set_tuple_root([z])
    return relayout(mb.text(), {h.name: in_layout, b.name: out_layout})


LAYOUTS_3D = [(2, 1, 0), (0, 1, 2), (0, 2, 1), (1, 0, 2), (1, 2, 0), (2, 0, 1)]


# ---- the oracle -------------------------------------------------------------------------------------------------
def test_oracle_memory_image_follows_the_strides():
    rng = np.random.default_rng(1)
    v = rng.normal(size=(2, 3, 4)).astype(np.float32)
    for lay in LAYOUTS_3D:
        sh = hlo_interp.Shape("f32", v.shape, layout=None if lay == (2, 1, 0) else list(lay))
        img = hlo_interp._memory_image(v, sh)
        assert img.shape == tuple(v.shape[d] for d in reversed(lay))
        assert np.array_equal(img, to_memory(v, lay)), lay
        assert np.array_equal(hlo_interp._from_memory(img, sh), v), lay


def test_oracle_parameters_and_results_are_memory_images():
    rng = np.random.default_rng(2)
    dims = (3, 4, 5)
    x = rng.normal(size=dims).astype(np.float32)
    y = rng.normal(size=dims).astype(np.float32)
    for lin, lout in itertools.product(LAYOUTS_3D[1:4], LAYOUTS_3D):
        text, _ = elementwise_module(dims, lin, lout)
        got = hlo_interp.evaluate(text, [to_memory(x, lin), y])[0]
        assert np.array_equal(got, to_memory(2 * x + y, lout)), (lin, lout)
    # two dimensions: a {0,1} buffer is the transposed array
    text, _ = elementwise_module((4, 6), (0, 1), (0, 1))
    base = np.arange(24, dtype=np.float32).reshape(4, 6)
    got = hlo_interp.evaluate(text, [np.ascontiguousarray(base.T), np.zeros((4, 6), np.float32)])[0]
    assert np.array_equal(got, (2 * base).T)


def test_oracle_bitcast_keeps_the_bytes():
    rng = np.random.default_rng(3)
    # the textbook case: [A,B]{0,1} -> [B,A]{1,0} is the logical transpose, and back
    x = rng.normal(size=(5, 7)).astype(np.float32)
    assert np.array_equal(hlo_interp.evaluate(bitcast_module((5, 7), (0, 1), (7, 5), (1, 0)), [x])[0], x.T)
    assert np.array_equal(hlo_interp.evaluate(bitcast_module((5, 7), (1, 0), (7, 5), (0, 1)), [x])[0], x.T)
    # descending on both sides: a reshape
    assert np.array_equal(hlo_interp.evaluate(bitcast_module((5, 7), (1, 0), (35,), (0,)), [x])[0], x.reshape(35))
    # general: the flat buffers under the two (shape, layout) pairs agree element by element (the module negates
    # before and after the bitcast, so values come back exactly)
    v = rng.normal(size=(2, 3, 4)).astype(np.float32)
    for lin, (out_dims, lout) in itertools.product(LAYOUTS_3D, [((4, 6), (0, 1)), ((6, 4), (1, 0)), ((3, 2, 4), (1, 2, 0)), ((4, 3, 2), (0, 1, 2))]):
        got = hlo_interp.evaluate(bitcast_module(v.shape, lin, out_dims, lout), [v])[0]
        assert np.array_equal(got, from_memory(to_memory(v, lin), out_dims, lout)), (lin, out_dims, lout)


GEMM_LAYOUT_CASES = [
    (dict(M=128, N=96, K=64), {"b": (0, 1)}),                               # B [K,N] held column-major: k-contiguous
    (dict(M=128, N=96, K=64), {"d": (0, 1)}),                               # column-major result, B strided: GEMM + transposing stage
    (dict(M=100, N=72, K=64, rhs_c=1), {"d": (0, 1)}),                      # column-major result by exchanging the operands
    (dict(M=40, N=24, K=64), {"a": (0, 1)}),                                # A held [K,M]
    (dict(M=128, N=96, K=64), {"a": (0, 1), "b": (0, 1), "d": (0, 1)}),     # everything column-major
    (dict(M=64, N=48, K=32, batch=(2, 3), rhs_c=3), {"d": (2, 3, 1, 0)}),   # batched, column-major result
    (dict(M=64, N=48, K=32, batch=(3,)), {"b": (1, 2, 0), "d": (1, 0, 2)}),  # batched: B k-contiguous by layout, batch innermost in D
    (dict(M=96, N=80, K=48, dtype="f32", rhs_c=1), {"a": (0, 1), "d": (0, 1)}),   # f32
]


def gemm_with_layouts(case, lays):
    mb, a_dims, b_dims, d_dims = parity.gemm_module(**case)
    text = mb.text()
    names = {"a": re.search(r"%(a\.\d+) =", text).group(1), "b": re.search(r"%(b\.\d+) =", text).group(1),
             "d": re.search(r"%(cublas-(?:batch-)?gemm\.\d+) =", text).group(1)}
    full = {k: tuple(lays.get(k, tuple(reversed(range(len(a_dims)))))) for k in "abd"}
    return relayout(text, {names[k]: full[k] for k in "abd"}), (a_dims, b_dims, d_dims), full


def gemm_reference(case, a, b):
    r = a.ndim
    sub_a = "...mk" if case.get("lhs_c", r - 1) == r - 1 else "...km"
    sub_b = "...kn" if case.get("rhs_c", r - 2) == r - 2 else "...nk"
    return np.einsum(f"{sub_a},{sub_b}->...mn", a.astype(np.float64), b.astype(np.float64)) * case.get("alpha", 1.0)


@pytest.mark.parametrize("case,lays", GEMM_LAYOUT_CASES)
def test_oracle_gemm_with_layouts_against_einsum(case, lays):
    text, (a_dims, b_dims, d_dims), full = gemm_with_layouts(case, lays)
    rng = np.random.default_rng(4)
    npdt = np.float32 if case.get("dtype") == "f32" else np.float16
    a = rng.normal(size=a_dims).astype(npdt)
    b = rng.normal(size=b_dims).astype(npdt)
    got = hlo_interp.evaluate(text, [to_memory(a, full["a"]), to_memory(b, full["b"])], precision="fp32")[0]
    want = to_memory(gemm_reference(case, a, b), full["d"])
    assert got.shape == want.shape and np.abs(got - want).max() <= 1e-4 * np.abs(want).max()


# ---- the compiler, on the CPU -----------------------------------------------------------------------------------
def test_layout_syntax_outside_the_dialect_is_refused():
    text, _ = elementwise_module((4, 6), (0, 1), (1, 0))
    with pytest.raises(MonoNNError, match="tiled or annotated"):
        MonoNNModule.compile(text.replace("f32[4,6]{0,1} parameter", "f32[4,6]{0,1:T(2,128)} parameter"), build=False)
    with pytest.raises(MonoNNError, match="not a permutation"):
        MonoNNModule.compile(text.replace("f32[4,6]{0,1} parameter", "f32[4,6]{1,1} parameter"), build=False)
    with pytest.raises(MonoNNError, match="rank mismatch"):
        MonoNNModule.compile(text.replace("f32[4,6]{0,1} parameter", "f32[4,6]{0} parameter"), build=False)


def test_transposes_next_to_a_gemm_go_into_the_call():
    def compiled(case, lays):
        m = MonoNNModule.compile(gemm_with_layouts(case, lays)[0], build=False)
        return m.get_source("main.hip"), m.launch_dims()["barriers"]
    # B [K,N]{0,1} is an [N,K] row-major buffer: the k-contiguous MFMA fetch, no gather, one stage
    src, barriers = compiled(dict(M=128, N=96, K=64), {"b": (0, 1)})
    tile = re.search(r"gemm_tile<([^>]*)>", src).group(1).split(", ")
    assert barriers == 0 and tile[-3] == "false" and "gemm_naive_element" not in src      # B_ALONG_N off
    # column-major D with both operands k-contiguous: operands exchanged, still one stage on the MFMAs
    src, barriers = compiled(dict(M=100, N=72, K=64, rhs_c=1), {"d": (0, 1)})
    assert barriers == 0 and "gemm_tile<" in src and "gemm_naive_element" not in src
    # column-major D with B strided along k: left as GEMM + transposing stage
    src, barriers = compiled(dict(M=128, N=96, K=64), {"d": (0, 1)})
    assert barriers == 1 and "gemm_tile<" in src
    # everything column-major: A^T and B^T folded, then exchanged
    src, barriers = compiled(dict(M=128, N=96, K=64), {"a": (0, 1), "b": (0, 1), "d": (0, 1)})
    assert barriers == 0 and "gemm_tile<" in src and "gemm_naive_element" not in src


@pytest.mark.parametrize("which", range(len(GEMM_LAYOUT_CASES)))
def test_gemm_layout_cases_stay_inside_their_buffers(which):
    case, lays = GEMM_LAYOUT_CASES[which]
    ok, msg = check_module(gemm_with_layouts(case, lays)[0])
    assert ok, msg


def test_elementwise_and_bitcast_layout_cases_stay_inside_their_buffers():
    ok, msg = check_module(elementwise_module((6, 10, 14), (0, 2, 1), (1, 0, 2))[0])
    assert ok, msg
    ok, msg = check_module(bitcast_module((6, 10, 14), (1, 2, 0), (14, 60), (0, 1)))
    assert ok, msg


# ---- the compiler, on the GPU -----------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("case,lays", GEMM_LAYOUT_CASES)
def test_gemm_layout_cases(gpu_device, case, lays):
    text, (a_dims, b_dims, d_dims), full = gemm_with_layouts(case, lays)
    rng = np.random.default_rng(5)
    f32 = case.get("dtype") == "f32"
    npdt = np.float32 if f32 else np.float16
    a = to_memory(rng.normal(size=a_dims).astype(npdt), full["a"])
    b = to_memory(rng.normal(size=b_dims).astype(npdt), full["b"])
    out_dims = [d_dims[d] for d in reversed(full["d"])]
    (got,), m = parity.run_module(text, [a, b], {}, [{"dtype": "f32" if f32 else "f16", "dims": out_dims}])
    m.close()
    want = hlo_interp.evaluate(text, [a, b], precision="fp32")[0]
    assert got.shape == want.shape
    if f32:
        assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()
    else:
        parity.check_close(got, want, atol=2e-2 * max(1.0, float(np.abs(want).max()) / 8))


@pytest.mark.gpu
def test_elementwise_and_bitcast_layouts(gpu_device):
    rng = np.random.default_rng(6)
    dims = (6, 10, 14)
    x = rng.normal(size=dims).astype(np.float32)
    y = rng.normal(size=dims).astype(np.float32)
    for lin, lout in [((0, 2, 1), (1, 0, 2)), ((1, 2, 0), (2, 1, 0)), ((2, 1, 0), (0, 1, 2))]:
        text, _ = elementwise_module(dims, lin, lout)
        ins = [to_memory(x, lin), y]
        want = hlo_interp.evaluate(text, ins)[0]
        (got,), m = parity.run_module(text, ins, {}, [{"dtype": "f32", "dims": list(want.shape)}])
        m.close()
        assert np.array_equal(got, want), (lin, lout)
    for lin, out_dims, lout in [((1, 2, 0), (14, 60), (0, 1)), ((0, 1, 2), (10, 6, 14), (1, 2, 0)), ((2, 1, 0), (84, 10), (0, 1))]:
        text = bitcast_module(dims, lin, out_dims, lout)
        want = hlo_interp.evaluate(text, [x])[0]
        (got,), m = parity.run_module(text, [x], {}, [{"dtype": "f32", "dims": list(want.shape)}])
        m.close()
        assert np.array_equal(got, want), (lin, out_dims, lout)
