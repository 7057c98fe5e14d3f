"""Differential tests on seeded random fused-HLO modules (tests/random_graphs.py): the oracle must evaluate them, the
host compiler must lower them, and on the GPU the generated kernel must agree with the oracle."""
import numpy as np
import pytest

from mononn_amd import MonoNNModule
from oracle import hlo_interp
from random_graphs import random_module

SEEDS = list(range(48))


def test_random_graphs_are_lowered_and_evaluated():
    kinds = set()
    for seed in SEEDS:
        text, inputs, descs = random_module(seed)
        want = hlo_interp.evaluate(text, inputs, {})
        assert [list(w.shape) for w in want] == [d["dims"] for d in descs]
        assert all(np.isfinite(w.astype(np.float64)).all() for w in want), seed
        m = MonoNNModule.compile(text, build=False)
        summary = m.summary()
        kinds.update(k for k in ("rowred", "elewise") if k in summary)
        m.close()
    assert kinds == {"rowred", "elewise"}          # the seeds cover row programs and plain element-wise stages


def test_random_graphs_stay_inside_their_buffers():
    # the generated kernels run thread by thread on the CPU with every buffer against guard pages (tests/cpu_bounds.py)
    from cpu_bounds import check_module
    from op_cases import arg_reduce_module, pool_module, update_slice_module
    cases = [(f"seed {s}", random_module(s)[0]) for s in SEEDS]
    cases += [("max pooling with padding", pool_module((2, 9, 10, 8), (1, 3, 3, 1), (1, 2, 2, 1), ((0, 0), (1, 1), (1, 1), (0, 0)))[0]),
              ("sum pooling, ragged", pool_module((3, 7, 5, 2), (1, 3, 2, 1), (1, 1, 2, 1), ((0, 0), (1, 1), (0, 1), (0, 0)), "sum")[0]),
              ("dynamic-update-slice", update_slice_module((6, 10, 8), (2, 4, 8), scale=2.0)),
              ("arg-max, wave per row", arg_reduce_module(7, 50)),
              ("arg-max, workgroup per row", arg_reduce_module(64, 2000)),
              ("arg-max over the major dimension", arg_reduce_module(40, 50, axis=0))]
    for name, text in cases:
        ok, msg = check_module(text)
        assert ok, f"{name}: {msg}"


def test_tuning_knobs_keep_random_graphs_inside_their_buffers():
    # the same bounds check under other specifications: vector widths, workgroup-per-row programs, small grids
    # (several units per workgroup), other workgroup sizes
    import json
    from cpu_bounds import check_module
    for seed in SEEDS[:10]:
        text = random_module(seed)[0]
        base = json.loads(MonoNNModule.compile(text, build=False).get_tuning_spec())
        for ilp, tier, grid, block in [(4, 2, 256, 256), (8, 1, 8, 256), (2, 2, 3, 512)]:
            spec = json.loads(json.dumps(base))
            for v in spec["cluster_reduce_spec"].values():
                v["ilp_factor"], v["locality_tier"] = ilp, tier
            for v in spec["cluster_elewise_spec"].values():
                v["ilp_factor"] = ilp
            spec["cuda_context"]["cuda_runtime_context"]["grid_dim"]["x"] = grid
            spec["cuda_context"]["cuda_runtime_context"]["block_dim"]["x"] = block
            ok, msg = check_module(text, json.dumps(spec))
            assert ok, f"seed {seed}, ilp {ilp}, tier {tier}, grid {grid}, block {block}: {msg}"


def _rotated_row_sum_module(R=70, C=257, k=10):
    """Row program over a row whose columns are rotated by k (slice + concatenate): the two slices are read under the
    branches of the concatenate, at addresses that are in range only where the branch is taken."""
    from mononn_amd.hlo.builder import HloModuleBuilder
    mb = HloModuleBuilder("cluster_77__rotated_rows.1")
    e = mb.entry
    x = e.parameter("f16", (R, C), "x")

    def body(f, p):
        a = f.convert(p, "f32")
        rot = f.concatenate([f.slice(a, [0, C - k], [R, C]), f.slice(a, [0, 0], [R, C - k])], 1)
        red = f.reduce(rot, f.scalar("f32", 0.0), 1, mb.reducer("add", "f32"))
        return f.convert(f.sub(rot, f.broadcast(red, (R, C), [0])), "f16")
    e.set_tuple_root([e.fusion("kInput", [x], body)])
    return mb.text()


def test_loads_under_a_condition_are_not_requested_ahead_of_it():
    # a row program asks for its operands at the top of the row; a load that sits in a branch of a concatenate is
    # only in range where the branch is taken and has to stay there
    from cpu_bounds import check_module
    text = _rotated_row_sum_module()
    src = MonoNNModule.compile(text, build=False).get_source("main.hip")
    body = src[src.index("node_fn_0("):]
    first_branch = body.index("if (q0 < 10)")
    assert "+ 247]" not in body[:first_branch] and "+ -10]" not in body[:first_branch]        # the two halves of the rotated row
    assert "+ 247]" in body[first_branch:] and "+ -10]" in body[first_branch:]
    ok, msg = check_module(text)
    assert ok, msg


@pytest.mark.gpu
def test_random_graphs_match_the_oracle(gpu_device):
    worst = 0.0
    for seed in SEEDS:
        text, inputs, descs = random_module(seed)
        want = hlo_interp.evaluate(text, inputs, {})
        m = MonoNNModule.compile(text)
        m.load(gpu_device)
        got = m.run(inputs, descs)
        m.close()
        for g, w in zip(got, want):
            g64, w64 = g.astype(np.float64), w.astype(np.float64)
            assert np.isfinite(g64).all(), seed
            # f16 results: the same rounding points as the oracle run as written, up to fast-math transcendental
            # functions and the summation order of the f32 row sums
            err = np.abs(g64 - w64) / (1.0 + np.abs(w64))
            worst = max(worst, float(err.max()))
            assert err.max() <= 2e-2, f"seed {seed}: relative error {err.max()} at {np.unravel_index(err.argmax(), err.shape)}"
    print(f"random graphs: worst relative error {worst:.3e} over {len(SEEDS)} modules")


@pytest.mark.gpu
def test_random_gemms_match_the_oracle(gpu_device):
    # the cases whose addresses tests/test_cpu_bounds.py checks on the CPU, here for their values
    import test_gpu_parity as parity
    from random_graphs import random_gemm_cases
    rng = np.random.default_rng(9)
    for case, text, spec in random_gemm_cases(5, 25):
        mb, a_dims, b_dims, d_dims = parity.gemm_module(**case)
        a = rng.normal(0, 1, a_dims).astype(np.float16)
        b = rng.normal(0, 1, b_dims).astype(np.float16)
        consts = {n: b for n in mb.constants}
        inputs = [a] if case.get("b_const") else [a, b]
        m = MonoNNModule.compile(text, spec)
        m.set_constants(consts)
        m.load(gpu_device)
        (got,) = m.run(inputs, [{"dtype": "f16", "dims": d_dims}])
        m.close()
        want = hlo_interp.evaluate(text, inputs, consts, "fp32")[0]
        scale = np.abs(want).max()
        assert np.abs(got.astype(np.float32) - want).max() <= 2e-3 * scale + 1e-3, case


@pytest.mark.gpu
def test_random_gemms_on_lds_staged_tiles_match_the_oracle(gpu_device):
    # the cases whose addresses tests/test_cpu_bounds.py checks on the CPU, here for their values
    import test_gpu_parity as parity
    from random_graphs import random_lds_gemm_cases
    rng = np.random.default_rng(10)
    for case, text, spec in random_lds_gemm_cases(6, 24):
        mb, a_dims, b_dims, d_dims = parity.gemm_module(**case)
        a = rng.normal(0, 1, a_dims).astype(np.float16)
        b = rng.normal(0, 1, b_dims).astype(np.float16)
        consts = {n: b for n in mb.constants}
        inputs = [a] if case.get("b_const") else [a, b]
        m = MonoNNModule.compile(text, spec)
        assert "gemm_tile_lds<" in m.get_source("main.hip"), case
        m.set_constants(consts)
        m.load(gpu_device)
        print(case, flush=True)
        (got,) = m.run(inputs, [{"dtype": "f16", "dims": d_dims}])
        m.close()
        want = hlo_interp.evaluate(text, inputs, consts, "fp32")[0]
        scale = np.abs(want).max()
        assert np.abs(got.astype(np.float32) - want).max() <= 2e-3 * scale + 1e-3, case


def _as_bf16(text, inputs, descs):
    """The same module with every f16 replaced by bf16; f16 inputs become bf16 bit patterns of the same values."""
    import re
    from mononn_amd import bf16
    text = re.sub(r"\bf16\b", "bf16", text)
    inputs = [bf16.to_bits(a.astype(np.float32)) if a.dtype == np.float16 else a for a in inputs]
    descs = [dict(d, dtype="bf16") if d["dtype"] == "f16" else d for d in descs]
    return text, inputs, descs


def test_random_graphs_in_bf16_are_lowered_and_stay_inside_their_buffers():
    from cpu_bounds import check_module
    for seed in SEEDS[:12]:
        text, inputs, descs = _as_bf16(*random_module(seed))
        want = hlo_interp.evaluate(text, inputs, {})
        assert all(np.isfinite(w.astype(np.float64)).all() for w in want), seed
        ok, msg = check_module(text)
        assert ok, f"seed {seed} in bf16: {msg}"


@pytest.mark.gpu
def test_random_graphs_in_bf16_match_the_oracle(gpu_device):
    from mononn_amd import bf16
    worst = 0.0
    for seed in SEEDS:
        text, inputs, descs = _as_bf16(*random_module(seed))
        want = hlo_interp.evaluate(text, inputs, {})          # as written: rounded to bf16 after every bf16 instruction
        m = MonoNNModule.compile(text)
        m.load(gpu_device)
        got = m.run(inputs, descs)
        m.close()
        for g, w, d in zip(got, want, descs):
            g64 = (bf16.from_bits(g) if d["dtype"] == "bf16" else g).astype(np.float64)
            w64 = w.astype(np.float64)
            assert np.isfinite(g64).all(), seed
            # the same rounding points on both sides; a fast-math transcendental or another summation order moves a
            # value by a bf16 spacing (2^-8 relative) here and there, and a few of those can meet in one result
            err = np.abs(g64 - w64) / (1.0 + np.abs(w64))
            worst = max(worst, float(err.max()))
            assert err.max() <= 2e-2, f"seed {seed}: relative error {err.max()} at {np.unravel_index(err.argmax(), err.shape)}"
    print(f"random graphs in bf16: worst relative error {worst:.3e} over {len(SEEDS)} modules")
