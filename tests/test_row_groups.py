"""Row programs with a wave on 8, 4 or 2 rows at once (cluster_reduce_spec reduce_implementation 1, 2, 3): 8, 16 or 32
lanes per row, 16-byte runs per lane, reductions over the lanes that share lane % 8 (4, 2).  Addresses on the CPU,
values against the oracle on the GPU; rows whose length does not split into whole runs, or gives a lane of the row
nothing to do, fall back to one row per wave."""
import json

import numpy as np
import pytest

import test_gpu_parity as parity
from cpu_bounds import check_module
from mononn_amd import MonoNNModule
from mononn_amd.hlo import models
from mononn_amd.hlo.builder import HloModuleBuilder
from op_cases import arg_reduce_module
from oracle import hlo_interp


ROWS_PER_WAVE = {1: 8, 2: 4, 3: 2}      # reduce_implementation -> rows a wave takes at once


def takes_row_groups(length, dtype, impl):
    run = 4 if dtype == "f32" else 8         # elements of a 16-byte run
    lanes = 64 // ROWS_PER_WAVE[impl]
    return length % run == 0 and length // run >= lanes and -(-(length // run) // lanes) * run <= 160


def rows8_spec(text, grid=None, impl=1):
    spec = json.loads(MonoNNModule.compile(text, build=False).get_tuning_spec())
    assert spec["cluster_reduce_spec"]
    for v in spec["cluster_reduce_spec"].values():
        v["locality_tier"], v["ilp_factor"], v["reduce_implementation"] = 1, 1, impl
    if grid:
        spec["cuda_context"]["cuda_runtime_context"]["grid_dim"]["x"] = grid
    return json.dumps(spec)


def normalise_module(rows, length, dtype="f16"):
    """Mean / variance normalisation of every row with a per-column scale (two dependent reductions, one full output
    and the row means as a second, per-row output)."""
    mb = HloModuleBuilder("cluster_5__rows8.1")
    e = mb.entry
    x = e.parameter(dtype, (rows, length), "x")
    g = e.parameter(dtype, (length,), "gamma")

    def body(f, px, pg):
        a = f.convert(px, "f32")
        s = f.reduce(a, f.scalar("f32", 0.0), 1, mb.reducer("add", "f32"))
        mean = f.mul(s, f.splat("f32", 1.0 / length, (rows,)))
        c = f.sub(a, f.broadcast(mean, (rows, length), [0]))
        var = f.mul(f.reduce(f.mul(c, c), f.scalar("f32", 0.0), 1, mb.reducer("add", "f32")), f.splat("f32", 1.0 / length, (rows,)))
        r = f.rsqrt(f.add(var, f.splat("f32", 1e-5, (rows,))))
        y = f.mul(f.mul(c, f.broadcast(r, (rows, length), [0])), f.broadcast(f.convert(pg, "f32"), (rows, length), [1]))
        return f.convert(y, dtype), mean
    y, mean = e.fusion("kInput", [x, g], body)
    e.set_tuple_root([y, mean])
    return mb.text(), [{"dtype": dtype, "dims": [rows, length]}, {"dtype": "f32", "dims": [rows]}]


CASES = [(100, 64, "f16"), (37, 256, "f16"), (16, 1024, "f16"), (2100, 768, "f16"), (50, 32, "f32"), (9, 1280, "f16")]


@pytest.mark.parametrize("impl", [1, 2, 3])
def test_rows8_programs_are_generated_and_stay_inside_their_buffers(impl):
    G = ROWS_PER_WAVE[impl]
    for rows, length, dtype in CASES:
        text, _ = normalise_module(rows, length, dtype)
        for grid in (256, 3):
            spec = rows8_spec(text, grid, impl)
            src = MonoNNModule.compile(text, spec, build=False).get_source("main.hip")
            if takes_row_groups(length, dtype, impl):
                assert f"lane_group_all_reduce<{G}>" in src and f"* {G} + (lane & {G - 1})" in src, (rows, length, dtype)
            else:
                assert "lane_group_all_reduce" not in src and "wave_all_reduce" in src, (rows, length, dtype)
            if rows <= 100 or grid == 256:
                ok, msg = check_module(text, spec)
                assert ok, f"{rows} x {length} {dtype}, grid {grid}: {msg}"
    # (value, index) reduce: the exchange stays inside the lanes of a row
    text = arg_reduce_module(21, 256)
    spec = rows8_spec(text, impl=impl)
    src = MonoNNModule.compile(text, spec, build=False).get_source("main.hip")
    assert f"off >= {G}" in src
    ok, msg = check_module(text, spec)
    assert ok, msg


def test_rows_that_do_not_split_into_whole_runs_keep_one_row_per_wave():
    for rows, length in ((40, 197), (40, 36), (40, 4096)):
        text, _ = normalise_module(rows, length)
        src = MonoNNModule.compile(text, rows8_spec(text), build=False).get_source("main.hip")
        assert "lane_group_all_reduce" not in src and "wave_all_reduce" in src, (rows, length)


def test_rows8_is_the_default_for_many_rows_and_feeds_fragment_order_operands():
    # BERT-large's shape: 6144 rows of 1024; the LayerNorm results go to the next GEMM in MFMA fragment order
    fx = models.bert_encoder(L=1, B=16, S=384, H=1024, NH=16, F=4096, mask_kind="length_mask")
    m = MonoNNModule.compile(fx.hlo_text, build=False)
    spec = json.loads(m.get_tuning_spec())
    assert all(v["reduce_implementation"] == 1 and v["locality_tier"] == 1 for v in spec["cluster_reduce_spec"].values())
    assert "lane_group_all_reduce<8>" in m.get_source("main.hip")
    # BERT-base's 128 rows stay on the workgroup-per-row programs
    spec = json.loads(MonoNNModule.compile(models.bert_layer().hlo_text, build=False).get_tuning_spec())
    assert all(v["reduce_implementation"] == 0 for v in spec["cluster_reduce_spec"].values())


def test_rows8_encoder_stays_inside_its_buffers():
    fx = models.bert_encoder(L=1, B=2, S=40, H=128, NH=2, F=256, vocab=100, max_pos=64)
    ok, msg = check_module(fx.hlo_text, rows8_spec(fx.hlo_text))
    assert ok, msg


@pytest.mark.gpu
@pytest.mark.parametrize("impl", [1, 2, 3])
def test_rows8_programs_match_the_oracle(gpu_device, impl):
    rng = np.random.default_rng(11)
    for rows, length, dtype in CASES:
        text, outs = normalise_module(rows, length, dtype)
        npdt = np.float32 if dtype == "f32" else np.float16
        x = (rng.normal(0.3, 1.5, (rows, length))).astype(npdt)
        g = rng.normal(1.0, 0.2, (length,)).astype(npdt)
        want = hlo_interp.evaluate(text, [x, g])
        for grid in (256, 3):
            got, m = parity.run_module(text, [x, g], {}, outs, rows8_spec(text, grid, impl))
            m.close()
            assert np.abs(got[0].astype(np.float32) - want[0].astype(np.float32)).max() <= (2e-5 if dtype == "f32" else 4e-3), (rows, length, dtype, grid)
            assert np.abs(got[1] - want[1]).max() <= 1e-5, (rows, length, dtype, grid)
    text = arg_reduce_module(21, 256)
    x = rng.integers(-6, 7, (21, 256)).astype(np.float16)        # many ties: the first index wins
    (v, i), m = parity.run_module(text, [x], {}, [{"dtype": "f16", "dims": [21]}, {"dtype": "s32", "dims": [21]}], rows8_spec(text, impl=impl))
    m.close()
    assert np.array_equal(i, np.argmax(x, axis=1).astype(np.int32)) and np.array_equal(v, x.max(axis=1))


@pytest.mark.gpu
def test_rows8_encoder_matches_the_oracle(gpu_device):
    # LayerNorm results stored in fragment order for the next GEMM, split-K partial sums added by the row program,
    # a soft-max outside the fused attention (fusion off)
    fx = models.bert_encoder(L=2, B=2, S=40, H=128, NH=2, F=256, vocab=100, max_pos=64)
    consts, inputs = fx.make_constants(5, "random"), fx.make_inputs(5)
    want = hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0]
    for hip in ({}, {"fuse_attention": False}):
        spec = json.loads(rows8_spec(fx.hlo_text))
        if hip:
            spec = json.loads(parity._spec_with(fx.hlo_text, hip=hip))
            for v in spec["cluster_reduce_spec"].values():
                v["locality_tier"], v["ilp_factor"], v["reduce_implementation"] = 1, 1, 1
            base = json.loads(MonoNNModule.compile(fx.hlo_text, json.dumps(spec), build=False).get_tuning_spec())
            for v in base["cluster_reduce_spec"].values():
                v["locality_tier"], v["ilp_factor"], v["reduce_implementation"] = 1, 1, 1
            spec = base
        (got,), m = parity.run_module(fx.hlo_text, inputs, consts, fx.outputs, json.dumps(spec))
        assert "lane_group_all_reduce<8>" in m.get_source("main.hip")
        m.close()
        parity.check_close(got, want, atol=3e-2)
