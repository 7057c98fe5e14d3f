"""Regional synchronisation (mononn_hip.regional_synchronization): chains of stages whose hand-overs stay inside one
XCD.  Counterpart of the reference's regional tier (mononn_engine/optimization/regional_synchronization_assignment_pass.cc:35-72,
global_synchronization_elimination_pass.cc:32-147): which barriers may be regional is decided from the data flow, here
element by element from where the writer's epilogue puts a value and which elements a reader's partition fetches.

CPU: the plan on an encoder (barrier tiers, partitions, plain stores only for values that stay inside an XCD), its
fall-backs, the bounds of the generated kernel.  GPU: parity with the oracle and with the same tiles under memory-side
barriers, and an exchange of integer-valued data through a regional barrier with inputs that change every launch."""
import json
import re

import numpy as np
import pytest

from mononn_amd import MonoNNModule
from mononn_amd.hlo import models
from mononn_amd.hlo.builder import HloModuleBuilder
from oracle import hlo_interp

import cpu_bounds

# 4 heads of 64, 128 rows: the heads go to 4 XCDs, FFN1's 1024 columns and FFN2's k range to 8
ENC = dict(L=2, B=1, S=128, H=256, NH=4, F=1024, vocab=300, max_pos=128)


def _gemm_nodes(summary):
    out = []
    for line in summary.splitlines():
        m = re.match(r"\s*stage (\d+)\s+gemm\s+(\S+)\s+\[(\S+)\] members=(\d+)", line)
        if m:
            out.append((int(m.group(1)), m.group(2), m.group(3), int(m.group(4))))
    return out


def encoder_spec(fx, regional=True, out_proj_split=4, ffn2_split=8, qkv_tile=(32, 32), ffn1_tile=(32, 32)):
    """Default specification of the encoder with the k splits and tiles the chains need."""
    base = MonoNNModule.compile(fx.hlo_text, build=False)
    spec = json.loads(base.get_tuning_spec())
    H, F = ENC["H"], ENC["F"]
    nodes = _gemm_nodes(base.summary())
    per_stage = {}
    for stage, _, _, _ in nodes:
        per_stage[stage] = per_stage.get(stage, 0) + 1

    def split(name, ways):
        # a GEMM split over k sheds its epilogue: its entry goes by the name of the GEMM instruction alone
        entry = spec["gemm_spec_list"].pop(name)
        entry["cutlass_config"]["split_k"] = ways
        spec["gemm_spec_list"][re.match(r"(cublas_gemm_\d+)", name).group(1)] = entry

    for stage, name, key, members in nodes:
        cc = spec["gemm_spec_list"][name]["cutlass_config"]
        tile = None
        if f"_n{F}_k{H}_" in key:
            tile = ffn1_tile
        elif f"_n{H}_k{F}_" in key:
            split(name, ffn2_split)
        elif f"_n{H}_k{H}_" in key and per_stage[stage] == 1:
            split(name, out_proj_split)
        elif f"_n{H}_k{H}_" in key:
            tile = qkv_tile
        if tile:
            cc["threadblockshape"].update(m=tile[0], n=tile[1])
            cc["warpshape"].update(m=tile[0], n=tile[1])
            cc["wave_arrangement"].update(m=1, n=1, k=4)
    base.close()
    spec["mononn_hip"]["regional_synchronization"] = regional
    return spec


def _settled_spec(fx, **kw):
    """A specification that names only nodes of the graph it produces (k splits rename nodes)."""
    spec = encoder_spec(fx, **kw)
    for _ in range(64):
        try:
            MonoNNModule.compile(fx.hlo_text, json.dumps(spec), build=False).close()
            return spec
        except Exception as e:
            m = re.search(r"names node '([^']+)'", str(e))
            if not m:
                raise
            for section in ("gemm_spec_list", "cluster_reduce_spec", "cluster_elewise_spec"):
                spec[section].pop(m.group(1), None)
    raise AssertionError("specification does not settle")


def _tiers(m):
    s = m.summary()
    g = re.search(r"barriers=(\d+)(?: \((\d+) of them over one XCD's workgroups\))?", s)
    return int(g.group(1)), int(g.group(2) or 0)


def test_three_boundaries_per_layer_become_regional():
    fx = models.bert_encoder(**ENC)
    spec = _settled_spec(fx)
    m = MonoNNModule.compile(fx.hlo_text, json.dumps(spec), build=False)
    total, regional = _tiers(m)
    # projections -> attention, attention -> output projection, FFN1 -> FFN2, in each of the two layers
    assert regional == 3 * ENC["L"] and total > regional
    src = m.get_source("main.hip")
    assert "#define MONONN_REGIONAL_SYNC 1" in src and "barrier.arrive_regional()" in src and "mononn_regional_flags" in src
    assert "parts = 4;" in src and "parts = 8;" in src
    # the same specification without the option: the kernel of before, text for text
    spec_off = json.loads(json.dumps(spec))
    spec_off["mononn_hip"]["regional_synchronization"] = False
    off = MonoNNModule.compile(fx.hlo_text, json.dumps(spec_off), build=False)
    assert _tiers(off) == (total, 0)
    src_off = off.get_source("main.hip")
    assert "regional" not in src_off and "parts" not in src_off
    # plain stores appear only where a value stays inside an XCD
    assert src.count("stN_plain<") > src_off.count("stN_plain<")
    assert json.loads(m.get_tuning_spec())["mononn_hip"]["regional_synchronization"] is True
    m.close()
    off.close()


def test_a_k_split_that_does_not_match_the_heads_keeps_its_barrier_on_the_memory_side():
    fx = models.bert_encoder(**ENC)
    # 4 heads but the output projection split 2 ways: its k slices are not head runs of the attention's partition
    m = MonoNNModule.compile(fx.hlo_text, json.dumps(_settled_spec(fx, out_proj_split=2)), build=False)
    _, regional = _tiers(m)
    assert regional == 2 * ENC["L"]
    m.close()
    # FFN1 tiles of 48 columns do not divide the 128 columns of an XCD's slice: FFN1 stays round-robin, FFN2's read crosses XCDs
    m = MonoNNModule.compile(fx.hlo_text, json.dumps(_settled_spec(fx, ffn1_tile=(32, 48))), build=False)
    _, regional = _tiers(m)
    assert regional == 2 * ENC["L"]
    m.close()


def test_projections_stay_round_robin_when_the_xcds_would_need_a_second_round():
    fx = models.bert_encoder(**ENC)
    # 32x16 tiles: 3 projections x 4 x 4 tiles = 48 units for the 32 workgroups of an XCD, two rounds, where the 192
    # units of the stage took one round of the grid: the projections stay as they were, the attention keeps its heads
    # on the XCDs for the output projection's sake
    m = MonoNNModule.compile(fx.hlo_text, json.dumps(_settled_spec(fx, qkv_tile=(32, 16))), build=False)
    assert _tiers(m)[1] == 2 * ENC["L"]
    m.close()


def test_generated_kernel_stays_inside_its_buffers():
    fx = models.bert_encoder(**ENC)
    ok, msg = cpu_bounds.check_module(fx.hlo_text, json.dumps(_settled_spec(fx)))
    assert ok, msg


def exchange_module(M=128, K=256, F=1024, N=256):
    """x[M,K] . w1[K,F] -> h (a GEMM whose column slices go to the XCDs) -> h . w2[F,N] split 8 ways over k -> sum of
    the partial sums + 1: two hand-overs, the first one regional."""
    mb = HloModuleBuilder("cluster_9__regional_exchange.1")
    e = mb.entry
    x = e.parameter("f16", (M, K), "x")
    w1 = e.elided_constant("f16", (K, F), "w1/kernel")
    w2 = e.elided_constant("f16", (F, N), "w2/kernel")
    h = e.gemm(x, w1, 1, 0)
    y = e.gemm(h, w2, 1, 0)
    z = e.fusion("kLoop", [y], lambda f, p: f.add(p, f.splat("f16", 1.0, p.dims)))
    e.set_tuple_root([z])
    return mb, (M, K, F, N)


def exchange_spec(text, regional):
    spec = json.loads(MonoNNModule.compile(text, build=False).get_tuning_spec())
    names = [n.replace(".", "_").replace("-", "_") for n in re.findall(r"%(cublas-gemm\.\d+) =", text)]
    g1, g2 = spec["gemm_spec_list"][names[0]], None
    g1["cutlass_config"]["threadblockshape"].update(m=32, n=32)
    g1["cutlass_config"]["warpshape"].update(m=32, n=32)
    template = json.loads(json.dumps(g1))
    spec["gemm_spec_list"] = {names[0]: g1, names[1]: template}
    spec["gemm_spec_list"][names[1]]["cutlass_config"]["split_k"] = 8
    spec["cluster_elewise_spec"] = {}
    spec["cluster_reduce_spec"] = {}
    spec["mononn_hip"]["regional_synchronization"] = regional
    return json.dumps(spec)


def test_exchange_module_has_one_regional_and_one_memory_side_barrier():
    mb, _ = exchange_module()
    m = MonoNNModule.compile(mb.text(), exchange_spec(mb.text(), True), build=False)
    assert _tiers(m) == (2, 1)
    ok, msg = cpu_bounds.check_module(mb.text(), exchange_spec(mb.text(), True))
    assert ok, msg
    m.close()


@pytest.mark.gpu
def test_regional_barrier_hands_over_complete_data(gpu_device):
    """Integer-valued f16 data (every product and sum exact) through GEMM -> regional barrier -> k-split GEMM ->
    memory-side barrier -> sum, 40 launches with fresh inputs: a store that is still on its way when the regional flag
    is seen, a reader that looks into another XCD's slice, or a line left from the launch before is a wrong value.
    Every consumer workgroup reads tiles that 4 to 8 other workgroups (compute units) of its XCD wrote.
    From launch 20 on a second stream exists and has run a kernel: the hardware then starts dealing the workgroups of
    a launch on this stream at another XCD (measured: workgroup b on XCD (b + 7) % 8 instead of b % 8), which must not
    matter, because workgroups with equal b % 8 still share an XCD."""
    import torch
    mb, (M, K, F, N) = exchange_module()
    rng = np.random.default_rng(5)
    w1 = rng.integers(-1, 2, (K, F)) * (rng.random((K, F)) < 0.05)
    w2 = rng.integers(-1, 2, (F, N)) * (rng.random((F, N)) < 0.02)
    names = list(mb.constants)
    m = MonoNNModule.compile(mb.text(), exchange_spec(mb.text(), True))
    assert _tiers(m) == (2, 1)
    m.set_constants({names[0]: w1.astype(np.float16), names[1]: w2.astype(np.float16)})
    m.load(gpu_device)
    for launch in range(40):
        if launch == 20:
            side = torch.cuda.Stream(device=torch.device("cuda", gpu_device))
            with torch.cuda.stream(side):
                torch.zeros(100 * 1024, device=torch.device("cuda", gpu_device)).add_(1.0)
            side.synchronize()
        x = rng.integers(-3, 4, (M, K))
        h = x @ w1
        want = h @ w2 + 1
        assert np.abs(h).max() < 2048 and np.abs(want).max() < 2048   # exactly representable all the way
        got = m.run([x.astype(np.float16)], [{"dtype": "f16", "dims": [M, N]}])[0]
        assert np.array_equal(got.astype(np.int64), want), f"launch {launch}: {(got.astype(np.int64) != want).sum()} wrong values"
    m.close()


@pytest.mark.gpu
def test_encoder_with_regional_barriers_matches_the_oracle_and_the_memory_side_build(gpu_device):
    fx = models.bert_encoder(**ENC)
    consts = fx.make_constants(21, "random")
    spec = _settled_spec(fx)
    outs = {}
    for regional in (True, False):
        s = json.loads(json.dumps(spec))
        s["mononn_hip"]["regional_synchronization"] = regional
        m = MonoNNModule.compile(fx.hlo_text, json.dumps(s))
        assert (_tiers(m)[1] > 0) == regional
        m.set_constants(consts)
        m.load(gpu_device)
        runs = []
        for seed in (21, 22, 23):
            runs.append(m.run(fx.make_inputs(seed), fx.outputs)[0])
        # and again: the temp arena now holds the values of the launch before
        again = m.run(fx.make_inputs(21), fx.outputs)[0]
        assert np.array_equal(again, runs[0])
        outs[regional] = runs
        m.close()
    for a, b in zip(outs[True], outs[False]):
        assert np.array_equal(a, b)   # same tiles, same order of every sum: bit for bit
    want = hlo_interp.evaluate(fx.hlo_text, fx.make_inputs(21), consts, "fp32")[0].astype(np.float64).ravel()
    got = outs[True][0].astype(np.float64).ravel()
    assert np.abs(got - want).max() <= 2e-2 and got @ want / (np.linalg.norm(got) * np.linalg.norm(want)) >= 0.9999
