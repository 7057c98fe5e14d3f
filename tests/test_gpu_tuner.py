"""GPU tests of the tuner (MonoNNModuleTuner::tune, mononn_module_tuner.cc:620-991): it must hand back a module that
computes the same function as the default one, leave the reference's dump tree behind, and that tree must be enough
to rebuild the same kernel (TF_MONONN_EXISTING_TUNING_SPEC_DIR contract, README.md:145-149)."""
import json
import os
import re

import numpy as np
import pytest

from mononn_amd import MonoNNModule, MonoNNModuleTuner
from mononn_amd.hlo import models
from oracle import hlo_interp

pytestmark = pytest.mark.gpu


def _check(got, want32):
    g, w = got.astype(np.float64).ravel(), want32.astype(np.float64).ravel()
    assert np.abs(g - w).max() <= 2e-2                                         # the north star's tolerance
    assert float(g @ w / (np.linalg.norm(g) * np.linalg.norm(w))) >= 0.9999


@pytest.fixture(scope="module")
def encoder():
    # FFN2 contracts over 1024: long enough for the split-K phase to consider it
    fx = models.bert_encoder(L=2, B=1, S=64, H=256, NH=4, F=1024, vocab=300, max_pos=64)
    consts, inputs = fx.make_constants(31, "random"), fx.make_inputs(31)
    return fx, consts, inputs, hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0]


def test_tuned_module_dump_tree_and_reload(gpu_device, encoder, tmp_path, monkeypatch):
    fx, consts, inputs, want = encoder
    monkeypatch.setenv("MONONN_TUNER_VERBOSE", "0")
    dump = str(tmp_path / "dump")
    tuned = MonoNNModuleTuner.tune(fx.hlo_text, gpu_device, dump, budget=2)   # fastest: one launch shape, few tiles
    tuned.set_constants(consts)
    tuned.load(gpu_device)
    got = tuned.run(inputs, fx.outputs)[0]
    _check(got, want)
    # dump tree (mononn_module_tuner.cc:374-383, 457-603)
    cluster = os.path.join(dump, "cluster_0")
    names = set(os.listdir(cluster))
    assert {"best_tuning_spec.json", "best_tuning_spec.hsaco", "best_tuning_spec_src", "tuning_log.log", "performance_report.csv"} <= names
    contexts = [n[:-5] for n in names if n.endswith(".json") and n != "best_tuning_spec.json"]
    assert contexts and all(f"{c}.hsaco" in names and f"{c}_src" in names for c in contexts)
    log = open(os.path.join(cluster, "tuning_log.log")).read()
    assert "Tuning result for each thread grid setting" in log and "gemm x" in log and " ms\n" in log
    assert "whole kernel" in log                         # the class winners were confirmed in the whole kernel
    # the stage-fusion decisions were tried as whole-kernel alternatives (tuning_space_generator.cc:139-307: per-node
    # implementation alternatives), each with a verdict, and the specification records what was kept
    import re
    verdicts = dict(re.findall(r"fusion decision (\w+), whole kernel: now [\d.]+ us;.*?-> (adopted|not adopted)", log))
    for line in log.splitlines():
        if "fusion decision" in line:
            print(line[:500], flush=True)
    hip = json.loads(tuned.get_tuning_spec())["mononn_hip"]
    # (the prologue fusion is not a question of its own once the folding, which implies it, has been adopted)
    assert {"regional_synchronization", "attention_out_proj_fusion", "layer_norm_folding"} <= set(verdicts), verdicts
    assert "gemm_prologue_fusion" in verdicts or hip["gemm_prologue_fusion"] is True
    for name, verdict in verdicts.items():
        if verdict == "adopted":
            assert hip[name] is True
    assert not re.search(r"=-1\.00(?! \[)", log)         # a candidate that produced no kernel says why
    report = open(os.path.join(cluster, "performance_report.csv")).read().splitlines()
    assert len(report) > 10 and all(len(r.split(",")) == 3 for r in report[1:])
    # the tree is enough to get the same kernel back, bit for bit
    again = MonoNNModule.from_spec_dir(fx.hlo_text, dump)
    assert json.loads(again.get_tuning_spec()) == json.loads(tuned.get_tuning_spec())
    again.set_constants(consts)
    again.load(gpu_device)
    assert np.array_equal(again.run(inputs, fx.outputs)[0].view(np.uint16), got.view(np.uint16))
    # and the tuned kernel is not slower than the default one (same launch shape family, 5% slack for noise)
    import torch
    default = MonoNNModule.compile(fx.hlo_text)
    default.set_constants(consts)
    default.load(gpu_device)
    default.run(inputs, fx.outputs)
    stream = torch.cuda.current_stream().cuda_stream
    t_def, _ = default.time_raw(default.buffer_pointers(), stream, 10, 100)
    t_tuned, _ = tuned.time_raw(tuned.buffer_pointers(), stream, 10, 100)
    print(f"default {t_def * 1e3:.1f} us, tuned {t_tuned * 1e3:.1f} us")
    assert t_tuned <= 1.05 * t_def


@pytest.fixture(scope="module")
def first_run(gpu_device, encoder, tmp_path_factory):
    """Dump directory of an unseeded tuning run (shared by the tests that start from a seed)."""
    fx, _, _, _ = encoder
    first = str(tmp_path_factory.mktemp("seed") / "first")
    MonoNNModuleTuner.tune(fx.hlo_text, gpu_device, first, budget=2).close()
    return first


def test_tuning_from_a_seed_specification(gpu_device, encoder, first_run, tmp_path, monkeypatch):
    fx, consts, inputs, want = encoder
    monkeypatch.setenv("MONONN_TUNER_SEED_SPEC_DIR", first_run)
    second = str(tmp_path / "second")
    tuned = MonoNNModuleTuner.tune(fx.hlo_text, gpu_device, second, budget=2)
    log = open(os.path.join(second, "cluster_0", "tuning_log.log")).read()
    assert "with the seed specification" in log
    tuned.set_constants(consts)
    tuned.load(gpu_device)
    _check(tuned.run(inputs, fx.outputs)[0], want)


def test_row_programs_and_fusion_decisions_from_a_seed(gpu_device, encoder, first_run, tmp_path, monkeypatch):
    """A run that keeps the seed's tiles and searches only the row programs and the stage-fusion decisions: it starts
    from the seed's decisions, and the rows-per-wave variants are among what it tries."""
    fx, consts, inputs, want = encoder
    monkeypatch.setenv("MONONN_TUNER_SEED_SPEC_DIR", first_run)
    monkeypatch.setenv("MONONN_TUNER_ONLY_FUSION_DECISIONS", "1")
    monkeypatch.setenv("MONONN_TUNER_ROW_PROGRAMS_TOO", "1")
    out = str(tmp_path / "rows")
    again = MonoNNModuleTuner.tune(fx.hlo_text, gpu_device, out, budget=2)
    log = open(os.path.join(out, "cluster_0", "tuning_log.log")).read()
    assert "tier1_rows2=" in log and "tier1_rows4=" in log and "fusion decision" in log
    assert not re.search(r"gemm x\d+ \([^)]*\): best \S+ [\d.]+ us per stage; default=[\d.]+ \S", log), "GEMM classes keep the seed's tiles"
    seed_hip = json.loads(open(os.path.join(first_run, "cluster_0", "best_tuning_spec.json")).read())["mononn_hip"]
    if any(seed_hip[k] for k in ("gemm_prologue_fusion", "layer_norm_folding", "attention_out_proj_fusion", "regional_synchronization")):
        assert "stage-fusion decisions taken from the seed specification" in log
    again.set_constants(consts)
    again.load(gpu_device)
    _check(again.run(inputs, fx.outputs)[0], want)


def test_launch_contexts_can_be_named(gpu_device, encoder, tmp_path, monkeypatch):
    # MONONN_TUNER_LAUNCH_CONTEXTS replaces the built-in list of (workgroups per CU) x (threads per workgroup)
    from mononn_amd import MonoNNError
    fx, consts, inputs, want = encoder
    monkeypatch.setenv("MONONN_TUNER_LAUNCH_CONTEXTS", "1x512")
    out = str(tmp_path / "ctx")
    tuned = MonoNNModuleTuner.tune(fx.hlo_text, gpu_device, out, budget=2)
    assert tuned.launch_dims()["block"] == 512
    files = os.listdir(os.path.join(out, "cluster_0"))
    assert any(f.endswith("__512_1_1.json") for f in files) and not any(f.endswith("__256_1_1.json") for f in files)
    tuned.set_constants(consts)
    tuned.load(gpu_device)
    _check(tuned.run(inputs, fx.outputs)[0], want)
    monkeypatch.setenv("MONONN_TUNER_LAUNCH_CONTEXTS", "two by four")
    with pytest.raises(MonoNNError) as ei:
        MonoNNModuleTuner.tune(fx.hlo_text, gpu_device, None, budget=2)
    assert "MONONN_TUNER_LAUNCH_CONTEXTS" in str(ei.value)


def test_attention_row_blocks_are_searched_on_many_rows(gpu_device, tmp_path, monkeypatch):
    # with many query rows per head the tuner also tries several row blocks per wave on one set of keys and values
    monkeypatch.setenv("MONONN_TUNER_LAUNCH_CONTEXTS", "1x256")
    monkeypatch.setenv("MONONN_TUNER_NO_SPLIT_K", "1")
    fx = models.bert_encoder(L=1, B=8, S=256, H=256, NH=4, F=512, vocab=300, max_pos=256, mask_kind="length_mask")
    consts, inputs = fx.make_constants(33, "random"), fx.make_inputs(33)
    out = str(tmp_path / "rows")
    tuned = MonoNNModuleTuner.tune(fx.hlo_text, gpu_device, out, budget=2)
    log = open(os.path.join(out, "cluster_0", "tuning_log.log")).read()
    line = next(l for l in log.splitlines() if "attention x1" in l)
    assert "_rows" in line, line                       # candidates like key_waves1_rows128 were timed
    tuned.set_constants(consts)
    tuned.load(gpu_device)
    _check(tuned.run(inputs, fx.outputs)[0], hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0])


def test_tuning_with_layer_norm_folding_and_the_seed_s_deep_splits(gpu_device, encoder, tmp_path, monkeypatch):
    # MONONN_TUNER_LAYER_NORM_FOLDING tunes the folded form; with a seed, MONONN_TUNER_KEEP_SEED_SPLIT_K keeps its k
    # splits of at least that factor from the start, and the LayerNorm behind such a GEMM stays a stage
    fx, consts, inputs, want = encoder
    monkeypatch.setenv("MONONN_TUNER_LAUNCH_CONTEXTS", "1x256")
    monkeypatch.setenv("MONONN_TUNER_LAYER_NORM_FOLDING", "1")
    folded_dir = str(tmp_path / "folded")
    folded = MonoNNModuleTuner.tune(fx.hlo_text, gpu_device, folded_dir, budget=2)
    spec = json.loads(folded.get_tuning_spec())
    assert spec["mononn_hip"]["layer_norm_folding"] is True and spec["mononn_hip"]["gemm_prologue_fusion"] is True
    assert "ln_stats[" in folded.get_source("main.hip")
    folded.set_constants(consts)
    folded.load(gpu_device)
    _check(folded.run(inputs, fx.outputs)[0], want)
    # a seed with FFN2 split by 4: kept from the start, so only the LayerNorm in front of FFN1 is folded
    seed = json.loads(MonoNNModule.compile(fx.hlo_text, build=False).get_tuning_spec())
    import re
    gemms = [n.replace(".", "_").replace("-", "_") for n in re.findall(r"%(cublas-gemm\.\d+) =", fx.hlo_text)]
    template = next(v for k, v in seed["gemm_spec_list"].items() if k.startswith("cublas_gemm_"))
    seed["gemm_spec_list"] = {k: v for k, v in seed["gemm_spec_list"].items() if not k.startswith("cublas_gemm_")}
    seed["cluster_reduce_spec"], seed["cluster_elewise_spec"] = {}, {}
    for layer in range(2):
        e = json.loads(json.dumps(template))
        e["cutlass_config"]["split_k"] = 4
        seed["gemm_spec_list"][gemms[layer * 6 + 5]] = e
    seed_dir = tmp_path / "seed" / "cluster_0"
    seed_dir.mkdir(parents=True)
    filled = MonoNNModule.compile(fx.hlo_text, json.dumps(seed), build=False).get_tuning_spec()
    (seed_dir / "best_tuning_spec.json").write_text(filled)
    monkeypatch.setenv("MONONN_TUNER_SEED_SPEC_DIR", str(tmp_path / "seed"))
    monkeypatch.setenv("MONONN_TUNER_KEEP_SEED_SPLIT_K", "4")
    monkeypatch.setenv("MONONN_TUNER_NO_SPLIT_K", "1")
    mixed_dir = str(tmp_path / "mixed")
    mixed = MonoNNModuleTuner.tune(fx.hlo_text, gpu_device, mixed_dir, budget=2)
    log = open(os.path.join(mixed_dir, "cluster_0", "tuning_log.log")).read()
    assert "2 k splits of the seed specification kept from the start" in log
    mspec = json.loads(mixed.get_tuning_spec())
    assert sum(1 for v in mspec["gemm_spec_list"].values() if v["cutlass_config"]["split_k"] == 4) == 2
    assert folded.launch_dims()["barriers"] < mixed.launch_dims()["barriers"] < MonoNNModule.compile(fx.hlo_text, build=False).launch_dims()["barriers"] + 1
    mixed.set_constants(consts)
    mixed.load(gpu_device)
    _check(mixed.run(inputs, fx.outputs)[0], want)
