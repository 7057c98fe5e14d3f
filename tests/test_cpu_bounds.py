"""Every generated kernel keeps its accesses inside its buffers: the generated translation units (with the device
prelude they ship with) run on the CPU, one thread at a time, every buffer against guard pages (tests/cpu_bounds.py).
Covers what a GPU test could only report as a memory fault: MFMA tiles on ragged shapes, fragment-order operands,
weights requested ahead of the barrier, fused attention, split-K, the launch variants and the tuned BERT-base kernel."""
import json

import numpy as np
import pytest

from cpu_bounds import check_module
from mononn_amd import MonoNNModule
from mononn_amd.hlo import models
import test_gpu_parity as parity

GEMM_CASES = [m for m in parity.test_gemm_cases.pytestmark if m.name == "parametrize"][0].args[1]


def test_the_check_itself_reports_an_access_past_a_buffer():
    mb, *_ = parity.gemm_module(M=100, N=52, K=96, rhs_c=1)
    ok, _ = check_module(mb.text())
    assert ok
    for which in ("live-out 0", "parameter 0", "parameter 1"):      # the same kernel, one buffer declared 32 bytes short
        ok, msg = check_module(mb.text(), shrink=(which, 32))
        assert not ok and "OUT OF BOUNDS: " + which in msg, msg
    ok, msg = check_module(models.bert_layer().hlo_text, shrink=("temp arena", 64))
    assert not ok and "temp arena" in msg
    # the constants of the module (arrays of the code object) and the workgroup's LDS are guarded like the arguments
    import re
    from mononn_amd import MonoNNModule
    layer = models.bert_layer().hlo_text
    m = MonoNNModule.compile(layer, build=False)
    weights = [(n, int(b)) for n, b in re.findall(r"unsigned char (buffer_for_\w+)\[(\d+)\];", m.get_source("main.hip")) if int(b) >= 4096]
    assert weights
    for name, _ in weights[:2]:
        ok, msg = check_module(layer, shrink=(name, 16))
        assert not ok and "OUT OF BOUNDS: " + name in msg, msg
    ok, msg = check_module(layer, shrink=("LDS", m.launch_dims()["smem"] // 2))
    assert not ok and "OUT OF BOUNDS: LDS" in msg, msg


@pytest.mark.parametrize("case", GEMM_CASES)
def test_gemm_layout_cases(case):
    ok, msg = check_module(parity.gemm_module(**case)[0].text())
    assert ok, msg


def test_random_gemm_shapes_layouts_and_tiles():
    from random_graphs import random_gemm_cases
    for case, text, spec in random_gemm_cases(5, 25):
        ok, msg = check_module(text, spec)
        assert ok, f"{case}: {msg}"


def test_fused_attention_with_key_counts_off_the_mfma_step():
    for kw in (dict(L=1, B=2, image=96, patch=16, H=128, NH=2, F=256), dict(L=1, B=1, image=224, patch=16, H=128, NH=2, F=256)):
        fx = models.vit(**kw)
        assert "colv[" in MonoNNModule.compile(fx.hlo_text, build=False).get_source("main.hip")
        ok, msg = check_module(fx.hlo_text, opt="-O1")
        assert ok, f"{kw}: {msg}"
    fx = models.bert_encoder(L=1, B=2, S=100, H=128, NH=2, F=256, vocab=97, max_pos=128, mask_kind="length_mask")
    assert "colv[" in MonoNNModule.compile(fx.hlo_text, build=False).get_source("main.hip")
    ok, msg = check_module(fx.hlo_text, opt="-O1")
    assert ok, msg


def test_random_gemms_on_lds_staged_tiles():
    from random_graphs import random_lds_gemm_cases
    for case, text, spec in random_lds_gemm_cases(6, 12):
        assert "gemm_tile_lds<" in MonoNNModule.compile(text, spec, build=False).get_source("main.hip"), case
        ok, msg = check_module(text, spec, opt="-O1")
        assert ok, f"{case}: {msg}"


def test_encoder_variants():
    fx = models.bert_encoder(L=2, B=1, S=64, H=256, NH=4, F=512, vocab=300, max_pos=64)
    variants = {
        "default": None,
        "8 workgroups": parity._spec_with(fx.hlo_text, grid=8),
        "2 workgroups per compute unit": parity._spec_with(fx.hlo_text, grid=512),
        "LayerNorm inside the GEMM": parity._spec_with(fx.hlo_text, hip={"gemm_prologue_fusion": True}),
        "LayerNorm folded into the GEMM": parity._spec_with(fx.hlo_text, hip={"gemm_prologue_fusion": True, "layer_norm_folding": True}),
        "output projection inside the attention": parity._spec_with(fx.hlo_text, hip={"attention_out_proj_fusion": True}),
        "no attention fusion": parity._spec_with(fx.hlo_text, hip={"fuse_attention": False}),
        "no epilogue fusion": parity._spec_with(fx.hlo_text, hip={"gemm_epilogue_fusion": False}),
        "plain layouts": parity._spec_with(fx.hlo_text, hip={"transpose_constant_b": False, "assign_operand_layouts": False}),
        "weights requested inside the tile": parity._spec_with(fx.hlo_text, hip={"operand_preload": False}),
        "row-major left operands": parity._spec_with(fx.hlo_text, hip={"pack_left_operands": False}),
    }
    for name, spec in variants.items():
        ok, msg = check_module(fx.hlo_text, spec)
        assert ok, f"{name}: {msg}"


def test_attention_with_several_row_blocks_per_wave():
    import json
    cases = [(models.bert_encoder(L=1, B=2, S=128, H=128, NH=2, F=256, vocab=300, max_pos=128, mask_kind="length_mask"), 3, 4),
             (models.gpt2(L=1, B=2, S=64, H=128, NH=2, F=256, vocab=300, max_pos=64), 4, 2),
             (models.vit(L=1, B=2, image=96, patch=16, H=128, NH=2, F=256), 2, 1)]
    for fx, row_blocks, key_waves in cases:
        spec = json.loads(MonoNNModule.compile(fx.hlo_text, build=False).get_tuning_spec())
        block = spec["cuda_context"]["cuda_runtime_context"]["block_dim"]["x"]
        for name, entry in spec["gemm_spec_list"].items():
            if name.count("batch_gemm") >= 2:
                c = entry["cutlass_config"]
                c["wave_arrangement"] = {"m": block // 64 // key_waves, "n": 1, "k": key_waves}
                c["threadblockshape"]["m"] = 16 * c["wave_arrangement"]["m"] * row_blocks
        text = json.dumps(spec)
        assert "for (int rb = 0; rb < %d; ++rb)" % row_blocks in MonoNNModule.compile(fx.hlo_text, text, build=False).get_source("main.hip")
        ok, msg = check_module(fx.hlo_text, text)
        assert ok, f"{row_blocks} row blocks, {key_waves} key waves: {msg}"


ODD_ENCODERS = [dict(B=1, S=17, H=64, NH=1, F=100), dict(B=3, S=50, H=96, NH=2, F=100), dict(B=1, S=100, H=120, NH=3, F=256),
                dict(B=3, S=64, H=128, NH=4, F=100), dict(B=1, S=50, H=120, NH=3, F=100), dict(B=3, S=17, H=96, NH=2, F=256)]


@pytest.mark.parametrize("shape", ODD_ENCODERS)
def test_encoders_with_sizes_off_the_mfma_steps(shape):
    # sequence lengths, hidden sizes and head sizes that are not multiples of 16 / 32: ragged tiles, unfused attention
    fx = models.bert_encoder(L=1, vocab=97, max_pos=128, **shape)
    ok, msg = check_module(fx.hlo_text)
    assert ok, msg


def test_other_model_families_and_the_tuned_bert_base_kernel():
    import os
    from mononn_amd import binding
    for name, fx in [("GPT-2 style decoder", models.gpt2(L=2, B=2, S=64, H=256, NH=4, F=512, vocab=1000, max_pos=128)),
                     ("ViT, 17 tokens", models.vit(L=2, B=2, image=64, patch=16, H=256, NH=4, F=512)),
                     ("ViT-B/16 layer, 197 tokens", models.vit(L=1, B=1))]:
        ok, msg = check_module(fx.hlo_text)
        assert ok, f"{name}: {msg}"
    spec = open(os.path.join(os.path.dirname(binding.__file__), "specs", "bert_base_b1_s128", "cluster_0", "best_tuning_spec.json")).read()
    ok, msg = check_module(models.bert_base().hlo_text, spec)
    assert ok, msg


def test_whatever_specification_is_accepted_stays_inside_the_buffers():
    # numbers of a valid specification replaced at random (tiles, wave arrangements, knobs, launch shape): the host
    # compiler either rejects the result or generates a kernel that passes the bounds check
    import random
    import re
    from mononn_amd import MonoNNError
    fx = models.bert_encoder(L=1, B=1, S=32, H=64, NH=2, F=128, vocab=50, max_pos=64)
    spec = json.dumps(json.loads(MonoNNModule.compile(fx.hlo_text, build=False).get_tuning_spec()), indent=1)
    numbers = list(re.finditer(r"(?<=: )-?\d+(?=,|\n)", spec))
    rnd = random.Random(3)
    accepted = 0
    for _ in range(60):
        t = spec
        for m in sorted(rnd.sample(numbers, rnd.randint(1, 3)), key=lambda m: -m.start()):
            t = t[:m.start()] + rnd.choice(["0", "1", "2", "3", "4", "5", "7", "8", "16", "17", "32", "48", "64", "96", "100", "128", "256", "512", "1024"]) + t[m.end():]
        try:
            MonoNNModule.compile(fx.hlo_text, t, build=False).close()
        except MonoNNError:
            continue
        accepted += 1
        ok, msg = check_module(fx.hlo_text, t)
        assert ok, msg + "\n" + t
    assert accepted >= 20


def test_bf16_encoder_and_gemms():
    import json
    fx = models.bert_encoder(L=1, B=2, S=64, H=128, NH=2, F=256, vocab=300, max_pos=64, ftype="bf16", mask_kind="length_mask")
    ok, msg = check_module(fx.hlo_text)
    assert ok, msg
    spec = json.loads(MonoNNModule.compile(fx.hlo_text, build=False).get_tuning_spec())
    for name, e in spec["gemm_spec_list"].items():
        c = e["cutlass_config"]
        if name.startswith("cublas_gemm_") and c["split_k"] == 1:
            c["threadblockshape"].update(m=64, n=64, k=32)
            c["wave_arrangement"] = {"m": 2, "n": 2, "k": 1}
            c["stages"] = 2
    ok, msg = check_module(fx.hlo_text, json.dumps(spec), opt="-O1")
    assert ok, "LDS-staged tiles: " + msg


def test_folded_layer_norm_on_lds_staged_tiles_that_store_their_rows():
    """Post-LN encoder, LayerNorms folded into LDS-staged tiles: the GEMMs that owe the normalised rows to a later stage
    re-read their left operand (stored in fragment order by the stage before) and store a share of the rows per column tile."""
    import json
    from mononn_amd import MonoNNModule
    fx = models.bert_encoder(L=2, B=4, S=128, H=256, NH=4, F=1024, vocab=300, max_pos=128)
    spec = json.loads(MonoNNModule.compile(fx.hlo_text, build=False).get_tuning_spec())
    spec["mononn_hip"].update(gemm_prologue_fusion=True, layer_norm_folding=True)
    spec["gemm_spec_list"], spec["cluster_reduce_spec"], spec["cluster_elewise_spec"] = {}, {}, {}
    spec = json.loads(MonoNNModule.compile(fx.hlo_text, json.dumps(spec), build=False).get_tuning_spec())
    for name, entry in spec["gemm_spec_list"].items():
        if name.startswith("fusion_"):
            c = entry["cutlass_config"]
            c["threadblockshape"], c["warpshape"] = dict(m=128, n=128, k=64), dict(m=64, n=64, k=256)
            c["wave_arrangement"], c["stages"] = dict(m=2, n=2, k=1), 2
    src = MonoNNModule.compile(fx.hlo_text, json.dumps(spec), build=False).get_source("main.hip")
    assert src.count("_rows {") == 2 and "_rows>(" in src
    ok, msg = check_module(fx.hlo_text, json.dumps(spec))
    assert ok, msg

