"""CPU tests of the host compiler and the C ABI: parsing, stage scheduling, specification handling,
dump tree, error codes.  No kernel is launched here; hipRTC cross-compiles for gfx950 without a GPU."""
import ctypes
import json
import os
import re
import subprocess

import pytest

from mononn_amd import MonoNNError, MonoNNModule, binding
from mononn_amd.hlo import models
from mononn_amd.hlo.builder import HloModuleBuilder

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def layer():
    return models.bert_layer(B=1, S=32, H=128, NH=4, F=256)


def test_abi_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "mononn_hip.h")).read()
    declared = set(re.findall(r"\b(mononn_[a-z_]+)\s*\(", header))
    assert declared, "no declarations found"
    lib = ctypes.CDLL(binding.LIB_PATH)
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} is declared in include/mononn_hip.h but not exported"
    assert declared == set(binding.EXPORTED_SYMBOLS)


def test_kernel_name_buffers_and_argument_order(layer):
    m = MonoNNModule.compile(layer.hlo_text, build=False)
    assert m.kernel_name == "mononn_cluster_0"          # README.md:186 naming convention
    info = m.buffer_info()
    assert info["parameters"] == [1 * 32 * 128 * 2, 32 * 4]
    assert info["liveouts"] == [32 * 128 * 2]
    src = m.get_source("main.hip")
    sig = re.search(r'extern "C" .*void mononn_cluster_0\(([^)]*)\)', src).group(1)
    assert [a.strip() for a in sig.split(",")] == ["void* arg0", "void* arg1", "void* liveout_buffer_0", "void* temp_buffer"]
    assert "buffer_for_constant_" in src                # constants are module globals filled by the host
    names = [c["name"] for c in m.constants()]
    assert len(names) == 16 and all(c["needs_payload"] for c in m.constants())


def test_bert_base_parameters_match_reference_log():
    m = MonoNNModule.compile(models.bert_base().hlo_text, build=False)
    info = m.buffer_info()
    assert info["parameters"] == [512, 512, 512]        # README.md:192-194
    assert info["liveouts"] == [196608]


def test_stage_structure_and_function_sharing(layer):
    m = MonoNNModule.compile(layer.hlo_text, build=False)
    s = m.summary()
    stages = [int(x) for x in re.findall(r"^\s+stage (\d+)", s, re.M)]
    assert stages == sorted(stages)
    # QKV | attention | out-proj(+residual) | LayerNorm | FFN1(+GELU) | FFN2(+residual) | LayerNorm
    assert max(stages) == 7 and m.launch_dims()["barriers"] == 6
    # Q, K and V projections share a stage; scores -> soft-max -> context became one attention node;
    # the LayerNorm chains were merged into row programs
    assert stages.count(1) == 3
    assert len(re.findall(r"\battn\b", s)) == 1 and len(re.findall(r"rowred", s)) == 2
    two = MonoNNModule.compile(models.bert_encoder(L=2, B=1, S=32, H=128, NH=4, F=256, vocab=100, max_pos=64).hlo_text, build=False)
    one = MonoNNModule.compile(models.bert_encoder(L=1, B=1, S=32, H=128, NH=4, F=256, vocab=100, max_pos=64).hlo_text, build=False)
    n2 = len(re.findall(r"__forceinline__ void node_fn_", two.get_source()))
    n1 = len(re.findall(r"__forceinline__ void node_fn_", one.get_source()))
    assert n1 >= 5
    assert n2 <= n1 + 1, "a repeated layer must reuse the device functions of the first one"


def test_disabled_pass_env(layer, monkeypatch):
    base = MonoNNModule.compile(layer.hlo_text, build=False).launch_dims()["barriers"]
    monkeypatch.setenv("MONONN_OPTIMIZATION_DISABLED_PASS", "AttentionFusionPass")
    no_attn = MonoNNModule.compile(layer.hlo_text, build=False).launch_dims()["barriers"]
    assert no_attn == base + 2
    monkeypatch.setenv("MONONN_OPTIMIZATION_DISABLED_PASS", "AttentionFusionPass,MergeDependentPass,GemmEpilogueFusionPass")
    unfused = MonoNNModule.compile(layer.hlo_text, build=False).launch_dims()["barriers"]
    assert unfused > no_attn


def test_fusion_decisions_in_spec(layer):
    spec = json.loads(MonoNNModule.compile(layer.hlo_text, build=False).get_tuning_spec())
    base = MonoNNModule.compile(layer.hlo_text, json.dumps(spec), build=False).launch_dims()["barriers"]
    spec["mononn_hip"]["gemm_prologue_fusion"] = True      # LayerNorm inside the FFN1 GEMM
    spec["gemm_spec_list"] = {}
    spec["cluster_reduce_spec"] = {}
    fused = MonoNNModule.compile(layer.hlo_text, json.dumps(spec), build=False)
    assert fused.launch_dims()["barriers"] == base - 1
    assert "+row-prologue(stores)" in fused.summary()


def test_spec_round_trip_and_reload(layer, tmp_path):
    m = MonoNNModule.compile(layer.hlo_text, build=False)
    spec = json.loads(m.get_tuning_spec())
    rt = spec["cuda_context"]["cuda_runtime_context"]
    assert rt["grid_dim"] == {"x": 256, "y": 1, "z": 1} and rt["block_dim"]["x"] == 256 and "smem_size" in rt
    assert spec["cuda_context"]["cuda_device_context"]["warp_size"] == 64
    for key in ("cluster_elewise_spec", "cluster_reduce_spec", "gemm_spec_list", "conv_spec_list", "codegen_allow_list",
                "codegen_reject_list", "feeds", "fetches", "input_data_files", "hlo_module_proto_file"):
        assert key in spec
    g = next(v for k, v in spec["gemm_spec_list"].items() if k.startswith("cublas_gemm_"))
    assert set(g["cutlass_config"]) >= {"threadblockshape", "warpshape", "instructionshape", "operatorclass", "archtag", "stages"}
    assert "alpha_real" in g["gemm_backend_config"]
    m2 = MonoNNModule.compile(layer.hlo_text, json.dumps(spec), build=False)
    assert json.loads(m2.get_tuning_spec()) == spec
    assert m2.get_source() == m.get_source()
    # dump tree (README.md:155-177, context string with a double underscore: mononn_module_tuner.cc:374-383)
    mb = MonoNNModule.compile(layer.hlo_text, json.dumps(spec), build=True)
    mb.dump(str(tmp_path))
    d = tmp_path / "cluster_0"
    for f in ("256_1_1__256_1_1.json", "256_1_1__256_1_1.hsaco", "256_1_1__256_1_1_src/main.hip", "256_1_1__256_1_1_src/headers.h",
              "best_tuning_spec.json", "best_tuning_spec.hsaco"):
        assert (d / f).exists(), f
    m3 = MonoNNModule.from_spec_dir(layer.hlo_text, str(tmp_path))
    assert m3.get_code_object() == mb.get_code_object()      # cached code object was picked up
    # ... because it was built from the sources this load generates: the key beside it says so.  A cache whose key
    # does not match (another specification, HLO, prelude or compiler options) is left alone and the kernel rebuilt
    assert (d / "best_tuning_spec.hsaco.key").read_text().startswith("fnv1a64:")
    good = (d / "best_tuning_spec.hsaco").read_bytes()
    (d / "best_tuning_spec.hsaco").write_bytes(b"stale code object")
    assert bytes(MonoNNModule.from_spec_dir(layer.hlo_text, str(tmp_path)).get_code_object()) == b"stale code object"    # the key still matches
    edited = json.loads((d / "best_tuning_spec.json").read_text())
    edited["mononn_hip"]["barrier_timeout_ms"] = 2000          # changes the generated preamble, hence the key
    (d / "best_tuning_spec.json").write_text(json.dumps(edited))
    rebuilt = bytes(MonoNNModule.from_spec_dir(layer.hlo_text, str(tmp_path)).get_code_object())
    assert rebuilt != b"stale code object" and rebuilt[:4] == b"\x7fELF"
    (d / "best_tuning_spec.json").write_text(json.dumps(spec if False else json.loads(mb.get_tuning_spec())))
    (d / "best_tuning_spec.hsaco").write_bytes(good)
    os.environ["TF_MONONN_EXISTING_TUNING_SPEC_DIR"] = str(tmp_path)
    try:
        m4 = MonoNNModule.from_spec_dir(layer.hlo_text, None)
        assert json.loads(m4.get_tuning_spec()) == json.loads(mb.get_tuning_spec())
    finally:
        del os.environ["TF_MONONN_EXISTING_TUNING_SPEC_DIR"]


def test_spec_changes_generated_code(layer):
    m = MonoNNModule.compile(layer.hlo_text, build=False)
    spec = json.loads(m.get_tuning_spec())
    name = next(n for n in spec["gemm_spec_list"] if n.startswith("cublas_gemm_") and "fusion" in n)
    cc = spec["gemm_spec_list"][name]["cutlass_config"]
    cc["threadblockshape"].update(m=16, n=64)
    cc["wave_arrangement"].update(m=1, n=2, k=2)
    src = MonoNNModule.compile(layer.hlo_text, json.dumps(spec), build=False).get_source()
    assert "gemm_tile<16, 64, 1, 2, 2," in src


@pytest.mark.parametrize("mutate,status", [
    (lambda s: s["gemm_spec_list"].update({"no_such_node": next(iter(s["gemm_spec_list"].values()))}), "SPEC_ERROR"),
    (lambda s: s.update({"unknown_field": 1}), "SPEC_ERROR"),
    (lambda s: s["cuda_context"]["cuda_runtime_context"]["block_dim"].update(x=100), "SPEC_ERROR"),
    (lambda s: s["cuda_context"]["cuda_runtime_context"]["grid_dim"].update(x=5000), "SPEC_ERROR"),
    (lambda s: s["codegen_allow_list"].append("ghost"), "SPEC_ERROR"),
    (lambda s: s["mononn_hip"].update(barrier="semaphore"), "SPEC_ERROR"),
    (lambda s: next(v for k, v in s["gemm_spec_list"].items() if k.startswith("cublas_gemm_"))["cutlass_config"]["wave_arrangement"].update(m=3), "SPEC_ERROR"),
    (lambda s: next(v for k, v in s["gemm_spec_list"].items() if k.startswith("cublas_batch_gemm_"))["cutlass_config"]["wave_arrangement"].update(k=3), "SPEC_ERROR"),
    # query rows per attention unit: whole rounds of 16 rows per wave along m
    (lambda s: next(v for k, v in s["gemm_spec_list"].items() if k.startswith("cublas_batch_gemm_"))["cutlass_config"]["threadblockshape"].update(m=24), "SPEC_ERROR"),
])
def test_bad_specs_are_rejected(layer, mutate, status):
    spec = json.loads(MonoNNModule.compile(layer.hlo_text, build=False).get_tuning_spec())
    mutate(spec)
    with pytest.raises(MonoNNError) as e:
        MonoNNModule.compile(layer.hlo_text, json.dumps(spec), build=False)
    assert e.value.status == status


HEAD = "HloModule cluster_9__t.1\n\n"


@pytest.mark.parametrize("text,status", [
    ("not hlo at all", "PARSE_ERROR"),
    (HEAD + "ENTRY %main {\n  %p = f32[4]{0} parameter(0)\n  ROOT %r = f32[4]{0} add(f32[4]{0} %p, f32[4]{0} %q)\n}\n", "PARSE_ERROR"),
    (HEAD + "ENTRY %main {\n  %p = f32[4]{0} parameter(0)\n  ROOT %r = f32[4]{0} cosine(f32[4]{0} %p)\n}\n", "UNSUPPORTED"),
    (HEAD + "ENTRY %main {\n  %p = f32[<=4]{0} parameter(0)\n  ROOT %r = f32[<=4]{0} negate(%p)\n}\n", "UNSUPPORTED"),
    (HEAD + "ENTRY %main {\n  %p = f32[4,4]{1,0:T(2,2)} parameter(0)\n  ROOT %r = f32[4,4]{1,0} negate(%p)\n}\n", "UNSUPPORTED"),
    (HEAD + "ENTRY %main {\n  %p = f32[4,4]{0,1:T(2,128)} parameter(0)\n  ROOT %r = f32[4,4]{0,1} negate(%p)\n}\n", "UNSUPPORTED"),
    (HEAD + "ENTRY %main {\n  %p = f8e4m3fn[4]{0} parameter(0)\n  ROOT %r = f8e4m3fn[4]{0} negate(%p)\n}\n", "UNSUPPORTED"),
    (HEAD + "ENTRY %main {\n  %p = f32[1,4,4,1]{3,2,1,0} parameter(0)\n  %w = f32[1,1,1,1]{3,2,1,0} parameter(1)\n"
            "  ROOT %r = f32[1,4,4,1]{3,2,1,0} convolution(%p, %w), window={size=1x1}, dim_labels=b01f_01io->b01f\n}\n", "UNSUPPORTED"),
    (HEAD + "ENTRY %main {\n  %p = f16[4,4]{1,0} parameter(0)\n  ROOT %r = f16[4,4]{1,0} custom-call(%p), custom_call_target=\"__my$thing\"\n}\n",
     "UNSUPPORTED"),
    (HEAD + "ENTRY %main {\n  %p = f32[4]{0} parameter(0)\n  ROOT %r = f32[4]{0} negate(%p)\n", "PARSE_ERROR"),
])
def test_bad_hlo_is_rejected_with_a_status(text, status):
    with pytest.raises(MonoNNError) as e:
        MonoNNModule.compile(text, build=False)
    assert e.value.status == status, str(e.value)


def test_gemm_stride_cross_check():
    # XLA's lhs_stride must agree with the shapes (the reference cross-checks it, gemm_impl.cc:380-393)
    mb = HloModuleBuilder("cluster_4__t.1")
    e = mb.entry
    a = e.parameter("f16", (2, 8, 32), "a")
    b = e.parameter("f16", (2, 32, 8), "b")
    e.set_tuple_root([e.gemm(a, b, 2, 1, batch_dims=(0,))])
    good = mb.text()
    MonoNNModule.compile(good, build=False)
    bad = good.replace('\\"lhs_stride\\":\\"256\\"', '\\"lhs_stride\\":\\"999\\"')
    assert bad != good
    with pytest.raises(MonoNNError) as ex:
        MonoNNModule.compile(bad, build=False)
    assert ex.value.status == "INVALID_ARGUMENT"


def test_errors_before_load(layer):
    m = MonoNNModule.compile(layer.hlo_text, build=False)
    with pytest.raises(MonoNNError) as e:
        m.get_code_object()
    assert e.value.status == "NOT_FOUND"
    with pytest.raises(MonoNNError) as e:
        m.set_constant("no_such_constant", __import__("numpy").zeros(4, "float16"))
    assert e.value.status == "NOT_FOUND"
    c = m.constants()[0]
    with pytest.raises(MonoNNError) as e:
        m.set_constant(c["name"], __import__("numpy").zeros(3, "float16"))
    assert e.value.status == "INVALID_ARGUMENT"
    with pytest.raises(MonoNNError) as e:
        m.launch_raw([0, 0, 0, 0])
    assert e.value.status == "INVALID_ARGUMENT"      # not loaded


def test_compile_error_is_reported_not_fatal(layer):
    # a kernel name that is not an identifier makes hipRTC fail; the process must survive with the log
    with pytest.raises(MonoNNError) as e:
        MonoNNModule.compile(layer.hlo_text, None, "not an identifier", build=True)
    assert e.value.status == "COMPILE_ERROR" and "error" in str(e.value)
    # what failed is kept for inspection (mononn_module_tuner.cc:261-285 dumps to /tmp/mononn_codegen/<uuid>)
    kept = re.search(r"kept in (/tmp/mononn_codegen/\S+)\]", str(e.value)).group(1)
    assert sorted(os.listdir(kept)) == ["graph_spec.json", "headers.h", "host_main.cpp", "main.hip"]
    assert "not an identifier" in open(os.path.join(kept, "main.hip")).read()


def test_cli_compiles_and_dumps(layer, tmp_path):
    hlo = tmp_path / "m.hlo"
    hlo.write_text(layer.hlo_text)
    exe = os.path.join(ROOT, "mononn_amd", "bin", "mononn_hipc")
    out = subprocess.run([exe, str(hlo), "--dump", str(tmp_path / "dump")], capture_output=True, text=True, check=True).stdout
    assert "Temporary buffer size:" in out and "Parameter 0:" in out
    assert (tmp_path / "dump" / "cluster_0" / "best_tuning_spec.json").exists()
    out2 = subprocess.run([exe, str(hlo), "--spec-dir", str(tmp_path / "dump")], capture_output=True, text=True, check=True).stdout
    assert "kernel mononn_cluster_0" in out2


def test_write_once_temp_addresses(layer):
    # the fence-free barrier relies on every temp address being written once per launch
    coherent = MonoNNModule.compile(layer.hlo_text, build=False)
    spec = json.loads(coherent.get_tuning_spec())
    assert spec["mononn_hip"]["barrier"] == "flags_coherent"
    src = coherent.get_source()
    sigs = {int(i): [p.strip() for p in sig.split(",") if not re.search(r"\b(smem|pre_b)$", p.strip())]
            for i, sig in re.findall(r"void node_fn_(\d+)\(int unit, ([^)]*)\)", src)}
    written = []
    for fn, rest in re.findall(r"case \d+: fn = (\d+); units = \d+; first = \d+; total = \d+; new_stage = \w+;(.*?) break;", src):
        ptrs = dict(re.findall(r"p(\d+) = ([^;]*);", rest))
        for i, prm in enumerate(sigs[int(fn)]):
            if not prm.startswith("const") and "temp_buffer" in ptrs[str(i)]:
                written.append(ptrs[str(i)])
    assert written and len(written) == len(set(written)), "a temp slot is written by two nodes"
    assert "MONONN_COHERENT_STORES 1" in coherent.get_source()
    spec["mononn_hip"]["barrier"] = "flags"
    fenced = MonoNNModule.compile(layer.hlo_text, json.dumps(spec), build=False)
    assert fenced.buffer_info()["temp"] < coherent.buffer_info()["temp"]     # slots are re-used again


def _conv_text(xd=(2, 64, 64, 8), fd=(64, 16, 16, 8), stride=(16, 16), pad=(0, 0)):
    mb = HloModuleBuilder("cluster_9__conv.1")
    e = mb.entry
    x = e.parameter("f16", xd, "x")
    f = e.parameter("f16", fd, "f")
    e.set_tuple_root([e.conv_forward(x, f, stride=stride, pad=pad)])
    return mb.text()


def test_convolution_call_is_lowered_as_implicit_gemm():
    # conv_impl.cc:51: forward convolution = GEMM over (output pixels) x (output channels) x (R*S*C)
    m = MonoNNModule.compile(_conv_text(), build=False)
    assert "f16_b1_m32_n64_k2048_ak_bk_conv16x16s16x16p0x0" in m.summary()
    src = m.get_source("main.hip")
    assert "_amap" in src and "gemm_tile<" in src          # patch convolution: MFMA tiles with gathered rows
    # padding breaks the fragment loads: per-element fallback, still one stage
    m2 = MonoNNModule.compile(_conv_text((2, 9, 10, 4), (6, 3, 3, 4), (2, 1), (1, 1)), build=False)
    assert "conv_naive_element" in m2.get_source("main.hip")
    assert m2.buffer_info()["liveouts"] == [2 * 5 * 10 * 6 * 2]


def test_contraction_length_off_the_mfma_step_still_takes_mfma_tiles():
    # ViT's P.V product contracts over 197 keys: the tile zero-fills the last step instead of falling back to one
    # thread per element; V is stored transposed by the stage that writes it, so both operands are k-contiguous
    # (with the attention left as separate stages; fused, the product never is a GEMM stage of its own)
    fx = models.vit(L=1, B=1)
    spec = json.loads(MonoNNModule.compile(fx.hlo_text, build=False).get_tuning_spec())
    spec["mononn_hip"]["fuse_attention"] = False
    spec["gemm_spec_list"], spec["cluster_reduce_spec"], spec["cluster_elewise_spec"] = {}, {}, {}
    src = MonoNNModule.compile(fx.hlo_text, json.dumps(spec), build=False).get_source("main.hip")
    assert "gemm_naive_element" not in src
    assert re.search(r"gemm_tile<\d+, \d+, \d+, \d+, \d+, 197, false, 197,", src)


SHIPPED_SPECS = {"bert_base_b1_s128": models.bert_base, "vit_b16_b8": models.vit, "gpt2_b4_s512": models.gpt2,
                 "bert_large_b16_s384": models.bert_large}


def test_results_only_the_host_reads_are_stored_through_the_cache():
    # a value that a later stage reads crosses XCDs through write-through stores; the last LayerNorm's result is read
    # by the host alone and is written with plain stores (the L2 merges them; all of it is written out at kernel end)
    fx = models.bert_encoder(L=2, B=1, S=64, H=256, NH=4, F=512, vocab=300, max_pos=64)
    src = MonoNNModule.compile(fx.hlo_text, build=False).get_source("main.hip")
    fns = re.split(r"(?=__device__ __forceinline__ void node_fn_\d+\()", src)
    plain = [f for f in fns if "stN_plain<" in f or "st1_plain(" in f]
    assert len(plain) == 1 and "mononn_dev::stN<" not in plain[0] and "mononn_dev::st1(" not in plain[0].split("extern \"C\"")[0]
    assert sum("mononn_dev::stN<" in f or "mononn_dev::st1(" in f for f in fns) >= 5
    # a module output that a later stage also reads keeps the write-through stores
    mb = HloModuleBuilder("cluster_6__two_readers.1")
    e = mb.entry
    x = e.parameter("f16", (64, 128), "x")
    w = e.elided_constant("f16", (128, 128), "w/kernel")
    h = e.fusion("kLoop", [x], lambda f, p: f.tanh(p))
    y = e.gemm(h, w, 1, 0)
    e.set_tuple_root([h, y])
    src = MonoNNModule.compile(mb.text(), build=False).get_source("main.hip")
    first = [f for f in re.split(r"(?=__device__ __forceinline__ void node_fn_\d+\()", src) if "fast_tanh" in f][0]
    first = re.split(r"\n(?:typedef|struct) ", first)[0]          # the next function's epilogue struct follows in the text
    assert "_plain" not in first and ("mononn_dev::stN<" in first or "mononn_dev::st1(" in first)


def test_register_budget_follows_the_workgroups_per_compute_unit():
    # a persistent grid must be resident as a whole: with more than one workgroup per CU (or 512-thread workgroups)
    # two waves share a SIMD, the kernel is compiled for 256 registers per wave and the GEMM tile loads smaller chunks
    layer = models.bert_layer()
    base = json.loads(MonoNNModule.compile(layer.hlo_text, build=False).get_tuning_spec())
    assert "__launch_bounds__(256)" in MonoNNModule.compile(layer.hlo_text, build=False).get_source("main.hip")
    for grid, block, bounds in [(512, 256, "__launch_bounds__(256, 2)"), (256, 512, "__launch_bounds__(512, 2)"), (768, 256, "__launch_bounds__(256, 3)")]:
        spec = json.loads(json.dumps(base))
        spec["cuda_context"]["cuda_runtime_context"]["grid_dim"]["x"] = grid
        spec["cuda_context"]["cuda_runtime_context"]["block_dim"]["x"] = block
        spec["gemm_spec_list"] = {}
        spec["cluster_reduce_spec"] = {}
        spec["cluster_elewise_spec"] = {}
        src = MonoNNModule.compile(layer.hlo_text, json.dumps(spec), build=False).get_source("main.hip")
        assert bounds in src and "#define MONONN_WAVES_PER_SIMD " + bounds[-2] in src, (grid, block)


def test_shipped_specifications_load_against_their_models():
    # every tuned specification in the package names the nodes of the model fixture it was tuned for: loading it
    # through the spec-dir path must compile (a renamed node or a tile the generator rejects fails here)
    root = os.path.join(os.path.dirname(binding.__file__), "specs")
    found = sorted(os.listdir(root))
    assert "bert_base_b1_s128" in found and set(found) <= set(SHIPPED_SPECS)
    for name in found:
        fx = SHIPPED_SPECS[name]()
        m = MonoNNModule.from_spec_dir(fx.hlo_text, os.path.join(root, name))
        spec = json.loads(m.get_tuning_spec())
        shipped = json.load(open(os.path.join(root, name, "cluster_0", "best_tuning_spec.json")))
        assert spec["gemm_spec_list"] == shipped["gemm_spec_list"] and spec["mononn_hip"] == shipped["mononn_hip"]
        assert len(m.get_code_object()) > 0
        m.close()


def test_reduce_window_update_slice_and_variadic_reduce_are_lowered():
    # index maps of index_tracer.cc for reduce-window / dynamic-update-slice, tuple reducers of
    # reduction_functor_generator.cc:246-283: each is one stage of plain per-element code
    from op_cases import pool_module, update_slice_module, arg_reduce_module
    text, od = pool_module((2, 9, 10, 8), (1, 3, 3, 1), (1, 2, 2, 1), ((0, 0), (1, 1), (1, 1), (0, 0)), "max")
    m = MonoNNModule.compile(text, build=False)
    src = m.get_source("main.hip")
    assert od == [2, 5, 5, 8] and m.buffer_info()["liveouts"] == [2 * 5 * 5 * 8 * 2]
    assert re.search(r"for \(int w\d+ = 0; w\d+ < 3; \+\+w\d+\)", src) and "* 2 + w" in src and ">= 0 &&" in src
    # without padding there is no bounds test
    text, _ = pool_module((1, 8, 8, 4), (1, 2, 2, 1), (1, 2, 2, 1), ((0, 0),) * 4, "sum")
    assert ">= 0 &&" not in MonoNNModule.compile(text, build=False).get_source("main.hip")
    src = MonoNNModule.compile(update_slice_module((6, 10, 8), (2, 4, 8)), build=False).get_source("main.hip")
    assert "mononn_dev::clamp_index(" in src and ", 4);" in src and ", 6);" in src and "else" in src     # starts clamped to extent - update
    # a tuple-valued reduce over the last dimension is a row program (the lanes exchange whole tuples, the reducer is
    # inlined as a local lambda); over another dimension it is a serial loop of the thread that owns the element
    src = MonoNNModule.compile(arg_reduce_module(7, 50), build=False).get_source("main.hip")
    assert "int32_t* out1" in src and "mononn_dev::lane_xor(" in src and re.search(r"auto comb\d+ = \[\]\(_Float16& a0, int32_t& a1, const _Float16 b0, const int32_t b1\)", src)
    src = MonoNNModule.compile(arg_reduce_module(64, 2000), build=False).get_source("main.hip")
    assert "reinterpret_cast<int32_t*>(smem + 32)[w]" in src                         # long rows: one workgroup per row
    src = MonoNNModule.compile(arg_reduce_module(7, 50, axis=0), build=False).get_source("main.hip")
    assert "lane_xor" not in src and re.search(r"for \(int rk\d+ = 0; rk\d+ < 50;", src)
    # what the reference rejects is rejected here too: window dilation (ir_parser_fused.cc:1246-1250)
    bad = pool_module((1, 8, 8, 4), (1, 2, 2, 1), (1, 2, 2, 1), ((0, 0),) * 4)[0].replace("stride=1x2x2x1", "stride=1x2x2x1 rhs_dilate=1x2x2x1")
    with pytest.raises(MonoNNError) as ei:
        MonoNNModule.compile(bad, build=False)
    assert "dilation" in str(ei.value)


@pytest.mark.parametrize("edit,fragment", [
    (lambda t: t.replace("window={size=16x16 stride=16x16}", "window={size=16x16 stride=16x16 rhs_dilate=2x2}"), "dilated"),
    (lambda t: t.replace("window={size=16x16 stride=16x16}", "window={size=16x16 stride=16x16 pad=0_1x0_0}"), "symmetric"),
    (lambda t: t.replace("b01f_o01i->b01f", "bf01_oi01->bf01"), "dim_labels"),
    (lambda t: t.replace("dim_labels=", "feature_group_count=2, dim_labels="), "grouped"),
    (lambda t: t.replace("index=0", "index=1").replace("f16[2,4,4,64]{3,2,1,0} get-tuple-element", "u8[0]{0} get-tuple-element", 1), "scratch"),
])
def test_unsupported_convolutions_are_rejected(edit, fragment):
    # the reference aborts on the same constructs (ir_parser_fused.cc:749-798)
    text = edit(_conv_text())
    assert text != _conv_text()
    with pytest.raises(MonoNNError) as e:
        MonoNNModule.compile(text, build=False)
    assert e.value.status == "UNSUPPORTED", str(e.value)
    assert fragment in str(e.value)


def test_plain_dot_and_nested_backend_config_are_gemms():
    mb = HloModuleBuilder("cluster_5__dot.1")
    e = mb.entry
    a = e.parameter("f16", (128, 256), "a")
    w = e.elided_constant("f16", (256, 512), "w/kernel")
    e.set_tuple_root([e.dot(a, w, 1, 0)])
    m = MonoNNModule.compile(mb.text(), build=False)
    assert "gemm    dot_" in m.summary() and "f16_b1_m128_n512_k256_ak_bp" in m.summary()   # constant packed for the MFMA path
    # newer XLA prints the cuBLAS fields one level down, under "gemm_backend_config"
    mb2 = HloModuleBuilder("cluster_5__gemm.1")
    e2 = mb2.entry
    a2 = e2.parameter("f16", (128, 256), "a")
    b2 = e2.parameter("f16", (256, 64), "b")
    e2.set_tuple_root([e2.gemm(a2, b2, 1, 0, alpha=0.5)])
    text = mb2.text()
    nested = text.replace('backend_config="{', 'backend_config="{\\"gemm_backend_config\\":{').replace('}", ', '}}", ', 1) \
        if '}", ' in text else text.replace('backend_config="{', 'backend_config="{\\"gemm_backend_config\\":{').replace('}"\n', '}}"\n', 1)
    assert nested != text and "gemm_backend_config" in nested
    m1 = MonoNNModule.compile(text, build=False)
    m2 = MonoNNModule.compile(nested, build=False)
    assert m1.summary() == m2.summary()
    assert m1.get_source("main.hip") == m2.get_source("main.hip")


def _lt_module(epilogue, beta=0.0, n_operands=None):
    mb = HloModuleBuilder("cluster_5__lt.1")
    e = mb.entry
    a = e.parameter("f16", (128, 256), "a")
    w = e.elided_constant("f16", (256, 512), "w/kernel")
    c = e.parameter("f16", (128, 512), "c") if beta else None
    bias = e.elided_constant("f16", (512,), "w/bias") if epilogue.startswith("BIAS") else None
    e.set_tuple_root([e.lt_matmul(a, w, 1, 0, epilogue=epilogue, bias=bias, beta=beta, addend=c)])
    return mb


def test_lt_matmul_becomes_a_gemm_with_a_fused_epilogue():
    # core/op/custom_call.cc:96-100 accepts __cublas$gemm only; the newer spelling lowers onto the same GEMM node with
    # its epilogue enum as an element-wise cluster behind it, which the GEMM-epilogue fusion takes into the tile
    plain = MonoNNModule.compile(_lt_module("DEFAULT").text(), build=False)
    assert "gemm    cublas_lt_matmul_" in plain.summary() and "members=1" in plain.summary() and "f16_b1_m128_n512_k256_ak_bp" in plain.summary()
    fused = MonoNNModule.compile(_lt_module("BIAS_GELU", beta=1.0).text(), build=False)
    s = fused.summary()
    assert "stages=1" in s and "members=2" in s            # one stage: bias, addend and GELU run in the GEMM's epilogue
    src = fused.get_source("main.hip")
    assert "fast_tanh" in src or "tanhf" in src
    for bad, code in ((_lt_module("BIAS").text().replace('\\"epilogue\\":\\"BIAS\\"', '\\"epilogue\\":\\"BIAS_GELU_AUX\\"'), "UNSUPPORTED"),
                      (_lt_module("BIAS").text().replace('\\"epilogue\\":\\"BIAS\\"', '\\"epilogue\\":\\"RELU\\"'), "PARSE_ERROR")):
        with pytest.raises(MonoNNError, match=code):
            MonoNNModule.compile(bad, build=False)


def test_dump_contains_a_standalone_driver_and_the_constants(layer, tmp_path):
    # host_codegen.cc:31-73 counterpart: the dump can be run without the library
    m = MonoNNModule.compile(layer.hlo_text, build=True)
    consts = layer.make_constants(3, "random")
    m.set_constants(consts)
    m.dump(str(tmp_path))
    cluster = os.path.join(tmp_path, "cluster_0")
    src = open(os.path.join(cluster, "best_tuning_spec_src", "host_main.cpp")).read()
    assert "hipModuleLoadData" in src and 'kKernel = "mononn_cluster_0"' in src
    info = m.buffer_info()
    assert f"kTempBytes = {info['temp']}" in src
    names = sorted(os.listdir(os.path.join(cluster, "constants")))
    assert len(names) == len(consts)
    # a packed GEMM weight is dumped in the layout of its module global (padded to 16 columns)
    for c in m.constants():
        path = os.path.join(cluster, "constants", "buffer_for_" + c["name"].lstrip("%").replace(".", "_").replace("-", "_") + ".bin")
        assert os.path.getsize(path) >= c["bytes"]


def test_split_k_consumer_without_a_following_gemm_stays_a_row_program(layer):
    # the last LayerNorm adds up split-K partial sums and feeds no GEMM: a stage of its own, LayerNorm-in-GEMM or not
    spec = json.loads(MonoNNModule.compile(layer.hlo_text, build=False).get_tuning_spec())
    template = next(v for k, v in spec["gemm_spec_list"].items() if k.startswith("cublas_gemm_"))
    gemms = [n.replace(".", "_").replace("-", "_") for n in re.findall(r"%(cublas-gemm\.\d+) =", layer.hlo_text)]
    ffn2 = gemms[-1]
    spec["gemm_spec_list"], spec["cluster_reduce_spec"], spec["cluster_elewise_spec"] = {}, {}, {}
    entry = json.loads(json.dumps(template))
    entry["cutlass_config"]["split_k"] = 2
    spec["gemm_spec_list"][ffn2] = entry
    spec["mononn_hip"]["gemm_prologue_fusion"] = True
    m = MonoNNModule.compile(layer.hlo_text, json.dumps(spec), build=False)
    text = m.summary()
    assert "+row-prologue" in text                      # the first LayerNorm went into FFN1
    assert re.search(rf"gemm\s+{ffn2}\s", text)          # FFN2 is split: bare node, no fused epilogue
    assert re.search(r"rowred\s+\S+\s+members=4", text)  # its consumer: bias + residual + LayerNorm over the partial sums


def _hip_spec(hlo_text, **hip):
    spec = json.loads(MonoNNModule.compile(hlo_text, build=False).get_tuning_spec())
    spec["gemm_spec_list"], spec["cluster_reduce_spec"], spec["cluster_elewise_spec"] = {}, {}, {}
    spec["mononn_hip"].update(hip)
    return spec


def test_hip_options_have_defaults_and_are_checked(layer):
    hip = json.loads(MonoNNModule.compile(layer.hlo_text, build=False).get_tuning_spec())["mononn_hip"]
    assert hip["operand_preload"] is True and hip["pack_left_operands"] is True and hip["stage_rotation"] is True
    assert hip["attention_out_proj_fusion"] is False and hip["gemm_prologue_fusion"] is False and hip["cooperative_launch"] is False
    with pytest.raises(MonoNNError) as e:
        MonoNNModule.compile(layer.hlo_text, json.dumps(_hip_spec(layer.hlo_text, operand_prefetch=True)), build=False)
    assert e.value.status == "SPEC_ERROR"


def test_weights_are_requested_between_arrive_and_wait(layer):
    src = MonoNNModule.compile(layer.hlo_text, build=False).get_source()
    # every packed-weight GEMM has a companion that loads the first chunk of its right operand ...
    pre = set(re.findall(r"void (node_fn_\d+)_pre\(", src))
    assert pre and all(f"typedef mononn_dev::PreB<" in src for _ in pre)
    # ... called in the dispatch switch before the pending barrier wait, the function proper after it
    for fn in pre:
        case = re.search(rf"case \d+: {{ {fn}_preb pre_b; {fn}_pre\(unit.*?pre_b\); if \(pending\) {{ barrier\.wait\(\); pending = false; }} {fn}\(unit.*?smem, pre_b\); }} break;", src)
        assert case, fn
    assert "barrier.arrive();" in src and "barrier.sync()" not in src
    off = MonoNNModule.compile(layer.hlo_text, json.dumps(_hip_spec(layer.hlo_text, operand_preload=False)), build=False).get_source()
    assert "_pre(" not in off and "barrier.sync();" in off and "barrier.arrive()" not in off


def test_fragment_order_writer_and_reader_agree(layer):
    """A left GEMM operand produced in the kernel is written by its producer through the index machinery of the
    code generator and read by the GEMM tile as block (row / 16) * (K / 32) + k / 32, lane (k % 32 / 8) * 16 + row % 16,
    element k % 8: both must name the same address for every (row, k)."""
    src = MonoNNModule.compile(layer.hlo_text, build=False).get_source()
    # the LayerNorm between attention and FFN1 writes [32, 128] f16 rows, 4 or 8 consecutive columns per store
    stores = re.findall(r"stN<_Float16, (\d)>\(out0 \+ ([^,]*\(row / 16\)[^,]*), pk\d+\)", src)
    assert stores, "no fragment-order store of a row program found"
    width, expr = int(stores[0][0]), stores[0][1]
    K, rows = 128, 32
    seen = set()
    for row in range(rows):
        for q0 in range(K // width):
            base = eval(expr.replace("/", "//"), {"row": row, "q0": q0})
            for e in range(width):
                k = q0 * width + e
                want = (((row // 16) * (K // 32) + k // 32) * 64 + ((k % 32) // 8) * 16 + row % 16) * 8 + k % 8
                assert base + e == want, (row, k)
                seen.add(base + e)
    assert seen == set(range(rows * K))
    plain = MonoNNModule.compile(layer.hlo_text, json.dumps(_hip_spec(layer.hlo_text, pack_left_operands=False)), build=False).get_source()
    assert "(row / 16)" not in plain


def test_stage_is_placed_on_idle_workgroups_when_it_fits(layer):
    # LayerNorm: 32 units; FFN1 with 32x64 tiles: 1 x 4 = 4 units: both fit into the grid side by side
    spec = _hip_spec(layer.hlo_text)
    m = MonoNNModule.compile(layer.hlo_text, json.dumps(spec), build=False)
    src = m.get_source()
    assert re.search(r"rot = \d+;", src) and "blockIdx.x >= rot ? blockIdx.x - rot : blockIdx.x + gridDim.x - rot" in src
    rots = [int(r) for r in re.findall(r" rot = (\d+);", src)]
    assert all(r % 8 == 0 for r in rots), "a unit must keep its XCD"
    spec["mononn_hip"]["stage_rotation"] = False
    assert " rot = " not in MonoNNModule.compile(layer.hlo_text, json.dumps(spec), build=False).get_source()


def test_output_projection_inside_the_attention_stage(layer):
    base = MonoNNModule.compile(layer.hlo_text, build=False)
    fused = MonoNNModule.compile(layer.hlo_text, json.dumps(_hip_spec(layer.hlo_text, attention_out_proj_fusion=True)))   # hipRTC build
    assert fused.launch_dims()["barriers"] == base.launch_dims()["barriers"] - 1
    src = fused.get_source()
    assert "float* prow" in src and "pre_w.v[" in src
    # one fp32 partial sum per head, added up by the row program that follows: 4 heads in this fixture
    assert fused.buffer_info()["temp"] > base.buffer_info()["temp"]


def test_layernorm_in_gemm_over_split_k_partial_sums():
    fx = models.bert_encoder(L=2, B=1, S=64, H=256, NH=4, F=512, vocab=300, max_pos=64)
    gemms = [n.replace(".", "_").replace("-", "_") for n in re.findall(r"%(cublas-gemm\.\d+) =", fx.hlo_text)]
    spec = _hip_spec(fx.hlo_text)
    template = next(v for k, v in json.loads(MonoNNModule.compile(fx.hlo_text, build=False).get_tuning_spec())["gemm_spec_list"].items()
                    if k.startswith("cublas_gemm_"))
    for g, s in ((gemms[3], 2), (gemms[5], 4)):
        entry = json.loads(json.dumps(template))
        entry["cutlass_config"]["split_k"] = s
        spec["gemm_spec_list"][g] = entry
    plain = MonoNNModule.compile(fx.hlo_text, json.dumps(spec), build=False)
    spec["mononn_hip"]["gemm_prologue_fusion"] = True
    fused = MonoNNModule.compile(fx.hlo_text, json.dumps(spec))   # hipRTC build
    assert fused.launch_dims()["barriers"] < plain.launch_dims()["barriers"]
    src = fused.get_source()
    # the partial sums of the split GEMMs are stored in fragment order for the row program in front of the next GEMM
    assert re.search(r"stN<float, 4>\(out \+ \(long\)ksplit \* \d+ \+ \(m % 16\) \* 8", src)


def norm_gemm_module(with_beta):
    """Mean / variance normalisation with a scale (and, with_beta, a shift: LayerNorm) feeding a weight GEMM."""
    mb = HloModuleBuilder("cluster_3__norm_gemm.1")
    e = mb.entry
    M, K, N = 64, 256, 128
    x = e.parameter("f16", (M, K), "x")
    gamma = e.elided_constant("f16", (K,), "ln/gamma")
    beta = e.elided_constant("f16", (K,), "ln/beta")
    add = mb.reducer("add", "f32")

    def sum_body(f, px):
        return f.reduce(f.convert(px, "f32"), f.scalar("f32", 0.0), 1, add)
    s = e.fusion("kInput", [x], sum_body)

    def centred(f, px, ps):
        return f.sub(f.convert(px, "f32"), f.broadcast(f.mul(ps, f.splat("f32", 1.0 / K, (M,))), (M, K), [0]))

    def var_body(f, px, ps):
        d = centred(f, px, ps)
        return f.reduce(f.mul(d, d), f.scalar("f32", 0.0), 1, add)
    v = e.fusion("kInput", [x, s], var_body)

    def norm_body(f, px, ps, pv, pg, pb):
        r = f.rsqrt(f.add(f.mul(pv, f.splat("f32", 1.0 / K, (M,))), f.splat("f32", 1e-5, (M,))))
        y = f.mul(f.broadcast(f.convert(pg, "f32"), (M, K), [1]), f.mul(f.broadcast(r, (M, K), [0]), centred(f, px, ps)))   # operands the other way round
        if with_beta:
            y = f.add(f.broadcast(f.convert(pb, "f32"), (M, K), [1]), y)
        return f.convert(y, "f16")
    h = e.fusion("kLoop", [x, s, v, gamma, beta], norm_body)
    w = e.elided_constant("f16", (K, N), "w/kernel")
    e.set_tuple_root([e.gemm(h, w, 1, 0)])
    return mb.text(), mb.constants


def test_layer_norm_in_front_of_a_gemm_is_recognised_and_other_row_programs_are_not():
    # with the prologue fusion on, a row program that is exactly LayerNorm takes the hand-laid-out form (sums by
    # v_dot2_f32_f16, one exchange); anything else - here the same normalisation without the shift - is generated
    # element by element from the HLO as before
    for with_beta in (True, False):
        text, _ = norm_gemm_module(with_beta)
        spec = json.loads(MonoNNModule.compile(text, build=False).get_tuning_spec())
        spec["mononn_hip"]["gemm_prologue_fusion"] = True
        spec["gemm_spec_list"], spec["cluster_reduce_spec"] = {}, {}
        m = MonoNNModule.compile(text, json.dumps(spec), build=False)
        src = m.get_source("main.hip")
        assert m.launch_dims()["barriers"] == 0 and "_pro {" in src          # one stage: the row program runs inside the GEMM
        assert ("__builtin_amdgcn_fdot2" in src) == with_beta


def test_layer_norm_folding_moves_the_scale_into_the_weights_and_the_rest_into_the_epilogue():
    # h = ((x - mean) * r) * gamma + beta in front of h @ W becomes r * (x @ (gamma o W) - mean * (gamma^T W)) + beta^T W:
    # the MFMAs read x as stored, the functor in front of them only computes (mean, r), the epilogue applies the
    # rank-1 correction, and the host derives the scaled weights and the two column sums when the payloads arrive
    text, _ = norm_gemm_module(True)
    spec = json.loads(MonoNNModule.compile(text, build=False).get_tuning_spec())
    spec["mononn_hip"]["gemm_prologue_fusion"] = True
    spec["mononn_hip"]["layer_norm_folding"] = True
    spec["gemm_spec_list"], spec["cluster_reduce_spec"] = {}, {}
    m = MonoNNModule.compile(text, json.dumps(spec), build=False)
    src = m.get_source("main.hip")
    assert m.launch_dims()["barriers"] == 0
    assert "after_mfma = true" in src and "ln_stats[" in src and "__builtin_amdgcn_fdot2" in src
    consts = {c["name"]: c for c in m.constants()}
    derived = [n for n in consts if n.endswith("_ln_gamma_sums") or n.endswith("_ln_beta_sums")]
    assert len(derived) == 2 and all(consts[n]["bytes"] == 128 * 4 and not consts[n]["needs_payload"] for n in derived)
    # gamma and beta themselves are still asked of the caller: the column sums are computed from them
    assert sum(c["needs_payload"] for c in consts.values()) == 3
    # without the shift it is not LayerNorm: the fold stays away and the generic prologue is generated
    text, _ = norm_gemm_module(False)
    m = MonoNNModule.compile(text, json.dumps(spec), build=False)
    assert "ln_stats[" not in m.get_source("main.hip") and "_pro {" in m.get_source("main.hip")
    # a spec that asks for the fold without the prologue fusion has nothing to fold
    spec["mononn_hip"]["gemm_prologue_fusion"] = False
    m = MonoNNModule.compile(norm_gemm_module(True)[0], json.dumps(spec), build=False)
    assert "ln_stats[" not in m.get_source("main.hip") and m.launch_dims()["barriers"] >= 1


def test_bf16_modules_take_the_bf16_mfma_on_the_same_tiles():
    # bf16 is parsed, element-wise code computes through float and rounds where the HLO says bf16, weight GEMMs run
    # on the direct tile or the LDS-staged tile with the bf16 form of the MFMA (last template argument), constants
    # are packed in fragment order like f16 ones, and the attention is one fused stage holding scores and
    # probabilities as bf16 between its two contractions
    fx = models.bert_encoder(L=1, B=2, S=64, H=128, NH=2, F=256, vocab=300, max_pos=64, ftype="bf16")
    m = MonoNNModule.compile(fx.hlo_text)          # hipRTC build
    src = m.get_source("main.hip")
    assert "__bf16" in src and "_Float16" not in src.split("extern \"C\"")[1]
    calls = src.count("mononn_dev::gemm_tile<")
    assert calls >= 4 and src.count(", true>(reinterpret_cast<const half_t*>(") == calls
    assert m.launch_dims()["barriers"] == 7 and "mononn_dev::mfma_16x16x32<true>(" in src   # as the f16 encoder
    packed = [c for c in m.constants() if c["role"].endswith("/kernel")]
    assert packed and all(c["needs_payload"] for c in packed)
    # the LDS-staged tile
    spec = json.loads(m.get_tuning_spec())
    n = 0
    for name, e in spec["gemm_spec_list"].items():
        c = e["cutlass_config"]
        if name.startswith("cublas_gemm_") and c["split_k"] == 1:
            c["threadblockshape"].update(m=64, n=64, k=32)
            c["wave_arrangement"] = {"m": 2, "n": 2, "k": 1}
            c["stages"] = 2
            n += 1
    assert n >= 4
    lds = MonoNNModule.compile(fx.hlo_text, json.dumps(spec)).get_source("main.hip")
    staged = lds.count("gemm_tile_lds<")
    # (a second `true`: the result is row-major and goes through LDS a fragment row at a time)
    assert staged >= 4 and len(re.findall(r"mononn_dev::RowMajorA, true(?:, true)?>\(reinterpret_cast<const half_t\*>\(", lds)) == staged
    # a mixed GEMM is refused
    bad = fx.hlo_text.replace("bf16[128,128]{1,0} custom-call(", "f16[128,128]{1,0} custom-call(", 1)
    if bad != fx.hlo_text:
        with pytest.raises(MonoNNError) as ei:
            MonoNNModule.compile(bad, build=False)
        assert ei.value.status in ("UNSUPPORTED", "PARSE_ERROR", "INVALID_ARGUMENT")
