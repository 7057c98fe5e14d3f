"""GPU parity: the generated monolithic kernel against the NumPy oracle on the same seeded inputs.
Tolerance (stated by the north star): max-abs-err <= 2e-2 and cosine >= 0.9999 against the fp32
evaluation of the HLO; integer / gather work bit-exact."""
import re

import numpy as np
import pytest

from mononn_amd import MonoNNModule
from mononn_amd.hlo import models
from mononn_amd.hlo.builder import HloModuleBuilder
from oracle import hlo_interp

pytestmark = pytest.mark.gpu


def run_module(hlo_text, inputs, constants, outputs, spec_json=None):
    m = MonoNNModule.compile(hlo_text, spec_json)
    m.set_constants(constants)
    m.load(0)
    return m.run(inputs, outputs), m


def check_close(got, want32, atol=2e-2, cos_min=0.9999):
    g = got.astype(np.float64).ravel()
    w = want32.astype(np.float64).ravel()
    assert np.all(np.isfinite(g))
    err = np.abs(g - w).max()
    cos = float(g @ w / (np.linalg.norm(g) * np.linalg.norm(w) + 1e-30))
    assert err <= atol, f"max abs err {err}"
    assert cos >= cos_min, f"cosine {cos}"
    return err, cos


def gemm_module(M, N, K, batch=(), lhs_c=None, rhs_c=None, alpha=1.0, b_const=False, as_dot=False, dtype="f16"):
    mb = HloModuleBuilder("cluster_7__gemm_test.1")
    e = mb.entry
    r = len(batch) + 2
    lhs_c = r - 1 if lhs_c is None else lhs_c
    rhs_c = r - 2 if rhs_c is None else rhs_c
    a_dims = list(batch) + ([M, K] if lhs_c == r - 1 else [K, M])
    b_dims = list(batch) + ([K, N] if rhs_c == r - 2 else [N, K])
    a = e.parameter(dtype, a_dims, "a")
    b = e.elided_constant(dtype, b_dims, "w/kernel") if b_const else e.parameter(dtype, b_dims, "b")
    if as_dot:
        d = e.dot(a, b, lhs_c, rhs_c, batch_dims=tuple(range(len(batch))))
    else:
        d = e.gemm(a, b, lhs_c, rhs_c, batch_dims=tuple(range(len(batch))), alpha=alpha)
    e.set_tuple_root([d])
    return mb, a_dims, b_dims, list(batch) + [M, N]


@pytest.mark.parametrize("case", [
    dict(M=128, N=768, K=768, b_const=True),                      # weight GEMM, constant transposed at upload
    dict(M=128, N=96, K=64),                                      # [K,N] parameter operand: gathered per lane, still on the MFMAs
    dict(M=128, N=128, K=64, batch=(1, 12), rhs_c=3, alpha=0.125),  # scores: both operands k-contiguous
    dict(M=128, N=64, K=128, batch=(2, 3)),                       # context: B stored [K,N]
    dict(M=100, N=52, K=96, rhs_c=1),                             # ragged M / N on the MFMA path
    dict(M=64, N=48, K=40, rhs_c=1),                              # K not a multiple of 32: zero-filled last MFMA step
    dict(M=197, N=64, K=197, batch=(2, 3), rhs_c=3),              # odd row length: fragments start at unaligned addresses
    dict(M=33, N=20, K=17, rhs_c=1),                              # K below one MFMA step
    dict(M=64, N=48, K=40),                                       # K not a multiple of 32 and B stored [K,N]: zero-filled gather
    dict(M=40, N=24, K=64, lhs_c=0, rhs_c=1),                     # A stored [K,M]: gathered per lane onto the MFMAs (gemm_impl.cc:408-469 takes either order)
    dict(M=128, N=96, K=256, lhs_c=0),                            # A stored [K,M] and B stored [K,N]: both gathered
    dict(M=100, N=52, K=72, lhs_c=0, rhs_c=1),                    # A stored [K,M], ragged M / N, K off the MFMA step
    dict(M=64, N=128, K=128, lhs_c=1, batch=(3,)),                # batched, A stored [b,K,M]
    dict(M=128, N=256, K=256, lhs_c=0, b_const=True),             # A stored [K,M] against constant weights (left as given: not packed)
    dict(M=128, N=256, K=256, b_const=True, as_dot=True),         # plain `dot` with a constant right operand
    dict(M=48, N=80, K=64, batch=(3,), rhs_c=2, as_dot=True),     # batched `dot`, both operands k-contiguous
    dict(M=200, N=136, K=256, dtype="f32", rhs_c=1),              # f32 on v_mfma_f32_16x16x4_f32, both operands k-contiguous
    dict(M=128, N=96, K=100, dtype="f32"),                        # f32, B stored [K,N], k extent off the chunk of 16
    dict(M=77, N=50, K=33, batch=(2,), dtype="f32", rhs_c=2),     # f32, batched, everything ragged
    dict(M=128, N=256, K=128, dtype="f32", b_const=True),         # f32 constant weights (not packed)
    dict(M=40, N=24, K=64, dtype="f32", lhs_c=0, rhs_c=1),        # f32 with A stored [K,M]: per-element fallback
    dict(M=256, N=1001, K=128, rhs_c=1, b_const=True),            # odd N: rows at 2-byte aligned addresses, 4 columns per store where they fit
    dict(M=70, N=50, K=64, batch=(2,), rhs_c=2),                  # N off the run of 4, batched
])
def test_gemm_cases(gpu_device, case):
    mb, a_dims, b_dims, d_dims = gemm_module(**case)
    rng = np.random.default_rng(3)
    dtype = case.get("dtype", "f16")
    npdt = np.float32 if dtype == "f32" else np.float16
    a = rng.normal(0, 1, a_dims).astype(npdt)
    b = rng.normal(0, 1, b_dims).astype(npdt)
    text = mb.text()
    consts = {n: b for n in mb.constants}
    inputs = [a] if case.get("b_const") else [a, b]
    (got,), _ = run_module(text, inputs, consts, [{"dtype": dtype, "dims": d_dims}])
    want = hlo_interp.evaluate(text, inputs, consts, "fp32")[0]
    scale = np.abs(want).max()
    if dtype == "f32":
        # f32 inputs and accumulation: only the summation order differs from the oracle's
        assert got.dtype == np.float32 and np.abs(got - want).max() <= 2e-5 * scale
    else:
        # fp16 output rounding of values up to ~sqrt(K): relative tolerance
        assert np.abs(got.astype(np.float32) - want).max() <= 2e-3 * scale + 1e-3


def test_f32_gemm_with_fused_epilogue(gpu_device):
    # f32 [M,K] x constant [K,N] with bias add and ReLU fused onto the accumulator tile
    M, N, K = 150, 200, 96
    mb = HloModuleBuilder("cluster_8__gemm_f32_epilogue.1")
    e = mb.entry
    a = e.parameter("f32", (M, K), "a")
    w = e.elided_constant("f32", (K, N), "w/kernel")
    bias = e.elided_constant("f32", (N,), "w/bias")
    d = e.gemm(a, w, 1, 0)

    def body(f, pd, pb):
        return f.maximum(f.add(pd, f.broadcast(pb, pd.dims, [1])), f.splat("f32", 0.0, pd.dims))
    y = e.fusion("kLoop", [d, bias], body)
    e.set_tuple_root([y])
    rng = np.random.default_rng(12)
    av = rng.normal(0, 1, (M, K)).astype(np.float32)
    consts = {}
    for name, meta in mb.constants.items():
        consts[name] = rng.normal(0, 1, meta["dims"]).astype(np.float32)
    (got,), m = run_module(mb.text(), [av], consts, [{"dtype": "f32", "dims": [M, N]}])
    src = m.get_source("main.hip")
    assert "gemm_tile_f32<" in src and m.launch_dims()["barriers"] == 0      # one stage: the epilogue is fused
    want = hlo_interp.evaluate(mb.text(), [av], consts, "fp32")[0]
    assert (want == 0).any() and (want > 0).any()
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()


@pytest.mark.parametrize("with_beta", [True, False])
def test_row_program_in_front_of_a_gemm(gpu_device, with_beta):
    # LayerNorm inside the GEMM in its hand-laid-out form (with_beta) and a row program that is not LayerNorm in the
    # generic form, both against the oracle
    import json
    from test_host_compiler import norm_gemm_module
    text, constants = norm_gemm_module(with_beta)
    spec = json.loads(MonoNNModule.compile(text, build=False).get_tuning_spec())
    spec["mononn_hip"]["gemm_prologue_fusion"] = True
    spec["gemm_spec_list"], spec["cluster_reduce_spec"] = {}, {}
    rng = np.random.default_rng(31)
    x = rng.normal(0.7, 2.0, (64, 256)).astype(np.float16)          # a mean well away from zero
    consts = {name: (rng.normal(1.0, 0.2, meta["dims"]) if len(meta["dims"]) == 1 else rng.normal(0, 0.05, meta["dims"])).astype(np.float16)
              for name, meta in constants.items()}
    want = hlo_interp.evaluate(text, [x], consts, "fp32")[0]
    (got,), m = run_module(text, [x], consts, [{"dtype": "f16", "dims": [64, 128]}], json.dumps(spec))
    assert ("__builtin_amdgcn_fdot2" in m.get_source("main.hip")) == with_beta
    m.close()
    check_close(got, want, atol=2e-2)


def test_bert_layer_parity(gpu_device):
    fx = models.bert_layer()
    consts = fx.make_constants(1234, "random")
    inputs = fx.make_inputs(1234)
    (got,), m = run_module(fx.hlo_text, inputs, consts, fx.outputs)
    want = hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0]
    err, cos = check_close(got, want)
    print(f"bert_layer: max_abs_err={err:.3e} cosine={cos:.6f} dims={m.launch_dims()}")


def test_gather_bit_exact(gpu_device):
    mb = HloModuleBuilder("cluster_3__gather_test.1")
    e = mb.entry
    ids = e.parameter("s32", (2, 37), "ids")
    table = e.elided_constant("f16", (1000, 96), "table")
    g = e.gather_rows(table, ids)
    e.set_tuple_root([g])
    rng = np.random.default_rng(5)
    t = rng.normal(0, 1, (1000, 96)).astype(np.float16)
    i = rng.integers(0, 1000, (2, 37), dtype=np.int32)
    consts = {n: t for n in mb.constants}
    (got,), _ = run_module(mb.text(), [i], consts, [{"dtype": "f16", "dims": [2, 37, 96]}])
    assert np.array_equal(got.view(np.uint16), t[i].view(np.uint16))


@pytest.mark.parametrize("epilogue,beta", [("DEFAULT", 0.0), ("BIAS", 0.0), ("RELU", 0.0), ("GELU", 0.0), ("BIAS_RELU", 2.0), ("BIAS_GELU", 0.0), ("BIAS_GELU", 0.5)])
def test_lt_matmul_cases(gpu_device, epilogue, beta):
    """__cublas$lt$matmul (a, b[, c][, bias]) with every epilogue of its enum that has one result, on the MFMA tile with
    the epilogue fused, against the oracle's own restatement of the call (core/op/custom_call.cc:96-100 knows only the
    older spelling; gemm_impl.cc:182-231 for alpha / beta)."""
    M, K, N = 128, 256, 384
    mb = HloModuleBuilder("cluster_7__lt_test.1")
    e = mb.entry
    a = e.parameter("f16", (M, K), "a")
    w = e.elided_constant("f16", (K, N), "w/kernel")
    c = e.parameter("f16", (M, N), "c") if beta else None
    bias = e.elided_constant("f16", (N,), "w/bias") if epilogue.startswith("BIAS") else None
    e.set_tuple_root([e.lt_matmul(a, w, 1, 0, epilogue=epilogue, bias=bias, alpha=0.25, beta=beta, addend=c)])
    rng = np.random.default_rng(11)
    A = rng.normal(0, 1, (M, K)).astype(np.float16)
    C = rng.normal(0, 1, (M, N)).astype(np.float16)
    names = list(mb.constants)
    consts = {names[0]: rng.normal(0, 1, (K, N)).astype(np.float16)}
    if bias is not None:
        consts[names[1]] = rng.normal(0, 2, (N,)).astype(np.float16)
    inputs = [A] + ([C] if beta else [])
    text = mb.text()
    assert MonoNNModule.compile(text, build=False).launch_dims()["barriers"] == 0   # one stage: the epilogue runs in the tile
    (got,), _ = run_module(text, inputs, consts, [{"dtype": "f16", "dims": [M, N]}])
    want = hlo_interp.evaluate(text, inputs, consts, "fp32")[0]
    assert np.abs(got.astype(np.float32) - want).max() <= 2e-3 * np.abs(want).max() + 1e-3


def _spec_with(hlo_text, gemm_overrides=None, hip=None, grid=None):
    """Default specification with some entries replaced; per-node maps are cleared so that nodes whose names
    change with the fusion decisions get fresh defaults."""
    import json
    spec = json.loads(MonoNNModule.compile(hlo_text, build=False).get_tuning_spec())
    template = next(iter(spec["gemm_spec_list"].values()))
    spec["gemm_spec_list"] = {}
    spec["cluster_reduce_spec"] = {}
    spec["cluster_elewise_spec"] = {}
    for name, cc in (gemm_overrides or {}).items():
        entry = json.loads(json.dumps(template))
        entry["cutlass_config"].update(cc)
        spec["gemm_spec_list"][name] = entry
    spec["mononn_hip"].update(hip or {})
    if grid:
        spec["cuda_context"]["cuda_runtime_context"]["grid_dim"]["x"] = grid
    return json.dumps(spec)


def _gemm_instr_names(hlo_text):
    import re
    return [n.replace(".", "_").replace("-", "_") for n in re.findall(r"%(cublas-gemm\.\d+) =", hlo_text)]


def test_folded_layer_norm_on_rows_far_from_zero(gpu_device):
    """LayerNorm folded into weights and epilogue, h.W = r (x.W' - mean colsum(W')) + beta^T W with W' = half(gamma o W):
    the column sums must belong to the weights the MFMAs multiply, or an error of r * mean * (sum of a column's
    rounding errors) stays behind.  Rows with |mean| = 40 sigma make that term visible: against the oracle the folded
    kernel must be as close as the kernel that runs the LayerNorm as written."""
    import json
    from test_host_compiler import norm_gemm_module
    text, declared = norm_gemm_module(True)
    M, K, N = 64, 256, 128
    rng = np.random.default_rng(71)
    x = (rng.normal(0, 0.25, (M, K)) + rng.choice([-10.0, 10.0], (M, 1))).astype(np.float16)
    by_role = {v["role"]: k for k, v in declared.items()}
    consts = {by_role["ln/gamma"]: rng.uniform(0.5, 1.5, (K,)).astype(np.float16),
              by_role["ln/beta"]: rng.normal(0, 0.5, (K,)).astype(np.float16),
              by_role["w/kernel"]: rng.normal(0, 0.05, (K, N)).astype(np.float16)}
    want = hlo_interp.evaluate(text, [x], consts, "fp32")[0].astype(np.float64)
    outs = [{"dtype": "f16", "dims": [M, N]}]
    (plain,), m1 = run_module(text, [x], consts, outs)
    spec = json.loads(MonoNNModule.compile(text, build=False).get_tuning_spec())
    spec["mononn_hip"].update(gemm_prologue_fusion=True, layer_norm_folding=True)
    spec["gemm_spec_list"], spec["cluster_reduce_spec"] = {}, {}
    (folded,), m2 = run_module(text, [x], consts, outs, json.dumps(spec))
    assert "ln_stats[" in m2.get_source("main.hip")
    err_plain = np.abs(plain.astype(np.float64) - want).max()
    err_folded = np.abs(folded.astype(np.float64) - want).max()
    print(f"rows at |mean| = 40 sigma: as written {err_plain:.3e}, folded {err_folded:.3e}", flush=True)
    assert err_folded <= max(2 * err_plain, 4e-3 * np.abs(want).max())
    m1.close()
    m2.close()


def test_fusion_variants_agree(gpu_device):
    """Every stage-fusion decision must leave the result unchanged (bit for bit where the arithmetic is the
    same, within fp16 rounding where a reduction order changes)."""
    fx = models.bert_encoder(L=2, B=1, S=64, H=256, NH=4, F=512, vocab=300, max_pos=64)
    consts = fx.make_constants(21, "random")
    inputs = fx.make_inputs(21)
    want = hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0]
    (base,), m0 = run_module(fx.hlo_text, inputs, consts, fx.outputs)
    check_close(base, want)
    gemms = _gemm_instr_names(fx.hlo_text)
    # out-projection and FFN2 of both layers: k split over workgroups, partial sums added by the LayerNorm stage
    split = {}
    for layer in range(2):
        split[gemms[layer * 6 + 3]] = {"split_k": 2}
        split[gemms[layer * 6 + 5]] = {"split_k": 4}
    variants = {
        "fenced barrier, reused temp slots": _spec_with(fx.hlo_text, hip={"barrier": "flags"}),
        "no attention fusion": _spec_with(fx.hlo_text, hip={"fuse_attention": False}),
        "no epilogue fusion": _spec_with(fx.hlo_text, hip={"gemm_epilogue_fusion": False}),
        "LayerNorm as GEMM prologue": _spec_with(fx.hlo_text, hip={"gemm_prologue_fusion": True}),
        "LayerNorm as GEMM prologue over split-K partial sums": _spec_with(fx.hlo_text, hip={"gemm_prologue_fusion": True}, gemm_overrides=split),
        "LayerNorm folded into weights and epilogue": _spec_with(fx.hlo_text, hip={"gemm_prologue_fusion": True, "layer_norm_folding": True}),
        # a LayerNorm fed by a k-split GEMM stays a stage that adds the partial sums up; the others are folded
        "LayerNorm folded where no k split feeds it": _spec_with(fx.hlo_text, hip={"gemm_prologue_fusion": True, "layer_norm_folding": True},
                                                              gemm_overrides={k: v for k, v in split.items() if v["split_k"] == 4}),
        "plain weight layout": _spec_with(fx.hlo_text, hip={"transpose_constant_b": False, "assign_operand_layouts": False}),
        "split-K": _spec_with(fx.hlo_text, gemm_overrides=split),
        "cooperative launch": _spec_with(fx.hlo_text, hip={"cooperative_launch": True}),
        # by default a GEMM stage asks for its packed weights before it waits at the grid barrier
        "weights requested inside the tile": _spec_with(fx.hlo_text, hip={"operand_preload": False}),
        "the same with split-K": _spec_with(fx.hlo_text, hip={"operand_preload": False}, gemm_overrides=split),
        # a grid of 8 workgroups: several units per workgroup and stage, only the first of them behind a barrier wait
        "small grid": _spec_with(fx.hlo_text, grid=8),
        # two workgroups per compute unit: the kernel is compiled for half the registers per wave, the whole grid
        # must still be resident for the barrier
        "two workgroups per compute unit": _spec_with(fx.hlo_text, grid=512),
        # the projection of the merged heads inside the attention stage: one stage less per layer, the LayerNorm
        # stage adds one fp32 partial sum per head
        "output projection inside the attention stage": _spec_with(fx.hlo_text, hip={"attention_out_proj_fusion": True}),
        "the same, weights requested inside the stage": _spec_with(fx.hlo_text, hip={"attention_out_proj_fusion": True, "operand_preload": False}),
    }
    for name, spec in variants.items():
        (got,), m = run_module(fx.hlo_text, inputs, consts, fx.outputs, spec)
        err, cos = check_close(got, want)
        diff = np.abs(got.astype(np.float32) - base.astype(np.float32)).max()
        print(f"{name}: barriers={m.launch_dims()['barriers']} max_abs_err={err:.2e} vs default {diff:.2e}")
        assert diff <= 8e-3, name
        if name.startswith("output projection inside"):
            assert m.launch_dims()["barriers"] == m0.launch_dims()["barriers"] - 2, "one stage less per layer"
    (fenced,), _ = run_module(fx.hlo_text, inputs, consts, fx.outputs, variants["fenced barrier, reused temp slots"])
    assert np.array_equal(fenced.view(np.uint16), base.view(np.uint16)), "barrier flavour must not change any bit"
    (coop,), _ = run_module(fx.hlo_text, inputs, consts, fx.outputs, variants["cooperative launch"])
    assert np.array_equal(coop.view(np.uint16), base.view(np.uint16)), "the launch entry point must not change any bit"
    for name in ("weights requested inside the tile", "small grid"):
        (other,), _ = run_module(fx.hlo_text, inputs, consts, fx.outputs, variants[name])
        assert np.array_equal(other.view(np.uint16), base.view(np.uint16)), f"{name}: when an operand is requested must not change any bit"
    # MFMA accumulators stored as they are (fp32 partial sums of a k-split GEMM, per-head partial sums of the projection
    # inside the attention stage): the 16-byte write-through store of the default barrier against the two plain
    # 8-byte stores of the fenced one, bit for bit
    import json
    for name in ("split-K", "output projection inside the attention stage"):
        fenced_spec = json.loads(variants[name])
        fenced_spec["mononn_hip"]["barrier"] = "flags"
        (a,), _ = run_module(fx.hlo_text, inputs, consts, fx.outputs, variants[name])
        (b,), mb = run_module(fx.hlo_text, inputs, consts, fx.outputs, json.dumps(fenced_spec))
        assert "#define MONONN_COHERENT_STORES 1" not in mb.get_source("main.hip")
        assert np.array_equal(a.view(np.uint16), b.view(np.uint16)), f"{name}: the store instruction must not change any bit"


def test_repeated_launches_are_bit_identical(gpu_device):
    fx = models.bert_encoder(L=2, B=1, S=64, H=256, NH=4, F=512, vocab=300, max_pos=64)
    consts = fx.make_constants(22, "random")
    inputs = fx.make_inputs(22)
    m = MonoNNModule.compile(fx.hlo_text)
    m.set_constants(consts)
    m.load(0)
    first = m.run(inputs, fx.outputs)[0]
    for _ in range(100):
        again = m.run(inputs, fx.outputs)[0]
        assert np.array_equal(first.view(np.uint16), again.view(np.uint16))
    other = fx.make_inputs(23)
    changed = m.run(other, fx.outputs)[0]
    want = hlo_interp.evaluate(fx.hlo_text, other, consts, "fp32")[0]
    check_close(changed, want)


@pytest.mark.parametrize("key_waves", [1, 2, 4])
def test_attention_key_wave_arrangements(gpu_device, key_waves):
    """The fused attention node with 1, 2 or 4 waves sharing a block of 16 query rows (the others take further
    row blocks): same result up to the order in which the key slices are added."""
    import json
    fx = models.bert_encoder(L=1, B=2, S=128, H=256, NH=4, F=512, vocab=300, max_pos=128, mask_kind="length_mask")
    consts = fx.make_constants(24, "random")
    inputs = fx.make_inputs(24)
    want = hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0]
    spec = json.loads(MonoNNModule.compile(fx.hlo_text, build=False).get_tuning_spec())
    names = [n for n in spec["gemm_spec_list"] if n.startswith("cublas_batch_gemm_")]
    assert names, "the attention block did not fuse"
    for n in names:
        spec["gemm_spec_list"][n]["cutlass_config"]["wave_arrangement"].update(k=key_waves, m=4 // key_waves)
        spec["gemm_spec_list"][n]["cutlass_config"]["threadblockshape"]["m"] = 16 * (4 // key_waves)   # query rows per unit
    (got,), m = run_module(fx.hlo_text, inputs, consts, fx.outputs, json.dumps(spec))
    assert f"kw = mononn_dev::wave_id() % {key_waves}" in m.get_source("main.hip")
    check_close(got, want)


@pytest.mark.parametrize("xd,size,stride,pad", [
    ((2, 9, 10, 8), (1, 3, 3, 1), (1, 2, 2, 1), ((0, 0), (1, 1), (1, 1), (0, 0))),
    ((4, 56, 56, 64), (1, 3, 3, 1), (1, 2, 2, 1), ((0, 0), (0, 1), (0, 1), (0, 0))),     # ResNet stem pooling
    ((3, 7, 5, 2), (1, 3, 2, 1), (1, 1, 2, 1), ((0, 0), (1, 1), (0, 1), (0, 0))),
])
def test_reduce_window_bit_exact(gpu_device, xd, size, stride, pad):
    # maximum never rounds; the f16 sum adds the window elements in the order the HLO's evaluation defines (ascending
    # window offsets, rounding after every add), so both are bit-exact against the oracle run "as written"
    from op_cases import pool_module
    x = np.random.default_rng(51).normal(0, 1, xd).astype(np.float16)
    for kind in ("max", "sum"):
        text, od = pool_module(xd, size, stride, pad, kind)
        (got,), _ = run_module(text, [x], {}, [{"dtype": "f16", "dims": od}])
        want = hlo_interp.evaluate(text, [x], {})[0]
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), kind
        want32 = hlo_interp.evaluate(text, [x], {}, "fp32")[0]
        assert np.abs(got.astype(np.float32) - want32).max() <= 2e-2


def test_dynamic_update_slice_bit_exact(gpu_device):
    from op_cases import update_slice_module
    rng = np.random.default_rng(53)
    x = rng.normal(0, 1, (6, 10, 8)).astype(np.float16)
    u = rng.normal(0, 1, (2, 4, 8)).astype(np.float16)
    for scale in (None, 2.0):
        text = update_slice_module(x.shape, u.shape, scale=scale)
        m = MonoNNModule.compile(text)
        m.load(0)
        for starts in [(1, 3, 0), (0, 0, 0), (4, 6, 0), (9, -5, 3)]:      # the last one is clamped to (4, 0, 0)
            ins = [x, u] + [np.array(s, np.int32) for s in starts]
            (got,) = m.run(ins, [{"dtype": "f16", "dims": list(x.shape)}])
            want = hlo_interp.evaluate(text, ins, {})[0]
            assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), (scale, starts)
        m.close()


@pytest.mark.parametrize("rows,n,direction,axis", [
    (7, 50, "GT", 1),          # one wave per row, partly filled
    (64, 1000, "GT", 1),       # one workgroup per row, register-resident
    (5, 333, "LT", 1),
    (16, 50257, "GT", 1),      # vocabulary-sized rows: column loop, exchange through LDS
    (40, 50, "GT", 0),         # not the last dimension: serial loop per output element
])
def test_variadic_reduce_bit_exact(gpu_device, rows, n, direction, axis):
    # (value, index) reduction: arg-max / arg-min with the first index on ties
    from op_cases import arg_reduce_module
    x = np.random.default_rng(57).integers(-6, 7, (rows, n) if axis == 1 else (n, rows)).astype(np.float16)      # many ties
    text = arg_reduce_module(rows, n, direction, axis=axis)
    (v, i), _ = run_module(text, [x], {}, [{"dtype": "f16", "dims": [rows]}, {"dtype": "s32", "dims": [rows]}])
    assert np.array_equal(i, (np.argmax if direction == "GT" else np.argmin)(x, axis=axis).astype(np.int32))
    assert np.array_equal(v, x.max(axis=axis) if direction == "GT" else x.min(axis=axis))
    if n <= 1000:
        wv, wi = hlo_interp.evaluate(text, [x], {})
        assert np.array_equal(i, wi) and np.array_equal(v.view(np.uint16), wv.view(np.uint16))


# ---- bf16 (not in the reference, whose tiles are half and float): the same kernels on the bf16 forms of the MFMAs ----
def _bf16_check(got_bits, want32, what, steps=4.0, atol=2e-2):
    """bf16 results against fp32 values: within `steps` bf16 spacings (2^-8 relative) of the value's magnitude, plus
    `atol` for sums whose terms cancel."""
    from mononn_amd import bf16
    assert got_bits.dtype == np.uint16
    g = bf16.from_bits(got_bits).astype(np.float64).ravel()
    w = want32.astype(np.float64).ravel()
    assert np.all(np.isfinite(g))
    err = np.abs(g - w)
    bound = steps * 2.0 ** -8 * np.abs(w) + atol
    cos = float(g @ w / (np.linalg.norm(g) * np.linalg.norm(w) + 1e-30))
    print(f"{what}: max_abs_err={err.max():.3e} cosine={cos:.6f}")
    assert (err <= bound).all(), f"{what}: {err.max()} at magnitude {np.abs(w)[err.argmax()]}"
    assert cos >= 0.9999


@pytest.mark.parametrize("case", [
    dict(M=128, N=768, K=768, b_const=True),                       # weight GEMM: constant packed in fragment order
    dict(M=128, N=96, K=64),                                       # [K,N] parameter operand, gathered per lane
    dict(M=128, N=128, K=64, batch=(2, 3), rhs_c=3, alpha=0.125),  # batched, both operands k-contiguous
    dict(M=100, N=52, K=96, rhs_c=1),                              # ragged M / N
    dict(M=64, N=48, K=40, rhs_c=1),                               # K off the MFMA step: zero-filled last step
    dict(M=256, N=1001, K=128, rhs_c=1, b_const=True),             # odd N: four columns per store where they fit
    dict(M=40, N=24, K=64, lhs_c=0, rhs_c=1),                      # A stored [K,M]: gathered per lane
])
def test_bf16_gemm_cases(gpu_device, case):
    from mononn_amd import bf16
    mb, a_dims, b_dims, d_dims = gemm_module(dtype="bf16", **case)
    rng = np.random.default_rng(5)
    a = bf16.to_bits(rng.normal(0, 1, a_dims))
    b = bf16.to_bits(rng.normal(0, 1, b_dims))
    text = mb.text()
    consts = {n: b for n in mb.constants}
    inputs = [a] if case.get("b_const") else [a, b]
    (got,), m = run_module(text, inputs, consts, [{"dtype": "bf16", "dims": d_dims}])
    assert ", true>(reinterpret_cast<const half_t*>(" in m.get_source("main.hip")
    want = hlo_interp.evaluate(text, inputs, consts, "fp32")[0]
    # one rounding of an exactly accumulated sum: half a bf16 spacing, a little more for the summation order
    _bf16_check(got, want, f"bf16 gemm {case}", steps=1.0, atol=2e-3 * float(np.abs(want).max()))


def test_bf16_gemm_on_lds_staged_tiles_with_split_k_neighbours(gpu_device):
    import json
    from mononn_amd import bf16
    M, N, K = 512, 384, 512
    mb, a_dims, b_dims, d_dims = gemm_module(M=M, N=N, K=K, b_const=True, dtype="bf16")
    text = mb.text()
    rng = np.random.default_rng(6)
    a = bf16.to_bits(rng.normal(0, 1, a_dims))
    consts = {n: bf16.to_bits(rng.normal(0, 1, b_dims)) for n in mb.constants}
    want = hlo_interp.evaluate(text, [a], consts, "fp32")[0]
    for tile in (dict(m=128, n=128, k=32), dict(m=64, n=192, k=64)):
        spec = json.loads(MonoNNModule.compile(text, build=False).get_tuning_spec())
        for e in spec["gemm_spec_list"].values():
            c = e["cutlass_config"]
            c["threadblockshape"].update(tile)
            c["wave_arrangement"] = {"m": 2, "n": 2, "k": 1}
            c["stages"] = 2
        (got,), m = run_module(text, [a], consts, [{"dtype": "bf16", "dims": d_dims}], json.dumps(spec))
        assert "gemm_tile_lds<" in m.get_source("main.hip")
        m.close()
        _bf16_check(got, want, f"bf16 LDS tile {tile}", steps=1.0, atol=2e-3 * float(np.abs(want).max()))


def test_bf16_encoder_parity(gpu_device):
    # two BERT layers with embeddings and padding masks, stored and multiplied in bf16: against the oracle run as
    # written (every bf16 instruction rounded, as the kernel does) and against the unrounded fp32 evaluation
    import json
    fx = models.bert_encoder(L=2, B=2, S=64, H=256, NH=4, F=512, vocab=300, max_pos=64, mask_kind="length_mask", ftype="bf16")
    consts = fx.make_constants(27, "random")
    inputs = fx.make_inputs(27)
    (got,), m = run_module(fx.hlo_text, inputs, consts, fx.outputs)
    assert m.get_source("main.hip").count(", true>(reinterpret_cast<const half_t*>(") >= 4   # the layers share their node functions
    written = hlo_interp.evaluate(fx.hlo_text, inputs, consts, "as_written")[0]
    _bf16_check(got, written, "bf16 encoder against the oracle as written", steps=4.0, atol=3e-2)
    free = hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0]
    _bf16_check(got, free, "bf16 encoder against the fp32 evaluation", steps=8.0, atol=6e-2)
    # split-K on the second feed-forward GEMM: fp32 partial sums, added by the LayerNorm stage, rounded once
    gemms = _gemm_instr_names(fx.hlo_text)
    split = {gemms[l * 6 + 5]: {"split_k": 4} for l in range(2)}
    (got2,), m2 = run_module(fx.hlo_text, inputs, consts, fx.outputs, _spec_with(fx.hlo_text, gemm_overrides=split))
    _bf16_check(got2, written, "bf16 encoder with split-K", steps=4.0, atol=3e-2)
    # the attention as three stages (scores GEMM, soft-max, context GEMM) instead of the fused node
    assert "mononn_dev::mfma_16x16x32<true>(" in m.get_source("main.hip")
    (got3,), m3 = run_module(fx.hlo_text, inputs, consts, fx.outputs, _spec_with(fx.hlo_text, hip={"fuse_attention": False}))
    assert m3.launch_dims()["barriers"] > m.launch_dims()["barriers"]
    _bf16_check(got3, written, "bf16 encoder without attention fusion", steps=4.0, atol=3e-2)


def test_bf16_attention_with_a_key_count_off_the_mfma_step(gpu_device):
    fx = models.bert_encoder(L=1, B=2, S=48, H=128, NH=2, F=256, vocab=97, max_pos=64, mask_kind="length_mask", ftype="bf16")
    consts = fx.make_constants(28, "random")
    inputs = fx.make_inputs(28)
    (got,), m = run_module(fx.hlo_text, inputs, consts, fx.outputs)
    src = m.get_source("main.hip")
    assert "colv[" in src and "mononn_dev::mfma_16x16x32<true>(" in src
    _bf16_check(got, hlo_interp.evaluate(fx.hlo_text, inputs, consts, "as_written")[0], "bf16 encoder, 48 keys", steps=4.0, atol=3e-2)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,N,K,tile", [
    (512, 384, 256, dict(m=128, n=128, k=64)),      # 64 columns per wave: 16 lanes per row
    (500, 392, 128, dict(m=128, n=192, k=32)),      # 96 columns per wave (24 lanes per row), M and N off the tile
    (300, 1001, 128, dict(m=64, n=256, k=32)),      # 128 columns per wave, odd N: rows at 2-byte aligned addresses
    (256, 64, 512, dict(m=64, n=64, k=64)),         # 32 columns per wave
])
def test_lds_tile_epilogue_through_lds_by_rows(gpu_device, dtype, M, N, K, tile):
    # a row-major result of the LDS-staged tile passes through LDS a fragment row at a time so that the epilogue
    # (here: bias + residual) loads and stores whole rows of the wave's tile; against the oracle
    import json
    from mononn_amd import bf16
    mb = HloModuleBuilder("cluster_9__gemm_rows.1")
    e = mb.entry
    a = e.parameter(dtype, (M, K), "a")
    res = e.parameter(dtype, (M, N), "res")
    w = e.elided_constant(dtype, (K, N), "w/kernel")
    bias = e.elided_constant(dtype, (N,), "w/bias")
    d = e.gemm(a, w, 1, 0)

    def body(f, pd, pb, pr):
        return f.convert(f.add(f.add(f.convert(pd, "f32"), f.broadcast(f.convert(pb, "f32"), (M, N), [1])), f.convert(pr, "f32")), dtype)
    e.set_tuple_root([e.fusion("kLoop", [d, bias, res], body)])
    text = mb.text()
    rng = np.random.default_rng(9)
    host = (lambda v: bf16.to_bits(v)) if dtype == "bf16" else (lambda v: v.astype(np.float16))
    av, rv = host(rng.normal(0, 1, (M, K))), host(rng.normal(0, 1, (M, N)))
    consts = {n: host(rng.normal(0, 0.1 if len(meta["dims"]) == 2 else 1.0, meta["dims"])) for n, meta in mb.constants.items()}
    spec = json.loads(MonoNNModule.compile(text, build=False).get_tuning_spec())
    for g in spec["gemm_spec_list"].values():
        c = g["cutlass_config"]
        c["threadblockshape"].update(tile)
        c["wave_arrangement"] = {"m": 2, "n": 2, "k": 1}
        c["stages"] = 2
    (got,), m = run_module(text, [av, rv], consts, [{"dtype": dtype, "dims": [M, N]}], json.dumps(spec))
    src = m.get_source("main.hip")
    assert "gemm_tile_lds<" in src and re.search(r"mononn_dev::RowMajorA, (true|false), true>\(", src)
    m.close()
    want = hlo_interp.evaluate(text, [av, rv], consts, "fp32")[0]
    if dtype == "bf16":
        _bf16_check(got, want, f"bf16 {M}x{N}x{K} {tile}", steps=1.0, atol=2e-3 * float(np.abs(want).max()))
    else:
        assert np.abs(got.astype(np.float32) - want).max() <= 2e-3 * np.abs(want).max() + 1e-3
