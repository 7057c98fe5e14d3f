"""What stands between a bad launch and a hung GPU: the co-residency check at load time, the bounded grid-barrier
wait (forced from the host: one workgroup's flag is set back so that the others can never see it arrive; every
workgroup still runs to the end of the kernel), and the store / flag ordering of the fence-free barrier under
inputs that change from launch to launch."""
import ctypes
import json
import time

import numpy as np
import pytest

from mononn_amd.hlo import models
from mononn_amd.hlo.builder import HloModuleBuilder
from oracle import hlo_interp

pytestmark = pytest.mark.gpu


def _small_encoder():
    fx = models.bert_encoder(L=1, B=1, S=32, H=128, NH=4, F=256, vocab=200, max_pos=64)
    return fx, fx.make_constants(3, "random"), fx.make_inputs(3)


def test_a_grid_that_cannot_be_resident_is_refused_at_load(gpu_device):
    from mononn_amd import MonoNNModule
    from mononn_amd.binding import MonoNNError
    fx, consts, inputs = _small_encoder()
    spec = json.loads(MonoNNModule.compile(fx.hlo_text, build=False).get_tuning_spec())
    spec["cuda_context"]["cuda_runtime_context"]["grid_dim"]["x"] = 4096      # 256 compute units hold far fewer workgroups of 256 threads
    m = MonoNNModule.compile(fx.hlo_text, json.dumps(spec))
    m.set_constants(consts)
    with pytest.raises(MonoNNError) as e:
        m.load(gpu_device)
    assert e.value.status == "RESOURCE_EXHAUSTED" and "co-resident" in str(e.value)
    with pytest.raises(MonoNNError):          # nothing was loaded, so nothing can be launched
        m.run(inputs, fx.outputs)
    m.close()


def test_a_wait_that_cannot_complete_gives_up_and_the_kernel_ends(gpu_device):
    from mononn_amd import MonoNNModule
    from mononn_amd.binding import MonoNNError
    fx, consts, inputs = _small_encoder()
    spec = json.loads(MonoNNModule.compile(fx.hlo_text, build=False).get_tuning_spec())
    spec["mononn_hip"]["barrier_timeout_ms"] = 50
    m = MonoNNModule.compile(fx.hlo_text, json.dumps(spec))
    m.set_constants(consts)
    m.load(gpu_device)
    want = hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0].astype(np.float64).ravel()

    def check_good():
        got = m.run(inputs, fx.outputs)[0].astype(np.float64).ravel()
        assert np.abs(got - want).max() <= 2e-2
    check_good()
    # Set workgroup 1's flag far back: it starts the next launch at that epoch and publishes values the other
    # workgroups' waits never accept, while its own waits pass at once.  No wait of the launch can complete.
    flags, nbytes = m.global_address("mononn_barrier_flags")
    stride = 64                                # unsigned words between the flags of consecutive workgroups
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    word = ctypes.c_uint32(0)
    assert hip.hipMemcpy(ctypes.byref(word), ctypes.c_void_p(flags + 4 * stride), 4, 2) == 0     # device to host
    back = ctypes.c_uint32((word.value - 100000) & 0xFFFFFFFF)
    assert hip.hipMemcpy(ctypes.c_void_p(flags + 4 * stride), ctypes.byref(back), 4, 1) == 0     # host to device
    t0 = time.perf_counter()
    with pytest.raises(MonoNNError) as e:
        m.run(inputs, fx.outputs)
    elapsed = time.perf_counter() - t0
    assert e.value.status == "RUNTIME_ERROR" and "grid barrier" in str(e.value)
    assert 0.04 < elapsed < 5.0, elapsed       # the budget, not a multiple of it per stage, and no hang
    # the barrier state was reset: the module works again
    check_good()
    m.close()


def test_stage_outputs_are_complete_when_the_flag_is_seen(gpu_device):
    """Three element-wise stages separated by grid barriers, each reading what other workgroups (other XCDs) wrote
    through a transpose, on integer data that differs in every launch: a store still on its way when the flag is
    published, or a line left over from the previous launch, shows up as a wrong word."""
    from mononn_amd import MonoNNModule
    R, C = 512, 768
    mb = HloModuleBuilder("cluster_7__exchange.1")
    e = mb.entry
    x = e.parameter("s32", (R, C), "x")

    def stage(mul, add):
        def body(f, p):
            t = f.transpose(p, (1, 0))
            return f.add(f.mul(t, f.splat("s32", mul, t.dims)), f.splat("s32", add, t.dims))
        return body
    a = e.fusion("kLoop", [x], stage(3, 1))          # [C, R]
    b = e.fusion("kLoop", [a], stage(5, -7))         # [R, C]
    c = e.fusion("kLoop", [b], stage(7, 11))         # [C, R]
    e.set_tuple_root([c])
    # the three fusions must stay three stages: no merging of dependent clusters into one loop nest
    spec = json.loads(MonoNNModule.compile(mb.text(), build=False).get_tuning_spec())
    spec["mononn_hip"]["merge_dependent"] = False
    spec["cluster_elewise_spec"] = {}
    m = MonoNNModule.compile(mb.text(), json.dumps(spec))
    assert m.launch_dims()["barriers"] == 2
    m.load(gpu_device)
    rng = np.random.default_rng(99)
    for launch in range(40):
        xv = rng.integers(-1000, 1000, (R, C)).astype(np.int32)
        got = m.run([xv], [{"dtype": "s32", "dims": [C, R]}])[0]
        want = (((xv.T * 3 + 1).T * 5 - 7).T * 7 + 11).astype(np.int32)
        assert np.array_equal(got, want), f"launch {launch}: {(got != want).sum()} wrong words"
    m.close()


@pytest.mark.gpu
def test_cooperative_launch_is_refused_while_a_profiler_tool_is_attached(gpu_device):
    """A process that used the cooperative launch entry point under a profiler tool died in an exit handler; the
    combination is refused at load time with a message that names the way out, and the ordinary launch is not
    affected.  (The tool is only named in the environment here: nothing is loaded.)"""
    import os
    import test_gpu_parity as parity
    from mononn_amd import MonoNNError, MonoNNModule
    mb, a_dims, b_dims, d_dims = parity.gemm_module(M=64, N=64, K=64)
    rng = np.random.default_rng(3)
    a, b = rng.normal(size=a_dims).astype(np.float16), rng.normal(size=b_dims).astype(np.float16)
    coop = MonoNNModule.compile(mb.text(), parity._spec_with(mb.text(), hip={"cooperative_launch": True}))
    plain = MonoNNModule.compile(mb.text())
    # run under a profiler itself (rocprofv3 names its tool in ROCP_TOOL_LIBRARIES), the test checks the refusal only
    under_profiler = bool(os.environ.get("HSA_TOOLS_LIB") or os.environ.get("ROCP_TOOL_LIBRARIES"))
    if not under_profiler:
        os.environ["HSA_TOOLS_LIB"] = "libsome-profiler-tool.so"
    try:
        with pytest.raises(MonoNNError, match="cooperative_launch is refused while a profiler tool"):
            coop.load(gpu_device)
        plain.load(gpu_device)
        want = plain.run([a, b], [{"dtype": "f16", "dims": d_dims}])[0]
    finally:
        if not under_profiler:
            del os.environ["HSA_TOOLS_LIB"]
    assert np.isfinite(want.astype(np.float32)).all()
    if not under_profiler:
        try:
            coop.load(gpu_device)      # without the tool the cooperative launch loads and agrees
        except MonoNNError as e:       # ... unless a tool library is mapped into this process without being named
            assert "profiler tool" in str(e)
        else:
            got = coop.run([a, b], [{"dtype": "f16", "dims": d_dims}])[0]
            assert np.array_equal(got, want)
    coop.close()
    plain.close()
