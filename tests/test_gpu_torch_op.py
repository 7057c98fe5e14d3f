"""The PyTorch front end (mononn_amd/torch_op.py): same kernel, torch tensors as buffers, torch's current stream."""
import numpy as np
import pytest

from mononn_amd.hlo import models
from oracle import hlo_interp

pytestmark = pytest.mark.gpu


def test_custom_op_matches_the_ctypes_path_bit_for_bit(gpu_device):
    import torch
    from mononn_amd import MonoNNModule
    from mononn_amd import torch_op
    fx = models.bert_encoder(L=2, B=1, S=64, H=256, NH=4, F=512, vocab=300, max_pos=64)
    consts = fx.make_constants(31, "random")
    inputs = fx.make_inputs(31)
    m = MonoNNModule.compile(fx.hlo_text)
    m.set_constants(consts)
    m.load(gpu_device)
    want = m.run(inputs, fx.outputs)[0]
    fn = torch_op.MonoNNFunction(m, fx.outputs, gpu_device)
    dev = torch.device("cuda", gpu_device)
    tin = [torch.from_numpy(a).to(dev) for a in inputs]
    (got,) = torch_op.forward(fn, *tin)
    assert got.dtype == torch.float16 and tuple(got.shape) == tuple(fx.outputs[0]["dims"])
    assert np.array_equal(got.cpu().numpy().view(np.uint16), want.view(np.uint16))
    # the operator's result against the fp32 oracle of the same HLO and weights
    from oracle import hlo_interp
    ref = hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0].astype(np.float64).ravel()
    g = got.cpu().numpy().astype(np.float64).ravel()
    assert np.abs(g - ref).max() <= 2e-2 and g @ ref / (np.linalg.norm(g) * np.linalg.norm(ref)) >= 0.9999
    # on a side stream, ordered after work that torch queued there
    side = torch.cuda.Stream(device=dev)
    with torch.cuda.stream(side):
        ids2 = (tin[0] + 1) % 300
        (got2,) = torch.ops.mononn.forward(fn.handle, [ids2, tin[1], tin[2]])
        back = (ids2 - 1) % 300
        (got3,) = torch.ops.mononn.forward(fn.handle, [back, tin[1], tin[2]])
    side.synchronize()
    assert not np.array_equal(got2.cpu().numpy(), want)
    assert np.array_equal(got3.cpu().numpy().view(np.uint16), want.view(np.uint16))
    with pytest.raises(AssertionError):
        fn(tin[0][:, :32], tin[1], tin[2])          # wrong size is refused before anything is launched
    fn.close()
    # checked mode: every call waits for its launch and would raise on a barrier wait that gave up
    checked = torch_op.MonoNNFunction(m, fx.outputs, gpu_device, checked=True)
    (got4,) = torch_op.forward(checked, *tin)
    assert np.array_equal(got4.cpu().numpy().view(np.uint16), want.view(np.uint16))
    checked.close()
    m.close()


def test_custom_op_with_bfloat16_tensors(gpu_device):
    # a bf16 module through the operator: torch.bfloat16 results, the same bits as the ctypes path hands back as uint16,
    # and against torch's own bf16 GEMM + bias on the same operands
    import torch
    from mononn_amd import MonoNNModule, bf16, torch_op
    from mononn_amd.hlo.builder import HloModuleBuilder
    M, K, N = 256, 512, 384
    mb = HloModuleBuilder("cluster_4__bf16_op.1")
    e = mb.entry
    a = e.parameter("bf16", (M, K), "a")
    w = e.elided_constant("bf16", (K, N), "w/kernel")
    bias = e.elided_constant("bf16", (N,), "w/bias")
    d = e.gemm(a, w, 1, 0)

    def body(f, pd, pb):
        return f.convert(f.add(f.convert(pd, "f32"), f.broadcast(f.convert(pb, "f32"), (M, N), [1])), "bf16")
    e.set_tuple_root([e.fusion("kLoop", [d, bias], body)])
    rng = np.random.default_rng(41)
    av = rng.normal(0, 1, (M, K)).astype(np.float32)
    consts = {n: bf16.to_bits(rng.normal(0, 0.1 if len(meta["dims"]) == 2 else 1.0, meta["dims"])) for n, meta in mb.constants.items()}
    outputs = [{"dtype": "bf16", "dims": [M, N]}]
    m = MonoNNModule.compile(mb.text())
    m.set_constants(consts)
    m.load(gpu_device)
    want_bits = m.run([bf16.to_bits(av)], outputs)[0]
    fn = torch_op.MonoNNFunction(m, outputs, gpu_device)
    dev = torch.device("cuda", gpu_device)
    ta = torch.from_numpy(av).to(dev).to(torch.bfloat16)
    (got,) = torch_op.forward(fn, ta)
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == (M, N)
    assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), want_bits)
    by_name = {meta["role"]: torch.from_numpy(consts[n].view(np.int16)).view(torch.bfloat16).to(dev) for n, meta in mb.constants.items()}
    # the HLO rounds twice: the GEMM's result is bf16, and so is the sum with the bias
    d = (ta.float() @ by_name["w/kernel"].float()).to(torch.bfloat16).float()
    ref = (d + by_name["w/bias"].float()).to(torch.bfloat16).float().cpu().numpy()
    g = got.float().cpu().numpy()
    spacing = 2.0 ** -7 * np.maximum(np.abs(ref), np.abs(d.cpu().numpy()))      # a bf16 step at the larger of the two magnitudes
    assert (np.abs(g - ref) <= spacing + 1e-6).all() and (g == ref).mean() > 0.9
    fn.close()
    m.close()


def test_perf_report_lists_every_stage(gpu_device, tmp_path):
    # the per-node report (perf dumper counterpart) of a small encoder: one row per stage, times positive
    import csv
    from mononn_amd import perf_report
    fx = models.bert_encoder(L=2, B=1, S=64, H=256, NH=4, F=512, vocab=300, max_pos=64)
    consts, inputs, details = fx.make_constants(5, "random"), fx.make_inputs(5), {}
    rows = perf_report.stage_report(fx.hlo_text, consts, inputs, fx.outputs, launches=20, device=gpu_device, details=details)
    assert len(rows) == 15 and [r["stage"] for r in rows] == list(range(15))
    # the profiled build computes what the module computes (mononn_module_tuner.cc:422-448 reports on the kernel it runs) ...
    want = hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0].astype(np.float64).ravel()
    got = details["outputs"][0].astype(np.float64).ravel()
    assert np.abs(got - want).max() <= 2e-2 and got @ want / (np.linalg.norm(got) * np.linalg.norm(want)) >= 0.9999
    # ... and its steps add up to that kernel: first workgroup in to last workgroup out, against the event-timed launch
    # period of the same build (which also holds the launch itself and the kernel's first and last instructions)
    steps = sum(r["step_us"] for r in rows)
    print(f"sum of steps {steps:.1f} us, event-timed kernel {details['kernel_us']:.1f} us", flush=True)
    assert 0.80 * details["kernel_us"] <= steps <= 1.02 * details["kernel_us"], (steps, details["kernel_us"])
    assert all(r["busy_us"] > 0 and r["mean_wg_us"] > 0 and r["step_us"] > 0 for r in rows)
    assert all(r["barrier_us"] > 0 for r in rows[:-1])
    assert any("cublas_gemm" in r["nodes"] for r in rows)
    hlo = tmp_path / "m.hlo"
    hlo.write_text(fx.hlo_text)
    out = tmp_path / "report.csv"
    perf_report.main(["--hlo", str(hlo), "--csv", str(out), "--launches", "3"])
    table = list(csv.reader(open(out)))
    assert table[0] == ["stage", "busy_us", "mean_workgroup_us", "barrier_us", "step_us", "nodes"] and len(table) == 16
