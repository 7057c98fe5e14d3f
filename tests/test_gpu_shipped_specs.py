"""The tuned specifications shipped under mononn_amd/specs/ -- the kernels bench.py times -- against the golden
vectors (BERT-base) and against the fp32 oracle at the full size each specification was tuned for."""
import importlib.util
import os

import numpy as np
import pytest

from mononn_amd.hlo import models
from oracle import hlo_interp

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")
SPECS = os.path.join(os.path.dirname(HERE), "mononn_amd", "specs")
_spec = importlib.util.spec_from_file_location("make_golden", os.path.join(GOLDEN, "make_golden.py"))
make_golden = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(make_golden)

TOL_ABS, TOL_COS = 2e-2, 0.9999   # fp16 storage, fp32 accumulation, against an fp32 evaluation


def _tuned(fx, consts, spec_name, device):
    from mononn_amd import MonoNNModule
    spec_dir = os.path.join(SPECS, spec_name)
    assert os.path.isdir(spec_dir), f"{spec_dir} is not shipped"
    m = MonoNNModule.from_spec_dir(fx.hlo_text, spec_dir)
    m.set_constants(consts)
    m.load(device)
    return m


def _check(got, want, what):
    g, w = got.astype(np.float64).ravel(), want.astype(np.float64).ravel()
    assert g.shape == w.shape
    err = np.abs(g - w).max()
    cos = g @ w / (np.linalg.norm(g) * np.linalg.norm(w))
    print(f"{what}: max_abs_err={err:.3e} cosine={cos:.6f}", flush=True)
    assert err <= TOL_ABS and cos >= TOL_COS


def test_shipped_bert_base_spec_matches_the_golden_vectors(gpu_device):
    # the specification bench.py loads, on the seeded ids and on the reference's example feed
    fx, consts, inputs = make_golden.case_data("bert_base_b1_s128")
    m = _tuned(fx, consts, "bert_base_b1_s128", gpu_device)
    for stem in ("bert_base_b1_s128", "bert_base_b1_s128_example_feed"):
        _, _, feed = make_golden.case_data(stem)
        want = np.load(os.path.join(GOLDEN, stem + ".npy")).astype(np.float32)
        _check(m.run(feed, fx.outputs)[0], want, f"shipped spec, {stem}")
    m.close()


@pytest.mark.parametrize("spec_name,make,seed", [
    ("gpt2_b4_s512", models.gpt2, 1237),
    ("vit_b16_b8", models.vit, 1238),
    ("bert_large_b16_s384", models.bert_large, 1236),
])
def test_shipped_spec_matches_the_oracle_at_full_size(gpu_device, spec_name, make, seed):
    if not os.path.isdir(os.path.join(SPECS, spec_name)):
        pytest.skip(f"no specification shipped for {spec_name}")
    fx = make()
    consts = fx.make_constants(seed, "random")
    inputs = fx.make_inputs(seed)
    m = _tuned(fx, consts, spec_name, gpu_device)
    got = m.run(inputs, fx.outputs)[0]
    m.close()
    print(f"{spec_name}: fp32 evaluation at full size ...", flush=True)
    if spec_name.startswith("bert"):
        # 3.9 TFLOP: the NumPy interpreter needs minutes, the torch fp32 restatement behind the golden vectors seconds
        want = make_golden.torch_encoder(fx, consts, inputs)
    else:
        want = hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0]
    _check(got, want, f"shipped spec {spec_name} vs fp32 evaluation")
