"""The standalone driver that the module dump contains (best_tuning_spec_src/host_main.cpp, built by
__graft_entry__.build() into mononn_amd/bin/host_driver_example/): plain HIP, no library, same kernel, same result."""
import os
import re
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

pytestmark = pytest.mark.gpu


def test_standalone_driver_reproduces_the_library_result(gpu_device, tmp_path):
    import __graft_entry__ as entry
    from mononn_amd import MonoNNModule
    exe = os.path.join(entry.HOST_DRIVER_DIR, "host_main")
    cluster = os.path.join(entry.HOST_DRIVER_DIR, "cluster_0")
    assert os.path.exists(exe), "the standalone driver example is not built; run __graft_entry__.build()"
    fx, consts, inputs = entry.host_driver_fixture()
    m = MonoNNModule.compile(fx.hlo_text)
    m.set_constants(consts)
    m.load(gpu_device)
    want = m.run(inputs, fx.outputs)[0]
    m.close()
    out = subprocess.run([exe, os.path.join(cluster, "best_tuning_spec.hsaco"), os.path.join(cluster, "constants"), "50"],
                         cwd=tmp_path, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    assert re.search(r"mononn_cluster_0: grid \d+ x block \d+, 50 iterations, [\d.]+ us per launch", out.stdout), out.stdout
    got = np.fromfile(os.path.join(tmp_path, "liveout_0.bin"), dtype=np.float16).reshape(want.shape)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    # and both against the fp32 oracle of the same HLO and weights
    from oracle import hlo_interp
    ref = hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0].astype(np.float64).ravel()
    g = got.astype(np.float64).ravel()
    assert np.abs(g - ref).max() <= 2e-2 and g @ ref / (np.linalg.norm(g) * np.linalg.norm(ref)) >= 0.9999
