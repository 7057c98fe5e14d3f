"""mononn_launch_static_temp: the launch path for callers that cannot allocate device memory.  Two calls in a row
through the C ABI -- a larger module first, then a smaller one, both sharing the library's static temp arena --
each checked bit for bit against mononn_launch of the same module with a caller-provided temp buffer, plus the
refusal of a module whose temp arena does not fit."""
import numpy as np
import pytest

from mononn_amd.hlo import models

pytestmark = pytest.mark.gpu


def _module(fx, seed, device):
    from mononn_amd import MonoNNModule
    m = MonoNNModule.compile(fx.hlo_text)
    m.set_constants(fx.make_constants(seed, "random"))
    m.load(device)
    return m


def _both_ways(m, fx, inputs, device):
    import torch
    want = m.run(inputs, fx.outputs)[0]                       # mononn_launch, temp buffer from the caller
    bufs = m._bufs
    for t in bufs["liveouts"]:
        t.zero_()
    torch.cuda.synchronize()
    ptrs = [t.data_ptr() for t in bufs["params"]] + [t.data_ptr() for t in bufs["liveouts"]]
    stream = torch.cuda.current_stream().cuda_stream
    # what the entry point exists for: the call takes no device memory (the driver's count of free bytes on the GPU
    # is the same before the launch and after it has finished)
    free_before, _ = torch.cuda.mem_get_info(device)
    m.launch_static_temp(ptrs, stream)                        # no temp slot: the library's static arena
    m.synchronize(stream)
    free_after, _ = torch.cuda.mem_get_info(device)
    assert free_after == free_before, f"launch_static_temp changed the free device memory by {free_before - free_after} bytes"
    got = bufs["liveouts"][0].cpu().numpy().view(np.float16).reshape(fx.outputs[0]["dims"])
    return got, want


def test_static_temp_launch_matches_the_ordinary_launch_twice_in_a_row(gpu_device):
    from mononn_amd import binding
    big = models.bert_encoder(L=2, B=2, S=128, H=256, NH=4, F=1024, vocab=1000, max_pos=128)
    small = models.bert_encoder(L=1, B=1, S=32, H=128, NH=4, F=256, vocab=200, max_pos=64)
    mb, ms = _module(big, 51, gpu_device), _module(small, 52, gpu_device)
    assert 0 < ms.buffer_info()["temp"] < mb.buffer_info()["temp"] <= binding._lib.mononn_static_temp_bytes()
    got, want = _both_ways(mb, big, big.make_inputs(51), gpu_device)
    assert np.isfinite(want.astype(np.float32)).all() and np.abs(want.astype(np.float32)).max() > 0.1
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    # second call, smaller input: the arena still holds the first call's intermediates
    got, want = _both_ways(ms, small, small.make_inputs(52), gpu_device)
    assert np.abs(want.astype(np.float32)).max() > 0.1
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    # and the first module again, with other inputs
    got, want = _both_ways(mb, big, big.make_inputs(53), gpu_device)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    mb.close()
    ms.close()


def test_static_temp_launch_refuses_a_temp_arena_beyond_its_size(gpu_device):
    import torch
    from mononn_amd import binding
    from mononn_amd.binding import MonoNNError
    fx = models.bert_encoder(L=4, B=8, S=384, H=1024, NH=16, F=4096, vocab=1000, max_pos=384)
    m = _module(fx, 54, gpu_device)
    assert m.buffer_info()["temp"] > binding._lib.mononn_static_temp_bytes()
    bufs = m.make_buffers(gpu_device)
    ptrs = [t.data_ptr() for t in bufs["params"]] + [t.data_ptr() for t in bufs["liveouts"]]
    with pytest.raises(MonoNNError) as e:
        m.launch_static_temp(ptrs, torch.cuda.current_stream().cuda_stream)
    assert e.value.status == "RESOURCE_EXHAUSTED" and "static arena" in str(e.value)
    with pytest.raises(MonoNNError) as e:                     # wrong count: the temp slot is not the caller's to pass
        m.launch_static_temp(ptrs + [bufs["temp"].data_ptr()], 0)
    assert e.value.status == "INVALID_ARGUMENT"
    m.close()
