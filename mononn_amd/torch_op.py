"""PyTorch front end over the C ABI: run a compiled module directly on ROCm tensors.

The reference's README suggests loading the dumped kernel "from PyTorch" (README.md:183); this is that hook.
`MonoNNFunction` wraps a loaded `MonoNNModule`: inputs and outputs are torch tensors on the GPU (no copies, the
launch goes onto torch's current stream), and the call is also registered as the custom operator
`mononn::forward(int handle, Tensor[] inputs) -> Tensor[]` so that it can sit inside a torch program or be A/B-timed
against `torch.nn.functional` on the same device.

torch is used for device memory and the stream only; all arithmetic happens in the generated HIP kernel.
"""
from __future__ import annotations

from typing import Dict, List, Sequence

import torch

from .binding import MonoNNModule

_TORCH_DTYPE = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32, "s32": torch.int32, "s64": torch.int64, "pred": torch.bool,
                "u8": torch.uint8, "s8": torch.int8}
_REGISTRY: Dict[int, "MonoNNFunction"] = {}


class MonoNNFunction:
    """Callable view of a module whose constants are uploaded and which is loaded on `device`."""

    def __init__(self, module: MonoNNModule, outputs: Sequence[dict], device: int = 0, checked: bool = False):
        """`checked`: every call waits for its launch through mononn_module_synchronize and raises when a grid-barrier
        wait gave up (the outputs are then invalid).  Unchecked calls stay asynchronous on torch's current stream, and
        such a failure only shows in the caller's next MonoNNModule.synchronize()."""
        self.module = module
        self.checked = checked
        self.outputs = list(outputs)
        self.device = torch.device("cuda", device)
        info = module.buffer_info()
        self._param_bytes = info["parameters"]
        self._out_bytes = info["liveouts"]
        assert len(self._out_bytes) == len(self.outputs), "one {dtype, dims} entry per live-out is required"
        self._temp = None if module.owns_temp else torch.zeros(max(info["temp"], 256), dtype=torch.uint8, device=self.device)
        self.handle = id(self)
        _REGISTRY[self.handle] = self

    def close(self):
        _REGISTRY.pop(self.handle, None)

    def __call__(self, *inputs: torch.Tensor) -> List[torch.Tensor]:
        assert len(inputs) == len(self._param_bytes), f"expected {len(self._param_bytes)} tensors"
        held = []
        ptrs = []
        for t, nbytes in zip(inputs, self._param_bytes):
            assert t.is_cuda and t.device == self.device, "inputs must live on the module's GPU"
            t = t.contiguous()
            assert t.numel() * t.element_size() == nbytes, f"parameter needs {nbytes} bytes, got {t.numel() * t.element_size()}"
            assert t.data_ptr() % 16 == 0, "buffers must be 16-byte aligned"
            held.append(t)
            ptrs.append(t.data_ptr())
        outs = []
        for o, nbytes in zip(self.outputs, self._out_bytes):
            t = torch.empty(o["dims"], dtype=_TORCH_DTYPE[o["dtype"]], device=self.device)
            assert t.numel() * t.element_size() == nbytes
            outs.append(t)
            ptrs.append(t.data_ptr())
        ptrs.append(0 if self._temp is None else self._temp.data_ptr())
        stream = torch.cuda.current_stream(self.device).cuda_stream
        self.module.launch_raw(ptrs, stream)
        if self.checked:
            self.module.synchronize(stream)
        return outs


@torch.library.custom_op("mononn::forward", mutates_args=())
def _forward(handle: int, inputs: Sequence[torch.Tensor]) -> List[torch.Tensor]:
    return _REGISTRY[handle](*inputs)


@_forward.register_fake
def _(handle: int, inputs: Sequence[torch.Tensor]) -> List[torch.Tensor]:
    fn = _REGISTRY[handle]
    return [torch.empty(o["dims"], dtype=_TORCH_DTYPE[o["dtype"]], device=fn.device) for o in fn.outputs]


def forward(fn: MonoNNFunction, *inputs: torch.Tensor) -> List[torch.Tensor]:
    """torch.ops.mononn.forward on a MonoNNFunction."""
    return torch.ops.mononn.forward(fn.handle, list(inputs))
