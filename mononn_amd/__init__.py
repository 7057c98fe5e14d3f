"""mononn_amd: MI355X-native monolithic-kernel backend with MonoNN's module API.

Host compiler and C ABI live in `csrc/` (built into `lib/libmononn_hip.so`); `binding` is the
ctypes mirror of the reference's MonoNNModule / MonoNNModuleTuner; `hlo` holds the HLO fixtures of
the measured models.
"""
from .binding import MonoNNError, MonoNNModule, MonoNNModuleTuner, device_count, device_info  # noqa: F401
