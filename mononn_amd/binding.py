"""ctypes binding of libmononn_hip.so and the host-side mirror of the reference's module API.

`MonoNNModule` / `MonoNNModuleTuner.tune` follow mononn_engine/module/mononn_module.h:31-87 and
mononn_engine/module/mononn_module_tuner.h:27-37.  All compute goes through the C ABI declared in
include/mononn_hip.h; there is no Python or CPU fallback: if the shared library is missing the
import fails, and launching without a GPU raises.
"""
from __future__ import annotations

import atexit
import ctypes
import os
import weakref
from typing import Dict, List, Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmononn_hip.so")

STATUS_NAMES = {0: "OK", 1: "INVALID_ARGUMENT", 2: "PARSE_ERROR", 3: "UNSUPPORTED", 4: "SPEC_ERROR",
                5: "COMPILE_ERROR", 6: "RUNTIME_ERROR", 7: "RESOURCE_EXHAUSTED", 8: "NOT_FOUND", 9: "INTERNAL"}


class MonoNNError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"[{STATUS_NAMES.get(code, code)}] {message}")
        self.code = code
        self.status = STATUS_NAMES.get(code, str(code))


def _load_library() -> ctypes.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is missing: build it with `make -C mononn_amd/csrc` "
                          "(or `python -c 'import __graft_entry__ as g; g.build()'`)")
    # PyTorch (used for device memory and streams) ships its own HIP runtime; two HIP runtimes in
    # one process cannot both own the GPU, so let torch's copy load first and bind to that one.
    import torch  # noqa: F401
    lib = ctypes.CDLL(LIB_PATH)
    c = ctypes
    P = c.POINTER
    lib.mononn_last_error.restype = c.c_char_p
    lib.mononn_version.restype = c.c_char_p
    lib.mononn_compile.argtypes = [c.c_char_p, c.c_size_t, c.c_char_p, c.c_char_p, c.c_int, P(c.c_void_p)]
    lib.mononn_tune.argtypes = [c.c_char_p, c.c_size_t, c.c_int, c.c_char_p, c.c_int, P(c.c_void_p)]
    lib.mononn_compile_from_spec_dir.argtypes = [c.c_char_p, c.c_size_t, c.c_char_p, P(c.c_void_p)]
    lib.mononn_module_destroy.argtypes = [c.c_void_p]
    lib.mononn_module_destroy.restype = None
    lib.mononn_module_kernel_name.argtypes = [c.c_void_p]
    lib.mononn_module_kernel_name.restype = c.c_char_p
    for fn in ("mononn_module_spec_json", "mononn_module_summary"):
        getattr(lib, fn).argtypes = [c.c_void_p, P(c.c_char_p), P(c.c_size_t)]
    lib.mononn_module_source.argtypes = [c.c_void_p, c.c_char_p, P(c.c_char_p), P(c.c_size_t)]
    lib.mononn_module_code_object.argtypes = [c.c_void_p, P(c.c_void_p), P(c.c_size_t)]
    lib.mononn_module_buffer_info.argtypes = [c.c_void_p, P(c.c_int), P(P(c.c_int64)), P(c.c_int), P(P(c.c_int64)),
                                              P(c.c_int64)]
    lib.mononn_module_launch_dims.argtypes = [c.c_void_p, P(c.c_int), P(c.c_int), P(c.c_int), P(c.c_int)]
    lib.mononn_module_regional_barriers.argtypes = [c.c_void_p, P(c.c_int)]
    lib.mononn_module_owns_temp.argtypes = [c.c_void_p]
    lib.mononn_module_num_constants.argtypes = [c.c_void_p]
    lib.mononn_module_constant_info.argtypes = [c.c_void_p, c.c_int, P(c.c_char_p), P(c.c_char_p), P(c.c_int64), P(c.c_int)]
    lib.mononn_module_set_constant.argtypes = [c.c_void_p, c.c_char_p, c.c_void_p, c.c_size_t]
    lib.mononn_module_load.argtypes = [c.c_void_p, c.c_int]
    lib.mononn_launch.argtypes = [c.c_void_p, P(c.c_void_p), c.c_size_t, c.c_void_p]
    lib.mononn_launch_static_temp.argtypes = [c.c_void_p, P(c.c_void_p), c.c_size_t, c.c_void_p]
    lib.mononn_static_temp_bytes.restype = c.c_size_t
    lib.mononn_module_synchronize.argtypes = [c.c_void_p, c.c_void_p]
    lib.mononn_module_global.argtypes = [c.c_void_p, c.c_char_p, P(c.c_void_p), P(c.c_size_t)]
    lib.mononn_time_kernel.argtypes = [c.c_void_p, P(c.c_void_p), c.c_size_t, c.c_void_p, c.c_int, c.c_int,
                                       P(c.c_float), P(c.c_float)]
    lib.mononn_module_stage_clock.argtypes = [c.c_void_p, P(c.c_uint64), c.c_size_t, P(c.c_int), P(c.c_int), P(c.c_double)]
    lib.mononn_module_stage_name.argtypes = [c.c_void_p, c.c_int]
    lib.mononn_module_stage_name.restype = c.c_char_p
    lib.mononn_module_dump.argtypes = [c.c_void_p, c.c_char_p]
    lib.mononn_device_count.restype = c.c_int
    lib.mononn_device_info.argtypes = [c.c_int, P(c.c_int), P(c.c_int), P(c.c_int), c.c_char_p, c.c_size_t]
    return lib


_lib = _load_library()

EXPORTED_SYMBOLS = [
    "mononn_last_error", "mononn_version", "mononn_compile", "mononn_tune", "mononn_compile_from_spec_dir",
    "mononn_module_destroy", "mononn_module_kernel_name", "mononn_module_spec_json", "mononn_module_source",
    "mononn_module_code_object", "mononn_module_summary", "mononn_module_buffer_info", "mononn_module_launch_dims", "mononn_module_regional_barriers", "mononn_module_owns_temp",
    "mononn_module_num_constants", "mononn_module_constant_info", "mononn_module_set_constant", "mononn_module_load",
    "mononn_launch", "mononn_launch_static_temp", "mononn_static_temp_bytes", "mononn_module_synchronize", "mononn_module_global", "mononn_time_kernel", "mononn_module_stage_clock", "mononn_module_stage_name", "mononn_module_dump", "mononn_device_count", "mononn_device_info"]


def _check(rc: int):
    if rc != 0:
        raise MonoNNError(rc, _lib.mononn_last_error().decode("utf-8", "replace"))


def device_count() -> int:
    return int(_lib.mononn_device_count())


def device_info(device: int = 0) -> dict:
    cu, ws, lds = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    arch = ctypes.create_string_buffer(64)
    _check(_lib.mononn_device_info(device, ctypes.byref(cu), ctypes.byref(ws), ctypes.byref(lds), arch, 64))
    return {"compute_units": cu.value, "wave_size": ws.value, "max_lds_per_block": lds.value,
            "arch": arch.value.decode()}


_live_modules: "weakref.WeakSet" = weakref.WeakSet()


@atexit.register
def _destroy_all_modules():
    # unload code objects while the HIP runtime is still alive (interpreter teardown order is arbitrary)
    for m in list(_live_modules):
        m.close()


class MonoNNModule:
    """One HLO module compiled into one monolithic kernel."""

    def __init__(self, handle: int):
        self._h = ctypes.c_void_p(handle)
        self._bufs = None
        self._ptr_array = None
        _live_modules.add(self)

    def close(self):
        h, self._h = getattr(self, "_h", None), None
        self._bufs = None
        if h and _lib is not None:
            _lib.mononn_module_destroy(h)

    # ---- construction ------------------------------------------------------------------------
    @classmethod
    def compile(cls, hlo_text: str, spec_json: Optional[str] = None, kernel_name: Optional[str] = None,
                build: bool = True) -> "MonoNNModule":
        """MonoNNModule(hlo, spec) + generate_code() + build_assembly()."""
        h = ctypes.c_void_p()
        t = hlo_text.encode()
        _check(_lib.mononn_compile(t, len(t), spec_json.encode() if spec_json else None,
                                   kernel_name.encode() if kernel_name else None, 1 if build else 0, ctypes.byref(h)))
        return cls(h.value)

    @classmethod
    def from_spec_dir(cls, hlo_text: str, spec_dir: Optional[str] = None) -> "MonoNNModule":
        """TF_MONONN_EXISTING_TUNING_SPEC_DIR path: no tuning, spec (and cached code object) from disk."""
        h = ctypes.c_void_p()
        t = hlo_text.encode()
        _check(_lib.mononn_compile_from_spec_dir(t, len(t), spec_dir.encode() if spec_dir else None, ctypes.byref(h)))
        return cls(h.value)

    def __del__(self):
        self.close()

    # ---- introspection -----------------------------------------------------------------------
    @property
    def kernel_name(self) -> str:
        return _lib.mononn_module_kernel_name(self._h).decode()

    def _text(self, fn, *args) -> str:
        p, n = ctypes.c_char_p(), ctypes.c_size_t()
        _check(fn(self._h, *args, ctypes.byref(p), ctypes.byref(n)))
        return ctypes.string_at(p, n.value).decode()

    def get_tuning_spec(self) -> str:
        return self._text(_lib.mononn_module_spec_json)

    def get_source(self, file: str = "main.hip") -> str:
        return self._text(_lib.mononn_module_source, file.encode())

    def summary(self) -> str:
        return self._text(_lib.mononn_module_summary)

    def get_code_object(self) -> bytes:
        p, n = ctypes.c_void_p(), ctypes.c_size_t()
        _check(_lib.mononn_module_code_object(self._h, ctypes.byref(p), ctypes.byref(n)))
        return ctypes.string_at(p, n.value)

    def buffer_info(self) -> dict:
        npar, nlo, temp = ctypes.c_int(), ctypes.c_int(), ctypes.c_int64()
        pp, lp = ctypes.POINTER(ctypes.c_int64)(), ctypes.POINTER(ctypes.c_int64)()
        _check(_lib.mononn_module_buffer_info(self._h, ctypes.byref(npar), ctypes.byref(pp), ctypes.byref(nlo),
                                              ctypes.byref(lp), ctypes.byref(temp)))
        return {"parameters": [pp[i] for i in range(npar.value)], "liveouts": [lp[i] for i in range(nlo.value)],
                "temp": temp.value}

    def launch_dims(self) -> dict:
        g, b, s, nb = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        _check(_lib.mononn_module_launch_dims(self._h, ctypes.byref(g), ctypes.byref(b), ctypes.byref(s), ctypes.byref(nb)))
        rb = ctypes.c_int()
        _check(_lib.mononn_module_regional_barriers(self._h, ctypes.byref(rb)))
        return {"grid": g.value, "block": b.value, "smem": s.value, "barriers": nb.value, "regional_barriers": rb.value}

    def constants(self) -> List[dict]:
        out = []
        for i in range(_lib.mononn_module_num_constants(self._h)):
            name, role, nbytes, need = ctypes.c_char_p(), ctypes.c_char_p(), ctypes.c_int64(), ctypes.c_int()
            _check(_lib.mononn_module_constant_info(self._h, i, ctypes.byref(name), ctypes.byref(role),
                                                    ctypes.byref(nbytes), ctypes.byref(need)))
            out.append({"name": name.value.decode(), "role": role.value.decode(), "bytes": nbytes.value,
                        "needs_payload": bool(need.value)})
        return out

    @property
    def owns_temp(self) -> bool:
        return bool(_lib.mononn_module_owns_temp(self._h))

    def dump(self, dump_dir: str):
        _check(_lib.mononn_module_dump(self._h, dump_dir.encode()))

    # ---- device side -------------------------------------------------------------------------
    def set_constant(self, name: str, array: np.ndarray):
        a = np.ascontiguousarray(array)
        _check(_lib.mononn_module_set_constant(self._h, name.encode(), a.ctypes.data_as(ctypes.c_void_p), a.nbytes))

    def set_constants(self, constants: Dict[str, np.ndarray]):
        for k, v in constants.items():
            self.set_constant(k, v)

    def load(self, device: int = 0):
        _check(_lib.mononn_module_load(self._h, device))
        self._device = device

    def launch_raw(self, device_ptrs: Sequence[int], stream: int = 0):
        arr = (ctypes.c_void_p * len(device_ptrs))(*device_ptrs)
        _check(_lib.mononn_launch(self._h, arr, len(device_ptrs), ctypes.c_void_p(stream)))

    def launch_static_temp(self, device_ptrs: Sequence[int], stream: int = 0):
        """mononn_launch_static_temp: parameters and live-outs only; the temp arena is the library's static device array."""
        arr = (ctypes.c_void_p * len(device_ptrs))(*device_ptrs)
        _check(_lib.mononn_launch_static_temp(self._h, arr, len(device_ptrs), ctypes.c_void_p(stream)))

    def synchronize(self, stream: int = 0):
        """Wait for `stream`; raises MonoNNError(RUNTIME_ERROR) when a grid-barrier wait of a launch gave up."""
        _check(_lib.mononn_module_synchronize(self._h, ctypes.c_void_p(stream)))

    def global_address(self, symbol: str):
        """(device pointer, bytes) of a module global of the loaded code object."""
        p, n = ctypes.c_void_p(), ctypes.c_size_t()
        _check(_lib.mononn_module_global(self._h, symbol.encode(), ctypes.byref(p), ctypes.byref(n)))
        return p.value, n.value

    def time_raw(self, device_ptrs: Sequence[int], stream: int = 0, warmup: int = 20, iters: int = 200):
        arr = (ctypes.c_void_p * len(device_ptrs))(*device_ptrs)
        avg = ctypes.c_float()
        each = (ctypes.c_float * iters)()
        _check(_lib.mononn_time_kernel(self._h, arr, len(device_ptrs), ctypes.c_void_p(stream), warmup, iters,
                                       ctypes.byref(avg), each))
        return float(avg.value), np.array(each[:], dtype=np.float32)

    def stage_profile(self) -> List[dict]:
        """Per-stage timing of the last launch (kernel compiled with mononn_hip.profile_stages):
        `busy_us` = first workgroup in to last workgroup done, `barrier_us` = last workgroup done to the
        first workgroup entering the next stage, `mean_wg_us` = average per-workgroup work time, `step_us` =
        last workgroup done in the previous stage to last workgroup done in this one (what the stage adds to
        the kernel's duration, whatever of its operand traffic overlaps the barrier).  Workgroups that had no
        unit in a stage leave zero stamps and are left out."""
        ns, grid, tpu = ctypes.c_int(), ctypes.c_int(), ctypes.c_double()
        _check(_lib.mononn_module_stage_clock(self._h, None, 0, ctypes.byref(ns), ctypes.byref(grid), ctypes.byref(tpu)))
        n = ns.value * grid.value * 2
        buf = (ctypes.c_uint64 * n)()
        _check(_lib.mononn_module_stage_clock(self._h, buf, n, ctypes.byref(ns), ctypes.byref(grid), ctypes.byref(tpu)))
        t = np.frombuffer(buf, dtype=np.uint64).astype(np.float64).reshape(ns.value, grid.value, 2) / tpu.value
        live = [(t[s, :, 0] > 0) & (t[s, :, 1] > 0) for s in range(ns.value)]
        begin = [t[s, live[s], 0].min() if live[s].any() else np.nan for s in range(ns.value)]
        done = [t[s, live[s], 1].max() if live[s].any() else np.nan for s in range(ns.value)]
        out = []
        for s in range(ns.value):
            nxt = begin[s + 1] if s + 1 < ns.value else done[s]
            prev = done[s - 1] if s > 0 else begin[s]
            out.append({"stage": s, "nodes": _lib.mononn_module_stage_name(self._h, s).decode(),
                        "busy_us": done[s] - begin[s], "barrier_us": nxt - done[s], "step_us": done[s] - prev,
                        "mean_wg_us": float((t[s, live[s], 1] - t[s, live[s], 0]).mean()) if live[s].any() else 0.0})
        return out

    # torch is used for device memory and streams only
    def make_buffers(self, device: int = 0):
        import torch
        info = self.buffer_info()
        dev = torch.device("cuda", device)
        bufs = {"params": [torch.zeros(max(n, 1), dtype=torch.uint8, device=dev) for n in info["parameters"]],
                "liveouts": [torch.zeros(max(n, 1), dtype=torch.uint8, device=dev) for n in info["liveouts"]],
                "temp": None if self.owns_temp else torch.zeros(max(info["temp"], 256), dtype=torch.uint8, device=dev)}
        self._bufs = bufs
        return bufs

    def buffer_pointers(self) -> List[int]:
        b = self._bufs
        temp = 0 if b["temp"] is None else b["temp"].data_ptr()
        return [t.data_ptr() for t in b["params"]] + [t.data_ptr() for t in b["liveouts"]] + [temp]

    def run(self, inputs: Sequence[np.ndarray], out_dtypes_dims: Sequence[dict]) -> List[np.ndarray]:
        """Copy `inputs` to the GPU, launch once on torch's current stream, return live-outs as NumPy."""
        import torch
        if self._bufs is None:
            self.make_buffers(getattr(self, "_device", 0))
        b = self._bufs
        assert len(inputs) == len(b["params"]), "wrong number of entry parameters"
        for t, a in zip(b["params"], inputs):
            a = np.ascontiguousarray(a)
            assert a.nbytes == t.numel(), f"parameter needs {t.numel()} bytes, got {a.nbytes}"
            t.copy_(torch.from_numpy(a.view(np.uint8).reshape(-1)))
        stream = torch.cuda.current_stream().cuda_stream
        self.launch_raw(self.buffer_pointers(), stream)
        self.synchronize(stream)
        outs = []
        # bf16 results come back as their uint16 bit patterns (NumPy has no bfloat16; mononn_amd.bf16 converts)
        npdt = {"f16": np.float16, "bf16": np.uint16, "f32": np.float32, "s32": np.int32, "pred": np.bool_, "s64": np.int64, "u8": np.uint8, "s8": np.int8}
        for t, o in zip(b["liveouts"], out_dtypes_dims):
            outs.append(t.cpu().numpy().view(npdt[o["dtype"]]).reshape(o["dims"]).copy())
        return outs


class MonoNNModuleTuner:
    """MonoNNModuleTuner::tune: search the tuning space on the GPU, return the best module."""

    @staticmethod
    def tune(hlo_text: str, device: int = 0, dump_dir: Optional[str] = None, budget: int = 0) -> MonoNNModule:
        h = ctypes.c_void_p()
        t = hlo_text.encode()
        _check(_lib.mononn_tune(t, len(t), device, dump_dir.encode() if dump_dir else None, budget, ctypes.byref(h)))
        return MonoNNModule(h.value)
