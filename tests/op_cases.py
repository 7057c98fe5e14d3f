"""HLO modules for the less common instructions (reduce-window, dynamic-update-slice, variadic reduce), shared by the
oracle's pinning tests, the host-compiler tests and the GPU parity tests."""
from mononn_amd.hlo.builder import HloModuleBuilder


def pool_module(xd, size, stride, pad, kind="max", dtype="f16", in_fusion=True):
    """N,H,W,C pooling as XLA writes it: reduce-window with a maximum (init -inf) or add (init 0) reducer."""
    mb = HloModuleBuilder("cluster_8__pool.1")
    e = mb.entry
    x = e.parameter(dtype, xd, "x")
    red = mb.reducer("maximum" if kind == "max" else "add", dtype)

    def body(f, p):
        init = f.scalar(dtype, float("-inf") if kind == "max" else 0.0)
        return f.reduce_window(p, init, size, stride, pad, red)
    out = e.fusion("kLoop", [x], body) if in_fusion else body(e, x)
    e.set_tuple_root([out])
    return mb.text(), list(out.dims)


def update_slice_module(xd, ud, dtype="f16", scale=None):
    """out = x with `update` (optionally scaled: an element-wise producer inside the fusion) written at run-time offsets."""
    mb = HloModuleBuilder("cluster_9__update_slice.1")
    e = mb.entry
    x = e.parameter(dtype, xd, "x")
    u = e.parameter(dtype, ud, "update")
    starts = [e.parameter("s32", (), f"start{i}") for i in range(len(xd))]

    def body(f, px, pu, *ps):
        if scale is not None:
            pu = f.mul(pu, f.splat(dtype, scale, ud))
        return f.dynamic_update_slice(px, pu, list(ps))
    out = e.fusion("kLoop", [x, u] + starts, body)
    e.set_tuple_root([out])
    return mb.text()


def arg_reduce_module(rows, n, direction="GT", dtype="f16", axis=1):
    """(value, index) of the largest (GT) / smallest (LT) element along `axis` of a [rows, n] (axis 1) or [n, rows]
    (axis 0) matrix, first one on ties."""
    mb = HloModuleBuilder("cluster_10__argmax.1")
    e = mb.entry
    xd = (rows, n) if axis == 1 else (n, rows)
    x = e.parameter(dtype, xd, "x")
    red = mb.arg_reducer(direction, dtype)

    def body(f, p):
        idx = f.iota("s32", xd, axis)
        init_v = f.scalar(dtype, float("-inf") if direction in ("GE", "GT") else float("inf"))
        init_i = f.scalar("s32", 0)
        return f.reduce_variadic([p, idx], [init_v, init_i], axis, red)
    vals = e.fusion("kInput", [x], body)
    e.set_tuple_root(list(vals))
    return mb.text()
