"""Seeded random fused-HLO modules for differential tests of the code generator against the oracle: chains of
element-wise ops, broadcasts, transposes, column rotations (slice + concatenate), index masks (iota + compare +
select) and row reductions, spread over one to three fusions.  Reductions and transcendental functions run in f32,
as XLA's mixed-precision rewrite leaves them; values are squashed now and then so that nothing overflows in f16."""
import numpy as np

from mononn_amd.hlo.builder import HloModuleBuilder


def random_module(seed: int):
    """Returns (hlo_text, inputs, output descriptors)."""
    rng = np.random.default_rng(seed)
    R = int(rng.choice([1, 3, 16, 37, 64, 70]))
    C = int(rng.choice([1, 5, 32, 64, 100, 257, 300, 768]))
    mb = HloModuleBuilder(f"cluster_{seed}__random_graph.1")
    e = mb.entry
    x0 = e.parameter("f16", (R, C), "x0")
    x1 = e.parameter("f16", (R, C), "x1")
    v = e.parameter("f16", (C,), "v")
    w = e.parameter("f16", (R,), "w")
    T = int(rng.choice([1, 7, 50]))
    table = e.parameter("f16", (T, C), "table")
    ids = e.parameter("s32", (R,), "ids")                 # partly out of range: row gathers clamp
    wide = e.parameter("f16", (R, C + 6), "wide")
    start = e.parameter("s32", (), "start")               # may be out of range: dynamic-slice clamps
    inputs = [rng.normal(0, 1, (R, C)).astype(np.float16), rng.normal(0, 1, (R, C)).astype(np.float16),
              rng.normal(0, 1, (C,)).astype(np.float16), rng.normal(0, 1, (R,)).astype(np.float16),
              rng.normal(0, 1, (T, C)).astype(np.float16), rng.integers(-3, T + 3, (R,)).astype(np.int32),
              rng.normal(0, 1, (R, C + 6)).astype(np.float16), np.array(int(rng.integers(-4, 12)), np.int32)]
    full = [x0, x1]          # entry-level [R, C] f16 values available to later fusions
    rows = []                # entry-level [R] f32 values
    n_fusions = int(rng.integers(1, 4))
    for fi in range(n_fusions):
        operands = list(full) + [v, w] + rows + [table, ids, wide, start]
        state = {"has_reduce": False}

        def body(f, *ps):
            pf = [f.convert(p, "f32") for p in ps[:len(full)]]
            pv = f.convert(ps[len(full)], "f32")
            pw = f.convert(ps[len(full) + 1], "f32")
            prow = list(ps[len(full) + 2:len(ps) - 4])
            ptable, pids, pwide, pstart = ps[len(ps) - 4:]
            vals = list(pf)

            def pick():
                return vals[int(rng.integers(0, len(vals)))]
            n_ops = int(rng.integers(3, 9))
            for _ in range(n_ops):
                kind = rng.choice(["binary", "unary", "rowvec", "colvec", "const", "select", "transpose", "rotate", "mask",
                                   "reduce", "rowin", "shift", "window", "gather", "dslice"])
                a = pick()
                if kind == "binary":
                    r = f.binary(str(rng.choice(["add", "subtract", "multiply", "maximum", "minimum"])), a, pick())
                elif kind == "unary":
                    op = str(rng.choice(["tanh", "negate", "abs", "exponential"]))
                    if op == "exponential":
                        a = f.binary("minimum", a, f.splat("f32", 3.0, (R, C)))
                    r = f.unary(op, a)
                elif kind == "rowvec":
                    r = f.binary(str(rng.choice(["add", "multiply"])), a, f.broadcast(pv, (R, C), [1]))
                elif kind == "colvec":
                    r = f.binary(str(rng.choice(["add", "multiply"])), a, f.broadcast(pw, (R, C), [0]))
                elif kind == "const":
                    r = f.binary(str(rng.choice(["add", "multiply"])), a, f.splat("f32", float(rng.choice([0.5, -1.25, 2.0])), (R, C)))
                elif kind == "select":
                    b = pick()
                    r = f.select(f.compare(a, b, str(rng.choice(["GT", "LE", "NE"]))), a, f.unary("negate", b))
                elif kind == "transpose":
                    t = f.transpose(a, [1, 0])
                    t = f.binary("add", t, f.broadcast(pw, (C, R), [1]))
                    r = f.transpose(t, [1, 0])
                elif kind == "rotate" and C >= 2:
                    c1 = int(rng.integers(1, C))
                    r = f.concatenate([f.slice(a, [0, c1], [R, C]), f.slice(a, [0, 0], [R, c1])], 1)
                elif kind == "shift" and C >= 2:
                    # shift the columns by k with zero fill: pad on one side, cut the other
                    k = int(rng.integers(1, min(C, 9)))
                    if rng.random() < 0.5:
                        r = f.slice(f.pad(a, f.scalar("f32", 0.0), [0, k], [0, 0]), [0, 0], [R, C])
                    else:
                        r = f.slice(f.pad(a, f.scalar("f32", 0.0), [0, 0], [0, k]), [0, k], [R, C + k])
                elif kind == "window" and C >= 3:
                    # moving maximum over three columns, same size (padding = -inf)
                    r = f.reduce_window(a, f.scalar("f32", float("-inf")), (1, 3), (1, 1), ((0, 0), (1, 1)), mb.reducer("maximum", "f32"))
                elif kind == "gather":
                    r = f.binary("add", a, f.convert(f.gather_rows(ptable, pids), "f32"))
                elif kind == "dslice":
                    zero = f.scalar("s32", 0)
                    r = f.binary("multiply", a, f.convert(f.dynamic_slice(pwide, [zero, pstart], (R, C)), "f32"))
                elif kind == "mask":
                    col = f.iota("s32", (R, C), 1)
                    lim = f.splat("s32", int(rng.integers(0, C + 1)), (R, C))
                    r = f.select(f.compare(col, lim, "LT"), a, f.splat("f32", 0.0, (R, C)))
                elif kind == "reduce":
                    which = str(rng.choice(["add", "maximum"]))
                    sq = f.unary("tanh", a)
                    init = f.scalar("f32", 0.0 if which == "add" else float("-inf"))
                    red = f.reduce(sq, init, 1, mb.reducer(which, "f32"))
                    if which == "add":
                        red = f.binary("multiply", red, f.splat("f32", 1.0 / C, (R,)))
                    r = f.binary("subtract", sq, f.broadcast(red, (R, C), [0]))
                    state["has_reduce"] = True
                elif kind == "rowin" and prow:
                    r = f.binary("add", a, f.broadcast(prow[int(rng.integers(0, len(prow)))], (R, C), [0]))
                else:
                    r = f.unary("negate", a)
                if rng.random() < 0.35:
                    r = f.unary("tanh", r)          # keep magnitudes bounded
                vals.append(r)
            out = f.convert(f.unary("tanh", vals[-1]) if rng.random() < 0.5 else f.binary("minimum", f.binary("maximum", vals[-1], f.splat("f32", -60000.0, (R, C))), f.splat("f32", 60000.0, (R, C))), "f16")
            if rng.random() < 0.4:
                # a second result: one value per row
                rr = f.reduce(f.unary("tanh", vals[-1]), f.scalar("f32", 0.0), 1, mb.reducer("add", "f32"))
                state["has_reduce"] = True
                return [out, rr]
            return out
        # the body draws from the generator, so the fusion kind is only known afterwards: build as kInput when the
        # body may reduce (a kLoop fusion must not contain a reduce root), which the parser treats alike
        res = e.fusion("kInput", operands, body)
        if isinstance(res, list):
            full.append(res[0])
            rows.append(res[1])
        else:
            full.append(res)
    outs = [full[-1]] + rows[-1:]
    e.set_tuple_root(outs)
    descs = [{"dtype": o.dtype, "dims": list(o.dims)} for o in outs]
    return mb.text(), inputs, descs


def random_gemm_cases(seed: int, count: int):
    """Seeded GEMM modules over shapes, batch ranks, operand layouts and (mostly) explicit tiles: yields
    (case dict for test_gpu_parity.gemm_module, hlo_text, specification json)."""
    import json
    from mononn_amd import MonoNNModule
    import test_gpu_parity as parity
    rng = np.random.default_rng(seed)
    for _ in range(count):
        batch = [(), (2,), (2, 3)][int(rng.integers(0, 3))]
        r = len(batch) + 2
        case = dict(M=int(rng.integers(1, 300)), N=int(rng.integers(1, 300)), K=int(rng.choice([8, 17, 32, 40, 64, 96, 100, 128, 197, 256])),
                    batch=batch, lhs_c=int(rng.choice([r - 1, r - 2])), rhs_c=int(rng.choice([r - 1, r - 2])))
        if not batch and rng.random() < 0.4:
            case.update(b_const=True, lhs_c=r - 1, rhs_c=r - 2)
        text = parity.gemm_module(**case)[0].text()
        spec = json.loads(MonoNNModule.compile(text, build=False).get_tuning_spec())
        if rng.random() < 0.7:
            c = next(iter(spec["gemm_spec_list"].values()))["cutlass_config"]
            wk = int(rng.choice([1, 2, 4]))
            wm = int(rng.choice([w for w in (1, 2, 4) if (4 // wk) % w == 0]))
            wn = 4 // wk // wm
            tm, tn = int(rng.integers(1, 5)), int(rng.integers(1, 5))
            c["threadblockshape"] = {"m": 16 * tm * wm, "n": 16 * tn * wn, "k": 32}
            c["warpshape"] = {"m": 16 * tm, "n": 16 * tn, "k": c["warpshape"]["k"]}
            c["wave_arrangement"] = {"m": wm, "n": wn, "k": wk}
        yield case, text, json.dumps(spec)


LDS_TILES = [(128, 128, 64), (128, 128, 32), (256, 128, 64), (128, 256, 32), (192, 128, 64), (192, 256, 32), (256, 256, 32), (128, 128, 128)]


def random_lds_gemm_cases(seed: int, count: int):
    """Seeded GEMM modules for the LDS-staged tile (k a multiple of 32, both operands k-contiguous or the right one a
    packed constant), ragged M / N, with and without batch dimensions: yields (case, hlo_text, specification json)."""
    import json
    from mononn_amd import MonoNNModule
    import test_gpu_parity as parity
    rng = np.random.default_rng(seed)
    for _ in range(count):
        batch = [(), (), (2,), (2, 2)][int(rng.integers(0, 4))]
        r = len(batch) + 2
        case = dict(M=int(rng.integers(1, 600)), N=int(rng.integers(1, 600)), K=int(rng.choice([32, 64, 96, 128, 160, 256, 320])),
                    batch=batch, lhs_c=r - 1, rhs_c=r - 1)
        if not batch and rng.random() < 0.5:
            case.update(b_const=True, rhs_c=r - 2)
        text = parity.gemm_module(**case)[0].text()
        spec = json.loads(MonoNNModule.compile(text, build=False).get_tuning_spec())
        bm, bn, bk = LDS_TILES[int(rng.integers(0, len(LDS_TILES)))]
        c = next(iter(spec["gemm_spec_list"].values()))["cutlass_config"]
        c["threadblockshape"] = {"m": bm, "n": bn, "k": bk}
        c["warpshape"] = {"m": bm // 2, "n": bn // 2, "k": case["K"]}
        c["wave_arrangement"] = {"m": 2, "n": 2, "k": 1}
        c["stages"] = 2
        yield case, text, json.dumps(spec)
