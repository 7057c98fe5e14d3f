"""CPU oracle: a NumPy evaluator for the fused-HLO dialect MonoNN consumes.

TEST INFRASTRUCTURE ONLY.  Nothing in the product (`mononn_amd/`, the C-ABI library) may import
this file; it is the checker used by `tests/`, `__graft_entry__.smoke()` and the `cpu_baseline`
leg of `bench.py`.

The reference has no CPU execution path of its own and cannot be built here (it needs its
TensorFlow and CUTLASS forks, both absent), so this is a restatement of the *semantics* the
reference attaches to each instruction when it lowers it:

  * opcode set ......................... mononn_engine/core/op/op_type.h:20-65
  * dtype / layout rules ............... mononn_engine/parser/ir_parser_fused.cc:68-152
    (a value with minor_to_major m lies in memory with dimension m[0] varying fastest; entry
    parameters, constant payloads and results are such memory images, `bitcast` keeps the bytes,
    every other instruction is defined on logical indices)
  * fusion -> called computation ....... ir_parser_fused.cc:490-539, :866-1019
  * reduce (one reduced dim, constant
    init, reducer = called computation)  ir_parser_fused.cc:1169-1213,
                                          mononn_engine/codegen/reduction_functor_generator.cc:224-294
  * broadcast/transpose/slice/pad/
    concatenate/gather/dynamic-slice/
    reduce-window index maps ........... mononn_engine/core/context/index_tracer.cc:67-456
  * reduce-window (operand + init, no
    dilation), dynamic-update-slice,
    variadic (value, index) reduce ..... ir_parser_fused.cc:1215-1262, :973-978, :1169-1213,
                                          reduction_functor_generator.cc:246-283
  * row gather ......................... index_tracer.cc:235-280
  * element-wise op -> functor ......... mononn_engine/core/gpu/functor.cc:42-88, :145-168
  * __cublas$gemm backend_config ....... mononn_engine/core/op_impl/gemm_impl.cc:182-231, :233-499
    (D = alpha * A.B + beta * C, fp32 accumulation, batch = leading dims)

The parser below is written independently of the product's C++ parser so that a parsing bug is
not shared between the thing under test and its checker.

Pinning (what fixes these functions besides the formulae above): tests/test_layouts.py checks the
layout handling against element offsets computed from strides by brute force, np.transpose and
np.einsum; tests/test_oracle_pinning.py
checks the evaluator against closed forms and library routines -- fp64 triple-loop GEMM on tiny
shapes, the two worked backend_config examples of gemm_impl.cc:290-316 against numpy einsum,
torch.nn.functional soft-max / layer_norm / gelu(tanh), brute-force gather, torch max/avg
pooling for reduce-window, NumPy slice assignment for dynamic-update-slice, np.argmax/argmin for
the variadic reduce, and a whole BERT layer against an independent torch restatement;
tests/test_oracle_pinning_ops.py checks the remaining branches on hand-written HLO text against
plain Python arithmetic and brute-force loops: integer divide (truncation toward zero), convert
(float -> int truncation, int -> half rounding and overflow), power / log / negate / abs / sign /
sqrt / exponential, the six compare directions, select, clamp, and / or / not, maximum / minimum,
dynamic-slice with clamped starts, pad (low / high / value), slice + concatenate + broadcast + iota +
transpose, and reduce with add / maximum / minimum / multiply / and / or reducers over the last and
over another dimension.  Bit-level results of the CUDA build (CUTLASS
accumulation order, -use_fast_math intrinsics) are not reproducible offline: parity unpinned at
that level; the north-star tolerance is defined against fp32 evaluation, which this is.

Reduce init values are used as the HLO writes them (XLA semantics).  The reference replaces an
infinite init by the type's finite extreme (ir_parser_fused.cc:182-204: -inf -> -65504 for f16,
-FLT_MAX for f32); the two readings differ only for a row that holds nothing but values beyond that
extreme (e.g. a maximum over a row of -inf gives -inf here, -65504 there).  The HIP kernels follow
the HLO as written, like this file; tests/test_oracle_pinning_ops.py pins that case.

precision="as_written": every f16-typed instruction result is rounded to IEEE half (what the
HLO says).  precision="fp32": f16 is carried as float32 without rounding (the "fp32 reference"
the tolerance max-abs-err <= 2e-2 / cosine >= 0.9999 is stated against).

bf16 (not a type of the reference; the HIP path adds it): carried as float32, rounded to nearest
even on the upper 16 bits of the pattern after every bf16-typed instruction in as_written mode,
handed in as uint16 bit patterns and returned as float32 values.  Pinned against torch.bfloat16
(conversions bit for bit including ties, infinities and NaN; a GEMM + element-wise program) in
tests/test_oracle_pinning.py.
"""
from __future__ import annotations

import json
import re
from typing import Dict, List, Optional, Sequence

import numpy as np

_NP = {"pred": np.bool_, "s8": np.int8, "u8": np.uint8, "s16": np.int16, "u16": np.uint16,
       "s32": np.int32, "u32": np.uint32, "s64": np.int64, "u64": np.uint64,
       "f16": np.float16, "f32": np.float32, "f64": np.float64,
       # NumPy has no bfloat16: bf16 values are carried as float32 and rounded to bf16 after every bf16-typed
       # instruction (round_to_bf16); host buffers of that type are uint16 bit patterns (bf16_from_bits)
       "bf16": np.float32}


def bf16_from_bits(bits) -> np.ndarray:
    """bf16 bit patterns (uint16) -> their values as float32: bf16 is the upper half of the f32 pattern."""
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def bf16_to_bits(values) -> np.ndarray:
    """float32 values -> bf16 bit patterns, round to nearest, ties to even, on the 16 bits that are dropped
    (what v_cvt_pk_bf16_f32 and XLA's convert do); NaN stays a quiet NaN."""
    u = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32)
    rounded = ((u + np.uint32(0x7FFF) + ((u >> 16) & np.uint32(1))) >> 16).astype(np.uint16)
    nan = np.isnan(np.asarray(values, dtype=np.float32))
    return np.where(nan, ((u >> 16) | np.uint32(0x40)).astype(np.uint16), rounded)


def round_to_bf16(values) -> np.ndarray:
    return bf16_from_bits(bf16_to_bits(values)).reshape(np.shape(values))


class Shape:
    __slots__ = ("dtype", "dims", "tuple_shapes", "layout")

    def __init__(self, dtype=None, dims=(), tuple_shapes=None, layout=None):
        self.dtype, self.dims, self.tuple_shapes = dtype, tuple(dims), tuple_shapes
        self.layout = layout     # minor-to-major list as written, None when descending (row-major)

    def major_to_minor(self):
        """Logical dimension numbers from the slowest-varying to the fastest-varying one in memory."""
        return list(range(len(self.dims))) if self.layout is None else list(reversed(self.layout))

    def memory_dims(self):
        return tuple(self.dims[d] for d in self.major_to_minor())


def _memory_image(a: np.ndarray, shape: "Shape") -> np.ndarray:
    """The value's elements in the order they lie in memory, as a row-major array of shape.memory_dims()."""
    return np.ascontiguousarray(np.transpose(a, shape.major_to_minor()))


def _from_memory(buf: np.ndarray, shape: "Shape") -> np.ndarray:
    """Inverse of _memory_image: logical array from its memory image (any shape with the right element count)."""
    order = shape.major_to_minor()
    return np.transpose(np.ascontiguousarray(buf).reshape(shape.memory_dims()), np.argsort(order))


class Instr:
    __slots__ = ("name", "shape", "opcode", "operands", "attrs", "literal", "is_root")


class Comp:
    def __init__(self, name):
        self.name = name
        self.instrs: List[Instr] = []
        self.root: Optional[Instr] = None


# ------------------------------------------------------------------------------------------
# text -> structures
# ------------------------------------------------------------------------------------------
def _split_top(s: str, sep: str = ",") -> List[str]:
    """Split on `sep` outside (), {}, [] and double-quoted strings."""
    out, depth, cur, i, in_q = [], 0, [], 0, False
    while i < len(s):
        c = s[i]
        if in_q:
            cur.append(c)
            if c == "\\" and i + 1 < len(s):
                cur.append(s[i + 1])
                i += 1
            elif c == '"':
                in_q = False
        elif c == '"':
            in_q = True
            cur.append(c)
        elif c in "({[":
            depth += 1
            cur.append(c)
        elif c in ")}]":
            depth -= 1
            cur.append(c)
        elif c == sep and depth == 0:
            out.append("".join(cur).strip())
            cur = []
        else:
            cur.append(c)
        i += 1
    tail = "".join(cur).strip()
    if tail:
        out.append(tail)
    return out


def _parse_shape(s: str) -> Shape:
    s = s.strip()
    if s.startswith("("):
        inner = s[1:s.rindex(")")]
        return Shape(tuple_shapes=[_parse_shape(p) for p in _split_top(inner)])
    m = re.match(r"([a-z]+\d*)\[([^\]]*)\](\{[^}]*\})?", s)
    if not m:
        raise ValueError(f"bad shape: {s!r}")
    dims = [int(d) for d in m.group(2).split(",") if d.strip()]
    layout = None
    if m.group(3):
        if ":" in m.group(3):
            raise ValueError(f"tiled or annotated layouts are not supported: {s}")
        lay = [int(x) for x in m.group(3)[1:-1].split(",") if x.strip()]
        if sorted(lay) != list(range(len(dims))):
            raise ValueError(f"layout is not a permutation of the dimensions: {s}")
        if lay != list(reversed(range(len(dims)))):
            layout = lay
    return Shape(m.group(1), dims, layout=layout)


def _match_paren(s: str, start: int) -> int:
    depth, i, in_q = 0, start, False
    while i < len(s):
        c = s[i]
        if in_q:
            if c == "\\":
                i += 1
            elif c == '"':
                in_q = False
        elif c == '"':
            in_q = True
        elif c in "({[":
            depth += 1
        elif c in ")}]":
            depth -= 1
            if depth == 0:
                return i
        i += 1
    raise ValueError("unbalanced parentheses")


def _parse_instr(line: str) -> Instr:
    ins = Instr()
    line = line.strip()
    ins.is_root = line.startswith("ROOT ")
    if ins.is_root:
        line = line[5:].strip()
    name, rest = line.split("=", 1)
    ins.name = name.strip().lstrip("%")
    rest = rest.strip()
    # shape: either a tuple "(...)" or token up to the first space
    if rest.startswith("("):
        end = _match_paren(rest, 0)
        shape_s, rest = rest[:end + 1], rest[end + 1:].strip()
    else:
        shape_s, rest = rest.split(" ", 1)
    ins.shape = _parse_shape(shape_s)
    p = rest.index("(")
    ins.opcode = rest[:p].strip()
    end = _match_paren(rest, p)
    body = rest[p + 1:end]
    tail = rest[end + 1:].strip()
    ins.literal = None
    ins.operands = []
    if ins.opcode in ("constant", "parameter"):
        ins.literal = body.strip()
    else:
        for o in _split_top(body):
            ins.operands.append(o.split()[-1].lstrip("%"))
    ins.attrs = {}
    if tail.startswith(","):
        for a in _split_top(tail[1:]):
            if "=" in a:
                k, v = a.split("=", 1)
                ins.attrs[k.strip()] = v.strip()
    return ins


def parse_module(text: str) -> Dict[str, object]:
    comps: Dict[str, Comp] = {}
    entry = None
    cur = None
    mod_name = None
    for raw in text.splitlines():
        line = raw.strip()
        if not line or line.startswith("//"):
            continue
        if line.startswith("HloModule"):
            mod_name = line.split()[1].rstrip(",")
            continue
        if cur is None:
            if line.endswith("{"):
                is_entry = line.startswith("ENTRY")
                head = line[5:].strip() if is_entry else line
                cname = re.split(r"[\s({]", head.lstrip("%"), 1)[0]
                cur = Comp(cname)
                if is_entry:
                    entry = cur
            continue
        if line == "}":
            if cur.root is None and cur.instrs:
                cur.root = cur.instrs[-1]
            comps[cur.name] = cur
            cur = None
            continue
        ins = _parse_instr(line)
        cur.instrs.append(ins)
        if ins.is_root:
            cur.root = ins
    if entry is None:
        raise ValueError("no ENTRY computation")
    return {"name": mod_name, "comps": comps, "entry": entry}


# ------------------------------------------------------------------------------------------
# evaluation
# ------------------------------------------------------------------------------------------
def _ints(attr: str) -> List[int]:
    return [int(x) for x in re.findall(r"-?\d+", attr)]


def _parse_literal(lit: str, dtype, dims):
    body = lit.replace("{", " ").replace("}", " ").replace(",", " ").split()
    conv = {"true": 1, "false": 0, "inf": np.inf, "-inf": -np.inf, "nan": np.nan}
    vals = [conv[t] if t in conv else float(t) if np.issubdtype(dtype, np.floating) else int(t)
            for t in body]
    with np.errstate(over="ignore"):
        return np.array(vals, dtype=np.float64 if np.issubdtype(dtype, np.floating) else np.int64
                        ).astype(dtype).reshape(dims)


_UNARY = {
    "abs": np.abs, "negate": np.negative, "exponential": np.exp, "log": np.log, "tanh": np.tanh,
    "sqrt": np.sqrt, "sign": np.sign, "not": np.logical_not, "copy": lambda x: x,
    "rsqrt": lambda x: (1.0 / np.sqrt(x)).astype(x.dtype),
}
_BINARY = {
    "add": np.add, "subtract": np.subtract, "multiply": np.multiply, "maximum": np.maximum,
    "minimum": np.minimum, "and": np.logical_and, "or": np.logical_or,
}
_CMP = {"EQ": np.equal, "NE": np.not_equal, "LT": np.less, "LE": np.less_equal,
        "GT": np.greater, "GE": np.greater_equal}
_REDUCERS = {"add": np.add, "maximum": np.maximum, "minimum": np.minimum, "multiply": np.multiply,
             "and": np.logical_and, "or": np.logical_or}


class Evaluator:
    def __init__(self, text: str, constants: Optional[Dict[str, np.ndarray]] = None,
                 precision: str = "as_written"):
        assert precision in ("as_written", "fp32")
        self.mod = parse_module(text)
        self.constants = constants or {}
        self.fp32 = precision == "fp32"
        self.trace: Dict[str, np.ndarray] = {}
        self._vector_depth = 0

    def np_dtype(self, hlo_dtype: str):
        if self.fp32 and hlo_dtype == "f16":
            return np.float32
        return _NP[hlo_dtype]

    def run(self, params: Sequence[np.ndarray], keep_trace: bool = False):
        self._keep = keep_trace
        res = self._run_comp(self.mod["entry"], list(params), top=True)
        return list(res) if isinstance(res, tuple) else [res]

    def _cast_in(self, a: np.ndarray, shape: Shape) -> np.ndarray:
        """A buffer handed in by the host (entry parameter, constant payload): its memory image, dims listed from the
        slowest-varying one; with the default layout that is the logical array itself."""
        a = np.asarray(a)
        if shape.dtype == "bf16":
            if a.dtype != np.uint16:
                raise ValueError("a bf16 buffer is handed in as uint16 bit patterns")
            a = bf16_from_bits(a)
        if tuple(a.shape) != tuple(shape.memory_dims()):
            raise ValueError(f"shape mismatch: got {a.shape}, HLO says {shape.dims} laid out as {shape.memory_dims()}")
        return _from_memory(a, shape).astype(self.np_dtype(shape.dtype), copy=False)

    def _run_comp(self, comp: Comp, args: List[np.ndarray], top: bool = False):
        env: Dict[str, object] = {}
        shapes = {i.name: i.shape for i in comp.instrs}
        for ins in comp.instrs:
            self._top, self._shapes = top, shapes
            env[ins.name] = self._eval(ins, env, args)
            if not self.fp32 and ins.shape.tuple_shapes is None and ins.shape.dtype == "bf16" and isinstance(env[ins.name], np.ndarray):
                env[ins.name] = round_to_bf16(env[ins.name])
            if top and self._keep and isinstance(env[ins.name], np.ndarray):
                self.trace[ins.name] = env[ins.name]
        res = env[comp.root.name]
        if top:     # results leave as memory images, like the parameters came in
            if isinstance(res, tuple):
                res = tuple(_memory_image(r, shapes[o]) for r, o in zip(res, comp.root.operands))
            else:
                res = _memory_image(res, comp.root.shape)
        return res

    def _eval(self, ins: Instr, env, args):
        op = ins.opcode
        x = [env[o] for o in ins.operands]
        sh = ins.shape
        dt = self.np_dtype(sh.dtype) if sh.tuple_shapes is None else None
        if op == "parameter":
            if self._vector_depth:   # a reducer body applied to whole arrays at once: its scalar shapes are not checked
                return np.asarray(args[int(ins.literal)]).astype(self.np_dtype(sh.dtype), copy=False)
            if not self._top:        # a called computation receives values, not buffers
                a = np.asarray(args[int(ins.literal)])
                if tuple(a.shape) != tuple(sh.dims):
                    raise ValueError(f"shape mismatch: got {a.shape}, HLO says {sh.dims}")
                return a.astype(self.np_dtype(sh.dtype), copy=False)
            return self._cast_in(args[int(ins.literal)], sh)
        if op == "constant":
            if ins.literal.replace(" ", "") == "{...}":
                if ins.name not in self.constants:
                    raise KeyError(f"payload for elided constant {ins.name} not supplied")
                return self._cast_in(self.constants[ins.name], sh)
            return _parse_literal(ins.literal, dt, sh.dims)
        if op in ("tuple",):
            return tuple(x)
        if op == "get-tuple-element":
            return x[0][int(ins.attrs["index"])]
        if op == "reshape":      # defined on logical row-major order whatever the layouts
            return np.ascontiguousarray(x[0]).reshape(sh.dims)
        if op == "bitcast":      # the same bytes under another shape and layout
            return _from_memory(_memory_image(x[0], self._shapes[ins.operands[0]]), sh)
        if op == "fusion" or op == "call":
            key = "calls" if "calls" in ins.attrs else "to_apply"
            return self._run_comp(self.mod["comps"][ins.attrs[key].lstrip("%")], x)
        if op == "convert":
            src = x[0]
            if np.issubdtype(dt, np.integer) and np.issubdtype(src.dtype, np.floating):
                src = np.trunc(src)
            with np.errstate(over="ignore"):
                return src.astype(dt)
        if op in _UNARY:
            with np.errstate(all="ignore"):
                return _UNARY[op](x[0]).astype(dt, copy=False)
        if op in _BINARY:
            with np.errstate(all="ignore"):
                return _BINARY[op](x[0], x[1]).astype(dt, copy=False)
        if op == "divide":
            with np.errstate(all="ignore"):
                if np.issubdtype(dt, np.integer):
                    q = np.trunc(x[0].astype(np.float64) / x[1].astype(np.float64))
                    return q.astype(dt)
                return np.divide(x[0], x[1]).astype(dt, copy=False)
        if op == "power":
            return np.power(x[0], x[1]).astype(dt, copy=False)
        if op == "compare":
            return _CMP[ins.attrs["direction"]](x[0], x[1])
        if op == "select":
            return np.where(x[0], x[1], x[2]).astype(dt, copy=False)
        if op == "clamp":
            return np.minimum(np.maximum(x[1], x[0]), x[2]).astype(dt, copy=False)
        if op == "broadcast":
            mapping = _ints(ins.attrs.get("dimensions", "{}"))
            shape1 = [1] * len(sh.dims)
            for i, m in enumerate(mapping):
                shape1[m] = x[0].shape[i]
            return np.broadcast_to(x[0].reshape(shape1), sh.dims)
        if op == "transpose":
            return np.transpose(x[0], _ints(ins.attrs["dimensions"]))
        if op == "iota":
            d = int(ins.attrs["iota_dimension"])
            shape1 = [1] * len(sh.dims)
            shape1[d] = sh.dims[d]
            return np.broadcast_to(np.arange(sh.dims[d], dtype=dt).reshape(shape1), sh.dims)
        if op == "slice":
            parts = re.findall(r"\[(\d+):(\d+)(?::(\d+))?\]", ins.attrs["slice"])
            idx = tuple(slice(int(a), int(b), int(c) if c else 1) for a, b, c in parts)
            return x[0][idx]
        if op == "concatenate":
            return np.concatenate(x, axis=_ints(ins.attrs["dimensions"])[0])
        if op == "pad":
            cfg = [tuple(int(v) for v in p.split("_")[:2]) for p in ins.attrs["padding"].split("x")]
            out = np.empty(sh.dims, dt)
            out[...] = x[1]
            idx = tuple(slice(lo, lo + n) for (lo, _), n in zip(cfg, x[0].shape))
            out[idx] = x[0]
            return out
        if op == "reduce":
            return self._reduce(ins, x, dt)
        if op == "gather":
            return self._gather(ins, x)
        if op == "dynamic-slice":
            sizes = _ints(ins.attrs["dynamic_slice_sizes"])
            starts = [int(np.clip(int(s), 0, x[0].shape[i] - sizes[i])) for i, s in enumerate(x[1:])]
            return x[0][tuple(slice(s, s + n) for s, n in zip(starts, sizes))]
        if op == "dynamic-update-slice":
            # start indices are clamped so that the update fits (XLA semantics, as for dynamic-slice)
            upd = x[1]
            starts = [int(np.clip(int(s), 0, x[0].shape[i] - upd.shape[i])) for i, s in enumerate(x[2:])]
            out = np.array(x[0], dtype=dt, copy=True)
            out[tuple(slice(s, s + n) for s, n in zip(starts, upd.shape))] = upd
            return out
        if op == "reduce-window":
            return self._reduce_window(ins, x, dt)
        if op == "dot":
            lc, rc = _ints(ins.attrs["lhs_contracting_dims"])[0], _ints(ins.attrs["rhs_contracting_dims"])[0]
            A, B = x[0].astype(np.float32), x[1].astype(np.float32)
            r = A.ndim
            if _ints(ins.attrs.get("lhs_batch_dims", "")) != list(range(r - 2)):
                raise NotImplementedError("dot: batch dims must be the leading dims")
            if lc == r - 2:
                A = np.swapaxes(A, -1, -2)
            if rc == r - 1:
                B = np.swapaxes(B, -1, -2)
            with np.errstate(over="ignore"):
                return np.matmul(A, B).astype(dt)
        if op == "custom-call":
            target = ins.attrs["custom_call_target"].strip('"')
            if target == "__cublas$gemm":
                return self._gemm(ins, x, dt)
            if target == "__cudnn$convForward":
                return self._conv_forward(ins, x)
            if target == "__cublas$lt$matmul":
                return self._lt_matmul(ins, x, dt)
            raise NotImplementedError(f"custom-call target {target}")
        raise NotImplementedError(f"opcode {op}")

    def _apply_reducer(self, red: Comp, args):
        self._vector_depth += 1
        try:
            return self._run_comp(red, list(args))
        finally:
            self._vector_depth -= 1

    def _reduce_window(self, ins: Instr, x, dt):
        # out[o] = reducer over w of padded(x)[o * stride + w], padding = the init value, the accumulator
        # starts at the init value (ir_parser_fused.cc:1215-1262: two operands, no dilation)
        if len(x) != 2:
            raise NotImplementedError("reduce-window takes one operand and one init value")
        win = dict(kv.split("=") for kv in ins.attrs["window"].strip("{}").split())
        if "lhs_dilate" in win or "rhs_dilate" in win:
            raise NotImplementedError("reduce-window with dilation")
        size = [int(v) for v in win["size"].split("x")]
        stride = [int(v) for v in win["stride"].split("x")] if "stride" in win else [1] * len(size)
        pad = [tuple(int(v) for v in p.split("_")) for p in win["pad"].split("x")] if "pad" in win else [(0, 0)] * len(size)
        red = self.mod["comps"][ins.attrs["to_apply"].lstrip("%")]
        init = np.asarray(x[1])
        padded = np.empty([lo + n + hi for (lo, hi), n in zip(pad, x[0].shape)], x[0].dtype)
        padded[...] = init
        padded[tuple(slice(lo, lo + n) for (lo, _), n in zip(pad, x[0].shape))] = x[0]
        acc = np.empty(ins.shape.dims, x[0].dtype)
        acc[...] = init
        with np.errstate(all="ignore"):
            for w in np.ndindex(*size):
                part = padded[tuple(slice(wi, wi + (o - 1) * st + 1, st) for wi, o, st in zip(w, ins.shape.dims, stride))]
                acc = self._apply_reducer(red, [acc, part])
        return np.asarray(acc).astype(dt, copy=False)

    def _reduce_variadic(self, ins: Instr, x, d):
        # N operands, N init values, a reducer of 2N parameters (accumulators first) returning an N-tuple
        # (ir_parser_fused.cc:1169-1213: tuple functors, e.g. (value, index) for arg-max); elements are
        # combined in ascending order of the reduced dimension
        n = len(x) // 2
        red = self.mod["comps"][ins.attrs["to_apply"].lstrip("%")]
        out_dims = [e for i, e in enumerate(x[0].shape) if i != d]
        acc = []
        for i in range(n):
            a = np.empty(out_dims, x[i].dtype)
            a[...] = x[n + i]
            acc.append(a)
        with np.errstate(all="ignore"):
            for k in range(x[0].shape[d]):
                res = self._apply_reducer(red, acc + [np.take(x[i], k, axis=d) for i in range(n)])
                acc = [np.asarray(r) for r in res]
        return tuple(a.astype(self.np_dtype(t.dtype), copy=False) for a, t in zip(acc, ins.shape.tuple_shapes))

    def _reduce(self, ins: Instr, x, dt):
        dims = _ints(ins.attrs["dimensions"])
        if len(dims) == 1 and len(x) > 2 and len(x) % 2 == 0:
            return self._reduce_variadic(ins, x, dims[0])
        if len(dims) != 1 or len(x) != 2:
            raise NotImplementedError("only single-dimension reduce")
        red = self.mod["comps"][ins.attrs["to_apply"].lstrip("%")]
        fn = _REDUCERS[red.root.opcode]
        init = x[1]
        with np.errstate(all="ignore"):
            r = fn.reduce(x[0], axis=dims[0], dtype=x[0].dtype if x[0].dtype != np.bool_ else None)
            return fn(r, init).astype(dt, copy=False)

    def _gather(self, ins: Instr, x):
        table, idx = x
        a = ins.attrs
        if (_ints(a["collapsed_slice_dims"]) != [0] or _ints(a["start_index_map"]) != [0]
                or int(a["index_vector_dim"]) != idx.ndim):
            raise NotImplementedError("only row gather")
        sizes = _ints(a["slice_sizes"])
        if sizes[0] != 1 or list(sizes[1:]) != list(table.shape[1:]):
            raise NotImplementedError("only whole-row slices")
        safe = np.clip(idx.astype(np.int64), 0, table.shape[0] - 1)   # XLA clamps start indices
        return table[safe]

    def _gemm(self, ins: Instr, x, dt):
        cfg = json.loads(ins.attrs["backend_config"][1:-1].replace('\\"', '"'))
        cfg = cfg.get("gemm_backend_config", cfg)
        dn = cfg["dot_dimension_numbers"]
        lc = int(dn["lhs_contracting_dimensions"][0])
        rc = int(dn["rhs_contracting_dimensions"][0])
        A = x[0].astype(np.float32, copy=False)
        B = x[1].astype(np.float32, copy=False)
        r = A.ndim
        if lc == r - 2:
            A = np.swapaxes(A, -1, -2)
        if rc == r - 1:
            B = np.swapaxes(B, -1, -2)
        D = np.matmul(A, B) * np.float32(cfg["alpha_real"])
        if len(x) > 2 and float(cfg["beta"]) != 0.0:
            D = D + np.float32(cfg["beta"]) * x[2].astype(np.float32, copy=False)
        with np.errstate(over="ignore"):
            return D.astype(dt, copy=False)


    def _lt_matmul(self, ins: Instr, x, dt):
        """__cublas$lt$matmul(a, b[, c][, bias]), the newer spelling of the cuBLAS call.  The reference accepts only
        __cublas$gemm (core/op/custom_call.cc:96-100); alpha / beta / dimension numbers are read as for that call
        (gemm_impl.cc:182-231), the `epilogue` field follows cuBLASLt as XLA's GEMM rewriter uses it:
        D = act(alpha * A.B + beta * C + bias[column]), act = identity | max(., 0) | tanh-GELU, evaluated in fp32 and
        rounded once to the result type.  Reconstructed without a dump of such a module: parity unpinned against XLA."""
        cfg = json.loads(ins.attrs["backend_config"][1:-1].replace('\\"', '"'))
        cfg = cfg.get("gemm_backend_config", cfg)
        ep = cfg.get("epilogue", "DEFAULT")
        if not isinstance(ep, str):
            ep = ["DEFAULT", "BIAS", "RELU", "BIAS_RELU", "GELU", "BIAS_GELU", "GELU_AUX", "BIAS_GELU_AUX"][int(ep)]
        if ep not in ("DEFAULT", "BIAS", "RELU", "GELU", "BIAS_RELU", "BIAS_GELU"):
            raise NotImplementedError(f"__cublas$lt$matmul epilogue {ep}")
        dn = cfg["dot_dimension_numbers"]
        lc, rc = int(dn["lhs_contracting_dimensions"][0]), int(dn["rhs_contracting_dimensions"][0])
        A, B = x[0].astype(np.float32), x[1].astype(np.float32)
        r = A.ndim
        A = np.swapaxes(A, -1, -2) if lc == r - 2 else A
        B = np.swapaxes(B, -1, -2) if rc == r - 1 else B
        D = np.einsum("...mk,...kn->...mn", A, B) * np.float32(cfg["alpha_real"])
        nxt = 2
        if float(cfg["beta"]) != 0.0:
            D = D + np.float32(cfg["beta"]) * x[nxt].astype(np.float32)
            nxt += 1
        if ep.startswith("BIAS"):
            D = D + x[nxt].astype(np.float32)[None, :]
            nxt += 1
        if len(x) != nxt:
            raise ValueError("__cublas$lt$matmul: operand count does not match beta and epilogue")
        if ep.endswith("RELU"):
            D = np.maximum(D, np.float32(0))
        if ep.endswith("GELU"):
            D = np.float32(0.5) * D * (np.float32(1) + np.tanh(np.float32(0.7978845608028654) * (D + np.float32(0.044715) * D * D * D)))
        out_sh = ins.shape.tuple_shapes[0] if ins.shape.tuple_shapes else ins.shape
        with np.errstate(over="ignore"):
            out = D.astype(self.np_dtype(out_sh.dtype))
        if ins.shape.tuple_shapes:
            return (out, np.zeros(ins.shape.tuple_shapes[1].dims, np.uint8))
        return out

    def _conv_forward(self, ins: Instr, x):
        """cuDNN forward convolution custom call as the reference lowers it (conv_impl.cc:252-324, attributes
        from ir_parser_fused.cc:749-823): input N,H,W,C; filter K,R,S,C; output N,P,Q,K;
        out[n,p,q,k] = scale * sum_{r,s,c} in[n, p*sh + r - ph, q*sw + s - pw, c] * filt[k,r,s,c], zero outside.
        Result is the tuple (output, scratch)."""
        a = ins.attrs
        if a.get("dim_labels", "").strip() != "b01f_o01i->b01f":
            raise NotImplementedError("only dim_labels=b01f_o01i->b01f")
        if int(a.get("feature_group_count", "1")) != 1:
            raise NotImplementedError("grouped convolution")
        win = a["window"].strip("{} ")
        fields = dict(f.split("=") for f in win.split())
        size = [int(v) for v in fields["size"].split("x")]
        stride = [int(v) for v in fields.get("stride", "1x1").split("x")]
        pad = [[int(t) for t in v.split("_")] for v in fields.get("pad", "0_0x0_0").split("x")]
        for key in ("lhs_dilate", "rhs_dilate"):
            if key in fields and any(int(v) != 1 for v in fields[key].split("x")):
                raise NotImplementedError("dilated convolution")
        cfg = json.loads(a["backend_config"][1:-1].replace('\\"', '"'))
        if float(cfg.get("side_input_scale", 0)) != 0.0 or str(cfg.get("activation_mode", "0")) != "0":
            raise NotImplementedError("side input / activation in the convolution call")
        inp = x[0].astype(np.float32)
        flt = x[1].astype(np.float32)
        N, H, W, C = inp.shape
        K, R, S, C2 = flt.shape
        assert C == C2 and [R, S] == size
        out_sh = ins.shape.tuple_shapes[0]
        P, Q = out_sh.dims[1], out_sh.dims[2]
        padded = np.zeros((N, H + pad[0][0] + pad[0][1], W + pad[1][0] + pad[1][1], C), np.float32)
        padded[:, pad[0][0]:pad[0][0] + H, pad[1][0]:pad[1][0] + W, :] = inp
        out = np.zeros((N, P, Q, K), np.float32)
        for r in range(R):
            for s_ in range(S):
                patch = padded[:, r:r + (P - 1) * stride[0] + 1:stride[0], s_:s_ + (Q - 1) * stride[1] + 1:stride[1], :]
                out += np.einsum("npqc,kc->npqk", patch, flt[:, r, s_, :], optimize=True)
        out *= np.float32(cfg.get("conv_result_scale", 1))
        with np.errstate(over="ignore"):
            res = out.astype(self.np_dtype(out_sh.dtype))
        scratch = np.zeros(ins.shape.tuple_shapes[1].dims, np.uint8)
        return (res, scratch)


def evaluate(text: str, params: Sequence[np.ndarray], constants: Optional[Dict[str, np.ndarray]] = None,
             precision: str = "as_written") -> List[np.ndarray]:
    """Evaluate the ENTRY computation; returns the list of outputs (root tuple flattened)."""
    return Evaluator(text, constants, precision).run(params)
