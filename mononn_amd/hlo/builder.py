"""Tiny XLA-HLO *text* builder.

MonoNN consumes an already optimised, already fused XLA-GPU HLO module
(reference: mononn_engine/parser/ir_parser_fused.cc:319-385).  XLA itself is not
available offline, so the model fixtures of this package are authored directly in
that dialect: `fusion` instructions with kind=kLoop|kInput calling fused
computations, `custom-call` GEMMs with custom_call_target="__cublas$gemm" and the
backend_config JSON of mononn_engine/core/op_impl/gemm_impl.cc:290-316, plain
`{n-1,...,0}` layouts, scalar constants inline and large constants elided
(`constant({...})`) with their payload supplied separately by the host, exactly as
the reference fills `buffer_for_<node>` before launch
(mononn_engine/codegen/graph_codegen.cc:71-86).

The builder only prints text and tracks shapes; it evaluates nothing.
"""
from __future__ import annotations

import json
from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence, Tuple

DTYPE_BYTES = {"pred": 1, "s8": 1, "u8": 1, "s16": 2, "u16": 2, "f16": 2, "s32": 4,
               "u32": 4, "f32": 4, "s64": 8, "u64": 8, "f64": 8}


@dataclass(frozen=True)
class Value:
    """A named HLO value with a static array shape."""
    name: str
    dtype: str
    dims: Tuple[int, ...]

    @property
    def shape_str(self) -> str:
        return shape_str(self.dtype, self.dims)

    @property
    def operand_str(self) -> str:
        return f"{self.shape_str} %{self.name}"

    @property
    def num_elements(self) -> int:
        n = 1
        for d in self.dims:
            n *= d
        return n

    @property
    def nbytes(self) -> int:
        return self.num_elements * DTYPE_BYTES[self.dtype]


def shape_str(dtype: str, dims: Sequence[int]) -> str:
    layout = ",".join(str(i) for i in reversed(range(len(dims))))
    return f"{dtype}[{','.join(str(d) for d in dims)}]{{{layout}}}"


def _fmt_scalar(dtype: str, v) -> str:
    if dtype == "pred":
        return "true" if v else "false"
    if dtype.startswith("f"):
        if v == float("inf"):
            return "inf"
        if v == float("-inf"):
            return "-inf"
        return repr(float(v))
    return str(int(v))


class Computation:
    """One HLO computation under construction (entry, fused or reducer)."""

    def __init__(self, module: "HloModuleBuilder", name: str):
        self.module = module
        self.name = name
        self.lines: List[str] = []
        self.params: List[Value] = []
        self.root: Optional[Value] = None
        self.root_is_tuple = False
        self.root_tuple: List[Value] = []

    # -- low level -----------------------------------------------------------------
    def _emit(self, opcode: str, dtype: str, dims: Sequence[int], operands: Sequence[Value],
              attrs: str = "", name_hint: Optional[str] = None, literal: Optional[str] = None) -> Value:
        name = self.module.fresh(name_hint or opcode)
        v = Value(name, dtype, tuple(int(d) for d in dims))
        body = literal if literal is not None else ", ".join(o.operand_str for o in operands)
        line = f"%{name} = {v.shape_str} {opcode}({body})"
        if attrs:
            line += ", " + attrs
        self.lines.append(line)
        self.root = v
        self.root_is_tuple = False
        return v

    # -- leaves --------------------------------------------------------------------
    def parameter(self, dtype: str, dims: Sequence[int], name_hint: str = "param") -> Value:
        idx = len(self.params)
        v = self._emit("parameter", dtype, dims, [], literal=str(idx), name_hint=name_hint)
        self.params.append(v)
        return v

    def scalar(self, dtype: str, value) -> Value:
        return self._emit("constant", dtype, (), [], literal=_fmt_scalar(dtype, value), name_hint="constant")

    def elided_constant(self, dtype: str, dims: Sequence[int], role: str) -> Value:
        """Large constant whose payload the host uploads by name; `role` is recorded in the
        module's constant table (and as metadata op_name) so a harness can find it."""
        v = self._emit("constant", dtype, dims, [], literal="{...}", name_hint="constant",
                       attrs=f'metadata={{op_type="Const" op_name="{role}"}}')
        self.module.constants[v.name] = {"role": role, "dtype": dtype, "dims": list(v.dims)}
        return v

    def literal_constant(self, dtype: str, dims: Sequence[int], flat_values: Sequence) -> Value:
        def nest(vals, ds):
            if len(ds) == 1:
                return "{" + ", ".join(_fmt_scalar(dtype, x) for x in vals) + "}"
            step = len(vals) // ds[0]
            return "{ " + ", ".join(nest(vals[i * step:(i + 1) * step], ds[1:]) for i in range(ds[0])) + " }"
        return self._emit("constant", dtype, dims, [], literal=nest(list(flat_values), list(dims)),
                          name_hint="constant")

    def iota(self, dtype: str, dims: Sequence[int], dim: int) -> Value:
        return self._emit("iota", dtype, dims, [], attrs=f"iota_dimension={dim}", literal="")

    # -- element-wise --------------------------------------------------------------
    def unary(self, opcode: str, x: Value) -> Value:
        return self._emit(opcode, x.dtype, x.dims, [x])

    def binary(self, opcode: str, a: Value, b: Value) -> Value:
        assert a.dims == b.dims and a.dtype == b.dtype, (opcode, a, b)
        return self._emit(opcode, a.dtype, a.dims, [a, b])

    def add(self, a, b): return self.binary("add", a, b)
    def sub(self, a, b): return self.binary("subtract", a, b)
    def mul(self, a, b): return self.binary("multiply", a, b)
    def div(self, a, b): return self.binary("divide", a, b)
    def maximum(self, a, b): return self.binary("maximum", a, b)
    def tanh(self, x): return self.unary("tanh", x)
    def exp(self, x): return self.unary("exponential", x)
    def rsqrt(self, x): return self.unary("rsqrt", x)
    def negate(self, x): return self.unary("negate", x)

    def convert(self, x: Value, dtype: str) -> Value:
        return self._emit("convert", dtype, x.dims, [x])

    def compare(self, a: Value, b: Value, direction: str) -> Value:
        assert a.dims == b.dims
        return self._emit("compare", "pred", a.dims, [a, b], attrs=f"direction={direction}")

    def select(self, p: Value, a: Value, b: Value) -> Value:
        return self._emit("select", a.dtype, a.dims, [p, a, b])

    # -- shape ops -----------------------------------------------------------------
    def broadcast(self, x: Value, dims: Sequence[int], mapping: Sequence[int]) -> Value:
        assert len(mapping) == len(x.dims)
        for i, m in enumerate(mapping):
            assert dims[m] == x.dims[i], (x, dims, mapping)
        return self._emit("broadcast", x.dtype, dims, [x],
                          attrs="dimensions={" + ",".join(str(m) for m in mapping) + "}")

    def splat(self, dtype: str, value, dims: Sequence[int]) -> Value:
        return self.broadcast(self.scalar(dtype, value), dims, [])

    def reshape(self, x: Value, dims: Sequence[int], opcode: str = "reshape") -> Value:
        n = 1
        for d in dims:
            n *= d
        assert n == x.num_elements, (x, dims)
        return self._emit(opcode, x.dtype, dims, [x])

    def bitcast(self, x: Value, dims: Sequence[int]) -> Value:
        return self.reshape(x, dims, opcode="bitcast")

    def transpose(self, x: Value, perm: Sequence[int]) -> Value:
        dims = [x.dims[p] for p in perm]
        return self._emit("transpose", x.dtype, dims, [x],
                          attrs="dimensions={" + ",".join(str(p) for p in perm) + "}")

    def slice(self, x: Value, starts: Sequence[int], limits: Sequence[int]) -> Value:
        dims = [l - s for s, l in zip(starts, limits)]
        spec = ", ".join(f"[{s}:{l}]" for s, l in zip(starts, limits))
        return self._emit("slice", x.dtype, dims, [x], attrs="slice={" + spec + "}")

    def pad(self, x: Value, value: Value, low: Sequence[int], high: Sequence[int]) -> Value:
        """Edge padding without interior padding (ir_parser_fused.cc:1143-1147)."""
        dims = [lo + n + hi for lo, n, hi in zip(low, x.dims, high)]
        return self._emit("pad", x.dtype, dims, [x, value], attrs="padding=" + "x".join(f"{lo}_{hi}" for lo, hi in zip(low, high)))

    def concatenate(self, xs: Sequence[Value], dim: int) -> Value:
        dims = list(xs[0].dims)
        dims[dim] = sum(x.dims[dim] for x in xs)
        return self._emit("concatenate", xs[0].dtype, dims, list(xs), attrs=f"dimensions={{{dim}}}")

    def reduce(self, x: Value, init: Value, dim: int, reducer: str) -> Value:
        dims = [d for i, d in enumerate(x.dims) if i != dim]
        return self._emit("reduce", x.dtype, dims, [x, init],
                          attrs=f"dimensions={{{dim}}}, to_apply=%{reducer}")

    def reduce_window(self, x: Value, init: Value, size: Sequence[int], stride: Sequence[int],
                      pad: Sequence[Sequence[int]], reducer: str) -> Value:
        """Window reduction without dilation (ir_parser_fused.cc:1215-1262): out = (in + lo + hi - size) / stride + 1."""
        dims = [(n + lo + hi - w) // st + 1 for n, w, st, (lo, hi) in zip(x.dims, size, stride, pad)]
        window = ("size=" + "x".join(map(str, size)) + " stride=" + "x".join(map(str, stride)) +
                  " pad=" + "x".join(f"{lo}_{hi}" for lo, hi in pad))
        return self._emit("reduce-window", x.dtype, dims, [x, init], attrs=f"window={{{window}}}, to_apply=%{reducer}")

    def dynamic_slice(self, x: Value, starts: Sequence[Value], sizes: Sequence[int]) -> Value:
        return self._emit("dynamic-slice", x.dtype, sizes, [x] + list(starts),
                          attrs="dynamic_slice_sizes={" + ",".join(str(n) for n in sizes) + "}")

    def dynamic_update_slice(self, x: Value, update: Value, starts: Sequence[Value]) -> Value:
        return self._emit("dynamic-update-slice", x.dtype, x.dims, [x, update] + list(starts))

    def reduce_variadic(self, xs: Sequence[Value], inits: Sequence[Value], dim: int, reducer: str) -> List[Value]:
        """N-operand reduce with a tuple-valued reducer, e.g. (value, index) for arg-max
        (ir_parser_fused.cc:1169-1213).  Returns the get-tuple-element values."""
        dims = tuple(d for i, d in enumerate(xs[0].dims) if i != dim)
        outs = [Value("", x.dtype, dims) for x in xs]
        tshape = "(" + ", ".join(o.shape_str for o in outs) + ")"
        name = self.module.fresh("reduce")
        ops = ", ".join(o.operand_str for o in list(xs) + list(inits))
        self.lines.append(f"%{name} = {tshape} reduce({ops}), dimensions={{{dim}}}, to_apply=%{reducer}")
        res = []
        for i, o in enumerate(outs):
            g = self.module.fresh("get-tuple-element")
            self.lines.append(f"%{g} = {o.shape_str} get-tuple-element({tshape} %{name}), index={i}")
            res.append(Value(g, o.dtype, o.dims))
        self.root = res[-1]
        self.root_is_tuple = False
        return res

    def gather_rows(self, table: Value, indices: Value) -> Value:
        """Row gather out[i..., :] = table[indices[i...], :] in XLA's gather form
        (dimension numbers as recorded by ir_parser_fused.cc:1034-1066)."""
        assert len(table.dims) == 2
        out_dims = list(indices.dims) + [table.dims[1]]
        r = len(indices.dims)
        attrs = (f"offset_dims={{{r}}}, collapsed_slice_dims={{0}}, start_index_map={{0}}, "
                 f"index_vector_dim={r}, slice_sizes={{1,{table.dims[1]}}}")
        return self._emit("gather", table.dtype, out_dims, [table, indices], attrs=attrs)

    # -- calls ---------------------------------------------------------------------
    def fusion(self, kind: str, operands: Sequence[Value],
               body: Callable[..., object], name_hint: str = "fusion"):
        """Create a fused computation; `body(f, *params)` builds it and returns the root Value or a
        list/tuple of Values for a multi-output fusion.  Returns Value or list of GTE Values."""
        fc = Computation(self.module, self.module.fresh("fused_computation"))
        params = [fc.parameter(o.dtype, o.dims, name_hint=f"param_{i}") for i, o in enumerate(operands)]
        out = body(fc, *params)
        if isinstance(out, (list, tuple)):
            fc.set_tuple_root(list(out))
            self.module.computations.append(fc)
            tshape = "(" + ", ".join(o.shape_str for o in out) + ")"
            name = self.module.fresh(name_hint)
            ops = ", ".join(o.operand_str for o in operands)
            self.lines.append(f"%{name} = {tshape} fusion({ops}), kind={kind}, calls=%{fc.name}")
            res = []
            for i, o in enumerate(out):
                g = self.module.fresh("get-tuple-element")
                self.lines.append(f"%{g} = {o.shape_str} get-tuple-element({tshape} %{name}), index={i}")
                res.append(Value(g, o.dtype, o.dims))
            self.root = res[-1]
            return res
        assert fc.root is not None and fc.root.name == out.name, "fusion body must return its last value"
        self.module.computations.append(fc)
        return self._emit("fusion", out.dtype, out.dims, list(operands),
                          attrs=f"kind={kind}, calls=%{fc.name}", name_hint=name_hint)

    def gemm(self, a: Value, b: Value, lhs_contract: int, rhs_contract: int,
             batch_dims: Sequence[int] = (), alpha: float = 1.0, beta: float = 0.0,
             addend: Optional[Value] = None) -> Value:
        """`__cublas$gemm` custom call.  Operands have equal rank; the two minor-most dims are the
        matrix dims, the leading ones the batch (gemm_impl.cc:252-253, :290-316)."""
        r = len(a.dims)
        assert len(b.dims) == r
        nb = len(batch_dims)
        assert list(batch_dims) == list(range(nb)) and nb == r - 2
        m_dim = r - 1 if lhs_contract == r - 2 else r - 2
        n_dim = r - 1 if rhs_contract == r - 2 else r - 2
        assert a.dims[lhs_contract] == b.dims[rhs_contract]
        out_dims = list(a.dims[:nb]) + [a.dims[m_dim], b.dims[n_dim]]
        batch = 1
        for d in a.dims[:nb]:
            batch *= d
        cfg = {
            "alpha_real": alpha, "alpha_imag": 0, "beta": beta,
            "dot_dimension_numbers": {
                "lhs_contracting_dimensions": [str(lhs_contract)],
                "rhs_contracting_dimensions": [str(rhs_contract)],
                "lhs_batch_dimensions": [str(d) for d in batch_dims],
                "rhs_batch_dimensions": [str(d) for d in batch_dims]},
            "batch_size": str(batch),
            "lhs_stride": str(a.dims[-1] * a.dims[-2]),
            "rhs_stride": str(b.dims[-1] * b.dims[-2]),
            "selected_algorithm": "-1"}
        cfg_s = json.dumps(cfg, separators=(",", ":")).replace('"', '\\"')
        ops = [a, b] + ([addend] if addend is not None else [])
        return self._emit("custom-call", a.dtype, out_dims, ops,
                          attrs=f'custom_call_target="__cublas$gemm", backend_config="{cfg_s}"',
                          name_hint="cublas-batch-gemm" if batch > 1 else "cublas-gemm")

    def lt_matmul(self, a: Value, b: Value, lhs_contract: int, rhs_contract: int, epilogue: str = "DEFAULT", bias: Optional[Value] = None,
                  alpha: float = 1.0, beta: float = 0.0, addend: Optional[Value] = None, nested_config: bool = True) -> Value:
        """`__cublas$lt$matmul` custom call as newer XLA versions print it: operands (a, b[, c][, bias]), the
        `gemm_backend_config` of `gemm` plus `epilogue` (DEFAULT, BIAS, RELU, GELU, BIAS_RELU, BIAS_GELU)."""
        r = len(a.dims)
        assert r == 2 and len(b.dims) == 2, "unbatched matrices"
        m_dim = 1 if lhs_contract == 0 else 0
        n_dim = 1 if rhs_contract == 0 else 0
        assert a.dims[lhs_contract] == b.dims[rhs_contract]
        out_dims = [a.dims[m_dim], b.dims[n_dim]]
        cfg = {"alpha_real": alpha, "alpha_imag": 0, "beta": beta,
               "dot_dimension_numbers": {"lhs_contracting_dimensions": [str(lhs_contract)], "rhs_contracting_dimensions": [str(rhs_contract)],
                                         "lhs_batch_dimensions": [], "rhs_batch_dimensions": []},
               "epilogue": epilogue}
        if nested_config:
            cfg = {"gemm_backend_config": cfg}
        cfg_s = json.dumps(cfg, separators=(",", ":")).replace('"', '\\"')
        ops = [a, b] + ([addend] if addend is not None else []) + ([bias] if bias is not None else [])
        return self._emit("custom-call", a.dtype, out_dims, ops,
                          attrs=f'custom_call_target="__cublas$lt$matmul", backend_config="{cfg_s}"', name_hint="cublas-lt-matmul")

    def dot(self, a: Value, b: Value, lhs_contract: int, rhs_contract: int, batch_dims: Sequence[int] = ()) -> Value:
        """Plain `dot` with the same operand conventions as `gemm` (what XLA prints before its GEMM rewriter)."""
        r = len(a.dims)
        nb = len(batch_dims)
        assert len(b.dims) == r and list(batch_dims) == list(range(nb)) and nb == r - 2
        m_dim = r - 1 if lhs_contract == r - 2 else r - 2
        n_dim = r - 1 if rhs_contract == r - 2 else r - 2
        out_dims = list(a.dims[:nb]) + [a.dims[m_dim], b.dims[n_dim]]
        attrs = ""
        if nb:
            bd = ",".join(str(d) for d in batch_dims)
            attrs = f"lhs_batch_dims={{{bd}}}, "
        attrs += f"lhs_contracting_dims={{{lhs_contract}}}, "
        if nb:
            attrs += f"rhs_batch_dims={{{bd}}}, "
        attrs += f"rhs_contracting_dims={{{rhs_contract}}}"
        return self._emit("dot", a.dtype, out_dims, [a, b], attrs=attrs, name_hint="dot")

    def conv_forward(self, x: Value, filt: Value, stride: Sequence[int] = (1, 1), pad: Sequence[int] = (0, 0),
                     result_scale: float = 1.0) -> Value:
        """`__cudnn$convForward` custom call on an N,H,W,C input and a K,R,S,C filter (dim_labels
        b01f_o01i->b01f), symmetric padding, no dilation, one feature group -- the form the reference accepts
        (ir_parser_fused.cc:749-823).  The call yields (output, scratch); the output is taken with
        get-tuple-element index 0, as XLA does."""
        n, h, w, c = x.dims
        k, r, s, c2 = filt.dims
        assert c == c2
        p = (h + 2 * pad[0] - r) // stride[0] + 1
        q = (w + 2 * pad[1] - s) // stride[1] + 1
        out = Value("", x.dtype, (n, p, q, k))
        window = f"size={r}x{s}"
        if tuple(stride) != (1, 1):
            window += f" stride={stride[0]}x{stride[1]}"
        if tuple(pad) != (0, 0):
            window += f" pad={pad[0]}_{pad[0]}x{pad[1]}_{pad[1]}"
        cfg = json.dumps({"conv_result_scale": result_scale, "activation_mode": "0", "side_input_scale": 0},
                         separators=(",", ":")).replace('"', '\\"')
        name = self.module.fresh("cudnn-conv")
        tshape = f"({out.shape_str}, u8[0]{{0}})"
        self.lines.append(f"%{name} = {tshape} custom-call({x.operand_str}, {filt.operand_str}), window={{{window}}}, "
                          f"dim_labels=b01f_o01i->b01f, custom_call_target=\"__cudnn$convForward\", backend_config=\"{cfg}\"")
        gte = self.module.fresh("get-tuple-element")
        v = Value(gte, x.dtype, out.dims)
        self.lines.append(f"%{gte} = {v.shape_str} get-tuple-element({tshape} %{name}), index=0")
        self.root = v
        self.root_is_tuple = False
        return v

    def set_tuple_root(self, values: Sequence[Value]):
        name = self.module.fresh("tuple")
        tshape = "(" + ", ".join(v.shape_str for v in values) + ")"
        self.lines.append(f"%{name} = {tshape} tuple({', '.join(v.operand_str for v in values)})")
        self.root = Value(name, "tuple", ())
        self.root_is_tuple = True
        self.root_tuple = list(values)

    def text(self, entry: bool = False) -> str:
        out = [("ENTRY " if entry else "") + f"%{self.name} {{"]
        for i, l in enumerate(self.lines):
            out.append(("  ROOT " if i == len(self.lines) - 1 else "  ") + l)
        out.append("}")
        return "\n".join(out)


class HloModuleBuilder:
    """Collects computations and prints one HLO module.  The module name must start with
    `cluster_<digits>` so the dump directory can be derived from it
    (mononn_engine/helpers/string_helpers.cc:34-48)."""

    def __init__(self, name: str = "cluster_0__XlaCompiledKernel_true__XlaNumConstantArgs_0_.1"):
        self.name = name
        self.computations: List[Computation] = []
        self.constants: Dict[str, dict] = {}
        self._ids: Dict[str, int] = {}
        self._counter = 0
        self.entry = Computation(self, "main")
        self._reducers: Dict[Tuple[str, str], str] = {}

    def fresh(self, hint: str) -> str:
        self._counter += 1
        return f"{hint}.{self._counter}"

    def reducer(self, opcode: str, dtype: str) -> str:
        """Scalar binary reducer computation (add / maximum / minimum), created on first use."""
        key = (opcode, dtype)
        if key not in self._reducers:
            c = Computation(self, self.fresh(f"{opcode}_{dtype}_reducer"))
            a = c.parameter(dtype, (), "x")
            b = c.parameter(dtype, (), "y")
            c.binary(opcode, a, b)
            self.computations.append(c)
            self._reducers[key] = c.name
        return self._reducers[key]

    def arg_reducer(self, direction: str, dtype: str, index_dtype: str = "s32") -> str:
        """(value, index) reducer: keeps the larger (direction GT) or smaller (LT) value, and on equal values the
        smaller index -- the form XLA gives tf.argmax / tf.argmin.  With GT / LT the reducer is commutative, which a
        reduction spread over lanes needs; GE / LE keep the accumulator on ties whatever its index and only mean
        "first index" when the elements arrive in ascending order."""
        key = ("arg", direction, dtype, index_dtype)
        if key not in self._reducers:
            c = Computation(self, self.fresh(f"arg_{direction.lower()}_{dtype}_reducer"))
            av = c.parameter(dtype, (), "acc_value")
            ai = c.parameter(index_dtype, (), "acc_index")
            xv = c.parameter(dtype, (), "value")
            xi = c.parameter(index_dtype, (), "index")
            better = c.compare(av, xv, direction)
            same = c.compare(av, xv, "EQ")
            first = c.compare(ai, xi, "LT")
            keep = c.binary("or", better, c.binary("and", same, first))
            c.set_tuple_root([c.select(keep, av, xv), c.select(keep, ai, xi)])
            self.computations.append(c)
            self._reducers[key] = c.name
        return self._reducers[key]

    def text(self) -> str:
        parts = [f"HloModule {self.name}", ""]
        for c in self.computations:
            parts.append(c.text())
            parts.append("")
        parts.append(self.entry.text(entry=True))
        parts.append("")
        return "\n".join(parts)
