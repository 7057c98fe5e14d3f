"""Pins the element-wise, slicing and reduce branches of the NumPy oracle that the model-level checks do not reach.
The HLO text is written out by hand (not by mononn_amd.hlo.builder) and every expected value comes from plain Python
arithmetic, a brute-force loop or a NumPy routine other than the one the oracle calls, chosen so that a plausible
mistake -- a wrong rounding direction, swapped select operands, an unclamped start index, low and high padding
exchanged -- fails."""
import math

import numpy as np
import pytest

from oracle import hlo_interp


def _module(body: str, params, root_shape: str, kind="kLoop", extra=""):
    """One fusion over `params` [(shape_text, ...)] whose computation is `body` (root named %r)."""
    ps = "\n".join(f"  %p{i} = {s} parameter({i})" for i, s in enumerate(params))
    ops = ", ".join(f"{s} %a{i}" for i, s in enumerate(params))
    es = "\n".join(f"  %a{i} = {s} parameter({i})" for i, s in enumerate(params))
    return f"""HloModule cluster_5__pin_ops.1
{extra}
%fc {{
{ps}
{body}
}}

ENTRY %main {{
{es}
  %f = {root_shape} fusion({ops}), kind={kind}, calls=%fc
  ROOT %t = ({root_shape}) tuple({root_shape} %f)
}}
"""


def _run(text, args):
    return hlo_interp.evaluate(text, args, {})[0]


def test_integer_divide_truncates_toward_zero():
    a = np.array([7, -7, 7, -7, 0, -1, 2147483647, -9], np.int32)
    b = np.array([2, 2, -2, -2, 5, 3, 2, 4], np.int32)
    got = _run(_module("  ROOT %r = s32[8]{0} divide(s32[8]{0} %p0, s32[8]{0} %p1)", ["s32[8]{0}", "s32[8]{0}"], "s32[8]{0}"), [a, b])
    want = [int(x / y) if abs(x) < 2 ** 30 else 1073741823 for x, y in zip(a.tolist(), b.tolist())]   # C semantics; floor would give -4 for -7/2
    assert got.dtype == np.int32 and got.tolist() == want
    assert got.tolist()[:4] == [3, -3, -3, 3]


def test_float_to_int_convert_truncates_and_int_to_float_is_exact():
    x = np.array([2.9, -2.9, 0.5, -0.5, 1e3 + 0.999, -7.0001], np.float32)
    got = _run(_module("  ROOT %r = s32[6]{0} convert(f32[6]{0} %p0)", ["f32[6]{0}"], "s32[6]{0}"), [x])
    assert got.dtype == np.int32 and got.tolist() == [2, -2, 0, 0, 1000, -7]        # rounding to nearest would give 3, -3
    i = np.array([3, -70000, 2049], np.int32)
    got = _run(_module("  ROOT %r = f16[3]{0} convert(s32[3]{0} %p0)", ["s32[3]{0}"], "f16[3]{0}"), [i])
    assert got.dtype == np.float16 and got[0] == 3 and np.isinf(got[1]) and got[1] < 0 and got[2] == 2048   # half: overflow, ties to even
    p = np.array([True, False], np.bool_)
    got = _run(_module("  ROOT %r = f32[2]{0} convert(pred[2]{0} %p0)", ["pred[2]{0}"], "f32[2]{0}"), [p])
    assert got.tolist() == [1.0, 0.0]


def test_power_log_negate_abs_sign_sqrt_against_python_math():
    x = np.array([0.25, 1.0, 2.5, 9.0, 100.0], np.float32)
    y = np.array([2.0, -3.0, 0.5, 1.5, 0.0], np.float32)
    body = """  %pw = f32[5]{0} power(f32[5]{0} %p0, f32[5]{0} %p1)
  %lg = f32[5]{0} log(f32[5]{0} %p0)
  %ng = f32[5]{0} negate(f32[5]{0} %lg)
  %sq = f32[5]{0} sqrt(f32[5]{0} %p0)
  %s1 = f32[5]{0} add(f32[5]{0} %pw, f32[5]{0} %ng)
  ROOT %r = f32[5]{0} subtract(f32[5]{0} %s1, f32[5]{0} %sq)"""
    got = _run(_module(body, ["f32[5]{0}", "f32[5]{0}"], "f32[5]{0}"), [x, y])
    want = [math.pow(a, b) - math.log(a) - math.sqrt(a) for a, b in zip(x.tolist(), y.tolist())]   # subtract order matters
    assert np.allclose(got, want, rtol=2e-6, atol=1e-6)
    z = np.array([-3.5, 0.0, 4.0], np.float32)
    body = """  %ab = f32[3]{0} abs(f32[3]{0} %p0)
  %sg = f32[3]{0} sign(f32[3]{0} %p0)
  %ex = f32[3]{0} exponential(f32[3]{0} %sg)
  ROOT %r = f32[3]{0} multiply(f32[3]{0} %ab, f32[3]{0} %ex)"""
    got = _run(_module(body, ["f32[3]{0}"], "f32[3]{0}"), [z])
    assert np.allclose(got, [3.5 * math.exp(-1.0), 0.0, 4.0 * math.e], rtol=1e-6)


def test_compare_select_clamp_and_logic():
    a = np.array([1, 5, 3, 3, -2, 9], np.int32)
    b = np.array([2, 4, 3, 1, -2, 0], np.int32)
    want_by_dir = {"EQ": [x == y for x, y in zip(a, b)], "NE": [x != y for x, y in zip(a, b)], "LT": [x < y for x, y in zip(a, b)],
                   "LE": [x <= y for x, y in zip(a, b)], "GT": [x > y for x, y in zip(a, b)], "GE": [x >= y for x, y in zip(a, b)]}
    for d, want in want_by_dir.items():
        got = _run(_module(f"  ROOT %r = pred[6]{{0}} compare(s32[6]{{0}} %p0, s32[6]{{0}} %p1), direction={d}", ["s32[6]{0}", "s32[6]{0}"], "pred[6]{0}"), [a, b])
        assert got.dtype == np.bool_ and got.tolist() == want, d
    # select(p, on_true, on_false); and / or / not on predicates
    body = """  %lt = pred[6]{0} compare(s32[6]{0} %p0, s32[6]{0} %p1), direction=LT
  %eq = pred[6]{0} compare(s32[6]{0} %p0, s32[6]{0} %p1), direction=EQ
  %nt = pred[6]{0} not(pred[6]{0} %eq)
  %an = pred[6]{0} and(pred[6]{0} %nt, pred[6]{0} %p2)
  %or = pred[6]{0} or(pred[6]{0} %lt, pred[6]{0} %an)
  ROOT %r = s32[6]{0} select(pred[6]{0} %or, s32[6]{0} %p0, s32[6]{0} %p1)"""
    c = np.array([True, False, True, True, False, True], np.bool_)
    got = _run(_module(body, ["s32[6]{0}", "s32[6]{0}", "pred[6]{0}"], "s32[6]{0}"), [a, b, c])
    want = [x if (x < y or ((not x == y) and z)) else y for x, y, z in zip(a.tolist(), b.tolist(), c.tolist())]
    assert got.tolist() == want and want == [1, 4, 3, 3, -2, 9]
    # clamp(lo, x, hi): operand order is (min, value, max)
    x = np.array([-5.0, 0.25, 7.0], np.float32)
    body = """  %lo = f32[] constant(-1)
  %hi = f32[] constant(2)
  %bl = f32[3]{0} broadcast(f32[] %lo), dimensions={}
  %bh = f32[3]{0} broadcast(f32[] %hi), dimensions={}
  ROOT %r = f32[3]{0} clamp(f32[3]{0} %bl, f32[3]{0} %p0, f32[3]{0} %bh)"""
    assert _run(_module(body, ["f32[3]{0}"], "f32[3]{0}"), [x]).tolist() == [-1.0, 0.25, 2.0]
    body = """  %mx = f32[3]{0} maximum(f32[3]{0} %p0, f32[3]{0} %p1)
  %mn = f32[3]{0} minimum(f32[3]{0} %p0, f32[3]{0} %p1)
  ROOT %r = f32[3]{0} subtract(f32[3]{0} %mx, f32[3]{0} %mn)"""
    y = np.array([1.0, -3.0, 7.5], np.float32)
    assert _run(_module(body, ["f32[3]{0}", "f32[3]{0}"], "f32[3]{0}"), [x, y]).tolist() == [6.0, 3.25, 0.5]


def test_dynamic_slice_clamps_its_start_indices():
    rng = np.random.default_rng(3)
    x = rng.integers(-100, 100, (5, 7)).astype(np.int32)
    body = "  ROOT %r = s32[2,3]{1,0} dynamic-slice(s32[5,7]{1,0} %p0, s32[] %p1, s32[] %p2), dynamic_slice_sizes={2,3}"
    text = _module(body, ["s32[5,7]{1,0}", "s32[]", "s32[]"], "s32[2,3]{1,0}")
    for i, j in [(0, 0), (1, 2), (3, 4), (4, 6), (-3, 9), (100, -100)]:
        got = _run(text, [x, np.array(i, np.int32), np.array(j, np.int32)])
        ci, cj = min(max(i, 0), 5 - 2), min(max(j, 0), 7 - 3)     # start clamped so that the slice fits
        want = [[int(x[ci + r][cj + c]) for c in range(3)] for r in range(2)]
        assert got.tolist() == want, (i, j)


def test_pad_low_high_and_value_against_np_pad():
    x = np.arange(6, dtype=np.float32).reshape(2, 3) + 1
    body = """  %v = f32[] constant(-2.5)
  ROOT %r = f32[5,6]{1,0} pad(f32[2,3]{1,0} %p0, f32[] %v), padding=1_2x3_0"""
    got = _run(_module(body, ["f32[2,3]{1,0}"], "f32[5,6]{1,0}"), [x])
    want = np.pad(x, ((1, 2), (3, 0)), constant_values=-2.5)
    assert np.array_equal(got, want) and got[1, 3] == 1.0 and got[0, 0] == -2.5


def test_slice_concatenate_broadcast_iota_transpose_by_brute_force():
    x = np.arange(24, dtype=np.int32).reshape(2, 3, 4)
    body = """  %tr = s32[4,2,3]{2,1,0} transpose(s32[2,3,4]{2,1,0} %p0), dimensions={2,0,1}
  %sl = s32[2,2,2]{2,1,0} slice(s32[4,2,3]{2,1,0} %tr), slice={[1:3], [0:2], [1:3]}
  %io = s32[2,2,1]{2,1,0} iota(), iota_dimension=1
  %cc = s32[2,2,3]{2,1,0} concatenate(s32[2,2,2]{2,1,0} %sl, s32[2,2,1]{2,1,0} %io), dimensions={2}
  %bc = s32[2,2,3]{2,1,0} broadcast(s32[3]{0} %p1), dimensions={2}
  ROOT %r = s32[2,2,3]{2,1,0} add(s32[2,2,3]{2,1,0} %cc, s32[2,2,3]{2,1,0} %bc)"""
    v = np.array([100, 200, 300], np.int32)
    got = _run(_module(body, ["s32[2,3,4]{2,1,0}", "s32[3]{0}"], "s32[2,2,3]{2,1,0}"), [x, v])
    want = np.zeros((2, 2, 3), np.int64)
    for i in range(2):
        for j in range(2):
            for k in range(3):
                # transposed[a,b,c] = x[b,c,a]; slice offsets (1,0,1); the third column is iota along dimension 1
                base = int(x[j, k + 1, i + 1]) if k < 2 else j
                want[i, j, k] = base + int(v[k])
    assert np.array_equal(got, want)


def _reducer(name, dtype, opcode):
    return f"""
%{name} {{
  %x = {dtype}[] parameter(0)
  %y = {dtype}[] parameter(1)
  ROOT %m = {dtype}[] {opcode}({dtype}[] %x, {dtype}[] %y)
}}
"""


REDUCERS = "".join(_reducer(n, t, o) for n, t, o in [("red_max", "f32", "maximum"), ("red_min", "f32", "minimum"), ("red_add", "f32", "add"),
                                                     ("red_mul", "f32", "multiply"), ("red_and", "pred", "and"), ("red_or", "pred", "or")])


@pytest.mark.parametrize("red,init,fold", [("red_max", "-inf", max), ("red_min", "inf", min), ("red_add", "0.5", lambda a, b: a + b),
                                           ("red_mul", "2", lambda a, b: a * b)])
def test_reduce_folds_the_init_value_into_every_row(red, init, fold):
    rng = np.random.default_rng(11)
    x = rng.integers(-3, 4, (4, 6)).astype(np.float32)
    body = f"""  %i = f32[] constant({init})
  ROOT %r = f32[4]{{0}} reduce(f32[4,6]{{1,0}} %p0, f32[] %i), dimensions={{1}}, to_apply=%{red}"""
    got = _run(_module(body, ["f32[4,6]{1,0}"], "f32[4]{0}", kind="kInput", extra=REDUCERS), [x])
    want = []
    for row in x.tolist():
        acc = float(init)
        for v in row:
            acc = fold(acc, v)
        want.append(acc)
    assert got.tolist() == want
    # the reduced dimension need not be the last one
    body = f"""  %i = f32[] constant({init})
  ROOT %r = f32[6]{{0}} reduce(f32[4,6]{{1,0}} %p0, f32[] %i), dimensions={{0}}, to_apply=%{red}"""
    got = _run(_module(body, ["f32[4,6]{1,0}"], "f32[6]{0}", kind="kInput", extra=REDUCERS), [x])
    for c in range(6):
        acc = float(init)
        for r in range(4):
            acc = fold(acc, float(x[r, c]))
        assert got[c] == acc


def test_predicate_reduces_and_infinite_inits_are_taken_as_written():
    p = np.array([[True, True, True], [True, False, True], [False, False, False]], np.bool_)
    for red, init, want in [("red_and", "true", [True, False, False]), ("red_or", "false", [True, True, False])]:
        body = f"""  %i = pred[] constant({init})
  ROOT %r = pred[3]{{0}} reduce(pred[3,3]{{1,0}} %p0, pred[] %i), dimensions={{1}}, to_apply=%{red}"""
        got = _run(_module(body, ["pred[3,3]{1,0}"], "pred[3]{0}", kind="kInput", extra=REDUCERS), [p])
        assert got.tolist() == want
    # A maximum over a row that holds nothing above -inf stays -inf: the init is used as written (XLA semantics).
    # The reference replaces an infinite init by the type's finite extreme (ir_parser_fused.cc:182-204: -65504 for
    # f16), which changes the result of exactly such rows and of no other; the oracle and the kernels do not.
    x = np.array([[-np.inf, -np.inf], [-np.inf, 3.0]], np.float16)
    body = """  %i = f16[] constant(-inf)
  ROOT %r = f16[2]{0} reduce(f16[2,2]{1,0} %p0, f16[] %i), dimensions={1}, to_apply=%red_max16"""
    extra = _reducer("red_max16", "f16", "maximum")
    got = _run(_module(body, ["f16[2,2]{1,0}"], "f16[2]{0}", kind="kInput", extra=extra), [x])
    assert np.isneginf(got[0]) and got[1] == 3.0
