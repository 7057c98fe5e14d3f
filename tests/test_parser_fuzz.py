"""Malformed HLO text must come back as an error code, never as a crash of the host process (the reference aborts
on every failure; this library's contract is `int` status + `mononn_last_error()`).  Seeded random edits of a valid
module - deleted spans, inserted tokens, swapped spans, dropped lines - run through the host compiler in a child
process, so that a segmentation fault fails the test instead of ending the test run."""
import subprocess
import sys
import textwrap

import pytest

from mononn_amd import MonoNNError, MonoNNModule
from mononn_amd.hlo import models

CHILD = textwrap.dedent('''
    import random, sys
    from mononn_amd import MonoNNModule, MonoNNError
    from mononn_amd.hlo import models
    text = models.bert_encoder(L=1, B=1, S=32, H=64, NH=2, F=128, vocab=50, max_pos=64).hlo_text
    rnd = random.Random(int(sys.argv[1]))
    toks = ["{", "}", "(", ")", ",", "[", "]", "=", "%", "f16", "s32", "fusion", "ROOT", "0", "-1", "99999999999", "kLoop", "dimensions={7}", "\\n", " "]
    ok = rejected = 0
    for it in range(int(sys.argv[2])):
        t = text
        for _ in range(rnd.randint(1, 4)):
            k, i = rnd.random(), rnd.randrange(len(t))
            if k < 0.3:
                t = t[:i] + t[i + rnd.randint(1, 30):]
            elif k < 0.6:
                t = t[:i] + rnd.choice(toks) + t[i:]
            elif k < 0.8:
                j = rnd.randrange(len(t))
                a, b = min(i, j), max(i, j)
                t = t[:a] + t[b:b + 20] + t[a + 20:b] + t[a:a + 20] + t[b + 20:]
            else:
                lines = t.split("\\n")
                lines.pop(rnd.randrange(len(lines)))
                t = "\\n".join(lines)
        print("case", it, flush=True)
        try:
            MonoNNModule.compile(t, build=False).close()
            ok += 1
        except MonoNNError:
            rejected += 1
    print("done", ok, rejected)
''')


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_edited_modules_are_rejected_or_compiled_never_a_crash(seed):
    r = subprocess.run([sys.executable, "-c", CHILD, str(seed), "120"], capture_output=True, text=True, timeout=600)
    last = r.stdout.strip().splitlines()[-1] if r.stdout.strip() else ""
    assert r.returncode == 0 and last.startswith("done"), f"host compiler crashed (exit {r.returncode}) after '{last}': {r.stderr[-500:]}"
    ok, rejected = (int(v) for v in last.split()[1:])
    assert rejected > 60          # most edits break the module, and each of those is an error return


def test_attributes_that_do_not_fit_the_shapes_are_parse_errors():
    # the case the random edits found first: a broadcast whose dimensions attribute is lost used to reach the index
    # maps with an empty vector
    text = models.bert_layer().hlo_text
    line = next(l for l in text.splitlines() if " broadcast(" in l and "dimensions={1}" in l)
    for bad in (line.replace("dimensions={1}", "dimenskLoopions={1}"), line.replace("dimensions={1}", "dimensions={5}"),
                line.replace("dimensions={1}", "dimensions={0,1}")):
        with pytest.raises(MonoNNError) as ei:
            MonoNNModule.compile(text.replace(line, bad), build=False)
        assert "broadcast" in str(ei.value) or "dimension" in str(ei.value)
    t = next(l for l in text.splitlines() if " transpose(" in l)
    import re
    perm = re.search(r"dimensions=\{([\d,]+)\}", t).group(1)
    with pytest.raises(MonoNNError):
        MonoNNModule.compile(text.replace(t, t.replace("{" + perm + "}", "{" + ",".join(["0"] * len(perm.split(","))) + "}")), build=False)


def test_misuse_of_the_c_abi_returns_error_codes():
    # NULL pointers, unknown names, calls in the wrong order: an error code and a message, never a crash
    import ctypes
    from mononn_amd import binding
    lib = binding._lib
    text = models.bert_layer().hlo_text.encode()
    h = ctypes.c_void_p()
    assert lib.mononn_compile(None, 0, None, None, 0, ctypes.byref(h)) != 0
    assert lib.mononn_compile(text, len(text), None, None, 0, None) != 0
    assert lib.mononn_compile(b"", 0, None, None, 0, ctypes.byref(h)) != 0 and b"HloModule" in lib.mononn_last_error()
    assert lib.mononn_compile(text, len(text), b"{not json", None, 0, ctypes.byref(h)) != 0 and b"JSON" in lib.mononn_last_error()
    assert lib.mononn_compile_from_spec_dir(text, len(text), b"/nonexistent/dir", ctypes.byref(h)) != 0
    assert lib.mononn_compile(text, len(text), None, None, 0, ctypes.byref(h)) == 0
    p, vp, n = ctypes.c_char_p(), ctypes.c_void_p(), ctypes.c_size_t()
    assert lib.mononn_module_source(h, None, ctypes.byref(p), ctypes.byref(n)) != 0
    assert lib.mononn_module_source(h, b"nope.txt", ctypes.byref(p), ctypes.byref(n)) != 0
    assert lib.mononn_module_code_object(h, ctypes.byref(vp), ctypes.byref(n)) != 0 and b"not been built" in lib.mononn_last_error()
    assert lib.mononn_module_set_constant(h, b"nope", b"abcd", 4) != 0 and b"no constant named" in lib.mononn_last_error()
    assert lib.mononn_module_set_constant(h, None, b"abcd", 4) != 0
    assert lib.mononn_module_load(h, 0) != 0                      # nothing built yet
    assert lib.mononn_launch(h, None, 0, None) != 0
    assert lib.mononn_module_dump(h, None) != 0
    assert lib.mononn_module_load(None, 0) != 0 and lib.mononn_launch(None, None, 0, None) != 0
    assert lib.mononn_module_summary(None, ctypes.byref(p), ctypes.byref(n)) != 0
    lib.mononn_module_destroy(None)
    lib.mononn_module_destroy(h)
