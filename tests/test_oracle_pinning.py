"""Pins the NumPy oracle (oracle/hlo_interp.py) against things it did not write itself: closed forms,
brute force in float64, torch library routines and an independent torch restatement of a whole
BERT layer.  A dropped term, a transposed operand or a wrong contraction index fails one of these."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from mononn_amd.hlo import models
from mononn_amd.hlo.builder import HloModuleBuilder
from oracle import hlo_interp


def _gemm_module(a_dims, b_dims, lhs_c, rhs_c, batch_dims=(), alpha=1.0, beta=0.0, with_c=False):
    mb = HloModuleBuilder("cluster_1__pin.1")
    e = mb.entry
    a = e.parameter("f32" if False else "f16", a_dims, "a")
    b = e.parameter("f16", b_dims, "b")
    c = None
    if with_c:
        r = len(a_dims)
        m = a_dims[r - 2] if lhs_c == r - 1 else a_dims[r - 1]
        n = b_dims[r - 1] if rhs_c == r - 2 else b_dims[r - 2]
        c = e.parameter("f16", list(a_dims[:r - 2]) + [m, n], "c")
    d = e.gemm(a, b, lhs_c, rhs_c, batch_dims=batch_dims, alpha=alpha, beta=beta, addend=c)
    e.set_tuple_root([d])
    return mb.text()


def test_gemm_brute_force_fp64_tiny():
    rng = np.random.default_rng(0)
    a = rng.normal(size=(5, 7)).astype(np.float16)
    b = rng.normal(size=(7, 3)).astype(np.float16)
    want = np.zeros((5, 3))
    for i in range(5):
        for j in range(3):
            for k in range(7):
                want[i, j] += float(a[i, k]) * float(b[k, j])
    got = hlo_interp.evaluate(_gemm_module([5, 7], [7, 3], 1, 0), [a, b], precision="fp32")[0]
    assert np.abs(got - want).max() < 1e-5


def test_f32_gemm_against_fp64_brute_force():
    # all-f32 GEMM (gemm_impl.cc:56, :229): no rounding to half anywhere, both right-operand layouts
    from test_gpu_parity import gemm_module
    rng = np.random.default_rng(21)
    for case in (dict(M=9, N=7, K=13, dtype="f32"), dict(M=6, N=5, K=11, dtype="f32", rhs_c=1), dict(M=4, N=3, K=5, batch=(2,), dtype="f32", rhs_c=2)):
        mb, a_dims, b_dims, d_dims = gemm_module(**case)
        a = rng.normal(size=a_dims).astype(np.float32) * 1000.0      # values a half would overflow or round visibly
        b = rng.normal(size=b_dims).astype(np.float32) + 1e-4
        for mode in ("fp32", "as_written"):
            got = hlo_interp.evaluate(mb.text(), [a, b], precision=mode)[0]
            bt = np.swapaxes(b, -1, -2) if case.get("rhs_c") == len(b_dims) - 1 else b
            want = np.zeros(d_dims)
            for idx in np.ndindex(*d_dims):
                lead, i, j = idx[:-2], idx[-2], idx[-1]
                want[idx] = sum(float(a[lead + (i, k)]) * float(bt[lead + (k, j)]) for k in range(case["K"]))
            assert got.dtype == np.float32 and np.abs(got - want).max() <= 1e-5 * np.abs(want).max(), (case, mode)


def test_gemm_row_major_example_shapes():
    # shapes / strides of the row-major worked example in the reference (gemm_impl.cc:290-303):
    # f16[512,384] = f16[512,128] x f16[128,384], contracting lhs 1 / rhs 0, lhs_stride 65536, rhs_stride 49152
    rng = np.random.default_rng(1)
    a = rng.normal(size=(512, 128)).astype(np.float16)
    b = rng.normal(size=(128, 384)).astype(np.float16)
    text = _gemm_module([512, 128], [128, 384], 1, 0)
    assert '\\"lhs_stride\\":\\"65536\\"' in text and '\\"rhs_stride\\":\\"49152\\"' in text
    got = hlo_interp.evaluate(text, [a, b], precision="fp32")[0]
    want = np.einsum("mk,kn->mn", a.astype(np.float64), b.astype(np.float64))
    assert got.shape == (512, 384) and np.abs(got - want).max() < 1e-3


def test_gemm_batched_transposed_example_shapes():
    # the column-major worked example (gemm_impl.cc:305-316): f16[4,2,128,128] from f16[4,2,64,128] and
    # f16[4,2,128,64], lhs contracting 2, rhs contracting 3, batch dims {0,1}, batch 8, strides 8192 / 8192
    rng = np.random.default_rng(2)
    a = rng.normal(size=(4, 2, 64, 128)).astype(np.float16)
    b = rng.normal(size=(4, 2, 128, 64)).astype(np.float16)
    text = _gemm_module([4, 2, 64, 128], [4, 2, 128, 64], 2, 3, batch_dims=(0, 1))
    assert '\\"batch_size\\":\\"8\\"' in text and '\\"lhs_stride\\":\\"8192\\"' in text
    got = hlo_interp.evaluate(text, [a, b], precision="fp32")[0]
    want = np.einsum("xykm,xynk->xymn", a.astype(np.float64), b.astype(np.float64))
    assert got.shape == (4, 2, 128, 128) and np.abs(got - want).max() < 1e-3


def test_gemm_alpha_beta_addend():
    rng = np.random.default_rng(3)
    a = rng.normal(size=(6, 8)).astype(np.float16)
    b = rng.normal(size=(8, 4)).astype(np.float16)
    c = rng.normal(size=(6, 4)).astype(np.float16)
    got = hlo_interp.evaluate(_gemm_module([6, 8], [8, 4], 1, 0, alpha=0.5, beta=2.0, with_c=True), [a, b, c],
                              precision="fp32")[0]
    want = 0.5 * a.astype(np.float64) @ b.astype(np.float64) + 2.0 * c.astype(np.float64)
    assert np.abs(got - want).max() < 1e-5


def test_as_written_rounds_to_half():
    rng = np.random.default_rng(4)
    a = rng.normal(size=(6, 64)).astype(np.float16)
    b = rng.normal(size=(64, 4)).astype(np.float16)
    got = hlo_interp.evaluate(_gemm_module([6, 64], [64, 4], 1, 0), [a, b])[0]
    assert got.dtype == np.float16
    want = (a.astype(np.float32) @ b.astype(np.float32)).astype(np.float16)
    assert np.array_equal(got, want)


def _single_fusion(build, params):
    mb = HloModuleBuilder("cluster_2__pin.1")
    e = mb.entry
    ps = [e.parameter(dt, dims, f"p{i}") for i, (dt, dims) in enumerate(params)]
    outs = build(e, mb, *ps)
    e.set_tuple_root(outs if isinstance(outs, list) else [outs])
    return mb.text()


def test_softmax_matches_torch():
    rng = np.random.default_rng(5)
    x = rng.normal(size=(2, 3, 8, 16)).astype(np.float32)

    def build(e, mb, px):
        full = (2, 3, 8, 16)
        mx = e.fusion("kInput", [px], lambda f, p: f.reduce(p, f.scalar("f32", float("-inf")), 3, mb.reducer("maximum", "f32")))
        sm = e.fusion("kInput", [px, mx], lambda f, p, m: f.reduce(f.exp(f.sub(p, f.broadcast(m, full, [0, 1, 2]))),
                                                                  f.scalar("f32", 0.0), 3, mb.reducer("add", "f32")))
        return e.fusion("kLoop", [px, mx, sm], lambda f, p, m, s: f.div(f.exp(f.sub(p, f.broadcast(m, full, [0, 1, 2]))),
                                                                         f.broadcast(s, full, [0, 1, 2])))
    got = hlo_interp.evaluate(_single_fusion(build, [("f32", (2, 3, 8, 16))]), [x])[0]
    want = torch.softmax(torch.tensor(x), -1).numpy()
    assert np.abs(got - want).max() < 1e-6
    assert np.abs(got.sum(-1) - 1).max() < 1e-5


def test_layer_norm_and_gelu_match_torch():
    rng = np.random.default_rng(6)
    x = rng.normal(size=(8, 32)).astype(np.float16)
    g = (1 + 0.1 * rng.normal(size=32)).astype(np.float16)
    b = (0.1 * rng.normal(size=32)).astype(np.float16)
    text = _single_fusion(lambda e, mb, px, pg, pb: models._layer_norm(e, mb, px, pg, pb, 1e-12),
                          [("f16", (8, 32)), ("f16", (32,)), ("f16", (32,))])
    got = hlo_interp.evaluate(text, [x, g, b], precision="fp32")[0]
    want = F.layer_norm(torch.tensor(x.astype(np.float32)), (32,), torch.tensor(g.astype(np.float32)),
                        torch.tensor(b.astype(np.float32)), 1e-12).numpy()
    assert np.abs(got - want).max() < 2e-5
    xs = rng.normal(size=(4, 16)).astype(np.float32) * 3
    text = _single_fusion(lambda e, mb, px: e.fusion("kLoop", [px], lambda f, p: models._gelu_tanh(f, p)), [("f32", (4, 16))])
    got = hlo_interp.evaluate(text, [xs])[0]
    assert np.abs(got - F.gelu(torch.tensor(xs), approximate="tanh").numpy()).max() < 1e-6


def test_gather_brute_force_and_clamp():
    rng = np.random.default_rng(7)
    table = rng.normal(size=(11, 5)).astype(np.float16)
    ids = np.array([[0, 10, 3], [7, 7, 2]], np.int32)
    text = _single_fusion(lambda e, mb, pt, pi: e.gather_rows(pt, pi), [("f16", (11, 5)), ("s32", (2, 3))])
    got = hlo_interp.evaluate(text, [table, ids])[0]
    for i in range(2):
        for j in range(3):
            assert np.array_equal(got[i, j], table[ids[i, j]])
    oob = np.array([[-4, 99, 3], [7, 7, 2]], np.int32)   # XLA clamps out-of-range start indices
    got = hlo_interp.evaluate(text, [table, oob])[0]
    assert np.array_equal(got[0, 0], table[0]) and np.array_equal(got[0, 1], table[10])


def test_shape_ops_against_numpy():
    rng = np.random.default_rng(8)
    x = rng.normal(size=(2, 3, 4)).astype(np.float32)

    def build(e, mb, px):
        def body(f, p):
            t = f.transpose(p, (2, 0, 1))                 # [4,2,3]
            r = f.reshape(t, (8, 3))
            s = f.slice(r, (2, 1), (6, 3))               # [4,2]
            c = f.concatenate([s, f.splat("f32", 7.0, (4, 1))], 1)   # [4,3]
            return f.add(c, f.convert(f.iota("s32", (4, 3), 1), "f32"))
        return e.fusion("kLoop", [px], body)
    got = hlo_interp.evaluate(_single_fusion(build, [("f32", (2, 3, 4))]), [x])[0]
    r = np.transpose(x, (2, 0, 1)).reshape(8, 3)[2:6, 1:3]
    want = np.concatenate([r, np.full((4, 1), 7.0, np.float32)], 1) + np.arange(3, dtype=np.float32)[None, :]
    assert np.array_equal(got, want)


def test_bert_layer_against_independent_torch_restatement():
    fx = models.bert_layer(B=1, S=32, H=128, NH=4, F=256)
    consts = fx.make_constants(11, "random")
    inputs = fx.make_inputs(11)
    got = hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0][0]
    R = {m["role"].split("layer_0/")[1]: torch.tensor(consts[n].astype(np.float32)) for n, m in fx.constants.items()}
    h = torch.tensor(inputs[0].astype(np.float32))[0]

    def lin(x, p):
        return x @ R[p + "/kernel"] + R[p + "/bias"]
    S, NH, D = 32, 4, 32
    q, k, v = (lin(h, "attention/" + n).view(S, NH, D).transpose(0, 1) for n in ("query", "key", "value"))
    p = torch.softmax(q @ k.transpose(1, 2) / math.sqrt(D), -1)
    ctx = (p @ v).transpose(0, 1).reshape(S, NH * D)
    x1 = F.layer_norm(lin(ctx, "attention/output") + h, (128,), R["attention/LayerNorm/gamma"], R["attention/LayerNorm/beta"], 1e-12)
    a = F.gelu(lin(x1, "intermediate"), approximate="tanh")
    x2 = F.layer_norm(lin(a, "output") + x1, (128,), R["output/LayerNorm/gamma"], R["output/LayerNorm/beta"], 1e-12)
    assert np.abs(got - x2.numpy()).max() < 2e-5


def test_masked_encoder_against_torch():
    # padding mask (1/0) -> additive -10000 on padded keys; embeddings gathered by id
    fx = models.bert_encoder(L=1, B=2, S=16, H=64, NH=2, F=128, vocab=50, max_pos=32, mask_kind="length_mask")
    consts = fx.make_constants(12, "random")
    inputs = fx.make_inputs(12)
    got = hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0]
    by_role = {m["role"]: torch.tensor(consts[n].astype(np.float32)) for n, m in fx.constants.items()}
    ids, mask, tt = (torch.tensor(a.astype(np.int64)) for a in inputs)
    emb = by_role["bert/embeddings/word_embeddings"][ids] + by_role["bert/embeddings/position_embeddings"][:16][None] + \
        by_role["bert/embeddings/token_type_embeddings"][tt]
    h = F.layer_norm(emb, (64,), by_role["bert/embeddings/LayerNorm/gamma"], by_role["bert/embeddings/LayerNorm/beta"], 1e-12)
    add = (1.0 - mask.float()) * -10000.0
    P = "bert/encoder/layer_0/"

    def lin(x, p):
        return x @ by_role[P + p + "/kernel"] + by_role[P + p + "/bias"]
    q, k, v = (lin(h, "attention/" + n).view(2, 16, 2, 32).transpose(1, 2) for n in ("query", "key", "value"))
    s = q @ k.transpose(2, 3) / math.sqrt(32) + add[:, None, None, :]
    ctx = (torch.softmax(s, -1) @ v).transpose(1, 2).reshape(2, 16, 64)
    x1 = F.layer_norm(lin(ctx, "attention/output") + h, (64,), by_role[P + "attention/LayerNorm/gamma"], by_role[P + "attention/LayerNorm/beta"], 1e-12)
    a = F.gelu(lin(x1, "intermediate"), approximate="tanh")
    x2 = F.layer_norm(lin(a, "output") + x1, (64,), by_role[P + "output/LayerNorm/gamma"], by_role[P + "output/LayerNorm/beta"], 1e-12)
    assert np.abs(got - x2.numpy()).max() < 3e-5


def test_reference_example_input_shape():
    ids, mask, seg = models.reference_example_inputs()
    assert ids.dtype == np.int32 and ids.shape == (1, 128) and ids.nbytes == 512
    assert ids[0, 0] == 101 and ids[0, -1] == 102 and (ids[0, 1:-1] == 7592).all()
    assert mask.all() and not seg.any()


def test_gpt2_decoder_against_torch():
    # pre-LN decoder, causal mask built from iota/compare/select, LM head tied to the token embedding
    B, S, H, NH, Fd, V = 2, 24, 64, 4, 128, 97
    fx = models.gpt2(L=2, B=B, S=S, H=H, NH=NH, F=Fd, vocab=V, max_pos=32)
    consts = fx.make_constants(21, "random")
    inputs = fx.make_inputs(21)
    got = hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0]
    R = {m["role"]: torch.tensor(consts[n].astype(np.float32)) for n, m in fx.constants.items()}
    ids = torch.tensor(inputs[0].astype(np.int64))
    h = R["gpt2/wte"][ids] + R["gpt2/wpe"][:S][None]
    D = H // NH
    causal = torch.tril(torch.ones(S, S, dtype=torch.bool))
    for l in range(2):
        P = f"gpt2/h_{l}/"

        def lin(x, p):
            return x @ R[P + p + "/kernel"] + R[P + p + "/bias"]
        a = F.layer_norm(h, (H,), R[P + "attention/LayerNorm/gamma"], R[P + "attention/LayerNorm/beta"], 1e-5)
        q, k, v = (lin(a, "attention/" + n).view(B, S, NH, D).transpose(1, 2) for n in ("query", "key", "value"))
        s = q @ k.transpose(2, 3) / math.sqrt(D)
        s = torch.where(causal, s, torch.tensor(-10000.0))
        ctx = (torch.softmax(s, -1) @ v).transpose(1, 2).reshape(B, S, H)
        h = h + lin(ctx, "attention/output")
        m = F.layer_norm(h, (H,), R[P + "output/LayerNorm/gamma"], R[P + "output/LayerNorm/beta"], 1e-5)
        h = h + lin(F.gelu(lin(m, "intermediate"), approximate="tanh"), "output")
    hf = F.layer_norm(h, (H,), R["gpt2/ln_f/gamma"], R["gpt2/ln_f/beta"], 1e-5)
    want = (hf @ R["gpt2/wte"].T).numpy()
    assert got.shape == want.shape
    assert np.abs(got - want).max() < 3e-5


def _conv_module(xd, fd, stride, pad):
    mb = HloModuleBuilder("cluster_9__conv.1")
    e = mb.entry
    x = e.parameter("f16", xd, "x")
    f = e.parameter("f16", fd, "f")
    e.set_tuple_root([e.conv_forward(x, f, stride=stride, pad=pad)])
    return mb.text()


@pytest.mark.parametrize("xd,fd,stride,pad", [((2, 9, 10, 4), (6, 3, 3, 4), (2, 1), (1, 1)),
                                              ((1, 12, 12, 3), (5, 4, 4, 3), (4, 4), (0, 0)),
                                              ((3, 7, 5, 2), (4, 1, 1, 2), (1, 1), (0, 0)),
                                              ((2, 8, 8, 8), (16, 5, 3, 8), (1, 2), (2, 1))])
def test_conv_forward_matches_torch_conv2d(xd, fd, stride, pad):
    # N,H,W,C input, K,R,S,C filter, N,P,Q,K output against the library routine on NCHW / OIHW
    rng = np.random.default_rng(31)
    x = rng.normal(0, 1, xd).astype(np.float16)
    w = rng.normal(0, 1, fd).astype(np.float16)
    got = hlo_interp.evaluate(_conv_module(xd, fd, stride, pad), [x, w], {}, "fp32")[0]
    want = F.conv2d(torch.tensor(x.astype(np.float32)).permute(0, 3, 1, 2), torch.tensor(w.astype(np.float32)).permute(0, 3, 1, 2),
                    stride=stride, padding=pad).permute(0, 2, 3, 1).numpy()
    assert got.shape == want.shape
    assert np.abs(got - want).max() < 2e-5


def test_vit_encoder_against_torch():
    B, image, patch, H, NH, Fd = 2, 32, 8, 64, 4, 128
    fx = models.vit(L=2, B=B, image=image, patch=patch, H=H, NH=NH, F=Fd)
    consts = fx.make_constants(23, "random")
    inputs = fx.make_inputs(23)
    got = hlo_interp.evaluate(fx.hlo_text, inputs, consts, "fp32")[0]
    R = {m["role"]: torch.tensor(consts[n].astype(np.float32)) for n, m in fx.constants.items()}
    px = torch.tensor(inputs[0].astype(np.float32))
    S, D = (image // patch) ** 2 + 1, H // NH
    emb = F.conv2d(px, R["vit/embeddings/patch_embeddings/kernel"].permute(0, 3, 1, 2), R["vit/embeddings/patch_embeddings/bias"], stride=patch)
    # the patch embedding is rounded to fp16 where the HLO says so only in "as_written" mode; fp32 mode keeps it wide
    tok = torch.cat([R["vit/embeddings/cls_token"].expand(B, 1, H), emb.flatten(2).transpose(1, 2)], 1)
    h = tok + R["vit/embeddings/position_embeddings"][None]
    for l in range(2):
        P = f"vit/encoder/layer_{l}/"

        def lin(x, p):
            return x @ R[P + p + "/kernel"] + R[P + p + "/bias"]
        a = F.layer_norm(h, (H,), R[P + "attention/LayerNorm/gamma"], R[P + "attention/LayerNorm/beta"], 1e-6)
        q, k, v = (lin(a, "attention/" + n).view(B, S, NH, D).transpose(1, 2) for n in ("query", "key", "value"))
        ctx = (torch.softmax(q @ k.transpose(2, 3) / math.sqrt(D), -1) @ v).transpose(1, 2).reshape(B, S, H)
        h = h + lin(ctx, "attention/output")
        m = F.layer_norm(h, (H,), R[P + "output/LayerNorm/gamma"], R[P + "output/LayerNorm/beta"], 1e-6)
        h = h + lin(F.gelu(lin(m, "intermediate"), approximate="tanh"), "output")
    want = F.layer_norm(h, (H,), R["vit/layernorm/gamma"], R["vit/layernorm/beta"], 1e-6).numpy()
    assert got.shape == want.shape
    assert np.abs(got - want).max() < 5e-5


def test_dot_matches_einsum_and_the_gemm_call():
    # a plain `dot` means the same contraction as the cuBLAS call with alpha 1 / beta 0
    rng = np.random.default_rng(33)
    A = rng.normal(0, 1, (3, 40, 64)).astype(np.float16)
    B = rng.normal(0, 1, (3, 24, 64)).astype(np.float16)
    texts = []
    for kind in ("dot", "gemm"):
        mb = HloModuleBuilder("cluster_5__dot.1")
        e = mb.entry
        a = e.parameter("f16", A.shape, "a")
        b = e.parameter("f16", B.shape, "b")
        d = e.dot(a, b, 2, 2, batch_dims=(0,)) if kind == "dot" else e.gemm(a, b, 2, 2, batch_dims=(0,))
        e.set_tuple_root([d])
        texts.append(mb.text())
    got_dot = hlo_interp.evaluate(texts[0], [A, B], {}, "fp32")[0]
    got_gemm = hlo_interp.evaluate(texts[1], [A, B], {}, "fp32")[0]
    want = np.einsum("bmk,bnk->bmn", A.astype(np.float64), B.astype(np.float64))
    assert np.abs(got_dot - want).max() < 2e-5
    assert np.array_equal(got_dot, got_gemm)


@pytest.mark.parametrize("epilogue", ["DEFAULT", "BIAS", "RELU", "GELU", "BIAS_RELU", "BIAS_GELU"])
def test_lt_matmul_matches_einsum_and_the_closed_forms(epilogue):
    # the newer spelling of the cuBLAS call: D = act(alpha A.B + beta C + bias) against einsum in fp64 and torch's
    # relu / tanh-approximated gelu as library routines (a dropped bias, a bias along the rows instead of the columns,
    # the erf form of GELU or an activation applied before the addend all fail here)
    rng = np.random.default_rng(47)
    M, K, N = 24, 40, 56
    A = rng.normal(0, 1, (M, K)).astype(np.float16)
    B = rng.normal(0, 1, (N, K)).astype(np.float16)          # stored [N, K]: contracting dimension 1
    C = rng.normal(0, 1, (M, N)).astype(np.float16)
    bias = rng.normal(0, 2, (N,)).astype(np.float16)
    mb = HloModuleBuilder("cluster_5__lt.1")
    e = mb.entry
    a, b, c = e.parameter("f16", A.shape, "a"), e.parameter("f16", B.shape, "b"), e.parameter("f16", C.shape, "c")
    bv = e.parameter("f16", bias.shape, "bias") if epilogue.startswith("BIAS") else None
    e.set_tuple_root([e.lt_matmul(a, b, 1, 1, epilogue=epilogue, bias=bv, alpha=0.5, beta=2.0, addend=c)])
    feeds = [A, B, C] + ([bias] if bv is not None else [])
    got = hlo_interp.evaluate(mb.text(), feeds, {}, "fp32")[0].astype(np.float64)
    want = 0.5 * np.einsum("mk,nk->mn", A.astype(np.float64), B.astype(np.float64)) + 2.0 * C.astype(np.float64)
    if bv is not None:
        want = want + bias.astype(np.float64)[None, :]
    t = torch.tensor(want)
    if epilogue.endswith("RELU"):
        want = torch.relu(t).numpy()
    if epilogue.endswith("GELU"):
        want = torch.nn.functional.gelu(t, approximate="tanh").numpy()
    assert np.abs(got - want).max() < 3e-5
    # as written (f16 result): one rounding of the fp32 value
    got16 = hlo_interp.evaluate(mb.text(), feeds, {})[0]
    assert got16.dtype == np.float16 and np.abs(got16.astype(np.float64) - want).max() <= 2.0 ** -11 * np.abs(want).max() + 1e-6


def test_lt_matmul_with_a_workspace_tuple_and_numbered_epilogue():
    # (matrix, workspace) result read through get-tuple-element, fields not nested, epilogue given by its enum number
    text = """HloModule cluster_5__lt2.1

ENTRY %main (a: f16[8,16], b: f16[16,4], bias: f16[4]) -> (f16[8,4]) {
  %a = f16[8,16]{1,0} parameter(0)
  %b = f16[16,4]{1,0} parameter(1)
  %bias = f16[4]{0} parameter(2)
  %lt = (f16[8,4]{1,0}, s8[256]{0}) custom-call(f16[8,16]{1,0} %a, f16[16,4]{1,0} %b, f16[4]{0} %bias), custom_call_target="__cublas$lt$matmul", backend_config="{\\"alpha_real\\":1,\\"alpha_imag\\":0,\\"beta\\":0,\\"dot_dimension_numbers\\":{\\"lhs_contracting_dimensions\\":[\\"1\\"],\\"rhs_contracting_dimensions\\":[\\"0\\"],\\"lhs_batch_dimensions\\":[],\\"rhs_batch_dimensions\\":[]},\\"epilogue\\":3}"
  %d = f16[8,4]{1,0} get-tuple-element((f16[8,4]{1,0}, s8[256]{0}) %lt), index=0
  ROOT %t = (f16[8,4]{1,0}) tuple(f16[8,4]{1,0} %d)
}
"""
    rng = np.random.default_rng(48)
    A, B, bias = rng.normal(0, 1, (8, 16)).astype(np.float16), rng.normal(0, 1, (16, 4)).astype(np.float16), rng.normal(0, 1, (4,)).astype(np.float16)
    got = hlo_interp.evaluate(text, [A, B, bias], {}, "fp32")[0]
    want = np.maximum(A.astype(np.float64) @ B.astype(np.float64) + bias.astype(np.float64), 0)   # 3 = BIAS_RELU
    assert np.abs(got - want).max() < 1e-5


@pytest.mark.parametrize("xd,size,stride,pad", [
    ((2, 9, 10, 8), (1, 3, 3, 1), (1, 2, 2, 1), ((0, 0), (1, 1), (1, 1), (0, 0))),
    ((1, 8, 8, 4), (1, 2, 2, 1), (1, 2, 2, 1), ((0, 0), (0, 0), (0, 0), (0, 0))),
    ((3, 7, 5, 2), (1, 3, 2, 1), (1, 1, 2, 1), ((0, 0), (1, 1), (0, 1), (0, 0))),
])
def test_reduce_window_matches_torch_pooling(xd, size, stride, pad):
    # max pooling against the library routine (padding = -inf); sum pooling against avg_pool2d * window size with
    # zero padding counted in (padding = the init value 0)
    from op_cases import pool_module
    rng = np.random.default_rng(41)
    x = rng.normal(0, 1, xd).astype(np.float16)
    t = torch.tensor(x.astype(np.float32)).permute(0, 3, 1, 2)
    sym = all(lo == hi for lo, hi in pad)
    text, od = pool_module(xd, size, stride, pad, "max")
    got = hlo_interp.evaluate(text, [x], {}, "fp32")[0]
    tp = F.pad(t, (pad[2][0], pad[2][1], pad[1][0], pad[1][1]), value=float("-inf"))
    want = F.max_pool2d(tp, size[1:3], stride[1:3]).permute(0, 2, 3, 1).numpy()
    assert list(got.shape) == od == list(want.shape)
    assert np.array_equal(got, want)
    text, _ = pool_module(xd, size, stride, pad, "sum", dtype="f32")
    got = hlo_interp.evaluate(text, [x.astype(np.float32)], {}, "fp32")[0]
    tz = F.pad(t, (pad[2][0], pad[2][1], pad[1][0], pad[1][1]), value=0.0)
    want = (F.avg_pool2d(tz, size[1:3], stride[1:3]) * (size[1] * size[2])).permute(0, 2, 3, 1).numpy()
    assert np.abs(got - want).max() < 1e-5
    assert sym or got.shape == want.shape


def test_dynamic_update_slice_matches_numpy_assignment_with_clamped_starts():
    from op_cases import update_slice_module
    rng = np.random.default_rng(43)
    x = rng.normal(0, 1, (6, 10, 8)).astype(np.float16)
    u = rng.normal(0, 1, (2, 4, 8)).astype(np.float16)
    text = update_slice_module(x.shape, u.shape)
    for starts in [(1, 3, 0), (0, 0, 0), (4, 6, 0), (9, -5, 3)]:      # the last one is clamped to (4, 0, 0)
        got = hlo_interp.evaluate(text, [x, u] + [np.array(s, np.int32) for s in starts], {})[0]
        s = [min(max(v, 0), n - m) for v, n, m in zip(starts, x.shape, u.shape)]
        want = x.copy()
        want[s[0]:s[0] + 2, s[1]:s[1] + 4, s[2]:s[2] + 8] = u
        assert np.array_equal(got, want)


def test_variadic_reduce_is_argmax_with_first_index_on_ties():
    from op_cases import arg_reduce_module
    rng = np.random.default_rng(47)
    x = rng.integers(-4, 5, (7, 50)).astype(np.float16)      # many ties
    v, i = hlo_interp.evaluate(arg_reduce_module(7, 50, "GT"), [x], {})
    assert np.array_equal(i, np.argmax(x, axis=1).astype(np.int32)) and np.array_equal(v, x.max(axis=1))
    v, i = hlo_interp.evaluate(arg_reduce_module(7, 50, "LT"), [x], {})
    assert np.array_equal(i, np.argmin(x, axis=1).astype(np.int32)) and np.array_equal(v, x.min(axis=1))


def test_bf16_conversions_match_torch_bfloat16():
    # bf16 has no NumPy type: the oracle and the product's boundary both carry it as uint16 bit patterns and convert by
    # rounding the float32 pattern to nearest even on its upper half.  torch.bfloat16 is the independent statement.
    from mononn_amd import bf16
    rng = np.random.default_rng(71)
    x = np.concatenate([rng.normal(0, 1, 4096), rng.normal(0, 1e-3, 1024), rng.normal(0, 1e4, 1024),
                        [0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, 65504.0, 3.3895314e38, 1e-40, -1e-40],
                        # exact ties between two bf16 neighbours: 1 + 2^-8 (down to even), 1 + 3 * 2^-8 (up to even)
                        [1.00390625, 1.01171875, -1.00390625, 257.0, 259.0]]).astype(np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    for to_bits, from_bits in ((hlo_interp.bf16_to_bits, hlo_interp.bf16_from_bits), (bf16.to_bits, bf16.from_bits)):
        got = to_bits(x)
        assert got.dtype == np.uint16 and np.array_equal(got, want)
        back = from_bits(got)
        assert np.array_equal(back, torch.from_numpy(want.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy())
    assert np.isnan(hlo_interp.bf16_from_bits(hlo_interp.bf16_to_bits(np.array([np.nan], np.float32))))[0]
    assert np.isnan(bf16.from_bits(bf16.to_bits(np.array([np.nan], np.float32))))[0]


def test_bf16_program_as_written_rounds_like_torch_bfloat16():
    # convert, an element-wise chain and a GEMM in bf16: every bf16-typed instruction result is a bf16 value
    M, K, N = 24, 40, 16
    mb = HloModuleBuilder("cluster_5__bf16_pin.1")
    e = mb.entry
    a = e.parameter("bf16", (M, K), "a")
    b = e.parameter("bf16", (K, N), "b")
    bias = e.parameter("f32", (N,), "bias")
    d = e.gemm(a, b, 1, 0)

    def body(f, pd, pb):
        y = f.add(f.convert(pd, "f32"), f.broadcast(pb, (M, N), [1]))
        h = f.convert(y, "bf16")                       # rounded
        return f.mul(h, h)                             # bf16 x bf16 -> bf16: the product rounded once
    out = e.fusion("kLoop", [d, bias], body)
    e.set_tuple_root([out])
    rng = np.random.default_rng(72)
    av, bv = rng.normal(0, 1, (M, K)).astype(np.float32), rng.normal(0, 1, (K, N)).astype(np.float32)
    biasv = rng.normal(0, 1, N).astype(np.float32)
    a_bits, b_bits = hlo_interp.bf16_to_bits(av), hlo_interp.bf16_to_bits(bv)
    got = hlo_interp.evaluate(mb.text(), [a_bits, b_bits, biasv], {}, "as_written")[0]
    ta = torch.from_numpy(av).to(torch.bfloat16).to(torch.float32)
    tb = torch.from_numpy(bv).to(torch.bfloat16).to(torch.float32)
    dd = (ta.double() @ tb.double()).to(torch.float32).to(torch.bfloat16)          # GEMM result stored as bf16
    h = (dd.to(torch.float32) + torch.from_numpy(biasv)).to(torch.bfloat16)
    want = (h.to(torch.float32) * h.to(torch.float32)).to(torch.bfloat16).to(torch.float32).numpy()
    assert got.dtype == np.float32
    # fp32 accumulation order may move a GEMM element by one bf16 step before the squaring
    steps = np.abs(got - want) / np.maximum(np.abs(want) * 2.0 ** -7, 1e-30)
    assert (steps <= 2.5).all() and (got == want).mean() > 0.97
    assert np.array_equal(hlo_interp.round_to_bf16(got), got)          # results are bf16 values
    # the fp32 mode carries the same program without intermediate rounding
    free = hlo_interp.evaluate(mb.text(), [a_bits, b_bits, biasv], {}, "fp32")[0]
    exact = ((ta.double() @ tb.double()).float() + torch.from_numpy(biasv)).numpy() ** 2
    assert np.allclose(free, exact, rtol=1e-5, atol=1e-5)
