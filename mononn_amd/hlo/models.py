"""HLO fixtures for the model configurations the backend is measured on.

These play the role of the frozen TensorFlow graphs the reference feeds through XLA
(reference: examples/utils/save_model.py:96-110, examples/run_mononn.py:44-87): each
function returns the post-fusion HLO text of one model plus the description of its
inputs and constants.  The structure follows what XLA-GPU emits for a Hugging Face
encoder under auto mixed precision: fp16 tensors feed `__cublas$gemm` custom calls,
element-wise math runs in fp32 between explicit converts (the convention visible in
mononn_engine/optimization/topology_simplification_pass.cc:41-50), soft-max and
LayerNorm are chains of kInput reduce fusions and kLoop fusions.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import numpy as np

from .builder import Computation, HloModuleBuilder, Value

NP_DTYPE = {"f16": np.float16, "f32": np.float32, "s32": np.int32, "pred": np.bool_, "s64": np.int64}

# storage type of activations and weights in the fixtures below: "f16", or "bf16" inside bert_encoder(ftype="bf16")
_FT = "f16"


def _host_array(values, dtype):
    """values as the host buffer of HLO type `dtype` (bf16: uint16 bit patterns)."""
    if dtype == "bf16":
        from .. import bf16
        return np.ascontiguousarray(bf16.to_bits(values))
    return np.ascontiguousarray(np.asarray(values).astype(NP_DTYPE[dtype]))


@dataclass
class ModelFixture:
    name: str
    hlo_text: str
    params: List[dict]                 # [{name, dtype, dims, kind}]
    constants: Dict[str, dict]         # hlo constant name -> {role, dtype, dims}
    outputs: List[dict]                # [{dtype, dims}]
    config: dict = field(default_factory=dict)

    # ---- synthetic data ------------------------------------------------------------
    def make_constants(self, seed: int, init: str = "baseline") -> Dict[str, np.ndarray]:
        """Seeded weights.  init="baseline": kernels and embedding tables ~N(0,0.02), biases 0,
        LayerNorm gamma 1 / beta 0 (the measured configuration).  init="random": biases, gamma and
        beta are perturbed too, so a dropped bias or scale shows up in a parity test."""
        rng = np.random.default_rng(seed)
        out = {}
        for name, meta in self.constants.items():
            role, dims = meta["role"], meta["dims"]
            if role.endswith("/bias") or role.endswith("/beta"):
                a = rng.normal(0.0, 0.05, dims) if init == "random" else np.zeros(dims)
            elif role.endswith("/gamma"):
                a = 1.0 + rng.normal(0.0, 0.1, dims) if init == "random" else np.ones(dims)
            else:
                a = rng.normal(0.0, 0.02, dims)
            out[name] = _host_array(a, meta["dtype"])
        return out

    def make_inputs(self, seed: int) -> List[np.ndarray]:
        rng = np.random.default_rng(seed + 7919)
        arrs = []
        for p in self.params:
            dims, kind = p["dims"], p["kind"]
            if kind == "token_ids":
                a = rng.integers(0, p["vocab"], dims, dtype=np.int32)
            elif kind == "ones_mask":
                a = np.ones(dims, np.int32)
            elif kind == "length_mask":
                lens = rng.integers(p["min_len"], p["max_len"] + 1, dims[0])
                a = (np.arange(dims[1])[None, :] < lens[:, None]).astype(np.int32)
            elif kind == "zeros":
                a = _host_array(np.zeros(dims), p["dtype"])
            elif kind == "normal":
                a = _host_array(rng.normal(0.0, 1.0, dims), p["dtype"])
            elif kind == "uniform_pm1":
                a = _host_array(rng.uniform(-1.0, 1.0, dims), p["dtype"])
            else:
                raise ValueError(kind)
            arrs.append(np.ascontiguousarray(a))
        return arrs


# ----------------------------------------------------------------------------------------
# shared transformer pieces
# ----------------------------------------------------------------------------------------
def _bias_add_f16(f: Computation, g: Value, bias: Value) -> Value:
    rows, cols = g.dims
    x = f.add(f.convert(g, "f32"), f.broadcast(f.convert(bias, "f32"), (rows, cols), [1]))
    return f.convert(x, _FT)


def _layer_norm(e: Computation, mb: HloModuleBuilder, x: Value, gamma: Value, beta: Value,
                eps: float) -> Value:
    """LayerNorm over the last dim of f16[M,H] as XLA emits it: two kInput reduce fusions (sum,
    centred sum of squares) and one kLoop fusion that normalises (eps inside the rsqrt)."""
    M, H = x.dims
    add = mb.reducer("add", "f32")
    inv_h = 1.0 / H

    def sum_body(f, px):
        return f.reduce(f.convert(px, "f32"), f.scalar("f32", 0.0), 1, add)
    s = e.fusion("kInput", [x], sum_body)

    def centred(f, px, ps):
        mean = f.mul(ps, f.splat("f32", inv_h, (M,)))
        return f.sub(f.convert(px, "f32"), f.broadcast(mean, (M, H), [0]))

    def var_body(f, px, ps):
        d = centred(f, px, ps)
        return f.reduce(f.mul(d, d), f.scalar("f32", 0.0), 1, add)
    v = e.fusion("kInput", [x, s], var_body)

    def norm_body(f, px, ps, pv, pg, pb):
        d = centred(f, px, ps)
        var = f.mul(pv, f.splat("f32", inv_h, (M,)))
        r = f.rsqrt(f.add(var, f.splat("f32", eps, (M,))))
        y = f.mul(d, f.broadcast(r, (M, H), [0]))
        y = f.mul(y, f.broadcast(f.convert(pg, "f32"), (M, H), [1]))
        y = f.add(y, f.broadcast(f.convert(pb, "f32"), (M, H), [1]))
        return f.convert(y, _FT)
    return e.fusion("kLoop", [x, s, v, gamma, beta], norm_body)


def _gelu_tanh(f: Computation, x: Value) -> Value:
    dims = x.dims
    c = math.sqrt(2.0 / math.pi)
    x3 = f.mul(f.mul(x, x), x)
    inner = f.mul(f.splat("f32", c, dims), f.add(x, f.mul(f.splat("f32", 0.044715, dims), x3)))
    t = f.add(f.splat("f32", 1.0, dims), f.tanh(inner))
    return f.mul(f.mul(f.splat("f32", 0.5, dims), x), t)


def _attention(e: Computation, mb: HloModuleBuilder, h: Value, mask_add: Optional[Value],
               B: int, S: int, NH: int, D: int, W: dict, causal: bool) -> Value:
    """Self-attention block on f16[M,H]; returns the f16[M,H] context (before the output
    projection).  Scores and probabilities are materialised [B,NH,S,S], as in the reference
    (two batched GEMMs with a soft-max reduce cluster between them)."""
    H = NH * D
    M = B * S

    def head_proj(w, bias):
        g = e.gemm(h, w, 1, 0)

        def body(f, pg, pb):
            x16 = _bias_add_f16(f, pg, pb)
            return f.transpose(f.reshape(x16, (B, S, NH, D)), (0, 2, 1, 3))
        return e.fusion("kLoop", [g, bias], body)
    q = head_proj(W["q_w"], W["q_b"])
    k = head_proj(W["k_w"], W["k_b"])
    v = head_proj(W["v_w"], W["v_b"])
    scores = e.gemm(q, k, 3, 3, batch_dims=(0, 1), alpha=1.0 / math.sqrt(D))
    full = (B, NH, S, S)

    def logits(f, ps, pm):
        x = f.convert(ps, "f32")
        if pm is not None:
            x = f.add(x, f.broadcast(pm, full, [0, 3]))
        if causal:
            qi = f.iota("s32", full, 2)
            ki = f.iota("s32", full, 3)
            x = f.select(f.compare(ki, qi, "LE"), x, f.splat("f32", -10000.0, full))
        return x
    ops = [scores] + ([mask_add] if mask_add is not None else [])

    def split(params):
        return params[0], (params[1] if mask_add is not None else None), params[len(ops):]
    mx_r = mb.reducer("maximum", "f32")
    add_r = mb.reducer("add", "f32")

    def max_body(f, *p):
        ps, pm, _ = split(p)
        return f.reduce(logits(f, ps, pm), f.scalar("f32", float("-inf")), 3, mx_r)
    mx = e.fusion("kInput", ops, max_body)

    def sum_body(f, *p):
        ps, pm, (pmx,) = split(p)
        ex = f.exp(f.sub(logits(f, ps, pm), f.broadcast(pmx, full, [0, 1, 2])))
        return f.reduce(ex, f.scalar("f32", 0.0), 3, add_r)
    sm = e.fusion("kInput", ops + [mx], sum_body)

    def prob_body(f, *p):
        ps, pm, (pmx, psm) = split(p)
        ex = f.exp(f.sub(logits(f, ps, pm), f.broadcast(pmx, full, [0, 1, 2])))
        return f.convert(f.div(ex, f.broadcast(psm, full, [0, 1, 2])), _FT)
    probs = e.fusion("kLoop", ops + [mx, sm], prob_body)
    ctx = e.gemm(probs, v, 3, 2, batch_dims=(0, 1))

    def merge_heads(f, pc):
        return f.reshape(f.transpose(pc, (0, 2, 1, 3)), (M, H))
    return e.fusion("kLoop", [ctx], merge_heads)


def _residual_f16(e: Computation, g: Value, bias: Value, res: Value) -> Value:
    def body(f, pg, pb, pr):
        rows, cols = pg.dims
        x = f.add(f.convert(pg, "f32"), f.broadcast(f.convert(pb, "f32"), (rows, cols), [1]))
        return f.convert(f.add(x, f.convert(pr, "f32")), _FT)
    return e.fusion("kLoop", [g, bias, res], body)


def _ffn_act(e: Computation, g: Value, bias: Value) -> Value:
    def body(f, pg, pb):
        rows, cols = pg.dims
        x = f.add(f.convert(pg, "f32"), f.broadcast(f.convert(pb, "f32"), (rows, cols), [1]))
        return f.convert(_gelu_tanh(f, x), _FT)
    return e.fusion("kLoop", [g, bias], body)


def _layer_weights(e: Computation, prefix: str, H: int, F: int) -> dict:
    c = lambda role, dims: e.elided_constant(_FT, dims, f"{prefix}/{role}")
    return {
        "q_w": c("attention/query/kernel", (H, H)), "q_b": c("attention/query/bias", (H,)),
        "k_w": c("attention/key/kernel", (H, H)), "k_b": c("attention/key/bias", (H,)),
        "v_w": c("attention/value/kernel", (H, H)), "v_b": c("attention/value/bias", (H,)),
        "o_w": c("attention/output/kernel", (H, H)), "o_b": c("attention/output/bias", (H,)),
        "ln1_g": c("attention/LayerNorm/gamma", (H,)), "ln1_b": c("attention/LayerNorm/beta", (H,)),
        "f1_w": c("intermediate/kernel", (H, F)), "f1_b": c("intermediate/bias", (F,)),
        "f2_w": c("output/kernel", (F, H)), "f2_b": c("output/bias", (H,)),
        "ln2_g": c("output/LayerNorm/gamma", (H,)), "ln2_b": c("output/LayerNorm/beta", (H,)),
    }


def _post_ln_layer(e, mb, h, mask_add, B, S, NH, D, F, W, eps):
    ctx = _attention(e, mb, h, mask_add, B, S, NH, D, W, causal=False)
    x1 = _residual_f16(e, e.gemm(ctx, W["o_w"], 1, 0), W["o_b"], h)
    h1 = _layer_norm(e, mb, x1, W["ln1_g"], W["ln1_b"], eps)
    act = _ffn_act(e, e.gemm(h1, W["f1_w"], 1, 0), W["f1_b"])
    x2 = _residual_f16(e, e.gemm(act, W["f2_w"], 1, 0), W["f2_b"], h1)
    return _layer_norm(e, mb, x2, W["ln2_g"], W["ln2_b"], eps)


def _additive_mask(e: Computation, mask: Value) -> Value:
    """s32[B,S] 1/0 attention mask -> f32[B,S] additive term (1-mask)*-10000 (fp16-safe)."""
    def body(f, pm):
        one = f.splat("f32", 1.0, pm.dims)
        return f.mul(f.sub(one, f.convert(pm, "f32")), f.splat("f32", -10000.0, pm.dims))
    return e.fusion("kLoop", [mask], body)


# ----------------------------------------------------------------------------------------
# models
# ----------------------------------------------------------------------------------------
def bert_layer(B=1, S=128, H=768, NH=12, F=3072, eps=1e-12) -> ModelFixture:
    """One BERT encoder layer (post-LN, tanh-GELU) on a given hidden state."""
    mb = HloModuleBuilder("cluster_0__XlaCompiledKernel_true__XlaNumConstantArgs_0_.1")
    e = mb.entry
    hidden = e.parameter(_FT, (B, S, H), "hidden_states")
    mask = e.parameter("s32", (B, S), "attention_mask")
    W = _layer_weights(e, "bert/encoder/layer_0", H, F)
    h = e.bitcast(hidden, (B * S, H))
    out = _post_ln_layer(e, mb, h, _additive_mask(e, mask), B, S, NH, H // NH, F, W, eps)
    e.set_tuple_root([e.bitcast(out, (B, S, H))])
    return ModelFixture(
        "bert_layer", mb.text(),
        [{"name": "hidden_states", "dtype": _FT, "dims": [B, S, H], "kind": "normal"},
         {"name": "attention_mask", "dtype": "s32", "dims": [B, S], "kind": "ones_mask"}],
        mb.constants, [{"dtype": _FT, "dims": [B, S, H]}],
        dict(B=B, S=S, H=H, NH=NH, F=F, L=1))


def bert_encoder(L=12, B=1, S=128, H=768, NH=12, F=3072, vocab=30522, max_pos=512, types=2,
                 eps=1e-12, mask_kind="ones_mask", ftype="f16") -> ModelFixture:
    """Full BERT encoder: word + position + segment embedding gather, LayerNorm, L layers.
    Entry parameters are the three s32[B,S] tensors of the reference's example input
    (examples/data/bert_bs1.npy; 512 B each at B=1,S=128, README.md:192-194).
    ftype: storage type of weights and activations, "f16" (the reference's) or "bf16"."""
    global _FT
    assert ftype in ("f16", "bf16")
    saved, _FT = _FT, ftype
    try:
        return _bert_encoder(L, B, S, H, NH, F, vocab, max_pos, types, eps, mask_kind)
    finally:
        _FT = saved


def _bert_encoder(L, B, S, H, NH, F, vocab, max_pos, types, eps, mask_kind) -> ModelFixture:
    mb = HloModuleBuilder("cluster_0__XlaCompiledKernel_true__XlaNumConstantArgs_0_.1")
    e = mb.entry
    ids = e.parameter("s32", (B, S), "input_ids")
    mask = e.parameter("s32", (B, S), "attention_mask")
    tts = e.parameter("s32", (B, S), "token_type_ids")
    word = e.elided_constant(_FT, (vocab, H), "bert/embeddings/word_embeddings")
    pos = e.elided_constant(_FT, (max_pos, H), "bert/embeddings/position_embeddings")
    typ = e.elided_constant(_FT, (types, H), "bert/embeddings/token_type_embeddings")
    emb_g = e.elided_constant(_FT, (H,), "bert/embeddings/LayerNorm/gamma")
    emb_b = e.elided_constant(_FT, (H,), "bert/embeddings/LayerNorm/beta")

    def emb_body(f, pi, pt, pw, pp, pty):
        w = f.convert(f.gather_rows(pw, pi), "f32")
        t = f.convert(f.gather_rows(pty, pt), "f32")
        p = f.convert(f.broadcast(f.slice(pp, (0, 0), (S, H)), (B, S, H), [1, 2]), "f32")
        return f.convert(f.add(f.add(w, p), t), _FT)
    emb = e.fusion("kLoop", [ids, tts, word, pos, typ], emb_body)
    h = _layer_norm(e, mb, e.bitcast(emb, (B * S, H)), emb_g, emb_b, eps)
    mask_add = _additive_mask(e, mask)
    for l in range(L):
        W = _layer_weights(e, f"bert/encoder/layer_{l}", H, F)
        h = _post_ln_layer(e, mb, h, mask_add, B, S, NH, H // NH, F, W, eps)
    e.set_tuple_root([e.bitcast(h, (B, S, H))])
    mparam = {"name": "attention_mask", "dtype": "s32", "dims": [B, S], "kind": mask_kind}
    if mask_kind == "length_mask":
        mparam.update(min_len=max(1, S // 3), max_len=S)
    return ModelFixture(
        f"bert_L{L}_H{H}", mb.text(),
        [{"name": "input_ids", "dtype": "s32", "dims": [B, S], "kind": "token_ids", "vocab": vocab},
         mparam,
         {"name": "token_type_ids", "dtype": "s32", "dims": [B, S], "kind": "zeros"}],
        mb.constants, [{"dtype": _FT, "dims": [B, S, H]}],
        dict(B=B, S=S, H=H, NH=NH, F=F, L=L, vocab=vocab))


def bert_base(B=1, S=128, ftype="f16") -> ModelFixture:
    return bert_encoder(L=12, B=B, S=S, ftype=ftype)


def bert_large(B=16, S=384) -> ModelFixture:
    return bert_encoder(L=24, B=B, S=S, H=1024, NH=16, F=4096, mask_kind="length_mask")


def gemm_stage(M=6144, N=4096, K=1024) -> ModelFixture:
    """One weight GEMM at the shape of BERT-large's first feed-forward projection (16 x 384 rows), fed by an
    element-wise stage the way every GEMM inside an encoder is fed by the stage before it: f16[M,K] activations,
    constant f16[K,N] weights, f16[M,N] result.  Two stages, one grid barrier."""
    mb = HloModuleBuilder("cluster_0__XlaCompiledKernel_true__XlaNumConstantArgs_0_.1")
    e = mb.entry
    x = e.parameter(_FT, (M, K), "activations")

    def body(f, p):
        return f.convert(f.mul(f.convert(p, "f32"), f.splat("f32", 0.5, p.dims)), _FT)
    a = e.fusion("kLoop", [x], body)
    w = e.elided_constant(_FT, (K, N), "gemm_stage/kernel")
    e.set_tuple_root([e.gemm(a, w, 1, 0)])
    return ModelFixture(
        f"gemm_stage_{M}x{N}x{K}", mb.text(),
        [{"name": "activations", "dtype": _FT, "dims": [M, K], "kind": "normal"}],
        mb.constants, [{"dtype": _FT, "dims": [M, N]}], dict(M=M, N=N, K=K))


def gpt2(L=12, B=4, S=512, H=768, NH=12, F=3072, vocab=50257, max_pos=1024, eps=1e-5) -> ModelFixture:
    """GPT-2 style decoder prefill: token + learned position embeddings, L pre-LayerNorm layers with causal
    self-attention and tanh-GELU MLP, final LayerNorm, LM head tied to the token embedding
    (logits = h . wte^T, a GEMM whose right operand is contracted over its minor dimension)."""
    mb = HloModuleBuilder("cluster_0__XlaCompiledKernel_true__XlaNumConstantArgs_0_.1")
    e = mb.entry
    ids = e.parameter("s32", (B, S), "input_ids")
    wte = e.elided_constant(_FT, (vocab, H), "gpt2/wte")
    wpe = e.elided_constant(_FT, (max_pos, H), "gpt2/wpe")

    def emb_body(f, pi, pw, pp):
        w = f.convert(f.gather_rows(pw, pi), "f32")
        p = f.convert(f.broadcast(f.slice(pp, (0, 0), (S, H)), (B, S, H), [1, 2]), "f32")
        return f.convert(f.add(w, p), _FT)
    h = e.bitcast(e.fusion("kLoop", [ids, wte, wpe], emb_body), (B * S, H))
    D = H // NH
    for l in range(L):
        W = _layer_weights(e, f"gpt2/h_{l}", H, F)
        a = _layer_norm(e, mb, h, W["ln1_g"], W["ln1_b"], eps)
        ctx = _attention(e, mb, a, None, B, S, NH, D, W, causal=True)
        h = _residual_f16(e, e.gemm(ctx, W["o_w"], 1, 0), W["o_b"], h)
        m = _layer_norm(e, mb, h, W["ln2_g"], W["ln2_b"], eps)
        act = _ffn_act(e, e.gemm(m, W["f1_w"], 1, 0), W["f1_b"])
        h = _residual_f16(e, e.gemm(act, W["f2_w"], 1, 0), W["f2_b"], h)
    lnf_g = e.elided_constant(_FT, (H,), "gpt2/ln_f/gamma")
    lnf_b = e.elided_constant(_FT, (H,), "gpt2/ln_f/beta")
    hf = _layer_norm(e, mb, h, lnf_g, lnf_b, eps)
    logits = e.gemm(hf, wte, 1, 1)
    e.set_tuple_root([e.bitcast(logits, (B, S, vocab))])
    return ModelFixture(
        f"gpt2_L{L}_H{H}", mb.text(),
        [{"name": "input_ids", "dtype": "s32", "dims": [B, S], "kind": "token_ids", "vocab": vocab}],
        mb.constants, [{"dtype": _FT, "dims": [B, S, vocab]}],
        dict(B=B, S=S, H=H, NH=NH, F=F, L=L, vocab=vocab, eps=eps))


def vit(L=12, B=8, image=224, patch=16, H=768, NH=12, F=3072, eps=1e-6) -> ModelFixture:
    """ViT-B/16 style encoder: NCHW pixels -> NHWC, patch embedding as a strided forward convolution
    (`__cudnn$convForward`, window = stride = patch), class token + learned positions, L pre-LayerNorm layers
    without masking, final LayerNorm.  Output f16[B, 1 + (image/patch)^2, H]."""
    mb = HloModuleBuilder("cluster_0__XlaCompiledKernel_true__XlaNumConstantArgs_0_.1")
    e = mb.entry
    G = image // patch
    S = G * G + 1
    pixels = e.parameter(_FT, (B, 3, image, image), "pixel_values")
    filt = e.elided_constant(_FT, (H, patch, patch, 3), "vit/embeddings/patch_embeddings/kernel")
    pbias = e.elided_constant(_FT, (H,), "vit/embeddings/patch_embeddings/bias")
    cls = e.elided_constant(_FT, (1, 1, H), "vit/embeddings/cls_token")
    pos = e.elided_constant(_FT, (S, H), "vit/embeddings/position_embeddings")
    nhwc = e.fusion("kLoop", [pixels], lambda f, px: f.transpose(px, (0, 2, 3, 1)))
    conv = e.conv_forward(nhwc, filt, stride=(patch, patch))

    def bias_body(f, pc, pb):
        x = f.add(f.convert(pc, "f32"), f.broadcast(f.convert(pb, "f32"), pc.dims, [3]))
        return f.convert(x, _FT)
    patches = e.fusion("kLoop", [conv, pbias], bias_body)

    def emb_body(f, pp, pc, ppos):
        tok = f.concatenate([f.broadcast(f.reshape(pc, (H,)), (B, 1, H), [2]), f.reshape(pp, (B, G * G, H))], 1)
        x = f.add(f.convert(tok, "f32"), f.broadcast(f.convert(ppos, "f32"), (B, S, H), [1, 2]))
        return f.convert(x, _FT)
    h = e.bitcast(e.fusion("kLoop", [patches, cls, pos], emb_body), (B * S, H))
    D = H // NH
    for l in range(L):
        W = _layer_weights(e, f"vit/encoder/layer_{l}", H, F)
        a = _layer_norm(e, mb, h, W["ln1_g"], W["ln1_b"], eps)
        ctx = _attention(e, mb, a, None, B, S, NH, D, W, causal=False)
        h = _residual_f16(e, e.gemm(ctx, W["o_w"], 1, 0), W["o_b"], h)
        m = _layer_norm(e, mb, h, W["ln2_g"], W["ln2_b"], eps)
        act = _ffn_act(e, e.gemm(m, W["f1_w"], 1, 0), W["f1_b"])
        h = _residual_f16(e, e.gemm(act, W["f2_w"], 1, 0), W["f2_b"], h)
    lnf_g = e.elided_constant(_FT, (H,), "vit/layernorm/gamma")
    lnf_b = e.elided_constant(_FT, (H,), "vit/layernorm/beta")
    out = _layer_norm(e, mb, h, lnf_g, lnf_b, eps)
    e.set_tuple_root([e.bitcast(out, (B, S, H))])
    return ModelFixture(
        f"vit_L{L}_H{H}", mb.text(),
        [{"name": "pixel_values", "dtype": _FT, "dims": [B, 3, image, image], "kind": "uniform_pm1"}],
        mb.constants, [{"dtype": _FT, "dims": [B, S, H]}],
        dict(B=B, S=S, H=H, NH=NH, F=F, L=L, image=image, patch=patch, eps=eps))


def reference_example_inputs(S=128) -> List[np.ndarray]:
    """The reference's example feed (examples/data/bert_bs1.npy): ids [101, 7592 x (S-2), 102],
    attention mask all ones, segment ids all zeros, int32 [1,S].  The file itself is a pickled
    dict which the pickle-free loader refuses, so its documented content is rebuilt here."""
    ids = np.full((1, S), 7592, np.int32)
    ids[0, 0], ids[0, -1] = 101, 102
    return [ids, np.ones((1, S), np.int32), np.zeros((1, S), np.int32)]
