"""Writes the golden vectors under tests/golden/.

    python tests/golden/make_golden.py

Expected outputs come from a torch (CPU, fp32) restatement of the BERT encoder written against the
textbook definitions -- F.layer_norm, F.gelu(approximate="tanh"), torch.softmax, `@` -- and never from the
HLO interpreter under oracle/ nor from the HIP kernels, so the same file pins both.  Inputs and weights are
not stored: they are regenerated from their seeds by ModelFixture.make_constants / make_inputs.

The reference ships no expected outputs for this path (its harness only times the model,
examples/run_mononn.py:74-87); its one data file, examples/data/bert_bs1.npy, is the input feed whose
documented content (README.md:192-194) models.reference_example_inputs() rebuilds.
"""
import math
import os
import sys

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from mononn_amd.hlo import models  # noqa: E402

# (file stem, fixture factory, seed, init, input override)
CASES = {
    "bert_layer_b1_s128": (lambda: models.bert_layer(), 1234, "baseline", None),
    "bert_base_b1_s128": (lambda: models.bert_base(), 1235, "baseline", None),
    "bert_base_b1_s128_example_feed": (lambda: models.bert_base(), 1235, "baseline", models.reference_example_inputs),
    "bert_small_masked_b2_s48": (lambda: models.bert_encoder(L=2, B=2, S=48, H=128, NH=4, F=512, vocab=1000, max_pos=64,
                                                             mask_kind="length_mask"), 77, "random", None),
}


def torch_encoder(fx, consts, inputs):
    """Post-LN BERT encoder in fp32.  Weights are the fp16 values widened, as the HLO reads them."""
    cfg = fx.config
    R = {m["role"]: torch.tensor(consts[n].astype(np.float32)) for n, m in fx.constants.items()}
    B, S, H, NH, L = cfg["B"], cfg["S"], cfg["H"], cfg["NH"], cfg["L"]
    D = H // NH
    if fx.name == "bert_layer":
        h = torch.tensor(inputs[0].astype(np.float32))
        mask = torch.tensor(inputs[1].astype(np.int64))
    else:
        ids, mask, tt = (torch.tensor(a.astype(np.int64)) for a in inputs)
        emb = R["bert/embeddings/word_embeddings"][ids] + R["bert/embeddings/position_embeddings"][:S][None] + \
            R["bert/embeddings/token_type_embeddings"][tt]
        h = F.layer_norm(emb, (H,), R["bert/embeddings/LayerNorm/gamma"], R["bert/embeddings/LayerNorm/beta"], 1e-12)
    add = (1.0 - mask.float()) * -10000.0
    for l in range(L):
        P = f"bert/encoder/layer_{l}/"

        def lin(x, p):
            return x @ R[P + p + "/kernel"] + R[P + p + "/bias"]
        q, k, v = (lin(h, "attention/" + n).view(B, S, NH, D).transpose(1, 2) for n in ("query", "key", "value"))
        s = q @ k.transpose(2, 3) / math.sqrt(D) + add[:, None, None, :]
        ctx = (torch.softmax(s, -1) @ v).transpose(1, 2).reshape(B, S, H)
        x1 = F.layer_norm(lin(ctx, "attention/output") + h, (H,), R[P + "attention/LayerNorm/gamma"],
                          R[P + "attention/LayerNorm/beta"], 1e-12)
        a = F.gelu(lin(x1, "intermediate"), approximate="tanh")
        h = F.layer_norm(lin(a, "output") + x1, (H,), R[P + "output/LayerNorm/gamma"], R[P + "output/LayerNorm/beta"], 1e-12)
    return h.numpy()


def case_data(stem):
    make, seed, init, feed = CASES[stem]
    fx = make()
    consts = fx.make_constants(seed, init)
    inputs = feed() if feed else fx.make_inputs(seed)
    return fx, consts, inputs


def main():
    torch.manual_seed(0)
    for stem in CASES:
        fx, consts, inputs = case_data(stem)
        out = torch_encoder(fx, consts, inputs).astype(np.float32)
        # fp16 storage halves the files; the tests compare with tolerances far above half an fp16 ulp
        np.save(os.path.join(HERE, stem + ".npy"), out.astype(np.float16))
        print(stem, out.shape, "abs max %.3f" % np.abs(out).max())
    # embedding gather: ids and the rows they must select, bit for bit
    rng = np.random.default_rng(5)
    table = rng.normal(0, 1, (97, 40)).astype(np.float16)
    ids = rng.integers(0, 97, (3, 11), dtype=np.int32)
    np.savez(os.path.join(HERE, "gather_rows.npz"), table=table, ids=ids, rows=table[ids])
    print("gather_rows", table[ids].shape)


if __name__ == "__main__":
    main()
