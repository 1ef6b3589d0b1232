"""Writes tests/golden/hotpath_golden.npz: seeded inputs and expected outputs.

The reference holds no golden vectors for these ops (its tests recompute every
expectation with numpy / PyTorch at run time), so the expectations here are
produced the way the reference's tests produce theirs -- with PyTorch's CPU
operators (``F.conv2d``, ``F.softmax``, ``F.layer_norm``, ``F.gelu``, ``@``,
``transformers`` BertLayer) -- evaluated in float64 and rounded once to float32.
Neither the oracle nor the HIP kernels take part in generating them.

Run from the repository root:  python tests/golden/make_golden.py
Also copies nothing from the reference: ``slice.onnx`` next to this file is the
168-byte data fixture of the reference's own tests (tests/onnx_files/slice.onnx).
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))


def f64(a):
    return torch.from_numpy(np.asarray(a)).double()


def main():
    out = {}
    # --- config 1: ONNXConv X[5,3,10,10] W[16,3,3,3] U[0,1), strides 2 -----------
    rng = np.random.default_rng(1)
    X = rng.random((5, 3, 10, 10), dtype=np.float32)
    W = rng.random((16, 3, 3, 3), dtype=np.float32)
    out["conv1_X"], out["conv1_W"] = X, W
    out["conv1_Y"] = F.conv2d(f64(X), f64(W), stride=2).numpy().astype(np.float32)
    # padded / biased / dilated conv + relu, small
    rng = np.random.default_rng(41)
    X = rng.normal(size=(2, 5, 9, 11)).astype(np.float32)
    W = rng.normal(size=(7, 5, 3, 2)).astype(np.float32)
    B = rng.normal(size=(7, )).astype(np.float32)
    out["conv2_X"], out["conv2_W"], out["conv2_B"] = X, W, B
    xp = F.pad(f64(X), (2, 1, 1, 0))  # pads = [top 1, left 2, bottom 0, right 1]
    out["conv2_Y"] = F.relu(F.conv2d(xp, f64(W), f64(B), stride=(2, 1), dilation=(1, 2))).numpy().astype(np.float32)
    # --- config 2: softmax / layernorm (reduced row counts, full row lengths) -----
    rng = np.random.default_rng(2)
    X = rng.normal(size=(2, 3, 8, 128)).astype(np.float32)
    out["softmax_X"] = X
    out["softmax_Y"] = F.softmax(f64(X), dim=-1).numpy().astype(np.float32)
    X = rng.normal(size=(2, 8, 768)).astype(np.float32)
    g = rng.normal(1.0, 0.02, size=768).astype(np.float32)
    b = rng.normal(0.0, 0.02, size=768).astype(np.float32)
    out["ln_X"], out["ln_gamma"], out["ln_beta"] = X, g, b
    out["ln_Y"] = F.layer_norm(f64(X), (768, ), f64(g), f64(b), eps=1e-12).numpy().astype(np.float32)
    X = rng.normal(scale=3.0, size=(4096, )).astype(np.float32)
    out["gelu_X"] = X
    out["gelu_Y"] = F.gelu(f64(X)).numpy().astype(np.float32)
    # --- matmul / gemm ---------------------------------------------------------------
    rng = np.random.default_rng(7)
    A = rng.normal(size=(2, 3, 16, 24)).astype(np.float32)
    Bm = rng.normal(size=(24, 20)).astype(np.float32)
    out["matmul_A"], out["matmul_B"] = A, Bm
    out["matmul_Y"] = (f64(A) @ f64(Bm)).numpy().astype(np.float32)
    A = rng.normal(size=(10, 12)).astype(np.float32)
    Bt = rng.normal(size=(9, 12)).astype(np.float32)
    C = rng.normal(size=(9, )).astype(np.float32)
    out["gemm_A"], out["gemm_B"], out["gemm_C"] = A, Bt, C
    out["gemm_Y"] = (f64(A) @ f64(Bt).T + f64(C)).numpy().astype(np.float32)
    # --- config 5 (reduced): MatMulInteger, zero points 3 / -2 ----------------------------
    rng = np.random.default_rng(5)
    A = rng.integers(-128, 128, size=(64, 48), dtype=np.int8)
    Bi = rng.integers(-128, 128, size=(48, 40), dtype=np.int8)
    out["mmi_A"], out["mmi_B"] = A, Bi
    out["mmi_Y"] = ((torch.from_numpy(A).long() - 3) @ (torch.from_numpy(Bi).long() + 2)).numpy().astype(np.int32)
    # --- config 3 (reduced): BERT encoder layer through transformers.BertLayer --------------
    from transformers import BertConfig
    from transformers.models.bert.modeling_bert import BertLayer
    hidden, heads, ffn, bsz, seq = 32, 4, 64, 2, 16
    cfg = BertConfig(hidden_size=hidden, num_attention_heads=heads, intermediate_size=ffn,
                     hidden_act="gelu", layer_norm_eps=1e-12, attention_probs_dropout_prob=0.0,
                     hidden_dropout_prob=0.0)
    cfg._attn_implementation = "eager"
    layer = BertLayer(cfg).eval().double()
    rng = np.random.default_rng(3)
    w = {}
    for name, shape in (("wq", (hidden, hidden)), ("wk", (hidden, hidden)), ("wv", (hidden, hidden)),
                        ("wo", (hidden, hidden)), ("w1", (hidden, ffn)), ("w2", (ffn, hidden))):
        w[name] = rng.normal(0.0, 0.02, size=shape).astype(np.float32)
    for name, n in (("bq", hidden), ("bk", hidden), ("bv", hidden), ("bo", hidden), ("b1", ffn), ("b2", hidden)):
        w[name] = rng.normal(0.0, 0.02, size=n).astype(np.float32)  # non-zero so a dropped bias shows
    for i in (1, 2):
        w[f"ln{i}_g"] = rng.normal(1.0, 0.02, size=hidden).astype(np.float32)
        w[f"ln{i}_b"] = rng.normal(0.0, 0.02, size=hidden).astype(np.float32)
    x = rng.normal(size=(bsz, seq, hidden)).astype(np.float32)
    with torch.no_grad():
        att, so = layer.attention.self, layer.attention.output
        for lin, wn, bn in ((att.query, "wq", "bq"), (att.key, "wk", "bk"), (att.value, "wv", "bv"),
                            (so.dense, "wo", "bo"), (layer.intermediate.dense, "w1", "b1"),
                            (layer.output.dense, "w2", "b2")):
            lin.weight.copy_(f64(w[wn]).T)  # nn.Linear stores [out, in]
            lin.bias.copy_(f64(w[bn]))
        so.LayerNorm.weight.copy_(f64(w["ln1_g"])); so.LayerNorm.bias.copy_(f64(w["ln1_b"]))
        layer.output.LayerNorm.weight.copy_(f64(w["ln2_g"])); layer.output.LayerNorm.bias.copy_(f64(w["ln2_b"]))
        y = layer(f64(x))
        y = y[0] if isinstance(y, (tuple, list)) else y
    for k, v in w.items():
        out["bert_" + k] = v
    out["bert_x"] = x
    out["bert_y"] = y.numpy().astype(np.float32)
    out["bert_meta"] = np.array([hidden, heads, ffn, bsz, seq], dtype=np.int64)

    path = os.path.join(HERE, "hotpath_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
