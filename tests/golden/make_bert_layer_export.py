"""Writes tests/golden/bert_layer_torch_export_opset12.{onnx,npz}: a `transformers` BertLayer exported by
`torch.onnx.export(opset_version=12)` (the TorchScript exporter, as the reference's DaceModule uses it,
daceml/pytorch/module.py:130-160), with one input and the output PyTorch computes for it on the CPU.

The file is what the ONNX reader, the importer and the fusion pass meet in practice: Constant nodes for
the Reshape shapes and scalars, Identity nodes for initializers the exporter found equal, bias as the
first Add operand, LayerNorm and Gelu in their decomposed form. Small enough to commit (hidden 128, two
heads of 64, FFN 256), yet with 128 keys and head size 64 so the fused attention kernel is on the path.

The exporter's last step attaches onnxscript functions through the `onnx` package, which this image does
not have and this model does not need: that step is skipped.

Run from the repository root:  python tests/golden/make_bert_layer_export.py
"""
import io
import os
import warnings

import numpy as np
import torch
from torch.onnx._internal.torchscript_exporter import onnx_proto_utils
from transformers import BertConfig
from transformers.models.bert.modeling_bert import BertLayer

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    warnings.filterwarnings("ignore")
    onnx_proto_utils._add_onnxscript_fn = lambda proto, custom_opsets: proto
    torch.manual_seed(20)
    cfg = BertConfig(hidden_size=128, num_attention_heads=2, intermediate_size=256)
    cfg._attn_implementation = "eager"
    layer = BertLayer(cfg).eval()
    with torch.no_grad():
        # the default init makes both LayerNorms identical; give every parameter its own values
        for p in layer.parameters():
            p.copy_(torch.randn_like(p) * (0.05 if p.dim() > 1 else 0.2))
        layer.attention.output.LayerNorm.weight.add_(1.0)
        layer.output.LayerNorm.weight.add_(1.0)
    x = torch.randn(2, 128, 128)
    with torch.no_grad():
        y = layer(x)
        y = y[0] if isinstance(y, (tuple, list)) else y
    buf = io.BytesIO()
    torch.onnx.export(layer, (x, ), buf, opset_version=12, dynamo=False, input_names=["hidden_states"],
                      output_names=["output"])
    with open(os.path.join(HERE, "bert_layer_torch_export_opset12.onnx"), "wb") as f:
        f.write(buf.getvalue())
    np.savez_compressed(os.path.join(HERE, "bert_layer_torch_export_opset12.npz"), hidden_states=x.numpy(),
                        output=y.numpy(), torch_version=np.array(torch.__version__))
    print("wrote", len(buf.getvalue()), "bytes of ONNX; output", tuple(y.shape))


if __name__ == "__main__":
    main()
