"""HuggingFace BertModel -> the .npz weight file that `BertModel.from_npz` and the C++
`BertModel(file, device, n_layers, n_heads)` read.

Same key scheme and orientation as the reference's converter
(tools/convert_huggingface_bert_pytorch_to_npz.py:44-71): query / key / value weights of a layer
are concatenated into `...attention.qkv.weight` of shape [hidden, 3*hidden] (and `qkv.bias`),
every other dense weight is stored transposed, [in, out]; everything else keeps its name.

    python -m turbotransformers_amd.convert_huggingface_bert_to_npz <local model directory> <output.npz>

The model is read from a local directory (config.json + weights); nothing is downloaded.
"""
import sys

import numpy as np


def bert_to_npz_arrays(model):
    """-> {name: float32 ndarray} for a transformers BertModel."""
    sd = {k: v.detach().float().cpu().numpy() for k, v in model.named_parameters()}
    out = {}
    for name, value in sd.items():
        if ".attention.self." in name:
            continue  # packed below
        if name.endswith("dense.weight"):
            value = np.ascontiguousarray(value.T)
        out[name] = value
    for i in range(model.config.num_hidden_layers):
        p = "encoder.layer.%d.attention." % i
        parts = ("query", "key", "value")
        out[p + "qkv.weight"] = np.ascontiguousarray(np.concatenate([sd[p + "self.%s.weight" % x] for x in parts], 0).T)
        out[p + "qkv.bias"] = np.concatenate([sd[p + "self.%s.bias" % x] for x in parts])
    return out


def save_bert_npz(model, file_name, compressed=True):
    """Write `model` (a transformers BertModel) to `file_name`; compressed like the reference's converter by default."""
    (np.savez_compressed if compressed else np.savez)(file_name, **bert_to_npz_arrays(model))


def main(argv):
    if len(argv) != 3:
        print(__doc__)
        return 2
    from transformers import BertModel
    model = BertModel.from_pretrained(argv[1], local_files_only=True)
    save_bert_npz(model, argv[2])
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
