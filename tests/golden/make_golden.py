"""Writes the small golden vectors under tests/golden/ from the torch float64 library
restatements in tests/torch_ref.py (the reference ships no usable vectors for this path:
its parity scripts need downloaded weights).  Run from the repo root:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import torch_ref  # noqa: E402


def bert_small():
    B, S, H, heads, F = 2, 8, 32, 4, 64
    rng = np.random.default_rng(20240)
    w = {"qkv_weight": rng.normal(0, 0.2, (3, H, H)), "qkv_bias": rng.normal(0, 0.3, 3 * H),
         "attn_fc_weight": rng.normal(0, 0.2, (H, H)), "attn_fc_bias": rng.normal(0, 0.3, H),
         "ln1_gamma": 1 + rng.normal(0, 0.2, H), "ln1_beta": rng.normal(0, 0.2, H),
         "fc1_weight": rng.normal(0, 0.2, (H, F)), "fc1_bias": rng.normal(0, 0.3, F),
         "fc2_weight": rng.normal(0, 0.2, (F, H)), "fc2_bias": rng.normal(0, 0.3, H),
         "ln2_gamma": 1 + rng.normal(0, 0.2, H), "ln2_beta": rng.normal(0, 0.2, H)}
    w = {k: v.astype(np.float32) for k, v in w.items()}
    x = rng.normal(size=(B * S, H)).astype(np.float32)
    mask = np.where(rng.random((B, S, S)) < 0.25, -1e4, 0.0).astype(np.float32)
    scale, eps = 0.35, 1e-12
    outs = torch_ref.bert_layer(x, w, B, S, heads, "gelu_tanh", scale, eps, mask=mask)
    d = {"B": B, "S": S, "H": H, "heads": heads, "F": F, "scale": scale, "eps": eps, "x": x, "mask": mask}
    d.update({"w_" + k: v for k, v in w.items()})
    d.update({"out_" + n: o.astype(np.float32) for n, o in zip(["qkv", "probs", "ctx", "ln1", "fc1", "out"], outs)})
    np.savez_compressed(os.path.join(HERE, "bert_layer_small.npz"), **d)


if __name__ == "__main__":
    bert_small()
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
