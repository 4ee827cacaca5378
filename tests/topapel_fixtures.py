"""Small Topapel configurations for tests, and model folders made from them.

A mixes all three mixers with and without feed-forwards: grouped and ungrouped attention heads, a rotation of part
of a head with scaled positions and of a whole head without, chunks of 7 positions (no multiple of the page size of
4) and no chunks at all, linear-attention heads whose key and value sizes differ, a decay of exactly one. B starts
with a recurrence, has six query heads on one key/value head, a chunk of one position (a token sees itself and the
sink), no embedding scale, no logit cap. C has sizes in no step of 8, a chunk longer than any request, a recurrence
seven wide. D has no attention at all (no pages, only state slots) and a head whose decay is zero. E has twenty
query heads on one key/value head: more than the matrix-core decode kernel takes.
"""

import json
import os

import torch

A = {
    "architecture": "Topapel", "vocab": 101, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 4.0},
    "logit_scale": 0.5, "logit_softcap": 12.0,
    "layers": [
        {"type": "attention",
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 16, "scale": 0.3, "mask": {"size": 7},
                   "rot": {"dims": 8, "base": 100.0, "scaling": {"factor": 1.5}}},
         "mlp": {"kind": "dense", "ff": 40}},
        {"type": "lightning", "mixer": {"heads": 2, "dim": 8, "vdim": 24, "decay": [0.5, 0.97]}, "mlp": None},
        {"type": "mingru", "mixer": {"width": 40}, "mlp": {"kind": "dense", "ff": 24}},
        {"type": "attention",
         "mixer": {"heads": 3, "kv_heads": 3, "dim": 32, "vdim": 32, "scale": 0.2,
                   "rot": {"dims": 32, "base": 10000.0}},
         "mlp": None},
        {"type": "lightning", "mixer": {"heads": 3, "dim": 20, "vdim": 12, "decay": [1.0, 0.9, 0.3]},
         "mlp": {"kind": "dense", "ff": 16}},
    ],
}
B = {
    "architecture": "Topapel", "vocab": 211, "width": 96, "norm": {"eps": 1e-6}, "logit_scale": 2.0,
    "layers": [
        {"type": "mingru", "mixer": {"width": 104}, "mlp": None},
        {"type": "attention",
         "mixer": {"heads": 6, "kv_heads": 1, "dim": 48, "vdim": 48, "scale": 0.15, "mask": {"size": 33},
                   "rot": {"dims": 24, "base": 5000.0, "scaling": {"factor": 4.0}}},
         "mlp": {"kind": "dense", "ff": 72}},
        {"type": "lightning", "mixer": {"heads": 1, "dim": 64, "vdim": 32, "decay": [0.95]}, "mlp": None},
        {"type": "attention",
         "mixer": {"heads": 2, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 0.125, "mask": {"size": 16},
                   "rot": {"dims": 64, "base": 777.0, "scaling": {"factor": 1.0}}},
         "mlp": {"kind": "dense", "ff": 48}},
        {"type": "mingru", "mixer": {"width": 32}, "mlp": {"kind": "dense", "ff": 64}},
        {"type": "attention",
         "mixer": {"heads": 8, "kv_heads": 2, "dim": 16, "vdim": 16, "scale": 0.4, "mask": {"size": 1}},
         "mlp": None},
    ],
}
C = {
    "architecture": "Topapel", "vocab": 333, "width": 100, "norm": {"eps": 1e-4}, "embedding": {"scale": 0.5},
    "logit_scale": 1.0, "logit_softcap": 3.0,
    "layers": [
        {"type": "lightning", "mixer": {"heads": 5, "dim": 12, "vdim": 40, "decay": [0.2, 0.6, 0.8, 0.99, 0.999]},
         "mlp": {"kind": "dense", "ff": 50}},
        {"type": "attention",
         "mixer": {"heads": 8, "kv_heads": 1, "dim": 40, "vdim": 40, "scale": 0.11, "mask": {"size": 200},
                   "rot": {"dims": 10, "base": 30.0, "scaling": {"factor": 0.5}}},
         "mlp": None},
        {"type": "mingru", "mixer": {"width": 7}, "mlp": {"kind": "dense", "ff": 9}},
    ],
}
D = {
    "architecture": "Topapel", "vocab": 64, "width": 48, "norm": {"eps": 1e-5}, "embedding": {"scale": 7.0},
    "layers": [
        {"type": "mingru", "mixer": {"width": 48}, "mlp": {"kind": "dense", "ff": 96}},
        {"type": "lightning", "mixer": {"heads": 2, "dim": 16, "vdim": 80, "decay": [0.0, 0.9]}, "mlp": None},
    ],
}
E = {
    "architecture": "Topapel", "vocab": 90, "width": 80, "norm": {"eps": 1e-5}, "logit_softcap": 8.0,
    "layers": [
        {"type": "attention",
         "mixer": {"heads": 20, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 0.25, "mask": {"size": 24},
                   "rot": {"dims": 16, "base": 50.0}},
         "mlp": {"kind": "dense", "ff": 32}},
        {"type": "mingru", "mixer": {"width": 24}, "mlp": None},
    ],
}
CONFIGS = {"A": A, "B": B, "C": C, "D": D, "E": E}
BLOCK_SIZE = {"A": 4, "B": 16, "C": 8, "D": 16, "E": 16}


def make_tensors(config: dict, seed: int, dtype: str):
    """Random tensors of the design, drawn wider than the serving default so that every mechanism moves the logits:
    matrices three times as wide, biases and sinks of the order of one, norm weights around zero."""
    from tie_amd.models.builder import expected_tensors_for_config
    from tie_amd.weights.random_init import random_tensors

    store = torch.float32 if dtype == "float32" else torch.bfloat16
    specs = expected_tensors_for_config(config)
    tensors = dict(random_tensors(specs, seed, torch.float32, vector_dtype=torch.float32))
    for name, t in tensors.items():
        if name.endswith(".b"):
            t.mul_(25.0)
        elif t.dim() == 2 and name != "embed":
            t.mul_(3.0)
    return {n: t.to(store) for n, t in tensors.items()}


def write_model(folder, config: dict, seed: int, dtype: str) -> str:
    from tie_amd.weights.safetensors_io import write_safetensors

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), list(make_tensors(config, seed, dtype).items()))
    return str(folder)


def load_plain(folder):
    from safetensors import safe_open

    weights = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name).to(torch.float64)
    return weights
