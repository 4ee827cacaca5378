"""Small Duzozen configurations for tests, and model folders made from them.

P mixes everything the design allows in four layers: grouped and ungrouped heads, key and value heads of unequal
size, a head size that is no multiple of 16, layers with and without a cap, a window, blended values or a
feed-forward, both kinds of feed-forward, routers with and without identity experts and groups. Q is seven layers of
which six are alike (routed), with other sizes throughout.
"""

import json
import os

import torch

P = {
    "architecture": "Duzozen", "vocab": 97, "width": 64, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "attention",
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 32, "scale": 0.3, "softcap": 5.0,
                   "mask": {"size": 7}, "v_mix": True},
         "mlp": {"kind": "moe", "expert": {"ff": 24},
                 "router": {"experts": 6, "identity": 2, "top": 3, "groups": {"count": 4, "keep": 2}}}},
        {"type": "attention",
         "mixer": {"heads": 4, "kv_heads": 4, "dim": 32, "vdim": 32, "scale": 0.2, "v_mix": False},
         "mlp": None},
        {"type": "attention",
         "mixer": {"heads": 2, "kv_heads": 2, "dim": 24, "vdim": 32, "scale": 0.25, "softcap": 30.0,
                   "mask": {"size": 5}, "v_mix": True},
         "mlp": {"kind": "dense", "ff": 40}},
        {"type": "attention",
         "mixer": {"heads": 6, "kv_heads": 2, "dim": 16, "vdim": 32, "scale": 0.35, "softcap": 2.0,
                   "mask": {"size": 16}, "v_mix": True},
         "mlp": {"kind": "moe", "expert": {"ff": 16},
                 "router": {"experts": 5, "identity": 0, "top": 2, "groups": {"count": 1, "keep": 1}}}},
    ],
}

_Q_LAYER = {"type": "attention",
            "mixer": {"heads": 3, "kv_heads": 3, "dim": 32, "vdim": 32, "scale": 0.17, "softcap": 12.0,
                      "mask": {"size": 9}, "v_mix": True},
            "mlp": {"kind": "moe", "expert": {"ff": 48},
                    "router": {"experts": 5, "identity": 3, "top": 2, "groups": {"count": 2, "keep": 1}}}}
Q = {
    "architecture": "Duzozen", "vocab": 211, "width": 96, "norm": {"eps": 1e-6},
    "layers": [dict(_Q_LAYER, mlp={"kind": "dense", "ff": 72})] + [_Q_LAYER] * 6,
}
# R: sizes at the edges. A stream of 100 (no multiple of 8), a vocabulary of 333; a window of one (a token sees only
# itself) and one longer than any test's request; 8 and 32 query heads on one key/value head, a single head; value heads
# smaller than key heads; one layer alone keeping values (nothing ever blends them); 72 router outputs in groups of 9;
# a single expert; a router most of whose outputs are identity experts, in groups of one; expert widths in no step of 8.
R = {
    "architecture": "Duzozen", "vocab": 333, "width": 100, "norm": {"eps": 1e-4},
    "layers": [
        {"type": "attention",
         "mixer": {"heads": 8, "kv_heads": 1, "dim": 40, "vdim": 40, "scale": 0.11, "softcap": 50.0, "mask": {"size": 1}},
         "mlp": {"kind": "moe", "expert": {"ff": 20},
                 "router": {"experts": 70, "identity": 2, "top": 6, "groups": {"count": 8, "keep": 3}}}},
        {"type": "attention",
         "mixer": {"heads": 32, "kv_heads": 1, "dim": 16, "vdim": 8, "scale": 0.5, "mask": {"size": 200}, "v_mix": True},
         "mlp": {"kind": "dense", "ff": 50}},
        {"type": "attention",
         "mixer": {"heads": 1, "kv_heads": 1, "dim": 64, "vdim": 16, "scale": 0.2, "softcap": 1.0},
         "mlp": {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 1, "top": 1}}},
        {"type": "attention",
         "mixer": {"heads": 2, "kv_heads": 2, "dim": 8, "vdim": 8, "scale": 0.4, "softcap": 3.0, "mask": {"size": 3}},
         "mlp": {"kind": "moe", "expert": {"ff": 16},
                 "router": {"experts": 2, "identity": 6, "top": 5, "groups": {"count": 8, "keep": 8}}}},
    ],
}
CONFIGS = {"P": P, "Q": Q, "R": R}
BLOCK_SIZE = {"P": 4, "Q": 16, "R": 8}


def make_tensors(config: dict, seed: int, dtype: str, decisive_router: bool):
    """Random tensors of the design. Matrices are drawn wider than the serving default so that every mechanism
    moves the logits; router rows wider still, so that choices differ from token to token. ``decisive_router``:
    the corrections are set far apart instead, so that rounding (bfloat16 runs) cannot change who is chosen; the
    weights of the chosen stay what the tokens make them."""
    from tie_amd.models.builder import expected_tensors_for_config
    from tie_amd.weights.random_init import random_tensors

    store = torch.float32 if dtype == "float32" else torch.bfloat16
    specs = expected_tensors_for_config(config)
    tensors = dict(random_tensors(specs, seed, torch.float32, vector_dtype=torch.float32))
    g = torch.Generator().manual_seed(seed)
    for name, t in tensors.items():
        if name.endswith(".router"):
            t.mul_(0.0 if decisive_router else 12.0)
            if decisive_router:
                t.add_(torch.randn(t.shape, generator=g) * 0.1)
        elif name.endswith(".correction"):
            if decisive_router:
                order = torch.randperm(t.numel(), generator=g).to(torch.float32)
                t.copy_(order * 1.5 - 2.0)                    # further apart than two scores can be; some negative:
                                                              # an excluded expert counts as -inf, not as 0
            else:
                t.copy_(torch.randn(t.shape, generator=g) * 0.05)
        elif name.endswith(".vmix"):
            t.fill_(0.15 + 0.6 * float(torch.rand((), generator=g)))
        elif t.dim() == 2 and name not in ("embed",):
            t.mul_(3.0)
    return {n: (t.to(store) if t.dim() == 2 else t.to(store)) for n, t in tensors.items()}


def write_model(folder, config: dict, seed: int, dtype: str, decisive_router: bool = False) -> str:
    from tie_amd.weights.safetensors_io import write_safetensors

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config, f)
    tensors = make_tensors(config, seed, dtype, decisive_router)
    write_safetensors(os.path.join(folder, "model.safetensors"), list(tensors.items()))
    return str(folder)


def load_plain(folder):
    from safetensors import safe_open

    weights = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name).to(torch.float64)
    return weights
