"""A plain, slow Duzozen for tests: whole sequences, no cache, one function per mechanism.

Written from the design's equations; it shares no code with the engine. Everything runs on the CPU in
float64. A model is a config dictionary (the keys of the design's config.json) and a dictionary of
tensors by their stored names.

The design in short. Every layer is ``x += post_a(mixer(pre_a(x)))`` and then, if it has a feed-forward,
``x += post_b(ff(pre_b(x)))`` with four RMS norms. The mixer is grouped-query attention without any position
encoding, with a fixed score scale, a tanh cap on the scores, a sliding window, and (optionally) values that are
blended with the values the first such layer computed for the same token. The feed-forward is either
``down(gelu(up(h)))`` or a routed mixture: softmax router over real and identity experts, a bias that
only steers the choice, a choice limited to the best groups of neighbouring experts, weights that are the
plain softmax scores of the chosen.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

F64 = torch.float64


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * w over the last dimension."""
    x = x.to(F64)
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w.to(F64)


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """W x for every row of x; W is stored [out, in]."""
    return x.to(F64) @ w.to(F64).T


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    """The exact gelu: z * Phi(z) with the normal distribution function written through erf."""
    z = z.to(F64)
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z: torch.Tensor) -> torch.Tensor:
    z = z.to(F64)
    return z / (1.0 + torch.exp(-z))


def capped_scores(q: torch.Tensor, k: torch.Tensor, scale: float, softcap: Optional[float]) -> torch.Tensor:
    """scores[i, j] = cap * tanh(scale * (q_i . k_j) / cap); without a cap the scaled product itself."""
    s = scale * (q.to(F64) @ k.to(F64).T)
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    return s


def window_mask(T: int, window: Optional[int]) -> torch.Tensor:
    """allowed[i, j]: j <= i and, with a window of w, i - j < w."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    allowed = j <= i
    if window is not None:
        allowed = allowed & (i - j < window)
    return allowed


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, softcap: Optional[float],
              window: Optional[int]) -> torch.Tensor:
    """q [T, H, D], k [T, G, D], v [T, G, Dv] -> [T, H, Dv]; query head h reads key/value head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    allowed = window_mask(T, window)
    for h in range(H):
        g = h // (H // G)
        s = capped_scores(q[:, h], k[:, g], scale, softcap).masked_fill(~allowed, -math.inf)
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g].to(F64)
    return out


def mix_values(v: torch.Tensor, v_first: torch.Tensor, lam) -> torch.Tensor:
    """(1 - lambda) v + lambda v_first, token by token."""
    lam = float(lam)
    return (1.0 - lam) * v.to(F64) + lam * v_first.to(F64)


def attention_mixer(h: torch.Tensor, weights: Dict[str, torch.Tensor], prefix: str, mixer: dict,
                    v_first: Optional[torch.Tensor]):
    """The whole mixer on normed rows h [T, width]; returns (output [T, width], the values it used [T, G, Dv])."""
    H, G, D, Dv = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    T = h.shape[0]
    q = linear(h, weights[prefix + "q"]).view(T, H, D)
    k = linear(h, weights[prefix + "k"]).view(T, G, D)
    v = linear(h, weights[prefix + "v"]).view(T, G, Dv)
    if mixer.get("v_mix") and v_first is not None:
        v = mix_values(v, v_first, weights[prefix + "vmix"])
    mask = mixer.get("mask") or {}
    o = attention(q, k, v, float(mixer["scale"]), mixer.get("softcap"), mask.get("size"))
    return linear(o.reshape(T, H * Dv), weights[prefix + "o"]), v


def dense_feed_forward(h: torch.Tensor, weights, prefix: str) -> torch.Tensor:
    return linear(gelu_erf(linear(h, weights[prefix + "up"])), weights[prefix + "down"])


def route(h: torch.Tensor, router_w: torch.Tensor, correction: torch.Tensor, router: dict):
    """For every row: the chosen experts (indices into real + identity experts) and their weights.

    s = softmax(W h) over all outputs. The choice looks at s + correction: a group of neighbours scores the
    largest of its members, only members of the ``keep`` best groups stay eligible, and the ``top`` largest of
    those are chosen. The weights are s at the chosen, as they are.
    """
    s = torch.softmax(linear(h, router_w), dim=-1)
    choice = s + correction.to(F64)
    T, E = s.shape
    groups = router.get("groups") or {"count": 1, "keep": 1}
    count, keep = int(groups["count"]), int(groups["keep"])
    size = E // count
    group_score = choice.view(T, count, size).max(dim=-1).values
    best = torch.topk(group_score, keep, dim=-1).indices
    eligible = torch.zeros(T, count, dtype=torch.bool)
    eligible.scatter_(1, best, True)
    eligible = eligible[:, :, None].expand(T, count, size).reshape(T, E)
    masked = choice.masked_fill(~eligible, -math.inf)
    chosen = torch.topk(masked, int(router["top"]), dim=-1).indices
    return chosen, torch.gather(s, 1, chosen)


def expert(h: torch.Tensor, weights, prefix: str) -> torch.Tensor:
    return linear(silu(linear(h, weights[prefix + "gate"])) * linear(h, weights[prefix + "up"]),
                  weights[prefix + "down"])


def routed_feed_forward(h: torch.Tensor, weights, prefix: str, mlp: dict) -> torch.Tensor:
    router = mlp["router"]
    real = int(router["experts"])
    chosen, w = route(h, weights[prefix + "router"], weights[prefix + "correction"], router)
    out = torch.zeros(h.shape[0], h.shape[1], dtype=F64)
    for t in range(h.shape[0]):
        for e, we in zip(chosen[t].tolist(), w[t].tolist()):
            row = h[t:t + 1].to(F64)
            out[t] += we * (expert(row, weights, f"{prefix}e{e}.")[0] if e < real else row[0])
    return out


def forward(config: dict, weights: Dict[str, torch.Tensor], tokens: Sequence[int],
            stream_after: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence; ``stream_after`` collects the residual stream after every layer."""
    eps = float(config["norm"]["eps"])
    x = weights["embed"][torch.as_tensor(list(tokens), dtype=torch.long)].to(F64)
    v_first = None
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        if layer["type"] != "attention":
            raise ValueError(f"layer {i}: unknown mixer '{layer['type']}'")
        mixer = layer["mixer"]
        y, v = attention_mixer(rms_norm(x, weights[p + "norm1"], eps), weights, p + "mix.", mixer, v_first)
        if mixer.get("v_mix") and v_first is None:
            v_first = v
        x = x + rms_norm(y, weights[p + "norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rms_norm(x, weights[p + "norm2"], eps)
            if mlp["kind"] == "dense":
                y = dense_feed_forward(h, weights, p + "mlp.")
            elif mlp["kind"] == "moe":
                y = routed_feed_forward(h, weights, p + "mlp.", mlp)
            else:
                raise ValueError(f"layer {i}: unknown feed-forward '{mlp['kind']}'")
            x = x + rms_norm(y, weights[p + "norm2b"], eps)
        if stream_after is not None:
            stream_after.append(x.clone())
    return linear(rms_norm(x, weights["final.norm"], eps), weights["head"])
