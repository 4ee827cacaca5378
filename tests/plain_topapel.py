"""A plain, slow Topapel for tests: whole sequences, no cache, one function per mechanism.

Written from the design's equations; it shares no code with the engine. Everything runs on the CPU in float64.
A model is a config dictionary (the keys of the design's config.json) and a dictionary of tensors by their
stored names.

The design in short. ``x = embed[token] * s``. Every layer is ``x += mixer(n1(x))`` and then, if it has a
feed-forward, ``x += ff(n2(x))``; the norms multiply by ``1 + w``. Three mixers: a linear attention with a fixed
decay per head and a gated, normed output (``lightning``); grouped-query softmax attention whose values are the
projected keys, with per-head q/k norms, a partial rotation, causal chunks and a sink in the softmax's
denominator (``attention``); and an element-wise gated recurrence (``mingru``). The feed-forward is
``down(polynorm(up(h)))``. The head reuses the embedding table, scales and tanh-caps the logits.
"""

from __future__ import annotations

import math
from typing import Dict, List, Sequence

import torch

F64 = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    x = x.to(F64)
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    return rms(x, eps) * (1.0 + w.to(F64))


def norm_plain(x, w, eps):
    return rms(x, eps) * w.to(F64)


def linear(x, w, b=None):
    y = x.to(F64) @ w.to(F64).T
    return y if b is None else y + b.to(F64)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z.to(F64)))


def silu(z):
    z = z.to(F64)
    return z * sigmoid(z)


# ------------------------------------------------------------------ lightning
def decayed_linear_attention(q, k, v, decay: float) -> torch.Tensor:
    """One head. ``S_t = decay * S_(t-1) + k_t v_t^T`` from zero; ``o_t = S_t^T q_t``. q, k ``[T, d]``, v ``[T, e]``."""
    T = q.shape[0]
    S = torch.zeros(k.shape[1], v.shape[1], dtype=F64)
    out = torch.zeros(T, v.shape[1], dtype=F64)
    for t in range(T):
        S = decay * S + torch.outer(k[t], v[t])
        out[t] = S.T @ q[t]
    return out


def lightning_mixer(h, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    q = silu(linear(h, W[p + "q"])).view(T, H, d)
    k = silu(linear(h, W[p + "k"])).view(T, H, d)
    v = silu(linear(h, W[p + "v"])).view(T, H, e)
    heads = [decayed_linear_attention(q[:, i], k[:, i], v[:, i], float(m["decay"][i])) for i in range(H)]
    o = torch.cat(heads, dim=1)                                  # head by head
    o = norm_plain(o, W[p + "norm"], eps) * sigmoid(linear(h, W[p + "g"]))
    return linear(o, W[p + "o"])


# ------------------------------------------------------------------ attention
def rotate_partial(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float, factor: float) -> torch.Tensor:
    """x ``[T, heads, d]``: dimension i < dims/2 pairs with i + dims/2; angle p * base^(-2i/dims) / factor."""
    half = dims // 2
    i = torch.arange(half, dtype=F64)
    freq = base ** (-2.0 * i / dims) / factor
    a = positions.to(F64)[:, None] * freq[None, :]               # [T, half]
    cos, sin = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, w = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = u * cos - w * sin
    out[..., half:dims] = w * cos + u * sin
    return out


def chunk_mask(T: int, size) -> torch.Tensor:
    """allowed[i, j]: j <= i and both in the same chunk of ``size`` positions counted from 0."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    allowed = j <= i
    if size:
        allowed = allowed & (i // size == j // size)
    return allowed


def softmax_with_sink(scores: torch.Tensor, allowed: torch.Tensor, sink: float) -> torch.Tensor:
    """Rows of weights ``exp(s_j) / (exp(sink) + sum_allowed exp(s_j'))``: they sum to less than one."""
    top = torch.where(allowed, scores, torch.full_like(scores, -math.inf)).max(dim=-1, keepdim=True).values
    top = torch.clamp(top, min=sink)
    e = torch.where(allowed, torch.exp(scores - top), torch.zeros_like(scores))
    return e / (e.sum(dim=-1, keepdim=True) + torch.exp(torch.as_tensor(sink, dtype=F64) - top))


def attention_mixer(h, W, p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, d = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
    e = m.get("vdim", d)
    assert e == d, "the values are the projected keys"
    q = linear(h, W[p + "q"], W[p + "q.b"]).view(T, H, d)
    k = linear(h, W[p + "k"], W[p + "k.b"]).view(T, G, d)
    v = k.clone()                                                 # as projected: before norm and rotation
    q = norm_plain(q, W[p + "q.norm"], eps)
    k = norm_plain(k, W[p + "k.norm"], eps)
    rot = m.get("rot")
    if rot:
        factor = float((rot.get("scaling") or {}).get("factor", 1.0))
        pos = torch.arange(T)
        q = rotate_partial(q, pos, rot["dims"], float(rot["base"]), factor)
        k = rotate_partial(k, pos, rot["dims"], float(rot["base"]), factor)
    allowed = chunk_mask(T, (m.get("mask") or {}).get("size"))
    out = torch.zeros(T, H, e, dtype=F64)
    per = H // G
    for i in range(H):
        g = i // per
        s = float(m["scale"]) * (q[:, i] @ k[:, g].T)
        out[:, i] = softmax_with_sink(s, allowed, float(W[p + "sink"][i])) @ v[:, g]
    return linear(out.reshape(T, H * e), W[p + "o"], W[p + "o.b"])


# --------------------------------------------------------------------- mingru
def mingru_candidate(u: torch.Tensor) -> torch.Tensor:
    """u + 1/2 where u >= 0, sigmoid(u) below: continuous and positive."""
    return torch.where(u >= 0, u + 0.5, sigmoid(u))


def mingru_scan(z: torch.Tensor, c: torch.Tensor) -> torch.Tensor:
    """``S_t = (1 - z_t) S_(t-1) + z_t c_t`` from zero, element by element; returns every S_t."""
    S = torch.zeros(z.shape[1], dtype=F64)
    out = torch.zeros_like(z)
    for t in range(z.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * c[t]
        out[t] = S
    return out


def mingru_mixer(h, W, p: str, m: dict) -> torch.Tensor:
    z = sigmoid(linear(h, W[p + "z"], W[p + "z.b"]))
    c = mingru_candidate(linear(h, W[p + "x"], W[p + "x.b"]))
    S = mingru_scan(z, c)
    return linear(S * silu(linear(h, W[p + "g"])), W[p + "o"])


# --------------------------------------------------------------- feed-forward
def polynorm(z: torch.Tensor, coeff: torch.Tensor, eps: float) -> torch.Tensor:
    """``a N(z) + b N(z^2) + c N(z^3) + e`` with N = division by the row's root mean square."""
    a, b, c, e = [float(x) for x in coeff.to(F64)]
    z = z.to(F64)
    return a * rms(z, eps) + b * rms(z * z, eps) + c * rms(z * z * z, eps) + e


def dense_ff(h, W, p: str, eps: float) -> torch.Tensor:
    return linear(polynorm(linear(h, W[p + "up"]), W[p + "act"], eps), W[p + "down"])


# ---------------------------------------------------------------------- model
def forward(config: dict, W: Dict[str, torch.Tensor], tokens: Sequence[int], streams: List[torch.Tensor] = None):
    """Logits ``[T, vocab]`` of a whole sequence; ``streams`` (a list) receives the stream after every layer."""
    eps = float(config["norm"]["eps"])
    ids = torch.as_tensor(list(tokens), dtype=torch.long)
    x = W["embed"].to(F64)[ids] * float((config.get("embedding") or {}).get("scale", 1.0))
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h = norm_one_plus(x, W[p + "norm1"], eps)
        kind = layer["type"]
        if kind == "lightning":
            y = lightning_mixer(h, W, p + "mix.", layer["mixer"], eps)
        elif kind == "attention":
            y = attention_mixer(h, W, p + "mix.", layer["mixer"], eps)
        elif kind == "mingru":
            y = mingru_mixer(h, W, p + "mix.", layer["mixer"])
        else:
            raise ValueError(kind)
        x = x + y
        if layer.get("mlp") is not None:
            x = x + dense_ff(norm_one_plus(x, W[p + "norm2"], eps), W, p + "mlp.", eps)
        if streams is not None:
            streams.append(x.clone())
    x = norm_one_plus(x, W["final.norm"], eps)
    logits = linear(x, W["embed"]) * float(config.get("logit_scale", 1.0))
    cap = config.get("logit_softcap")
    if cap:
        logits = float(cap) * torch.tanh(logits / float(cap))
    return logits
