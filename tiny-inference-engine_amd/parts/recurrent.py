"""Mixers whose memory is a state of fixed size per request instead of a cache of keys.

``decay_attention`` is a linear attention with a fixed decay per head and a gated, normed output:

    q, k = act(Wq h), act(Wk h)   (heads x key_dim)        v = act(Wv h)   (heads x value_dim)
    per head   S_t = decay[head] * S_(t-1) + k_t v_t^T ,   o_t = S_t^T q_t          (no other scale)
    y = Wo ( RMSNorm(o_t, all heads side by side; weight ``norm``) * sigmoid(Wg h) )

``min_gru`` is a gated recurrence whose gates read the current token only:

    z = sigmoid(Wz h + bz),   u = Wx h + bx,   candidate = u + 1/2 for u >= 0, sigmoid(u) below
    S_t = (1 - z) S_(t-1) + z * candidate   element by element,      y = Wo (S_t * silu(Wg h))

Both states start at zero (a slot is cleared when a request takes it), live in float32 whatever the compute mode,
and are carried from step to step in the request's state slot. The projections of a mixer run as one product; the
recurrences, their gates, activations and the norm are float32 on the product's float32 sums. Everything that
differs between steps is read on the device (``query_start``, ``state_slots``), so decode steps are recorded. A
step with a long prompt portion runs the recurrences chunk beside chunk (``kernels.scan_chunks``: three launches
instead of one token after the other in a handful of waves); such steps are never recorded.

Parameters. ``decay_attention``: ``hidden``, ``heads``, ``key_dim``, ``value_dim``, ``decay`` (one number a head),
``activation`` ("silu" or "none"), ``eps``, ``names`` (``q``, ``k``, ``v``, ``g``, ``o``, ``norm``).
``min_gru``: ``hidden``, ``width``, ``names`` (``z``, ``x``, ``g``, ``o``) and ``bias`` (``z``, ``x``).
"""

from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..cache.spec import FixedState
from ..errors import InvalidArgument
from .base import Mixer, StepContext, TensorSpec, register_part
from .linear import Linear


def _finish(ctx: StepContext, out: Linear, rows: torch.Tensor, residual: Optional[torch.Tensor], name: str):
    """The output projection: added to ``residual``, or (None) returned as float32 rows."""
    if residual is not None:
        out(rows, residual, accumulate=True, ctx=ctx)
        return None
    ctx.settle()
    result = ctx.scratch(name, (rows.shape[0], out.total_out), torch.float32)
    out(rows, result, accumulate=False, ctx=ctx)
    return result


@register_part("mixer", "decay_attention")
class DecayAttention(Mixer):
    capturable = True      # reads the step on the device only: may be recorded into a HIP graph
    takes_row_scale = True   # h goes into the one projection only, through Linear with the step context
    returns_result = True

    def __init__(self, params):
        super().__init__(params)
        self.hidden = int(params["hidden"])
        self.heads = int(params["heads"])
        self.key_dim = int(params["key_dim"])
        self.value_dim = int(params.get("value_dim") or self.key_dim)
        self.decay_values = [float(d) for d in params["decay"]]
        self.activation = params.get("activation", "silu")
        self.eps = float(params["eps"])
        if len(self.decay_values) != self.heads:
            raise InvalidArgument(f"{self.heads} heads need {self.heads} decays, got {len(self.decay_values)}")
        if self.key_dim > kernels.DECAY_ATTENTION_MAX_DIM:
            raise InvalidArgument(f"a key size of {self.key_dim} exceeds {kernels.DECAY_ATTENTION_MAX_DIM}")
        names = params["names"]
        self.qk_width, self.v_width = self.heads * self.key_dim, self.heads * self.value_dim
        self.inputs = Linear([names["q"], names["k"], names["v"], names["g"]],
                             [self.qk_width, self.qk_width, self.v_width, self.v_width], self.hidden)
        self.out = Linear([names["o"]], [self.hidden], self.v_width)
        self.norm_name = names["norm"]
        self.norm_weight: torch.Tensor = None
        self.decay: torch.Tensor = None

    def cache_need(self):
        return FixedState((self.heads, self.key_dim, self.value_dim))

    def tensors(self) -> List[TensorSpec]:
        return self.inputs.tensors() + self.out.tensors() + \
            [TensorSpec(self.norm_name, (self.v_width,), "vector", ("one_plus_uniform", 0.1))]

    def load(self, fetch, mode, device) -> None:
        self.inputs.load(fetch)
        self.out.load(fetch)
        self.norm_weight = fetch(self.norm_name, "vector")
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32).to(device)

    def forward(self, ctx: StepContext, h: torch.Tensor, cache, residual: Optional[torch.Tensor]):
        T = h.shape[0]
        proj = ctx.scratch("decay_attention.proj", (T, self.inputs.total_out), torch.float32)
        self.inputs(h, proj, ctx=ctx)
        o = ctx.scratch("decay_attention.o", (T, self.v_width), torch.float32)
        kernels.decay_attention_scan(proj, o, cache.state, ctx.batch.query_start, cache.state_slots, self.decay,
                                     ctx.batch.num_seqs, self.heads, self.key_dim, self.value_dim, self.activation,
                                     chunks=kernels.scan_chunks(ctx.batch, ctx.device), scratch=ctx.scratch)
        gated = ctx.scratch("decay_attention.gated", (T, self.v_width))
        kernels.gated_rms_norm(o, self.norm_weight, self.eps, proj[:, 2 * self.qk_width + self.v_width:], gated)
        return _finish(ctx, self.out, gated, residual, "decay_attention.result")


@register_part("mixer", "min_gru")
class MinGru(Mixer):
    capturable = True
    takes_row_scale = True
    returns_result = True

    def __init__(self, params):
        super().__init__(params)
        self.hidden = int(params["hidden"])
        self.width = int(params["width"])
        names = params["names"]
        bias = params.get("bias") or {}
        # The projection itself carries no bias: the recurrence kernel adds the vectors as it reads the sums, so the
        # product keeps its ways of running at decode sizes (planes of partial sums are not used here: the kernel
        # reads plain rows) and no pass over the rows is spent on the addition.
        self.inputs = Linear([names["z"], names["x"], names["g"]], [self.width] * 3, self.hidden)
        self.bias_names = [bias.get("z"), bias.get("x"), bias.get("g")] if bias else None
        self.bias: torch.Tensor = None
        self.out = Linear([names["o"]], [self.hidden], self.width)

    def cache_need(self):
        return FixedState((self.width,))

    def tensors(self) -> List[TensorSpec]:
        specs = self.inputs.tensors() + self.out.tensors()
        for name in self.bias_names or ():
            if name is not None:
                specs.append(TensorSpec(name, (self.width,), "vector", ("normal", 0.02)))
        return specs

    def load(self, fetch, mode, device) -> None:
        self.inputs.load(fetch)
        self.out.load(fetch)
        if self.bias_names is not None:
            self.bias = torch.cat([fetch(name, "vector").to(torch.float32) if name is not None else
                                   torch.zeros(self.width, dtype=torch.float32, device=device)
                                   for name in self.bias_names]).contiguous()

    def forward(self, ctx: StepContext, h: torch.Tensor, cache, residual: Optional[torch.Tensor]):
        T = h.shape[0]
        proj = ctx.scratch("min_gru.proj", (T, 3 * self.width), torch.float32)
        self.inputs(h, proj, ctx=ctx)
        rows = ctx.scratch("min_gru.rows", (T, self.width))
        kernels.min_gru_scan(proj, rows, cache.state, ctx.batch.query_start, cache.state_slots, ctx.batch.num_seqs,
                             self.width, chunks=kernels.scan_chunks(ctx.batch, ctx.device), scratch=ctx.scratch,
                             bias=self.bias)
        return _finish(ctx, self.out, rows, residual, "min_gru.result")
