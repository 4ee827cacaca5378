"""Topapel as a ModelSpec.

A decoder whose config.json lists its layers one by one. The embedded rows are scaled by a constant. Every layer is
the ``pre_norm`` arrangement, ``x += mixer(norm1(x))`` and, where the layer has a feed-forward,
``x += ff(norm2(x))``, with RMS norms whose weights are stored around zero (``1 + w`` multiplies). A layer's mixer is

* ``lightning``: linear attention with a fixed decay per head, SiLU on q, k and v, the heads' outputs normed
  together, gated by ``sigmoid(Wg h)`` and projected (``decay_attention``);
* ``attention``: grouped-query softmax attention with biased q, k and o projections, whose values are the projected
  keys; per-head RMS norms on q and k, a rotation of the first ``rot.dims`` dimensions with linearly scaled
  positions, causal chunks of ``mask.size`` positions, and a learned sink per head in the softmax's denominator
  (``paged_attention`` with ``values_are_keys``, ``chunk`` and ``sink``);
* ``mingru``: an element-wise gated recurrence (``min_gru``).

The feed-forward is ``down(polynorm(up(h)))`` (``mlp`` with the ``poly_norm`` activation). The head norms the last
rows, multiplies by the embedding table itself, scales the logits and caps them with a tanh.

Tensor names: ``embed``; ``l<i>.norm1``, ``l<i>.norm2``; lightning ``l<i>.mix.{q,k,v,g,o,norm}``; attention
``l<i>.mix.{q,k,o}`` with ``.b`` biases, ``l<i>.mix.{q.norm,k.norm,sink}``; mingru ``l<i>.mix.{z,x,g,o}`` with
``z.b``, ``x.b``; ``l<i>.mlp.{up,down,act}``; ``final.norm``.
"""

from __future__ import annotations

from ..config.registry import register_architecture
from ..config.topapel import TopapelConfig
from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec

NAME = "Topapel"


def build_topapel_spec(config: TopapelConfig) -> ModelSpec:
    width, eps = config.width, config.norm_eps

    def norm(name: str) -> PartSpec:
        return PartSpec("rms_norm", {"dim": width, "eps": eps, "weight": name, "one_plus": True})

    layers = []
    for i, layer in enumerate(config.layers):
        p = f"l{i}.mix."
        m = layer.mixer
        if layer.kind == "lightning":
            mixer = PartSpec("decay_attention", {
                "hidden": width, "heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim, "decay": list(m.decay),
                "activation": "silu", "eps": eps,
                "names": {k: p + k for k in ("q", "k", "v", "g", "o", "norm")},
            })
        elif layer.kind == "attention":
            position = PartSpec("none")
            if m.rotation is not None:
                position = PartSpec("rope_neox", {"head_dim": m.dim, "theta": m.rotation.base,
                                                  "rotary_dim": m.rotation.dims, "scaling_factor": m.rotation.factor})
            mixer = PartSpec("paged_attention", {
                "hidden": width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                "scale": m.scale, "window": None, "chunk": m.chunk, "sink": p + "sink", "values_are_keys": True,
                "qk_norm": {"eps": eps, "q_weight": p + "q.norm", "k_weight": p + "k.norm"},
                "position": position,
                "names": {"q": p + "q", "k": p + "k", "o": p + "o"},
                "bias": {"q": p + "q.b", "k": p + "k.b", "o": p + "o.b"},
            })
        else:
            mixer = PartSpec("min_gru", {
                "hidden": width, "width": m.width,
                "names": {k: p + k for k in ("z", "x", "g", "o")},
                "bias": {"z": p + "z.b", "x": p + "x.b"},
            })
        norms = {"pre_mixer": norm(f"l{i}.norm1")}
        feed_forward = None
        if layer.mlp is not None:
            f = f"l{i}.mlp."
            feed_forward = PartSpec("mlp", {"hidden": width, "intermediate": layer.mlp.ff, "activation": "poly_norm",
                                            "activation_weight": f + "act", "activation_eps": eps,
                                            "names": {"up": f + "up", "down": f + "down"}})
            norms["pre_feed_forward"] = norm(f"l{i}.norm2")
        layers.append(LayerSpec(block=PartSpec("pre_norm"), mixer=mixer, feed_forward=feed_forward, norms=norms))
    return ModelSpec(
        architecture=NAME,
        vocab_size=config.vocab,
        hidden_size=width,
        max_positions=config.max_positions,
        embedding=PartSpec("token_embedding", {"vocab": config.vocab, "hidden": width, "weight": "embed",
                                               "scale": config.embedding_scale}),
        layers=tuple(layers),
        order=tuple(LayerCall(i) for i in range(len(layers))),
        head=PartSpec("lm_head", {"vocab": config.vocab, "hidden": width, "norm": norm("final.norm"),
                                  "weight": None, "tied_to": "embed", "logit_scale": config.logit_scale,
                                  "softcap": config.logit_softcap}),
    )


register_architecture(NAME, TopapelConfig.from_json, build_topapel_spec)
