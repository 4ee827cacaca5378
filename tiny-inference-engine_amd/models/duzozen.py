"""Duzozen as a ModelSpec.

A decoder whose config.json lists its layers one by one. Every layer norms both the input and the output of each
sub-layer (``x += post(sublayer(pre(x)))``, four RMS norms a layer, the ``sandwich_norm`` arrangement). The mixer
is grouped-query attention without a position encoding: a score scale given as a number, a tanh cap on the
scores, a sliding window, value heads whose size may differ from the key heads', and, where a layer says so,
values blended with those the first such layer computed for the same token (``.vmix`` holds the weight). The
feed-forward is ``down(gelu(up(h)))`` or a routed mixture of SiLU-gated experts (``routed_experts``), or absent.

Tensor names: ``embed``; ``l<i>.norm1``, ``norm1b`` (before / after the mixer), ``norm2``, ``norm2b`` (before /
after the feed-forward); ``l<i>.mix.{q,k,v,o,vmix}``; ``l<i>.mlp.{up,down}`` or ``l<i>.mlp.{router,correction}``
and ``l<i>.mlp.e<j>.{gate,up,down}``; ``final.norm``; ``head``.
"""

from __future__ import annotations

from ..config.duzozen import DenseMlpConfig, DuzozenConfig, RoutedMlpConfig
from ..config.registry import register_architecture
from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec

NAME = "Duzozen"


def build_duzozen_spec(config: DuzozenConfig) -> ModelSpec:
    width, eps = config.width, config.norm_eps

    def norm(name: str) -> PartSpec:
        return PartSpec("rms_norm", {"dim": width, "eps": eps, "weight": name})

    layers = []
    first_mixing = next((i for i, l in enumerate(config.layers) if l.mixer.v_mix), None)
    for i, layer in enumerate(config.layers):
        p = f"l{i}."
        m = layer.mixer
        value_mix = None
        if m.v_mix:
            # every blending layer owns a weight tensor; the first one's is stored and never used
            value_mix = {"role": "keep" if i == first_mixing else "blend", "weight": p + "mix.vmix", "share": "v_first"}
        mixer = PartSpec("paged_attention", {
            "hidden": width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
            "value_dim": m.vdim, "scale": m.scale, "softcap": m.softcap, "window": m.window,
            "qk_norm": None, "position": PartSpec("none"), "value_mix": value_mix,
            "names": {"q": p + "mix.q", "k": p + "mix.k", "v": p + "mix.v", "o": p + "mix.o"},
        })
        norms = {"pre_mixer": norm(p + "norm1"), "post_mixer": norm(p + "norm1b")}
        feed_forward = None
        if isinstance(layer.mlp, DenseMlpConfig):
            feed_forward = PartSpec("mlp", {"hidden": width, "intermediate": layer.mlp.ff, "activation": "gelu",
                                            "names": {"up": p + "mlp.up", "down": p + "mlp.down"}})
        elif isinstance(layer.mlp, RoutedMlpConfig):
            r = layer.mlp
            feed_forward = PartSpec("routed_experts", {
                "hidden": width, "expert_intermediate": r.expert_ff, "experts": r.experts,
                "identity_experts": r.identity, "top": r.top, "groups": r.group_count, "keep_groups": r.group_keep,
                "scoring": "softmax", "renormalize": False,
                "names": {"router": p + "mlp.router", "correction": p + "mlp.correction",
                          "gate": [f"{p}mlp.e{e}.gate" for e in range(r.experts)],
                          "up": [f"{p}mlp.e{e}.up" for e in range(r.experts)],
                          "down": [f"{p}mlp.e{e}.down" for e in range(r.experts)]},
            })
        if feed_forward is not None:
            norms["pre_feed_forward"] = norm(p + "norm2")
            norms["post_feed_forward"] = norm(p + "norm2b")
        layers.append(LayerSpec(block=PartSpec("sandwich_norm"), mixer=mixer, feed_forward=feed_forward, norms=norms))
    return ModelSpec(
        architecture=NAME,
        vocab_size=config.vocab,
        hidden_size=width,
        max_positions=config.max_positions,
        embedding=PartSpec("token_embedding", {"vocab": config.vocab, "hidden": width, "weight": "embed"}),
        layers=tuple(layers),
        order=tuple(LayerCall(i) for i in range(len(layers))),
        head=PartSpec("lm_head", {"vocab": config.vocab, "hidden": width, "norm": norm("final.norm"),
                                  "weight": "head", "tied_to": None}),
    )


register_architecture(NAME, DuzozenConfig.from_json, build_duzozen_spec)
