"""The plain Duzozen pinned by hand-made cases, and the configuration reader, registry and spec of the design.

The plain implementation is the oracle of the GPU tests, so its mechanisms are held against numbers worked out
here by other means: a window by counting, a capped score by its limits, a routing choice by hand.
"""

import copy
import math

import pytest
import torch

import plain_duzozen as plain
from duzozen_fixtures import CONFIGS

F64 = torch.float64


def test_rms_norm_has_eps_inside_the_root_and_multiplies_the_weight_last():
    x = torch.tensor([[3.0, 4.0]], dtype=F64)
    w = torch.tensor([2.0, 0.5], dtype=F64)
    got = plain.rms_norm(x, w, 0.5)
    inv = 1.0 / math.sqrt((9 + 16) / 2 + 0.5)
    assert torch.allclose(got, torch.tensor([[3 * inv * 2, 4 * inv * 0.5]], dtype=F64), atol=1e-15)


def test_gelu_is_the_exact_form_and_silu_is_z_sigmoid_z():
    z = torch.tensor([-3.0, -0.5, 0.0, 0.7, 4.0], dtype=F64)
    normal = torch.distributions.Normal(torch.tensor(0.0, dtype=F64), torch.tensor(1.0, dtype=F64))
    assert torch.allclose(plain.gelu_erf(z), z * normal.cdf(z), atol=1e-14)
    tanh_form = 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))
    assert float((plain.gelu_erf(z) - tanh_form).abs().max()) > 1e-5          # not the tanh approximation
    assert torch.allclose(plain.silu(z), z * torch.sigmoid(z), atol=1e-15)


def test_the_window_counts_the_query_itself():
    allowed = plain.window_mask(6, 3)
    assert allowed[5].tolist() == [False, False, False, True, True, True]     # positions 3, 4 and 5 itself
    assert allowed[1].tolist() == [True, True, False, False, False, False]
    assert plain.window_mask(4, None)[3].tolist() == [True] * 4
    assert plain.window_mask(4, 1)[2].tolist() == [False, False, True, False]  # a window of one: only itself


def test_the_cap_bends_large_scores_and_leaves_small_ones():
    q = torch.tensor([[1.0, 0.0]], dtype=F64)
    k = torch.tensor([[0.01, 0.0], [1000.0, 0.0], [-1000.0, 0.0]], dtype=F64)
    s = plain.capped_scores(q, k, 0.5, 4.0)
    assert abs(float(s[0, 0]) - 0.005) < 1e-8
    assert abs(float(s[0, 1]) - 4.0) < 1e-9 and abs(float(s[0, 2]) + 4.0) < 1e-9
    assert torch.equal(plain.capped_scores(q, k, 0.5, None), 0.5 * q @ k.T)


def test_query_heads_share_key_value_heads_in_runs():
    T, H, G, D, Dv = 3, 4, 2, 2, 3
    g = torch.Generator().manual_seed(1)
    q = torch.randn(T, H, D, generator=g, dtype=F64)
    k = torch.randn(T, G, D, generator=g, dtype=F64)
    v = torch.randn(T, G, Dv, generator=g, dtype=F64)
    out = plain.attention(q, k, v, 0.7, None, None)
    assert out.shape == (T, H, Dv)
    # head 1 reads key/value head 0 and head 2 reads head 1: the last row by hand
    for h, kv in ((1, 0), (2, 1)):
        s = 0.7 * (k[:, kv] @ q[2, h])
        assert torch.allclose(out[2, h], torch.softmax(s, 0) @ v[:, kv], atol=1e-14)
    # the first row sees only itself
    assert torch.allclose(out[0, 3], v[0, 1], atol=1e-14)


def test_values_blend_with_the_first_layers_and_only_in_later_layers():
    v = torch.tensor([[1.0, 2.0]], dtype=F64)
    first = torch.tensor([[10.0, 20.0]], dtype=F64)
    assert torch.allclose(plain.mix_values(v, first, 0.25), torch.tensor([[3.25, 6.5]], dtype=F64))
    assert torch.equal(plain.mix_values(v, first, 0.0), v)


def test_routing_by_hand():
    # 8 router outputs in 4 groups of 2, keep 2, top 3. h is a unit vector, so the logits are a column of W.
    logits = torch.tensor([2.0, 0.0, 1.0, 1.5, -1.0, 3.0, 0.5, 0.2], dtype=F64)
    w = logits[:, None].clone()
    h = torch.ones(1, 1, dtype=F64)
    s = torch.softmax(logits, 0)
    router = {"experts": 6, "identity": 2, "top": 3, "groups": {"count": 4, "keep": 2}}
    zero = torch.zeros(8, dtype=F64)
    chosen, weights = plain.route(h, w, zero, router)
    # group scores: max of (2, 0), (1, 1.5), (-1, 3), (.5, .2) -> groups 2 and 0 stay; top 3 of {0, 1, 4, 5}
    assert chosen[0].tolist() == [5, 0, 1]
    assert torch.allclose(weights[0], s[[5, 0, 1]], atol=1e-15)
    assert abs(float(weights.sum()) - 1.0) > 1e-3                     # not renormalised
    # a correction steers the choice and leaves the weights alone; it may be negative without freeing a group
    correction = torch.tensor([-0.9, 0.0, 0.5, 0.0, 0.0, -0.95, 0.0, 0.0], dtype=F64)
    chosen, weights = plain.route(h, w, correction, router)
    # choice scores: s + c. Group 1 now scores s[2] + .5, the best; then group 3 or 0...
    choice = s + correction
    group = choice.view(4, 2).max(dim=1).values
    best = set(torch.topk(group, 2).indices.tolist())
    want = sorted((e for e in range(8) if e // 2 in best), key=lambda e: -float(choice[e]))[:3]
    assert chosen[0].tolist() == want
    assert torch.allclose(weights[0], s[want], atol=1e-15)            # s without the correction
    # all choice scores negative: an excluded expert counts as -inf, not as 0
    negative = torch.full((8,), -5.0, dtype=F64)
    chosen, _ = plain.route(h, w, negative, router)
    assert chosen[0].tolist() == [5, 0, 1]


def test_identity_experts_return_their_input():
    # one expert with weights and one identity expert, both always chosen
    g = torch.Generator().manual_seed(2)
    weights = {"m.router": torch.randn(2, 4, generator=g, dtype=F64), "m.correction": torch.zeros(2, dtype=F64),
               "m.e0.gate": torch.randn(3, 4, generator=g, dtype=F64), "m.e0.up": torch.randn(3, 4, generator=g, dtype=F64),
               "m.e0.down": torch.randn(4, 3, generator=g, dtype=F64)}
    mlp = {"router": {"experts": 1, "identity": 1, "top": 2, "groups": {"count": 1, "keep": 1}}}
    h = torch.randn(2, 4, generator=g, dtype=F64)
    out = plain.routed_feed_forward(h, weights, "m.", mlp)
    s = torch.softmax(h @ weights["m.router"].T, dim=-1)
    want = s[:, :1] * plain.expert(h, weights, "m.e0.") + s[:, 1:] * h
    assert torch.allclose(out, want, atol=1e-13)


# --------------------------------------------------------------------------- configuration, registry, spec
def test_the_registry_finds_the_design_by_its_singular_key():
    from tie_amd.config.registry import resolve_architecture
    from tie_amd.errors import LoadError, UnsupportedError

    assert resolve_architecture(CONFIGS["P"]).name == "Duzozen"
    with pytest.raises(UnsupportedError):
        resolve_architecture({"architecture": "NoSuchDesign"})
    with pytest.raises(LoadError):
        resolve_architecture({"architecture": 7})


def test_the_reader_takes_every_size_and_constant_from_the_file():
    from tie_amd.config.duzozen import DenseMlpConfig, DuzozenConfig, RoutedMlpConfig

    c = DuzozenConfig.from_json(CONFIGS["P"])
    assert (c.vocab, c.width, c.norm_eps) == (CONFIGS["P"]["vocab"], CONFIGS["P"]["width"], CONFIGS["P"]["norm"]["eps"])
    for got, want in zip(c.layers, CONFIGS["P"]["layers"]):
        m = want["mixer"]
        assert (got.mixer.heads, got.mixer.kv_heads, got.mixer.dim, got.mixer.vdim) == \
            (m["heads"], m["kv_heads"], m["dim"], m["vdim"])
        assert got.mixer.scale == m["scale"] and got.mixer.softcap == m.get("softcap")
        assert got.mixer.window == (m.get("mask") or {}).get("size") and got.mixer.v_mix == bool(m.get("v_mix"))
        if want["mlp"] is None:
            assert got.mlp is None
        elif want["mlp"]["kind"] == "dense":
            assert got.mlp == DenseMlpConfig(want["mlp"]["ff"])
        else:
            r = want["mlp"]["router"]
            assert got.mlp == RoutedMlpConfig(want["mlp"]["expert"]["ff"], r["experts"], r["identity"], r["top"],
                                              r["groups"]["count"], r["groups"]["keep"])


@pytest.mark.parametrize("change, message", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["layers"][0].update(type="recurrent"), "recurrent"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"].update(scale=0.0), "scale"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "mask"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=3), "groups"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "chooses"),
    (lambda c: c["layers"][2]["mlp"].update(kind="glu"), "glu"),
    (lambda c: c["layers"][3]["mixer"].update(vdim=16), "v_mix"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_the_reader_refuses_what_does_not_fit(change, message):
    from tie_amd.config.duzozen import DuzozenConfig
    from tie_amd.errors import TieError

    broken = copy.deepcopy(CONFIGS["P"])
    change(broken)
    with pytest.raises(TieError, match=message):
        DuzozenConfig.from_json(broken)


def test_the_spec_names_the_designs_tensors_and_plans_a_cache_group_per_need():
    from tie_amd.cache.spec import PagedKV
    from tie_amd.models.builder import model_from_config

    model = model_from_config(CONFIGS["P"])
    names = {s.name: tuple(s.shape) for s in model.expected_tensors()}
    W = CONFIGS["P"]["width"]
    l0 = CONFIGS["P"]["layers"][0]
    m, r = l0["mixer"], l0["mlp"]["router"]
    assert names["embed"] == (CONFIGS["P"]["vocab"], W) and names["head"] == (CONFIGS["P"]["vocab"], W)
    assert names["final.norm"] == (W,)
    assert names["l0.mix.q"] == (m["heads"] * m["dim"], W) and names["l0.mix.k"] == (m["kv_heads"] * m["dim"], W)
    assert names["l0.mix.v"] == (m["kv_heads"] * m["vdim"], W) and names["l0.mix.o"] == (W, m["heads"] * m["vdim"])
    assert names["l0.mix.vmix"] == (1,)
    assert names["l0.mlp.router"] == (r["experts"] + r["identity"], W)
    assert names["l0.mlp.correction"] == (r["experts"] + r["identity"],)
    assert names[f"l0.mlp.e{r['experts'] - 1}.down"] == (W, l0["mlp"]["expert"]["ff"])
    assert f"l0.mlp.e{r['experts']}.gate" not in names                  # identity experts have no tensors
    assert not any(n.startswith("l1.mlp") or n.startswith("l1.norm2") for n in names)    # layer 1 has no feed-forward
    assert "l1.mix.vmix" not in names                                   # nor does it blend values
    assert names["l2.mlp.up"] == (CONFIGS["P"]["layers"][2]["mlp"]["ff"], W)
    # one cache group per (heads, head size, window); sizes in steps of 16 where nothing rotates the heads
    needs = [g.need for g in model.cache_plan.groups]
    assert all(isinstance(n, PagedKV) and n.head_dim % 16 == 0 for n in needs)
    windows = sorted((n.window or 0) for n in needs)
    assert windows == sorted({(l["mixer"].get("mask") or {}).get("size") or 0 for l in CONFIGS["P"]["layers"]})
    assert model.capturable()


def test_a_random_model_of_the_design_is_written_and_read_back(tmp_path):
    from tie_amd.weights.loader import load_model_folder
    from tie_amd.weights.random_init import write_random_model

    write_random_model(tmp_path, CONFIGS["Q"], seed=3, dtype="bfloat16")
    files = load_model_folder(tmp_path)
    assert files.config_values["architecture"] == "Duzozen"
    assert files.tensors["l0.mix.vmix"].shape == (1,)
