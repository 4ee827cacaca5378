"""The plain Topapel pinned by cases worked out by hand, and the design's reader, spec and cache needs (CPU)."""

import copy
import math

import pytest
import torch

import plain_topapel as plain
from topapel_fixtures import CONFIGS

F64 = torch.float64


def test_decayed_linear_attention_by_hand():
    q = torch.tensor([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0]], dtype=F64)
    k = torch.tensor([[1.0, 2.0], [3.0, 0.0], [0.0, 1.0]], dtype=F64)
    v = torch.tensor([[1.0], [10.0], [100.0]], dtype=F64)
    out = plain.decayed_linear_attention(q, k, v, 0.5)
    # S_0 = k0 v0 = [1, 2];  S_1 = 0.5 S_0 + k1 v1 = [30.5, 1];  S_2 = 0.5 S_1 + k2 v2 = [15.25, 100.5]
    assert out.flatten().tolist() == [1.0, 1.0, 115.75]
    # the same as a sum over earlier tokens with weights decay^(t-s) (q_t . k_s)
    t = 2
    direct = sum(0.5 ** (t - s) * float(q[t] @ k[s]) * float(v[s]) for s in range(3))
    assert direct == 115.75


def test_chunks_are_counted_from_position_zero():
    allowed = plain.chunk_mask(7, 3)
    assert allowed[2].tolist() == [True, True, True, False, False, False, False]
    assert allowed[3].tolist() == [False, False, False, True, False, False, False]
    assert allowed[5].tolist() == [False, False, False, True, True, True, False]
    assert plain.chunk_mask(4, None)[3].tolist() == [True] * 4


def test_the_sink_counts_once_unscaled_and_has_no_value():
    scores = torch.tensor([[0.0, math.log(2.0)]], dtype=F64)
    w = plain.softmax_with_sink(scores, torch.tensor([[True, True]]), math.log(5.0))
    assert torch.allclose(w, torch.tensor([[1 / 8, 2 / 8]], dtype=F64))
    w = plain.softmax_with_sink(scores, torch.tensor([[True, False]]), -1e9)        # a sink far below: a plain softmax
    assert torch.allclose(w, torch.tensor([[1.0, 0.0]], dtype=F64))
    w = plain.softmax_with_sink(scores, torch.tensor([[True, True]]), 800.0)        # a sink far above: nothing passes
    assert float(w.sum()) < 1e-300 or float(w.sum()) == 0.0


def test_rotation_of_part_of_a_head():
    x = torch.arange(1, 7, dtype=F64).view(1, 1, 6)
    out = plain.rotate_partial(x.repeat(2, 1, 1), torch.tensor([0, 3]), dims=4, base=100.0, factor=2.0)
    assert out[0].flatten().tolist() == [1, 2, 3, 4, 5, 6]                 # position 0 turns nothing
    a0, a1 = 3 * 1.0 / 2.0, 3 * 100.0 ** (-0.5) / 2.0
    want = [1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
            3 * math.cos(a0) + 1 * math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 5, 6]
    assert torch.allclose(out[1].flatten(), torch.tensor(want, dtype=F64))


def test_the_recurrences_candidate_and_scan():
    u = torch.tensor([-2.0, 0.0, 1.5], dtype=F64)
    c = plain.mingru_candidate(u)
    assert torch.allclose(c, torch.tensor([1 / (1 + math.exp(2.0)), 0.5, 2.0], dtype=F64))
    z = torch.tensor([[0.5], [0.25], [1.0]], dtype=F64)
    cand = torch.tensor([[4.0], [8.0], [-1.0]], dtype=F64)
    assert plain.mingru_scan(z, cand).flatten().tolist() == [2.0, 3.5, -1.0]


def test_polynorm_by_hand():
    z = torch.tensor([[1.0, -1.0, 2.0, -2.0]], dtype=F64)
    out = plain.polynorm(z, torch.tensor([2.0, 3.0, 5.0, 7.0]), 0.0)
    r1, r2, r3 = math.sqrt(2.5), math.sqrt(8.5), math.sqrt(32.5)
    want = [2 * a / r1 + 3 * a * a / r2 + 5 * a ** 3 / r3 + 7 for a in (1.0, -1.0, 2.0, -2.0)]
    assert torch.allclose(out.flatten(), torch.tensor(want, dtype=F64))


def test_norm_weights_are_stored_around_zero():
    x = torch.tensor([[3.0, 4.0]], dtype=F64)
    out = plain.norm_one_plus(x, torch.tensor([0.0, 1.0]), 0.0)
    assert torch.allclose(out, torch.tensor([[3.0, 8.0]], dtype=F64) / math.sqrt(12.5))


# ----------------------------------------------------------------------------------- reader, registry, spec
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_the_reader_and_the_spec(name):
    import tie_amd  # noqa: F401
    from tie_amd.cache.spec import FixedState, PagedKV
    from tie_amd.models.builder import model_from_config

    config = CONFIGS[name]
    model = model_from_config(config)
    assert model.spec.architecture == "Topapel"
    names = {s.name for s in model.expected_tensors()}
    assert "embed" in names and "final.norm" in names and "head" not in names
    needs = [g.need for g in model.cache_plan.groups]
    for i, layer in enumerate(config["layers"]):
        m = layer["mixer"]
        p = f"l{i}.mix."
        if layer["type"] == "lightning":
            assert {p + k for k in ("q", "k", "v", "g", "o", "norm")} <= names
            assert FixedState((m["heads"], m["dim"], m["vdim"])) in needs
        elif layer["type"] == "attention":
            assert {p + k for k in ("q", "q.b", "k", "k.b", "o", "o.b", "q.norm", "k.norm", "sink")} <= names
            assert p + "v" not in names
            assert PagedKV(m["kv_heads"], m["dim"], None, (m.get("mask") or {}).get("size")) in needs
        else:
            assert {p + k for k in ("z", "z.b", "x", "x.b", "g", "o")} <= names and p + "g.b" not in names
            assert FixedState((m["width"],)) in needs
        assert (f"l{i}.mlp.act" in names) == (layer["mlp"] is not None)
        assert (f"l{i}.norm2" in names) == (layer["mlp"] is not None)
    assert model.capturable()


def test_what_does_not_fit_is_refused():
    import tie_amd  # noqa: F401
    from tie_amd.errors import LoadError, UnsupportedError
    from tie_amd.models.builder import model_from_config

    def changed(path, value):
        config = copy.deepcopy(CONFIGS["A"])
        node = config
        for key in path[:-1]:
            node = node[key]
        node[path[-1]] = value
        return config

    for path, value, error in [
        (("layers", 1, "mixer", "decay"), [0.5], LoadError),                  # one decay a head
        (("layers", 0, "mixer", "vdim"), 8, LoadError),                       # the values are the keys
        (("layers", 0, "mixer", "kv_heads"), 3, LoadError),
        (("layers", 0, "mixer", "rot", "dims"), 7, LoadError),
        (("layers", 0, "mixer", "rot", "dims"), 18, LoadError),
        (("layers", 0, "mixer", "mask", "size"), 0, LoadError),
        (("layers", 2, "type"), "lstm", UnsupportedError),
        (("layers", 2, "mlp", "kind"), "moe", UnsupportedError),
        (("layers", 2, "mixer", "width"), 0, LoadError),
        (("norm", "eps"), 0.0, LoadError),
        (("logit_softcap",), -1.0, LoadError),
    ]:
        with pytest.raises(error):
            model_from_config(changed(path, value))


def test_pages_of_chunks_left_behind_go_back():
    from tie_amd.cache.manager import FREED, CacheManager
    from tie_amd.cache.spec import FixedState, PagedKV, plan_cache

    need = PagedKV(2, 16, None, 10)
    assert need.reach == 10 and [need.first_needed(p) for p in (0, 9, 10, 25)] == [0, 0, 10, 20]
    with pytest.raises(Exception):
        PagedKV(2, 16, 5, 10)
    plan = plan_cache([need, FixedState((3,)), PagedKV(2, 16)], [None, None, None])
    cache = CacheManager(plan, block_size=4, num_blocks=12, max_state_slots=2)
    req = cache.new_request()
    assert cache.reserve(req, 23)
    assert cache.trim(req, 23) == 5                      # chunk 20..29 is current: positions 0..19 are five pages
    assert req.tables[0][:6] == [FREED] * 5 + [req.tables[0][5]] and FREED not in req.tables[1]
    assert cache.trim(req, 29) == 0 and cache.reserve(req, 31) and cache.trim(req, 31) == 2
    assert cache.capacity_tokens == 48                   # the group that keeps every key limits a request
    other = cache.new_request()
    assert cache.reserve(other, 16) and other.state_slot != req.state_slot
    third = cache.new_request()
    assert not cache.reserve(third, 4)                   # no state slot left
    cache.release(req)
    assert cache.reserve(third, 4) and third.state_slot >= 0
    cache.release(other)
    cache.release(third)
    assert cache.all_free()
