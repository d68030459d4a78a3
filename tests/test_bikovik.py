"""Bikovik without a GPU: the configuration reader, the tensors it expects, the cache manager's
pages for a window that keeps the first tokens, and pins of the plain implementation (each
mechanism against a second, independent formulation)."""

from __future__ import annotations

import copy
import json

import pytest
import torch

from bikovik_cases import CASES, SINGLE, make_tensors, write_model
from plain import bikovik_plain as plain

F64 = torch.float64


# -- configuration and weights ---------------------------------------------------------

def test_config_is_found_by_its_architecture_key_and_states_the_layers_as_parts():
    from lockstep_amd.config import BikovikConfig, config_from_dict

    cfg = config_from_dict(CASES["A"]["raw"])
    assert isinstance(cfg, BikovikConfig)
    spec = cfg.model_spec()
    assert [layer.mixer.kind for layer in spec.layers] == ["hgrn2", "talking_attention", "retention", "talking_attention"]
    assert [layer.mixer.params.get("v_mix") for layer in spec.layers] == [None, "source", None, "mix"]
    attn = spec.layers[1].mixer
    assert (attn["num_heads"], attn["num_kv_heads"], attn["head_dim"], attn["value_dim"]) == (4, 2, 32, 16)
    assert (attn["window"], attn["keep_first"], attn["scale"]) == (24, 3, 0.25)
    assert attn["position"].params == {"rotary_dim": 8, "theta": 10000.0}
    assert spec.layers[2].mixer["decay"] == (0.9, 0.99)
    assert spec.embedding["scale"] == 4.0 and spec.head["softcap"] == 20.0
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()


def test_a_layer_without_feed_forward_and_a_config_without_soft_cap():
    from lockstep_amd.config import config_from_dict
    from lockstep_amd.engine.model import collect_weight_specs

    raw = copy.deepcopy(CASES["B"]["raw"])
    del raw["logit_softcap"]
    spec = config_from_dict(raw).model_spec()
    assert spec.head["softcap"] is None
    assert spec.layers[1].feed_forward is None
    names = {w.name: w for w in collect_weight_specs(spec)}
    assert "l1.mlp.gate" not in names and "l0.mlp.gate" in names
    assert names["l1.norm2"].optional and not names["l0.norm2"].optional
    assert names["l3.mix.talk"].shape == (3, 3) and names["l0.mix.v"].shape == (3 * 24, 96)
    assert "l0.mix.vmix" not in names and "l3.mix.vmix" in names


@pytest.mark.parametrize("breakage, message", [
    (lambda raw: raw["layers"][0].update(type="mamba"), "not one of"),
    (lambda raw: raw["layers"][1]["mixer"].pop("kv_heads"), "kv_heads"),
    (lambda raw: raw["layers"][1]["mixer"]["rot"].update(dims=7), "even"),
    (lambda raw: raw["layers"][0]["mlp"].update(kind="experts"), "not built"),
    (lambda raw: raw.pop("width"), "width"),
    (lambda raw: raw["layers"][3]["mixer"].update(vdim=32), "agree"),
])
def test_config_errors_name_what_is_wrong(breakage, message):
    from lockstep_amd.config import ConfigError, config_from_dict

    raw = copy.deepcopy(CASES["A"]["raw"])
    breakage(raw)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(raw).model_spec()


def test_random_weights_folder_loads_and_a_missing_tensor_is_named(tmp_path):
    from lockstep_amd.config import config_from_dir
    from lockstep_amd.engine.model import collect_weight_specs
    from lockstep_amd.weights import WeightError, load_weights

    raw = CASES["B"]["raw"]
    tensors = make_tensors(raw, seed=3)
    assert tensors["l0.norm1.alpha"].shape == () and tensors["l3.mix.talk"].shape == (3, 3)
    assert 0 < float(tensors["l2.mix.lower"].float().min()) and float(tensors["l2.mix.lower"].float().max()) < 1
    folder = write_model(tmp_path / "m", raw, tensors)
    specs = collect_weight_specs(config_from_dir(folder).model_spec())
    store = load_weights(folder, specs)
    assert store.get("l1.mix.g").shape == (3 * 40, 96)
    del tensors["l2.mix.f.b"]
    broken = write_model(tmp_path / "broken", raw, tensors)
    with pytest.raises(WeightError, match="l2.mix.f.b"):
        load_weights(broken, specs)


# -- cache pages under a window that keeps the first tokens -------------------------------

def test_pages_a_window_has_passed_are_given_back_except_those_of_the_kept_tokens():
    from lockstep_amd.cache import CacheManager
    from lockstep_amd.parts import PagedKVSpec, StateSpec

    units = [PagedKVSpec(2, 32, window=24, value_dim=16, keep_first=10), StateSpec((2, 16, 32)),
             PagedKVSpec(2, 32, window=24, value_dim=16, keep_first=10), PagedKVSpec(2, 32, window=24, value_dim=16)]
    cache = CacheManager(units, page_size=8, num_pages=12, max_requests=2, max_tokens_per_request=400)
    assert len(cache.groups) == 2 and cache.groups[0].units == [0, 2]
    cache.open("a")
    for end in range(5, 200, 7):
        cache.reserve("a", end)
        cache.commit("a", end)
        cache.audit()
        kept, plain_window = cache.request_pages("a", 0), cache.request_pages("a", 1)
        first_needed = max(0, end - 24 + 1) // 8
        for logical, page in enumerate(kept):
            assert (page >= 0) == (logical < 2 or logical >= first_needed), (end, logical)
        for logical, page in enumerate(plain_window):
            assert (page >= 0) == (logical >= first_needed), (end, logical)
        assert sum(p >= 0 for p in kept) <= 2 + 5       # the pool never holds more than the window and the kept pages
    cache.close("a")
    cache.audit()
    assert cache.free_pages == [12, 12] and cache.free_slots == 2


def test_a_request_that_starts_far_in_reserves_the_kept_pages_too():
    from lockstep_amd.cache import CacheManager
    from lockstep_amd.parts import PagedKVSpec

    cache = CacheManager([PagedKVSpec(1, 16, window=16, value_dim=8, keep_first=4)], page_size=8, num_pages=16,
                         max_requests=1, max_tokens_per_request=256)
    assert cache.pages_to_reserve(None, 0, 100) == [13]
    assert cache.pages_to_reserve(None, 90, 100) == [1 + 4]     # the kept page, and pages 9..12 of the window
    cache.open("r")
    cache.reserve("r", 100, start=90)
    pages = cache.request_pages("r")
    assert [p >= 0 for p in pages] == [True] + [False] * 8 + [True] * 4
    cache.audit()


# -- pins of the plain implementation -------------------------------------------------------

def test_visibility_at_the_edges_of_the_window_and_of_the_kept_tokens():
    visible = plain.window_with_kept_first(40, size=8, keep_first=3)
    assert visible[30, 30] and visible[30, 23] and not visible[30, 22]       # i - j < 8
    assert visible[30, 2] and not visible[30, 3]                             # j < 3 stays
    assert not visible[5, 6] and visible[7, 0] and visible[12, 5]
    assert int(visible[30].sum()) == 8 + 3


def test_rotation_turns_pairs_by_position_and_leaves_the_rest():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 2, 12, generator=g, dtype=F64)
    pos = torch.tensor([0, 1, 7, 100, 1000])
    y = plain.rotate_pairs(x, pos, dims=8, base=100.0)
    assert torch.equal(y[..., 8:], x[..., 8:]) and torch.allclose(y[0], x[0])
    assert torch.allclose((y[..., :8] ** 2).sum(-1), (x[..., :8] ** 2).sum(-1))
    # pair (1, 5) at position 7: angle 7 * 100^(-2/8)
    a = 7 * 100.0 ** (-2.0 / 8)
    u, v = x[2, 0, 1], x[2, 0, 5]
    assert torch.allclose(y[2, 0, 1], u * torch.cos(torch.tensor(a)) - v * torch.sin(torch.tensor(a)))
    assert torch.allclose(y[2, 0, 5], v * torch.cos(torch.tensor(a)) + u * torch.sin(torch.tensor(a)))
    # the scalar product of two rotated vectors depends on the distance of their positions only
    q = torch.randn(1, 1, 8, generator=g, dtype=F64).expand(2, 1, 8)
    k = torch.randn(1, 1, 8, generator=g, dtype=F64).expand(2, 1, 8)
    near = (plain.rotate_pairs(q, torch.tensor([9, 59]), 8, 100.0) * plain.rotate_pairs(k, torch.tensor([4, 54]), 8, 100.0)).sum(-1)
    assert torch.allclose(near[0], near[1])


def test_talking_heads_with_the_identity_is_plain_grouped_attention():
    g = torch.Generator().manual_seed(1)
    n, heads, groups, d, dv = 9, 4, 2, 6, 5
    q, k, v = (torch.randn(n, h, s, generator=g, dtype=F64) for h, s in ((heads, d), (groups, d), (groups, dv)))
    visible = plain.window_with_kept_first(n, 4, 1)
    out = plain.talking_heads_attention(q, k, v, 0.3, torch.eye(heads, dtype=F64), visible)
    for h in range(heads):
        for i in range(n):
            js = [j for j in range(n) if visible[i, j]]
            s = torch.stack([0.3 * (q[i, h] @ k[j, h // 2]) for j in js])
            want = (torch.softmax(s, 0)[:, None] * torch.stack([v[j, h // 2] for j in js])).sum(0)
            assert torch.allclose(out[i, h], want)
    # and a mixing matrix that swaps two heads swaps their weights (values stay with the reading head's group)
    swap = torch.eye(heads, dtype=F64)[[1, 0, 2, 3]]
    mixed = plain.talking_heads_attention(q, k, v, 0.3, swap, visible)
    assert torch.allclose(mixed[:, 0], out[:, 1]) and torch.allclose(mixed[:, 1], out[:, 0]) and torch.allclose(mixed[:, 2:], out[:, 2:])


def test_the_recurrence_equals_its_sum_over_the_past_and_can_be_cut():
    g = torch.Generator().manual_seed(2)
    n, d, dv = 11, 4, 3
    q, k = torch.randn(n, d, generator=g, dtype=F64), torch.randn(n, d, generator=g, dtype=F64)
    v = torch.randn(n, dv, generator=g, dtype=F64)
    decay = torch.full((n, d), 0.9, dtype=F64)
    out, last = plain.gated_outer_product_recurrence(q, decay, k, v)
    for t in range(n):          # retention: o_t = sum_(s <= t) decay^(t-s) (q_t . k_s) v_s
        want = sum(0.9 ** (t - s) * (q[t] @ k[s]) * v[s] for s in range(t + 1))
        assert torch.allclose(out[t], want)
    f = torch.rand(n, d, generator=g, dtype=F64)
    whole, _ = plain.gated_outer_product_recurrence(q, f, 1 - f, v)
    head, state = plain.gated_outer_product_recurrence(q[:6], f[:6], 1 - f[:6], v[:6])
    tail, _ = plain.gated_outer_product_recurrence(q[6:], f[6:], 1 - f[6:], v[6:], state)
    assert torch.allclose(torch.cat([head, tail]), whole)
    # a gate of one keeps a row for ever and writes nothing into it
    ones = torch.ones(n, d, dtype=F64)
    kept, _ = plain.gated_outer_product_recurrence(q, ones, 1 - ones, v)
    assert float(kept.abs().max()) == 0.0


def test_small_functions():
    x = torch.tensor([-3.0, -0.5, 0.0, 0.5, 3.0], dtype=F64)
    assert torch.allclose(plain.dynamic_tanh(x, torch.tensor(2.0), torch.tensor(0.5), torch.tensor(0.1)),
                          torch.tanh(0.1 * x) * 2.0 + 0.5)
    y = plain.clamped_gated_unit(torch.tensor([5.0, -5.0, 0.5], dtype=F64), torch.tensor([9.0, -9.0, 0.25], dtype=F64), 1.0)
    want = [1.0 / (1 + torch.exp(torch.tensor(-1.702, dtype=F64))) * 2.0, -5.0 / (1 + torch.exp(torch.tensor(8.51, dtype=F64))) * 0.0,
            0.5 / (1 + torch.exp(torch.tensor(-0.851, dtype=F64))) * 1.25]
    assert torch.allclose(y, torch.stack([torch.as_tensor(w, dtype=F64) for w in want]))
    assert torch.allclose(plain.soft_cap(torch.tensor([1e6, 0.1], dtype=F64), 17.0), torch.tensor([17.0, 17 * torch.tanh(torch.tensor(0.1 / 17, dtype=F64))], dtype=F64))
    r = plain.root_mean_square_norm(torch.tensor([[3.0, 4.0]], dtype=F64), 0.0)
    assert torch.allclose(r, torch.tensor([[3.0, 4.0]], dtype=F64) / (12.5 ** 0.5))


def test_plain_model_runs_every_case_and_later_tokens_do_not_change_earlier_logits():
    for case in list(CASES.values()) + list(SINGLE.values()):
        raw = case["raw"]
        model = plain.PlainBikovik(raw, make_tensors(raw, seed=5))
        tokens = torch.randint(0, raw["vocab"], (30,), generator=torch.Generator().manual_seed(9)).tolist()
        whole, layers = model.forward(tokens, return_layers=True)
        assert whole.shape == (30, raw["vocab"]) and layers.shape[0] == len(raw["layers"])
        assert float(whole.abs().max()) < raw["logit_softcap"]
        assert torch.allclose(model.forward(tokens[:17]), whole[:17], atol=1e-12)
