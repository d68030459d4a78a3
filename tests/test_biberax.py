"""Biberax without a GPU: the configuration reader, the tensors it expects, the cache manager's pages
under a chunked mask, the table of distances that the attention part hands its kernel, the scaled
rotation tables, and pins of the plain implementation (each mechanism against a second, independent
formulation)."""

from __future__ import annotations

import copy
import math

import pytest
import torch

from biberax_cases import CASES, SINGLE, make_tensors, write_model
from plain import biberax_plain as plain

F64 = torch.float64


# -- configuration and weights ---------------------------------------------------------

def test_config_is_found_by_its_architecture_key_and_states_the_layers_as_parts():
    from lockstep_amd.config import BiberaxConfig, config_from_dict

    cfg = config_from_dict(CASES["A"]["raw"])
    assert isinstance(cfg, BiberaxConfig)
    spec = cfg.model_spec()
    assert [layer.mixer.kind for layer in spec.layers] == ["sink_attention"] * 3
    assert [layer.feed_forward.kind for layer in spec.layers] == ["gated_mlp", "routed_experts", "routed_experts"]
    first, second = spec.layers[0].mixer, spec.layers[1].mixer
    assert (first["num_heads"], first["num_kv_heads"], first["head_dim"], first["value_dim"]) == (4, 2, 32, 16)
    assert (first["chunk"], first["sink"], first["scale"], first["gate"]) == (24, "zero", 0.25, True)
    assert first["position"].kind == "rope_scaled" and first["position"]["pairing"] == "neighbours"
    assert first["position"]["scaling"] == {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64.0}
    assert (second["sink"], second["shared_kv"], second["bias"], second["out_bias"]) == ("learned", True, True, True)
    assert second["distance_bias"] == {"farthest": 60.0, "rows": 12} and second["qk_norm"] == 1e-5
    assert second["position"].kind == "no_position" and second.params.get("chunk") is None
    experts = spec.layers[1].feed_forward
    assert (experts["experts"], experts["top"], experts["limit"], experts["alpha"]) == (6, 2, 2.0, 1.702)
    assert experts["shared"].kind == "clamped_gated_mlp" and experts["shared"]["limit"] == 1.0
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()


def test_layers_without_feed_forward_shared_expert_mask_or_rotation():
    from lockstep_amd.config import config_from_dict
    from lockstep_amd.engine.model import collect_weight_specs

    spec = config_from_dict(CASES["B"]["raw"]).model_spec()
    assert spec.layers[1].feed_forward is None and spec.layers[0].feed_forward["shared"] is None
    names = {w.name: w for w in collect_weight_specs(spec)}
    assert "l1.mlp.gate" not in names and names["l1.norm2"].optional and not names["l0.norm2"].optional
    assert "l0.mlp.shared.gate" not in names and names["l3.mlp.shared.down"].shape == (96, 24)
    assert names["l0.mix.rel"].shape == (-1, 6) and names["l0.mix.rel"].free == 20
    assert "l0.mix.v" not in names and "l0.mix.k.b" in names and "l0.mix.o.b" in names
    assert names["l1.mix.v"].shape == (40, 96) and names["l1.mix.g"].shape == (6 * 40, 96)
    assert [n for n in names if n.startswith("l0.mlp.e")] == [f"l0.mlp.e{i}.{m}" for i in range(5) for m in ("gate", "up", "down")]
    spec = config_from_dict(CASES["C"]["raw"]).model_spec()
    assert spec.layers[0].mixer["position"].kind == "no_position" and spec.layers[0].mixer["chunk"] is None


@pytest.mark.parametrize("breakage, message", [
    (lambda raw: raw["layers"][0].update(type="mamba"), "not one of"),
    (lambda raw: raw["layers"][1]["mixer"].pop("kv_heads"), "kv_heads"),
    (lambda raw: raw["layers"][0]["mixer"]["rot"].update(dims=7), "even"),
    (lambda raw: raw["layers"][0]["mlp"].update(kind="experts"), "not one of"),
    (lambda raw: raw.pop("width"), "width"),
    (lambda raw: raw["layers"][1]["mixer"].update(vdim=32), "vdim"),
    (lambda raw: raw["layers"][1]["mlp"]["router"].update(top=9), "exceeds"),
    (lambda raw: raw["layers"][1]["mixer"].pop("bias_max"), "bias_max"),
    (lambda raw: raw["layers"][0]["mixer"]["rot"]["scaling"].pop("low"), "low"),
])
def test_config_errors_name_what_is_wrong(breakage, message):
    from lockstep_amd.config import ConfigError, config_from_dict

    raw = copy.deepcopy(CASES["A"]["raw"])
    breakage(raw)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(raw)


def test_random_weights_folder_loads_and_a_table_may_have_any_number_of_rows(tmp_path):
    from lockstep_amd.config import config_from_dir
    from lockstep_amd.engine.model import collect_weight_specs
    from lockstep_amd.weights import WeightError, load_weights

    raw = CASES["A"]["raw"]
    tensors = make_tensors(raw, seed=3)
    assert tensors["l1.mix.rel"].shape == (12, 4)
    folder = write_model(tmp_path / "m", raw, tensors)
    specs = collect_weight_specs(config_from_dir(folder).model_spec())
    store = load_weights(folder, specs)
    assert store.get("l1.mix.sink").shape == (4,)
    other = dict(tensors)
    other["l1.mix.rel"] = torch.zeros(30, 4, dtype=torch.bfloat16)          # the checkpoint decides the rows ...
    load_weights(write_model(tmp_path / "n", raw, other), specs)
    other["l1.mix.rel"] = torch.zeros(30, 5, dtype=torch.bfloat16)          # ... but not the heads
    with pytest.raises(WeightError, match="l1.mix.rel"):
        load_weights(write_model(tmp_path / "o", raw, other), specs)
    del other["l1.mix.rel"], other["l2.mlp.e3.up"]
    with pytest.raises(WeightError, match="l2.mlp.e3.up"):
        load_weights(write_model(tmp_path / "p", raw, other), specs)


# -- the cache manager under a chunked mask ------------------------------------------------------

def test_pages_before_the_current_chunk_are_given_back():
    from lockstep_amd.cache import CacheManager
    from lockstep_amd.parts import PagedKVSpec

    cache = CacheManager([PagedKVSpec(2, 16, value_dim=8, chunk=20), PagedKVSpec(2, 16, value_dim=8)], page_size=8,
                         num_pages=40, max_requests=2, max_tokens_per_request=256)
    assert len(cache.groups) == 2
    cache.open("a")
    for end in range(3, 200, 7):
        cache.reserve("a", end)
        cache.commit("a", end)
        cache.audit()
        chunked, full = cache.request_pages("a", 0), cache.request_pages("a", 1)
        first_needed = (end // 20 * 20) // 8           # the page that holds the first key of the next query's chunk
        for logical, page in enumerate(chunked):
            assert (page >= 0) == (logical >= first_needed), (end, logical)
        assert all(page >= 0 for page in full)
        assert sum(p >= 0 for p in chunked) <= 4       # a chunk of 20 never spans more than four pages of 8
    cache.close("a")
    cache.audit()
    assert cache.free_pages == [40, 40] and cache.free_slots == 2


def test_a_portion_that_starts_inside_a_late_chunk_reserves_from_that_chunk_on():
    from lockstep_amd.cache import CacheManager
    from lockstep_amd.parts import PagedKVSpec

    cache = CacheManager([PagedKVSpec(1, 16, chunk=30)], page_size=8, num_pages=16, max_requests=1, max_tokens_per_request=256)
    assert cache.pages_to_reserve(None, 0, 100) == [13]
    assert cache.pages_to_reserve(None, 95, 100) == [13 - 90 // 8]     # chunk 3 starts at 90, on page 11
    assert cache.why_not_shareable() is not None


# -- what the attention part hands its kernel ---------------------------------------------------------

@pytest.mark.parametrize("rows, farthest", [(12, 60.0), (6, 90.0), (8, 16.0), (20, 5000.0), (32, 256.0), (2, 3.0)])
def test_the_table_by_distance_follows_the_bucket_rule(rows, farthest):
    from lockstep_amd.parts.sink_attention import distance_buckets

    table = distance_buckets(rows, farthest)
    assert table[-1] == rows - 1 and rows - 1 not in table[:-1]
    assert table[:rows // 2] == list(range(rows // 2))
    for n in range(0, int(farthest) + 50):
        assert table[min(n, len(table) - 1)] == plain.distance_bucket(n, rows, farthest), n
    assert all(b >= a for a, b in zip(table, table[1:]))


def test_scaled_rotation_tables_match_the_plain_frequencies():
    from lockstep_amd.config.base import PartSpec
    from lockstep_amd.parts import build_part

    scaling = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
    part = build_part(PartSpec("rope_scaled", {"rotary_dim": 16, "theta": 100.0, "pairing": "neighbours", "scaling": scaling}))
    want = plain.scaled_frequencies(16, 100.0, scaling)
    assert torch.allclose(part.frequencies(), want, rtol=1e-14, atol=0)
    plain_freq = plain.scaled_frequencies(16, 100.0)
    ratio = (want / plain_freq).tolist()
    assert ratio[0] == 1.0 and ratio[-1] == 1 / 8.0 and any(1 / 8.0 < r < 1.0 for r in ratio)      # all three ranges
    cos, sin = part.tables(torch.tensor([0, 3, 1000]))
    assert torch.allclose(cos[1].double(), torch.cos(3 * want), atol=1e-7) and torch.allclose(sin[2].double(), torch.sin(1000 * want), atol=1e-7)
    assert part.neighbours and part.dim_order(20) == [0, 2, 4, 6, 8, 10, 12, 14, 1, 3, 5, 7, 9, 11, 13, 15, 16, 17, 18, 19]
    unscaled = build_part(PartSpec("rope_scaled", {"rotary_dim": 16, "theta": 100.0, "pairing": "half", "scaling": None}))
    assert torch.allclose(unscaled.frequencies(), plain_freq) and unscaled.dim_order(20) is None


# -- pins of the plain implementation -------------------------------------------------------

def test_visibility_inside_chunks():
    visible = plain.same_chunk(40, size=7)
    assert visible[13, 13] and visible[13, 7] and not visible[13, 6]         # 13 lies in 7..13
    assert visible[14, 14] and not visible[14, 13]                           # 14 starts a chunk
    assert not visible[5, 6] and int(visible[20].sum()) == 7 and int(visible[21].sum()) == 1
    assert torch.equal(plain.same_chunk(10, 100), plain.causal(10))


def test_rotation_turns_neighbouring_pairs_by_position_and_leaves_the_rest():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 2, 12, generator=g, dtype=F64)
    pos = torch.tensor([0, 1, 7, 100, 1000])
    f = plain.scaled_frequencies(8, 100.0)
    y = plain.rotate_neighbours(x, pos, f)
    assert torch.equal(y[..., 8:], x[..., 8:]) and torch.allclose(y[0], x[0])
    assert torch.allclose((y[..., :8] ** 2).sum(-1), (x[..., :8] ** 2).sum(-1))
    a = torch.tensor(7 * 100.0 ** (-2.0 * 1 / 8))                             # pair (2, 3) at position 7
    u, v = x[2, 0, 2], x[2, 0, 3]
    assert torch.allclose(y[2, 0, 2], u * torch.cos(a) - v * torch.sin(a))
    assert torch.allclose(y[2, 0, 3], v * torch.cos(a) + u * torch.sin(a))
    q = torch.randn(1, 1, 8, generator=g, dtype=F64).expand(2, 1, 8)
    k = torch.randn(1, 1, 8, generator=g, dtype=F64).expand(2, 1, 8)
    near = (plain.rotate_neighbours(q, torch.tensor([9, 59]), f) * plain.rotate_neighbours(k, torch.tensor([4, 54]), f)).sum(-1)
    assert torch.allclose(near[0], near[1])                                   # only the distance enters a score


def test_a_sink_is_a_key_with_a_zero_value():
    """The softmax with a sink equals the plain softmax over the keys and one more key per head whose
    score is the sink and whose value is zero; with a sink far below every score it is the plain softmax."""
    g = torch.Generator().manual_seed(1)
    n, heads, groups, d, dv = 9, 4, 2, 6, 5
    q, k, v = (torch.randn(n, h, s, generator=g, dtype=F64) for h, s in ((heads, d), (groups, d), (groups, dv)))
    sink = torch.randn(heads, generator=g, dtype=F64)
    got = plain.attention_with_sink(q, k, v, 0.3, plain.causal(n), sink)
    for h in range(heads):
        for i in range(n):
            scores = torch.cat([(q[i, h] @ k[:i + 1, h // 2].T) * 0.3, sink[h:h + 1]])
            weights = torch.softmax(scores, dim=0)
            assert torch.allclose(got[i, h], weights[:-1] @ v[:i + 1, h // 2])
            assert float(weights[:-1].sum()) < 1.0
    none = plain.attention_with_sink(q, k, v, 0.3, plain.causal(n), None)
    far = plain.attention_with_sink(q, k, v, 0.3, plain.causal(n), torch.full((heads,), -200.0, dtype=F64))
    assert torch.allclose(none, far)
    assert torch.allclose(none[0, :, :], v[0].repeat_interleave(2, dim=0))    # one key: its value


def test_distance_buckets_by_hand():
    # 8 rows up to distance 32: 0..3 themselves, then four rows in equal steps of ln(8)/4 from distance 4 on
    edges = [4 * math.exp(j * math.log(32 / 4) / 4) for j in range(5)]       # 4, 6.7, 11.3, 19.0, 32
    for n in range(0, 70):
        want = n if n < 4 else min(7, 4 + max(j for j in range(5) if n >= edges[j] - 1e-9))
        assert plain.distance_bucket(n, 8, 32.0) == want, n
    bias = plain.distance_bias(6, torch.arange(16, dtype=F64).reshape(8, 2), 32.0)
    assert bias[1, 5, 5] == 1 and bias[1, 5, 1] == 2 * 4 + 1 and bias[0, 5, 0] == 2 * 4 and bias[0, 2, 4] == 0


def test_routing_picks_the_largest_logits_and_weighs_them_among_themselves():
    g = torch.Generator().manual_seed(2)
    width, experts, ff = 10, 5, 6
    weights = {"m.router": torch.randn(experts, width, generator=g), "m.router.b": torch.randn(experts, generator=g)}
    for e in range(experts):
        weights.update({f"m.e{e}.gate": torch.randn(ff, width, generator=g), f"m.e{e}.up": torch.randn(ff, width, generator=g),
                        f"m.e{e}.down": torch.randn(width, ff, generator=g)})
    h = torch.randn(4, width, generator=g, dtype=F64)
    mlp = {"router": {"experts": experts, "top": 2}, "expert": {"limit": 1.5}}
    got = plain.routed_feed_forward(h, mlp, weights, "m")
    z = h @ weights["m.router"].double().T + weights["m.router.b"].double()
    for t in range(4):
        top = torch.topk(z[t], 2)
        share = torch.softmax(top.values, dim=0)
        want = sum(share[j] * plain.bounded_gated_unit(h[t:t + 1], weights, f"m.e{int(top.indices[j])}", 1.5)[0] for j in range(2))
        assert torch.allclose(got[t], want)
    everyone = plain.routed_feed_forward(h, dict(mlp, router={"experts": experts, "top": experts}), weights, "m")
    share = torch.softmax(z, dim=1)
    want = sum(share[:, e:e + 1] * plain.bounded_gated_unit(h, weights, f"m.e{e}", 1.5) for e in range(experts))
    assert torch.allclose(everyone, want)


def test_small_functions():
    z = torch.linspace(-4, 4, 9, dtype=F64)
    assert torch.allclose(plain.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))
    x = torch.tensor([[3.0, -4.0]], dtype=F64)
    assert torch.allclose(plain.root_mean_square_norm(x, 0.0), x / math.sqrt(12.5))
    w = {"u.gate": torch.tensor([[2.0]]), "u.up": torch.tensor([[-3.0]]), "u.down": torch.tensor([[1.0]])}
    one = torch.tensor([[1.0]], dtype=F64)
    assert torch.allclose(plain.bounded_gated_unit(one, w, "u", 1.5), torch.tensor([[1.5 / (1 + math.exp(-1.702 * 1.5)) * (-1.5 + 1)]], dtype=F64))


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_plain_model_runs_every_case_and_later_tokens_do_not_change_earlier_logits(name):
    raw = CASES[name]["raw"]
    tensors = make_tensors(raw, seed=4)
    g = torch.Generator().manual_seed(5)
    tokens = torch.randint(0, raw["vocab"], (50,), generator=g).tolist()
    whole = plain.forward(raw, tensors, tokens)
    assert whole.shape == (50, raw["vocab"]) and bool(torch.isfinite(whole).all())
    assert torch.allclose(plain.forward(raw, tensors, tokens[:31]), whole[:31], atol=1e-9)
