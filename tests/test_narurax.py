"""Narurax without a GPU: the configuration reader and its errors, the tensors it expects, the cache units
that the shifts and the embedding keep beside the mixers' own, kept first pages under a window, the
random-weights folder, and pins of the plain implementation (each mechanism against a second, independent
formulation)."""

from __future__ import annotations

import copy
import math

import pytest
import torch

from narurax_cases import CASES, SINGLE, make_tensors
from plain import narurax_plain as plain

F64 = torch.float64


# -- configuration and weights ---------------------------------------------------------

def test_config_is_found_by_its_architecture_key_and_states_the_layers_as_parts():
    from lockstep_amd.config import NaruraxConfig, config_from_dict

    cfg = config_from_dict(CASES["A"]["raw"])
    assert isinstance(cfg, NaruraxConfig)
    spec = cfg.model_spec()
    assert [layer.mixer.kind for layer in spec.layers] == ["gated_delta", "talking_attention", "sink_attention", "sink_attention"]
    assert all(layer.arrangement.kind == "prenorm_residual" and layer.arrangement["token_shift"] == "shift" for layer in spec.layers)
    first, second, third, fourth = (layer.mixer for layer in spec.layers)
    assert (first["num_heads"], first["num_kv_heads"], first["head_dim"], first["value_dim"], first["taps"]) == (4, 2, 24, 16, 3)
    assert (first["decay"], first["gate_act"], first["decay_rank"], first["gate_rank"], first["unit_eps"]) == ("channel", "sigmoid", -1, -1, 1e-6)
    assert (second["mix"], second["sink"], second["gate"], second["shared_kv"]) == ("weights", "learned", True, True)
    assert (second["window"], second["keep_first"], second["scale"]) == (21, 3, 0.3)
    assert second["position"].kind == "rope_scaled" and second["position"]["pairing"] == "neighbours"
    assert second["position"]["rotary_dim"] == 16 and second["position"]["scaling"] is None
    assert (third["sink"], third["bias"], third["out_bias"], third["head_norm"], third["head_norm_weights"]) == ("zero", True, True, 1e-5, True)
    assert (third["window"], third["keep_first"]) == (13, 5) and (fourth["window"], fourth["keep_first"]) == (50, 0)
    assert third["position"]["scaling"] == {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64.0}
    experts = spec.layers[0].feed_forward
    assert (experts["experts"], experts["top"], experts["limit"], experts["score"], experts["weigh"], experts["router_bias"]) == (
        6, 2, None, "sigmoid", "input", False)
    assert spec.layers[3].feed_forward is None
    pairs = spec.embedding["pairs"]
    assert (pairs["name"], pairs["buckets"], pairs["mul_prev"], pairs["mul_cur"]) == ("bigram", 61, 31, 5)
    # the mixers' units, then one unit a layer for what its shift keeps, then the embedding's
    assert [(e.layer, e.cache, e.state) for e in spec.schedule] == [(0, 0, 4), (1, 1, 5), (2, 2, 6), (3, 3, 7)]
    assert spec.embedding_state == 8 and spec.cache_units() == 9
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()


def test_the_expected_tensors():
    from lockstep_amd.config import config_from_dict
    from lockstep_amd.engine.model import collect_weight_specs

    names = {w.name: w for w in collect_weight_specs(config_from_dict(CASES["B"]["raw"]).model_spec())}
    assert names["bigram"].shape == (8, 96) and names["embed"].shape == (200, 96)
    assert names["l0.shift"].shape == (96,) and names["l0.shift"].kind == "vector"
    assert names["l0.mix.q.b"].shape == (120,) and names["l0.mix.o.b"].shape == (96,) and names["l0.mix.v"].shape == (72, 96)
    assert names["l0.mix.q.norm"].shape == (40,) and names["l0.mix.k.norm"].shape == (40,) and "l0.mix.sink" not in names
    assert "l0.mlp.router.b" not in names and names["l0.mlp.router"].shape == (3, 96) and names["l0.mlp.e2.down"].shape == (96, 48)
    assert names["l1.mix.a1"].shape == (-1, 96) and names["l1.mix.a2"].shape == (80, -1) and names["l1.mix.dt_bias"].shape == (80,)
    assert names["l1.mix.g1"].shape == (-1, 96) and names["l1.mix.g2"].shape == (48, -1) and names["l1.mix.A_log"].shape == (2,)
    assert names["l1.mix.q.conv"].shape == (80, 2) and "l1.mix.a" not in names and "l1.mix.g" not in names
    assert names["l1.norm2"].optional and "l1.mlp.router" not in names
    assert names["l2.mix.talk"].shape == (6, 6) and names["l2.mix.sink"].shape == (6,) and names["l2.mix.g"].shape == (72, 96)
    assert "l2.mix.v" not in names and "l2.mix.q.b" not in names and names["l2.mix.k"].shape == (12, 96)


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="delta"), "type"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"].update(vdim=16), "vdim"),
    (lambda c: c["layers"][1]["mixer"].pop("mask"), "mask"),
    (lambda c: c["layers"][2]["mixer"].update(heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"].pop("conv"), "conv"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "top"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "moe"),
    (lambda c: c["embedding"]["bigram"].pop("mul_prev"), "mul_prev"),
    (lambda c: c["embedding"]["bigram"].update(buckets=0), "buckets"),
    (lambda c: c["norm"].update(eps=0.0), "eps"),
    (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=18), "dims"),
    (lambda c: c["layers"][2]["mixer"]["mask"].update(keep_first=-1), "keep_first"),
])
def test_a_wrong_or_missing_key_is_named_when_the_configuration_is_read(change, message):
    from lockstep_amd.config import ConfigError, config_from_dict

    raw = copy.deepcopy(CASES["A"]["raw"])
    change(raw)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(raw)


def test_state_units_of_shifts_and_embedding_and_the_pages_a_window_keeps():
    """The cache manager gets a paged unit for each attention layer (with the kept first tokens declared), a state
    unit for the delta layer, one a layer for the shift's last row and one int for the embedding's last token."""
    from lockstep_amd.cache import CacheManager
    from lockstep_amd.config import config_from_dict
    from lockstep_amd.parts import PagedKVSpec, StateSpec, build_part, part_class

    spec = config_from_dict(CASES["A"]["raw"]).model_spec()
    units = [None] * spec.cache_units()
    for run in spec.schedule:
        layer = part_class(spec.layers[run.layer].arrangement.kind)(spec.layers[run.layer])
        units[run.cache] = layer.mixer.cache_spec()
        units[run.state] = layer.state_spec()
    units[spec.embedding_state] = build_part(spec.embedding).state_spec()
    assert isinstance(units[0], StateSpec) and units[0].shape == (4 * 24 * 16 + 2 * (2 * 2 * 24 + 4 * 16),)
    assert units[1] == PagedKVSpec(2, 24, 21, value_dim=24, keep_first=3)
    assert units[2] == PagedKVSpec(2, 16, 13, value_dim=40, keep_first=5) and units[3].keep_first == 0
    assert all(units[u] == StateSpec((64,), "float32") for u in range(4, 8)) and units[8] == StateSpec((1,), "int32")
    cache = CacheManager(units, page_size=8, num_pages=32, max_requests=2, max_tokens_per_request=256)
    cache.open("r")
    cache.reserve("r", 100)
    cache.commit("r", 100)
    by_window = {g.spec.window: cache.request_pages("r", g.index) for g in cache.groups}
    # the window of 13 with 5 kept tokens: the first page stays, then nothing up to the page of position 100 - 13 + 1
    assert [p >= 0 for p in by_window[13]] == [True] + [False] * 10 + [True, True]
    assert [p >= 0 for p in by_window[21]] == [True] + [False] * 9 + [True, True, True]
    assert all(p >= 0 for p in by_window[50][6:]) and all(p < 0 for p in by_window[50][:6])
    cache.audit()


def test_random_weights_folder_round_trip(tmp_path):
    from lockstep_amd.config import config_from_dict, config_from_dir
    from lockstep_amd.engine.model import collect_weight_specs
    from lockstep_amd.weights import load_weights, write_random_model

    cfg = config_from_dict(SINGLE["delta"]["raw"])
    folder = write_random_model(cfg, tmp_path / "m", seed=3)
    assert config_from_dir(folder).to_dict() == cfg.to_dict()
    weights = load_weights(folder, collect_weight_specs(cfg.model_spec()), {})
    assert weights.get("l0.mix.a1").shape == (16, 64) and weights.get("l0.mix.g2").shape == (64, 16)
    assert weights.get("bigram").shape == (62, 64) and weights.get("l0.shift").shape == (64,)


def test_a_checkpoint_decides_the_ranks_of_the_bottlenecks(tmp_path):
    from lockstep_amd.config import config_from_dict
    from lockstep_amd.engine.model import collect_weight_specs
    from lockstep_amd.weights import weights_from_dict

    case = CASES["A"]
    tensors = make_tensors(case["raw"], seed=1, ranks=case["ranks"])
    assert tensors["l0.mix.a1"].shape == (5, 64) and tensors["l0.mix.g2"].shape == (64, 12)
    weights = weights_from_dict(tensors, collect_weight_specs(config_from_dict(case["raw"]).model_spec()), {})
    assert weights.get("l0.mix.a2").shape == (96, 5)


# -- pins of the plain implementation -----------------------------------------------------

def test_pair_embedding_by_hand():
    table = torch.arange(12, dtype=F64).view(4, 3)
    pairs = torch.arange(100, 118, dtype=F64).view(6, 3)
    out = plain.pair_embedding(torch.tensor([2, 3, 0, 3]), table, pairs, 7, 2)
    rows = [5, (2 * 7 + 3 * 2) % 5, (3 * 7 + 0) % 5, (0 + 3 * 2) % 5]
    assert torch.equal(out, table[[2, 3, 0, 3]] + pairs[rows])


def test_the_shift_is_a_blend_with_the_row_before():
    n = torch.randn((5, 7), dtype=F64)
    assert torch.equal(plain.shift_towards_previous(n, torch.zeros(7, dtype=F64)), n)
    moved = plain.shift_towards_previous(n, torch.ones(7, dtype=F64))
    assert torch.allclose(moved[1:], n[:-1]) and float(moved[0].abs().max()) == 0.0
    half = plain.shift_towards_previous(n, torch.full((7,), 0.25, dtype=F64))
    assert torch.allclose(half[2], 0.75 * n[2] + 0.25 * n[1])


def test_rotation_of_neighbours_is_a_complex_product():
    x = torch.randn((6, 2, 10), dtype=F64)
    f = plain.frequencies(6, 50.0)
    out = plain.rotate_neighbours(x, torch.arange(6), f)
    z = torch.view_as_complex(x[..., :6].reshape(6, 2, 3, 2).contiguous())
    turned = z * torch.polar(torch.ones((6, 1, 3), dtype=F64), torch.arange(6, dtype=F64)[:, None, None] * f[None, None, :])
    assert torch.allclose(torch.view_as_real(turned).reshape(6, 2, 6), out[..., :6]) and torch.equal(out[..., 6:], x[..., 6:])


def test_stretched_frequencies_have_three_ranges():
    scaling = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
    plain_f = plain.frequencies(16, 100.0)
    got = plain.frequencies(16, 100.0, scaling)
    wavelength = 2 * math.pi / plain_f
    kinds = set()
    for i in range(8):
        if wavelength[i] < 16:
            kinds.add("kept")
            assert got[i] == plain_f[i]
        elif wavelength[i] > 64:
            kinds.add("divided")
            assert got[i] == plain_f[i] / 8
        else:
            kinds.add("between")
            assert plain_f[i] / 8 < got[i] < plain_f[i]
    assert kinds == {"kept", "divided", "between"}


def test_the_sink_is_a_key_with_a_zero_value_and_the_window_keeps_first_tokens():
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn((9, 4), generator=g, dtype=F64) for _ in range(3))
    seen = plain.visible(9, 3, 2)
    assert seen[8].tolist() == [True, True, False, False, False, False, True, True, True]
    w = plain.head_weights(q, k, 0.7, seen, 1.3)
    # the same with one more key whose score is the sink and whose value is zero
    scores = torch.cat([(q @ k.T * 0.7).masked_fill(~seen, -math.inf), torch.full((9, 1), 1.3, dtype=F64)], dim=1)
    full = torch.softmax(scores, dim=-1)
    assert torch.allclose(full[:, :9], w) and torch.allclose(w.sum(-1), 1 - full[:, 9])
    assert torch.allclose(w @ v, full @ torch.cat([v, torch.zeros((1, 4), dtype=F64)]))


def test_mixing_the_weights_is_mixing_the_heads_outputs_over_one_value_head():
    """With one key/value head, sum_g T[h, g] (P_g V) equals (sum_g T[h, g] P_g) V; the identity mixes nothing."""
    case = SINGLE["mixing"]
    raw = copy.deepcopy(case["raw"])
    raw["layers"][0]["mixer"]["kv_heads"] = 1
    tensors = make_tensors(raw, seed=2)
    model = plain.PlainNarurax(raw, tensors)
    m = raw["layers"][0]["mixer"]
    h = torch.randn((12, raw["width"]), dtype=F64)
    positions = torch.arange(12)
    mixed = model.attention(0, m, h, positions)
    q = (h @ model.t("l0.mix.q").T).view(12, 4, 24)
    k = (h @ model.t("l0.mix.k").T).view(12, 1, 24)
    f = plain.frequencies(16, 10000.0)
    qr, kr = plain.rotate_neighbours(q, positions, f), plain.rotate_neighbours(k, positions, f)
    seen = plain.visible(12, 20, 4)
    sink = model.t("l0.mix.sink")
    each = torch.stack([plain.head_weights(qr[:, a], kr[:, 0], 0.5, seen, sink[a]) @ k[:, 0] for a in range(4)], dim=1)
    want = torch.einsum("ab,tbe->tae", model.t("l0.mix.talk"), each).reshape(12, -1)
    gate = plain.sigmoid(h @ model.t("l0.mix.g").T)
    assert torch.allclose((want * gate) @ model.t("l0.mix.o").T, mixed, atol=1e-10)
    assert not torch.allclose((each.reshape(12, -1) * gate) @ model.t("l0.mix.o").T, mixed, atol=1e-3)


def test_the_delta_rule_retrieves_with_orthonormal_keys_and_forgets_by_channel():
    d, e = 4, 3
    keys = torch.eye(d, dtype=F64)
    values = torch.randn((d, e), dtype=F64)
    ones = torch.ones((d, d), dtype=F64)
    out = plain.delta_rule_with_channel_decay(keys, keys, values, torch.ones(d, dtype=F64), ones)
    assert torch.allclose(out, values)                      # each token reads what it has just written
    # one more token that writes nothing (beta 0) and decays channel 1 alone: key 1's value shrinks, the others stay
    q = torch.cat([keys, torch.ones((1, d), dtype=F64)])
    k = torch.cat([keys, keys[:1]])
    v = torch.cat([values, torch.zeros((1, e), dtype=F64)])
    g = torch.cat([ones, torch.tensor([[1.0, 0.25, 1.0, 1.0]], dtype=F64)])
    out = plain.delta_rule_with_channel_decay(q, k, v, torch.tensor([1.0] * d + [0.0], dtype=F64), g)
    assert torch.allclose(out[-1], values[0] + 0.25 * values[1] + values[2] + values[3])


def test_scored_experts_against_dense_products():
    g = torch.Generator().manual_seed(3)
    h = torch.randn((6, 5), generator=g, dtype=F64)
    router = torch.randn((4, 5), generator=g, dtype=F64)
    experts = [tuple(torch.randn(s, generator=g, dtype=F64) for s in ((7, 5), (7, 5), (5, 7))) for _ in range(4)]
    out = plain.scored_experts(h, router, experts, 4)        # all experts: no choice is made
    s = torch.sigmoid(h @ router.T)
    want = sum((torch.nn.functional.silu((s[:, e:e + 1] * h) @ gate.T) * ((s[:, e:e + 1] * h) @ up.T)) @ down.T
               for e, (gate, up, down) in enumerate(experts))
    assert torch.allclose(out, want)
    one = plain.scored_experts(h, router, experts, 1)
    best = s.argmax(-1)
    for t in range(6):
        gate, up, down = experts[int(best[t])]
        x = s[t, best[t]] * h[t]
        assert torch.allclose(one[t], down @ (torch.nn.functional.silu(gate @ x) * (up @ x)))
