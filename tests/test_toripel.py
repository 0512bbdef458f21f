"""Toripel without a GPU: the configuration reader, the tensors it expects, the cache units of layers
that share a latent, the random-weights folder, the ramped rotation tables, and pins of the plain
implementation (each mechanism against a second, independent formulation)."""

from __future__ import annotations

import copy
import json
import math

import pytest
import torch

from plain import toripel_plain as plain
from toripel_cases import CASES, SINGLE, make_tensors

F64 = torch.float64


# -- configuration and weights ---------------------------------------------------------

def test_config_is_found_by_its_architecture_key_and_states_the_layers_as_parts():
    from lockstep_amd.config import ToripelConfig, config_from_dict

    cfg = config_from_dict(CASES["A"]["raw"])
    assert isinstance(cfg, ToripelConfig)
    spec = cfg.model_spec()
    assert [layer.mixer.kind for layer in spec.layers] == ["gated_delta", "sink_attention", "latent_attention", "latent_attention"]
    assert all(layer.arrangement.kind == "hyper_connections" and layer.arrangement["copies"] == 3 for layer in spec.layers)
    assert spec.residual_copies == 3 and spec.embedding["copies"] == 3 and spec.embedding["scale"] == 4.0
    assert spec.final_norm["copies"] == 3 and spec.final_norm["offset"] == 1.0
    first, second, third, fourth = (layer.mixer for layer in spec.layers)
    assert (first["num_heads"], first["num_kv_heads"], first["head_dim"], first["value_dim"], first["taps"]) == (4, 2, 24, 16, 3)
    assert (second["window"], second["sink"], second["bias"], second["head_norm"], second["scale"]) == (21, None, True, 1e-5, 0.7)
    assert second["position"].kind == "no_position"
    assert third["position"].kind == "rope_ramped" and third["position"]["pairing"] == "neighbours"
    assert third["position"]["scaling"] == {"factor": 8.0, "original": 64.0, "fast": 4.0, "slow": 1.0}
    assert (third["q_rank"], third["kv_rank"], third["rot_dim"], third["window"], third["sink"]) == (40, 32, 8, 37, "learned")
    # the fourth layer reads the third's latent: the unit keeps what the wider of the two windows needs
    assert not third["reads_other"] and fourth["reads_other"] and third["cache_window"] == fourth["cache_window"] == 50
    assert [(e.layer, e.cache, e.writes_cache) for e in spec.schedule] == [(0, 0, True), (1, 1, True), (2, 2, True), (3, 2, False)]
    experts = spec.layers[0].feed_forward
    assert (experts["experts"], experts["top"], experts["limit"], experts["router"], experts["vocab_size"]) == (6, 2, None, "table", 128)
    assert spec.layers[3].feed_forward is None
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()


def test_one_copy_no_copies_and_the_expected_tensors():
    from lockstep_amd.config import config_from_dict
    from lockstep_amd.engine.model import collect_weight_specs

    spec = config_from_dict(CASES["B"]["raw"]).model_spec()
    assert spec.residual_copies == 1 and spec.layers[0].arrangement.kind == "hyper_connections"
    names = {w.name: w for w in collect_weight_specs(spec)}
    assert names["l0.hc1.mix"].shape == (1, 1) and names["l2.hc2.in"].optional and names["l2.norm2"].optional
    assert names["l0.mix.dkv"].shape == (36 + 12, 96) and names["l0.mix.uq"].shape == (6 * 32, 24)
    assert names["l0.mix.uk"].shape == (6 * 20, 36) and names["l0.mix.uv"].shape == (6 * 10, 36) and names["l0.mix.sink"].shape == (6,)
    assert names["l0.mlp.table"].shape == (200, 3) and names["l0.mlp.table"].kind == "int" and "l0.mlp.router" not in names
    assert names["l1.mix.q.b"].shape == (120,) and names["l2.mix.q.conv"].shape == (80, 2) and names["l2.mix.A_log"].shape == (2,)
    plain_stream = config_from_dict(CASES["C"]["raw"]).model_spec()
    assert plain_stream.residual_copies == 1 and plain_stream.layers[0].arrangement.kind == "prenorm_residual"
    assert not any(".hc" in w.name for w in collect_weight_specs(plain_stream))
    spec = config_from_dict(CASES["A"]["raw"]).model_spec()
    names = {w.name for w in collect_weight_specs(spec)}
    assert "l3.mix.dkv" not in names and "l3.mix.dkv.norm" not in names and "l3.mix.uk" in names and "l2.mix.dkv" in names


@pytest.mark.parametrize("breakage, message", [
    (lambda raw: raw["layers"][0].update(type="mamba"), "not one of"),
    (lambda raw: raw["layers"][1]["mixer"].pop("kv_heads"), "kv_heads"),
    (lambda raw: raw["layers"][2]["mixer"]["rot"].update(dims=7), "even"),
    (lambda raw: raw["layers"][0]["mlp"].update(kind="dense"), "not moe"),
    (lambda raw: raw.pop("width"), "width"),
    (lambda raw: raw["layers"][0]["mlp"]["router"].update(top=9), "exceeds"),
    (lambda raw: raw["layers"][2]["mixer"]["rot"]["scaling"].pop("fast"), "fast"),
    (lambda raw: raw["layers"][3]["mixer"].update(kv_from=1), "no latent of its own"),
    (lambda raw: raw["layers"][3]["mixer"].update(kv_rank=16), "differs in kv_rank"),
    (lambda raw: raw["layers"][0]["mixer"].update(heads=3), "multiple"),
    (lambda raw: raw.update(streams=0), "streams"),
    (lambda raw: raw.pop("embedding"), "embedding"),
])
def test_config_errors_name_what_is_wrong(breakage, message):
    from lockstep_amd.config import ConfigError, config_from_dict

    raw = copy.deepcopy(CASES["A"]["raw"])
    breakage(raw)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(raw)


def test_random_weights_folder_and_cache_units(tmp_path):
    """The seeded folder loads through the package's reader with the expected dtypes (a table of different
    experts a row); the cache manager gives the layers that share a latent one unit with the wider window, and
    the delta layer a state of its matrices and its convolutions' last inputs."""
    from lockstep_amd.cache import CacheManager
    from lockstep_amd.config import config_from_dict
    from lockstep_amd.parts import PagedKVSpec, StateSpec, build_part
    from lockstep_amd.weights import write_random_model
    from lockstep_amd.weights.safetensors_io import open_model_tensors

    cfg = config_from_dict(CASES["A"]["raw"])
    write_random_model(cfg, tmp_path, seed=3)
    assert json.loads((tmp_path / "config.json").read_text())["streams"] == 3
    tensors = {name: handle.get(key) for name, (handle, key) in open_model_tensors(tmp_path).items()}
    table = tensors["l0.mlp.table"]
    assert table.dtype == torch.int32 and table.shape == (128, 2) and int(table.min()) >= 0 and int(table.max()) < 6
    assert bool((table[:, 0] != table[:, 1]).all()) and tensors["l0.norm1"].dtype == torch.bfloat16
    assert float(tensors["l0.norm1"].float().abs().mean()) < 0.5          # (stored around zero)
    spec = cfg.model_spec()
    units = [None] * spec.cache_units()
    for run in spec.schedule:
        if run.writes_cache:
            units[run.cache] = build_part(spec.layers[run.layer].mixer, "x").cache_spec()
    assert units[0] == StateSpec((4 * 24 * 16 + 2 * (2 * 2 * 24 + 4 * 16),), "float32")
    assert units[1] == PagedKVSpec(2, 24, 21, value_dim=40)
    assert units[2] == PagedKVSpec(1, 40, 50, value_dim=32) and len(units) == 3
    cache = CacheManager(units, page_size=8, num_pages=16, max_requests=2, max_tokens_per_request=128)
    cache.open("r")
    cache.reserve("r", 100)
    cache.commit("r", 100)
    # positions 0 .. 49 are beyond the latent unit's window of 50 for the next query at 100: pages 0 .. 5 are back
    latent_group = cache.unit_group(2)
    held = list(cache.request_pages("r", latent_group.index))
    assert latent_group.spec.window == 50 and all(p < 0 for p in held[:6]) and all(p >= 0 for p in held[6:13])


def test_ramped_frequencies_against_values_by_hand():
    from lockstep_amd.config.base import PartSpec
    from lockstep_amd.parts import build_part

    part = build_part(PartSpec("rope_ramped", {"rotary_dim": 8, "theta": 100.0, "pairing": "neighbours",
                                               "scaling": {"factor": 8.0, "original": 64, "fast": 4.0, "slow": 1.0}}))
    # pair index at which a rotation makes t turns in 64 positions: 8 ln(64 / (2 pi t)) / (2 ln 100)
    lo = math.floor(8 * math.log(64 / (2 * math.pi * 4.0)) / (2 * math.log(100.0)))
    hi = math.ceil(8 * math.log(64 / (2 * math.pi * 1.0)) / (2 * math.log(100.0)))
    assert (lo, hi) == (0, 3)
    want = []
    for i in range(4):
        f = 100.0 ** (-2 * i / 8)
        r = min(1.0, max(0.0, (i - lo) / (hi - lo)))
        want.append(f / 8.0 * r + f * (1 - r))
    assert torch.allclose(part.frequencies(), torch.tensor(want, dtype=F64), rtol=1e-14)
    mine, magnitude = plain.stretched_frequencies(8, 100.0, {"factor": 8.0, "original": 64, "fast": 4.0, "slow": 1.0})
    assert torch.allclose(mine, part.frequencies(), rtol=1e-14) and magnitude == pytest.approx(0.1 * math.log(8.0) + 1.0)
    cos, sin = part.tables(torch.arange(5))
    assert torch.allclose(cos[3].double(), torch.cos(3 * mine) * magnitude, atol=1e-7)
    assert torch.allclose(sin[4].double(), torch.sin(4 * mine) * magnitude, atol=1e-7)
    unscaled = build_part(PartSpec("rope_ramped", {"rotary_dim": 8, "theta": 100.0, "pairing": "neighbours", "scaling": None}))
    assert torch.allclose(unscaled.frequencies(), torch.tensor([100.0 ** (-2 * i / 8) for i in range(4)], dtype=F64))
    assert unscaled.magnitude() == 1.0 and unscaled.share_key() != part.share_key()


# -- the plain implementation against second formulations --------------------------------

def test_plain_rotation_is_a_turn_of_every_pair_by_its_angle():
    g = torch.Generator().manual_seed(1)
    x = torch.randn((6, 3, 10), generator=g, dtype=F64)
    f = torch.tensor([1.0, 0.3, 0.01], dtype=F64)
    positions = torch.tensor([0, 1, 2, 7, 30, 31])
    out = plain.rotate_pairs(x, positions, f, magnitude=1.25)
    z = torch.view_as_complex(x[..., :6].reshape(6, 3, 3, 2).contiguous())
    turned = z * torch.polar(torch.full((6, 3), 1.25, dtype=F64), positions[:, None].double() * f[None, :])[:, None, :]
    assert torch.allclose(out[..., :6], torch.view_as_real(turned).reshape(6, 3, 6), atol=1e-12)
    assert torch.equal(out[..., 6:], x[..., 6:])


def test_plain_sink_is_a_key_with_a_zero_value_and_windows_count_the_query_itself():
    g = torch.Generator().manual_seed(2)
    n, heads, d, dv = 9, 2, 4, 3
    q, k, v = (torch.randn((n, h, s), generator=g, dtype=F64) for h, s in ((heads, d), (1, d), (1, dv)))
    sink = torch.tensor([0.3, -1.0], dtype=F64)
    visible = plain.in_window(n, 4)
    assert visible[5].tolist() == [False, False, True, True, True, True, False, False, False]
    got = plain.softmax_attention(q, k, v, 0.5, visible, sink)
    for h in range(heads):
        for i in range(n):
            seen = [j for j in range(n) if visible[i, j]]
            scores = torch.stack([q[i, h] @ k[j, 0] * 0.5 for j in seen] + [sink[h]])
            weights = torch.softmax(scores, dim=0)
            want = sum(weights[a] * v[j, 0] for a, j in enumerate(seen))         # the sink's share goes nowhere
            assert torch.allclose(got[i, h], want, atol=1e-12)
    assert plain.in_window(5, None).sum() == 15


def test_plain_convolution_against_the_library_and_the_delta_rule_against_retrieval():
    g = torch.Generator().manual_seed(3)
    x, taps = torch.randn((11, 5), generator=g, dtype=F64), torch.randn((5, 4), generator=g, dtype=F64)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(x.T[None], (3, 0)), taps[:, None, :], groups=5)[0].T
    assert torch.allclose(plain.short_convolution(x, taps), want, atol=1e-12)
    # orthonormal keys, no decay, full step size: the state stores every value under its key, a repeated key
    # replaces its value, and a query that is a key reads the value back
    keys = torch.linalg.qr(torch.randn((6, 6), generator=g, dtype=F64))[0]
    order = [0, 1, 2, 1, 3]
    k = keys[order][:, None, :]
    v = torch.randn((5, 1, 4), generator=g, dtype=F64)
    ones = torch.ones((5, 1), dtype=F64)
    out = plain.gated_delta_rule(k, k, v, ones, ones)
    assert torch.allclose(out, v, atol=1e-12)                      # the read-out sees the current token's write
    probe = plain.gated_delta_rule(torch.cat([k, keys[1][None, None]]), torch.cat([k, keys[5][None, None]]),
                                   torch.cat([v, torch.zeros((1, 1, 4), dtype=F64)]), torch.ones((6, 1), dtype=F64),
                                   torch.ones((6, 1), dtype=F64))
    assert torch.allclose(probe[5, 0], v[3, 0], atol=1e-12)        # key 1 holds its second value
    # with a decay g and a step size of zero the state only fades: o_t = g^(t - s) (S_s^T q)
    fade = plain.gated_delta_rule(k[:1].repeat(4, 1, 1), k[:1].repeat(4, 1, 1), v[:1].repeat(4, 1, 1),
                                  torch.tensor([[1.0], [0.0], [0.0], [0.0]], dtype=F64), torch.full((4, 1), 0.5, dtype=F64))
    assert torch.allclose(fade[3, 0], v[0, 0] * 0.125, atol=1e-12)


def test_plain_streams_of_one_copy_are_the_residual_sum_and_the_table_picks_the_experts():
    g = torch.Generator().manual_seed(4)
    x, y = torch.randn((5, 1, 7), generator=g, dtype=F64), torch.randn((5, 7), generator=g, dtype=F64)
    one = torch.ones(1, dtype=F64)
    assert torch.equal(plain.read_streams(x, one), x[:, 0])
    assert torch.allclose(plain.write_streams(x, y, one.view(1, 1), one)[:, 0], x[:, 0] + y)
    X = torch.randn((2, 3, 4), generator=g, dtype=F64)
    mix = torch.randn((3, 3), generator=g, dtype=F64)
    out = plain.write_streams(X, torch.zeros((2, 4), dtype=F64), mix, torch.zeros(3, dtype=F64))
    assert torch.allclose(out[1, 2], sum(mix[s, 2] * X[1, s] for s in range(3)))         # indexed [from, to]
    h = torch.randn((4, 6), generator=g, dtype=F64)
    experts = [tuple(torch.randn(s, generator=g, dtype=F64) for s in ((5, 6), (5, 6), (6, 5))) for _ in range(3)]
    table = torch.tensor([[0, 1], [2, 0], [1, 2]])
    got = plain.tabled_experts(h, torch.tensor([2, 0, 0, 1]), table, experts)
    one_expert = lambda e, t: experts[e][2] @ (plain.silu(experts[e][0] @ h[t]) * (experts[e][1] @ h[t]))  # noqa: E731
    assert torch.allclose(got[0], (one_expert(1, 0) + one_expert(2, 0)) / 2, atol=1e-12)
    assert torch.allclose(got[3], (one_expert(2, 3) + one_expert(0, 3)) / 2, atol=1e-12)


def test_plain_latent_attention_in_the_latents_space_equals_keys_and_values_a_head():
    """What the engine computes (queries multiplied into the latent's space, one shared key/value head, the heads'
    outputs multiplied out afterwards) against the plain model's keys and values a head."""
    raw = SINGLE["latent"]["raw"]
    tensors = make_tensors(raw, seed=5)
    model = plain.PlainToripel(raw, tensors)
    m = raw["layers"][0]["mixer"]
    g = torch.Generator().manual_seed(6)
    n = 40
    h = torch.randn((n, raw["width"]), generator=g, dtype=F64)
    positions = torch.arange(n)
    want = model.latent_attention(0, m, h, positions, {})
    heads, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    c, shared = model.latent(0, m, h, positions)
    f, magnitude = plain.stretched_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    a = plain.rms(h @ model.t("l0.mix.dq").T, model.eps) * model.t("l0.mix.dq.norm")
    q = (a @ model.t("l0.mix.uq").T).reshape(n, heads, d + r)
    uk, uv = model.t("l0.mix.uk").reshape(heads, d, rank), model.t("l0.mix.uv").reshape(heads, dv, rank)
    moved = torch.einsum("thd,hdc->thc", q[:, :, :d], uk)
    q_all = torch.cat([moved, plain.rotate_pairs(q[:, :, d:], positions, f, magnitude)], dim=-1)
    keys = torch.cat([c, shared], dim=-1)[:, None, :]
    mixed = plain.softmax_attention(q_all, keys, c[:, None, :], float(m["scale"]), plain.in_window(n, m["mask"]["size"]),
                                    sink=model.t("l0.mix.sink"))
    out = torch.einsum("thc,hvc->thv", mixed, uv).reshape(n, heads * dv) @ model.t("l0.mix.o").T
    assert torch.allclose(out, want, atol=1e-10)


def test_plain_model_prefix_property_and_generation():
    """Logits at a position depend on earlier tokens only (every mechanism is causal), and greedy generation
    feeds its own tokens back."""
    raw = CASES["A"]["raw"]
    model = plain.PlainToripel(raw, make_tensors(raw, seed=7))
    tokens = [5, 17, 3, 100, 41, 9, 77, 2, 2, 64, 31, 8]
    whole = model.forward(tokens)
    assert torch.allclose(model.forward(tokens[:7]), whole[:7], atol=1e-10)
    new = model.generate_greedy(tokens[:5], 3)
    assert new[0] == int(torch.argmax(model.forward(tokens[:5])[-1])) and len(new) == 3
