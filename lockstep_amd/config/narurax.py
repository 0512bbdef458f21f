"""Narurax: a decoder whose layers each name one of three mixers, with an embedding that also looks at
the token before, an input to every mixer that is shifted towards the token before, and routed experts
as the feed-forward.

* embedding: ``embed[token]`` plus a row of a second table chosen by a hash of (token before, token),
  ``(prev * mul_prev + cur * mul_cur) mod buckets``; a request's first token takes the table's last row.
* a layer: ``x += mixer(shift(norm1(x)))``, then ``x += ff(norm2(x))``; ``shift`` moves every element
  of the normed row towards the same element of the token before by a learned share (``l<i>.shift``).
* ``attention``: grouped heads, no biases, unrotated keys that double as the values (there is no value
  projection), rotation of neighbouring pairs, a sliding window that keeps the first tokens, a
  learned sink a head in the softmax, the heads' weights mixed after the softmax, a sigmoid gate on
  the heads' outputs.
* ``attention_2``: biased projections, a root-mean-square norm a head on queries and keys with one
  weight vector for all heads, rotation of neighbouring pairs with frequencies stretched by wavelength,
  the same kind of window, a softmax with a one in its denominator.
* ``channel_delta``: the gated delta rule with a decay for every head and key channel (through a
  bottleneck), short convolutions in front of q, k and v, a per-head norm with a sigmoid gate (through
  a bottleneck) behind.
* feed-forward ``moe``: a router's sigmoid scores pick ``top`` of ``experts`` plain gated units (SiLU);
  a chosen expert's score multiplies what the expert reads.

``config.json`` is nested: ``architecture`` (the name), ``vocab``, ``width``, ``norm.eps``,
``embedding.bigram`` (``buckets``, ``mul_prev``, ``mul_cur``) and ``layers``, a list whose entries give
``type``, the mixer's sizes and constants under ``mixer`` and the feed-forward under ``mlp`` (null for a
layer without one).  Layer ``i``'s tensors start with ``l<i>.``: ``norm1``, ``norm2``, ``shift``,
``mix.*``, ``mlp.*``; beside them ``embed``, ``bigram``, ``final.norm`` and ``head``.  The ranks of the
bottlenecks are the checkpoint's (the shapes of ``mix.a1`` and ``mix.g1``).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

from .base import ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry
from .registry import register_architecture

#: inside the root that makes the delta rule's queries and keys unit vectors; fixed by the design
UNIT_EPS = 1e-6
MIXERS = ("attention", "attention_2", "channel_delta")


def _need(mapping, key: str, where: str):
    if not isinstance(mapping, dict) or key not in mapping:
        raise ConfigError(f"config.json: {where} lacks the key {key!r}")
    return mapping[key]


def _positive_int(value, what: str) -> int:
    if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
        raise ConfigError(f"{what} must be a positive integer, got {value!r}")
    return value


def _count(value, what: str) -> int:
    if not isinstance(value, int) or isinstance(value, bool) or value < 0:
        raise ConfigError(f"{what} must be an integer that is not negative, got {value!r}")
    return value


@register_architecture
@dataclass(frozen=True)
class NaruraxConfig(ModelConfig):
    architecture: str
    vocab: int
    width: int
    norm: Any
    embedding: Any
    layers: Any

    architecture_names = ("Narurax", "narurax")

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "norm": dict(self.norm), "embedding": {k: dict(v) if isinstance(v, dict) else v for k, v in self.embedding.items()},
                "layers": [dict(layer) for layer in self.layers]}

    def init_scheme(self):
        return {"std": 0.05, "norm_std": 0.1}

    def validate(self) -> None:
        _positive_int(self.vocab, "vocab")
        _positive_int(self.width, "width")
        if not float(_need(self.norm, "eps", "norm")) > 0:
            raise ConfigError("norm.eps must be positive")
        pairs = _need(self.embedding, "bigram", "embedding")
        _positive_int(_need(pairs, "buckets", "embedding.bigram"), "embedding.bigram.buckets")
        for key in ("mul_prev", "mul_cur"):
            _count(_need(pairs, key, "embedding.bigram"), f"embedding.bigram.{key}")
        if not isinstance(self.layers, (list, tuple)) or not self.layers:
            raise ConfigError("layers must be a non-empty list")
        for i, layer in enumerate(self.layers):
            kind = _need(layer, "type", f"layers[{i}]")
            if kind not in MIXERS:
                raise ConfigError(f"layers[{i}].type {kind!r} is not one of {', '.join(MIXERS)}")
            _need(layer, "mixer", f"layers[{i}]")
            mlp = layer.get("mlp")
            if mlp is not None and _need(mlp, "kind", f"layers[{i}].mlp") != "moe":
                raise ConfigError(f"layers[{i}].mlp.kind {mlp['kind']!r} is not moe")
        self.model_spec()        # every key the layers need, now rather than at the first step

    # -- the mixers as parts ------------------------------------------------------------
    def _rotation(self, m, where: str) -> PartSpec:
        rot = m.get("rot")
        if rot is None or not rot.get("dims"):
            return PartSpec("no_position", {})
        dims = _positive_int(_need(rot, "dims", where + ".rot"), where + ".rot.dims")
        if dims % 2 or dims > int(m["dim"]):
            raise ConfigError(f"{where}.rot.dims {dims} must be even and at most dim {m['dim']}")
        scaling = rot.get("scaling")
        if scaling is not None:
            scaling = {key: float(_need(scaling, key, where + ".rot.scaling")) for key in ("factor", "low", "high", "original")}
        return PartSpec("rope_scaled", {"rotary_dim": dims, "theta": float(_need(rot, "base", where + ".rot")),
                                        "pairing": "neighbours", "scaling": scaling})

    def _heads(self, m, where: str) -> dict:
        sizes = {"hidden_size": self.width,
                 "num_heads": _positive_int(_need(m, "heads", where), where + ".heads"),
                 "num_kv_heads": _positive_int(_need(m, "kv_heads", where), where + ".kv_heads"),
                 "head_dim": _positive_int(_need(m, "dim", where), where + ".dim"),
                 "value_dim": _positive_int(_need(m, "vdim", where), where + ".vdim")}
        if sizes["num_heads"] % sizes["num_kv_heads"]:
            raise ConfigError(f"{where}: {sizes['num_heads']} heads are not a multiple of {sizes['num_kv_heads']} kv_heads")
        return sizes

    def _mixer(self, i: int, layer) -> PartSpec:
        kind, m, where = layer["type"], layer["mixer"], f"layers[{i}].mixer"
        sizes = self._heads(m, where)
        eps = float(self.norm["eps"])
        if kind == "channel_delta":
            return PartSpec("gated_delta", dict(
                sizes, taps=_positive_int(_need(m, "conv", where), where + ".conv"), eps=eps, unit_eps=UNIT_EPS,
                decay="channel", decay_rank=-1, gate_rank=-1, gate_act="sigmoid"))
        mask = _need(m, "mask", where)
        window = _positive_int(_need(mask, "size", where + ".mask"), where + ".mask.size")
        keep_first = _count(mask.get("keep_first", 0), where + ".mask.keep_first")
        common = dict(sizes, position=self._rotation(m, where), scale=float(_need(m, "scale", where)),
                      window=window, keep_first=keep_first)
        if kind == "attention":
            if sizes["value_dim"] != sizes["head_dim"]:
                raise ConfigError(f"{where}: the values are the keys, so vdim {sizes['value_dim']} must equal dim {sizes['head_dim']}")
            return PartSpec("talking_attention", dict(common, mix="weights", sink="learned", gate=True, shared_kv=True))
        return PartSpec("sink_attention", dict(common, sink="zero", bias=True, out_bias=True, head_norm=eps,
                                               head_norm_weights=True))

    def _feed_forward(self, i: int, mlp) -> PartSpec:
        where = f"layers[{i}].mlp"
        router, expert = _need(mlp, "router", where), _need(mlp, "expert", where)
        experts = _positive_int(_need(router, "experts", where + ".router"), where + ".router.experts")
        top = _positive_int(_need(router, "top", where + ".router"), where + ".router.top")
        if top > experts:
            raise ConfigError(f"{where}.router.top {top} exceeds its {experts} experts")
        return PartSpec("routed_experts", {
            "hidden_size": self.width,
            "intermediate_size": _positive_int(_need(expert, "ff", where + ".expert"), where + ".expert.ff"),
            "experts": experts, "top": top, "limit": None, "alpha": 1.0, "shared": None,
            "score": "sigmoid", "weigh": "input", "router_bias": False})

    def model_spec(self) -> ModelSpec:
        width, eps = self.width, float(self.norm["eps"])
        arrangement = PartSpec("prenorm_residual", {"mixer_prefix": "mix", "feed_forward_prefix": "mlp",
                                                    "mixer_norm_name": "norm1", "feed_forward_norm_name": "norm2",
                                                    "token_shift": "shift"})
        layers = []
        for i, layer in enumerate(self.layers):
            mlp = layer.get("mlp")
            layers.append(LayerSpec(
                prefix=f"l{i}", arrangement=arrangement, mixer=self._mixer(i, layer),
                feed_forward=None if mlp is None else self._feed_forward(i, mlp),
                mixer_norm=PartSpec("rmsnorm", {"size": width, "eps": eps, "name": f"l{i}.norm1"}),
                feed_forward_norm=PartSpec("rmsnorm", {"size": width, "eps": eps, "name": f"l{i}.norm2",
                                                       "optional": mlp is None})))
        pairs = self.embedding["bigram"]
        n = len(layers)
        # cache units: layer i's mixer in unit i, what its shift keeps in unit n + i, the embedding's token in unit 2 n
        return ModelSpec(
            hidden_size=width, vocab_size=self.vocab,
            embedding=PartSpec("token_embedding", {
                "name": "embed", "vocab_size": self.vocab, "hidden_size": width,
                "pairs": {"name": "bigram", "buckets": int(pairs["buckets"]), "mul_prev": int(pairs["mul_prev"]),
                          "mul_cur": int(pairs["mul_cur"])}}),
            layers=tuple(layers),
            schedule=tuple(ScheduleEntry(layer=i, cache=i, state=n + i) for i in range(n)),
            final_norm=PartSpec("rmsnorm", {"size": width, "eps": eps, "name": "final.norm"}),
            head=PartSpec("linear_head", {"name": "head", "tied_to": None, "vocab_size": self.vocab, "hidden_size": width}),
            max_positions=None, embedding_state=2 * n)
