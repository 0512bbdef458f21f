"""Toripel: a decoder whose layers each name one of three mixers, over a residual stream of several
copies (hyper-connections), with a feed-forward of experts that a table assigns to token ids.

* ``attention``: grouped heads with biased projections, no position encoding, queries and keys
  divided by their root mean square a head, a sliding window, an ordinary softmax.
* ``latent_attention``: queries through a normalised latent; keys and values as projections of one
  cached latent plus one rotated key part shared by the heads (neighbouring pairs, frequencies
  stretched along a ramp); a sliding window; a learned sink a head in the softmax.  With ``kv_from``
  the layer reads the latent that another such layer caches.
* ``delta``: the gated delta rule with short convolutions in front of q, k and v.
* feed-forward: ``experts`` plain gated units of which a token uses the ``top`` that a table names
  for its id, each weighing 1/top; or none.

Norms are root-mean-square norms whose weight is stored around zero (the factor is 1 + w).

``config.json`` is nested: ``architecture``, ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``,
``streams`` (the copies of the residual stream; absent: one plain residual stream) and ``layers``, a
list whose entries give ``type``, the mixer's sizes and constants under ``mixer`` and the feed-forward
under ``mlp`` (null for a layer without one).  Layer ``i``'s tensors start with ``l<i>.``: ``norm1``,
``norm2``, ``mix.*``, ``mlp.*``, ``hc1.*``, ``hc2.*``; beside them ``embed``, ``final.norm`` and ``head``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

from .base import ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry
from .registry import register_architecture

#: inside the root that makes unit vectors of the delta rule's queries and keys; fixed by the design
UNIT_EPS = 1e-6


def _need(mapping, key: str, where: str):
    if not isinstance(mapping, dict) or key not in mapping:
        raise ConfigError(f"config.json: {where} lacks the key {key!r}")
    return mapping[key]


def _positive_int(value, what: str) -> int:
    if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
        raise ConfigError(f"{what} must be a positive integer, got {value!r}")
    return value


@register_architecture
@dataclass(frozen=True)
class ToripelConfig(ModelConfig):
    architecture: str
    vocab: int
    width: int
    norm: Any
    embedding: Any
    layers: Any
    streams: Any = None

    architecture_names = ("Toripel", "toripel")

    @classmethod
    def from_dict(cls, raw):
        if "streams" not in raw:
            raw = dict(raw, streams=None)
        return super().from_dict(raw)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": dict(self.norm),
               "embedding": dict(self.embedding), "layers": [dict(layer) for layer in self.layers]}
        if self.streams is not None:
            out["streams"] = self.streams
        return out

    def init_scheme(self):
        return {"std": 0.05, "norm_std": 0.1}

    def validate(self) -> None:
        _positive_int(self.vocab, "vocab")
        _positive_int(self.width, "width")
        if not float(_need(self.norm, "eps", "norm")) > 0:
            raise ConfigError("norm.eps must be positive")
        float(_need(self.embedding, "scale", "embedding"))
        if self.streams is not None:
            _positive_int(self.streams, "streams")
        if not isinstance(self.layers, (list, tuple)) or not self.layers:
            raise ConfigError("layers must be a non-empty list")
        for i, layer in enumerate(self.layers):
            kind = _need(layer, "type", f"layers[{i}]")
            if kind not in ("attention", "latent_attention", "delta"):
                raise ConfigError(f"layers[{i}].type {kind!r} is not one of attention, latent_attention, delta")
            _need(layer, "mixer", f"layers[{i}]")
            mlp = layer.get("mlp")
            if mlp is not None and _need(mlp, "kind", f"layers[{i}].mlp") != "moe":
                raise ConfigError(f"layers[{i}].mlp.kind {mlp['kind']!r} is not moe")
        self.model_spec()        # every key the layers need, now rather than at the first step

    # -- the mixers as parts ------------------------------------------------------------
    @staticmethod
    def _window(m, where: str):
        mask = m.get("mask")
        return _positive_int(_need(mask, "size", where + ".mask"), where + ".mask.size") if mask else None

    def _source(self, i: int) -> int:
        """The layer whose cache unit layer ``i`` (attention over a latent) uses: itself, or its ``kv_from``."""
        m = self.layers[i]["mixer"]
        source = m.get("kv_from")
        if source is None:
            return i
        where = f"layers[{i}].mixer.kv_from"
        if not isinstance(source, int) or isinstance(source, bool) or not 0 <= source < len(self.layers) or source == i:
            raise ConfigError(f"{where} {source!r} is not another layer")
        other = self.layers[source]
        if other.get("type") != "latent_attention" or other["mixer"].get("kv_from") is not None:
            raise ConfigError(f"{where}: layer {source} has no latent of its own")
        if source > i:
            raise ConfigError(f"{where}: layer {source} runs after layer {i}")
        for key in ("kv_rank", "rot_dim", "rot"):
            if other["mixer"].get(key) != m.get(key):
                raise ConfigError(f"{where}: layer {source} differs in {key}")
        return source

    def _mixer(self, i: int, layer) -> PartSpec:
        kind, m, where = layer["type"], layer["mixer"], f"layers[{i}].mixer"
        eps = float(self.norm["eps"])
        need = lambda key: _positive_int(_need(m, key, where), f"{where}.{key}")  # noqa: E731
        if kind == "delta":
            heads, kv_heads = need("heads"), need("kv_heads")
            if heads % kv_heads:
                raise ConfigError(f"{where}: {heads} heads are not a multiple of {kv_heads} kv_heads")
            return PartSpec("gated_delta", {
                "hidden_size": self.width, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": need("dim"),
                "value_dim": need("vdim"), "taps": need("conv"), "eps": eps, "unit_eps": UNIT_EPS})
        if kind == "attention":
            heads, kv_heads = need("heads"), need("kv_heads")
            if heads % kv_heads:
                raise ConfigError(f"{where}: {heads} heads are not a multiple of {kv_heads} kv_heads")
            return PartSpec("sink_attention", {
                "hidden_size": self.width, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": need("dim"),
                "value_dim": need("vdim"), "scale": float(_need(m, "scale", where)), "position": PartSpec("no_position", {}),
                "window": self._window(m, where), "sink": None, "bias": True, "head_norm": eps})
        rot_dim = need("rot_dim")
        rot = _need(m, "rot", where)
        dims = _positive_int(_need(rot, "dims", where + ".rot"), where + ".rot.dims")
        if dims % 2 or dims > rot_dim:
            raise ConfigError(f"{where}.rot.dims {dims} must be even and at most rot_dim {rot_dim}")
        scaling = rot.get("scaling")
        if scaling is not None:
            scaling = {key: float(_need(scaling, key, where + ".rot.scaling")) for key in ("factor", "original", "fast", "slow")}
        position = PartSpec("rope_ramped", {"rotary_dim": dims, "theta": float(_need(rot, "base", where + ".rot")),
                                            "pairing": "neighbours", "scaling": scaling})
        source = self._source(i)
        # the cache unit keeps what the widest window among its readers needs
        windows = [self._window(self.layers[j]["mixer"], f"layers[{j}].mixer")
                   for j in range(len(self.layers))
                   if self.layers[j].get("type") == "latent_attention" and (j == source or self.layers[j]["mixer"].get("kv_from") == source)]
        return PartSpec("latent_attention", {
            "hidden_size": self.width, "num_heads": need("heads"), "head_dim": need("dim"), "rot_dim": rot_dim,
            "value_dim": need("vdim"), "q_rank": need("q_rank"), "kv_rank": need("kv_rank"), "eps": eps,
            "position": position, "scale": float(_need(m, "scale", where)), "window": self._window(m, where),
            "sink": "learned", "reads_other": source != i,
            "cache_window": None if any(w is None for w in windows) else max(windows)})

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
            "experts": experts, "top": top, "limit": None, "alpha": 1.0, "shared": None, "router": "table",
            "vocab_size": self.vocab})

    def model_spec(self) -> ModelSpec:
        width, eps = self.width, float(self.norm["eps"])
        names = {"mixer_prefix": "mix", "feed_forward_prefix": "mlp", "mixer_norm_name": "norm1",
                 "feed_forward_norm_name": "norm2"}
        copies = 1
        if self.streams is None:
            arrangement = PartSpec("prenorm_residual", names)
        else:
            copies = int(self.streams)
            arrangement = PartSpec("hyper_connections", dict(names, copies=copies, mixer_streams_prefix="hc1",
                                                             feed_forward_streams_prefix="hc2"))
        norm = lambda name, **more: PartSpec("rmsnorm", dict(size=width, eps=eps, name=name, offset=1.0, **more))  # noqa: E731
        layers, schedule = [], []
        for i, layer in enumerate(self.layers):
            mlp = layer.get("mlp")
            layers.append(LayerSpec(
                prefix=f"l{i}", arrangement=arrangement, mixer=self._mixer(i, layer),
                feed_forward=None if mlp is None else self._feed_forward(i, mlp),
                mixer_norm=norm(f"l{i}.norm1"), feed_forward_norm=norm(f"l{i}.norm2", optional=mlp is None)))
            source = self._source(i) if layer["type"] == "latent_attention" else i
            schedule.append(ScheduleEntry(layer=i, cache=source, writes_cache=source == i))
        return ModelSpec(
            hidden_size=width, vocab_size=self.vocab,
            embedding=PartSpec("token_embedding", {"name": "embed", "vocab_size": self.vocab, "hidden_size": width,
                                                   "scale": float(self.embedding["scale"]), "copies": copies}),
            layers=tuple(layers), schedule=tuple(schedule),
            final_norm=PartSpec("rmsnorm", {"size": width, "eps": eps, "name": "final.norm", "offset": 1.0, "copies": copies}),
            head=PartSpec("linear_head", {"name": "head", "tied_to": None, "vocab_size": self.vocab, "hidden_size": width}),
            max_positions=None, residual_copies=copies)
