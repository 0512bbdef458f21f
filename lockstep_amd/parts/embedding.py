"""Token embedding and output head."""

from __future__ import annotations

from ..config.base import PartSpec
from ..ops import STORE_F32
from .base import Part, StateSpec, WeightSpec, register_part


@register_part("token_embedding")
class TokenEmbedding(Part):
    """``h[t] = E[token[t]] * scale``; without ``scale`` no scaling (reference
    engine/model/qwen3.py:319).  Parameters: ``name``, ``vocab_size``, ``hidden_size``,
    ``scale`` (optional), ``copies`` (optional: the residual stream holds that many copies of a row,
    ``[T, copies * hidden_size]``, which all start as the embedding).

    ``pairs`` (optional, ``{"name", "buckets", "mul_prev", "mul_cur"}``): a second table ``[buckets + 1,
    hidden_size]`` is added, row ``(token before * mul_prev + token * mul_cur) mod buckets``, and its last
    row for a request's first token.  The token before a step's first one is kept per request (one int:
    the part then has a ``state_spec`` and the model names a cache unit for it)."""

    graph_safe = True
    state_unit = None       # the cache unit of the kept token, set by the model

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        self.table = self.pair_table = None
        self.scale = float(spec.params.get("scale", 1.0))
        self.copies = int(spec.params.get("copies") or 1)
        self.pairs = spec.params.get("pairs")
        if self.pairs is not None:
            if self.copies != 1:
                raise ValueError("an embedding with a table of pairs fills one copy of the stream")
            if int(self.pairs["buckets"]) <= 0:
                raise ValueError(f"the table of pairs needs a positive number of buckets, got {self.pairs['buckets']!r}")

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        out = [WeightSpec(spec["name"], (int(spec["vocab_size"]), int(spec["hidden_size"])))]
        pairs = spec.params.get("pairs")
        if pairs is not None:
            out.append(WeightSpec(pairs["name"], (int(pairs["buckets"]) + 1, int(spec["hidden_size"]))))
        return out

    def state_spec(self):
        return None if self.pairs is None else StateSpec((1,), "int32")

    def load(self, weights, rt) -> None:
        self.table = rt.matrix(weights.get(self.spec["name"]), share_key=weights.source_name(self.spec["name"]))
        if self.pairs is not None:
            self.pair_table = rt.matrix(weights.get(self.pairs["name"]))
            rt.kernels.mixers_lib()

    def forward(self, ctx, tokens, out) -> None:
        if self.pairs is None:
            ctx.rt.kernels.embed(tokens, self.table, out, self.scale, self.copies)
            return
        ctx.rt.kernels.embed_pair(tokens, ctx.tok_seq, ctx.tok_pos, ctx.seqs, self.table, self.pair_table,
                                  int(self.pairs["mul_prev"]), int(self.pairs["mul_cur"]),
                                  ctx.cache.unit_state(self.state_unit), out, self.scale)


@register_part("linear_head")
class LinearHead(Part):
    """``logits = x @ W^T`` in float32, no bias and no scaling (reference
    engine/model/qwen3.py:373); with ``softcap`` (optional, a positive number c) the
    logits are then bent into (-c, c): ``c * tanh(logits / c)``.  Parameters: ``name``,
    ``tied_to`` (a tensor name the head aliases when the checkpoint does not hold its
    own, or None), ``vocab_size``, ``hidden_size``, ``softcap``."""

    graph_safe = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        self.weight = None
        self.vocab = int(spec["vocab_size"])
        cap = spec.params.get("softcap")
        self.softcap = float(cap) if cap else None
        if self.softcap is not None and not self.softcap > 0:
            raise ValueError(f"the logits' soft cap must be positive, got {cap!r}")

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        return [WeightSpec(spec["name"], (int(spec["vocab_size"]), int(spec["hidden_size"])))]

    @classmethod
    def ties(cls, spec: PartSpec) -> dict[str, str]:
        return {spec["name"]: spec["tied_to"]} if spec.params.get("tied_to") else {}

    def load(self, weights, rt) -> None:
        self.weight = rt.matrix(weights.get(self.spec["name"]), share_key=weights.source_name(self.spec["name"]))

    def forward(self, ctx, x, logits) -> None:
        ctx.rt.kernels.gemm(x, self.weight, logits, STORE_F32)
        if self.softcap is not None:
            ctx.rt.kernels.softcap(logits, self.softcap)
