"""A feed-forward of many small experts of which each token uses a few, with an optional expert
that every token uses.

    z[t]      = router(x[t]) + router bias                       (float32)
    chosen(t) = the ``top`` experts with the largest z[t], largest first (the lower index wins a tie)
    w[t, k]   = softmax over the chosen logits alone
    out[t]    = sum_k w[t, k] * expert_chosen(t)[k](x[t])  +  shared(x[t])

With ``score = "sigmoid"`` a chosen expert weighs ``sigmoid(z)`` of its own logit instead, and a token's weights need not add up to one
(the experts with the largest scores are those with the largest logits).  With ``weigh = "input"`` a weight
multiplies what its expert reads and not what it returns: ``out[t] = sum_k expert_chosen(t)[k](w[t, k] x[t])``.

With ``router = "table"`` there is no router: row ``token id`` of an integer table ``[vocab, top]`` names
the token's experts (the entries of a row differ) and each weighs ``1 / top``.

Every expert is the clamped gated unit of ``clamped_gated_mlp`` (``down(g sigmoid(alpha g) (u + 1))``,
``g = min(gate x, limit)``, ``u = clamp(up x, -limit, limit)``) without biases, or, without a ``limit``,
the plain gated unit ``down(silu(gate x) * (up x))``; the shared expert is a
``clamped_gated_mlp`` part with sizes and constants of its own.  Routing, grouping of the tokens by
expert and the experts' products all run on the device (csrc/experts.hip), so a decode step can be
replayed from a graph.  The result is left as ``top`` (+ 1) slices, one for a token's k-th expert
(and one for the shared expert), which are added to the residual stream in this order: a token's sum
depends on its own choices only.
"""

from __future__ import annotations

import torch

from ..config.base import PartSpec
from ..ops import STORE_F32
from .base import FeedForward, PendingAdd, WeightSpec, build_part, part_class, register_part

DEFER_ROWS = 256     # steps of at most this many tokens leave the addition of the slices to the next norm


@register_part("routed_experts")
class RoutedExperts(FeedForward):
    """Parameters: ``hidden_size``, ``intermediate_size`` (of one expert), ``experts``, ``top``, ``limit``,
    ``alpha``, ``shared`` (None or the ``PartSpec`` of a feed-forward that runs for every token, built
    below ``<prefix>.shared``).  Tensors below the prefix: ``e<i>.gate``, ``e<i>.up`` ``[F, H]``,
    ``e<i>.down`` ``[H, F]`` for every expert ``i``, ``router`` ``[E, H]`` and ``router.b`` ``[E]``.
    ``limit`` None: the plain gated unit with SiLU.  ``router`` ``"table"`` (default ``"linear"``): the
    tensor ``table`` ``[vocab_size, top]`` (int) instead of the router's, with the parameter ``vocab_size``.
    ``score`` (``"softmax"`` over the chosen logits, the default, or ``"sigmoid"`` of each), ``weigh`` (``"output"``,
    the default, or ``"input"``), ``router_bias`` (default True; False: there is no tensor ``router.b``)."""

    graph_safe = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.inter = int(p["intermediate_size"])
        self.experts, self.top = int(p["experts"]), int(p["top"])
        self.plain = p.get("limit") is None
        # (the plain unit is the clamped one with no clamp, a slope of one and nothing added to the up half)
        self.limit, self.alpha = (float("inf"), 1.0) if self.plain else (float(p["limit"]), float(p["alpha"]))
        self.shift = 0.0 if self.plain else 1.0
        self.tabled = p.get("router", "linear") == "table"
        if p.get("router", "linear") not in ("linear", "table"):
            raise ValueError(f"router {p['router']!r} is not one of linear, table")
        self.score, self.weigh = p.get("score") or "softmax", p.get("weigh") or "output"
        self.router_bias = p.get("router_bias", True) is not False
        if self.score not in ("softmax", "sigmoid") or self.weigh not in ("output", "input"):
            raise ValueError(f"score {self.score!r} is not softmax or sigmoid, or weigh {self.weigh!r} not output or input")
        if self.tabled and self.score != "softmax":
            raise ValueError("experts that a table names have no scores")
        if not 0 < self.top <= self.experts:
            raise ValueError(f"a token cannot use {self.top} of {self.experts} experts")
        if not self.limit > 0:
            raise ValueError(f"the experts' limit must be positive, got {self.limit}")
        self.shared = build_part(p["shared"], self.join(prefix, "shared")) if p.get("shared") is not None else None
        self.w_router = self.b_router = self.w_gate = self.w_up = self.w_down = None

    def parts(self):
        return () if self.shared is None else (self.shared,)

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        p = spec.params
        h, f, e = int(p["hidden_size"]), int(p["intermediate_size"]), int(p["experts"])
        out = []
        for i in range(e):
            out += [WeightSpec(f"{prefix}.e{i}.gate", (f, h)), WeightSpec(f"{prefix}.e{i}.up", (f, h)),
                    WeightSpec(f"{prefix}.e{i}.down", (h, f))]
        if p.get("router", "linear") == "table":
            out.append(WeightSpec(f"{prefix}.table", (int(p["vocab_size"]), int(p["top"])), kind="int", init="distinct", free=e))
        else:
            out.append(WeightSpec(f"{prefix}.router", (e, h)))
            if p.get("router_bias", True) is not False:
                out.append(WeightSpec(f"{prefix}.router.b", (e,), kind="vector"))
        if p.get("shared") is not None:
            out += part_class(p["shared"].kind).weight_specs(p["shared"], cls.join(prefix, "shared"))
        return out

    def load(self, weights, rt) -> None:
        def stacked(name):
            mats = [weights.get(f"{self.prefix}.e{i}.{name}") for i in range(self.experts)]
            if len({m.dtype for m in mats}) > 1:
                mats = [m.to(torch.float32) for m in mats]
            return rt.matrix(torch.stack(mats, dim=0))

        self.w_gate, self.w_up, self.w_down = stacked("gate"), stacked("up"), stacked("down")
        if self.tabled:
            table = weights.get(f"{self.prefix}.table").to(torch.int32)
            if int(table.min()) < 0 or int(table.max()) >= self.experts:
                raise ValueError(f"{self.prefix}.table names experts outside [0, {self.experts})")
            if self.top > 1 and bool((table.sort(dim=1).values.diff(dim=1) == 0).any()):
                raise ValueError(f"{self.prefix}.table names an expert twice in a row")
            self.table = table.to(rt.device).contiguous()
            rt.kernels.experts_lib()
        else:
            self.w_router = rt.matrix(weights.get(f"{self.prefix}.router"))
            self.b_router = rt.vector(weights.get(f"{self.prefix}.router.b")) if self.router_bias else None
            rt.kernels.experts_lib()
        if not self.tabled and self.top > rt.kernels.experts_max_top():
            raise ValueError(f"{self.top} experts a token exceed the {rt.kernels.experts_max_top()} the routing kernel picks")
        if self.shared is not None:
            self.shared.load(weights, rt)

    @staticmethod
    def rows_a_tile(n_tokens: int, top: int, experts: int) -> int:
        """Rows of a tile of the experts' products: larger where an expert gets many tokens."""
        each = n_tokens * top / experts
        return 16 if each <= 16 else 32 if each <= 64 else 64

    def forward(self, ctx, x, out, accumulate: bool, defer=False):
        """``defer``: True leaves the slices to the next reader of the stream in steps of up to ``DEFER_ROWS`` tokens;
        ``"any"`` in every step (a reader that takes slices of any number of rows)."""
        rt = ctx.rt
        k = rt.kernels
        t, e, top = ctx.n_tokens, self.experts, self.top
        rows = self.rows_a_tile(t, top, e)
        cap = k.experts_tile_capacity(t, e, top, rows)
        chosen = ctx.buf("experts.chosen", (t * top,), torch.int32)
        share = ctx.buf("experts.share", (t * top,), torch.float32)
        order = ctx.buf("experts.order", (t * top,), torch.int32)
        tiles = ctx.buf("experts.tiles", (4 * cap,), torch.int32)
        counts = ctx.buf("experts.counts", (e,), torch.int32)
        if self.tabled:
            k.experts_route_table(ctx.token_ids, self.table, e, rows, chosen, share, order, tiles, counts)
        else:
            logits = ctx.buf("experts.logits", (t, e), torch.float32)
            k.gemm(x, self.w_router, logits, STORE_F32)
            k.experts_route(logits, self.b_router, top, rows, chosen, share, order, tiles, counts, scoring=self.score)
        slices = top + (1 if self.shared is not None else 0)
        partials = ctx.buf("experts.slices", (slices * t, self.hidden), torch.float32).view(slices, t, self.hidden)
        act = ctx.buf("experts.act", (t * top, self.inter), rt.dtype)
        k.experts_apply(x, self.w_gate, self.w_up, self.w_down, top, rows, order, tiles, share, self.limit, self.alpha,
                        act, partials[:top], shift=self.shift, weigh_input=self.weigh == "input")
        if self.shared is not None:
            self.shared.forward(ctx, x, partials[top], accumulate=False)
        pending = PendingAdd(partials)
        if defer == "any" or (defer and t <= DEFER_ROWS and self.hidden % 4 == 0):
            return pending                 # (the slices are the result: ``out`` is not touched)
        if not accumulate:
            out.zero_()
        pending.flush(ctx, out)
        return None
