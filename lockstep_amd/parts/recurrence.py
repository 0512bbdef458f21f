"""Linear-attention mixers that keep a matrix of fixed size per request and head instead of keys
and values.  ``gated_delta`` (at the end of this file) is the delta rule with a decay a head and short
convolutions in front; the two others share one recurrence with a decay and a write gate for every row of the state,

    S_t = diag(a_t) S_(t-1) + b_t v_t^T          S [dim, vdim] in float32, zero at the start
    o_t = S_t^T q_t

of which HGRN2 and retention are two choices of (q, a, b):

``hgrn2``      q = silu(W_q h); the forget gate f = lower + (1 - lower) * sigmoid(W_f h + bias) is both
               the decay and, as 1 - f, what is written: a = f, b = 1 - f.  Each head's o is
               RMS-normed over vdim with one weight for all heads, then W_o.
``retention``  q = rotate(W_q h), b = rotate(W_k h) / sqrt(dim), a = the head's constant decay.  Each
               head's o is divided by its root mean square (no weight), multiplied by
               silu(W_g h), then W_o.

The projections are one matrix product stored in float32; gates, rotation, the recurrence, the
state and the per-head norm are computed in 32-bit.  The state lives in the cache manager's state
slots: it is read at the start of a request's tokens of the step and left for the next step.
"""

from __future__ import annotations

import torch

from ..config.base import PartSpec
from ..ops import STORE_F32
from .base import Mixer, StateSpec, WeightSpec, build_part, project_out, register_part


class _LinearRecurrence(Mixer):
    """What both mixers share: sizes, the state's declaration, the order of the launches."""

    graph_safe = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads, self.d, self.dv = int(p["num_heads"]), int(p["head_dim"]), int(p["value_dim"])
        self.eps = float(p["eps"])
        if min(self.heads, self.d, self.dv) <= 0:
            raise ValueError("heads and sizes of a recurrent mixer must be positive")
        self.w_in = self.w_o = None

    def cache_spec(self):
        return StateSpec((self.heads, self.d, self.dv), "float32")

    def mixing_flops(self, tokens: int, start: int) -> float:
        """Decay, write and read of every state element per token."""
        return 5.0 * self.heads * self.d * self.dv * tokens

    def _check_dim(self, rt) -> None:
        most = rt.kernels.linrec_max_dim()
        if self.d > most:
            raise ValueError(f"a state of {self.d} rows a head is not supported: the recurrence kernel takes up to {most}")


@register_part("hgrn2")
class HGRN2(_LinearRecurrence):
    """Parameters: ``hidden_size``, ``num_heads``, ``head_dim``, ``value_dim``, ``eps`` (of the per-head
    norm).  Tensors below the prefix: ``q``, ``f`` ``[heads*dim, hidden]``, ``f.b``, ``lower``
    ``[heads*dim]``, ``v`` ``[heads*vdim, hidden]``, ``norm`` ``[vdim]``, ``o`` ``[hidden, heads*vdim]``."""

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        p = spec.params
        h, n, d, dv = int(p["hidden_size"]), int(p["num_heads"]), int(p["head_dim"]), int(p["value_dim"])
        return [WeightSpec(f"{prefix}.q", (n * d, h)), WeightSpec(f"{prefix}.f", (n * d, h)),
                WeightSpec(f"{prefix}.f.b", (n * d,), kind="vector"), WeightSpec(f"{prefix}.lower", (n * d,), kind="vector", init="unit"),
                WeightSpec(f"{prefix}.v", (n * dv, h)), WeightSpec(f"{prefix}.norm", (dv,), kind="vector", init="norm"),
                WeightSpec(f"{prefix}.o", (h, n * dv))]

    def load(self, weights, rt) -> None:
        self._check_dim(rt)
        q, f, v = (weights.get(f"{self.prefix}.{n}") for n in "qfv")
        if len({q.dtype, f.dtype, v.dtype}) > 1:
            q, f, v = q.to(torch.float32), f.to(torch.float32), v.to(torch.float32)
        self.w_in = rt.matrix(torch.cat([q, f, v], dim=0))
        self.w_o = rt.matrix(weights.get(f"{self.prefix}.o"))
        self.f_bias = rt.vector(weights.get(f"{self.prefix}.f.b"))
        self.lower = rt.vector(weights.get(f"{self.prefix}.lower"))
        self.norm = rt.vector(weights.get(f"{self.prefix}.norm"))
        rt.kernels.mixers_lib()

    def forward(self, ctx, run, x, out, accumulate: bool, defer: bool = False):
        rt, k, t = ctx.rt, ctx.rt.kernels, ctx.n_tokens
        n, d, dv = self.heads, self.d, self.dv
        raw = ctx.buf("recurrence.in_f32", (t, 2 * n * d + n * dv), torch.float32)
        k.gemm(x, self.w_in, raw, STORE_F32)
        o = ctx.buf("recurrence.o_f32", (t, n * dv), torch.float32)
        gates = ctx.buf("recurrence.gates", (k.linrec_gate_floats(t, n, d),), torch.float32)
        k.linrec(k.LINREC_HGRN2, raw, 0, n * d, 2 * n * d, n, d, dv, self.lower, self.f_bias, None, None, 0,
                 ctx.max_position, ctx.tok_pos, ctx.seqs, ctx.n_seqs, ctx.cache.unit_state(run.cache), gates, o)
        normed = ctx.buf("recurrence.normed", (t, n * dv), rt.dtype)
        k.head_norm_gate(o, n, dv, self.norm, None, self.eps, normed)
        return project_out(ctx, normed, self.w_o, out, accumulate, defer, "recurrence.out_slices")


@register_part("retention")
class Retention(_LinearRecurrence):
    """Parameters: ``hidden_size``, ``num_heads``, ``head_dim``, ``value_dim``, ``eps``, ``decay`` (one
    number a head), ``position`` (a position-encoding ``PartSpec`` for q and k).  Tensors below the
    prefix: ``q``, ``k`` ``[heads*dim, hidden]``, ``v``, ``g`` ``[heads*vdim, hidden]``, ``o``."""

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        self.decay = [float(v) for v in spec["decay"]]
        if len(self.decay) != self.heads:
            raise ValueError(f"{len(self.decay)} decays for {self.heads} heads")
        self.position = build_part(spec["position"], prefix)
        if self.position.rotary_dim > self.d:
            raise ValueError(f"rotary_dim {self.position.rotary_dim} exceeds head size {self.d}")

    def parts(self):
        return (self.position,)

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        p = spec.params
        h, n, d, dv = int(p["hidden_size"]), int(p["num_heads"]), int(p["head_dim"]), int(p["value_dim"])
        return [WeightSpec(f"{prefix}.q", (n * d, h)), WeightSpec(f"{prefix}.k", (n * d, h)),
                WeightSpec(f"{prefix}.v", (n * dv, h)), WeightSpec(f"{prefix}.g", (n * dv, h)),
                WeightSpec(f"{prefix}.o", (h, n * dv))]

    def load(self, weights, rt) -> None:
        self._check_dim(rt)
        tensors = [weights.get(f"{self.prefix}.{n}") for n in "qkvg"]
        if len({t.dtype for t in tensors}) > 1:
            tensors = [t.to(torch.float32) for t in tensors]
        self.w_in = rt.matrix(torch.cat(tensors, dim=0))
        self.w_o = rt.matrix(weights.get(f"{self.prefix}.o"))
        self.decays = rt.vector(torch.tensor(self.decay, dtype=torch.float64))
        rt.kernels.mixers_lib()
        if hasattr(self.position, "bind"):
            self.position.bind(rt)

    def prepare_group(self):
        share = getattr(self.position, "share_key", None)
        return None if share is None else ("retention", share())

    def prepare(self, ctx) -> None:
        self.position.ensure(ctx.max_position + 1, ctx.rt)

    def forward(self, ctx, run, x, out, accumulate: bool, defer: bool = False):
        rt, k, t = ctx.rt, ctx.rt.kernels, ctx.n_tokens
        n, d, dv = self.heads, self.d, self.dv
        raw = ctx.buf("recurrence.in_f32", (t, 2 * n * d + 2 * n * dv), torch.float32)
        k.gemm(x, self.w_in, raw, STORE_F32)
        o = ctx.buf("recurrence.o_f32", (t, n * dv), torch.float32)
        gates = ctx.buf("recurrence.gates", (k.linrec_gate_floats(t, n, d),), torch.float32)
        k.linrec(k.LINREC_RETENTION, raw, 0, n * d, 2 * n * d, n, d, dv, self.decays, None, self.position.cos,
                 self.position.sin, self.position.rotary_dim, ctx.max_position, ctx.tok_pos, ctx.seqs, ctx.n_seqs,
                 ctx.cache.unit_state(run.cache), gates, o)
        gated = ctx.buf("recurrence.normed", (t, n * dv), rt.dtype)
        k.head_norm_gate(o, n, dv, None, raw[:, 2 * n * d + n * dv:], self.eps, gated)
        return project_out(ctx, gated, self.w_o, out, accumulate, defer, "recurrence.out_slices")


@register_part("gated_delta")
class GatedDelta(Mixer):
    """The gated delta rule: a state matrix a head that forgets by a decay and is corrected, not
    just added to, by every token:

        S <- g_t S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t

    ``q = W_q h`` and ``k = W_k h`` (``num_kv_heads`` heads of ``head_dim``; head ``n`` of ``num_heads`` uses
    q/k head ``n // (num_heads / num_kv_heads)``) and ``v = W_v h`` (``num_heads`` of ``value_dim``) pass a
    short causal convolution a channel (``<tensor>.conv`` ``[channels, taps]``, the last column is the
    current token's, zeros before the start) and SiLU; q and k are then unit vectors a head, ``x /
    sqrt(sum x^2 + unit_eps)``, q also times ``head_dim^-1/2``.  ``beta = sigmoid(W_b h)``, ``g =
    exp(-exp(A_log) softplus(W_a h + dt_bias))``, one of each a head.  Each head's ``o`` is divided by its
    root mean square (``eps``), multiplied by ``norm [value_dim]`` and by ``silu(W_g h)``; then ``W_o``.

    Parameters: ``hidden_size``, ``num_heads``, ``num_kv_heads``, ``head_dim``, ``value_dim``, ``taps``,
    ``eps``, ``unit_eps``.  Tensors below the prefix: ``q``, ``k``, ``v`` with ``q.conv``, ``k.conv``,
    ``v.conv``; ``b``, ``a`` ``[heads, hidden]``; ``A_log``, ``dt_bias`` ``[heads]``; ``g`` ``[heads*vdim,
    hidden]``; ``norm`` ``[vdim]``; ``o``.

    ``decay = "channel"`` (default ``"head"``): one decay for every head and key channel, which multiplies
    the rows of ``S``: ``g = exp(-exp(A_log_h) softplus(W_a2 (W_a1 h) + dt_bias))``, laid out heads x
    ``head_dim``, through a bottleneck of ``decay_rank`` (tensors ``a1 [decay_rank, hidden]``, ``a2 [heads *
    head_dim, decay_rank]``, ``dt_bias [heads * head_dim]`` instead of ``a`` and ``dt_bias [heads]``).
    ``gate_rank`` (default None): the output gate's logits come through a bottleneck as well, ``W_g2 (W_g1
    h)`` (tensors ``g1 [gate_rank, hidden]``, ``g2 [heads * vdim, gate_rank]`` instead of ``g``).
    ``gate_act`` (``"silu"``, the default, or ``"sigmoid"``): what is applied to the gate's logits.
    A size of -1 for a rank is one that the checkpoint's tensors decide.

    The projections are one matrix product stored in float32; convolutions, gates, the recurrence and
    the per-head norm are computed in 32-bit.  A request's state slot holds the matrices and, behind
    them, the last ``taps - 1`` inputs of every convolution channel."""

    graph_safe = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads, self.kv_heads = int(p["num_heads"]), int(p["num_kv_heads"])
        self.d, self.dv, self.taps = int(p["head_dim"]), int(p["value_dim"]), int(p["taps"])
        self.eps, self.unit_eps = float(p["eps"]), float(p["unit_eps"])
        self.decay = p.get("decay") or "head"
        self.gate_act = p.get("gate_act") or "silu"
        self.gate_rank = p.get("gate_rank")
        if self.decay not in ("head", "channel") or self.gate_act not in ("silu", "sigmoid"):
            raise ValueError(f"decay {self.decay!r} is not head or channel, or gate_act {self.gate_act!r} not silu or sigmoid")
        if min(self.heads, self.kv_heads, self.d, self.dv, self.taps) <= 0 or self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads over {self.kv_heads} query/key heads with sizes {self.d}, {self.dv} "
                             f"and {self.taps} taps are not a gated delta mixer")
        self.channels = 2 * self.kv_heads * self.d + self.heads * self.dv
        self.w_in = self.w_o = self.conv = self.a_log = self.dt_bias = self.norm = self.w_a2 = self.w_g2 = None

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        p = spec.params
        h, n, g, d, dv, m = (int(p[key]) for key in ("hidden_size", "num_heads", "num_kv_heads", "head_dim", "value_dim", "taps"))
        out = [WeightSpec(f"{prefix}.q", (g * d, h)), WeightSpec(f"{prefix}.q.conv", (g * d, m), kind="vector", init="unit"),
               WeightSpec(f"{prefix}.k", (g * d, h)), WeightSpec(f"{prefix}.k.conv", (g * d, m), kind="vector", init="unit"),
               WeightSpec(f"{prefix}.v", (n * dv, h)), WeightSpec(f"{prefix}.v.conv", (n * dv, m), kind="vector", init="unit"),
               WeightSpec(f"{prefix}.b", (n, h)), WeightSpec(f"{prefix}.A_log", (n,), kind="vector"),
               WeightSpec(f"{prefix}.norm", (dv,), kind="vector", init="norm")]
        if (p.get("decay") or "head") == "channel":
            rank = int(p["decay_rank"])
            out += [WeightSpec(f"{prefix}.a1", (rank, h), free=16), WeightSpec(f"{prefix}.a2", (n * d, rank), free=16),
                    WeightSpec(f"{prefix}.dt_bias", (n * d,), kind="vector")]
        else:
            out += [WeightSpec(f"{prefix}.a", (n, h)), WeightSpec(f"{prefix}.dt_bias", (n,), kind="vector")]
        if p.get("gate_rank") is not None:
            rank = int(p["gate_rank"])
            out += [WeightSpec(f"{prefix}.g1", (rank, h), free=16), WeightSpec(f"{prefix}.g2", (n * dv, rank), free=16)]
        else:
            out.append(WeightSpec(f"{prefix}.g", (n * dv, h)))
        return out + [WeightSpec(f"{prefix}.o", (h, n * dv))]

    def cache_spec(self):
        return StateSpec((self.heads * self.d * self.dv + (self.taps - 1) * self.channels,), "float32")

    def mixing_flops(self, tokens: int, start: int) -> float:
        """Decay, two reads and a write of every state element per token."""
        return 7.0 * self.heads * self.d * self.dv * tokens

    def load(self, weights, rt) -> None:
        if self.d > rt.kernels.delta_max_dim():
            raise ValueError(f"a state of {self.d} rows a head is not supported: the delta rule kernel takes up to "
                             f"{rt.kernels.delta_max_dim()}")
        # one product, stored in float32, for what the 32-bit passes read: q | k | v | b, then a (a decay a head),
        # then g (a gate without a bottleneck); a second one, in the compute dtype, for the bottlenecks a1 | g1,
        # which the products with a2 and g2 read
        names = ["q", "k", "v", "b"] + ([] if self.decay == "channel" else ["a"]) + (["g"] if self.gate_rank is None else [])
        tensors = [weights.get(f"{self.prefix}.{n}") for n in names]
        if len({t.dtype for t in tensors}) > 1:
            tensors = [t.to(torch.float32) for t in tensors]
        self.w_in = rt.matrix(torch.cat(tensors, dim=0))
        low = [weights.get(f"{self.prefix}.{n}") for n in (["a1"] if self.decay == "channel" else []) +
               (["g1"] if self.gate_rank is not None else [])]
        if len({t.dtype for t in low}) > 1:
            low = [t.to(torch.float32) for t in low]
        self.decay_rank = low[0].shape[0] if self.decay == "channel" else 0
        # (zero rows behind a1, so that the gate's part of the product's rows starts on a 16-byte boundary)
        self.low_gate_at = -(-self.decay_rank // 8) * 8
        if self.decay == "channel" and len(low) > 1 and self.low_gate_at > self.decay_rank:
            low.insert(1, low[0].new_zeros((self.low_gate_at - self.decay_rank, low[0].shape[1])))
        self.w_low = rt.matrix(torch.cat(low, dim=0)) if low else None
        if self.decay == "channel":
            self.w_a2 = rt.matrix(weights.get(f"{self.prefix}.a2"))
        if self.gate_rank is not None:
            self.w_g2 = rt.matrix(weights.get(f"{self.prefix}.g2"))
        self.w_o = rt.matrix(weights.get(f"{self.prefix}.o"))
        self.conv = rt.vector(torch.cat([weights.get(f"{self.prefix}.{n}.conv").to(torch.float32) for n in "qkv"], dim=0))
        self.a_log = rt.vector(weights.get(f"{self.prefix}.A_log"))
        self.dt_bias = rt.vector(weights.get(f"{self.prefix}.dt_bias"))
        self.norm = rt.vector(weights.get(f"{self.prefix}.norm"))
        rt.kernels.mixers_lib()

    def forward(self, ctx, run, x, out, accumulate: bool, defer: bool = False):
        rt, k, t = ctx.rt, ctx.rt.kernels, ctx.n_tokens
        n, g, d, dv = self.heads, self.kv_heads, self.d, self.dv
        raw = ctx.buf("delta.in_f32", (t, self.w_in.shape[0]), torch.float32)
        k.gemm(x, self.w_in, raw, STORE_F32)
        o = ctx.buf("delta.o_f32", (t, n * dv), torch.float32)
        channel = self.decay == "channel"
        scratch = ctx.buf("delta.scratch", (k.delta_scratch_floats(t, g, n, d, dv, channel),), torch.float32)
        decay_logits = None
        if self.w_low is not None:
            from ..ops import STORE

            low = ctx.buf("delta.low", (t, self.w_low.shape[0]), rt.dtype)
            k.gemm(x, self.w_low, low, STORE)
        if channel:
            decay_logits = ctx.buf("delta.decay_f32", (t, n * d), torch.float32)
            k.gemm(low[:, :self.decay_rank], self.w_a2, decay_logits, STORE_F32)
        gate = raw[:, self.channels + (1 if channel else 2) * n:]
        if self.gate_rank is not None:
            gate = ctx.buf("delta.gate_f32", (t, n * dv), torch.float32)
            k.gemm(low[:, self.low_gate_at:], self.w_g2, gate, STORE_F32)
        k.delta_rule(raw, g, n, d, dv, self.conv, self.a_log, self.dt_bias, self.unit_eps, ctx.tok_seq, ctx.tok_pos,
                     ctx.seqs, ctx.n_seqs, ctx.cache.unit_state(run.cache), scratch, o, channel_decay=decay_logits)
        gated = ctx.buf("delta.normed", (t, n * dv), rt.dtype)
        k.head_norm_gate(o, n, dv, self.norm, gate, self.eps, gated, gate_act=self.gate_act)
        return project_out(ctx, gated, self.w_o, out, accumulate, defer, "delta.out_slices")
