"""Norms of the residual stream.  RMSNorm: ``y = x * 1/sqrt(mean(x^2) + eps) * w`` in 32-bit
(reference engine/kernels/rmsnorm.py:30-38).  Dynamic Tanh: ``y = tanh(alpha x) * w + b``, which
takes no statistics of the row."""

from __future__ import annotations

from ..config.base import PartSpec
from .base import Norm, WeightSpec, register_part


@register_part("rmsnorm")
class RMSNorm(Norm):
    """Parameters: ``size``, ``eps``; ``name`` overrides the tensor name.  With ``optional`` the
    weight may be absent (a layer whose second half is missing never runs the norm).  ``offset``
    (default 0): the stored weight is the distance of the factor from this number, the row is
    multiplied by ``offset + w`` (1 for weights stored around zero).  ``copies`` (default 1): the
    stream holds that many copies ``[T, copies * size]`` and the norm reads their sum."""

    graph_safe = True
    repeatable = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        self.size = int(spec["size"])
        self.eps = float(spec["eps"])
        self.offset = float(spec.params.get("offset") or 0.0)
        self.copies = int(spec.params.get("copies") or 1)
        self.weight = None

    @staticmethod
    def tensor_name(spec: PartSpec, prefix: str) -> str:
        return spec.params.get("name") or f"{prefix}.weight"

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        return [WeightSpec(cls.tensor_name(spec, prefix), (int(spec["size"]),), kind="vector",
                           init="around_zero" if spec.params.get("offset") else "norm",
                           optional=bool(spec.params.get("optional")))]

    def load(self, weights, rt) -> None:
        name = self.tensor_name(self.spec, self.prefix)
        if self.spec.params.get("optional") and name not in weights:
            return
        self.weight = rt.vector(weights.get(name))
        if self.offset:
            self.weight = self.weight + self.offset          # (float32: the factor as 32-bit arithmetic forms it)

    def forward(self, ctx, x, out, rows=None, pending=None) -> None:
        """``pending`` (a ``PendingAdd``): added to ``x`` first, in the same launch."""
        if self.copies > 1 or hasattr(pending, "mix"):
            # the sum of the copies, after what the last sublayer still has to write into them
            if pending is not None and not hasattr(pending, "mix"):
                raise ValueError("a stream of several copies takes the pending write of its own arrangement only")
            ctx.rt.kernels.streams_step(x, self.copies, None if pending is None else pending.partials,
                                        None if pending is None else pending.mix, None if pending is None else pending.gain,
                                        None, self.weight, self.eps, out, rows)
            return
        if pending is not None:
            ctx.rt.kernels.add_rmsnorm(x, pending.partials, self.weight, out, self.eps, rows)
        else:
            ctx.rt.kernels.rmsnorm(x, self.weight, out, self.eps, rows)


@register_part("dynamic_tanh")
class DynamicTanh(Norm):
    """``y = tanh(alpha * x) * w + b`` elementwise, in 32-bit: a norm without mean or variance.
    Parameters: ``size``; ``name`` overrides the weight's tensor name (default: the prefix itself).
    The bias ``[size]`` and the scalar ``alpha`` are stored beside the weight as ``<name>.b`` and
    ``<name>.alpha``.  With ``optional`` the tensors may be absent (a layer whose second half is
    missing never runs the norm)."""

    graph_safe = True
    repeatable = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        self.size = int(spec["size"])
        self.weight = self.bias = self.alpha = None

    @staticmethod
    def tensor_name(spec: PartSpec, prefix: str) -> str:
        return spec.params.get("name") or prefix

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        name, size, optional = cls.tensor_name(spec, prefix), int(spec["size"]), bool(spec.params.get("optional"))
        return [WeightSpec(name, (size,), kind="vector", init="norm", optional=optional),
                WeightSpec(f"{name}.b", (size,), kind="vector", optional=optional),
                WeightSpec(f"{name}.alpha", (), kind="vector", init="norm", optional=optional)]

    def load(self, weights, rt) -> None:
        name = self.tensor_name(self.spec, self.prefix)
        if self.spec.params.get("optional") and name not in weights:
            return
        self.weight = rt.vector(weights.get(name))
        self.bias = rt.vector(weights.get(f"{name}.b"))
        self.alpha = rt.vector(weights.get(f"{name}.alpha").reshape(1))

    def forward(self, ctx, x, out, rows=None, pending=None) -> None:
        """``pending`` (a ``PendingAdd``): added to ``x`` first, in the same launch."""
        ctx.rt.kernels.dyt(x, self.weight, self.bias, self.alpha, out, rows,
                           partials=None if pending is None else pending.partials)
