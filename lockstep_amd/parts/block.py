"""Arrangements: how a layer's parts are wired around the residual stream."""

from __future__ import annotations

from .base import Arrangement, PendingAdd, StateSpec, WeightSpec, build_part, register_part, takes


@register_part("prenorm_residual")
class PreNormResidual(Arrangement):
    """``h += mixer(norm_1(h)); h += feed_forward(norm_2(h))``
    (reference engine/model/qwen3.py:324-370).

    Parameters name the parts' tensor prefixes below the layer's prefix:
    ``mixer_prefix``, ``feed_forward_prefix``, ``mixer_norm_name``,
    ``feed_forward_norm_name``.  A layer without a ``feed_forward`` part is the first half alone.

    ``token_shift`` (optional, a tensor name below the layer's prefix): what the mixer reads, ``n =
    norm_1(h)``, is replaced by ``n[t] + (n[t-1] - n[t]) * mu`` with the tensor ``mu [width]`` and the
    unshifted ``n[t-1]`` of the same request's token before (zeros for its first token).  The last
    ``n`` of a request is kept between steps: the arrangement then has a ``state_spec`` and its
    schedule entry names a unit for it.
    """

    graph_safe = True
    repeatable = True

    def __init__(self, layer_spec, prefix: str = ""):
        super().__init__(layer_spec, build_part)
        p = layer_spec.arrangement.params
        base = layer_spec.prefix
        self.mixer_norm = build_part(layer_spec.part("mixer_norm"), self.join(base, p["mixer_norm_name"]))
        self._mixer = build_part(layer_spec.part("mixer"), self.join(base, p["mixer_prefix"]))
        self.feed_forward = self.feed_forward_norm = None
        if layer_spec.has("feed_forward"):
            self.feed_forward_norm = build_part(layer_spec.part("feed_forward_norm"),
                                                self.join(base, p["feed_forward_norm_name"]))
            self.feed_forward = build_part(layer_spec.part("feed_forward"), self.join(base, p["feed_forward_prefix"]))
        self._fuse_mixer = self._fuses(self._mixer, self.mixer_norm)
        self._fuse_ff = self.feed_forward is not None and self._fuses(self.feed_forward, self.feed_forward_norm)
        # parts that can leave their residual addition to the next norm (see PendingAdd)
        self._defer_mixer = takes(self._mixer.forward, "defer")
        self._defer_ff = self.feed_forward is not None and takes(self.feed_forward.forward, "defer")
        self._norm1_pending = takes(self.mixer_norm.forward, "pending")
        self._norm2_pending = self.feed_forward is not None and takes(self.feed_forward_norm.forward, "pending")
        self.shift_name = p.get("token_shift")
        self.shift = None
        self.width = None
        if self.shift_name:
            self.width = int(layer_spec.part("mixer_norm")["size"])
            self._fuse_mixer = False          # (the shift stands between the norm and the mixer)
        # one launch for addition, norm and shift where the norm is a plain RMS norm over rows of whole vectors of four
        norm = self.mixer_norm
        self._shift_fused = bool(self.shift_name) and getattr(norm, "kind", "") == "rmsnorm" and norm.copies == 1 \
            and self._norm1_pending and self.width % 4 == 0

    def state_spec(self):
        return StateSpec((self.width,), "float32") if self.shift_name else None

    @classmethod
    def weight_specs(cls, layer_spec, prefix: str = ""):
        from .base import part_class

        p = layer_spec.arrangement.params
        base = layer_spec.prefix
        out = []
        if p.get("token_shift"):
            out.append(WeightSpec(cls.join(base, p["token_shift"]), (int(layer_spec.part("mixer_norm")["size"]),),
                                  kind="vector", init="unit"))
        wired = [(layer_spec.part("mixer_norm"), p["mixer_norm_name"]), (layer_spec.part("mixer"), p["mixer_prefix"])]
        if layer_spec.has("feed_forward"):
            wired += [(layer_spec.part("feed_forward_norm"), p["feed_forward_norm_name"]),
                      (layer_spec.part("feed_forward"), p["feed_forward_prefix"])]
        elif layer_spec.has("feed_forward_norm"):
            # a norm the checkpoint may hold although nothing follows it: its tensors are accepted, never used
            wired.append((layer_spec.part("feed_forward_norm"), p["feed_forward_norm_name"]))
        for spec, name in wired:
            out += part_class(spec.kind).weight_specs(spec, cls.join(base, name))
        return out

    def parts(self):
        if self.feed_forward is None:
            return (self.mixer_norm, self._mixer)
        return (self.mixer_norm, self._mixer, self.feed_forward_norm, self.feed_forward)

    @property
    def mixer(self):
        return self._mixer

    def load(self, weights, rt) -> None:
        for part in self.parts():
            part.load(weights, rt)
        if self.shift_name:
            self.shift = rt.vector(weights.get(self.join(self.layer_spec.prefix, self.shift_name)))
            rt.kernels.mixers_lib()

    #: a step of at most this many tokens lets the consumer's first matrix
    #: product normalise its input itself (one launch less per norm).  Off by
    #: default: on MI355X the longer dependent chain inside the product costs
    #: more than the launch it saves (Qwen3-0.6B sizes, batch 1 and 8: 7 % slower).
    FUSE_NORM_ROWS = int(__import__("os").environ.get("LOCKSTEP_FUSE_NORM_ROWS", "0"))

    @staticmethod
    def _fuses(part, norm) -> bool:
        import inspect

        return (getattr(norm, "kind", "") == "rmsnorm"
                and "norm" in inspect.signature(part.forward).parameters)

    def forward(self, ctx, run, h, pending=None):
        """``pending``: an addition to ``h`` that the previous layer left to its reader.  Returns
        the one this layer leaves (or None)."""
        rt = ctx.rt
        small = ctx.n_tokens <= self.FUSE_NORM_ROWS
        if pending is not None and (small and self._fuse_mixer or not self._norm1_pending):
            pending.flush(ctx, h)
            pending = None
        if small and self._fuse_mixer:
            mixed = self._mixer.forward(ctx, run, h, h, accumulate=True, norm=self.mixer_norm)
        else:
            x = ctx.buf("block.normed", (ctx.n_tokens, h.shape[1]), rt.dtype)
            if self._shift_fused and ctx.single_tokens:
                # a step of single tokens: the addition that is still open, the norm and the shift in one launch
                rt.kernels.add_rmsnorm_shift(h, None if pending is None else pending.partials, self.mixer_norm.weight,
                                             self.mixer_norm.eps, self.shift, ctx.tok_seq, ctx.tok_pos, ctx.seqs,
                                             ctx.cache.unit_state(run.state), x)
            else:
                # (with a token shift the norm's rows stay in float32, and the shift writes what the mixer reads)
                n = ctx.buf("block.unshifted", (ctx.n_tokens, h.shape[1]), __import__("torch").float32) if self.shift_name else x
                if pending is not None:
                    self.mixer_norm.forward(ctx, h, n, pending=pending)
                else:
                    self.mixer_norm.forward(ctx, h, n)
                if self.shift_name:
                    rt.kernels.token_shift(n, self.shift, ctx.tok_seq, ctx.tok_pos, ctx.seqs, ctx.cache.unit_state(run.state), x)
            if self._defer_mixer:
                mixed = self._mixer.forward(ctx, run, x, h, accumulate=True, defer=True)
            else:
                mixed = self._mixer.forward(ctx, run, x, h, accumulate=True)
        mixed = mixed if isinstance(mixed, PendingAdd) else None
        if self.feed_forward is None:
            return mixed
        if mixed is not None and (small and self._fuse_ff or not self._norm2_pending):
            mixed.flush(ctx, h)
            mixed = None
        if small and self._fuse_ff:
            left = self.feed_forward.forward(ctx, h, h, accumulate=True, norm=self.feed_forward_norm)
        else:
            x = ctx.buf("block.normed", (ctx.n_tokens, h.shape[1]), rt.dtype)
            if mixed is not None:
                self.feed_forward_norm.forward(ctx, h, x, pending=mixed)
            else:
                self.feed_forward_norm.forward(ctx, h, x)
            if self._defer_ff:
                left = self.feed_forward.forward(ctx, x, h, accumulate=True, defer=True)
            else:
                left = self.feed_forward.forward(ctx, x, h, accumulate=True)
        return left if isinstance(left, PendingAdd) else None


class PendingWrite(PendingAdd):
    """A sublayer's output that still has to be written into a residual stream of several copies:
    ``x'_t = sum_s mix[s, t] x_s + gain[t] y`` with ``y`` the sum of ``partials`` in ascending order.
    The next reader of the stream does it on its way (the next sublayer's read, or the final norm)."""

    def __init__(self, partials, mix, gain, copies: int):
        super().__init__(partials)
        self.mix, self.gain, self.copies = mix, gain, copies

    def flush(self, ctx, stream, rows=None) -> None:
        ctx.rt.kernels.streams_step(stream, self.copies, self.partials, self.mix, self.gain, None, None, 0.0, None, rows)


@register_part("hyper_connections")
class HyperConnections(Arrangement):
    """A layer over a residual stream of ``copies`` copies ``x_1 .. x_n`` (``h [T, copies * width]``, all
    equal to the embedding at the start; the model's last norm reads their sum).  Each sublayer
    ``f`` (the mixer, then the feed-forward, if any) with its norm reads one weighted sum and writes to
    all copies at once:

        u = sum_s take[s] x_s;   y = f(norm(u));   x'_t = sum_s mix[s, t] x_s + gain[t] y

    ``mix`` is indexed ``[from, to]``.  The write of a sublayer is left to the launch that reads the
    stream next, which also normalises what it read: one launch a sublayer.

    Parameters: ``copies``; ``mixer_prefix``, ``feed_forward_prefix``, ``mixer_norm_name``,
    ``feed_forward_norm_name`` as for ``prenorm_residual``; ``mixer_streams_prefix``,
    ``feed_forward_streams_prefix``: below them the tensors ``in [n]`` (take), ``out [n]`` (gain) and
    ``mix [n, n]``.  The norms must be ``rmsnorm`` parts (their weight and eps are applied by the read)."""

    graph_safe = True

    def __init__(self, layer_spec, prefix: str = ""):
        super().__init__(layer_spec, build_part)
        p = layer_spec.arrangement.params
        base = layer_spec.prefix
        self.copies = int(p["copies"])
        if self.copies < 1:
            raise ValueError(f"a residual stream of {self.copies} copies")
        self.mixer_norm = build_part(layer_spec.part("mixer_norm"), self.join(base, p["mixer_norm_name"]))
        self._mixer = build_part(layer_spec.part("mixer"), self.join(base, p["mixer_prefix"]))
        self.feed_forward = self.feed_forward_norm = None
        if layer_spec.has("feed_forward"):
            self.feed_forward_norm = build_part(layer_spec.part("feed_forward_norm"),
                                                self.join(base, p["feed_forward_norm_name"]))
            self.feed_forward = build_part(layer_spec.part("feed_forward"), self.join(base, p["feed_forward_prefix"]))
        for norm in (self.mixer_norm, self.feed_forward_norm):
            if norm is not None and getattr(norm, "kind", "") != "rmsnorm":
                raise ValueError("the sublayers of a stream of several copies are normalised by rmsnorm parts")
        self._defer_mixer = takes(self._mixer.forward, "defer")
        self._defer_ff = self.feed_forward is not None and takes(self.feed_forward.forward, "defer")
        self.streams = {}        # sublayer -> (take, gain, mix) on the device

    @classmethod
    def _stream_specs(cls, prefix: str, n: int, optional: bool = False):
        from .base import WeightSpec

        return [WeightSpec(f"{prefix}.in", (n,), kind="vector", init="unit", optional=optional),
                WeightSpec(f"{prefix}.out", (n,), kind="vector", init="norm", optional=optional),
                WeightSpec(f"{prefix}.mix", (n, n), kind="vector", init="identity", optional=optional)]

    @classmethod
    def weight_specs(cls, layer_spec, prefix: str = ""):
        from .base import part_class

        p = layer_spec.arrangement.params
        base, n = layer_spec.prefix, int(p["copies"])
        out = []
        wired = [(layer_spec.part("mixer_norm"), p["mixer_norm_name"]), (layer_spec.part("mixer"), p["mixer_prefix"])]
        out += cls._stream_specs(cls.join(base, p["mixer_streams_prefix"]), n)
        if layer_spec.has("feed_forward"):
            wired += [(layer_spec.part("feed_forward_norm"), p["feed_forward_norm_name"]),
                      (layer_spec.part("feed_forward"), p["feed_forward_prefix"])]
            out += cls._stream_specs(cls.join(base, p["feed_forward_streams_prefix"]), n)
        else:
            # what the checkpoint may hold for a second half that never runs is accepted, never used
            if layer_spec.has("feed_forward_norm"):
                wired.append((layer_spec.part("feed_forward_norm"), p["feed_forward_norm_name"]))
            out += cls._stream_specs(cls.join(base, p["feed_forward_streams_prefix"]), n, optional=True)
        for spec, name in wired:
            out += part_class(spec.kind).weight_specs(spec, cls.join(base, name))
        return out

    def parts(self):
        if self.feed_forward is None:
            return (self.mixer_norm, self._mixer)
        return (self.mixer_norm, self._mixer, self.feed_forward_norm, self.feed_forward)

    @property
    def mixer(self):
        return self._mixer

    def load(self, weights, rt) -> None:
        for part in self.parts():
            part.load(weights, rt)
        p = self.layer_spec.arrangement.params
        most, widest = rt.kernels.streams_max()
        if self.copies > most:
            raise ValueError(f"a residual stream of {self.copies} copies; the kernel takes up to {most}")
        names = [("mixer", p["mixer_streams_prefix"])]
        if self.feed_forward is not None:
            names.append(("feed_forward", p["feed_forward_streams_prefix"]))
        for sublayer, name in names:
            full = self.join(self.layer_spec.prefix, name)
            self.streams[sublayer] = tuple(rt.vector(weights.get(f"{full}.{t}").reshape(-1)) for t in ("in", "out", "mix"))

    def _run(self, ctx, sublayer, defers: bool, call, width: int):
        """One sublayer's output as slice sums ``[slices, T, width]``."""
        import torch

        t = ctx.n_tokens
        y = ctx.buf(f"streams.y.{sublayer}", (t, width), torch.float32)
        # (a part that defers leaves slice sums and does not touch y; else it stores its output there)
        left = call(y, False, "any") if defers else call(y, False, False)
        if isinstance(left, PendingAdd):
            return left.partials
        return y.view(1, t, width)

    def forward(self, ctx, run, h, pending=None):
        """``pending``: the write the previous layer left (a ``PendingWrite``).  Returns this layer's last one."""
        rt = ctx.rt
        k = rt.kernels
        n = self.copies
        width = h.shape[1] // n
        if pending is not None and not isinstance(pending, PendingWrite):
            pending.flush(ctx, h)
            pending = None
        take, gain, mix = self.streams["mixer"]
        x = ctx.buf("block.normed", (ctx.n_tokens, width), rt.dtype)
        k.streams_step(h, n, None if pending is None else pending.partials, None if pending is None else pending.mix,
                       None if pending is None else pending.gain, take, self.mixer_norm.weight, self.mixer_norm.eps, x)
        if self._defer_mixer:
            call = lambda y, acc, defer: self._mixer.forward(ctx, run, x, y, accumulate=acc, defer=defer)  # noqa: E731
        else:
            call = lambda y, acc, defer: self._mixer.forward(ctx, run, x, y, accumulate=acc)  # noqa: E731
        left = PendingWrite(self._run(ctx, "mixer", self._defer_mixer, call, width), mix, gain, n)
        if self.feed_forward is None:
            return left
        take, gain, mix = self.streams["feed_forward"]
        x = ctx.buf("block.normed", (ctx.n_tokens, width), rt.dtype)
        k.streams_step(h, n, left.partials, left.mix, left.gain, take, self.feed_forward_norm.weight,
                       self.feed_forward_norm.eps, x)
        if self._defer_ff:
            call = lambda y, acc, defer: self.feed_forward.forward(ctx, x, y, accumulate=acc, defer=defer)  # noqa: E731
        else:
            call = lambda y, acc, defer: self.feed_forward.forward(ctx, x, y, accumulate=acc)  # noqa: E731
        return PendingWrite(self._run(ctx, "feed_forward", self._defer_ff, call, width), mix, gain, n)
