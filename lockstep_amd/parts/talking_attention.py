"""Attention whose heads exchange their scores before the softmax ("talking heads"), over the
paged cache, with a sliding window that keeps the first tokens, keys and values of different
sizes, biased projections, partial rotation and value mixing across layers.

For the step's queries ``q_h`` (head h of H) and all cached keys ``k_g`` / values ``v_g`` (head g of
G, query head h reads kv head ``h // (H/G)``):

    raw_h[i, j] = scale * <q_h[i], k_kv(h)[j]>
    s_h[i, j]   = sum_g talk[h, g] * raw_g[i, j]
    j is visible to i  iff  j <= i and (i - j < window or j < keep_first)      (true positions)
    o_h[i]      = sum_j softmax_j(s_h[i, :])[j] * v_kv(h)[j]

Value mixing: the first layer of a model that mixes values keeps this step's values (``v_mix =
"source"``); every later one (``v_mix = "mix"``) replaces its own by ``(1 - lambda) v + lambda
v_first`` of the same token before they are cached, with its scalar ``lambda``.

The projections are one matrix product over ``[Wq; Wk; Wv]`` stored in float32; one pass adds the
biases, rotates, mixes values and writes queries, keys and values; one launch runs the attention
of all requests of the step.

With ``mix = "weights"`` the heads exchange their weights after each head's own softmax instead:

    p_g[i, j]   = exp(raw_g[i, j]) / (exp(sink_g) + sum_j' exp(raw_g[i, j']))   (visible j'; the sink is optional)
    o_h[i]      = sigmoid(gate_h[i]) * sum_j (sum_g talk[h, g] p_g[i, j]) v_kv(h)[j]    (the gate is optional)

A head's mixed weights are applied to the values of its own key/value head.  The sink is a bare score in a head's
denominator: nothing is read for it and it takes no part in the mixing.  This form may also have ``shared_kv`` (the
unrotated keys double as the values, and there is no tensor ``v``) and rotates neighbouring pairs where the position encoding says so;
its pass in front of the attention is the one that the attention with a sink uses.  The keys are walked
twice (statistics, then weights), because a mixed weight needs every head's finished sum.
"""

from __future__ import annotations

import numpy as np
import torch

from ..config.base import PartSpec
from ..ops import STORE_F32
from .base import Mixer, PagedKVSpec, WeightSpec, build_part, project_out, register_part

ROWS_A_BLOCK = 16      # query rows of a work item of the attention kernel
TILE_KEYS = 32         # keys of a tile of the attention kernel
MAX_RUNS = 16          # the most runs the keys of a row block are dealt to
TILES_A_RUN = 8        # a row block of a prompt portion is cut into runs of at least this many tiles
TILES_A_DECODE_RUN = int(__import__("os").environ.get("LOCKSTEP_TALK_DECODE_TILES", "2"))   # ... of a decoded token


@register_part("talking_attention")
class TalkingAttention(Mixer):
    """Parameters: ``hidden_size``, ``num_heads``, ``num_kv_heads``, ``head_dim`` (queries and keys),
    ``value_dim``, ``position`` (a position-encoding ``PartSpec``), ``window``, ``keep_first``,
    ``scale``, ``bias`` (biases of q, k, v), ``v_mix`` (None, ``"source"`` or ``"mix"``).  Tensors below
    the prefix: ``q``, ``k``, ``v``, ``o``, ``talk`` ``[H, H]``, with ``bias`` also ``q.b``, ``k.b``,
    ``v.b``, with ``v_mix`` also the scalar ``vmix`` (unused by the source layer).
    ``mix`` (``"scores"``, the default, or ``"weights"``); with ``"weights"`` also ``sink`` (None, ``"zero"``
    or ``"learned"``: the tensor ``sink [H]``), ``gate`` (the tensor ``g [H*vdim, hidden]``) and ``shared_kv``
    (no tensor ``v``), and no ``v_mix``."""

    graph_safe = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.nq, self.nkv = int(p["num_heads"]), int(p["num_kv_heads"])
        self.d, self.dv = int(p["head_dim"]), int(p["value_dim"])
        self.window, self.keep_first = int(p["window"]), int(p.get("keep_first") or 0)
        self.scale = float(p["scale"])
        self.bias = bool(p.get("bias"))
        self.v_mix = p.get("v_mix")
        if self.nq % self.nkv:
            raise ValueError(f"{self.nq} query heads are not a multiple of {self.nkv} kv heads")
        if self.window <= 0 or self.keep_first < 0:
            raise ValueError(f"window {self.window} must be positive and keep_first {self.keep_first} not negative")
        if self.v_mix not in (None, "source", "mix"):
            raise ValueError(f"v_mix must be None, 'source' or 'mix', got {self.v_mix!r}")
        self.mix = p.get("mix") or "scores"
        self.sink_kind, self.gate, self.shared_kv = p.get("sink"), bool(p.get("gate")), bool(p.get("shared_kv"))
        if self.mix not in ("scores", "weights"):
            raise ValueError(f"mix must be 'scores' or 'weights', got {self.mix!r}")
        if self.sink_kind not in (None, "zero", "learned"):
            raise ValueError(f"sink must be None, 'zero' or 'learned', got {self.sink_kind!r}")
        if self.mix == "scores" and (self.sink_kind or self.gate or self.shared_kv):
            raise ValueError("a sink, a gate and keys as values come with mix = 'weights'")
        if self.mix == "weights" and self.v_mix is not None:
            raise ValueError("values are mixed across layers with mix = 'scores' only")
        if self.shared_kv and self.d != self.dv:
            raise ValueError(f"keys of {self.d} elements cannot be the values of {self.dv}")
        # (the pass in front of mixed weights pads a head of the queries and the cached keys to 16 bytes' worth)
        self.dk = -(-self.d // 8) * 8 if self.mix == "weights" else self.d
        self.position = build_part(p["position"], prefix)
        if self.position.rotary_dim > self.d:
            raise ValueError(f"rotary_dim {self.position.rotary_dim} exceeds head size {self.d}")
        self.neighbours = bool(getattr(self.position, "neighbours", False))
        if self.neighbours and self.mix == "scores":
            raise ValueError("mix = 'scores' rotates the halves of a head; neighbouring pairs come with mix = 'weights'")
        self.w_qkv = self.w_o = self.b_qkv = self.talk = self.vmix = self.sink = None

    def parts(self):
        return (self.position,)

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        p = spec.params
        h, nq, nkv = int(p["hidden_size"]), int(p["num_heads"]), int(p["num_kv_heads"])
        d, dv = int(p["head_dim"]), int(p["value_dim"])
        out = [WeightSpec(f"{prefix}.q", (nq * d, h)), WeightSpec(f"{prefix}.k", (nkv * d, h)),
               WeightSpec(f"{prefix}.o", (h, nq * dv)),
               WeightSpec(f"{prefix}.talk", (nq, nq), kind="vector", init="identity")]
        if not p.get("shared_kv"):
            out.append(WeightSpec(f"{prefix}.v", (nkv * dv, h)))
        if p.get("gate"):
            out.append(WeightSpec(f"{prefix}.g", (nq * dv, h)))
        if p.get("sink") == "learned":
            out.append(WeightSpec(f"{prefix}.sink", (nq,), kind="vector"))
        if p.get("bias"):
            out += [WeightSpec(f"{prefix}.q.b", (nq * d,), kind="vector"), WeightSpec(f"{prefix}.k.b", (nkv * d,), kind="vector")]
            if not p.get("shared_kv"):
                out.append(WeightSpec(f"{prefix}.v.b", (nkv * dv,), kind="vector"))
        if p.get("v_mix"):
            out.append(WeightSpec(f"{prefix}.vmix", (), kind="vector", init="unit"))
        return out

    def cache_spec(self):
        return PagedKVSpec(self.nkv, self.dk, self.window, value_dim=self.dv, keep_first=self.keep_first)

    def load(self, weights, rt) -> None:
        names = ["q", "k"] + ([] if self.shared_kv else ["v"]) + (["g"] if self.gate else [])
        mats = [weights.get(f"{self.prefix}.{n}") for n in names]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.to(torch.float32) for m in mats]
        self.w_qkv = rt.matrix(torch.cat(mats, dim=0))
        self.w_o = rt.matrix(weights.get(f"{self.prefix}.o"))
        self.talk = rt.vector(weights.get(f"{self.prefix}.talk"))
        if self.bias:
            biased = ["q", "k"] + ([] if self.shared_kv else ["v"])
            self.b_qkv = rt.vector(torch.cat([weights.get(f"{self.prefix}.{n}.b").to(torch.float32) for n in biased]))
        if self.v_mix == "mix":
            self.vmix = rt.vector(weights.get(f"{self.prefix}.vmix").reshape(1))
        if self.sink_kind == "learned":
            self.sink = rt.vector(weights.get(f"{self.prefix}.sink"))
        elif self.sink_kind == "zero":
            self.sink = rt.vector(torch.zeros(self.nq, dtype=torch.float32))
        rt.kernels.mixers_lib()
        rt.kernels.talking_lib(self.nq, self.nkv, self.dk, self.dv)
        if hasattr(self.position, "bind"):
            self.position.bind(rt)

    def mixing_flops(self, tokens: int, start: int) -> float:
        """Scores, their mixing over the heads and value products over the (query, key) pairs a query sees."""
        pairs = sum(min(start + i + 1, self.window + min(self.keep_first, max(0, start + i + 1 - self.window)))
                    for i in range(tokens))
        # (mixed weights walk the keys twice: the scores are formed once more)
        return ((4.0 if self.mix == "weights" else 2.0) * self.d + 2.0 * self.dv + 2.0 * self.nq) * self.nq * pairs

    def prepare_group(self):
        share = getattr(self.position, "share_key", None)
        return None if share is None else ("talking_attention", self.window, self.keep_first, share())

    def _block_key(self):
        return ("talking_attention", "work", self.window, self.keep_first)

    def prepare(self, ctx) -> None:
        """The step's work items, shared by the layers with this window and these kept tokens: (request of the
        step, block of its rows, run, runs), and the fold items of the row blocks that were cut into runs."""
        self.position.ensure(ctx.max_position + 1, ctx.rt)
        key = self._block_key()
        if ctx.declared(key):
            return
        cus = ctx.rt.kernels.compute_units()
        if ctx.single_tokens:
            # one row block a request: deal its visible keys to several items while the GPU has room for them
            # (a number of runs that many steps share: it depends on the number of requests and on a power of
            # two above the longest context only)
            longest = min(int(ctx.kv_len.max()) + ctx.horizon, self.window + self.keep_first)
            tiles = 1 << max(0, (-(-longest // TILE_KEYS) - 1).bit_length())
            runs = max(1, min(MAX_RUNS, (2 * cus) // ctx.n_seqs, tiles // TILES_A_DECODE_RUN))
            seq = np.repeat(np.arange(ctx.n_seqs), runs)
            items = np.stack([seq, np.zeros_like(seq), np.tile(np.arange(runs), ctx.n_seqs), np.full_like(seq, runs)], axis=1)
            rows = np.arange(ctx.n_seqs)            # a request's one row is packed row i
            folds = np.stack([rows * runs, np.full_like(rows, runs), rows, np.ones_like(rows)], axis=1) if runs > 1 else None
            part_rows = 1
        else:
            counts = -(-ctx.q_len // ROWS_A_BLOCK)
            seq = np.repeat(np.arange(ctx.n_seqs), counts)
            block = np.arange(int(counts.sum())) - np.repeat(np.cumsum(counts) - counts, counts)
            first = ctx.q_start[seq] + block * ROWS_A_BLOCK                       # position of a block's first row
            rows = np.minimum(ROWS_A_BLOCK, ctx.q_len[seq] - block * ROWS_A_BLOCK)
            last = first + rows - 1
            # the tiles a block walks: the kept ones below the window's first, then the window's (as the kernel counts)
            lo = np.maximum(0, first - self.window + 1) // TILE_KEYS
            kept = np.minimum(-(-self.keep_first // TILE_KEYS), lo)
            tiles = kept + last // TILE_KEYS - lo + 1
            # runs of at least TILES_A_RUN tiles, longer where the step has more work than a few items a CU
            a_run = max(TILES_A_RUN, -(-int(tiles.sum()) // (4 * cus)))
            runs = np.minimum(MAX_RUNS, np.maximum(1, tiles // a_run))
            item_block = np.repeat(np.arange(len(seq)), runs)
            run = np.arange(int(runs.sum())) - np.repeat(np.cumsum(runs) - runs, runs)
            items = np.stack([seq[item_block], block[item_block], run, runs[item_block]], axis=1)
            cut = runs > 1
            folds = None
            if cut.any():
                first_item = (np.cumsum(runs) - runs)[cut]
                folds = np.stack([first_item, runs[cut], (ctx.q_off[seq] + block * ROWS_A_BLOCK)[cut], rows[cut]], axis=1)
            part_rows = ROWS_A_BLOCK
        n_folds = 0 if folds is None else len(folds)
        ints = items.reshape(-1) if folds is None else np.concatenate([items.reshape(-1), folds.reshape(-1)])
        ctx.declare(key, ints, signature=("talking_attention", len(items), n_folds, part_rows))
        ctx.notes[key] = (len(items), n_folds, part_rows)

    def forward(self, ctx, run, x, out, accumulate: bool, defer: bool = False):
        rt = ctx.rt
        k = rt.kernels
        t = ctx.n_tokens
        nq, nkv, d, dv = self.nq, self.nkv, self.d, self.dv
        group, key_pages, value_pages = ctx.cache.unit_pages(run.cache)
        if not run.writes_cache:
            raise ValueError("a talking-heads attention layer writes its own keys and values")
        if self.mix == "weights":
            return self._forward_mixed_weights(ctx, run, x, out, accumulate, defer)
        raw = ctx.buf("talking.qkv_f32", (t, nq * d + nkv * (d + dv)), torch.float32)
        k.gemm(x, self.w_qkv, raw, STORE_F32)
        q = ctx.buf("talking.q", (t, nq * d), rt.dtype)
        v_first = None
        if self.v_mix is not None:
            # this step's values of the first mixing layer: every token of the step, for the layers that follow
            v_first = ctx.buf("talking.v_first", (t, nkv * dv), torch.float32)
        k.talk_qkv(raw, t, nq, nkv, d, dv, self.b_qkv, self.position.cos, self.position.sin, self.position.rotary_dim,
                   ctx.max_position, ctx.tok_seq, ctx.tok_pos, ctx.seqs, group.table, q, key_pages, value_pages,
                   group.page_size, {None: 0, "source": 1, "mix": 2}[self.v_mix], self.vmix, v_first)
        key = self._block_key()
        attn = ctx.buf("talking.out", (t, nq * dv), rt.dtype)
        n_items, n_folds, part_rows = ctx.notes[key]
        work = ctx.block(key)
        part = ctx.buf("talking.part", (n_items * part_rows * nq * (dv + 2),), torch.float32) if n_folds else None
        k.talk_attention(q, nq, nkv, d, dv, key_pages, value_pages, group.page_size, group.table, ctx.seqs,
                         work[:4 * n_items], n_items, self.talk, self.scale, self.window, self.keep_first, attn,
                         work[4 * n_items:] if n_folds else None, n_folds, part, part_rows)
        return project_out(ctx, attn, self.w_o, out, accumulate, defer, "talking.out_slices")

    def _forward_mixed_weights(self, ctx, run, x, out, accumulate: bool, defer: bool):
        """``mix = "weights"``: the projection (with the gate's logits behind it), the pass that rotates and writes the
        cache, the two passes of the attention, the output projection."""
        rt = ctx.rt
        k = rt.kernels
        t = ctx.n_tokens
        nq, nkv, d, dv = self.nq, self.nkv, self.d, self.dv
        group, key_pages, value_pages = ctx.cache.unit_pages(run.cache)
        raw = ctx.buf("talking.in_f32", (t, self.w_qkv.shape[0]), torch.float32)
        k.gemm(x, self.w_qkv, raw, STORE_F32)
        q = ctx.buf("talking.q", (t, nq * self.dk), rt.dtype)
        k.qkv_post(raw, t, nq, nkv, d, dv, self.b_qkv, None, None, 0.0, self.position.cos, self.position.sin,
                   self.position.rotary_dim, self.neighbours, ctx.max_position, ctx.tok_seq, ctx.tok_pos, ctx.seqs,
                   group.table, q, key_pages, value_pages, group.page_size, keys_are_values=self.shared_kv,
                   key_pad=self.dk)
        key = self._block_key()
        attn = ctx.buf("talking.out", (t, nq * dv), rt.dtype)
        n_items, n_folds, part_rows = ctx.notes[key]
        work = ctx.block(key)
        part = ctx.buf("talking.part", (n_items * part_rows * nq * (dv + 2),), torch.float32) if n_folds else None
        stats = ctx.buf("talking.stats", (n_items * 16 * nq * 2,), torch.float32)
        gate = raw[:, raw.shape[1] - nq * dv:] if self.gate else None
        k.talk_attention(q, nq, nkv, self.dk, dv, key_pages, value_pages, group.page_size, group.table, ctx.seqs,
                         work[:4 * n_items], n_items, self.talk, self.scale, self.window, self.keep_first, attn,
                         work[4 * n_items:] if n_folds else None, n_folds, part, part_rows, mix_weights=True,
                         sink=self.sink, stats=stats, gate=gate)
        return project_out(ctx, attn, self.w_o, out, accumulate, defer, "talking.out_slices")
