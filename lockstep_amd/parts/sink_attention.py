"""Grouped-query attention over the paged cache whose softmax has a sink, with the choices that
decoders of this family make layer by layer.

For the step's queries ``q_h`` (head h of H) and the cached keys ``k_g`` / values ``v_g`` (head g of G,
query head h reads kv head ``h // (H/G)``), at true positions i (query) and j (key):

    s_h[i, j] = scale * <q_h[i], k_kv(h)[j]> + rel[bucket(i - j), h]            (the bias is optional)
    j is visible to i  iff  lo(i) <= j <= i, where lo(i) is 0, i - window + 1, or the start of i's chunk
                            (with a window, also if j < keep_first: the first tokens stay visible)
    p_h[i, j] = exp(s_h[i, j]) / (exp(sink_h) + sum_j' exp(s_h[i, j']))         (sink: none, zero, or learned)
    o_h[i]    = sigmoid(g_h[i]) * sum_j p_h[i, j] v_kv(h)[j]                    (the gate is optional)

``bucket``: a table of B rows serves all distances; the first B/2 rows are the distances 0 .. B/2 - 1
themselves, the others are spaced evenly in the logarithm of the distance up to ``farthest``, beyond
which everything shares the last row: ``min(B - 1, B/2 + floor(ln(n / (B/2)) / ln(farthest / (B/2)) *
(B - B/2)))``.  The part turns the table into one row a head indexed by the distance itself (up to
the first distance of the last bucket), so that the kernel needs no logarithm.

Before the attention: one matrix product over ``[Wq; Wk; (Wv;) Wg]`` stored in float32, then one pass
that adds biases, applies a root-mean-square norm over the whole of q and of k (``qk_norm``), rotates,
and writes queries, keys and values; with ``shared_kv`` there is no value projection and the values
are the keys as projected (biased, before the norm).  The gate logits stay in the product's float32
rows, where the attention kernel reads them.
"""

from __future__ import annotations

import math

import numpy as np
import torch

from ..config.base import PartSpec
from ..ops import STORE_F32
from .base import Mixer, PagedKVSpec, WeightSpec, build_part, project_out, register_part

TILE_KEYS = 32         # keys of a tile of the attention kernel
MAX_RUNS = 16          # the most runs the keys of a row block are dealt to
TILES_A_RUN = 8        # a row block of a prompt portion is cut into runs of at least this many tiles
TILES_A_DECODE_RUN = 2  # ... of a decoded token
ROW_TILES = int(__import__("os").environ.get("LOCKSTEP_SINK_ROW_TILES", "0"))   # 0: chosen by the step's size
STAGED = 8             # the value of row_tiles that names the kernel with tiles staged in LDS


def distance_buckets(rows: int, farthest: float) -> list[int]:
    """``bucket(n)`` for n = 0 .. the first distance of the last bucket."""
    half = rows // 2
    out = []
    n = 0
    while True:
        if n < half:
            b = n
        else:
            b = min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(farthest / half) * (rows - half))))
        out.append(b)
        if b >= rows - 1:
            return out
        n += 1


@register_part("sink_attention")
class SinkAttention(Mixer):
    """Parameters: ``hidden_size``, ``num_heads``, ``num_kv_heads``, ``head_dim`` (queries and keys),
    ``value_dim``, ``position`` (a position-encoding ``PartSpec``), ``scale``, ``window`` / ``chunk``
    (None or a size; at most one of them), ``keep_first`` (with a window: the first that many tokens stay visible), ``sink`` (None, ``"zero"`` or ``"learned"``), ``gate``,
    ``bias`` (biases of q, k, v), ``out_bias``, ``qk_norm`` (None or the eps of a norm over the whole
    projection), ``head_norm`` (None or the eps of a norm over every head of q and of k; without weights, or with ``head_norm_weights`` times
    ``q.norm`` / ``k.norm`` of ``head_dim`` elements that all heads share), ``shared_kv`` (the values are the keys as projected), ``distance_bias`` (None or
    ``{"farthest": D, "rows": B}``; ``rows`` only sizes random weights, a checkpoint's table says it itself).
    Tensors below the prefix: ``q``, ``k``, ``v``, ``o``; ``g`` (gate); ``q.b``, ``k.b``, ``v.b``;
    ``o.b``; ``q.norm``, ``k.norm``; ``rel [B, H]``; ``sink [H]``."""

    graph_safe = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.nq, self.nkv = int(p["num_heads"]), int(p["num_kv_heads"])
        self.d, self.dv = int(p["head_dim"]), int(p["value_dim"])
        self.dk = -(-self.d // 8) * 8       # a head of the queries and of the cached keys: the kernel loads 16 bytes at a time
        self.scale = float(p["scale"])
        self.window = int(p.get("window") or 0)
        self.chunk = int(p.get("chunk") or 0)
        self.keep_first = int(p.get("keep_first") or 0)
        self.sink_kind = p.get("sink")
        self.gate = bool(p.get("gate"))
        self.bias = bool(p.get("bias"))
        self.out_bias = bool(p.get("out_bias"))
        self.qk_norm = None if p.get("qk_norm") is None else float(p["qk_norm"])
        self.head_norm = None if p.get("head_norm") is None else float(p["head_norm"])
        if self.qk_norm is not None and self.head_norm is not None:
            raise ValueError("a norm over the whole projection and a norm over every head: at most one")
        self.head_norm_weights = bool(p.get("head_norm_weights"))
        if self.head_norm_weights and self.head_norm is None:
            raise ValueError("head_norm_weights belong to a head_norm")
        if self.keep_first < 0 or (self.keep_first and not self.window):
            raise ValueError(f"keep_first {self.keep_first} must not be negative and needs a window")
        self.shared_kv = bool(p.get("shared_kv"))
        self.distance_bias = p.get("distance_bias")
        if self.nq % self.nkv:
            raise ValueError(f"{self.nq} query heads are not a multiple of {self.nkv} kv heads")
        if self.window < 0 or self.chunk < 0 or (self.window and self.chunk):
            raise ValueError(f"window {self.window} and chunk {self.chunk}: at most one, and not negative")
        if self.sink_kind not in (None, "zero", "learned"):
            raise ValueError(f"sink must be None, 'zero' or 'learned', got {self.sink_kind!r}")
        if self.shared_kv and self.d != self.dv:
            raise ValueError(f"keys of {self.d} elements cannot be the values of {self.dv}")
        if self.distance_bias is not None and not float(self.distance_bias["farthest"]) > 1:
            raise ValueError("distance_bias.farthest must exceed 1")
        self.position = build_part(p["position"], prefix)
        if self.position.rotary_dim > self.d:
            raise ValueError(f"rotary_dim {self.position.rotary_dim} exceeds head size {self.d}")
        self.neighbours = bool(getattr(self.position, "neighbours", False))
        self.w_in = self.w_o = self.b_in = self.b_o = self.q_norm = self.k_norm = self.sink = self.by_distance = None

    def parts(self):
        return (self.position,)

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        p = spec.params
        h, nq, nkv = int(p["hidden_size"]), int(p["num_heads"]), int(p["num_kv_heads"])
        d, dv = int(p["head_dim"]), int(p["value_dim"])
        out = [WeightSpec(f"{prefix}.q", (nq * d, h)), WeightSpec(f"{prefix}.k", (nkv * d, h)),
               WeightSpec(f"{prefix}.o", (h, nq * dv))]
        if not p.get("shared_kv"):
            out.append(WeightSpec(f"{prefix}.v", (nkv * dv, h)))
        if p.get("gate"):
            out.append(WeightSpec(f"{prefix}.g", (nq * dv, h)))
        if p.get("bias"):
            out += [WeightSpec(f"{prefix}.q.b", (nq * d,), kind="vector"), WeightSpec(f"{prefix}.k.b", (nkv * d,), kind="vector")]
            if not p.get("shared_kv"):
                out.append(WeightSpec(f"{prefix}.v.b", (nkv * dv,), kind="vector"))
        if p.get("out_bias"):
            out.append(WeightSpec(f"{prefix}.o.b", (h,), kind="vector"))
        if p.get("qk_norm") is not None:
            out += [WeightSpec(f"{prefix}.q.norm", (nq * d,), kind="vector", init="norm"),
                    WeightSpec(f"{prefix}.k.norm", (nkv * d,), kind="vector", init="norm")]
        if p.get("head_norm") is not None and p.get("head_norm_weights"):
            out += [WeightSpec(f"{prefix}.q.norm", (d,), kind="vector", init="norm"),
                    WeightSpec(f"{prefix}.k.norm", (d,), kind="vector", init="norm")]
        if p.get("distance_bias") is not None:
            out.append(WeightSpec(f"{prefix}.rel", (-1, nq), kind="vector", free=int(p["distance_bias"].get("rows") or 32)))
        if p.get("sink") == "learned":
            out.append(WeightSpec(f"{prefix}.sink", (nq,), kind="vector"))
        return out

    def cache_spec(self):
        return PagedKVSpec(self.nkv, self.dk, self.window or None, value_dim=self.dv, chunk=self.chunk or None,
                           keep_first=self.keep_first)

    def load(self, weights, rt) -> None:
        names = ["q", "k"] + ([] if self.shared_kv else ["v"]) + (["g"] if self.gate else [])
        mats = [weights.get(f"{self.prefix}.{n}") for n in names]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.to(torch.float32) for m in mats]
        self.w_in = rt.matrix(torch.cat(mats, dim=0))
        self.w_o = rt.matrix(weights.get(f"{self.prefix}.o"))
        if self.bias:
            biased = ["q", "k"] + ([] if self.shared_kv else ["v"])
            self.b_in = rt.vector(torch.cat([weights.get(f"{self.prefix}.{n}.b").to(torch.float32) for n in biased]))
        if self.out_bias:
            self.b_o = rt.vector(weights.get(f"{self.prefix}.o.b"))
        if self.qk_norm is not None or self.head_norm_weights:
            self.q_norm = rt.vector(weights.get(f"{self.prefix}.q.norm"))
            self.k_norm = rt.vector(weights.get(f"{self.prefix}.k.norm"))
        if self.sink_kind == "learned":
            self.sink = rt.vector(weights.get(f"{self.prefix}.sink"))
        elif self.sink_kind == "zero":
            self.sink = rt.vector(torch.zeros(self.nq, dtype=torch.float32))
        if self.distance_bias is not None:
            table = weights.get(f"{self.prefix}.rel").to(torch.float32)            # [B, H]
            if table.dim() != 2 or table.shape[0] < 2 or float(self.distance_bias["farthest"]) <= table.shape[0] // 2:
                raise ValueError(f"{self.prefix}.rel must have at least two rows and its farthest distance must lie beyond "
                                 f"the first half of them, got {tuple(table.shape)} and {self.distance_bias['farthest']}")
            rows = distance_buckets(table.shape[0], float(self.distance_bias["farthest"]))
            self.by_distance = rt.vector(table[torch.tensor(rows)].T.contiguous())   # [H, distances]
        rt.kernels.mixers_lib()
        rt.kernels.sink_lib(self.dk, self.dv)
        if hasattr(self.position, "bind"):
            self.position.bind(rt)

    def _seen(self, position: int) -> int:
        """Keys that a query at ``position`` sees."""
        lo = 0
        if self.window:
            lo = max(lo, position - self.window + 1)
        if self.chunk:
            lo = max(lo, position // self.chunk * self.chunk)
        return position - lo + 1 + min(self.keep_first, lo)

    def mixing_flops(self, tokens: int, start: int) -> float:
        pairs = sum(self._seen(start + i) for i in range(tokens))
        return (2.0 * self.d + 2.0 * self.dv) * self.nq * pairs

    def prepare_group(self):
        share = getattr(self.position, "share_key", None)
        return None if share is None else ("sink_attention", self.window, self.chunk, self.keep_first, self.nq, self.nkv,
                                           self.dk, self.dv, share())

    def _block_key(self):
        # (the blocks of rows and the tiles of keys depend on the heads and the sizes as well)
        return ("sink_attention", "work", self.window, self.chunk, self.keep_first, self.nq, self.nkv, self.dk, self.dv)

    def _first_seen(self, positions):
        lo = np.zeros_like(positions)
        if self.window:
            lo = np.maximum(lo, positions - self.window + 1)
        if self.chunk:
            lo = np.maximum(lo, positions // self.chunk * self.chunk)
        return lo

    def prepare(self, ctx) -> None:
        """The step's work items, shared by the layers with this window or chunk: (request of the step, block
        of its rows, run, runs), and the fold items of the row blocks that were cut into runs."""
        self.position.ensure(ctx.max_position + 1, ctx.rt)
        key = self._block_key()
        if ctx.declared(key):
            return
        cus = ctx.rt.kernels.compute_units()
        groups = self.nkv
        if ctx.single_tokens:
            # one row block a request: deal its visible keys to several items while the GPU has room for them
            # (a number of runs that many steps share: it depends on the number of requests and on a power of
            # two above the longest context only)
            longest = int(ctx.kv_len.max()) + ctx.horizon
            if self.window:
                longest = min(longest, self.window + self.keep_first)
            if self.chunk:
                longest = min(longest, self.chunk)
            tiles = 1 << max(0, (-(-longest // TILE_KEYS) - 1).bit_length())
            runs = max(1, min(MAX_RUNS, (2 * cus) // max(1, ctx.n_seqs * groups), tiles // TILES_A_DECODE_RUN))
            seq = np.repeat(np.arange(ctx.n_seqs), runs)
            items = np.stack([seq, np.zeros_like(seq), np.tile(np.arange(runs), ctx.n_seqs), np.full_like(seq, runs)], axis=1)
            rows = np.arange(ctx.n_seqs)            # a request's one row is packed row i
            folds = np.stack([rows * runs, np.full_like(rows, runs), rows, np.ones_like(rows)], axis=1) if runs > 1 else None
            row_tiles = 0
        else:
            longest_portion = int(ctx.q_len.max())
            kernels = ctx.rt.kernels
            page = ctx.cache.page_size
            staged_keys = kernels.sink_staged_keys(self.dk, self.dv, ctx.rt.dtype)
            # portions of more than 16 tokens: tiles staged in LDS where the sizes fit; else fragments straight from
            # global memory, two row tiles a wave (one for short portions; four remain for measurements)
            if ROW_TILES:
                row_tiles = ROW_TILES
            elif longest_portion <= 16:
                row_tiles = 1
            elif staged_keys and page % (8 if ctx.rt.dtype == torch.bfloat16 else 4) == 0:
                row_tiles = STAGED
            else:
                row_tiles = 2
            block_rows = kernels.sink_staged_rows(self.nq, self.nkv) if row_tiles == STAGED else 16 * row_tiles
            tile_keys = staged_keys if row_tiles == STAGED else TILE_KEYS
            counts = -(-ctx.q_len // block_rows)
            seq = np.repeat(np.arange(ctx.n_seqs), counts)
            block = np.arange(int(counts.sum())) - np.repeat(np.cumsum(counts) - counts, counts)
            first = ctx.q_start[seq] + block * block_rows                          # position of a block's first row
            rows = np.minimum(block_rows, ctx.q_len[seq] - block * block_rows)
            last = first + rows - 1
            lo_tile = self._first_seen(first) // tile_keys
            tiles = last // tile_keys - lo_tile + 1 + np.minimum(-(-self.keep_first // tile_keys), lo_tile)    # (as the kernel counts them)
            # runs of at least TILES_A_RUN tiles of 32 keys, longer where the step has more work than a few items a CU
            a_run = max(TILES_A_RUN * TILE_KEYS // tile_keys, -(-int(tiles.sum()) * groups // (4 * cus)))
            runs = np.minimum(MAX_RUNS, np.maximum(1, tiles // a_run))
            item_block = np.repeat(np.arange(len(seq)), runs)
            run = np.arange(int(runs.sum())) - np.repeat(np.cumsum(runs) - runs, runs)
            items = np.stack([seq[item_block], block[item_block], run, runs[item_block]], axis=1)
            cut = runs > 1
            folds = None
            if cut.any():
                first_item = (np.cumsum(runs) - runs)[cut]
                folds = np.stack([first_item, runs[cut], (ctx.q_off[seq] + block * block_rows)[cut], rows[cut]], axis=1)
        n_folds = 0 if folds is None else len(folds)
        ints = items.reshape(-1) if folds is None else np.concatenate([items.reshape(-1), folds.reshape(-1)])
        ctx.declare(key, ints, signature=("sink_attention", len(items), n_folds, row_tiles))
        ctx.notes[key] = (len(items), n_folds, row_tiles)

    def forward(self, ctx, run, x, out, accumulate: bool, defer: bool = False):
        rt = ctx.rt
        k = rt.kernels
        t = ctx.n_tokens
        nq, nkv, d, dv = self.nq, self.nkv, self.d, self.dv
        group, key_pages, value_pages = ctx.cache.unit_pages(run.cache)
        if not run.writes_cache:
            raise ValueError("a sink attention layer writes its own keys and values")
        raw = ctx.buf("sink.in_f32", (t, self.w_in.shape[0]), torch.float32)
        k.gemm(x, self.w_in, raw, STORE_F32)
        q = ctx.buf("sink.q", (t, nq * self.dk), rt.dtype)
        k.qkv_post(raw, t, nq, nkv, d, dv, self.b_in, self.q_norm, self.k_norm, self.qk_norm or self.head_norm or 0.0, self.position.cos,
                   self.position.sin, self.position.rotary_dim, self.neighbours, ctx.max_position, ctx.tok_seq,
                   ctx.tok_pos, ctx.seqs, group.table, q, key_pages, value_pages, group.page_size,
                   keys_are_values=self.shared_kv, key_pad=self.dk, per_head=self.head_norm is not None,
                   head_weights=self.head_norm_weights)
        key = self._block_key()
        attn = ctx.buf("sink.out", (t, nq * dv), rt.dtype)
        n_items, n_folds, row_tiles = ctx.notes[key]
        work = ctx.block(key)
        part_rows = k.sink_staged_rows(nq, nkv) if row_tiles == STAGED else 16 * row_tiles if row_tiles else 1
        part = ctx.buf("sink.part", (n_items * part_rows * nq * (dv + 2),), torch.float32) if n_folds else None
        gate = raw[:, raw.shape[1] - nq * dv:] if self.gate else None
        k.sink_attention(q, nq, nkv, self.dk, dv, key_pages, value_pages, group.page_size, group.table, ctx.seqs,
                         work[:4 * n_items], n_items, row_tiles, self.scale, self.window, self.chunk, self.sink,
                         self.by_distance, gate, attn, work[4 * n_items:] if n_folds else None, n_folds, part,
                         keep_first=self.keep_first)
        if self.b_o is not None:
            # (a product with an output bias is added to the stream at once, then the bias: the same order
            # of additions at every batch size)
            from ..ops import ADD_F32

            k.gemm(attn, self.w_o, out, ADD_F32 if accumulate else STORE_F32)
            k.bias_act(out, self.b_o, out)
            return None
        return project_out(ctx, attn, self.w_o, out, accumulate, defer, "sink.out_slices")
