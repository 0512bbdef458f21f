"""Attention whose keys and values are projections of one small latent a token, which is all the
cache holds; the softmax has a sink, the mask a window.

For a token with input ``h`` at position ``p``:

    a  = rmsnorm(W_dq h) * w_dq                 the query latent                       [q_rank]
    q  = W_uq a                                  per head: ``dim`` plain dimensions, then ``rot_dim`` rotated ones
    (c_raw | r_raw) = W_dkv h                    [kv_rank + rot_dim]
    c  = rmsnorm(c_raw) * w_dkv                 the latent: cached
    r  = rotate(r_raw, p)                        one key part shared by all heads: cached
    head n:  k_n = (W_uk,n c | r),  v_n = W_uv,n c
    s_n[i, j] = scale * (q_plain,n[i] . W_uk,n c[j]  +  rotate(q_rot,n[i], i) . r[j])

The products with ``W_uk`` and ``W_uv`` are moved to the query's side, so that no key or value of a
head is ever formed: with ``q'_n = W_uk,n^T q_plain,n`` the score is ``q'_n . c + q_rot,n . r``, which is
attention with one key/value head whose keys are ``(c | r)`` and whose values are ``c``, over ``H``
query heads of ``kv_rank + rot_dim`` elements; the head's output in the latent's space, ``sum_j p_j
c[j]``, is then multiplied by ``W_uv,n``.  The attention itself is the sink attention kernel
(csrc/sink_attention.hip); ``q'`` and the outputs are one launch each of a product a head.

A layer with ``kv_from`` has no ``W_dkv``: it reads the cache unit that another such layer writes
(same latent size, same shared key part, same rotation) with its own ``W_uk``, ``W_uv``, queries,
mask and sink.
"""

from __future__ import annotations

import torch

from ..config.base import PartSpec
from ..ops import STORE_F32
from .base import PagedKVSpec, WeightSpec, project_out, register_part
from .sink_attention import STAGED, SinkAttention


@register_part("latent_attention")
class LatentAttention(SinkAttention):
    """Parameters: ``hidden_size``, ``num_heads``, ``head_dim`` (plain dimensions of a query/key head),
    ``rot_dim`` (rotated ones), ``value_dim``, ``q_rank``, ``kv_rank``, ``eps`` (of the latents' norms),
    ``position`` (a position-encoding ``PartSpec`` over ``rot_dim`` elements, neighbouring pairs),
    ``scale``, ``window`` (None or a size), ``sink`` (None, ``"zero"`` or ``"learned"``), ``reads_other``
    (True for a layer that uses another layer's cache unit), ``cache_window`` (the window the cache
    unit keeps: the largest of the layers that read it; None: everything).
    Tensors below the prefix: ``dq`` ``[q_rank, hidden]``, ``dq.norm``, ``uq`` ``[H*(dim+rot_dim), q_rank]``,
    ``dkv`` ``[kv_rank+rot_dim, hidden]``, ``dkv.norm``, ``uk`` ``[H*dim, kv_rank]``, ``uv`` ``[H*vdim,
    kv_rank]``, ``sink [H]``, ``o`` ``[hidden, H*vdim]``."""

    graph_safe = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        p = spec.params
        self.plain_dim, self.rot_dim = int(p["head_dim"]), int(p["rot_dim"])
        self.q_rank, self.kv_rank = int(p["q_rank"]), int(p["kv_rank"])
        self.out_dim = int(p["value_dim"])
        self.eps = float(p["eps"])
        self.reads_other = bool(p.get("reads_other"))
        self.cache_window = p.get("cache_window")
        if min(self.plain_dim, self.q_rank, self.kv_rank, self.out_dim) <= 0 or self.rot_dim < 0:
            raise ValueError("the sizes of attention over a latent must be positive")
        # the attention as the kernel sees it: one key/value head (c | r), values c
        super().__init__(PartSpec(spec.kind, {
            "hidden_size": p["hidden_size"], "num_heads": p["num_heads"], "num_kv_heads": 1,
            "head_dim": self.kv_rank + self.rot_dim, "value_dim": self.kv_rank, "position": p["position"],
            "scale": p["scale"], "window": p.get("window"), "sink": p.get("sink")}), prefix)
        self.spec = spec
        if self.position.rotary_dim > self.rot_dim:
            raise ValueError(f"{self.position.rotary_dim} rotated dimensions exceed rot_dim {self.rot_dim}")
        if self.position.rotary_dim and not self.neighbours:
            raise ValueError("the shared key part is rotated in neighbouring pairs")
        self.w_down = self.w_uq = self.w_uk = self.w_uv = self.q_weight = self.kv_weight = None

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        p = spec.params
        h, n, d, r, dv = int(p["hidden_size"]), int(p["num_heads"]), int(p["head_dim"]), int(p["rot_dim"]), int(p["value_dim"])
        qr, cr = int(p["q_rank"]), int(p["kv_rank"])
        out = [WeightSpec(f"{prefix}.dq", (qr, h)), WeightSpec(f"{prefix}.dq.norm", (qr,), kind="vector", init="norm"),
               WeightSpec(f"{prefix}.uq", (n * (d + r), qr))]
        if not p.get("reads_other"):
            out += [WeightSpec(f"{prefix}.dkv", (cr + r, h)), WeightSpec(f"{prefix}.dkv.norm", (cr,), kind="vector", init="norm")]
        out += [WeightSpec(f"{prefix}.uk", (n * d, cr)), WeightSpec(f"{prefix}.uv", (n * dv, cr)),
                WeightSpec(f"{prefix}.o", (h, n * dv))]
        if p.get("sink") == "learned":
            out.append(WeightSpec(f"{prefix}.sink", (n,), kind="vector"))
        return out

    def cache_spec(self):
        return PagedKVSpec(1, self.dk, self.cache_window, value_dim=self.kv_rank)

    def load(self, weights, rt) -> None:
        get = lambda name: weights.get(f"{self.prefix}.{name}")  # noqa: E731
        down = [get("dq")] + ([] if self.reads_other else [get("dkv")])
        if len({m.dtype for m in down}) > 1:
            down = [m.to(torch.float32) for m in down]
        self.w_down = rt.matrix(torch.cat(down, dim=0))
        self.w_uq = rt.matrix(get("uq"))
        n, d, cr = self.nq, self.plain_dim, self.kv_rank
        # W_uk,n^T [kv_rank, dim] a head: the operand of q' = W_uk,n^T q_plain,n;  W_uv,n [vdim, kv_rank] as stored
        self.w_uk = rt.matrix(get("uk").reshape(n, d, cr).transpose(1, 2).contiguous())
        self.w_uv = rt.matrix(get("uv").reshape(n, self.out_dim, cr).contiguous())
        self.w_o = rt.matrix(get("o"))
        self.q_weight = rt.vector(get("dq.norm"))
        if not self.reads_other:
            self.kv_weight = rt.vector(get("dkv.norm"))
        if self.sink_kind == "learned":
            self.sink = rt.vector(get("sink"))
        elif self.sink_kind == "zero":
            self.sink = rt.vector(torch.zeros(self.nq, dtype=torch.float32))
        rt.kernels.mixers_lib()
        rt.kernels.sink_lib(self.dk, self.kv_rank)
        if hasattr(self.position, "bind"):
            self.position.bind(rt)

    def mixing_flops(self, tokens: int, start: int) -> float:
        pairs = sum(self._seen(start + i) for i in range(tokens))
        per_token = 2.0 * self.nq * self.kv_rank * (self.plain_dim + self.out_dim)     # the products a head
        return (2.0 * self.dk + 2.0 * self.kv_rank) * self.nq * pairs + per_token * tokens

    def forward(self, ctx, run, x, out, accumulate: bool, defer: bool = False):
        rt = ctx.rt
        k = rt.kernels
        t = ctx.n_tokens
        n, d, r, cr, dk = self.nq, self.plain_dim, self.rot_dim, self.kv_rank, self.dk
        if run.writes_cache == self.reads_other:
            raise ValueError("a layer over a latent writes its cache unit exactly when it has a projection into it")
        group, key_pages, value_pages = ctx.cache.unit_pages(run.cache)
        raw = ctx.buf("latent.down_f32", (t, self.w_down.shape[0]), torch.float32)
        k.gemm(x, self.w_down, raw, STORE_F32)
        q_latent = ctx.buf("latent.q_latent", (t, self.q_rank), rt.dtype)
        k.latent_post(raw, t, self.q_rank, cr, r, dk, not self.reads_other, self.q_weight, self.kv_weight, self.eps,
                      self.position.cos, self.position.sin, self.position.rotary_dim, ctx.max_position, ctx.tok_seq,
                      ctx.tok_pos, ctx.seqs, group.table, q_latent, key_pages, value_pages, group.page_size)
        qf = ctx.buf("latent.q_f32", (t, n * (d + r)), torch.float32)
        k.gemm(q_latent, self.w_uq, qf, STORE_F32)
        plain = ctx.buf("latent.q_plain", (t, n * d), rt.dtype)
        q = ctx.buf("latent.q", (t, n * dk), rt.dtype)
        k.latent_query(qf, t, n, d, r, cr, dk, self.position.cos, self.position.sin, self.position.rotary_dim,
                       ctx.max_position, ctx.tok_pos, plain, q)
        k.heads_product(plain, d, self.w_uk, q, dk)
        key = self._block_key()
        mixed = ctx.buf("latent.mixed", (t, n * cr), rt.dtype)
        n_items, n_folds, row_tiles = ctx.notes[key]
        work = ctx.block(key)
        part_rows = k.sink_staged_rows(n, 1) if row_tiles == STAGED else 16 * row_tiles if row_tiles else 1
        part = ctx.buf("sink.part", (n_items * part_rows * n * (cr + 2),), torch.float32) if n_folds else None
        k.sink_attention(q, n, 1, dk, cr, key_pages, value_pages, group.page_size, group.table, ctx.seqs,
                         work[:4 * n_items], n_items, row_tiles, self.scale, self.window, 0, self.sink, None, None, mixed,
                         work[4 * n_items:] if n_folds else None, n_folds, part)
        heads_out = ctx.buf("latent.heads_out", (t, n * self.out_dim), rt.dtype)
        k.heads_product(mixed, cr, self.w_uv, heads_out, self.out_dim)
        return project_out(ctx, heads_out, self.w_o, out, accumulate, defer, "latent.out_slices")
