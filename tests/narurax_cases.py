"""Small Narurax configurations and weights for the tests.  The configurations differ from each other in
every size and option: the order of the layers, heads (grouped, as many key/value heads as query heads,
sixteen on one, a single head whose mixing matrix is one number), key and value sizes (equal and unequal,
no multiples of 16 or of 8), windows (shorter than a page, no multiple of a page or of a key tile, longer
than any sequence), kept first tokens (none, fewer and more than the window holds), rotation of a whole
head or of a part, with and without stretched frequencies, convolutions of two to five taps (and of one:
none), bottlenecks of several ranks, experts (one a token, several, all, a single expert), layers without a
feed-forward, tables of pairs of several sizes with multipliers that are zero, one or large."""

from __future__ import annotations

import json

import torch


def mixing(heads, kv_heads, dim, window, keep_first, scale, dims=None, base=10000.0):
    """``attention``: weights mixed over the heads, a sink, a gate; the values are the keys."""
    return {"type": "attention", "mixer": {
        "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale,
        "mask": {"size": window, "keep_first": keep_first}, "rot": {"dims": dim if dims is None else dims, "base": base}}}


def normed(heads, kv_heads, dim, vdim, window, keep_first, scale, dims=None, base=10000.0, scaling=None):
    """``attention_2``: biases, a norm a head, a one in the denominator."""
    rot = {"dims": dim if dims is None else dims, "base": base}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return {"type": "attention_2", "mixer": {
        "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
        "mask": {"size": window, "keep_first": keep_first}, "rot": rot}}


def delta(heads, kv_heads, dim, vdim, taps):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps}}


def routed(layer, ff, experts, top):
    return dict(layer, mlp={"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}})


def bare(layer):
    return dict(layer, mlp=None)


def config(width, vocab, layers, buckets=61, mul_prev=31, mul_cur=5, eps=1e-5):
    return {"architecture": "Narurax", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}, "layers": layers}


#: ranks of the bottlenecks (decay, gate) of a layer's delta mixer, by (case, layer); others take RANKS_DEFAULT
RANKS_DEFAULT = (6, 10)

CASES = {
    # every mixer; windows of 21 and 13 on pages of 8 with 3 and 5 kept tokens; a part of the head rotated;
    # stretched frequencies with all three ranges; a layer without a feed-forward
    "A": dict(page_size=8, ranks={0: (5, 12)}, raw=config(64, 128, [
        routed(delta(4, 2, 24, 16, taps=3), 32, experts=6, top=2),
        routed(mixing(4, 2, 24, window=21, keep_first=3, scale=0.3, dims=16, base=100.0), 24, experts=5, top=1),
        routed(normed(4, 2, 16, 40, window=13, keep_first=5, scale=0.4, base=100.0, scaling=(8.0, 1.0, 4.0, 64)), 32,
               experts=6, top=2),
        bare(normed(4, 2, 16, 40, window=50, keep_first=0, scale=0.4, base=100.0, scaling=(8.0, 1.0, 4.0, 64))),
    ])),
    # as many key/value heads as query heads and a window longer than any sequence; a delta layer of two taps
    # without a feed-forward; six heads on one key/value head, more kept tokens than the window holds, a key size
    # that is no multiple of 8; all experts for every token; multipliers 1 and 0
    "B": dict(page_size=16, ranks={1: (9, 3)}, raw=config(96, 200, [
        routed(normed(3, 3, 40, 24, window=1000, keep_first=0, scale=0.25, dims=8, base=500.0), 48, experts=3, top=3),
        bare(delta(2, 2, 40, 24, taps=2)),
        routed(mixing(6, 1, 12, window=7, keep_first=9, scale=0.5), 16, experts=9, top=4),
    ], buckets=7, mul_prev=1, mul_cur=0, eps=1e-6)),
    # a single head whose mixing matrix is one number; sixteen heads on one key/value head with a window shorter
    # than a page; a delta head with a wide value and five taps, another with one tap (no convolution); a single
    # expert; large multipliers
    "C": dict(page_size=16, ranks={}, raw=config(32, 64, [
        routed(mixing(1, 1, 16, window=11, keep_first=2, scale=0.6), 16, experts=2, top=1),
        routed(delta(1, 1, 16, 72, taps=5), 16, experts=4, top=2),
        bare(normed(16, 1, 16, 8, window=5, keep_first=1, scale=0.9)),
        routed(delta(3, 1, 8, 8, taps=1), 8, experts=1, top=1),
    ], buckets=1000, mul_prev=100003, mul_cur=7919)),
}

SINGLE = {
    "mixing": dict(page_size=8, ranks={}, raw=config(64, 96, [bare(mixing(4, 2, 24, window=20, keep_first=4, scale=0.5, dims=16))])),
    "normed": dict(page_size=8, ranks={}, raw=config(64, 96, [
        bare(normed(4, 2, 16, 40, window=26, keep_first=3, scale=0.5, scaling=(4.0, 1.0, 8.0, 32)))])),
    "delta": dict(page_size=8, ranks={}, raw=config(64, 96, [bare(delta(4, 2, 24, 16, taps=4))])),
    "routed": dict(page_size=8, ranks={}, raw=config(64, 96, [routed(normed(3, 3, 40, 24, window=1000, keep_first=0, scale=0.3), 40,
                                                                    experts=7, top=3)])),
}


def make_tensors(raw: dict, seed: int, spread: float = 1.0, ranks=None) -> dict:
    """Random bfloat16 weights for ``raw`` through the package's seeded random-weights mode, then: the bottlenecks take
    the ranks of the case, sinks, biases, the decay's parameters and the shifts are drawn wide enough to matter, the
    convolutions' taps around zero, the mixing matrices well away from the identity, and the matrices into the delta
    rule's gates larger (decays and step sizes that differ from token to token and from channel to channel)."""
    from lockstep_amd.config import config_from_dict
    from lockstep_amd.weights import random_tensors

    cfg = config_from_dict(raw)
    tensors = random_tensors(cfg, seed, std=0.08 * spread, norm_std=0.2, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(seed + 1000)

    def draw(name, width, centre=0.0, shape=None):
        if name in tensors:
            shape = tensors[name].shape if shape is None else shape
            tensors[name] = (centre + torch.randn(shape, generator=g) * width).to(torch.bfloat16)

    for i, layer in enumerate(raw["layers"]):
        p = f"l{i}.mix"
        if layer["type"] == "channel_delta":
            m = layer["mixer"]
            decay_rank, gate_rank = (ranks or {}).get(i, RANKS_DEFAULT)
            draw(f"{p}.a1", 0.3, shape=(decay_rank, raw["width"]))
            draw(f"{p}.a2", 0.8, shape=(m["heads"] * m["dim"], decay_rank))
            draw(f"{p}.g1", 0.3, shape=(gate_rank, raw["width"]))
            draw(f"{p}.g2", 0.8, shape=(m["heads"] * m["vdim"], gate_rank))
        draw(f"{p}.sink", 1.5)
        for name in ("q.b", "k.b", "v.b", "o.b"):
            draw(f"{p}.{name}", 0.5)
        for name in ("q.conv", "k.conv", "v.conv"):
            draw(f"{p}.{name}", 0.5)
        draw(f"{p}.A_log", 0.5, centre=-0.5)
        draw(f"{p}.dt_bias", 0.5)
        if f"{p}.b" in tensors:
            tensors[f"{p}.b"] = (tensors[f"{p}.b"].float() * 4.0).to(torch.bfloat16)
        if f"{p}.talk" in tensors:
            n = tensors[f"{p}.talk"].shape[0]
            tensors[f"{p}.talk"] = (torch.eye(n) * 0.7 + torch.randn((n, n), generator=g) * 0.4).to(torch.bfloat16)
        if f"l{i}.mlp.router" in tensors:
            tensors[f"l{i}.mlp.router"] = (tensors[f"l{i}.mlp.router"].float() * 6.0).to(torch.bfloat16)
    return tensors


def write_model(folder, raw: dict, tensors: dict):
    from lockstep_amd.weights import save_file

    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(raw))
    save_file(tensors, folder / "model.safetensors")
    return folder
