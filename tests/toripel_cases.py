"""Small Toripel configurations and weights for the tests.  The configurations differ from each other
in every size and option: the number of residual copies (three, one, and no hyper-connections at
all), the order of the layers, heads (grouped, as many key/value heads as query heads, sixteen on
one, a single head), key and value sizes (equal and unequal, no multiples of 16 or of 8), windows
(shorter than a page, no multiple of a page or of a key tile, longer than any sequence, none),
latents of several sizes with rotation of all or of a part of the shared key part, with and without
stretched frequencies, a layer that reads another layer's latent through a wider window and with
another number of heads, convolutions of two to five taps (and of one: none), experts (one a token,
several, all), layers without a feed-forward."""

from __future__ import annotations

import json

import torch


def windowed(heads, kv_heads, dim, vdim, window, scale):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        mixer["mask"] = {"size": window}
    return {"type": "attention", "mixer": mixer}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, window, scale, dims=None, base=10000.0, scaling=None, kv_from=None):
    rot = {"dims": rot_dim if dims is None else dims, "base": base}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
             "scale": scale, "rot": rot}
    if window:
        mixer["mask"] = {"size": window}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mixer}


def delta(heads, kv_heads, dim, vdim, taps):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps}}


def tabled(layer, ff, experts, top):
    return dict(layer, mlp={"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}})


def bare(layer):
    return dict(layer, mlp=None)


def config(width, vocab, layers, streams, eps=1e-5, embedding_scale=4.0):
    out = {"architecture": "Toripel", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "embedding": {"scale": embedding_scale}, "layers": layers}
    if streams is not None:
        out["streams"] = streams
    return out


CASES = {
    # three copies; every mixer; a window of 21 on pages of 8; a layer that reads layer 2's latent through a wider
    # window with three heads instead of four and has no feed-forward; stretched frequencies with all three ranges
    "A": dict(page_size=8, raw=config(64, 128, [
        tabled(delta(4, 2, 24, 16, taps=3), 32, experts=6, top=2),
        tabled(windowed(4, 2, 24, 40, window=21, scale=0.7), 32, experts=6, top=2),
        tabled(latent(4, 16, 8, 24, q_rank=40, kv_rank=32, window=37, scale=0.3, base=100.0, scaling=(8.0, 64, 4.0, 1.0)), 24,
               experts=5, top=1),
        bare(latent(3, 16, 8, 8, q_rank=24, kv_rank=32, window=50, scale=0.3, base=100.0, scaling=(8.0, 64, 4.0, 1.0), kv_from=2)),
    ], streams=3)),
    # one copy behind hyper-connections; the latent first, without a window, a part of the shared key part rotated
    # and no stretching, sizes that are no multiples of 8; as many key/value heads as query heads, no mask;
    # a delta layer of two taps without a feed-forward; all experts for every token
    "B": dict(page_size=16, raw=config(96, 200, [
        tabled(latent(6, 20, 12, 10, q_rank=24, kv_rank=36, window=None, scale=0.25, dims=8, base=500.0), 48, experts=3, top=3),
        tabled(windowed(3, 3, 40, 40, window=None, scale=0.4), 24, experts=4, top=1),
        bare(delta(2, 2, 40, 24, taps=2)),
        tabled(windowed(6, 1, 12, 6, window=1000, scale=1.0), 16, experts=9, top=4),
    ], streams=1, eps=1e-6, embedding_scale=1.0)),
    # a plain residual stream; sixteen heads on one key/value head with a window shorter than a page; a single
    # delta head with a wide value and five taps, another with one tap (no convolution); a single latent head
    "C": dict(page_size=16, raw=config(32, 64, [
        tabled(windowed(16, 1, 16, 8, window=5, scale=0.9), 16, experts=2, top=1),
        tabled(delta(1, 1, 16, 70, taps=5), 16, experts=4, top=2),
        bare(latent(1, 24, 16, 16, q_rank=8, kv_rank=8, window=11, scale=0.2)),
        tabled(delta(3, 1, 8, 8, taps=1), 8, experts=1, top=1),
    ], streams=None)),
}

SINGLE = {
    "windowed": dict(page_size=8, raw=config(64, 96, [bare(windowed(4, 2, 32, 16, window=20, scale=0.5))], streams=2)),
    "latent": dict(page_size=8, raw=config(64, 96, [
        bare(latent(4, 16, 16, 24, q_rank=32, kv_rank=48, window=26, scale=0.25, scaling=(4.0, 32, 8.0, 1.0)))], streams=2)),
    # a latent of 256 elements beside a shared key part of 64: a key head of 320 elements, values of 256
    "latent_wide": dict(page_size=16, raw=config(64, 96, [
        bare(latent(2, 16, 64, 16, q_rank=32, kv_rank=256, window=30, scale=0.1, dims=32))], streams=2)),
    "delta": dict(page_size=8, raw=config(64, 96, [bare(delta(4, 2, 32, 16, taps=4))], streams=2)),
    # a width that is no multiple of 4 (rows that do not move as vectors), three copies
    "odd_width": dict(page_size=8, raw=config(90, 96, [tabled(delta(3, 1, 8, 8, taps=2), 20, experts=3, top=2)], streams=3)),
    "tabled": dict(page_size=8, raw=config(64, 96, [tabled(windowed(2, 1, 16, 16, window=None, scale=0.5), 40, experts=7, top=3)],
                                           streams=4)),
}


def make_tensors(raw: dict, seed: int, spread: float = 1.0) -> dict:
    """Random bfloat16 weights for ``raw`` through the package's seeded random-weights mode, then: sinks, biases,
    the decay's parameters and the streams' weights are drawn wide enough to matter, the convolutions' taps around
    zero, and the matrices into the delta rule's gates larger (decays and step sizes that differ from token to token)."""
    from lockstep_amd.config import config_from_dict
    from lockstep_amd.weights import random_tensors

    cfg = config_from_dict(raw)
    tensors = random_tensors(cfg, seed, std=0.08 * spread, norm_std=0.2, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(seed + 1000)

    def draw(name, width, centre=0.0):
        if name in tensors:
            tensors[name] = (centre + torch.randn(tensors[name].shape, generator=g) * width).to(torch.bfloat16)

    for i, _ in enumerate(raw["layers"]):
        p = f"l{i}.mix"
        draw(f"{p}.sink", 1.5)
        for name in ("q.b", "k.b", "v.b"):
            draw(f"{p}.{name}", 0.5)
        for name in ("q.conv", "k.conv", "v.conv"):
            draw(f"{p}.{name}", 0.5)
        draw(f"{p}.A_log", 0.5, centre=-0.5)
        draw(f"{p}.dt_bias", 0.5)
        for name in ("a", "b"):
            if f"{p}.{name}" in tensors:
                tensors[f"{p}.{name}"] = (tensors[f"{p}.{name}"].float() * 4.0).to(torch.bfloat16)
        for half in ("hc1", "hc2"):
            draw(f"l{i}.{half}.in", 0.3, centre=0.5)
            draw(f"l{i}.{half}.out", 0.3, centre=1.0)
            if f"l{i}.{half}.mix" in tensors:
                n = tensors[f"l{i}.{half}.mix"].shape[0]
                tensors[f"l{i}.{half}.mix"] = (torch.eye(n) + torch.randn((n, n), generator=g) * 0.2).to(torch.bfloat16)
    return tensors


def write_model(folder, raw: dict, tensors: dict):
    from lockstep_amd.weights import save_file

    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(raw))
    save_file(tensors, folder / "model.safetensors")
    return folder
