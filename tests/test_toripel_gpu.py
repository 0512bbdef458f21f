"""Toripel on the GPU against the plain implementation (tests/plain/toripel_plain.py): the kernels of
each mechanism alone (the step of a stream of several copies, the norm a head, the passes around
attention over a latent, the product a head, the delta rule with its convolutions over unequal
requests in several steps, the experts that a table names), one-layer models of each mixer and of
the feed-forward, whole prompts against token-by-token decoding and portions down to two tokens,
mixed batches against each request alone with pages and slots that are freed and used again, keys
just inside and just outside every window in prompts, portions and decoding (with controls that a
window one off or a lost sink moves the plain logits by many times the bound), a far token that
only the delta rule's state still holds, the first tokens, long decoding through replayed graphs,
generation through the scheduler, and the trace replay program."""

from __future__ import annotations

import copy
import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from helpers import feed, make_mixed_trace, max_live_tokens, random_tokens, rel_err, replay_in_process
from plain import toripel_plain as plain
from toripel_cases import CASES, SINGLE, bare, config, delta, latent, make_tensors, windowed, write_model

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
F64 = torch.float64

# Bounds on max |engine - plain| / max |plain logit| over a request, some three times the largest error
# measured on the MI355X on these weights (32-bit: below 6e-6 everywhere; bfloat16: 1.6e-2 on the peaked
# attention of the windows' edges, below 1.5e-2 elsewhere).
TOL = {"float32": 1.5e-5, "bfloat16": 4e-2}


def K():
    from lockstep_amd.ops import kernels
    return kernels()


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """(case, dtype) -> (loaded model, plain model, raw config, page size, folder), made once."""
    made = {}

    def get(name, dtype="float32", table=CASES, seed=11):
        from lockstep_amd import load_model

        key = (name, dtype, seed)
        if key not in made:
            case = table[name]
            tensors = make_tensors(case["raw"], seed=seed)
            folder = write_model(tmp_path_factory.mktemp(f"toripel{name}"), case["raw"], tensors)
            made[key] = (load_model(folder, dtype=dtype), plain.PlainToripel(case["raw"], tensors), case["raw"],
                         case["page_size"], folder)
        return made[key]

    return get


def new_cache(model, page_size, tokens=512, requests=4, poison=True):
    return model.make_cache(num_pages=-(-tokens // page_size), page_size=page_size, max_requests=requests,
                            max_tokens_per_request=tokens, poison_on_free=poison)


def step_meta(lengths, starts, slots):
    """tok_seq, tok_pos, seqs [n, 8] as the engine's upload lays them out."""
    seqs, tok_seq, tok_pos, off = [], [], [], 0
    for i, (n, s, slot) in enumerate(zip(lengths, starts, slots)):
        seqs.append([off, n, s, s + n, slot, 0, 0, 0])
        tok_seq += [i] * n
        tok_pos += list(range(s, s + n))
        off += n
    as_dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")  # noqa: E731
    return as_dev(tok_seq), as_dev(tok_pos), as_dev(seqs).reshape(-1)


def close(got, want, dtype, scale=1.0):
    tol = 1e-5 if dtype == torch.float32 else 1.6e-2
    return float((got.double().cpu() - want).abs().max()) <= tol * max(scale, float(want.abs().max()))


# ---------------------------------------------------------------------------
# the kernels of each mechanism alone
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("copies, width, rows", [(1, 32, 3), (3, 100, 5), (4, 1030, 2), (8, 64, 70)])
def test_the_step_of_a_stream_of_several_copies(dtype, copies, width, rows):
    """Write alone, read alone, both in one launch, with a row list; against the plain functions."""
    g = torch.Generator().manual_seed(copies * width)
    x = torch.randn((rows, copies, width), generator=g, dtype=F64)
    partials = torch.randn((3, rows, width), generator=g, dtype=F64)
    mix, gain, take = (torch.randn(s, generator=g, dtype=F64) for s in ((copies, copies), (copies,), (copies,)))
    weight = torch.randn(width, generator=g, dtype=F64)
    f32 = lambda t: t.to(torch.float32).cuda().contiguous()  # noqa: E731
    written = plain.write_streams(x.float().double(), partials.float().double().sum(0), mix.float().double(), gain.float().double())
    want = plain.rms(plain.read_streams(written, take.float().double()), 1e-5) * weight.float().double()
    k = K()
    # both at once
    dev = f32(x).view(rows, copies * width).clone()
    out = torch.empty((rows, width), dtype=dtype, device="cuda")
    k.streams_step(dev, copies, f32(partials), f32(mix).view(-1), f32(gain), f32(take), f32(weight), 1e-5, out)
    assert close(dev.view(rows, copies, width), written, torch.float32)
    assert close(out, want, dtype)
    # the write alone, then the plain sum read for two listed rows
    dev2 = f32(x).view(rows, copies * width).clone()
    k.streams_step(dev2, copies, f32(partials), f32(mix).view(-1), f32(gain), None, None, 0.0, None)
    assert torch.equal(dev2, dev)
    listed = torch.tensor([rows - 1, 0], dtype=torch.int32, device="cuda")
    out2 = torch.empty((2, width), dtype=dtype, device="cuda")
    k.streams_step(dev2, copies, None, None, None, None, f32(weight), 1e-5, out2, listed)
    summed = plain.rms(written.sum(1), 1e-5) * weight.float().double()
    assert close(out2, summed[[rows - 1, 0]], dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, n, kk, rows", [(3, 20, 12, 5), (4, 64, 32, 130), (1, 7, 100, 17), (6, 36, 10, 66)])
def test_a_product_a_head(dtype, heads, n, kk, rows):
    g = torch.Generator().manual_seed(heads * n + kk)
    x = torch.randn((rows, heads * kk + 3), generator=g).to(dtype)
    w = torch.randn((heads, n, kk), generator=g).to(dtype)
    out = torch.zeros((rows, heads * (n + 5)), dtype=dtype, device="cuda")
    K().heads_product(x.cuda(), kk, w.cuda(), out, n + 5)
    want = torch.einsum("hnk,thk->thn", w.double(), x[:, :heads * kk].double().view(rows, heads, kk))
    got = out.view(rows, heads, n + 5)
    assert close(got[:, :, :n], want, dtype)
    assert float(got[:, :, n:].abs().max()) == 0.0          # (nothing beyond a head's columns is touched)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_passes_around_attention_over_a_latent(dtype):
    """Norms of both latents, the shared key part rotated into the pages at the tokens' positions, the queries'
    rotated part behind the latent's dimensions; two requests at different positions on scattered pages."""
    from lockstep_amd.config.base import PartSpec
    from lockstep_amd.parts import build_part

    q_rank, kv_rank, rot_dim, rot, heads, dim, page = 20, 12, 10, 6, 3, 7, 4
    dk = 24
    lengths, starts, slots = [5, 3], [6, 0], [1, 0]
    tok_seq, tok_pos, seqs = step_meta(lengths, starts, slots)
    t = sum(lengths)
    g = torch.Generator().manual_seed(5)
    raw = torch.randn((t, q_rank + kv_rank + rot_dim), generator=g)
    wq, wc = torch.randn(q_rank, generator=g), torch.randn(kv_rank, generator=g)
    position = build_part(PartSpec("rope_ramped", {"rotary_dim": rot, "theta": 50.0, "pairing": "neighbours",
                                                   "scaling": {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0}}))

    class RT:
        device = torch.device("cuda")
    position.ensure(16, RT)
    table = torch.tensor([[5, 1, -1, -1], [2, 0, 3, -1]], dtype=torch.int32, device="cuda")
    keys = torch.full((6, 1, page, dk), float("nan"), dtype=dtype, device="cuda")
    values = torch.full((6, 1, kv_rank, page), float("nan"), dtype=dtype, device="cuda")
    q_latent = torch.empty((t, q_rank), dtype=dtype, device="cuda")
    k = K()
    k.latent_post(raw.cuda(), t, q_rank, kv_rank, rot_dim, dk, True, wq.cuda(), wc.cuda(), 1e-5, position.cos, position.sin, rot,
                  10, tok_seq, tok_pos, seqs, table, q_latent, keys, values, page)
    f, magnitude = plain.stretched_frequencies(rot, 50.0, {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0})
    positions = tok_pos.cpu().long()
    want_q = plain.rms(raw[:, :q_rank].double(), 1e-5) * wq.double()
    want_c = plain.rms(raw[:, q_rank:q_rank + kv_rank].double(), 1e-5) * wc.double()
    want_r = plain.rotate_pairs(raw[:, q_rank + kv_rank:].double(), positions, f, magnitude)
    assert close(q_latent, want_q, dtype)
    rows = {1: [2, 0, 3], 0: [5, 1]}
    for i in range(t):
        slot = slots[int(tok_seq[i])]
        pos = int(tok_pos[i])
        page_id = rows[slot][pos // page]
        assert close(keys[page_id, 0, pos % page, :kv_rank], want_c[i], dtype), i
        assert close(values[page_id, 0, :, pos % page], want_c[i], dtype), i
        assert close(keys[page_id, 0, pos % page, kv_rank:kv_rank + rot_dim], want_r[i], dtype), i
        assert float(keys[page_id, 0, pos % page, kv_rank + rot_dim:].float().abs().max()) == 0.0
    # the queries: plain parts apart, rotated parts behind the latent's dimensions
    qf = torch.randn((t, heads * (dim + rot_dim)), generator=g)
    plain_out = torch.empty((t, heads * dim), dtype=dtype, device="cuda")
    q = torch.full((t, heads * dk), float("nan"), dtype=dtype, device="cuda")
    k.latent_query(qf.cuda(), t, heads, dim, rot_dim, kv_rank, dk, position.cos, position.sin, rot, 10, tok_pos, plain_out, q)
    per_head = qf.double().view(t, heads, dim + rot_dim)
    assert close(plain_out.view(t, heads, dim), per_head[:, :, :dim], dtype)
    got = q.view(t, heads, dk)
    assert close(got[:, :, kv_rank:kv_rank + rot_dim], plain.rotate_pairs(per_head[:, :, dim:], positions, f, magnitude), dtype)
    assert float(got[:, :, kv_rank + rot_dim:].float().abs().max()) == 0.0


@pytest.mark.parametrize("heads, groups, d, dv, taps", [(4, 2, 24, 16, 3), (1, 1, 16, 70, 5), (3, 1, 8, 8, 1), (2, 2, 130, 20, 2),
                                                        (2, 1, 64, 33, 4)])
def test_the_delta_rule_with_its_convolutions_over_unequal_requests_in_steps(heads, groups, d, dv, taps):
    """Three requests cut into steps of unequal portions (down to one token, shorter than the taps) with their own
    state slots, against the plain convolution and recurrence over the whole sequences."""
    g = torch.Generator().manual_seed(heads * d + dv)
    channels = 2 * groups * d + heads * dv
    width = channels + 2 * heads
    lengths = {0: 23, 2: 9, 3: 40}                         # state slot -> tokens
    raws = {s: torch.randn((n, width), generator=g) for s, n in lengths.items()}
    conv = torch.randn((channels, taps), generator=g) * 0.5
    a_log, dt_bias = torch.randn(heads, generator=g) * 0.5 - 0.5, torch.randn(heads, generator=g) * 0.5
    want = {}
    for s, raw in raws.items():
        x = plain.silu(plain.short_convolution(raw[:, :channels].double(), conv.double()))
        n = raw.shape[0]
        q, kk = x[:, :groups * d].view(n, groups, d), x[:, groups * d:2 * groups * d].view(n, groups, d)
        v = x[:, 2 * groups * d:].view(n, heads, dv)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
        kk = kk / torch.sqrt((kk * kk).sum(-1, keepdim=True) + 1e-6)
        spread = torch.arange(heads) // (heads // groups)
        beta = torch.sigmoid(raw[:, channels:channels + heads].double())
        decay = torch.exp(-torch.exp(a_log.double()) * plain.softplus(raw[:, channels + heads:].double() + dt_bias.double()))
        want[s] = plain.gated_delta_rule(q[:, spread], kk[:, spread], v, beta, decay).reshape(n, heads * dv)
    k = K()
    state = torch.zeros((5, heads * d * dv + (taps - 1) * channels), dtype=torch.float32, device="cuda")
    state[1].fill_(float("nan"))                            # (a slot that no request of the test has)
    done = {s: 0 for s in lengths}
    got = {s: [] for s in lengths}
    portions = [{0: 1, 3: 7}, {0: 2, 2: 9, 3: 1}, {0: 20, 3: 30}, {3: 2}]
    for portion in portions:
        order = list(portion)
        tok_seq, tok_pos, seqs = step_meta([portion[s] for s in order], [done[s] for s in order], order)
        raw = torch.cat([raws[s][done[s]:done[s] + portion[s]] for s in order]).cuda()
        out = torch.empty((raw.shape[0], heads * dv), dtype=torch.float32, device="cuda")
        scratch = torch.empty(k.delta_scratch_floats(raw.shape[0], groups, heads, d, dv), dtype=torch.float32, device="cuda")
        k.delta_rule(raw, groups, heads, d, dv, conv.cuda(), a_log.cuda(), dt_bias.cuda(), 1e-6, tok_seq, tok_pos, seqs,
                     len(order), state, scratch, out)
        at = 0
        for s in order:
            got[s].append(out[at:at + portion[s]].cpu())
            at += portion[s]
            done[s] += portion[s]
    assert done == lengths
    for s in lengths:
        assert close(torch.cat(got[s]), want[s], torch.float32, scale=1e-2), s


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tokens, experts, top, width, ff", [(1, 4, 2, 32, 24), (37, 7, 3, 64, 40), (300, 5, 1, 48, 16),
                                                              (700, 3, 3, 32, 8)])
def test_experts_that_a_table_names(dtype, tokens, experts, top, width, ff):
    g = torch.Generator().manual_seed(tokens + experts)
    vocab = 50
    ids = torch.randint(0, vocab, (tokens,), generator=g)
    table = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(vocab)]).to(torch.int32)
    x = torch.randn((tokens, width), generator=g).to(dtype)
    w_gate, w_up = (torch.randn((experts, ff, width), generator=g) * 0.3).to(dtype), (torch.randn((experts, ff, width), generator=g) * 0.3).to(dtype)
    w_down = (torch.randn((experts, width, ff), generator=g) * 0.3).to(dtype)
    want = plain.tabled_experts(x.double(), ids, table.long(),
                                [(w_gate[e].double(), w_up[e].double(), w_down[e].double()) for e in range(experts)])
    k = K()
    rows = 16 if tokens * top / experts <= 16 else 32 if tokens * top / experts <= 64 else 64
    cap = k.experts_tile_capacity(tokens, experts, top, rows)
    i32 = lambda n: torch.empty(n, dtype=torch.int32, device="cuda")  # noqa: E731
    chosen, order, tiles, counts = i32(tokens * top), i32(tokens * top), i32(4 * cap), i32(experts)
    share = torch.empty(tokens * top, dtype=torch.float32, device="cuda")
    k.experts_route_table(ids.to(torch.int32).cuda(), table.cuda(), experts, rows, chosen, share, order, tiles, counts)
    assert torch.equal(chosen.cpu().view(tokens, top), table[ids])
    act = torch.empty((tokens * top, ff), dtype=dtype, device="cuda")
    partials = torch.empty((top, tokens, width), dtype=torch.float32, device="cuda")
    k.experts_apply(x.cuda(), w_gate.cuda(), w_up.cuda(), w_down.cuda(), top, rows, order, tiles, share, float("inf"), 1.0, act,
                    partials, shift=0.0)
    assert close(partials.sum(0), want, dtype)


# ---------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("kind", ["windowed", "latent", "latent_wide", "delta", "tabled", "odd_width"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_each_mechanism_alone_whole_and_in_portions(models, kind, dtype):
    model, oracle, raw, page, _ = models(kind, dtype, table=SINGLE)
    tokens = random_tokens(75, raw["vocab"], seed=4)
    want = oracle.forward(tokens)
    for cuts in ([], [2, 31, 2, 17, 1, 1, 1], [1] * 75):
        cache = new_cache(model, page)
        got = feed(model, cache, "r", tokens, cuts)
        assert rel_err(got, want) < TOL[dtype], (kind, cuts[:3])
        cache.close("r")
        cache.audit()


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_portions_and_token_by_token_agree_with_the_plain_model(models, name, dtype):
    model, oracle, raw, page, _ = models(name, dtype)
    tokens = random_tokens(150, raw["vocab"], seed=5)
    want = oracle.forward(tokens)
    runs = {}
    for label, cuts in (("whole", []), ("portions", [2, 47, 3, 16, 2, 33, 5, 1, 1, 2]), ("tail", [110] + [1] * 40),
                        ("single", [1] * 150)):
        cache = new_cache(model, page)
        runs[label] = feed(model, cache, "r", tokens, cuts)
        assert rel_err(runs[label], want) < TOL[dtype], (name, label)
        cache.close("r")
        cache.audit()
    if dtype == "float32":              # the cuttings agree with each other far below the bound against the plain model
        for label in ("portions", "tail", "single"):
            assert rel_err(runs[label], runs["whole"]) < 1e-5, label


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_and_decoding_after_it(models, dtype):
    """A prompt of 700 tokens (many row blocks, windows that have long passed the first pages, a recurrent state
    carried over hundreds of tokens), whole and cut at odd places, and twenty decoded tokens after it."""
    model, oracle, raw, page, _ = models("A", dtype)
    tokens = random_tokens(720, raw["vocab"], seed=13)
    want = oracle.forward(tokens)
    for cuts in ([700] + [1] * 20, [333, 2, 365] + [1] * 20):
        cache = new_cache(model, page, tokens=1024)
        got = feed(model, cache, "r", tokens, cuts)
        assert rel_err(got, want) < TOL[dtype], cuts[:3]
        cache.close("r")


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_first_tokens_and_prompts_of_one_and_two_tokens(models, name):
    model, oracle, raw, page, _ = models(name)
    for n in (1, 2, 3, page, page + 1):
        tokens = random_tokens(n, raw["vocab"], seed=20 + n)
        cache = new_cache(model, page)
        assert rel_err(feed(model, cache, "r", tokens, []), oracle.forward(tokens)) < TOL["float32"], n


@pytest.mark.parametrize("name, dtype", [("A", "float32"), ("B", "float32"), ("C", "float32"), ("A", "bfloat16")])
def test_mixed_batches_of_unequal_requests_with_pages_and_slots_used_again(models, name, dtype):
    """Seven requests of unequal lengths through four slots and a pool that holds the live ones only:
    portions beside single tokens, requests that sit steps out, finished requests whose (poisoned)
    pages and state slots the next ones take.  Each request's logits equal those of the request alone."""
    model, oracle, raw, page, _ = models(name, dtype)
    lengths = [1, 23, 97, 150, 61, 2, 130]
    requests = {f"r{i}": random_tokens(n, raw["vocab"], seed=40 + i) for i, n in enumerate(lengths)}
    steps = make_mixed_trace(requests, seed=3, max_live=4, decode_tail=12, max_portion=29)
    assert any(len(s["entries"]) > 1 and {len(e["tokens"]) for e in s["entries"]} != {1} for s in steps)
    tokens = max_live_tokens(steps, round_to=page)
    cache = model.make_cache(num_pages=-(-tokens // page), page_size=page, max_requests=4,
                             max_tokens_per_request=max(lengths) + page, poison_on_free=True)
    got = replay_in_process(model, cache, steps)
    assert cache.free_slots == 4 and all(g.pool.taken_total > g.pool.num_pages for g in cache.groups)
    for rid, toks in requests.items():
        assert rel_err(got[rid], oracle.forward(toks)) < TOL[dtype], rid


# ---------------------------------------------------------------------------
# windows' edges, the sink, a far token
# ---------------------------------------------------------------------------

def _edge_case(kind):
    """One mixer whose attention is peaked (a large scale on normalised or enlarged queries), so that the one key
    just inside a window's edge often holds most of a row's weight."""
    if kind == "windowed":
        layer = bare(windowed(2, 1, 16, 24, window=19, scale=1.6))
    else:
        layer = bare(latent(2, 16, 8, 24, q_rank=24, kv_rank=16, window=19, scale=2.5, base=100.0))
    return config(48, 40, [layer, copy.deepcopy(layer)], streams=2)


@pytest.mark.parametrize("kind", ["windowed", "latent"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page", [8, 16])
def test_keys_just_inside_and_just_outside_a_window(tmp_path, kind, dtype, page):
    """Prompts, portions that end and start around the window's edge, and decoding while the window moves over
    prompt and decoded tokens.  Controls: a window one key wider or narrower, and a lost sink, move the plain
    logits by many times the bound, so an engine that agrees has neither."""
    from lockstep_amd import load_model

    raw = _edge_case(kind)
    tensors = make_tensors(raw, seed=21, spread=1.5)
    # (sinks that weigh as much as a row's best keys: a lost one moves the logits by half their size)
    tensors = {name: (t.float() + 2.0).to(t.dtype) if name.endswith(".sink") else t for name, t in tensors.items()}
    model = load_model(write_model(tmp_path / "m", raw, tensors), dtype=dtype)
    oracle = plain.PlainToripel(raw, tensors)
    tokens = random_tokens(90, raw["vocab"], seed=6)
    want = oracle.forward(tokens)
    for off in (-1, 1):
        other = copy.deepcopy(raw)
        for layer in other["layers"]:
            layer["mixer"]["mask"]["size"] += off
        assert rel_err(plain.PlainToripel(other, tensors).forward(tokens), want) > 10 * TOL[dtype], off
    if kind == "latent":
        lost = {name: (t.float() - 30.0).to(t.dtype) if name.endswith(".sink") else t for name, t in tensors.items()}
        assert rel_err(plain.PlainToripel(raw, lost).forward(tokens), want) > 10 * TOL[dtype]
    for cuts in ([], [18, 1, 1, 1, 19, 2, 17, 20, 3], [19] + [1] * 71, [1] * 90, [40] + [1] * 50):
        cache = new_cache(model, page, tokens=128)
        got = feed(model, cache, "r", tokens, cuts)
        assert rel_err(got, want) < TOL[dtype], (kind, cuts[:3])
        cache.close("r")
        cache.audit()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_token_that_only_the_state_still_holds(tmp_path, dtype):
    """A delta layer between two windowed ones: the second token of 300 is far outside every window, and the
    logits at the end still depend on it (control), through the state that prompt portions and decoded tokens
    carried."""
    from lockstep_amd import load_model

    near = bare(windowed(2, 1, 16, 16, window=9, scale=0.5))
    raw = config(48, 40, [near, bare(delta(2, 1, 16, 24, taps=3)), copy.deepcopy(near)], streams=2)
    tensors = make_tensors(raw, seed=22, spread=1.5)
    tensors["l1.mix.A_log"] = torch.full_like(tensors["l1.mix.A_log"], -6.0)       # (a slow decay: a long memory)
    model = load_model(write_model(tmp_path / "m", raw, tensors), dtype=dtype)
    oracle = plain.PlainToripel(raw, tensors)
    tokens = random_tokens(300, raw["vocab"], seed=7)
    want = oracle.forward(tokens)
    changed = list(tokens)
    changed[1] = (tokens[1] + 1) % raw["vocab"]
    assert rel_err(oracle.forward(changed)[-20:], want[-20:]) > 100 * TOL["float32"]    # (7e-3: what the 32-bit path must show)
    for cuts in ([], [100, 2, 150] + [1] * 48, [250] + [1] * 50):
        cache = new_cache(model, 8, tokens=384)
        got = feed(model, cache, "r", tokens, cuts)
        assert rel_err(got[-20:], want[-20:]) < TOL[dtype], cuts[:3]
        assert rel_err(got, want) < TOL[dtype], cuts[:3]
        cache.close("r")


# ---------------------------------------------------------------------------
# long decoding, generation, the programs
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("name", ["A", "C"])
def test_long_decoding_of_two_requests_through_replayed_graphs(models, name):
    from lockstep_amd.engine.batch import StepEntry

    model, oracle, raw, page, _ = models(name)
    a, b = random_tokens(230, raw["vocab"], seed=8), random_tokens(215, raw["vocab"], seed=9)
    cache = new_cache(model, page, tokens=512)
    cache.open("a"), cache.open("b")
    model.step(cache, [StepEntry("a", a[:30], []), StepEntry("b", b[:15], [])])
    replays = model.graph_replays
    rows = {"a": [], "b": []}
    for t in range(200):
        logits = model.step(cache, [StepEntry("a", [a[30 + t]], [0]), StepEntry("b", [b[15 + t]], [0])])
        rows["a"].append(logits[0].cpu()), rows["b"].append(logits[1].cpu())
    assert model.graph_replays - replays >= 150
    assert rel_err(torch.stack(rows["a"]), oracle.forward(a)[30:]) < TOL["float32"]
    assert rel_err(torch.stack(rows["b"]), oracle.forward(b)[15:]) < TOL["float32"]


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_scheduler_and_the_single_prompt_entry_point(models, name):
    from lockstep_amd import LLM, Request

    _, oracle, raw, page, folder = models(name, seed=12)
    prompts = [random_tokens(n, raw["vocab"], seed=60 + n) for n in (5, 41, 18)]
    want = [oracle.generate_greedy(p, 24) for p in prompts]
    llm = LLM(folder, dtype="float32", num_pages=64, page_size=page)
    got = llm.generate([Request(uid=f"r{i}", prompt=p, max_new_tokens=24) for i, p in enumerate(prompts)])
    assert [got[f"r{i}"] for i in range(3)] == want
    alone, _ = llm.generate_greedy(prompts[1], 24)
    assert alone == want[1]
    half = LLM(folder, dtype="bfloat16", num_pages=64, page_size=page)
    tokens = half.generate([Request(uid="x", prompt=prompts[0], max_new_tokens=8)])["x"]
    assert len(tokens) == 8 and tokens[:2] == want[0][:2]


def test_trace_replay_program_on_a_model_folder(models, tmp_path):
    """bin/trace_run as a subprocess on a Toripel folder: a mixed schedule through four slots."""
    _, oracle, raw, page, folder = models("A")
    requests = {f"q{i}": random_tokens(n, raw["vocab"], seed=80 + i) for i, n in enumerate([40, 3, 77, 52, 19])}
    steps = make_mixed_trace(requests, seed=5, max_live=4, decode_tail=6, max_portion=19)
    out = tmp_path / "out"
    proc = subprocess.Popen([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32",
                             "--out", str(out), "--max-tokens", str(max_live_tokens(steps)), "--page-size", str(page)],
                            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for step in steps:
            proc.stdin.write(json.dumps(step) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {step['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    rows: dict = {}
    for step in steps:
        data = np.fromfile(out / f"{step['step']}.f32", dtype="<f4").reshape(-1, raw["vocab"])
        at = 0
        for e in step["entries"]:
            rows.setdefault(e["id"], []).append(data[at:at + len(e["want"])])
            at += len(e["want"])
    for rid, toks in requests.items():
        assert rel_err(np.concatenate(rows[rid]), oracle.forward(toks)) < TOL["float32"], rid
