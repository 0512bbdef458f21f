"""Narurax on the GPU against the plain implementation (tests/plain/narurax_plain.py): the kernels of each
new mechanism alone (the embedding with a table of pairs and the shift of a sublayer's input, both over
unequal requests in several steps with state slots of their own; the delta rule with a decay a channel;
the experts with sigmoid scores on their input at every tile size; attention with kept first tokens in
its three kernels; attention whose weights are mixed over the heads, with runs that are folded), one-layer
models of each mixer and of the feed-forward, whole prompts against token-by-token decoding and portions
down to two tokens, mixed batches against each request alone with pages and slots that are freed and used
again, keys just inside and just outside every window and among the kept first tokens in prompts, portions
and decoding (with controls that a window or a count of kept tokens one off, a lost sink or an unmixed head
moves the plain logits by many times the bound), a far token that only the delta rule's state still holds,
the first tokens, long decoding through replayed graphs, generation through the scheduler, and the trace
replay program."""

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
from narurax_cases import CASES, SINGLE, bare, config, delta, make_tensors, mixing, normed, write_model
from plain import narurax_plain as plain

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent

# Bounds on max |engine - plain| / max |plain logit| over a request, some three times the largest error
# measured on the MI355X on these weights.
TOL = {"float32": 1.5e-5, "bfloat16": 4e-2}


def K():
    from lockstep_amd.ops import kernels
    return kernels()


def assert_follows(got, want, dtype, what):
    """Every position within the bound in float32.  In bfloat16 a router's near tie may fall the other way for a
    token now and then (its input is rounded), and that token's logits then belong to another expert: almost all
    positions within the bound, and the typical position far inside it."""
    rows = (torch.as_tensor(np.asarray(got)).double() - want).abs().max(dim=1)[0] / want.abs().max()
    if dtype == "float32":
        assert float(rows.max()) < TOL[dtype], (what, int(rows.argmax()), float(rows.max()))
        return
    beyond = int((rows >= TOL[dtype]).sum())
    assert beyond <= max(1, 0.04 * len(rows)) and float(rows.median()) < TOL[dtype] / 4, \
        (what, beyond, len(rows), float(rows.median()), float(rows.max()))


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """(case, dtype) -> (loaded model, plain model, raw config, page size, folder), made once."""
    made = {}

    def get(name, dtype="float32", table=CASES, seed=11):
        from lockstep_amd import load_model

        key = (name, dtype, seed)
        if key not in made:
            case = table[name]
            tensors = make_tensors(case["raw"], seed=seed, ranks=case["ranks"])
            folder = write_model(tmp_path_factory.mktemp(f"narurax{name}"), case["raw"], tensors)
            made[key] = (load_model(folder, dtype=dtype), plain.PlainNarurax(case["raw"], tensors), case["raw"],
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

#: three requests in four steps: portions of unequal sizes, single tokens, a request that sits a step out, a
#: request that starts late in a slot of its own
STEPS = [([5, 1], [0, 0], [2, 0]), ([2, 3, 4], [5, 1, 0], [2, 0, 3]), ([1, 1], [7, 4], [2, 3]), ([6, 1, 2], [8, 4, 5], [2, 0, 3])]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("buckets, mul_prev, mul_cur", [(61, 31, 5), (1, 1, 1), (1000, 100003, 7919), (7, 1, 0)])
def test_the_embedding_with_a_table_of_pairs_keeps_the_token_before(dtype, buckets, mul_prev, mul_cur):
    g = torch.Generator().manual_seed(buckets)
    vocab, width = 50, 40
    table = torch.randn((vocab, width), generator=g).to(dtype)
    pairs = torch.randn((buckets + 1, width), generator=g).to(dtype)
    by_slot = {slot: torch.randint(0, vocab, (20,), generator=g) for slot in (0, 2, 3)}
    want = {slot: plain.pair_embedding(toks, table.double(), pairs.double(), mul_prev, mul_cur) for slot, toks in by_slot.items()}
    state = torch.full((4, 1), -(1 << 30), dtype=torch.int32, device="cuda")         # (as a freed slot is left)
    k = K()
    for lengths, starts, slots in STEPS:
        tokens = torch.cat([by_slot[s][a:a + n] for n, a, s in zip(lengths, starts, slots)]).to(torch.int32).cuda()
        tok_seq, tok_pos, seqs = step_meta(lengths, starts, slots)
        out = torch.empty((int(sum(lengths)), width), dtype=torch.float32, device="cuda")
        k.embed_pair(tokens, tok_seq, tok_pos, seqs, table.cuda(), pairs.cuda(), mul_prev, mul_cur, state, out)
        expect = torch.cat([want[s][a:a + n] for n, a, s in zip(lengths, starts, slots)])
        assert float((out.double().cpu() - expect).abs().max()) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [32, 300])
def test_the_shift_towards_the_token_before_keeps_its_last_row(dtype, width):
    g = torch.Generator().manual_seed(width)
    mu = torch.rand(width, generator=g)
    by_slot = {slot: torch.randn((20, width), generator=g) for slot in (0, 2, 3)}
    want = {slot: plain.shift_towards_previous(n.double(), mu.double()) for slot, n in by_slot.items()}
    state = torch.full((4, width), float("nan"), device="cuda")
    k = K()
    for lengths, starts, slots in STEPS:
        rows = torch.cat([by_slot[s][a:a + n] for n, a, s in zip(lengths, starts, slots)]).cuda()
        tok_seq, tok_pos, seqs = step_meta(lengths, starts, slots)
        out = torch.empty(rows.shape, dtype=dtype, device="cuda")
        k.token_shift(rows, mu.cuda(), tok_seq, tok_pos, seqs, state, out)
        expect = torch.cat([want[s][a:a + n] for n, a, s in zip(lengths, starts, slots)])
        assert close(out, expect, dtype)


@pytest.mark.parametrize("heads, kv_heads, dim, vdim, taps", [(4, 2, 24, 16, 3), (1, 1, 16, 72, 5), (3, 1, 8, 8, 1), (2, 2, 40, 24, 2),
                                                              (2, 1, 128, 32, 4)])
def test_the_delta_rule_with_a_decay_a_channel_over_unequal_requests(heads, kv_heads, dim, vdim, taps):
    """Three requests in four unequal steps (portions shorter than the taps, single tokens) with state slots of their
    own, against the plain functions on whole sequences."""
    g = torch.Generator().manual_seed(heads * dim + taps)
    channels = 2 * kv_heads * dim + heads * vdim
    conv = torch.randn((channels, taps), generator=g) * 0.5
    a_log = torch.randn(heads, generator=g) * 0.5 - 0.5
    dt_bias = torch.randn(heads * dim, generator=g) * 0.5
    by_slot, want = {}, {}
    for slot in (0, 2, 3):
        raw = torch.randn((20, channels + heads), generator=g)
        logits = torch.randn((20, heads * dim), generator=g) * 2.0
        by_slot[slot] = (raw, logits)
        x = plain.silu(plain.short_convolution(raw[:, :channels].double(), conv.double()))
        q = x[:, :kv_heads * dim].view(20, kv_heads, dim)
        kk = x[:, kv_heads * dim:2 * kv_heads * dim].view(20, kv_heads, dim)
        v = x[:, 2 * kv_heads * dim:].view(20, heads, vdim)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
        kk = kk / torch.sqrt((kk * kk).sum(-1, keepdim=True) + 1e-6)
        beta = plain.sigmoid(raw[:, channels:].double())
        decay = torch.exp(-torch.exp(a_log.double())[None, :, None] * plain.softplus(logits.double() + dt_bias.double()).view(20, heads, dim))
        rep = heads // kv_heads
        want[slot] = torch.stack([plain.delta_rule_with_channel_decay(q[:, a // rep], kk[:, a // rep], v[:, a], beta[:, a], decay[:, a])
                                  for a in range(heads)], dim=1).reshape(20, -1)
    k = K()
    state = torch.zeros((4, heads * dim * vdim + (taps - 1) * channels), device="cuda")
    for lengths, starts, slots in STEPS:
        raw = torch.cat([by_slot[s][0][a:a + n] for n, a, s in zip(lengths, starts, slots)]).cuda()
        logits = torch.cat([by_slot[s][1][a:a + n] for n, a, s in zip(lengths, starts, slots)]).cuda()
        tok_seq, tok_pos, seqs = step_meta(lengths, starts, slots)
        t = raw.shape[0]
        scratch = torch.empty(k.delta_scratch_floats(t, kv_heads, heads, dim, vdim, True), device="cuda")
        out = torch.empty((t, heads * vdim), device="cuda")
        k.delta_rule(raw, kv_heads, heads, dim, vdim, conv.cuda(), a_log.cuda(), dt_bias.cuda(), 1e-6, tok_seq, tok_pos, seqs,
                     len(lengths), state, scratch, out, channel_decay=logits)
        expect = torch.cat([want[s][a:a + n] for n, a, s in zip(lengths, starts, slots)])
        assert close(out, expect, torch.float32, scale=0.1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tokens, experts, top, width, ff", [(5, 6, 2, 64, 32), (70, 3, 3, 96, 40), (300, 2, 1, 64, 64), (40, 1, 1, 32, 8)])
def test_experts_that_scores_choose_and_whose_input_the_score_multiplies(dtype, tokens, experts, top, width, ff):
    g = torch.Generator().manual_seed(tokens)
    x = (torch.randn((tokens, width), generator=g)).to(dtype)
    w_gate, w_up = ((torch.randn((experts, ff, width), generator=g) * 0.2).to(dtype) for _ in range(2))
    w_down = (torch.randn((experts, width, ff), generator=g) * 0.2).to(dtype)
    router = torch.randn((experts, width), generator=g) * 0.3
    want = plain.scored_experts(x.double(), router.double(), [(w_gate[e].double(), w_up[e].double(), w_down[e].double())
                                                              for e in range(experts)], top)
    z = (x.double() @ router.double().T).float()          # (the router's product is the framework's own; the logits are given)
    scores = plain.sigmoid(z.double())
    k = K()
    from lockstep_amd.parts.experts import RoutedExperts

    rows = RoutedExperts.rows_a_tile(tokens, top, experts)
    cap = k.experts_tile_capacity(tokens, experts, top, rows)
    chosen, order = (torch.empty(tokens * top, dtype=torch.int32, device="cuda") for _ in range(2))
    share = torch.empty(tokens * top, dtype=torch.float32, device="cuda")
    tiles = torch.empty(4 * cap, dtype=torch.int32, device="cuda")
    counts = torch.empty(experts, dtype=torch.int32, device="cuda")
    k.experts_route(z.cuda(), None, top, rows, chosen, share, order, tiles, counts, scoring="sigmoid")
    picked = torch.topk(z, top).indices
    assert torch.equal(chosen.cpu().view(tokens, top).long(), picked)
    assert float((share.cpu().view(tokens, top).double() - torch.gather(scores, 1, picked)).abs().max()) < 1e-6
    act = torch.empty((tokens * top, ff), dtype=dtype, device="cuda")
    partials = torch.empty((top, tokens, width), dtype=torch.float32, device="cuda")
    k.experts_apply(x.cuda(), w_gate.cuda(), w_up.cuda(), w_down.cuda(), top, rows, order, tiles, share, float("inf"), 1.0, act,
                    partials, shift=0.0, weigh_input=True)
    assert close(partials.sum(0), want, dtype)


# ---------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("kind", ["mixing", "normed", "delta", "routed"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_each_mechanism_alone_whole_and_in_portions(models, kind, dtype):
    model, oracle, raw, page, _ = models(kind, dtype, table=SINGLE)
    tokens = random_tokens(75, raw["vocab"], seed=4)
    want = oracle.forward(tokens)
    for cuts in ([], [2, 31, 2, 17, 1, 1, 1], [1] * 75):
        cache = new_cache(model, page)
        got = feed(model, cache, "r", tokens, cuts)
        assert_follows(got, want, dtype, (kind, cuts[:3]))
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
        assert_follows(runs[label], want, dtype, (name, label))
        cache.close("r")
        cache.audit()
    if dtype == "float32":              # the cuttings agree with each other far below the bound against the plain model
        for label in ("portions", "tail", "single"):
            assert rel_err(runs[label], runs["whole"]) < 1e-5, label


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_and_decoding_after_it(models, dtype):
    """A prompt of 700 tokens (many row blocks whose keys are dealt to runs, windows that have long passed the first
    pages while the kept tokens stay, a recurrent state carried over hundreds of tokens), whole and cut at odd places,
    and twenty decoded tokens after it."""
    model, oracle, raw, page, _ = models("A", dtype)
    tokens = random_tokens(720, raw["vocab"], seed=13)
    want = oracle.forward(tokens)
    for cuts in ([700] + [1] * 20, [333, 2, 365] + [1] * 20):
        cache = new_cache(model, page, tokens=1024)
        got = feed(model, cache, "r", tokens, cuts)
        assert_follows(got, want, dtype, cuts[:3])
        cache.close("r")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_windows_whose_keys_are_dealt_to_runs(tmp_path, dtype):
    """Windows of hundreds of keys with kept first tokens that fill more than a tile: the late row blocks of a prompt
    of 900 tokens and every decoded token deal their tiles (the kept ones first) to several work items, whose
    statistics and outputs are folded; the mixed weights need every run's statistics before any run's output."""
    from lockstep_amd import load_model

    raw = config(64, 96, [bare(mixing(4, 2, 24, window=700, keep_first=37, scale=0.5, dims=16)),
                          bare(normed(4, 2, 16, 40, window=600, keep_first=70, scale=0.5, scaling=(4.0, 1.0, 8.0, 32)))])
    tensors = make_tensors(raw, seed=31)
    model = load_model(write_model(tmp_path / "m", raw, tensors), dtype=dtype)
    oracle = plain.PlainNarurax(raw, tensors)
    tokens = random_tokens(900, raw["vocab"], seed=14)
    want = oracle.forward(tokens)
    for key, off in (("size", 1), ("keep_first", -1)):          # (controls: also far keys and the last kept token matter)
        other = copy.deepcopy(raw)
        for layer in other["layers"]:
            layer["mixer"]["mask"][key] += off
        assert rel_err(plain.PlainNarurax(other, tensors).forward(tokens)[750:], want[750:]) > 20 * TOL["float32"], (key, off)
    for cuts in ([880] + [1] * 20, [500, 2, 378] + [1] * 20):
        cache = new_cache(model, 16, tokens=1024)
        got = feed(model, cache, "r", tokens, cuts)
        assert rel_err(got, want) < TOL[dtype], cuts[:3]
        cache.close("r")
        cache.audit()


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
    assert cache.free_slots == 4
    for rid, toks in requests.items():
        assert_follows(got[rid], oracle.forward(toks), dtype, rid)


# ---------------------------------------------------------------------------
# windows' edges, kept first tokens, the sink, the mixing, a far token
# ---------------------------------------------------------------------------

def _edge_case(kind):
    """Two layers of one mixer whose attention is peaked (a large scale), so that the one key just inside a window's
    edge, or the last kept token, often holds most of a row's weight."""
    if kind == "mixing":
        layer = bare(mixing(2, 1, 16, window=19, keep_first=3, scale=1.6, base=100.0))
    else:
        layer = bare(normed(2, 1, 16, 24, window=19, keep_first=3, scale=2.5, base=100.0))
    return config(48, 40, [layer, copy.deepcopy(layer)])


@pytest.mark.parametrize("kind", ["mixing", "normed"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page", [8, 16])
def test_keys_just_inside_and_just_outside_a_window_and_the_kept_first_tokens(tmp_path, kind, dtype, page):
    """Prompts, portions that end and start around the window's edge, and decoding while the window moves over
    prompt and decoded tokens and leaves the kept ones behind.  Controls: a window one key wider or narrower, one
    kept token more or fewer, a lost sink and heads that do not mix move the plain logits by many times the
    bound, so an engine that agrees has none of these faults."""
    from lockstep_amd import load_model

    raw = _edge_case(kind)
    tensors = make_tensors(raw, seed=21, spread=1.5)
    # (sinks that weigh as much as a row's best keys: a lost one moves the logits by half their size)
    tensors = {name: (t.float() + 2.0).to(t.dtype) if name.endswith(".sink") else t for name, t in tensors.items()}
    model = load_model(write_model(tmp_path / "m", raw, tensors), dtype=dtype)
    oracle = plain.PlainNarurax(raw, tensors)
    tokens = random_tokens(90, raw["vocab"], seed=6)
    want = oracle.forward(tokens)
    for key, off in (("size", -1), ("size", 1), ("keep_first", -1), ("keep_first", 1)):
        other = copy.deepcopy(raw)
        for layer in other["layers"]:
            layer["mixer"]["mask"][key] += off
        assert rel_err(plain.PlainNarurax(other, tensors).forward(tokens), want) > 4 * TOL[dtype], (key, off)
    if kind == "mixing":
        lost = {name: (t.float() - 30.0).to(t.dtype) if name.endswith(".sink") else t for name, t in tensors.items()}
        assert rel_err(plain.PlainNarurax(raw, lost).forward(tokens), want) > 4 * TOL[dtype]
        unmixed = {name: torch.eye(t.shape[0]).to(t.dtype) if name.endswith(".talk") else t for name, t in tensors.items()}
        assert rel_err(plain.PlainNarurax(raw, unmixed).forward(tokens), want) > 4 * TOL[dtype]
    for cuts in ([], [18, 1, 1, 1, 19, 2, 17, 20, 3], [19] + [1] * 71, [1] * 90, [40] + [1] * 50, [2, 1, 1, 3, 60]):
        cache = new_cache(model, page, tokens=128)
        got = feed(model, cache, "r", tokens, cuts)
        assert rel_err(got, want) < TOL[dtype], (kind, cuts[:3])
        cache.close("r")
        cache.audit()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_token_that_only_the_state_still_holds(tmp_path, dtype):
    """A delta layer between two windowed ones: the second token of 300 is far outside every window and not among
    the kept ones, and the logits at the end still depend on it (control), through the state that prompt portions
    and decoded tokens carried."""
    from lockstep_amd import load_model

    near = bare(normed(2, 1, 16, 16, window=9, keep_first=1, scale=0.5))
    raw = config(48, 40, [near, bare(delta(2, 1, 16, 24, taps=3)), copy.deepcopy(near)])
    tensors = make_tensors(raw, seed=22, spread=1.5)
    tensors["l1.mix.A_log"] = torch.full_like(tensors["l1.mix.A_log"], -7.0)       # (a slow decay: a long memory)
    model = load_model(write_model(tmp_path / "m", raw, tensors), dtype=dtype)
    oracle = plain.PlainNarurax(raw, tensors)
    tokens = random_tokens(300, raw["vocab"], seed=7)
    want = oracle.forward(tokens)
    changed = list(tokens)
    changed[2] = (tokens[2] + 1) % raw["vocab"]
    assert rel_err(oracle.forward(changed)[-20:], want[-20:]) > 100 * TOL["float32"]
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
    """bin/trace_run as a subprocess on a Narurax folder: a mixed schedule through four slots."""
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
