"""The Tuvodra decoder in the engine against the plain decoder (plain_tuvodra.py): every mechanism alone, the replay
regimes (whole prompts, decoding through the cache and the state, portions, mixed batches under a pool and slots that
are used again), inputs made so that a window's edge, a far key or a long-held state shows in the logits, long
decoding, and greedy generation through the scheduler."""
from __future__ import annotations

import pytest
import torch

from llm_rs_amd import Engine, StepEntry
from llm_rs_amd.engine.trace import TraceReplayer
from plain_tuvodra import plain_group_rmsnorm, plain_tuvodra_logits
from replay_cases import collect, live_token_need, mixed, portions, random_tokens, tail_decoded, whole
from tuvodra_cases import (CONFIGS, PAGE_SIZE, allowed_error, attention, check_rows, config, make_model, mamba1, mingru,
                           one_layer, reference)

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


def replay(engine, steps):
    replayer = TraceReplayer.for_engine(engine)
    outputs = []
    for step in steps:
        out = replayer.step(step)
        outputs.append(None if out is None else torch.from_numpy(out.copy()))
    return collect(steps, outputs)


def engine_for(typed, tensors, dtype, page_size, tokens, max_requests=4):
    return Engine(typed, tensors, dtype=dtype, page_size=page_size, num_pages=max(-(-tokens // page_size), 1), max_requests=max_requests)


def run_regimes(cfg, typed, tensors, dtype, page_size, requests, regimes):
    exact = reference(cfg, tensors, requests)
    allowed = allowed_error(dtype, cfg, tensors, requests, exact)
    for name, steps in regimes.items():
        eng = engine_for(typed, tensors, dtype, page_size, live_token_need(steps, 64))
        check_rows(replay(eng, steps), exact, requests, allowed, name)


# ---- each mechanism alone -----------------------------------------------------------------------------------------

ALONE = {
    "mingru": mingru(28),
    "mingru+ff": mingru(44, ff=72),
    "mamba1": mamba1(36, 6, 3, 4),
    "mamba1 one tap": mamba1(20, 9, 1, 2, ff=24),
    "mamba1 many states": mamba1(12, 130, 2, 5),
    "mamba1 many taps": mamba1(20, 3, 9, 2),
    "mamba1 six taps": mamba1(28, 2, 6, 1, ff=16),
    "attention": attention(4, 2, 12, 12, 0.4, 7),
    "attention wide values": attention(3, 3, 8, 24, 1.3, 50, ff=32),
    "attention narrow values, one kv head": attention(5, 1, 20, 4, 0.05, 3),
    "attention window of one": attention(2, 2, 16, 16, 0.25, 1),
    "attention, heads of 32 in fours": attention(4, 1, 32, 32, 0.2, 21),
    "attention, heads of 128": attention(6, 2, 128, 128, 0.09, 70, ff=48),
    "attention, heads of 64, window of a page": attention(8, 4, 64, 64, 0.11, 16),
    "attention, heads of 64 in threes": attention(6, 2, 64, 64, 0.13, 29),
    "attention, heads of 32, fourteen to a key head": attention(14, 1, 32, 32, 0.3, 40),
    "attention, heads of 96": attention(4, 2, 96, 96, 0.1, 23),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", list(ALONE))
def test_one_layer_of_each_kind(which, dtype):
    for streams, groups in ((1, 1), (2, 4), (5, 2)):
        cfg = one_layer(ALONE[which], streams=streams, groups=groups)
        typed, tensors = make_model(cfg, seed=streams)
        requests = {"a": random_tokens(cfg["vocab"], 45, 1), "b": random_tokens(cfg["vocab"], 3, 2)}
        run_regimes(cfg, typed, tensors, dtype, 4, requests,
                    {"whole": whole(requests), "decoded": tail_decoded(requests, tail=20), "portions": portions(requests, (2, 5, 2, 9, 3))})


# ---- whole models in every regime -----------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", list(CONFIGS))
def test_replay_regimes(which, dtype):
    cfg = CONFIGS[which]
    typed, tensors = make_model(cfg, seed=3)
    lengths = [1, 2, 23, 70, 131, 40, 17]          # more requests than slots: slots and pages are used again
    requests = {f"r{i}": random_tokens(cfg["vocab"], n, 10 + i) for i, n in enumerate(lengths)}
    run_regimes(cfg, typed, tensors, dtype, PAGE_SIZE[which], requests,
                {"whole": whole(requests), "decoded": tail_decoded(requests, tail=32), "portions": portions(requests),
                 "portions of two and three": portions(requests, (2, 3)), "mixed": mixed(requests, live=4),
                 "mixed, two live": mixed(requests, live=2, prefill_sizes=(2, 31, 4))})


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_batch_of_unequal_requests_equals_each_alone(dtype):
    cfg = CONFIGS["odd"]
    typed, tensors = make_model(cfg, seed=5)
    requests = {"long": random_tokens(cfg["vocab"], 90, 1), "short": random_tokens(cfg["vocab"], 2, 2),
                "one": random_tokens(cfg["vocab"], 1, 3), "mid": random_tokens(cfg["vocab"], 33, 4)}
    eng = engine_for(typed, tensors, dtype, 4, 4 * 128)
    together = [{"step": 0, "entries": [{"id": r, "tokens": t, "want": list(range(len(t)))} for r, t in requests.items()], "end": list(requests)}]
    rows_together = replay(eng, together)
    rows_alone = replay(eng, whole(requests))        # the same engine: the slots and pages of the batch, used again
    exact = reference(cfg, tensors, requests)
    allowed = allowed_error(dtype, cfg, tensors, requests, exact)
    check_rows(rows_together, exact, requests, allowed, "together")
    check_rows(rows_alone, exact, requests, allowed, "alone")
    for rid, toks in requests.items():            # and beyond rounding, being in a batch changes nothing
        for p in range(len(toks)):
            d = float((rows_together[rid][p] - rows_alone[rid][p]).abs().max()) / float(exact[rid].abs().max())
            assert d <= allowed, (rid, p, d)


# ---- inputs under which an edge shows ------------------------------------------------------------------------------

def marked_attention_model(window, dim=16, vdim=12, heads=2, kv_heads=1, scale=2.0, width=32, vocab=50, mark=7):
    """One attention layer in which the key of token `mark` stands out for every query: q's bias points where that
    key points, so the marked key scores scale * dim and any other key about scale * sqrt(dim) * N(0, 1); with the
    marked token inside the window the output is its value, outside it a mix of the others."""
    cfg = config(width, vocab, 2, 2, 4.0, [attention(heads, kv_heads, dim, vdim, scale, window)])

    def change(t):
        x = t["embed"].double()[mark] * 4.0 * float(t["l0.hc1.in"].double().sum())
        h = plain_group_rmsnorm(x, t["l0.norm1"].double(), 1e-5, 2)
        key = (t["l0.mix.k"].double() @ h + t["l0.mix.k.b"].double()).reshape(kv_heads, dim)
        t["l0.mix.q.b"] = (50.0 * key.repeat_interleave(heads // kv_heads, dim=0).reshape(-1)).to(torch.bfloat16)
        t["l0.mix.v"] = (t["l0.mix.v"].double() * 20.0).to(torch.bfloat16)      # values that tell tokens apart in the logits
        t["l0.mix.o"] = (t["l0.mix.o"].double() * 20.0).to(torch.bfloat16)
    typed, tensors = make_model(cfg, seed=11, change=change)
    return cfg, typed, tensors


def sequence_with_mark(vocab, n, at, mark, seed):
    toks = [t if t != mark else (t + 1) % vocab for t in random_tokens(vocab, n, seed)]
    toks[at] = mark
    return toks


# head shapes: values narrower than keys (the kernel for any sizes) and heads the matrix-core kernels take
HEAD_SHAPES = {"any sizes": dict(dim=16, vdim=12, heads=2, kv_heads=1, width=32), "matrix cores": dict(dim=64, vdim=64, heads=4, kv_heads=2, width=64)}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", list(HEAD_SHAPES))
@pytest.mark.parametrize("window,at", [(9, 3), (16, 0), (17, 15), (33, 16), (40, 31), (64, 1), (65, 30)])
def test_a_key_just_inside_and_just_outside_the_window(window, at, shape, dtype):
    cfg, typed, tensors = marked_attention_model(window, **HEAD_SHAPES[shape])
    toks = sequence_with_mark(cfg["vocab"], at + window + 6, at, 7, seed=window)
    requests = {"m": toks}
    exact = reference(cfg, tensors, requests)
    inside, outside = at + window - 1, at + window
    # the plain decoder itself: the marked key's leaving the window moves the logits by much more than any bound below
    gap = float((exact["m"][inside] - exact["m"][outside]).abs().max()) / float(exact["m"].abs().max())
    unmarked = {"m": [t if i != at else (t + 2) % cfg["vocab"] for i, t in enumerate(toks)]}
    moved = float((reference(cfg, tensors, unmarked)["m"][inside] - exact["m"][inside]).abs().max()) / float(exact["m"].abs().max())
    assert gap > 0.05 and moved > 0.05, (gap, moved)
    allowed = allowed_error(dtype, cfg, tensors, requests, exact)
    assert allowed < min(gap, moved) / 2, (allowed, gap, moved)
    regimes = {"whole": whole(requests), "decoded over the edge": tail_decoded(requests, tail=8),
               "portions of two": portions(requests, (2,)), "a portion that ends inside": portions(requests, (inside + 1, 1, 2)),
               "a portion that starts outside": portions(requests, (outside, 3))}
    for name, steps in regimes.items():
        eng = engine_for(typed, tensors, dtype, 16, 256)
        check_rows(replay(eng, steps), exact, requests, allowed, name)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", list(HEAD_SHAPES))
def test_a_far_key_among_hundreds_across_pages(shape, dtype):
    cfg, typed, tensors = marked_attention_model(window=1000, **HEAD_SHAPES[shape])
    for at in (0, 15, 16, 250):
        toks = sequence_with_mark(cfg["vocab"], 600, at, 7, seed=at)
        requests = {"m": toks}
        exact = reference(cfg, tensors, requests)
        unmarked = {"m": [t if i != at else (t + 2) % cfg["vocab"] for i, t in enumerate(toks)]}
        moved = float((reference(cfg, tensors, unmarked)["m"][599] - exact["m"][599]).abs().max()) / float(exact["m"].abs().max())
        assert moved > 0.05, moved
        allowed = allowed_error(dtype, cfg, tensors, requests, exact)
        for name, steps in {"whole": whole(requests), "decoded": tail_decoded(requests, tail=40),
                            "portions": portions(requests, (64, 3, 130, 2))}.items():
            eng = engine_for(typed, tensors, dtype, 16, 640)
            check_rows(replay(eng, steps), exact, requests, allowed, f"mark at {at}, {name}")


def held_state(t, dt_rank=2):
    """Two marked tokens (the last two ids) carry features that no other token has: feature 0 opens the recurrence
    for them (a gate near 1, an input many times the others'), feature 1 tells them apart; every other token leaves
    the state nearly as it was (gates near 0, slow decay), and what reads the state is made large enough to show."""
    e = t["embed"].double()
    e[:, 0:2] = 0.0
    e[-2, 0], e[-2, 1], e[-1, 0], e[-1, 1] = 1.0, 1.0, 1.0, -1.0
    t["embed"] = e.to(torch.bfloat16)
    g = torch.Generator().manual_seed(0)
    signs = lambda n: torch.sign(torch.randn(n, generator=g, dtype=torch.float64))
    for name in list(t):
        w = t[name].double()
        if name.endswith(".mix.z.b"): w = torch.full_like(w, -12.0)
        elif name.endswith(".mix.z"): w[:, 0] = 8.0
        elif name.endswith(".mix.x") and w.shape[1] == e.shape[1]: w[:, 1] = signs(w.shape[0]) * 3.0      # minGRU's candidate
        elif name.endswith(".mix.x"): w[dt_rank:] *= 20                                                   # the scan's B and C
        elif name.endswith((".mix.g", ".mix.o")): w = w * 20
        elif name.endswith(".mix.in"):
            C = w.shape[0] // 2
            w[C:] *= 20
            w[:C, 0] = 5.0
            w[:C, 1] = signs(C) * 2.0
        elif name.endswith(".mix.conv"): w = w.abs()
        elif name.endswith(".mix.dt.b"): w = torch.full_like(w, -3.0)
        elif name.endswith(".mix.A_log"): w = torch.full_like(w, -5.0)
        else: continue
        t[name] = w.to(torch.bfloat16)


def long_memory(t):
    """Gates and step sizes so small that a state holds what it saw long ago."""
    for name in t:
        if name.endswith(".mix.z.b"):
            t[name] = torch.full_like(t[name], -5.0)
        if name.endswith(".mix.dt.b"):
            t[name] = torch.full_like(t[name], -6.0)
        if name.endswith(".mix.A_log"):
            t[name] = torch.full_like(t[name], -3.0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("layer", ["mingru", "mamba1"])
def test_the_first_token_is_still_in_the_state_after_hundreds(layer, dtype):
    cfg = one_layer(mingru(24) if layer == "mingru" else mamba1(24, 4, 3, 2), width=32, vocab=40)
    typed, tensors = make_model(cfg, seed=2, change=held_state)
    toks = [38] + [t % 38 for t in random_tokens(40, 299, 9)]
    other = [39] + toks[1:]
    requests = {"a": toks, "b": other}
    exact = reference(cfg, tensors, requests)
    moved = float((exact["a"][299] - exact["b"][299]).abs().max()) / float(exact["a"].abs().max())
    allowed = allowed_error(dtype, cfg, tensors, requests, exact)
    assert moved > 0.05 and allowed < moved / 2, (moved, allowed)          # what the first token was still shows at the end
    for name, steps in {"whole": whole(requests), "decoded": tail_decoded(requests, tail=64), "portions": portions(requests, (2, 97, 3, 50)),
                        "both at once": mixed(requests, live=2, prefill_sizes=(40, 2, 7))}.items():
        eng = engine_for(typed, tensors, dtype, 16, 1024)
        check_rows(replay(eng, steps), exact, requests, allowed, name)


@pytest.fixture
def chunk_length(request):
    from llm_rs_amd.kernels import kernels
    kernels().scan_set_chunk(request.param)
    yield request.param
    kernels().scan_set_chunk(0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk_length", [32, 64], indirect=True)
@pytest.mark.parametrize("layer", ["mingru", "mamba1", "mamba1 many states"])
def test_portions_longer_than_a_chunk_of_the_recurrences(layer, chunk_length, dtype):
    """Entries of 64 tokens and more run their recurrences in chunks side by side: lengths at the chunks' edges, side
    by side with short entries in one step, portions that start in the middle of a sequence, and a state (slow gates,
    slow decay) in which everything before still counts."""
    mixer = {"mingru": mingru(70), "mamba1": mamba1(72, 5, 4, 3), "mamba1 many states": mamba1(10, 70, 2, 2)}[layer]
    cfg = one_layer(mixer, width=32, vocab=40)
    typed, tensors = make_model(cfg, seed=8, change=long_memory)
    lengths = {"a": 64, "b": 65, "c": 128, "d": 129, "e": 200, "f": 1, "g": 3, "h": 321}
    requests = {r: random_tokens(40, n, 20 + i) for i, (r, n) in enumerate(lengths.items())}
    exact = reference(cfg, tensors, requests)
    allowed = allowed_error(dtype, cfg, tensors, requests, exact)
    together = [{"step": 0, "entries": [{"id": r, "tokens": t, "want": list(range(len(t)))} for r, t in requests.items()], "end": list(requests)}]
    eng = engine_for(typed, tensors, dtype, 16, sum(-(-n // 16) * 16 for n in lengths.values()), max_requests=8)
    check_rows(replay(eng, together), exact, requests, allowed, "together")
    for name, steps in {"whole": whole(requests), "portions": portions(requests, (3, 66, 2, 127, 64, 65)),
                        "mixed": mixed(requests, live=3, prefill_sizes=(70, 2, 130))}.items():
        eng = engine_for(typed, tensors, dtype, 16, live_token_need(steps, 64))
        check_rows(replay(eng, steps), exact, requests, allowed, name)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_slot_used_again_starts_from_nothing(dtype):
    cfg = CONFIGS["plain"]
    typed, tensors = make_model(cfg, seed=4, change=long_memory)
    first, second = random_tokens(cfg["vocab"], 50, 1), random_tokens(cfg["vocab"], 30, 2)
    eng = Engine(typed, tensors, dtype=dtype, page_size=16, num_pages=8, max_requests=1)      # one slot, pages for one request
    exact = reference(cfg, tensors, {"first": first, "second": second})
    allowed = allowed_error(dtype, cfg, tensors, {"first": first, "second": second}, exact)
    for rid, toks in (("first", first), ("second", second), ("first", first)):
        slot = eng.open_request()
        assert slot == 0
        head = eng.step([StepEntry(slot, 0, toks[:20], list(range(20)))]).cpu().clone()
        tail = eng.step([StepEntry(slot, 20, toks[20:], list(range(len(toks) - 20)))]).cpu()
        eng.close_request(slot)
        got = torch.cat([head, tail]).double()
        err = float((got - exact[rid]).abs().max()) / float(exact[rid].abs().max())
        assert err <= allowed, (rid, err, allowed)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_with_recorded_steps(dtype):
    cfg = CONFIGS["odd"]
    typed, tensors = make_model(cfg, seed=6)
    requests = {"a": random_tokens(cfg["vocab"], 330, 1), "b": random_tokens(cfg["vocab"], 321, 2)}
    exact = reference(cfg, tensors, requests)
    allowed = allowed_error(dtype, cfg, tensors, requests, exact)
    steps = [{"step": 0, "entries": [{"id": r, "tokens": t[:9], "want": list(range(9))} for r, t in requests.items()], "end": []}]
    for i in range(9, 330):
        live = [r for r, t in requests.items() if i < len(t)]
        steps.append({"step": len(steps), "entries": [{"id": r, "tokens": [requests[r][i]], "want": [0]} for r in live],
                      "end": [r for r in live if i == len(requests[r]) - 1]})
    eng = engine_for(typed, tensors, dtype, 4, 704)
    check_rows(replay(eng, steps), exact, requests, allowed, "decoding")
    assert eng.runner.graph_replays > 100           # the single-token steps were recorded and replayed


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("streams,width,groups", [(5, 42, 3), (2, 40, 2), (4, 36, 1), (1, 44, 2)])
def test_steps_of_many_rows_mix_the_streams_inside_the_next_norm(streams, width, groups, dtype):
    """From 128 rows on, a sublayer's mix of the streams runs in the launch of the norm that reads them next: rows of
    a length that is and is not a multiple of four, few and many streams, steps just below and above that bound."""
    cfg = config(width, 53, streams, groups, 1.5, [mingru(24, ff=32), attention(2, 1, 8, 8, 0.5, 11), mamba1(16, 3, 2, 2, ff=20)])
    typed, tensors = make_model(cfg, seed=streams)
    requests = {"a": random_tokens(53, 127, 1), "b": random_tokens(53, 128, 2), "c": random_tokens(53, 300, 3)}
    run_regimes(cfg, typed, tensors, dtype, 16, requests,
                {"whole": whole(requests), "portions": portions(requests, (128, 2, 129, 41))})


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_step_of_more_than_a_thousand_tokens(dtype):
    """Steps this long take the convolution several tokens a block: a long portion beside a short one, both continued
    in the next step, over narrow and wide channels and several tap counts."""
    cfg = config(32, 40, 2, 2, 2.0, [mamba1(72, 5, 4, 3), mamba1(320, 4, 3, 2), mingru(40), mamba1(24, 20, 2, 2, ff=48)])
    typed, tensors = make_model(cfg, seed=12)
    requests = {"a": random_tokens(40, 1100, 1), "b": random_tokens(40, 40, 2)}
    exact = reference(cfg, tensors, requests)
    allowed = allowed_error(dtype, cfg, tensors, requests, exact)
    cuts = {"a": 1031, "b": 5}
    steps = [{"step": 0, "entries": [{"id": r, "tokens": t[:cuts[r]], "want": list(range(cuts[r]))} for r, t in requests.items()], "end": []},
             {"step": 1, "entries": [{"id": r, "tokens": t[cuts[r]:], "want": list(range(len(t) - cuts[r]))} for r, t in requests.items()], "end": list(requests)}]
    eng = engine_for(typed, tensors, dtype, 16, 1280)
    check_rows(replay(eng, steps), exact, requests, allowed, "two steps")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["even", "odd"])
def test_sizes_that_are_no_multiples_of_four(which, dtype):
    """No vector load fits these rows: every kernel's narrow path, also in steps long enough for chunks and fused norms."""
    cfg = {"even": config(46, 51, 3, 2, 1.0, [mingru(30), mamba1(26, 3, 3, 3, ff=22), attention(3, 1, 10, 6, 0.3, 9, ff=14)]),
           "odd": config(45, 37, 2, 3, 2.5, [attention(2, 2, 7, 5, 0.4, 6), mingru(17, ff=9), mamba1(15, 5, 2, 1)])}[which]
    typed, tensors = make_model(cfg, seed=13)
    requests = {"a": random_tokens(cfg["vocab"], 140, 1), "b": random_tokens(cfg["vocab"], 21, 2), "c": random_tokens(cfg["vocab"], 2, 3)}
    run_regimes(cfg, typed, tensors, dtype, 16, requests,
                {"whole": whole(requests), "decoded": tail_decoded(requests, tail=20), "portions": portions(requests, (3, 131, 2)),
                 "mixed": mixed(requests, live=3)})


# ---- configurations drawn at random -----------------------------------------------------------------------------------

def random_configuration(seed):
    import random
    r = random.Random(seed)
    width = r.choice([24, 40, 64, 96, 136])
    groups = r.choice([g for g in (1, 2, 3, 4, 8) if width % g == 0])
    layers = []
    for _ in range(r.randint(2, 5)):
        ff = r.choice([None, None, 8 * r.randint(2, 12)])
        kind = r.choice(["mingru", "mamba1", "attention"])
        if kind == "mingru":
            layers.append(mingru(4 * r.randint(3, 30), ff=ff))
        elif kind == "mamba1":
            layers.append(mamba1(4 * r.randint(3, 30), r.choice([1, 4, 16, 24, 33, 70]), r.randint(1, 5), r.randint(1, 9), ff=ff))
        else:
            kv = r.choice([1, 2, 3])
            dim = r.choice([8, 20, 32, 64, 128])
            vdim = r.choice([dim, dim, 4 * r.randint(1, 10)])
            layers.append(attention(kv * r.choice([1, 2, 4]), kv, dim, vdim, r.uniform(0.05, 0.5), r.choice([1, 5, 16, 17, 31, 32, 48, 100, 500]), ff=ff))
    return config(width, r.randint(30, 200), r.randint(1, 6), groups, r.uniform(0.5, 10.0), layers, eps=r.choice([1e-5, 1e-6, 1e-3]))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(seed, dtype):
    cfg = random_configuration(seed)
    typed, tensors = make_model(cfg, seed=seed)
    requests = {f"r{i}": random_tokens(cfg["vocab"], n, 70 + i) for i, n in enumerate([150, 3, 66, 1, 35])}
    run_regimes(cfg, typed, tensors, dtype, 16, requests,
                {"whole": whole(requests), "decoded": tail_decoded(requests, tail=36), "portions": portions(requests, (2, 70, 3, 33)),
                 "mixed": mixed(requests, live=3)})


# ---- generation through the scheduler --------------------------------------------------------------------------------

def plain_greedy(cfg, tensors, prompt, n):
    toks, margins = list(prompt), []
    for _ in range(n):
        row = plain_tuvodra_logits(cfg, tensors, toks)[-1]
        top = torch.topk(row, 2).values
        margins.append(float(top[0] - top[1]) / float(row.abs().max()))
        toks.append(int(torch.argmax(row)))
    return toks[len(prompt):], margins


@pytest.mark.parametrize("which", ["odd", "plain"])
def test_greedy_generation_through_the_scheduler(which):
    cfg = CONFIGS[which]
    typed, tensors = make_model(cfg, seed=8)
    prompts = [random_tokens(cfg["vocab"], n, 20 + n) for n in (1, 5, 19, 40, 3, 27)]
    eng = Engine(typed, tensors, dtype="float32", page_size=PAGE_SIZE[which], num_pages=64, max_requests=3, max_batch_tokens=24)
    outs = eng.generate(prompts, max_new_tokens=12)
    for prompt, out in zip(prompts, outs):
        want, margins = plain_greedy(cfg, tensors, prompt, 12)
        out = list(out.tokens if hasattr(out, "tokens") else out)
        for i, (a, b) in enumerate(zip(out, want)):
            if a != b:
                assert margins[i] < 1e-4, (prompt, i, out, want)       # a tie within rounding may fall either way
                break


# ---- the programs, on a model folder ----------------------------------------------------------------------------------

def test_the_programs_on_a_model_folder(tmp_path):
    """A folder with config.json and model.safetensors through `bin/trace_run` (a mixed trace under a small pool, both
    dtypes) and through `bin/llm-rs complete` (greedy): the architecture is chosen by the file."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np
    from tuvodra_cases import make_folder
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = CONFIGS["plain"]
    folder = make_folder(tmp_path, cfg, seed=11)
    typed, tensors = make_model(cfg, seed=11)
    requests = {f"r{i}": random_tokens(cfg["vocab"], n, 50 + i) for i, n in enumerate([33, 2, 90, 47, 18])}
    exact = reference(cfg, tensors, requests)
    steps = mixed(requests, live=3)
    text = "".join(json.dumps(s) + "\n" for s in steps)
    for dtype in DTYPES:
        out = tmp_path / f"out_{dtype}"
        p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out),
                            "--max-tokens", str(live_token_need(steps, 64))], input=text, capture_output=True, text=True, timeout=600)
        assert p.returncode == 0, p.stderr[-2000:]
        assert [l for l in p.stdout.split("\n") if l.startswith("done")] == [f"done {s['step']}" for s in steps]
        outputs = []
        for s in steps:
            n = sum(len(e["want"]) for e in s["entries"])
            outputs.append(torch.from_numpy(np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(n, cfg["vocab"]).copy()) if n else None)
        check_rows(collect(steps, outputs), exact, requests, allowed_error(dtype, cfg, tensors, requests, exact), f"trace_run {dtype}")
    prompt = requests["r3"]
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "llm-rs"), "-m", folder, "--dtype", "float32", "--num-pages", "64", "complete",
                        "--prompt-ids", " ".join(map(str, prompt)), "-n", "10", "--temperature", "0"], capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    got = [int(t) for t in p.stdout.split()]
    want, margins = plain_greedy(cfg, tensors, prompt, 10)
    for i, (a, b) in enumerate(zip(got, want)):
        if a != b:
            assert margins[i] < 1e-4, (i, got, want)
            break
    assert len(got) == 10
