"""The Lilatar decoder in the engine against the plain decoder (plain_lilatar.py): the new kernels one by one, every
mechanism alone, the replay regimes (whole prompts, decoding through the cache and the state, portions down to two
tokens, mixed batches under a pool and slots that are used again), inputs made so that a window's edge, a kept first
token, a far key or a long-held state shows in the logits, long decoding, and greedy generation through the scheduler."""
from __future__ import annotations

import pytest
import torch

from emulated_kernels import EmulatedKernels
from llm_rs_amd import Engine, StepEntry
from llm_rs_amd.engine.trace import TraceReplayer
from llm_rs_amd.kernels import kernels
from lilatar_cases import (CONFIGS, PAGE_SIZE, SCALED, allowed_error, check_rows, config, dense, left, lightning, make_folder, make_model,
                           moe, one_layer, parallel, reference, right)
from plain_lilatar import plain_lilatar_logits, plain_rmsnorm
from replay_cases import collect, live_token_need, mixed, portions, random_tokens, tail_decoded, whole

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


def run_regimes(cfg, typed, tensors, dtype, page_size, requests, regimes, allowed=None):
    exact = reference(cfg, tensors, requests)
    allowed = allowed if allowed is not None else allowed_error(dtype, cfg, tensors, requests, exact)
    for name, steps in regimes.items():
        eng = engine_for(typed, tensors, dtype, page_size, live_token_need(steps, 64))
        check_rows(replay(eng, steps), exact, requests, allowed, name)
        core = eng.cache.core
        assert core.slots_in_use() == 0 and all(core.pages_free(g) == core.pages_total(g) for g in range(core.n_groups)), name


# ---- the kernels one by one, against the same operation in plain tensor code ---------------------------------------

def entries_of(lengths, slots):
    starts = [0]
    for n in lengths:
        starts.append(starts[-1] + n)
    dev = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
    return dev(starts), dev(slots), torch.tensor(starts, dtype=torch.int32), torch.tensor(slots, dtype=torch.int32)


@pytest.mark.parametrize("heads,qk_heads,dk,dv", [(1, 1, 1, 1), (3, 1, 5, 7), (4, 2, 16, 33), (2, 2, 32, 32), (2, 1, 64, 40), (6, 3, 100, 12),
                                                  (2, 2, 128, 128), (1, 1, 256, 64), (2, 1, 36, 130)])
@pytest.mark.parametrize("kind", ["decay", "none", "delta", "delta by channel", "decay by channel"])
def test_linear_scan(heads, qk_heads, dk, dv, kind):
    g = torch.Generator().manual_seed(dk * 7 + dv)
    lengths, slots = [37, 1, 2, 64], [2, 0, 5, 3]
    T = sum(lengths)
    r = lambda *s: torch.randn(*s, generator=g)
    q, k, v = r(T, qk_heads * dk) * 0.5, r(T, qk_heads * dk) * 0.5, r(T, heads * dv)
    state = r(6, heads * dk * dv + 3) * 0.3           # (a slot's row is longer than the state: what follows is another's)
    decay = torch.rand(heads, generator=g) * 0.5 + 0.5 if kind == "decay" else None
    chan = torch.rand(T, heads * dk, generator=g) * 0.3 + 0.7 if "by channel" in kind else None
    beta = torch.rand(T, heads, generator=g) if "delta" in kind else None
    if "delta" in kind:      # unit keys keep the rule contractive
        k = (k.view(T, qk_heads, dk) / k.view(T, qk_heads, dk).norm(dim=-1, keepdim=True)).reshape(T, -1)
    qs_d, sl_d, qs_h, sl_h = entries_of(lengths, slots)
    want_state, want = state.double(), torch.zeros(T, heads * dv, dtype=torch.float64)
    dbl = lambda t: None if t is None else t.double()
    EmulatedKernels().linear_scan(q.double(), k.double(), v.double(), want_state, qs_h, sl_h, heads, qk_heads, dk, dv, want,
                                  decay=dbl(decay), g=dbl(chan), beta=dbl(beta))
    cuda = lambda t: None if t is None else t.cuda()
    got_state, got = state.cuda(), torch.empty(T, heads * dv, device="cuda")
    kernels().linear_scan(q.cuda(), k.cuda(), v.cuda(), got_state, qs_d, sl_d, heads, qk_heads, dk, dv, got, decay=cuda(decay), g=cuda(chan), beta=cuda(beta))
    scale = float(want.abs().max())
    assert float((got.cpu().double() - want).abs().max()) <= 2e-5 * scale
    assert float((got_state.cpu().double() - want_state).abs().max()) <= 2e-5 * max(float(want_state.abs().max()), 1.0)
    assert torch.equal(got_state.cpu()[[1, 4]], state[[1, 4]]) and torch.equal(got_state.cpu()[:, -3:], state[:, -3:])     # other rows untouched


def test_linear_scan_on_rows_inside_wider_rows():
    """q, k and v as column ranges of one wider buffer whose row length is no multiple of four."""
    g = torch.Generator().manual_seed(1)
    heads, dk, dv, T = 2, 8, 6, 19
    buf = torch.randn(T, 2 * heads * dk + heads * dv + 3, generator=g)
    q, k, v = buf[:, 1:1 + heads * dk], buf[:, 1 + heads * dk:1 + 2 * heads * dk], buf[:, 1 + 2 * heads * dk:1 + 2 * heads * dk + heads * dv]
    qs_d, sl_d, qs_h, sl_h = entries_of([T], [0])
    want_state, want = torch.zeros(1, heads * dk * dv, dtype=torch.float64), torch.zeros(T, heads * dv, dtype=torch.float64)
    decay = torch.tensor([0.9, 0.5])
    EmulatedKernels().linear_scan(q.double(), k.double(), v.double(), want_state, qs_h, sl_h, heads, heads, dk, dv, want, decay=decay.double())
    d = buf.cuda()
    got_state, got = torch.zeros(1, heads * dk * dv, device="cuda"), torch.empty(T, heads * dv, device="cuda")
    kernels().linear_scan(d[:, 1:1 + heads * dk], d[:, 1 + heads * dk:1 + 2 * heads * dk], d[:, 1 + 2 * heads * dk:1 + 2 * heads * dk + heads * dv],
                          got_state, qs_d, sl_d, heads, heads, dk, dv, got, decay=decay.cuda())
    assert float((got.cpu().double() - want).abs().max()) <= 2e-5 * float(want.abs().max())


@pytest.mark.parametrize("E,top,renormalize", [(1, 1, False), (5, 5, False), (16, 4, False), (64, 7, True), (100, 3, False), (300, 9, True)])
def test_route_topk(E, top, renormalize):
    g = torch.Generator().manual_seed(E)
    logits = torch.randn(33, E, generator=g) * 3
    logits[0] = 0.0                          # all equal: the lowest indices are chosen
    if E > 3:
        logits[1, [E - 1, 2]] = 50.0         # two equal maxima
    want = torch.zeros(33, E)
    EmulatedKernels().route_topk(logits, want, top, renormalize)
    got = torch.full((33, E), -1.0, device="cuda")
    kernels().route_topk(logits.cuda(), got, top, renormalize)
    assert torch.equal(got.cpu() > 0, want > 0)
    assert float((got.cpu() - want).abs().max()) <= 1e-6
    assert (got.cpu()[0] > 0).nonzero().flatten().tolist() == list(range(top))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_small_kernels_around_the_recurrences(dtype):
    g = torch.Generator().manual_seed(0)
    emu, k = EmulatedKernels(), kernels()
    T = 21
    # the norm in groups under a gate: a weight per column of a group, and of the row
    for groups, width, per_row in ((3, 10, False), (1, 70, True), (4, 64, False), (2, 300, True)):
        x, gate = torch.randn(T, groups * width, generator=g), torch.randn(T, groups * width, generator=g)
        w = torch.randn(groups * width if per_row else width, generator=g)
        group = groups * width if per_row else width
        want, got = torch.empty(T, groups * width), torch.empty(T, groups * width, dtype=dtype, device="cuda")
        emu.gated_rmsnorm(want, x, gate, w, group, 1e-5)
        k.gated_rmsnorm(got, x.cuda(), gate.cuda(), w.cuda(), group, 1e-5)
        assert float((got.cpu().float() - want).abs().max()) <= (1e-5 if dtype == torch.float32 else 1e-2) * float(want.abs().max())
    # sums of normed rows into the stream, one and two inputs, with and without a bias
    for D, T in ((7, 21), (64, 21), (1000, 21), (1030, 21), (4100, 21), (72, 300)):       # (few rows and many: two ways through the rows)
        for n_in in (1, 2):
            ins = [(torch.randn(T, D, generator=g), torch.randn(D, generator=g) if i == 0 and D != 64 else None, torch.randn(D, generator=g)) for i in range(n_in)]
            base = torch.randn(T, D, generator=g)
            want, got = base.clone(), base.cuda()
            emu.rmsnorm_sum(want, ins, 1.0 / n_in, 1e-6)
            k.rmsnorm_sum(got, [tuple(None if t is None else t.cuda() for t in row) for row in ins], 1.0 / n_in, 1e-6)
            assert float((got.cpu() - want).abs().max()) <= 1e-5 * float(want.abs().max())
    # squared relu times the expert's weight
    up, w = torch.randn(T, 5 * 12, generator=g), torch.rand(T, 5, generator=g)
    for weights in (None, w):
        want, got = torch.empty(T, 60), torch.empty(T, 60, dtype=dtype, device="cuda")
        emu.act_weight(want, up, weights, 12)
        k.act_weight(got, up.cuda(), None if weights is None else weights.cuda(), 12)
        assert float((got.cpu().float() - want).abs().max()) <= (1e-6 if dtype == torch.float32 else 1e-2) * float(want.abs().max())
    # what the delta rule needs: unit vectors, decays, write strengths
    heads, qk_heads, dk = 4, 2, 9
    q, kk = torch.randn(T, qk_heads * dk, generator=g), torch.randn(T, qk_heads * dk, generator=g)
    a, b = torch.randn(T, heads * dk, generator=g) * 3, torch.randn(T, heads, generator=g) * 3
    A_log, dt_bias = torch.randn(heads, generator=g), torch.randn(heads * dk, generator=g)
    want = [t.clone() for t in (q, kk, a, b)]
    got = [t.cuda() for t in (q, kk, a, b)]
    emu.delta_prepare(*want, A_log, dt_bias, heads, qk_heads, dk, 1e-6)
    k.delta_prepare(*got, A_log.cuda(), dt_bias.cuda(), heads, qk_heads, dk, 1e-6)
    for w_, g_ in zip(want, got):
        assert float((g_.cpu() - w_).abs().max()) <= 2e-6
    x = torch.randn(T, 30, generator=g)
    want, got = x.clone(), x.cuda()
    emu.silu_columns(want, 4, 20)
    k.silu_columns(got, 4, 20)
    assert float((got.cpu() - want).abs().max()) <= 1e-6 and torch.equal(got.cpu()[:, :4], x[:, :4]) and torch.equal(got.cpu()[:, 24:], x[:, 24:])


# ---- each mechanism alone -----------------------------------------------------------------------------------------

L0, R0 = left(4, 2, 12, 12, 0.4, 20.0, 7, 2, rot_dims=6), right(2, 1, 8, 6, 3)
ALONE = {
    "lightning": lightning(3, 8, 6),
    "lightning, one head, slow decay, dense ff": lightning(1, 20, 12, [0.999], mlp=dense(24)),
    "lightning, no decay at all": lightning(2, 6, 10, [1.0, 1.0]),
    "lightning, heads of 64": lightning(2, 64, 64, mlp=dense(48)),
    "lightning, wide keys": lightning(1, 130, 3),
    "attention beside a delta rule": parallel(L0, R0),
    "no rotation, no kept tokens, wide values": parallel(left(3, 3, 8, 24, 1.3, 5.0, 50, 0, rot_dims=0), R0, dense(32)),
    "full rotation with scaled frequencies, one kv head": parallel(left(5, 1, 20, 4, 0.05, 100.0, 3, 1, scaling=SCALED, base=50.0), R0),
    "window of one with kept tokens": parallel(left(2, 2, 16, 16, 0.25, 30.0, 1, 3, rot_dims=4), R0),
    "more kept tokens than the window": parallel(left(2, 1, 16, 16, 0.25, 30.0, 5, 21, rot_dims=16), R0),
    "heads of 64 in pairs (matrix cores in 32-bit)": parallel(left(4, 2, 64, 64, 0.11, 20.0, 16, 4, rot_dims=32), R0, dense(16)),
    "heads of 32, seven to a key head": parallel(left(7, 1, 32, 32, 0.3, 8.0, 40, 2, rot_dims=10), R0),
    "heads of 128": parallel(left(2, 1, 128, 128, 0.09, 25.0, 70, 6, rot_dims=64), R0),
    "delta rule: one tap, rank one": parallel(L0, right(1, 1, 5, 9, 1, 1, 1)),
    "delta rule: five taps, many heads to a key head": parallel(L0, right(6, 2, 10, 4, 5, 7, 2), dense(20)),
    "delta rule: heads of 64 and 128": parallel(L0, right(2, 2, 64, 128, 4, 16, 16)),
    "experts: all chosen": lightning(2, 8, 8, mlp=moe(12, 3, 3)),
    "experts: one of one": lightning(2, 8, 8, mlp=moe(9, 1, 1)),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", list(ALONE))
def test_one_layer_of_each_kind(which, dtype):
    for width, scale in ((40, 2.0), (66, 1.0)):
        cfg = one_layer(ALONE[which], width=width, logit_scale=scale)
        typed, tensors = make_model(cfg, seed=width)
        requests = {"a": random_tokens(cfg["vocab"], 45, 1), "b": random_tokens(cfg["vocab"], 3, 2)}
        run_regimes(cfg, typed, tensors, dtype, 4, requests,
                    {"whole": whole(requests), "decoded": tail_decoded(requests, tail=20), "portions": portions(requests, (2, 5, 2, 9, 3))})


def routed_layer_margin(cfg, tensors, toks) -> float:
    """For a model of one lightning layer with experts: the router's smallest margin over the tokens."""
    from plain_lilatar import _under, plain_lightning
    w = {n: t.double() for n, t in tensors.items()}
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.tensor(toks)]
    lw = _under(w, "l0.")
    x = x + plain_rmsnorm(plain_lightning(plain_rmsnorm(x, lw["norm1"], eps), _under(lw, "mix."), cfg["layers"][0]["mixer"], eps), lw["norm1b"], eps)
    z = plain_rmsnorm(x, lw["norm2"], eps) @ lw["mlp.router"].T
    top = cfg["layers"][0]["mlp"]["router"]["top"]
    s = torch.sort(z, dim=-1, descending=True).values
    return float(((s[:, top - 1] - s[:, top]) / (s[:, 0] - s[:, -1])).min())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("experts,top", [(4, 1), (4, 2), (7, 3), (16, 4)])
def test_experts_of_which_some_are_chosen(experts, top, dtype):
    """Random weights put some token's last chosen expert and the next one within rounding of each other; the
    sequence is drawn again until no choice is that close, so that the comparison is of the arithmetic."""
    cfg = one_layer(lightning(2, 8, 8, mlp=moe(10, experts, top)), width=48)
    typed, tensors = make_model(cfg, seed=experts)
    need = 1e-4 if dtype == "float32" else 0.03
    for seed in range(400):
        toks = random_tokens(cfg["vocab"], 8 if dtype == "bfloat16" else 40, seed)
        if routed_layer_margin(cfg, tensors, toks) > need:
            break
    else:
        pytest.fail("no sequence with clear choices found")
    requests = {"a": toks}
    run_regimes(cfg, typed, tensors, dtype, 4, requests,
                {"whole": whole(requests), "decoded": tail_decoded(requests, tail=5), "portions": portions(requests, (2, 3))})


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("experts,top", [(4, 1), (5, 2), (16, 4)])
def test_experts_run_one_by_one_over_their_own_tokens(experts, top, dtype, monkeypatch):
    """Steps with prompt portions lay the chosen (token, expert) pairs out expert by expert (here from the first row on,
    not only for long steps); single decoded tokens beside them keep to the product over all experts."""
    from llm_rs_amd.parts import RoutedFF
    monkeypatch.setattr(RoutedFF, "SORT_FROM_ROWS", 0)
    monkeypatch.setattr(RoutedFF, "SORT_FROM_WEIGHT", 0)
    cfg = one_layer(lightning(2, 8, 8, mlp=moe(10, experts, top)), width=48)
    typed, tensors = make_model(cfg, seed=experts)
    need = 1e-4 if dtype == "float32" else 0.03
    found = []
    for seed in range(2000):
        toks = random_tokens(cfg["vocab"], 8 if dtype == "bfloat16" else 70, seed)
        if routed_layer_margin(cfg, tensors, toks) > need:
            found.append(toks)
            if len(found) == 3:
                break
    assert len(found) == 3, "no sequences with clear choices found"
    requests = {f"r{i}": t for i, t in enumerate(found)}
    run_regimes(cfg, typed, tensors, dtype, 4, requests,
                {"whole": whole(requests), "decoded": tail_decoded(requests, tail=5), "portions": portions(requests, (2, 3, 30)),
                 "mixed": mixed(requests, live=3, prefill_sizes=(3, 2, 9))})


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


# ---- inputs under which an edge shows ------------------------------------------------------------------------------

def marked_attention_model(window, keep_first, dim=16, vdim=12, heads=2, kv_heads=1, rot_dims=8, softcap=25.0, width=32, vocab=50, mark=7):
    """One parallel layer whose right branch is switched off (its output norm's weight is zero) and in whose left
    branch the key of token `mark` stands out for every query: on the features that are not rotated, q's bias points
    where that key points, so the marked key's score sits at the soft cap and every other key's near zero.  With the
    marked token visible the attention's output is its value, otherwise a mix of the others'."""
    cfg = one_layer(parallel(left(heads, kv_heads, dim, vdim, 1.0, softcap, window, keep_first, rot_dims=rot_dims), right(1, 1, 4, 4, 2, 1, 1)),
                    width=width, vocab=vocab)

    def change(t):
        h = plain_rmsnorm(t["embed"].double()[mark], t["l0.norm1"].double(), 1e-5)
        key = (t["l0.mix.left.k"].double() @ h + t["l0.mix.left.k.b"].double()).reshape(kv_heads, dim)
        key[:, :rot_dims] = 0.0
        t["l0.mix.left.q.b"] = (300.0 * key.repeat_interleave(heads // kv_heads, dim=0).reshape(-1)).to(torch.bfloat16)
        t["l0.mix.left.v"] = (t["l0.mix.left.v"].double() * 20.0).to(torch.bfloat16)      # values that tell tokens apart in the logits
        t["l0.mix.right.out"] = torch.zeros_like(t["l0.mix.right.out"])
    typed, tensors = make_model(cfg, seed=11, change=change)
    return cfg, typed, tensors


def sequence_with_mark(vocab, n, at, mark, seed):
    toks = [t if t != mark else (t + 1) % vocab for t in random_tokens(vocab, n, seed)]
    toks[at] = mark
    return toks


def shows(cfg, tensors, toks, at, where):
    """How far the logits at `where` move when the token at `at` is another one, as a part of the largest logit."""
    exact = reference(cfg, tensors, {"m": toks})["m"]
    other = [t if i != at else (t + 2) % cfg["vocab"] for i, t in enumerate(toks)]
    return float((reference(cfg, tensors, {"m": other})["m"][where] - exact[where]).abs().max()) / float(exact.abs().max())


# head shapes: values narrower than keys (the kernel for any sizes) and heads the matrix-core kernels take
HEAD_SHAPES = {"any sizes": dict(dim=16, vdim=12, heads=2, kv_heads=1, width=32, rot_dims=8),
               "matrix cores": dict(dim=64, vdim=64, heads=4, kv_heads=2, width=64, rot_dims=32),
               "matrix cores, heads of 128": dict(dim=128, vdim=128, heads=2, kv_heads=1, width=64, rot_dims=64),
               "matrix cores, heads of 32 in threes": dict(dim=32, vdim=32, heads=3, kv_heads=1, width=64, rot_dims=16),
               "matrix cores, twenty heads to a key head": dict(dim=32, vdim=32, heads=20, kv_heads=1, width=64, rot_dims=32)}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", list(HEAD_SHAPES))
@pytest.mark.parametrize("window,at", [(9, 3), (16, 2), (17, 15), (33, 16), (40, 31), (64, 1), (65, 30)])
def test_a_key_just_inside_and_just_outside_the_window(window, at, shape, dtype):
    keep = min(at, 2)           # the marked token is not among the kept ones
    cfg, typed, tensors = marked_attention_model(window, keep, **HEAD_SHAPES[shape])
    toks = sequence_with_mark(cfg["vocab"], at + window + 6, at, 7, seed=window)
    requests = {"m": toks}
    exact = reference(cfg, tensors, requests)
    inside, outside = at + window - 1, at + window
    seen, unseen = shows(cfg, tensors, toks, at, inside), shows(cfg, tensors, toks, at, outside)
    assert seen > 0.03 and unseen < 1e-9, (seen, unseen)
    allowed = allowed_error(dtype, cfg, tensors, requests, exact)
    assert allowed < seen / 2, (allowed, seen)
    regimes = {"whole": whole(requests), "decoded over the edge": tail_decoded(requests, tail=8),
               "portions of two": portions(requests, (2,)), "a portion that ends inside": portions(requests, (inside + 1, 1, 2)),
               "a portion that starts outside": portions(requests, (outside, 3))}
    for name, steps in regimes.items():
        eng = engine_for(typed, tensors, dtype, 16, 256)
        check_rows(replay(eng, steps), exact, requests, allowed, name)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", list(HEAD_SHAPES))
@pytest.mark.parametrize("keep,window", [(1, 5), (4, 16), (16, 16), (17, 3), (33, 40)])
def test_the_last_kept_token_and_the_first_that_is_not(keep, window, shape, dtype):
    """The marked token at the last kept position shows hundreds of tokens later, across many pages that the window has
    given back; at the next position it is gone as soon as the window has passed it."""
    cfg, typed, tensors = marked_attention_model(window, keep, **HEAD_SHAPES[shape])
    n = 300
    for at, stays in ((keep - 1, True), (keep, False), (0, True)):
        toks = sequence_with_mark(cfg["vocab"], n, at, 7, seed=keep + at)
        requests = {"m": toks}
        exact = reference(cfg, tensors, requests)
        late = shows(cfg, tensors, toks, at, n - 1)
        assert (late > 0.03) if stays else (late < 1e-9), (at, late)
        allowed = allowed_error(dtype, cfg, tensors, requests, exact)
        assert allowed < (late / 2 if stays else 0.2), (allowed, late)      # (less than half of what the marked token moves where it is seen)
        for name, steps in {"whole": whole(requests), "decoded": tail_decoded(requests, tail=40), "portions": portions(requests, (64, 3, 130, 2)),
                            "portions of two": portions(requests, (2,)) if keep == 4 else None}.items():
            if steps is None:
                continue
            eng = engine_for(typed, tensors, dtype, 16, 320)
            check_rows(replay(eng, steps), exact, requests, allowed, f"mark at {at}, {name}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_key_among_hundreds_across_pages(dtype):
    cfg, typed, tensors = marked_attention_model(1000, 0, **HEAD_SHAPES["matrix cores"])
    for at in (0, 15, 16, 250):
        toks = sequence_with_mark(cfg["vocab"], 600, at, 7, seed=at)
        requests = {"m": toks}
        exact = reference(cfg, tensors, requests)
        assert shows(cfg, tensors, toks, at, 599) > 0.05
        allowed = allowed_error(dtype, cfg, tensors, requests, exact)
        for name, steps in {"whole": whole(requests), "decoded": tail_decoded(requests, tail=40),
                            "portions": portions(requests, (64, 3, 130, 2))}.items():
            eng = engine_for(typed, tensors, dtype, 16, 640)
            check_rows(replay(eng, steps), exact, requests, allowed, f"mark at {at}, {name}")


def long_memory(t):
    """Decays so close to one that a state holds what it saw long ago, and read-outs large enough to show it."""
    for name in t:
        if name.endswith(".A_log"):
            t[name] = torch.full_like(t[name], -7.0)
        if name.endswith((".mix.v", ".right.v")):
            t[name] = (t[name].double() * 10).to(torch.bfloat16)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("layer", ["lightning", "delta rule"])
def test_the_first_token_is_still_in_the_state_after_hundreds(layer, dtype):
    mixer = lightning(2, 12, 10, [0.9995, 0.998]) if layer == "lightning" else parallel(left(2, 1, 8, 8, 0.3, 10.0, 4, 0, rot_dims=4), right(2, 1, 12, 10, 3, 2, 2))

    def change(t):
        long_memory(t)
        if layer == "delta rule":       # only the recurrent branch speaks
            t["l0.mix.left.out"] = torch.zeros_like(t["l0.mix.left.out"])
    cfg = one_layer(mixer, width=32, vocab=40)
    typed, tensors = make_model(cfg, seed=2, change=change)
    toks = random_tokens(40, 300, 9)
    requests = {"a": toks, "b": [(toks[0] + 1) % 40] + toks[1:]}
    exact = reference(cfg, tensors, requests)
    moved = float((exact["a"][299] - exact["b"][299]).abs().max()) / float(exact["a"].abs().max())
    allowed = allowed_error(dtype, cfg, tensors, requests, exact)
    if dtype == "float32":
        assert moved > 50 * allowed, (moved, allowed)          # what the first token was still shows at the end
    for name, steps in {"whole": whole(requests), "decoded": tail_decoded(requests, tail=64), "portions": portions(requests, (2, 97, 3, 50)),
                        "both at once": mixed(requests, live=2, prefill_sizes=(40, 2, 7))}.items():
        eng = engine_for(typed, tensors, dtype, 16, 1024)
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
def test_a_step_of_more_than_a_thousand_tokens(dtype):
    cfg = config(32, 40, [parallel(left(2, 1, 16, 16, 0.2, 10.0, 70, 3, rot_dims=8), right(2, 1, 8, 12, 4, 2, 3), dense(24)), lightning(2, 8, 12, mlp=moe(8, 3, 3))])
    typed, tensors = make_model(cfg, seed=12)
    requests = {"a": random_tokens(40, 1100, 1), "b": random_tokens(40, 40, 2)}
    exact = reference(cfg, tensors, requests)
    allowed = allowed_error(dtype, cfg, tensors, requests, exact)
    cuts = {"a": 1031, "b": 5}
    steps = [{"step": 0, "entries": [{"id": r, "tokens": t[:cuts[r]], "want": list(range(cuts[r]))} for r, t in requests.items()], "end": []},
             {"step": 1, "entries": [{"id": r, "tokens": t[cuts[r]:], "want": list(range(len(t) - cuts[r]))} for r, t in requests.items()], "end": list(requests)}]
    eng = engine_for(typed, tensors, dtype, 16, 1280)
    check_rows(replay(eng, steps), exact, requests, allowed, "two steps")


# ---- configurations drawn at random -----------------------------------------------------------------------------------

def random_configuration(seed):
    import random
    r = random.Random(seed)
    width = r.choice([24, 40, 64, 96, 136])
    layers = []
    for _ in range(r.randint(2, 4)):
        E = r.randint(1, 6)
        mlp = r.choice([None, dense(8 * r.randint(2, 12)), moe(4 * r.randint(2, 8), E, E)])
        if r.random() < 0.4:
            heads = r.randint(1, 4)
            layers.append(lightning(heads, r.choice([4, 8, 20, 32, 64]), r.choice([4, 12, 32, 64]), [r.uniform(0.5, 1.0) for _ in range(heads)], mlp))
            continue
        kv = r.choice([1, 2, 3])
        dim = r.choice([8, 20, 32, 64, 128])
        vdim = r.choice([dim, dim, 4 * r.randint(1, 10)])
        l = left(kv * r.choice([1, 2, 4]), kv, dim, vdim, r.uniform(0.05, 0.5), r.choice([3.0, 20.0, 50.0]), r.choice([1, 5, 16, 17, 31, 32, 48, 100, 500]),
                 r.choice([0, 1, 4, 19]), rot_dims=r.choice([0, dim // 2 // 2 * 2, dim]), base=r.choice([100.0, 10000.0]), scaling=r.choice([None, SCALED]))
        qk = r.choice([1, 2])
        rr = right(qk * r.choice([1, 2, 3]), qk, r.choice([4, 8, 24, 64]), r.choice([4, 12, 32, 64]), r.randint(1, 5), r.randint(1, 9), r.randint(1, 9))
        layers.append(parallel(l, rr, mlp))
    return config(width, r.randint(30, 200), layers, logit_scale=r.uniform(0.5, 4.0), eps=r.choice([1e-5, 1e-6, 1e-3]))


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
        row = plain_lilatar_logits(cfg, tensors, toks)[-1]
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
