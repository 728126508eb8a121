"""The Lilatar configuration, what the model asks of weights and cache, the plain decoder's own invariants, and the
engine's host logic on the emulated kernels (CPU)."""
from __future__ import annotations

import copy
import math

import pytest
import torch

from emulated_kernels import EmulatedKernels
from llm_rs_amd import ConfigError, Engine, FixedState, LilatarConfig, Model, PagedKV, config_from_dict, load_config, use_kernels
from llm_rs_amd.cache.native import HostCore
from llm_rs_amd.engine.trace import TraceReplayer
from lilatar_cases import (CONFIGS, check_rows, config, dense, left, lightning, make_folder, make_model, moe, one_layer, parallel,
                           reference, right)
from plain_lilatar import (plain_delta_rule, plain_lightning, plain_lilatar_logits, plain_rotary_frequencies, plain_rotate,
                           plain_routed_ff, plain_short_conv, plain_softmax_attention, plain_visible)
from replay_cases import collect, live_token_need, mixed, portions, random_tokens, tail_decoded, whole


def test_the_registry_finds_the_architecture():
    cfg = config_from_dict(CONFIGS["odd"])
    assert isinstance(cfg, LilatarConfig) and cfg.to_dict() == CONFIGS["odd"]


@pytest.mark.parametrize("path", [("vocab",), ("width",), ("norm", "eps"), ("layers", 0, "type"), ("layers", 0, "mixer", "left", "vdim"),
                                  ("layers", 0, "mixer", "left", "mask", "size"), ("layers", 0, "mixer", "left", "rot", "base"),
                                  ("layers", 0, "mixer", "right", "conv"), ("layers", 0, "mixer", "right", "decay_rank"),
                                  ("layers", 1, "mixer", "decay"), ("layers", 1, "mlp", "router", "top"), ("layers", 0, "mlp", "ff")])
def test_a_missing_key_is_named(path):
    d = copy.deepcopy(CONFIGS["odd"])
    at = d
    for key in path[:-1]:
        at = at[key]
    del at[path[-1]]
    with pytest.raises(ConfigError, match=str(path[-1])):
        LilatarConfig.from_dict(d).model_spec()


def test_what_a_file_may_leave_out():
    d = copy.deepcopy(CONFIGS["plain"])
    del d["layers"][1]["mixer"]["right"]["kv_heads"], d["layers"][2]["mixer"]["left"]["kv_heads"], d["logit_scale"]
    d["layers"][0]["mixer"]["decay"] = 0.9
    d["layers"][1]["mixer"]["left"]["softcap"] = None
    cfg = LilatarConfig.from_dict(d)
    spec = cfg.model_spec()
    assert spec.logit_scale == 1.0 and spec.layers[0].mixer.params["decay"] == [0.9] * 4
    branches = spec.layers[1].mixer.params["branches"]
    assert branches[1]["mixer"].params["kv_heads"] == 4 and branches[0]["mixer"].params["softcap"] == 0.0
    assert spec.layers[2].mixer.params["branches"][0]["mixer"].params["num_kv_heads"] == 2
    assert cfg.to_dict()["layers"][0]["mixer"]["decay"] == [0.9] * 4


def test_what_does_not_fit_is_refused():
    for change in (lambda d: d["layers"][0].update(type="attention"), lambda d: d["layers"][0]["mixer"]["left"].update(kv_heads=4),
                   lambda d: d["layers"][1]["mlp"].update(kind="gated"), lambda d: d["layers"][1]["mixer"].update(decay=[0.5]),
                   lambda d: d["layers"][0]["mixer"]["left"]["rot"].update(dims=7), lambda d: d["layers"][1]["mlp"]["router"].update(top=6),
                   lambda d: d["layers"][0]["mixer"]["right"].update(conv=0)):
        d = copy.deepcopy(CONFIGS["odd"])
        change(d)
        with pytest.raises(ConfigError):
            LilatarConfig.from_dict(d)


def test_tensors_and_cache_needs_follow_the_file():
    cfg = LilatarConfig.from_dict(CONFIGS["odd"])
    model = Model(cfg.model_spec(), torch.bfloat16, "cpu")
    t = {n: tuple(s.shape) for n, s in model.tensors().items()}
    assert t["embed"] == (97, 46) and t["head"] == (97, 46) and t["final.norm"] == (46,) and t["l0.norm1b"] == (46,)
    assert "l2.norm2" not in t and "l2.norm2b" not in t and t["l1.norm2b"] == (46,)
    assert t["l0.mix.left.q"] == (60, 46) and t["l0.mix.left.k.b"] == (20,) and t["l0.mix.left.v"] == (12, 46) and t["l0.mix.left.o"] == (46, 36)
    assert t["l0.mix.left.o.b"] == (46,) and t["l0.mix.left.out"] == (46,) and t["l0.mix.right.out"] == (46,)
    assert t["l0.mix.right.q"] == (7, 46) and t["l0.mix.right.v.conv"] == (15, 4) and t["l0.mix.right.b"] == (3, 46)
    assert t["l0.mix.right.a1"] == (2, 46) and t["l0.mix.right.a2"] == (21, 2) and t["l0.mix.right.g2"] == (15, 1)
    assert t["l0.mix.right.A_log"] == (3,) and t["l0.mix.right.dt_bias"] == (21,) and t["l0.mix.right.norm"] == (5,)
    assert t["l1.mix.q"] == (15, 46) and t["l1.mix.g"] == (27, 46) and t["l1.mix.norm"] == (27,) and t["l1.mix.o"] == (46, 27)
    assert t["l1.mlp.router"] == (5, 46) and t["l1.mlp.e4.up"] == (11, 46) and t["l1.mlp.e0.down"] == (46, 11) and t["l0.mlp.up"] == (30, 46)
    needs = [n for n, _ in model.cache_needs()]
    assert needs[0] == (PagedKV(2, 10, 9, 6, 2), FixedState((3 * 7 * 5 + 3 * (7 + 7 + 15),)))
    assert needs[1] == FixedState((3 * 5 * 9,)) and needs[2] == (PagedKV(2, 12, 21, 20, 0), FixedState((2 * 9 * 6,)))
    assert model.spec.logit_scale == 3.0 and model.spec.head_name == "head" and set(model.spec.ignorable_tensors) == {"l2.norm2", "l2.norm2b"}


def test_the_ranks_come_from_the_tensors_of_a_folder(tmp_path):
    """A file that does not name the ranks of the low-rank projections: the tensors' shapes give them."""
    import json
    import os
    folder = make_folder(tmp_path, CONFIGS["odd"], seed=1)
    with open(os.path.join(folder, "config.json")) as f:
        d = json.load(f)
    for layer in d["layers"]:
        if layer["type"] == "parallel":
            del layer["mixer"]["right"]["decay_rank"], layer["mixer"]["right"]["gate_rank"]
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(d, f)
    cfg = load_config(folder)
    assert cfg.layers[0]["mixer"]["right"]["decay_rank"] == 2 and cfg.layers[2]["mixer"]["right"]["gate_rank"] == 3
    with pytest.raises(ConfigError, match="decay_rank"):
        LilatarConfig.from_dict(d).model_spec()


# ---- the plain decoder's mechanisms, each pinned by a case that can be worked out by hand -------------------------

def test_plain_visibility_and_frequencies():
    assert [j for j in range(10) if plain_visible(9, j, 3, 2)] == [0, 1, 7, 8, 9]
    assert [j for j in range(10) if plain_visible(2, j, 3, 2)] == [0, 1, 2]
    assert not plain_visible(3, 4, 100, 100)
    f = plain_rotary_frequencies({"dims": 8, "base": 100.0, "scaling": None})
    assert torch.allclose(f, torch.tensor([1.0, 100 ** -0.25, 0.1, 100 ** -0.75], dtype=torch.float64))
    s = plain_rotary_frequencies({"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}})
    # wavelengths 6.3, 19.9, 62.8, 198.7 against 64 / 4 = 16 and 64 / 1 = 64: kept, blended, blended, divided
    assert s[0] == f[0] and s[3] == f[3] / 4 and f[1] / 4 < s[1] < f[1] and f[2] / 4 < s[2] < f[2]
    blend = (64 / (2 * math.pi / float(f[1])) - 1.0) / 3.0
    assert abs(float(s[1]) - ((1 - blend) * float(f[1]) / 4 + blend * float(f[1]))) < 1e-15


def test_plain_rotation_turns_neighbours_and_leaves_the_rest():
    x = torch.zeros(2, 1, 6, dtype=torch.float64)
    x[:, 0, 0] = 1.0
    x[:, 0, 5] = 3.0
    y = plain_rotate(x, torch.tensor([math.pi / 2], dtype=torch.float64), [0, 1])
    assert torch.allclose(y[0], x[0]) and torch.allclose(y[1, 0], torch.tensor([0.0, 1.0, 0, 0, 0, 3.0], dtype=torch.float64), atol=1e-15)


def test_plain_lightning_is_a_decayed_sum():
    """One head, one key and one value channel, q = k = silu(1 * h): o_t = q_t sum_j decay^(t - j) k_j v_j."""
    silu = lambda v: v / (1 + math.exp(-v))
    h = torch.tensor([[1.0], [2.0], [0.5]], dtype=torch.float64)
    one = torch.ones(1, 1, dtype=torch.float64)
    w = {"q": one, "k": one, "v": one, "g": torch.zeros(1, 1, dtype=torch.float64), "o": one, "norm": torch.ones(1, dtype=torch.float64)}
    m = {"heads": 1, "dim": 1, "vdim": 1, "decay": [0.5]}
    got = plain_lightning(h, w, m, eps=0.0)
    a = [silu(1.0), silu(2.0), silu(0.5)]
    o = [a[0] ** 3, a[1] * (0.5 * a[0] ** 2 + a[1] ** 2), a[2] * (0.25 * a[0] ** 2 + 0.5 * a[1] ** 2 + a[2] ** 2)]
    # a single channel normed to +-1, times sigmoid(0)
    assert torch.allclose(got[:, 0], torch.tensor([math.copysign(0.5, v) for v in o], dtype=torch.float64))


def test_plain_short_conv_weighs_the_current_token_last():
    x = torch.tensor([[1.0], [10.0], [100.0]], dtype=torch.float64)
    y = plain_short_conv(x, torch.tensor([[3.0, 2.0, 1.0]], dtype=torch.float64))
    assert y[:, 0].tolist() == [1.0, 12.0, 123.0]


def test_plain_routing_takes_the_largest_scores_as_they_are():
    h = torch.eye(3, dtype=torch.float64)
    w = {"router": torch.tensor([[2.0, 0, 0], [1.0, 3.0, 0], [0.0, 1.0, 1.0]], dtype=torch.float64)}
    for e in range(3):      # expert e writes (e + 1) * relu(sum h)^2 into channel 0
        w[f"e{e}.up"] = torch.ones(1, 3, dtype=torch.float64)
        w[f"e{e}.down"] = torch.tensor([[e + 1.0], [0.0], [0.0]], dtype=torch.float64)
    out = plain_routed_ff(h, w, {"router": {"experts": 3, "top": 2}})
    s = torch.softmax(h @ w["router"].T, dim=-1)
    assert abs(float(out[0, 0]) - float(s[0, 0] * 1 + s[0, 1] * 2)) < 1e-12           # experts 0 and 1
    assert abs(float(out[1, 0]) - float(s[1, 1] * 2 + s[1, 2] * 3)) < 1e-12           # experts 1 and 2
    assert abs(float(out[2, 0]) - float(s[2, 2] * 3 + s[2, 0] * 1)) < 1e-12           # expert 2, then the lower of two equal scores


def test_plain_delta_rule_overwrites_what_a_key_held():
    """With decay 1 and beta 1, writing the same unit key twice leaves the second value: the read-out is q.k times it."""
    H, dk, dv = 1, 2, 2
    m = {"heads": 1, "kv_heads": 1, "dim": dk, "vdim": dv, "conv": 1}
    big = 40.0
    eye = torch.eye(2, dtype=torch.float64)
    w = {"q": eye, "k": eye, "v": eye, "q.conv": torch.ones(2, 1, dtype=torch.float64), "k.conv": torch.ones(2, 1, dtype=torch.float64),
         "v.conv": torch.ones(2, 1, dtype=torch.float64), "b": torch.tensor([[big, big]], dtype=torch.float64),
         "A_log": torch.tensor([-50.0], dtype=torch.float64), "a1": torch.zeros(1, 2, dtype=torch.float64), "a2": torch.zeros(2, 1, dtype=torch.float64),
         "dt_bias": torch.zeros(2, dtype=torch.float64), "g1": torch.zeros(1, 2, dtype=torch.float64), "g2": torch.zeros(2, 1, dtype=torch.float64),
         "norm": torch.ones(2, dtype=torch.float64), "o": eye}
    h = torch.tensor([[3.0, 0.0], [5.0, 0.0]], dtype=torch.float64)      # both tokens: key along channel 0
    out = plain_delta_rule(h, w, m, eps=0.0)
    # o_t = (q.k) v_t with unit q, k: v_t = silu(h_t) has one channel, the norm over vdim makes it sqrt(2), the gate halves it
    assert torch.allclose(out, torch.tensor([[math.sqrt(2) / 2, 0.0], [math.sqrt(2) / 2, 0.0]], dtype=torch.float64), atol=1e-6)


# ---- the cache manager keeps the first pages of a window group ----------------------------------------------------

def test_a_window_that_keeps_first_tokens_keeps_their_pages():
    core = HostCore([(4, 64, 6, 5)], max_requests=2)        # pages of 4, window 6, the first 5 positions stay
    s = core.acquire_slot()
    for pos in range(40):
        assert core.ensure(s, pos, 1)
        table = core.table(s, 0)
        first_visible = max(0, pos + 1 - 6)
        for i, page in enumerate(table):
            assert (page >= 0) == (i >= first_visible // 4 or i * 4 < 5), f"pos {pos}: logical page {i} -> {page}"
    assert core.pages_held(s, 0) == 2 + len([i for i in range(10) if i >= (40 - 6) // 4])
    core.release_slot(s)
    assert core.pages_free(0) == 64


def test_a_request_that_starts_late_still_gets_its_first_pages():
    core = HostCore([(4, 16, 6, 3)], max_requests=1)
    s = core.acquire_slot()
    assert core.ensure(s, 0, 30)                 # (a recompute: the whole span in one portion)
    assert all(p >= 0 for p in core.table(s, 0))
    assert core.ensure(s, 30, 1)
    table = core.table(s, 0)
    assert table[0] >= 0 and all(p < 0 for p in table[1:6]) and all(p >= 0 for p in table[6:])


# ---- the engine's host logic on the emulated kernels ---------------------------------------------------------------

def replay_cpu(typed, tensors, dtype, page_size, steps, max_requests=4):
    with use_kernels(EmulatedKernels()):
        eng = Engine(typed, tensors, dtype=dtype, device="cpu", page_size=page_size, num_pages=max(-(-live_token_need(steps, 64) // page_size), 1),
                     max_requests=max_requests)
        rep = TraceReplayer.for_engine(eng)
        outputs = []
        for step in steps:
            out = rep.step(step)
            outputs.append(None if out is None else torch.from_numpy(out.copy()))
        core = eng.cache.core
        assert core.slots_in_use() == 0 and all(core.pages_free(g) == core.pages_total(g) for g in range(core.n_groups))
    return collect(steps, outputs)


@pytest.mark.parametrize("which", ["odd", "plain"])
def test_replay_regimes_on_the_host_logic(which):
    cfg = CONFIGS[which]
    typed, tensors = make_model(cfg, seed=3)
    lengths = [1, 2, 23, 50, 40, 17]            # more requests than slots: slots and pages are used again
    requests = {f"r{i}": random_tokens(cfg["vocab"], n, 10 + i) for i, n in enumerate(lengths)}
    exact = reference(cfg, tensors, requests)
    for name, steps in {"whole": whole(requests), "decoded": tail_decoded(requests, tail=12), "portions": portions(requests, (2, 3, 7)),
                        "mixed": mixed(requests, live=3)}.items():
        check_rows(replay_cpu(typed, tensors, "float32", {"odd": 4, "plain": 16}[which], steps), exact, requests, 3e-5, name)
