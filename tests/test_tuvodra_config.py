"""The Tuvodra configuration, what the model asks of weights and cache, and the plain decoder's own invariants (CPU)."""
from __future__ import annotations

import copy

import pytest
import torch

from llm_rs_amd import ConfigError, FixedState, Model, PagedKV, TuvodraConfig, config_from_dict
from plain_tuvodra import (plain_causal_conv, plain_group_rmsnorm, plain_hyper_step, plain_mamba1, plain_mingru,
                           plain_tuvodra_logits, plain_window_attention)
from tuvodra_cases import CONFIGS, attention, config, mamba1, mingru, make_model


def test_the_registry_finds_the_architecture_by_its_singular_key():
    cfg = config_from_dict(CONFIGS["odd"])
    assert isinstance(cfg, TuvodraConfig) and cfg.to_dict() == CONFIGS["odd"]
    with pytest.raises(ConfigError, match="architectures"):
        config_from_dict({k: v for k, v in CONFIGS["odd"].items() if k != "architecture"})


@pytest.mark.parametrize("path", [("vocab",), ("width",), ("streams",), ("embedding", "scale"), ("norm", "eps"), ("norm", "groups"),
                                  ("layers", 0, "type"), ("layers", 0, "mixer", "vdim"), ("layers", 0, "mixer", "mask", "size"),
                                  ("layers", 1, "mixer", "dt_rank"), ("layers", 2, "mixer", "width"), ("layers", 1, "mlp", "ff")])
def test_a_missing_key_is_named(path):
    d = copy.deepcopy(CONFIGS["odd"])
    at = d
    for key in path[:-1]:
        at = at[key]
    del at[path[-1]]
    with pytest.raises(ConfigError, match=str(path[-1])):
        TuvodraConfig.from_dict(d)


def test_what_does_not_fit_is_refused():
    for change in (lambda d: d["norm"].update(groups=5), lambda d: d["layers"][0].update(type="lstm"),
                   lambda d: d["layers"][0]["mixer"].update(kv_heads=3), lambda d: d["layers"][1]["mlp"].update(kind="routed"),
                   lambda d: d.update(streams=0)):
        d = copy.deepcopy(CONFIGS["odd"])
        change(d)
        with pytest.raises(ConfigError):
            TuvodraConfig.from_dict(d)


def test_tensors_and_cache_needs_follow_the_file():
    cfg = TuvodraConfig.from_dict(CONFIGS["odd"])
    model = Model(cfg.model_spec(), torch.bfloat16, "cpu")
    t = {n: tuple(s.shape) for n, s in model.tensors().items()}
    assert t["embed"] == (97, 48) and t["final.norm"] == (48,) and "l0.norm2" not in t and t["l1.norm2"] == (48,)
    assert t["l0.mix.q"] == (48, 48) and t["l0.mix.v"] == (80, 48) and t["l0.mix.o"] == (48, 80) and t["l0.mix.v.b"] == (80,)
    assert t["l0.mix.r1"] == (4,) and t["l0.hc1.mix"] == (3, 3) and t["l1.hc2.in"] == (3,) and "l0.hc2.in" not in t
    assert t["l1.mix.in"] == (80, 48) and t["l1.mix.conv"] == (40, 4) and t["l1.mix.x"] == (3 + 10, 40) and t["l1.mix.dt"] == (40, 3)
    assert t["l1.mix.A_log"] == (40, 5) and t["l2.mix.z"] == (36, 48) and t["l2.mix.o"] == (48, 36) and t["l2.mlp.down"] == (48, 40)
    needs = [n for n, _ in model.cache_needs()]
    assert needs == [PagedKV(4, 12, 9, 20), FixedState((40 * 5 + 3 * 40,)), FixedState((36,)), FixedState((24 * 70,)), PagedKV(2, 10, 21, 6)]
    assert model.spec.embedding_scale == 3.5 and model.spec.streams == 3 and model.spec.head_name is None


# ---- the plain decoder's mechanisms, each pinned by a case that can be worked out by hand -------------------------

def test_group_norm_by_hand():
    x = torch.tensor([3.0, 4.0, 0.0, 2.0], dtype=torch.float64)
    y = plain_group_rmsnorm(x, torch.tensor([1.0, 2.0, 1.0, 0.5], dtype=torch.float64), 0.0, 2)
    r0, r1 = (12.5) ** 0.5, 2.0 ** 0.5
    assert torch.allclose(y, torch.tensor([3 / r0, 8 / r0, 0.0, 1 / r1], dtype=torch.float64))
    assert torch.allclose(plain_group_rmsnorm(x, None, 0.0, 1), x / (29.0 / 4) ** 0.5)


def test_hyper_step_by_hand():
    xs = torch.tensor([[[1.0]], [[10.0]]], dtype=torch.float64)       # two streams, one token, one feature
    hc = {"in": torch.tensor([2.0, 0.5]), "out": torch.tensor([1.0, -1.0]), "mix": torch.tensor([[1.0, 3.0], [0.0, 2.0]])}
    hc = {k: v.double() for k, v in hc.items()}
    new = plain_hyper_step(xs, hc, lambda u: u * 100.0)              # u = 7, y = 700
    assert torch.allclose(new.flatten(), torch.tensor([1.0 + 700.0, 3.0 + 20.0 - 700.0], dtype=torch.float64))


def test_mingru_by_hand():
    W = 1
    w = {"z": torch.zeros(W, 1), "z.b": torch.zeros(W), "x": torch.ones(W, 1), "x.b": torch.zeros(W), "g": torch.zeros(W, 1), "o": torch.ones(1, W)}
    w = {k: v.double() for k, v in w.items()}
    h = torch.tensor([[1.0], [-30.0]], dtype=torch.float64)
    # z = 1/2 always; candidate 1.5 then sigmoid(-30) ~ 0; the output gate silu(0) = 0 hides the state
    assert torch.allclose(plain_mingru(h, w), torch.zeros(2, 1, dtype=torch.float64))
    w["g"] = torch.full((W, 1), 50.0, dtype=torch.float64)          # silu(50 h) ~ 50 h for h > 0
    out = plain_mingru(torch.tensor([[1.0], [1.0]], dtype=torch.float64), w)
    assert torch.allclose(out.flatten(), torch.tensor([0.75 * 50.0, (0.375 + 0.75) * 50.0], dtype=torch.float64))


def test_conv_last_tap_is_the_current_token():
    x = torch.tensor([[1.0], [2.0], [4.0]], dtype=torch.float64)
    y = plain_causal_conv(x, torch.tensor([[100.0, 10.0, 1.0]], dtype=torch.float64), torch.tensor([0.5], dtype=torch.float64))
    assert torch.allclose(y.flatten(), torch.tensor([1.5, 12.5, 124.5], dtype=torch.float64))


def test_attention_window_and_distance_by_hand():
    # one head, keys all alike: the weights are softmax(-r1 ln(1 + r2 d)) = (1 + r2 d)^(-r1) normalised
    w = {"q": torch.zeros(2, 1), "q.b": torch.ones(2), "k": torch.zeros(2, 1), "k.b": torch.ones(2), "v": torch.ones(1, 1), "v.b": torch.zeros(1),
         "o": torch.ones(1, 1), "r1": torch.tensor([2.0]), "r2": torch.tensor([1.0])}
    w = {k: v.double() for k, v in w.items()}
    h = torch.tensor([[1.0], [2.0], [4.0], [8.0]], dtype=torch.float64)
    out = plain_window_attention(h, w, 1, 1, 2, 1, 0.3, 2, 0.0)
    wts = torch.tensor([1.0, 0.25], dtype=torch.float64) / 1.25        # the key itself, the one before; nothing older
    want = [1.0, wts[0] * 2 + wts[1] * 1, wts[0] * 4 + wts[1] * 2, wts[0] * 8 + wts[1] * 4]
    assert torch.allclose(out.flatten(), torch.tensor(want, dtype=torch.float64))


def test_the_scan_equals_its_closed_form_for_a_constant_input():
    C, N = 1, 1
    w = {"in": torch.tensor([[1.0], [0.0]]), "conv": torch.tensor([[1.0]]), "conv.b": torch.zeros(1), "x": torch.tensor([[0.0], [1.0], [1.0]]),
         "dt": torch.zeros(1, 1), "dt.b": torch.tensor([0.0]), "A_log": torch.zeros(1, 1), "D": torch.zeros(1), "o": torch.ones(1, 1)}
    w = {k: v.double() for k, v in w.items()}
    h = torch.ones(3, 1, dtype=torch.float64)
    x = 1.0 / (1.0 + torch.exp(torch.tensor(-1.0, dtype=torch.float64)))          # silu(1)
    step = torch.log(torch.tensor(2.0, dtype=torch.float64))                      # softplus(0); decay exp(-step) = 1/2
    S, want = 0.0, []
    for _ in range(3):
        S = 0.5 * S + step * x * x
        want.append(S * x * 0.0)                                                  # the gate silu(0) = 0 closes the output
    assert torch.allclose(plain_mamba1(h, w, 1, 1).flatten(), torch.tensor(want, dtype=torch.float64))


def test_whole_model_is_causal_and_windows_forget():
    cfg = config(32, 40, 2, 2, 2.0, [attention(2, 1, 8, 8, 0.5, 4)])
    _, tensors = make_model(cfg, seed=1)
    a = [1, 2, 3, 4, 5, 6, 7, 8]
    b = [9] + a[1:]
    la, lb = plain_tuvodra_logits(cfg, tensors, a), plain_tuvodra_logits(cfg, tensors, b)
    assert not torch.allclose(la[3], lb[3]) and torch.allclose(la[4:], lb[4:])     # position 0 is out of every window from 4 on
    assert torch.allclose(plain_tuvodra_logits(cfg, tensors, a[:5]), la[:5])
