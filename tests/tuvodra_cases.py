"""Small Tuvodra configurations for the tests, their random weights, and the comparison with the plain decoder.

The configurations differ from one another in every size and option: streams 1 and 3, norm groups 1 and 3, keys and
values of different widths, scales that are not 1/sqrt(dim), one, several or all query heads to a kv head, windows
shorter and longer than the sequences, convolutions of one to four taps, more states than one pass of the scan kernel
holds, layers with and without a feed-forward after every kind of mixer, sizes that are multiples of nothing.
"""
from __future__ import annotations

import os
from typing import Dict, List

import torch

from llm_rs_amd import TuvodraConfig, random_model_tensors, write_model_folder
from plain_tuvodra import bf16_rounding, plain_tuvodra_logits


def attention(heads, kv_heads, dim, vdim, scale, window, ff=None):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                                            "mask": {"size": window}}, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def mamba1(inner, state, conv, dt_rank, ff=None):
    return {"type": "mamba1", "mixer": {"inner": inner, "state": state, "conv": conv, "dt_rank": dt_rank},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def mingru(width, ff=None):
    return {"type": "mingru", "mixer": {"width": width}, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def config(width, vocab, streams, groups, scale, layers, eps=1e-5):
    return {"architecture": "Tuvodra", "vocab": vocab, "width": width, "streams": streams, "embedding": {"scale": scale},
            "norm": {"eps": eps, "groups": groups}, "layers": layers}


ODD = config(48, 97, 3, 3, 3.5, [attention(4, 4, 12, 20, 0.3, 9), mamba1(40, 5, 4, 3, ff=56), mingru(36, ff=40),
                                   mamba1(24, 70, 1, 7), attention(6, 2, 10, 6, 0.7, 21, ff=30)])
PLAIN = config(64, 128, 1, 1, 1.0, [mingru(64), attention(6, 2, 16, 8, 1.0, 37, ff=96), attention(2, 1, 32, 32, 0.2, 1000),
                                     mamba1(64, 16, 2, 1)], eps=1e-6)
# widths at which the bfloat16 products go to the matrix cores
WIDE = config(256, 320, 2, 4, 8.0, [mamba1(384, 16, 4, 24), attention(8, 2, 64, 32, 0.125, 48, ff=512), mingru(320)])
CONFIGS = {"odd": ODD, "plain": PLAIN, "wide": WIDE}
PAGE_SIZE = {"odd": 4, "plain": 16, "wide": 16}


def one_layer(layer, width=40, vocab=61, streams=2, groups=2):
    return config(width, vocab, streams, groups, 2.0, [layer])


def make_model(cfg: dict, seed: int = 0, change=None):
    """(typed config, {name: bfloat16 tensor}); `change(tensors)` may put values of its own in."""
    typed = TuvodraConfig.from_dict(cfg)
    tensors = random_model_tensors(typed, seed)
    if change is not None:
        change(tensors)
    return typed, tensors


def make_folder(tmp_path, cfg: dict, seed: int = 0, change=None, name: str = "model") -> str:
    typed, tensors = make_model(cfg, seed, change)
    folder = os.path.join(str(tmp_path), name)
    write_model_folder(folder, typed, tensors)
    return folder


def reference(cfg: dict, tensors, requests: Dict[str, List[int]], rnd=None):
    kw = {} if rnd is None else {"rnd": rnd}
    return {rid: plain_tuvodra_logits(cfg, tensors, toks, **kw) for rid, toks in requests.items()}


def allowed_error(dtype: str, cfg: dict, tensors, requests, exact) -> float:
    """How far the engine may be from the exact logits, as a part of a sequence's largest logit.  float32: 3e-5.
    bfloat16: twice as far as the plain decoder gets when every activation that passes through memory between two
    stages is rounded to bfloat16 (the engine keeps some of those in 32-bit and sums in other orders; it does not
    round more often)."""
    if dtype == "float32":
        return 3e-5
    rounded = reference(cfg, tensors, requests, rnd=bf16_rounding)
    return 2.0 * max(float((rounded[r] - exact[r]).abs().max()) / float(exact[r].abs().max()) for r in requests)


def check_rows(rows, exact, requests, allowed: float, what: str = "") -> float:
    worst = 0.0
    for rid, toks in requests.items():
        ref = exact[rid]
        scale = float(ref.abs().max())
        assert sorted(rows[rid]) == list(range(len(toks))), f"{what} request {rid}: not every position came back"
        got = torch.stack([rows[rid][p] for p in range(len(toks))]).double()
        assert torch.isfinite(got).all(), f"{what} request {rid}: logits that are not numbers"
        err = (got - ref).abs().max(dim=1).values / scale
        bad = (err > allowed).nonzero()
        assert len(bad) == 0, (f"{what} request {rid}: first wrong position {int(bad[0])} of {len(toks)} (error "
                               f"{float(err[int(bad[0])]):.3e} of the largest logit, allowed {allowed:.1e}); {len(bad)} positions wrong")
        worst = max(worst, float(err.max()))
    return worst
