"""Small Lilatar configurations for the tests, their random weights, and the comparison with the plain decoder.

The configurations differ from one another in every size and option: heads of several sizes with keys and values of
different widths, one, several or all query heads to a key head on both sides of a parallel layer, windows shorter and
longer than the sequences with and without kept first tokens, rotations over none, part or all of a head with and
without scaled frequencies, soft caps small and large, convolutions of one to five taps, ranks of one and many, dense
feed-forwards, experts of which some or all are chosen, layers without a feed-forward, sizes that are multiples of
nothing, a logit scale that is and is not 1.
"""
from __future__ import annotations

import os
from typing import Dict, List

import torch

from llm_rs_amd import LilatarConfig, random_model_tensors, write_model_folder
from plain_lilatar import bf16_rounding, plain_lilatar_logits


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def lightning(heads, dim, vdim, decay=None, mlp=None):
    decay = decay if decay is not None else [0.5 + 0.499 * (i + 1) / heads for i in range(heads)]
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}, "mlp": mlp}


def left(heads, kv_heads, dim, vdim, scale, softcap, size, keep_first=0, rot_dims=None, base=10000.0, scaling=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap,
            "mask": {"size": size, "keep_first": keep_first},
            "rot": {"dims": dim if rot_dims is None else rot_dims, "base": base, "scaling": scaling}}


def right(heads, kv_heads, dim, vdim, conv, decay_rank=3, gate_rank=5):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "decay_rank": decay_rank, "gate_rank": gate_rank}


def parallel(l, r, mlp=None):
    return {"type": "parallel", "mixer": {"left": l, "right": r}, "mlp": mlp}


def config(width, vocab, layers, logit_scale=1.0, eps=1e-5):
    return {"architecture": "Lilatar", "vocab": vocab, "width": width, "logit_scale": logit_scale, "norm": {"eps": eps}, "layers": layers}


SCALED = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}

ODD = config(46, 97, [
    parallel(left(6, 2, 10, 6, 0.3, 7.0, 9, 2, rot_dims=6, base=100.0, scaling=SCALED), right(3, 1, 7, 5, 4, 2, 1), dense(30)),
    lightning(3, 5, 9, mlp=moe(11, 5, 5)),
    parallel(left(2, 2, 12, 20, 0.7, 50.0, 21, 0, rot_dims=12), right(2, 2, 9, 6, 1, 4, 3)),
    lightning(1, 13, 4, [0.97], mlp=dense(17)),
], logit_scale=3.0)
PLAIN = config(64, 128, [
    lightning(4, 16, 16, mlp=dense(96)),
    parallel(left(4, 1, 16, 16, 0.25, 30.0, 37, 5, rot_dims=8), right(4, 2, 16, 8, 3, 8, 8), moe(32, 4, 4)),
    parallel(left(2, 2, 32, 32, 0.2, 10.0, 1000, 3, rot_dims=0), right(1, 1, 32, 32, 2, 1, 1), dense(64)),
], eps=1e-6)
# widths at which the bfloat16 products go to the matrix cores, heads the matrix-core attention takes in 32-bit
WIDE = config(256, 320, [
    parallel(left(8, 2, 64, 64, 0.125, 20.0, 48, 4, rot_dims=32, scaling=SCALED), right(4, 2, 64, 32, 4, 16, 24), moe(64, 6, 6)),
    lightning(4, 64, 64, mlp=dense(512)),
    parallel(left(4, 4, 32, 32, 0.2, 15.0, 16, 17, rot_dims=32), right(2, 1, 32, 128, 3, 8, 8), dense(256)),
], logit_scale=0.5)
CONFIGS = {"odd": ODD, "plain": PLAIN, "wide": WIDE}
PAGE_SIZE = {"odd": 4, "plain": 16, "wide": 16}


def one_layer(layer, width=40, vocab=61, logit_scale=2.0):
    return config(width, vocab, [layer], logit_scale)


def make_model(cfg: dict, seed: int = 0, change=None):
    """(typed config, {name: bfloat16 tensor}); `change(tensors)` may put values of its own in."""
    typed = LilatarConfig.from_dict(cfg)
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
    return {rid: plain_lilatar_logits(cfg, tensors, toks, **kw) for rid, toks in requests.items()}


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
