"""A plain, slow Tuvodra decoder for the tests to compare the engine with.

Whole sequences, no cache, no batching, one function per mechanism, in ordinary
tensor operations and explicit loops over time.  It shares no code with the
package.  Computation is in `compute` (float64 by default) from the weights as
stored.

The design: a token table whose rows are scaled on the way in; `streams` copies
of the residual stream mixed by small per-sublayer matrices (hyper-connections);
RMS norms taken over equal consecutive groups of the vector; layers whose mixer
is one of a minGRU recurrence, a selective state-space scan with a short causal
convolution, or windowed attention with unit-norm queries and keys and a
logarithmic distance penalty; an optional gated feed-forward; logits through the
(unscaled) token table.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, List, Optional, Sequence

import torch

# `rnd` in the functions below: applied to every activation that one stage hands the next through memory in an
# implementation that keeps such hand-overs in 16 bits (never to the streams, to a state, or to anything the design
# wants in 32-bit).  The identity by default; the tests pass a rounding to bfloat16 to learn how far rounding alone
# takes a model from its exact logits.
_same = lambda x: x


def bf16_rounding(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16).to(x.dtype)


def plain_group_rmsnorm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float, groups: int) -> torch.Tensor:
    """x: [..., D].  D is cut into `groups` equal consecutive parts; each part p becomes
    p / sqrt(mean(p^2) + eps); the whole is then multiplied by w (if any)."""
    D = x.shape[-1]
    parts = x.reshape(*x.shape[:-1], groups, D // groups)
    inv = 1.0 / torch.sqrt((parts * parts).mean(dim=-1, keepdim=True) + eps)
    y = (parts * inv).reshape(x.shape)
    return y if w is None else y * w


def plain_silu(x: torch.Tensor) -> torch.Tensor:
    return x / (1.0 + torch.exp(-x))


def plain_sigmoid(x: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-x))


def plain_softplus(x: torch.Tensor) -> torch.Tensor:
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def plain_mingru(h: torch.Tensor, w: Dict[str, torch.Tensor], rnd: Callable = _same) -> torch.Tensor:
    """h: [T, D].  gate z_t = sigmoid(Wz h_t + bz); u_t = Wx h_t + bx; candidate c_t = u_t + 1/2 where u_t >= 0,
    sigmoid(u_t) elsewhere; s_t = (1 - z_t) s_{t-1} + z_t c_t from s = 0; out_t = Wo (s_t * silu(Wg h_t))."""
    z = plain_sigmoid(h @ w["z"].T + w["z.b"])
    u = h @ w["x"].T + w["x.b"]
    cand = torch.where(u >= 0, u + 0.5, plain_sigmoid(u))
    gate = plain_silu(h @ w["g"].T)
    s = torch.zeros(z.shape[1], dtype=h.dtype)
    rows = []
    for t in range(h.shape[0]):
        s = (1.0 - z[t]) * s + z[t] * cand[t]
        rows.append(s * gate[t])
    return rnd(torch.stack(rows)) @ w["o"].T


def plain_causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """x: [T, C]; taps: [C, K], the last column weighs the current token, the one before it the token before, ...;
    inputs before the sequence's start are zero."""
    T, C = x.shape
    K = taps.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        acc = bias.clone()
        for j in range(K):
            src = t - (K - 1 - j)
            if src >= 0:
                acc = acc + taps[:, j] * x[src]
        y[t] = acc
    return y


def plain_mamba1(h: torch.Tensor, w: Dict[str, torch.Tensor], dt_rank: int, n_state: int, rnd: Callable = _same) -> torch.Tensor:
    """Selective scan.  [x | g] = Win h; x <- silu(conv(x)); [d | B | C] = Wx x; step = softplus(Wdt d + bdt) per
    channel; A = -exp(A_log); S[c, n] <- exp(step_c A[c, n]) S[c, n] + step_c x_c B_n; y_c = sum_n S[c, n] C_n +
    D_c x_c; out = Wo (y * silu(g))."""
    inner = w["in"].shape[0] // 2
    xg = h @ w["in"].T
    x, g = xg[:, :inner], xg[:, inner:]
    x = rnd(plain_silu(plain_causal_conv(x, w["conv"], w["conv.b"])))
    p = rnd(x @ w["x"].T)
    d, B, C = p[:, :dt_rank], p[:, dt_rank:dt_rank + n_state], p[:, dt_rank + n_state:dt_rank + 2 * n_state]
    step = plain_softplus(d @ w["dt"].T + w["dt.b"])
    A = -torch.exp(w["A_log"])
    S = torch.zeros(inner, n_state, dtype=h.dtype)
    rows = []
    for t in range(h.shape[0]):
        S = torch.exp(step[t][:, None] * A) * S + (step[t] * x[t])[:, None] * B[t][None, :]
        rows.append(S @ C[t] + w["D"] * x[t])
    y = rnd(torch.stack(rows) * plain_silu(g))
    return y @ w["o"].T


def plain_window_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], heads: int, kv_heads: int, dim: int, vdim: int,
                           scale: float, window: int, eps: float, rnd: Callable = _same) -> torch.Tensor:
    """q, k, v with biases; q and k divided by their root mean square over `dim`, head by head; score(i, j) =
    q_i . k_j * scale - r1_h ln(1 + r2_h (i - j)) for 0 <= i - j < window; softmax over those j; heads side by side
    through Wo.  Query head a reads key/value head a // (heads / kv_heads)."""
    T = h.shape[0]
    q = (h @ w["q"].T + w["q.b"]).reshape(T, heads, dim)
    k = (h @ w["k"].T + w["k.b"]).reshape(T, kv_heads, dim)
    v = (h @ w["v"].T + w["v.b"]).reshape(T, kv_heads, vdim)
    q = rnd(plain_group_rmsnorm(q, None, eps, 1))
    k = rnd(plain_group_rmsnorm(k, None, eps, 1))
    v = rnd(v)
    per = heads // kv_heads
    out = torch.zeros(T, heads, vdim, dtype=h.dtype)
    for a in range(heads):
        g = a // per
        for i in range(T):
            lo = max(0, i - window + 1)
            dist = torch.arange(i - lo, -1, -1, dtype=h.dtype)           # i - j for j = lo..i
            s = (k[lo:i + 1, g] @ q[i, a]) * scale - w["r1"][a] * torch.log(1.0 + w["r2"][a] * dist)
            p = torch.softmax(s, dim=0)
            out[i, a] = p @ v[lo:i + 1, g]
    return rnd(out.reshape(T, heads * vdim)) @ w["o"].T


def plain_gated_mlp(h: torch.Tensor, w: Dict[str, torch.Tensor], rnd: Callable = _same) -> torch.Tensor:
    return rnd(plain_silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def plain_hyper_step(xs: torch.Tensor, hc: Dict[str, torch.Tensor], sublayer) -> torch.Tensor:
    """xs: [S, T, D] streams.  u = sum_s in[s] xs[s]; y = sublayer(u); new[t] = sum_s mix[s, t] xs[s] + out[t] y,
    every new stream from the old ones."""
    u = torch.einsum("s,std->td", hc["in"], xs)
    y = sublayer(u)
    return torch.einsum("sr,std->rtd", hc["mix"], xs) + hc["out"][:, None, None] * y[None]


def _sub(tensors, prefix, compute):
    n = len(prefix) + 1
    return {k[n:]: v.to(compute) for k, v in tensors.items() if k.startswith(prefix + ".")}


def plain_tuvodra_logits(cfg: dict, tensors: Dict[str, torch.Tensor], tokens: Sequence[int], compute=torch.float64,
                         layers_out: Optional[List[torch.Tensor]] = None, rnd: Callable = _same) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  `layers_out`, if a list, gets the sum of the streams after each layer."""
    eps, groups, S = float(cfg["norm"]["eps"]), int(cfg["norm"]["groups"]), int(cfg["streams"])
    table = tensors["embed"].to(compute)
    x0 = table[torch.tensor(list(tokens), dtype=torch.long)] * float(cfg["embedding"]["scale"])
    xs = x0[None].repeat(S, 1, 1)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        m, kind = layer["mixer"], layer["type"]
        mw = _sub(tensors, f"{p}.mix", compute)
        if kind == "mingru":
            mixer = lambda h: plain_mingru(h, mw, rnd)
        elif kind == "mamba1":
            mixer = lambda h: plain_mamba1(h, mw, int(m["dt_rank"]), int(m["state"]), rnd)
        elif kind == "attention":
            mixer = lambda h: plain_window_attention(h, mw, int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]),
                                                     float(m["scale"]), int(m["mask"]["size"]), eps, rnd)
        else:
            raise ValueError(kind)
        n1 = tensors[f"{p}.norm1"].to(compute)
        xs = plain_hyper_step(xs, _sub(tensors, f"{p}.hc1", compute), lambda u: mixer(rnd(plain_group_rmsnorm(u, n1, eps, groups))))
        if layer.get("mlp") is not None:
            n2 = tensors[f"{p}.norm2"].to(compute)
            fw = _sub(tensors, f"{p}.mlp", compute)
            xs = plain_hyper_step(xs, _sub(tensors, f"{p}.hc2", compute), lambda u: plain_gated_mlp(rnd(plain_group_rmsnorm(u, n2, eps, groups)), fw, rnd))
        if layers_out is not None:
            layers_out.append(xs.sum(dim=0))
    x = rnd(plain_group_rmsnorm(xs.sum(dim=0), tensors["final.norm"].to(compute), eps, groups))
    return x @ table.T
