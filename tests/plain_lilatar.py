"""A plain, slow Lilatar decoder for the tests to compare the engine with.

Whole sequences, no cache, no batching, one function per mechanism, in ordinary
tensor operations and explicit loops over time.  It shares no code with the
package.  Computation is in `compute` (float64 by default) from the weights as
stored.

The design: a token table; layers with an RMS norm before and after each
sublayer; a mixer that is either linear attention with a fixed decay per head
("lightning") or two mixers side by side whose normed outputs are averaged
("parallel": softmax attention with biases, a partial interleaved rotation with
scaled frequencies, soft-capped scores and a sliding window that keeps the
first tokens, beside a gated delta rule with short convolutions and a decay per
key channel); a feed-forward with squared-relu activation, dense or routed over
experts by an un-renormalised softmax; a final norm and a scaled output matrix.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, List, Optional, Sequence

import torch

# `rnd`: applied to every activation that one stage hands the next through memory in an implementation that keeps
# such hand-overs in 16 bits (never to the stream, a state, a score, a norm's sum or anything that enters a
# recurrence).  The identity by default.
_same = lambda x: x


def bf16_rounding(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16).to(x.dtype)


def plain_rmsnorm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def plain_silu(x):
    return x / (1.0 + torch.exp(-x))


def plain_sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def plain_softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def plain_relu2(x):
    r = torch.clamp(x, min=0.0)
    return r * r


# -- linear attention with a fixed decay per head ----------------------------------------------------------------------
def plain_lightning(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float, rnd: Callable = _same) -> torch.Tensor:
    """h: [T, D].  q, k = silu(Wq h), silu(Wk h) [heads, dim]; v = silu(Wv h) [heads, vdim]; per head
    S_t = decay S_(t-1) + k_t v_t^T; o_t = S_t^T q_t; the heads side by side are RMS-normed together, times
    sigmoid(Wg h), through Wo."""
    T = h.shape[0]
    H, dk, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = rnd(plain_silu(h @ w["q"].T)).view(T, H, dk)
    k = rnd(plain_silu(h @ w["k"].T)).view(T, H, dk)
    v = rnd(plain_silu(h @ w["v"].T)).view(T, H, dv)
    decay = torch.tensor([float(d) for d in m["decay"]], dtype=h.dtype)
    S = torch.zeros(H, dk, dv, dtype=h.dtype)
    rows = []
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        rows.append(torch.einsum("hkv,hk->hv", S, q[t]).reshape(H * dv))
    o = plain_rmsnorm(torch.stack(rows), w["norm"], eps) * plain_sigmoid(h @ w["g"].T)
    return rnd(o) @ w["o"].T


# -- softmax attention -------------------------------------------------------------------------------------------------
def plain_rotary_frequencies(rot: dict) -> torch.Tensor:
    """f_i = base^(-2i/dims), i < dims/2, then scaled by wavelength: short waves kept, long ones divided by the
    factor, a linear blend between."""
    dims, base = int(rot["dims"]), float(rot["base"])
    out = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if sc is not None:
            factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
            wave = 2.0 * math.pi / f
            if wave > orig / low:
                f = f / factor
            elif not wave < orig / high:
                s = (orig / wave - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64)


def plain_rotate(x: torch.Tensor, freqs: torch.Tensor, positions: Sequence[int]) -> torch.Tensor:
    """x: [T, heads, dim]; features (2i, 2i+1), i < len(freqs), of every head are turned by the angle position * f_i;
    the others pass."""
    out = x.clone()
    pos = torch.tensor(list(positions), dtype=torch.float64)
    ang = (pos[:, None] * freqs[None, :]).to(x.dtype)       # [T, dims/2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    n = 2 * freqs.shape[0]
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    out[..., 0:n:2] = u * c - v * s
    out[..., 1:n:2] = v * c + u * s
    return out


def plain_visible(i: int, j: int, size: int, keep_first: int) -> bool:
    return j <= i and (i - j < size or j < keep_first)


def plain_softmax_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, rnd: Callable = _same) -> torch.Tensor:
    T = h.shape[0]
    H, G, dk, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w["q"].T + w["q.b"]).view(T, H, dk)
    k = (h @ w["k"].T + w["k.b"]).view(T, G, dk)
    v = (h @ w["v"].T + w["v.b"]).view(T, G, dv)
    freqs = plain_rotary_frequencies(m["rot"])
    q = rnd(plain_rotate(q, freqs, range(T)))
    k = rnd(plain_rotate(k, freqs, range(T)))
    v = rnd(v)
    scale, cap = float(m["scale"]), float(m["softcap"])
    size, keep = int(m["mask"]["size"]), int(m["mask"]["keep_first"])
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head, :] @ k[:, g, :].T) * scale
        s = cap * torch.tanh(s / cap)
        mask = torch.tensor([[plain_visible(i, j, size, keep) for j in range(T)] for i in range(T)])
        s = s.masked_fill(~mask, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, head, :] = rnd(p) @ v[:, g, :]
    return rnd(out.reshape(T, H * dv)) @ w["o"].T + w["o.b"]


# -- gated delta rule --------------------------------------------------------------------------------------------------
def plain_short_conv(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x: [T, C]; taps [C, K]: the last column weighs the current token, the one before it the token before; zeros
    before the start; no bias."""
    T, C = x.shape
    K = taps.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(K):
            src = t - (K - 1 - j)
            if src >= 0:
                y[t] += taps[:, j] * x[src]
    return y


def plain_delta_rule(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float, rnd: Callable = _same) -> torch.Tensor:
    T = h.shape[0]
    H, G, dk, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = rnd(plain_silu(plain_short_conv(h @ w["q"].T, w["q.conv"]))).view(T, G, dk)
    k = rnd(plain_silu(plain_short_conv(h @ w["k"].T, w["k.conv"]))).view(T, G, dk)
    v = rnd(plain_silu(plain_short_conv(h @ w["v"].T, w["v.conv"]))).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(dim=-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(dim=-1, keepdim=True) + 1e-6)
    beta = plain_sigmoid(h @ w["b"].T)                                                  # [T, H]
    a = rnd(h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]                                    # [T, H * dk]
    g = torch.exp(-torch.exp(w["A_log"])[None, :, None] * plain_softplus(a).view(T, H, dk))
    gate = plain_sigmoid(rnd(h @ w["g1"].T) @ w["g2"].T).view(T, H, dv)
    S = torch.zeros(H, dk, dv, dtype=h.dtype)
    rows = []
    rep = H // G
    for t in range(T):
        kt = k[t].repeat_interleave(rep, dim=0)            # head -> its q/k head
        qt = q[t].repeat_interleave(rep, dim=0)
        S = g[t][:, :, None] * S
        u = beta[t][:, None] * (v[t] - torch.einsum("hkv,hk->hv", S, kt))
        S = S + kt[:, :, None] * u[:, None, :]
        rows.append(torch.einsum("hkv,hk->hv", S, qt))
    o = torch.stack(rows)                                  # [T, H, dv]
    o = plain_rmsnorm(o, w["norm"], eps) * gate
    return rnd(o.reshape(T, H * dv)) @ w["o"].T


def _under(w: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {n[len(prefix):]: t for n, t in w.items() if n.startswith(prefix)}


def plain_parallel(h, w, m, eps, rnd=_same):
    left = plain_softmax_attention(h, _under(w, "left."), m["left"], rnd)
    right = plain_delta_rule(h, _under(w, "right."), m["right"], eps, rnd)
    return 0.5 * (plain_rmsnorm(left, w["left.out"], eps) + plain_rmsnorm(right, w["right.out"], eps))


# -- feed-forwards -----------------------------------------------------------------------------------------------------
def plain_dense_ff(h, w, rnd=_same):
    return rnd(plain_relu2(h @ w["up"].T)) @ w["down"].T


def plain_routed_ff(h, w, mlp: dict, rnd=_same):
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    s = torch.softmax(h @ w["router"].T, dim=-1)
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        chosen = sorted(range(E), key=lambda e: (-float(s[t, e]), e))[:top]
        for e in chosen:
            out[t] += s[t, e] * plain_dense_ff(h[t:t + 1], _under(w, f"e{e}."), rnd)[0]
    return out


# -- the model ---------------------------------------------------------------------------------------------------------
def plain_lilatar_logits(cfg: dict, tensors: Dict[str, torch.Tensor], tokens: Sequence[int], compute=torch.float64,
                         rnd: Callable = _same, layers_out: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from position 0.  `layers_out`: gets the stream after every layer."""
    w = {n: t.to(compute) for n, t in tensors.items()}
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.tensor(list(tokens))]
    for i, layer in enumerate(cfg["layers"]):
        lw = _under(w, f"l{i}.")
        hin = rnd(plain_rmsnorm(x, lw["norm1"], eps))
        mw = _under(lw, "mix.")
        if layer["type"] == "lightning":
            y = plain_lightning(hin, mw, layer["mixer"], eps, rnd)
        elif layer["type"] == "parallel":
            y = plain_parallel(hin, mw, layer["mixer"], eps, rnd)
        else:
            raise ValueError(layer["type"])
        x = x + plain_rmsnorm(y, lw["norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            hin = rnd(plain_rmsnorm(x, lw["norm2"], eps))
            fw = _under(lw, "mlp.")
            y = plain_dense_ff(hin, fw, rnd) if mlp["kind"] == "dense" else plain_routed_ff(hin, fw, mlp, rnd)
            x = x + plain_rmsnorm(y, lw["norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return (rnd(plain_rmsnorm(x, w["final.norm"], eps)) @ w["head"].T) * float(cfg["logit_scale"])
