"""Recurrent mixers: each keeps a state of fixed size per request (in the request's slot, 32-bit), reads it at the
start of a step's portion and leaves it for the next; nothing is paged.

"mingru"(hidden_size, width): gate z = sigmoid(Wz x + bz), candidate c = g(Wc x + bc) with g(u) = u + 1/2 for u >= 0
and sigmoid(u) below; s_t = (1 - z) s_{t-1} + z c; h += Wo (s_t * silu(Wg x)).  One product gives the three
projections' 32-bit sums; the scan kernel does the rest in 32-bit and writes the gated state in the activation type.

"mamba1"(hidden_size, inner, state, conv, dt_rank): the selective scan.  [x | g] = Win h (32-bit sums); x <-
silu(causal conv over `conv` taps, last tap the current token); [d | B | C] = Wx x; step = softplus(Wdt d + bdt);
S[c, n] <- exp(step_c A[c, n]) S[c, n] + step_c x_c B_n with A = -exp(A_log); y_c = sum_n S[c, n] C_n + D_c x_c;
h += Wo (y * silu(g)).  The request's state is S and the convolution's last conv - 1 inputs.
"""
from __future__ import annotations

import torch

from ..cache.spec import FixedState
from ..kernels import EPI_ACCUM_F32, EPI_STORE, EPI_STORE_F32, kernels
from .base import Mixer, TensorSpec, place, register_mixer


def _leaves(defaults: dict, given) -> dict:
    return {**defaults, **(given or {})}


class MinGRU(Mixer):
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        p = spec.params
        self.hidden, self.width = int(p["hidden_size"]), int(p["width"])
        leaves = _leaves({"gate": "z", "gate_bias": "z.b", "candidate": "x", "candidate_bias": "x.b", "out_gate": "g", "out": "o"}, p.get("names"))
        self.names = {k: self.name(v) for k, v in leaves.items()}
        self.w_in = self.w_o = self.bias_z = self.bias_c = None

    def tensors(self):
        n, W, H = self.names, self.width, self.hidden
        return {n["gate"]: TensorSpec((W, H)), n["gate_bias"]: TensorSpec((W,)), n["candidate"]: TensorSpec((W, H)),
                n["candidate_bias"]: TensorSpec((W,)), n["out_gate"]: TensorSpec((W, H)), n["out"]: TensorSpec((H, W))}

    def load(self, tensors, device):
        n = self.names
        get = lambda key: place(tensors[n[key]], device, self.dtype)
        self.w_in = torch.cat([get("gate"), get("candidate"), get("out_gate")], dim=0).contiguous()
        self.w_o = get("out")
        self.bias_z = place(tensors[n["gate_bias"]], device, torch.float32)
        self.bias_c = place(tensors[n["candidate_bias"]], device, torch.float32)

    def export(self):
        n, W = self.names, self.width
        w = self.w_in.cpu()
        return {n["gate"]: w[:W].contiguous(), n["candidate"]: w[W:2 * W].contiguous(), n["out_gate"]: w[2 * W:].contiguous(),
                n["out"]: self.w_o.cpu(), n["gate_bias"]: self.bias_z.cpu(), n["candidate_bias"]: self.bias_c.cpu()}

    def cache_need(self):
        return FixedState((self.width,), torch.float32)

    def forward(self, ctx, x, h, cache):
        k = kernels()
        T = x.shape[0]
        sums = ctx.workspace("mingru.sums", (T, 3 * self.width), torch.float32)
        k.gemm(x, self.w_in, sums, EPI_STORE_F32, ctx.gemm_workspace(x, self.w_in))
        gated = ctx.workspace("mingru.gated", (T, self.width), self.dtype)
        need = k.scan_carry_floats(T, ctx.n_entries, ctx.longest, 2 * self.width)
        carry = ctx.workspace("scan.carry", (need,), torch.float32) if need else None
        k.mingru_scan(sums, self.bias_z, self.bias_c, cache.state, ctx.q_starts, ctx.slots, self.width, gated, ctx.longest, carry)
        k.gemm(gated, self.w_o, h, EPI_ACCUM_F32, ctx.gemm_workspace(gated, self.w_o))
        ctx.note_left(h, None)


class Mamba1(Mixer):
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        p = spec.params
        self.hidden, self.inner, self.n_state = int(p["hidden_size"]), int(p["inner"]), int(p["state"])
        self.taps, self.dt_rank = int(p["conv"]), int(p["dt_rank"])
        if self.taps < 1:
            raise ValueError("the convolution has at least one tap")
        leaves = _leaves({"in": "in", "conv": "conv", "conv_bias": "conv.b", "x": "x", "dt": "dt", "dt_bias": "dt.b",
                          "A_log": "A_log", "D": "D", "out": "o"}, p.get("names"))
        self.names = {k: self.name(v) for k, v in leaves.items()}
        self.w_in = self.w_x = self.w_dt = self.w_o = None
        self.conv = self.conv_bias = self.dt_bias = self.A = self.A_log = self.D = None

    def tensors(self):
        n, C, H, N, R = self.names, self.inner, self.hidden, self.n_state, self.dt_rank
        return {n["in"]: TensorSpec((2 * C, H)), n["conv"]: TensorSpec((C, self.taps), "normal:0.0:0.3"), n["conv_bias"]: TensorSpec((C,)),
                n["x"]: TensorSpec((R + 2 * N, C)), n["dt"]: TensorSpec((C, R), "normal:0.0:0.1"), n["dt_bias"]: TensorSpec((C,), "normal:-2.0:0.5"),
                n["A_log"]: TensorSpec((C, N), "normal:0.0:0.5"), n["D"]: TensorSpec((C,), "norm"), n["out"]: TensorSpec((H, C))}

    def load(self, tensors, device):
        n = self.names
        get = lambda key: place(tensors[n[key]], device, self.dtype)
        get32 = lambda key: place(tensors[n[key]], device, torch.float32)
        self.w_in, self.w_x, self.w_dt, self.w_o = get("in"), get("x"), get("dt"), get("out")
        self.conv, self.conv_bias, self.dt_bias, self.D = get32("conv"), get32("conv_bias"), get32("dt_bias"), get32("D")
        self.A_log = get32("A_log")
        self.A = (-torch.exp(self.A_log)).t().contiguous()      # 32-bit, once; [state, inner] as the scan reads it

    def export(self):
        n = self.names
        return {n["in"]: self.w_in.cpu(), n["x"]: self.w_x.cpu(), n["dt"]: self.w_dt.cpu(), n["out"]: self.w_o.cpu(),
                n["conv"]: self.conv.cpu(), n["conv_bias"]: self.conv_bias.cpu(), n["dt_bias"]: self.dt_bias.cpu(),
                n["D"]: self.D.cpu(), n["A_log"]: self.A_log.cpu()}

    def step_weight_bytes(self, seen):
        seen.add(self.A_log.data_ptr())      # a step reads A, not its logarithm
        return super().step_weight_bytes(seen)

    def cache_need(self):
        # one row per request: the scan's state [state, inner], then the convolution's last inputs [conv - 1, inner]
        return FixedState((self.inner * self.n_state + (self.taps - 1) * self.inner,), torch.float32)

    def forward(self, ctx, x, h, cache):
        k = kernels()
        T, C, N, R = x.shape[0], self.inner, self.n_state, self.dt_rank
        sums = ctx.workspace("mamba.sums", (T, 2 * C), torch.float32)
        k.gemm(x, self.w_in, sums, EPI_STORE_F32, ctx.gemm_workspace(x, self.w_in))
        scan_state, conv_state = cache.state[:, :C * N], cache.state[:, C * N:]
        xc = ctx.workspace("mamba.x", (T, C), self.dtype)
        k.causal_conv_silu(sums, self.conv, self.conv_bias, conv_state, ctx.q_starts, ctx.slots, ctx.token_entry, C, xc)
        dbc = ctx.workspace("mamba.dbc", (T, R + 2 * N), self.dtype)
        k.gemm(xc, self.w_x, dbc, EPI_STORE, ctx.gemm_workspace(xc, self.w_x))
        dt = ctx.workspace("mamba.dt", (T, C), torch.float32)
        d = dbc[:, :R]
        k.gemm(d, self.w_dt, dt, EPI_STORE_F32, ctx.gemm_workspace(d, self.w_dt))
        y = ctx.workspace("mamba.y", (T, C), self.dtype)
        ypart = ctx.workspace("mamba.ypart", (T, C), torch.float32) if N > 64 else None
        need = k.scan_carry_floats(T, ctx.n_entries, ctx.longest, (N + 1) * C)
        carry = ctx.workspace("scan.carry", (need,), torch.float32) if need else None
        k.selective_scan(xc, dbc, R, R + N, dt, self.dt_bias, self.A, self.D, sums[:, C:], scan_state, ctx.q_starts, ctx.slots, y, ypart,
                         ctx.longest, carry)
        k.gemm(y, self.w_o, h, EPI_ACCUM_F32, ctx.gemm_workspace(y, self.w_o))
        ctx.note_left(h, None)


register_mixer("mingru", MinGRU)
register_mixer("mamba1", Mamba1)
