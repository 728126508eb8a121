"""SwiGLU feed-forward(hidden_size, intermediate_size):
h += (silu(x Wg^T) * (x Wu^T)) Wd^T, silu(v) = v / (1 + exp(-v))
(src/arch/llama.rs:165-170, shaders/ops.metal:762-793).  The gate and up weights
are interleaved row by row at load, so one product yields (gate_j, up_j) side by
side and its epilogue writes silu(gate) * up, computed in 32-bit, once; the down
product adds into the 32-bit residual stream.  No biases."""
from __future__ import annotations

import torch

from ..kernels import EPI_ACCUM_F32, EPI_STORE_F32, EPI_SWIGLU, kernels
from .base import FeedForward, TensorSpec, place, register_feed_forward


class SwiGLU(FeedForward):
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        # the leaves of the three tensors' names, for files that call them otherwise: {"gate": ..., "up": ..., "down": ...}
        leaves = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight", **(spec.params.get("names") or {})}
        self.n_gate, self.n_up, self.n_down = (self.name(leaves[k]) for k in ("gate", "up", "down"))
        self.w_gate_up = None
        self.w_down = None

    def tensors(self):
        return {self.n_gate: TensorSpec((self.inter, self.hidden)),
                self.n_up: TensorSpec((self.inter, self.hidden)),
                self.n_down: TensorSpec((self.hidden, self.inter))}

    def load(self, tensors, device):
        gate = place(tensors[self.n_gate], device, self.dtype)
        up = place(tensors[self.n_up], device, self.dtype)
        self.w_gate_up = torch.stack([gate, up], dim=1).reshape(2 * self.inter, self.hidden).contiguous()
        self.w_down = place(tensors[self.n_down], device, self.dtype)

    def export(self):
        both = self.w_gate_up.cpu().view(self.inter, 2, self.hidden)
        return {self.n_gate: both[:, 0, :].contiguous(), self.n_up: both[:, 1, :].contiguous(),
                self.n_down: self.w_down.cpu()}

    def takes_normed_rows(self, ctx, rows):
        return kernels().product_norms_its_rows(rows, 2 * self.inter, self.hidden, self.dtype)

    def forward(self, ctx, x, h):
        k = kernels()
        act = ctx.workspace("mlp.act", (x.shape[0], self.inter), self.dtype)
        k.gemm(x, self.w_gate_up, act, EPI_SWIGLU, ctx.gemm_workspace(x, self.w_gate_up))
        leave = ctx.room_for_next_norm(h, self.w_down)
        k.gemm(act, self.w_down, h, EPI_ACCUM_F32, ctx.gemm_workspace(act, self.w_down), **({} if leave is None else {"leave": leave}))
        ctx.note_left(h, leave)


register_feed_forward("swiglu", SwiGLU)


ACTIVATIONS = ("relu2",)        # relu(x)^2


class PlainFF(FeedForward):
    """Feed-forward without a gate(hidden_size, intermediate_size, activation): h += Wdown act(Wup x).  The up product
    leaves 32-bit sums; the activation is computed on them and rounded once to the activation type."""
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        self.activation = spec.params.get("activation", "relu2")
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"unknown activation {self.activation!r} (known: {', '.join(ACTIVATIONS)})")
        leaves = {"up": "up_proj.weight", "down": "down_proj.weight", **(spec.params.get("names") or {})}
        self.n_up, self.n_down = self.name(leaves["up"]), self.name(leaves["down"])
        self.w_up = self.w_down = None

    def tensors(self):
        return {self.n_up: TensorSpec((self.inter, self.hidden)), self.n_down: TensorSpec((self.hidden, self.inter))}

    def load(self, tensors, device):
        self.w_up = place(tensors[self.n_up], device, self.dtype)
        self.w_down = place(tensors[self.n_down], device, self.dtype)

    def export(self):
        return {self.n_up: self.w_up.cpu(), self.n_down: self.w_down.cpu()}

    def forward(self, ctx, x, h):
        k = kernels()
        T = x.shape[0]
        up = ctx.workspace("mlp.up", (T, self.inter), torch.float32)
        k.gemm(x, self.w_up, up, EPI_STORE_F32, ctx.gemm_workspace(x, self.w_up))
        act = ctx.workspace("mlp.act", (T, self.inter), self.dtype)
        k.act_weight(act, up, None, self.inter)
        k.gemm(act, self.w_down, h, EPI_ACCUM_F32, ctx.gemm_workspace(act, self.w_down))
        ctx.note_left(h, None)


class RoutedFF(FeedForward):
    """Mixture of experts(hidden_size, intermediate_size, experts, top, activation, renormalize): each expert is a
    feed-forward without a gate; scores = softmax(Wrouter x) over all experts in 32-bit, the `top` largest are chosen,
    and the output is the sum of the chosen experts' outputs, each weighed by its score (as it is, or with
    `renormalize` divided by the chosen scores' sum).

    The experts' up matrices are laid one under the other and their down matrices side by side at load, so a step's
    experts are one up product of experts * intermediate_size columns, one pass that applies the activation and each
    column's expert weight (zero where the token did not choose the expert), and one down product: w_e Wdown_e act(.)
    = Wdown_e (w_e act(.)).  Names: `router`, and `expert` with a place for the expert's number (e.g. "e{}")."""
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        p = spec.params
        self.hidden, self.inter = int(p["hidden_size"]), int(p["intermediate_size"])
        self.experts, self.top = int(p["experts"]), int(p["top"])
        self.renormalize = bool(p.get("renormalize", False))
        self.activation = p.get("activation", "relu2")
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"unknown activation {self.activation!r} (known: {', '.join(ACTIVATIONS)})")
        if not 1 <= self.top <= self.experts:
            raise ValueError(f"top = {self.top} of {self.experts} experts")
        leaves = {"router": "router.weight", "expert": "experts.{}", "up": "up_proj.weight", "down": "down_proj.weight", **(p.get("names") or {})}
        self.n_router = self.name(leaves["router"])
        self.n_up = [self.name(leaves["expert"].format(e) + "." + leaves["up"]) for e in range(self.experts)]
        self.n_down = [self.name(leaves["expert"].format(e) + "." + leaves["down"]) for e in range(self.experts)]
        self.w_router = self.w_up = self.w_down = None

    def tensors(self):
        t = {self.n_router: TensorSpec((self.experts, self.hidden), "normal:0.0:0.1")}
        for e in range(self.experts):
            t[self.n_up[e]] = TensorSpec((self.inter, self.hidden))
            t[self.n_down[e]] = TensorSpec((self.hidden, self.inter))
        return t

    def load(self, tensors, device):
        self.w_router = place(tensors[self.n_router], device, self.dtype)
        self.w_up = torch.cat([place(tensors[n], device, self.dtype) for n in self.n_up], dim=0).contiguous()
        self.w_down = torch.cat([place(tensors[n], device, self.dtype) for n in self.n_down], dim=1).contiguous()

    def export(self):
        up, down = self.w_up.cpu(), self.w_down.cpu()
        t = {self.n_router: self.w_router.cpu()}
        for e in range(self.experts):
            t[self.n_up[e]] = up[e * self.inter:(e + 1) * self.inter].contiguous()
            t[self.n_down[e]] = down[:, e * self.inter:(e + 1) * self.inter].contiguous()
        return t

    def step_weight_bytes(self, seen):
        # a single token reads the router and the experts it chose
        total = super().step_weight_bytes(seen)
        experts = (self.w_up.numel() + self.w_down.numel()) * self.w_up.element_size()
        return total - experts + experts * self.top // self.experts

    def forward(self, ctx, x, h):
        k = kernels()
        T, N = x.shape[0], self.experts * self.inter
        logits = ctx.workspace("moe.logits", (T, self.experts), torch.float32)
        k.gemm(x, self.w_router, logits, EPI_STORE_F32, ctx.gemm_workspace(x, self.w_router))
        weights = ctx.workspace("moe.weights", (T, self.experts), torch.float32)
        k.route_topk(logits, weights, self.top, self.renormalize)
        up = ctx.workspace("mlp.up", (T, N), torch.float32)
        k.gemm(x, self.w_up, up, EPI_STORE_F32, ctx.gemm_workspace(x, self.w_up))
        act = ctx.workspace("mlp.act", (T, N), self.dtype)
        k.act_weight(act, up, weights, self.inter)
        k.gemm(act, self.w_down, h, EPI_ACCUM_F32, ctx.gemm_workspace(act, self.w_down))
        ctx.note_left(h, None)


register_feed_forward("plain_ff", PlainFF)
register_feed_forward("routed_ff", RoutedFF)
