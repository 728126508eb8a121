"""Hyper-connections: the residual stream kept as several copies that every sublayer reads through weights of its own
and writes back through a small mixing matrix.

For a sublayer f with its norm and its connection (in [S], out [S], mix [S, S] indexed [from, to]):
    u = sum_s in[s] x_s;   y = f(norm(u));   x_r <- sum_s mix[s, r] x_s + out[r] y     (all r from the old copies)
The block arrangement "hyper" runs a mixer and, where the layer has one, a feed-forward this way.  The copies, the
combination and the mix are 32-bit.  The connection is a part of its own family ("connection"), so that its three
tensors are loaded, checked and given back like any other part's.
"""
from __future__ import annotations

import torch

from ..kernels import kernels
from .base import Block, Part, TensorSpec, place, register_block, register_part_family


class HyperConnection(Part):
    """streams: how many copies.  Tensors: `in` [S], `out` [S], `mix` [S, S]."""
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        self.streams = int(spec.params["streams"])
        self.w_in = self.w_out = self.mix = None

    def tensors(self):
        S = self.streams
        return {self.name("in"): TensorSpec((S,), "normal:0.3:0.1"), self.name("out"): TensorSpec((S,), "normal:1.0:0.1"),
                self.name("mix"): TensorSpec((S, S), "normal:0.25:0.1")}

    def load(self, tensors, device):
        self.w_in = place(tensors[self.name("in")], device, torch.float32)
        self.w_out = place(tensors[self.name("out")], device, torch.float32)
        self.mix = place(tensors[self.name("mix")], device, torch.float32)

    def export(self):
        return {self.name("in"): self.w_in.cpu(), self.name("out"): self.w_out.cpu(), self.name("mix"): self.mix.cpu()}

    def write(self, ctx, hs: torch.Tensor, y: torch.Tensor) -> None:
        """The mix is left to whoever reads the streams next: a norm that reads every row does it in its own
        launch; anyone else asks the context to do it first (`flush_streams`)."""
        ctx.defer_streams_mix(hs, self.mix, self.w_out, y)


register_connection = register_part_family("connection")
register_connection("hyper", HyperConnection)


class HyperBlock(Block):
    """h: [streams, T, hidden].  Parts: mixer, mixer_norm, mixer_connection; feed_forward, feed_forward_norm and
    feed_forward_connection together or not at all.  The norms must read several copies (`Norm.forward_streams`)."""
    needs = ("mixer", "mixer_norm", "mixer_connection")
    takes_streams = True

    def __init__(self, named):
        super().__init__(named)
        self.mixer_connection = self.named["mixer_connection"]
        self.feed_forward_connection = self.named.get("feed_forward_connection")
        if self.feed_forward is not None and (self.feed_forward_norm is None or self.feed_forward_connection is None):
            raise ValueError("a feed-forward on hyper-connections needs its norm and its connection")

    def _half(self, ctx, hs, norm, connection, run) -> None:
        T, D = hs.shape[1], hs.shape[2]
        x = ctx.workspace("block.x", (T, D), self.mixer.dtype)
        y = ctx.workspace("block.y", (T, D), torch.float32)      # the sublayer adds its result into y, cleared by the norm's kernel
        ctx.note_left(hs, None)
        ctx.upcoming_norm = None
        if not norm.forward_streams(ctx, hs, connection.w_in, x, zero=y):
            raise ValueError(f"{type(norm).__name__} cannot read a stream kept in several copies")
        run(x, y)
        connection.write(ctx, hs, y)

    def forward(self, ctx, hs, cache):
        self._half(ctx, hs, self.mixer_norm, self.mixer_connection, lambda x, y: self.mixer.forward(ctx, x, y, cache))
        if self.feed_forward is not None:
            self._half(ctx, hs, self.feed_forward_norm, self.feed_forward_connection, lambda x, y: self.feed_forward.forward(ctx, x, y))
        ctx.upcoming_norm = None


register_block("hyper", HyperBlock)
