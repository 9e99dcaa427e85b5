"""Gated feed-forward: down( act(gate(x)) * up(x) ), gate and up fused into one
[2I, hidden] operand with the gate rows first (crates/layers/src/nn.rs:272-390).
Plain feed-forward ("mlp"): down( act(up(x)) ) with an activation of one argument (silu, the square of relu, gelu)."""
from __future__ import annotations

import torch

from ..kernels import gemm, ops
from .base import Carried, FeedForward
from .linear import Linear
from .registry import FEED_FORWARDS
from .spec import TensorSpec


@FEED_FORWARDS.register("gated_mlp")
class GatedMLP(FeedForward):
    carries_norms = True   # the gate/up product takes a Carried, the down product an Into

    def __init__(self, hidden: int, intermediate: int, act: str = "silu",
                 names: tuple = ("gate_proj.weight", "up_proj.weight", "down_proj.weight"), out_name: str = "ffn_out"):
        if act not in ops.GATED_ACTS:   # said when the model is built, not at its first step
            raise ValueError(f"gated feed-forward: activation {act!r} has no kernel (known: {sorted(ops.GATED_ACTS)})")
        self.hidden, self.intermediate, self.act = hidden, intermediate, act
        self.names, self.out_name = tuple(names), out_name
        self.gate_up = Linear(hidden, 2 * intermediate)
        self.down = Linear(intermediate, hidden)

    def tensors(self):
        g, u, d = self.names
        return {
            g: TensorSpec((self.intermediate, self.hidden)),
            u: TensorSpec((self.intermediate, self.hidden)),
            d: TensorSpec((self.hidden, self.intermediate)),
        }

    def load(self, get):
        g, u, d = self.names
        self.gate_up.set_weight(torch.cat([get(g, compute=True), get(u, compute=True)], dim=0))
        self.down.set_weight(get(d, compute=True))

    def bind(self, ctx):
        ws = ctx.workspace
        self.gu_buf = ws.buffer("gate_up", 2 * self.intermediate)
        self.act_buf = ws.buffer("act", self.intermediate)
        self.out_buf = ws.buffer(self.out_name, self.hidden)

    def forward(self, x, batch, into=None):
        T = batch.num_tokens
        w = self.gate_up.weight
        if isinstance(x, Carried):
            if not (x.scaled and self.act == "silu" and gemm.scaled_nt(x.xg, x.stats, x.cols, x.eps, x.width, w, self.act_buf, T, gated=True)):
                x = x.materialise()
        if not isinstance(x, Carried):
            # decode-sized steps: both projections and the activation in one weight-streaming kernel
            gemm.gated_nt(x, w, self.act_buf, self.gu_buf, T, self.act)
        if into is not None:
            done = self.down.forward_into(self.act_buf, into, T)
            if done is not None:
                return done
        return self.down.forward(self.act_buf, self.out_buf, T, scratch=True)


@FEED_FORWARDS.register("mlp")
class MLP(FeedForward):
    """down( act(up(x)) ), no gate. act: a name of ops.ACTS."""

    def __init__(self, hidden: int, intermediate: int, act: str = "relu2", names: tuple = ("up", "down"),
                 out_name: str = "ffn_out", act_name: str = "act"):
        if act not in ops.ACTS:
            raise ValueError(f"feed-forward: activation {act!r} has no kernel (known: {sorted(ops.ACTS)})")
        self.hidden, self.intermediate, self.act, self.names = hidden, intermediate, act, tuple(names)
        self.out_name, self.act_name = out_name, act_name
        self.up = Linear(hidden, intermediate)
        self.down = Linear(intermediate, hidden)

    def tensors(self):
        u, d = self.names
        return {u: TensorSpec((self.intermediate, self.hidden)), d: TensorSpec((self.hidden, self.intermediate))}

    def load(self, get):
        u, d = self.names
        self.up.set_weight(get(u, compute=True))
        self.down.set_weight(get(d, compute=True))

    def bind(self, ctx):
        ws = ctx.workspace
        self.act_buf = ws.buffer(self.act_name, self.intermediate)
        self.out_buf = ws.buffer(self.out_name, self.hidden)

    def forward(self, x, batch, into=None):
        T = batch.num_tokens
        self.up.forward(x, self.act_buf, T, scratch=True)
        ops.act(self.act_buf, self.act_buf, T, self.act)
        return self.down.forward(self.act_buf, self.out_buf, T, scratch=True)


@FEED_FORWARDS.register("none")
class NoFeedForward(FeedForward):
    """A layer without a feed-forward: the block arrangement skips it and the norm before it."""
    absent = True

    def __init__(self, hidden: int):
        self.hidden = hidden
