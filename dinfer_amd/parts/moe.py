"""Routed feed-forward (mixture of experts).

    z = Wr x  (float)            the `top` experts with the largest z are chosen per token,
    p = softmax over the chosen z only
    y = sum_chosen p_e * down_e( silu(gate_e x) * up_e x )
        + sigmoid(wsg . x) * shared(x)          (a gated feed-forward every token runs, where the layer has one)

(The softmax over the chosen logits is the softmax over all experts with the chosen scores divided by their sum.)
With `gated=False` an expert, and the shared one, is down_e( act(up_e x) ) with act "silu" or "gelu" (error function);
with `shared_gate=False` the shared expert's output is added as it is.

Another rule of routing (`scores="all"`): the scores are the softmax of z over all router outputs; the `top` largest
of score + correction are chosen (`correction`, a tensor of one number a router output, only moves the choice), and a
chosen expert's weight is its score as it is, so a token's weights need not sum to one. `identity` experts: the router
has `experts + identity` outputs, and the last `identity` of them stand for experts without tensors whose output is
their input (times the weight).

Per step: one kernel routes (logits, choice, weights, the shared gate), one sorts the (token, choice) entries by
expert and writes the work list of row tiles, two launches run the products of all experts (gate and up with the
activation, then down, each row computed alone and written to its entry's place), and one sums a token's entries in
the order of its choices. Launch shapes depend on the step's token count alone; which expert gets which rows is read
from device memory, so the step may be captured. No atomics on results: a token's output does not depend on what
else is in the batch.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import FeedForward
from .mlp import MLP, GatedMLP
from .registry import FEED_FORWARDS
from .spec import TensorSpec


@FEED_FORWARDS.register("moe")
class RoutedExperts(FeedForward):
    """Tensors: e<i>.gate / .up / .down per expert, router [experts, hidden]; shared.gate / .up / .down and shared.sg
    [1, hidden] where `shared_intermediate` is given."""

    def __init__(self, hidden: int, experts: int, top: int, intermediate: int, shared_intermediate: int | None = None,
                 act: str = "silu", gated: bool = True, shared_gate: bool = True, scores: str = "chosen",
                 correction: bool = False, identity: int = 0):
        if gated and act != "silu":
            raise ValueError(f"routed feed-forward: gated activation {act!r} has no kernel (known: ['silu'])")
        if not gated and act not in ops.EXPERT_ACTS:
            raise ValueError(f"routed feed-forward: activation {act!r} has no kernel (known: {sorted(ops.EXPERT_ACTS)})")
        if scores not in ("chosen", "all") or identity < 0 or (scores != "all" and (correction or identity)):
            raise ValueError(f"routed feed-forward: scores {scores!r} with correction {correction} and {identity} identity "
                             "experts: a correction and identity experts go with scores over all router outputs")
        self.all_scores, self.has_correction, self.identity = scores == "all", bool(correction), int(identity)
        self.outputs = experts + self.identity          # what the router gives a token
        if not (0 < top <= self.outputs) or self.outputs > ops.MOE_MAX_EXPERTS or top > ops.MOE_MAX_TOP:
            raise ValueError(f"routed feed-forward: {top} of {experts} experts has no kernel (up to {ops.MOE_MAX_TOP} of "
                             f"{ops.MOE_MAX_EXPERTS})")
        self.hidden, self.experts, self.top, self.intermediate = hidden, experts, top, intermediate
        self.gated, self.act, self.shared_gate_on = bool(gated), act, bool(shared_gate)
        self.shared = None
        if shared_intermediate and gated:
            self.shared = GatedMLP(hidden, shared_intermediate, act, names=("shared.gate", "shared.up", "shared.down"),
                                   out_name="shared_out")
        elif shared_intermediate:
            self.shared = MLP(hidden, shared_intermediate, act, names=("shared.up", "shared.down"), out_name="shared_out",
                              act_name="shared_act")

    def tensors(self):
        t = {"router": TensorSpec((self.outputs, self.hidden))}
        if self.has_correction:
            t["correction"] = TensorSpec((self.outputs,), init="zeros")
        for e in range(self.experts):
            if self.gated:
                t[f"e{e}.gate"] = TensorSpec((self.intermediate, self.hidden))
            t[f"e{e}.up"] = TensorSpec((self.intermediate, self.hidden))
            t[f"e{e}.down"] = TensorSpec((self.hidden, self.intermediate))
        if self.shared is not None:
            t.update(self.shared.tensors())
            if self.shared_gate_on:
                t["shared.sg"] = TensorSpec((1, self.hidden))
        return t

    def load(self, get):
        self.router = get("router").float().contiguous()       # routing runs in 32 bits
        self.correction = get("correction").float().contiguous() if self.has_correction else None
        E = range(self.experts)
        # [experts, 2 I, hidden]: an expert's gate rows, then its up rows (not gated: [experts, I, hidden]); [experts, hidden, I]
        if self.gated:
            self.w_in = torch.stack([torch.cat([get(f"e{e}.gate", compute=True), get(f"e{e}.up", compute=True)], dim=0)
                                     for e in E]).contiguous()
        else:
            self.w_in = torch.stack([get(f"e{e}.up", compute=True) for e in E]).contiguous()
        self.w_out = torch.stack([get(f"e{e}.down", compute=True) for e in E]).contiguous()
        self.sg = None
        if self.shared is not None:
            self.shared.load(get)
            if self.shared_gate_on:
                self.sg = get("shared.sg").float().reshape(-1).contiguous()

    def bind(self, ctx):
        ws, dev = ctx.workspace, ctx.device
        n = ctx.max_tokens * self.top
        i32 = torch.int32
        self.idx = torch.zeros(n, dtype=i32, device=dev)
        self.share = torch.zeros(n, dtype=torch.float32, device=dev)
        self.logits = torch.zeros(ctx.max_tokens * (self.outputs + 1), dtype=torch.float32, device=dev)
        self.shared_gate = torch.zeros(ctx.max_tokens, dtype=torch.float32, device=dev)
        self.offsets = torch.zeros(self.outputs + 1, dtype=i32, device=dev)
        self.perm = torch.zeros(n, dtype=i32, device=dev)
        self.dtype = ctx.dtype
        self.tiles = torch.zeros((ops.moe_max_tiles(n, self.outputs, 16), 2), dtype=i32, device=dev)   # the smallest tile: the longest list
        self.act_buf = ws.buffer("moe_act", self.intermediate, rows=n)
        self.y_buf = ws.buffer("moe_y", self.hidden, rows=n)
        self.out_buf = ws.buffer("ffn_out", self.hidden)
        if self.shared is not None:
            self.shared.bind(ctx)

    def forward(self, x, batch, into=None):
        T, top = batch.num_tokens, self.top
        n = T * top
        ops.moe_route(x, self.router, self.sg, self.idx, self.share, self.shared_gate, T, top, self.logits,
                      all_scores=self.all_scores, correction=self.correction)
        rows = ops.moe_tile_rows(self.dtype, n, self.outputs, self.hidden, self.intermediate)   # follows the step's count alone
        ops.moe_scatter(self.idx, n, self.outputs, self.offsets, self.perm, self.tiles, rows, real_experts=self.experts)
        ops.experts_nt(x, self.w_in, self.act_buf, n, self.tiles, self.offsets, self.perm, gated=self.gated, a_div=top,
                       c_to_perm=False, tile_rows=rows, act=None if self.gated else self.act)
        ops.experts_nt(self.act_buf, self.w_out, self.y_buf, n, self.tiles, self.offsets, self.perm, gated=False, a_div=0,
                       c_to_perm=True, tile_rows=rows)
        shared = self.shared.forward(x, batch) if self.shared is not None else None
        same = dict(idx=self.idx, real_experts=self.experts, x=x) if self.identity else {}
        return ops.moe_combine(self.y_buf, self.share, top, shared, self.shared_gate if self.sg is not None else None,
                               self.out_buf, T, **same)
