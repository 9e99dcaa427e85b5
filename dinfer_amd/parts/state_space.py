"""State-space mixer with a scalar decay a head and token ("Mamba-2", state-space duality).

With h the mixer's input, H heads of size P, state size N, G groups (head i reads group i // (H / G)), inner = H P:

    z | x | B | C | dt = W_in h          (inner | inner | G N | G N | H)
    x, B, C <- silu(conv(x | B | C) + bias)      conv: a few taps a channel over time, causal, zeros before the start
    dt <- softplus(dt + dt_bias)                 (float, no clamp)
    S <- exp(-exp(A_log) dt) S + dt B x^T;   y = S^T C + D x             (per head, token by token, S float32 [N, P])
    out = W_o( norm_groups( y * silu(z) ) * w )    the gate comes before the norm; the norm divides each of `norm_groups`
                                                   equal parts of the inner columns by its own root mean square

One product makes all five; everything after it up to the operand of W_o is float (csrc/decay.hip): the recurrence is
the one of the retention mixer with q = C, k = B, v = x, a decay and a step size a token. The state and the
convolution's last taps - 1 inputs live in the request's state slot (DeltaStateSpec); a request's first step
(position 0) starts from zeros.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import CacheView, Mixer
from .linear import Linear
from .registry import MIXERS
from .spec import DeltaStateSpec, TensorSpec


@MIXERS.register("state_space")
class StateSpace(Mixer):
    capturable = True            # every kernel reads slots, lengths and row counts from the batch's device buffers
    capturable_portions = True

    NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "A_log": "A_log", "D": "D",
             "norm": "norm", "o": "o"}

    def __init__(self, hidden: int, heads: int, vdim: int, state: int, groups: int, taps: int, norm_groups: int,
                 norm_eps: float, conv_bias: bool = True, names: dict | None = None):
        if heads % groups:
            raise ValueError(f"state space: heads {heads} not divisible by groups {groups}")
        if (heads * vdim) % norm_groups:
            raise ValueError(f"state space: {norm_groups} norm groups do not divide heads * vdim {heads * vdim}")
        if not (0 < state <= ops.DECAY_MAX_DIM and vdim > 0 and 0 < taps <= ops.DELTA_MAX_TAPS):
            raise ValueError(f"state space: state {state} or {taps} taps have no kernel (state up to {ops.DECAY_MAX_DIM}, "
                             f"taps up to {ops.DELTA_MAX_TAPS})")
        self.hidden, self.heads, self.vdim, self.state, self.groups, self.taps = hidden, heads, vdim, state, groups, taps
        self.norm_groups, self.norm_eps, self.conv_bias = norm_groups, float(norm_eps), bool(conv_bias)
        self.names = dict(self.NAMES, **(names or {}))
        self.inner, self.gn = heads * vdim, groups * state
        self.channels = self.inner + 2 * self.gn
        self.x_off = self.inner                      # z | x | B | C | dt
        self.dt_off = self.inner + self.channels
        self.used = self.dt_off + heads
        self.proj = Linear(hidden, -(-self.used // 8) * 8)     # rows padded to 8 with zeros
        self.o = Linear(self.inner, hidden)

    def cache_spec(self):
        return DeltaStateSpec(self.heads, self.state, self.vdim, self.channels, self.taps)

    def tensors(self):
        n, Hd = self.names, self.hidden
        t = {n["in"]: TensorSpec((self.used, Hd)), n["conv"]: TensorSpec((self.channels, self.taps)),
             n["dt_bias"]: TensorSpec((self.heads,)), n["A_log"]: TensorSpec((self.heads,)),
             n["D"]: TensorSpec((self.heads,), init="ones"), n["norm"]: TensorSpec((self.inner,), init="gain"),
             n["o"]: TensorSpec((Hd, self.inner))}
        if self.conv_bias:
            t[n["conv_bias"]] = TensorSpec((self.channels,), init="zeros")
        return t

    def load(self, get):
        n = self.names
        w = get(n["in"], compute=True)
        if w.shape[0] < self.proj.out_features:
            w = torch.cat([w, w.new_zeros(self.proj.out_features - w.shape[0], self.hidden)], dim=0)
        self.proj.set_weight(w)
        self.o.set_weight(get(n["o"], compute=True))
        # small parameters in 32 bits (exact for a bfloat16 file): they enter the recurrence
        self.conv_taps = get(n["conv"]).float().contiguous()
        self.conv_b = get(n["conv_bias"]).float().contiguous() if self.conv_bias else None
        self.a_log = get(n["A_log"]).float().contiguous()
        self.dt_bias = get(n["dt_bias"]).float().contiguous()
        self.skip = get(n["D"]).float().contiguous()
        self.norm_weight = get(n["norm"]).float().contiguous()

    def bind(self, ctx):
        ws = ctx.workspace
        self.proj_buf = ws.buffer("ssm_proj", self.proj.out_features)
        self.gated_buf = ws.buffer("ssm_gated", self.inner)
        self.out_buf = ws.buffer("mixer_out", self.hidden)
        self.work = ws.buffer("ssm_work", self.channels + 2 * self.heads, dtype=torch.float32)
        self.y_buf = ws.buffer("ssm_y", self.inner, dtype=torch.float32)

    def forward(self, x, batch, cache: CacheView):
        T, B = batch.num_tokens, batch.num_reqs
        common = dict(state_slots=batch.state_slots, cu_seqlens=batch.cu_seqlens, seq_lens=batch.seq_lens, num_reqs=B)
        self.proj.forward(x, self.proj_buf, T, scratch=True)
        ops.conv_silu(self.proj_buf, T, x_off=self.x_off, dt_off=self.dt_off, taps=self.conv_taps, bias=self.conv_b,
                      a_log=self.a_log, dt_bias=self.dt_bias, conv_state=cache.conv, work=self.work, **common)
        if cache.owner:
            ops.delta_conv_update(self.proj_buf, qkv_off=self.x_off, conv_state=cache.conv, **common)
        w, inner, gn, H = self.work, self.inner, self.gn, self.heads
        xs, bs, cs = w[:, :inner], w[:, inner:inner + gn], w[:, inner + gn:inner + 2 * gn]
        dt, decay = w[:, self.channels:self.channels + H], w[:, self.channels + H:self.channels + 2 * H]
        ops.decay_recurrence(cs, bs, xs, decay, dt, cache.state, self.y_buf, groups=self.groups, heads=H, dim=self.state,
                             vdim=self.vdim, **common)
        ops.gated_group_norm(self.y_buf, self.proj_buf, 0, self.gated_buf, T, groups=self.norm_groups,
                             group=inner // self.norm_groups, eps=self.norm_eps, weight=self.norm_weight, x=xs,
                             skip=self.skip, vdim=self.vdim)
        return self.o.forward(self.gated_buf, self.out_buf, T, scratch=True)
