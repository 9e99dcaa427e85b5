"""Retention: linear attention with a fixed decay a head, no softmax and no denominator.

With h the mixer's input, H heads, p the position:

    q, k = Wq h, Wk h  (H x dim)      v = Wv h  (H x vdim)
    q, k rotated: of the first rot entries of a head, entry i and entry i + rot/2 turn by p base^(-2i/rot)
    k <- k * dim^-1/2
    S <- decay_h S + k v^T;   o = S^T q                          (per head, token by token, S float32 [dim, vdim])
    y = Wo concat_h( o_h / rms(o_h) * act(Wg h)_h )              (no gain on the norm; act silu)

One product makes q | k | v | gate; rotation, scale and everything after them up to the operand of Wo is float
(csrc/decay.hip). The state lives in the request's state slot (DeltaStateSpec without a convolution); a request's first
step (position 0) starts from zeros. Prompt portions of any size and single rows run the same kernels.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import CacheView, Mixer
from .linear import Linear
from .registry import MIXERS, POSITION_ENCODINGS
from .spec import DeltaStateSpec, PartSpec, TensorSpec


@MIXERS.register("retention")
class Retention(Mixer):
    capturable = True            # every kernel reads slots, lengths and row counts from the batch's device buffers
    capturable_portions = True

    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o"}

    def __init__(self, hidden: int, heads: int, dim: int, vdim: int, decay, position: PartSpec, norm_eps: float,
                 out_scale: float = 1.0, names: dict | None = None):
        decay = tuple(float(d) for d in decay)
        if len(decay) != heads or not all(0.0 < d <= 1.0 for d in decay):
            raise ValueError(f"retention: one decay in (0, 1] a head ({heads}), got {decay!r}")
        if not (0 < dim <= ops.DECAY_MAX_DIM and vdim > 0):
            raise ValueError(f"retention: dim {dim} or vdim {vdim} has no kernel (dim up to {ops.DECAY_MAX_DIM})")
        self.hidden, self.heads, self.dim, self.vdim, self.decay = hidden, heads, dim, vdim, decay
        self.norm_eps, self.out_scale = float(norm_eps), float(out_scale)
        self.names = dict(self.NAMES, **(names or {}))
        self.position = POSITION_ENCODINGS.get(position.kind)(head_dim=dim, **position.params)
        if not self.position.fused or self.position.style != 0:
            raise ValueError("retention: takes a rotation by a table with pairs (i, i + rot/2), or none")
        self.qk_size, self.v_size = heads * dim, heads * vdim
        self.g_off = 2 * self.qk_size + self.v_size
        self.proj = Linear(hidden, -(-(self.g_off + self.v_size) // 8) * 8)
        self.o = Linear(self.v_size, hidden)

    def cache_spec(self):
        return DeltaStateSpec(self.heads, self.dim, self.vdim, 0, 1)

    def tensors(self):
        n, Hd = self.names, self.hidden
        return {n["q"]: TensorSpec((self.qk_size, Hd)), n["k"]: TensorSpec((self.qk_size, Hd)),
                n["v"]: TensorSpec((self.v_size, Hd)), n["g"]: TensorSpec((self.v_size, Hd)),
                n["o"]: TensorSpec((Hd, self.v_size))}

    # ---- the middle part alone, for a mixer that joins several (parts/joined.py) ------------------
    @property
    def in_columns(self) -> int:
        return self.proj.out_features

    @property
    def out_columns(self) -> int:
        return self.v_size

    def out_weight(self, get) -> torch.Tensor:
        return get(self.names["o"], compute=True)

    def weight_rows(self, get) -> torch.Tensor:
        n = self.names
        w = torch.cat([get(n[k], compute=True) for k in ("q", "k", "v", "g")], dim=0)
        if w.shape[0] < self.proj.out_features:
            w = torch.cat([w, w.new_zeros(self.proj.out_features - w.shape[0], self.hidden)], dim=0)
        return w

    def load_small(self, get) -> None:
        some = get(self.names["q"], compute=True)
        self.decay_vec = torch.tensor(self.decay, dtype=torch.float32, device=some.device)
        self.position.load(lambda n, **kw: get("position." + n, **kw))

    def load(self, get):
        self.proj.set_weight(self.weight_rows(get))
        self.load_small(get)
        self.o.set_weight(self.out_weight(get))

    def bind(self, ctx):
        ws = ctx.workspace
        self.proj_buf = ws.buffer("retention_proj", self.proj.out_features)
        self.gated_buf = ws.buffer("retention_gated", self.v_size)
        self.out_buf = ws.buffer("mixer_out", self.hidden)
        self.bind_core(ctx)

    def bind_core(self, ctx):
        ws = ctx.workspace
        self.position.bind(ctx)
        self.work = ws.buffer("retention_work", 2 * self.qk_size + self.v_size, dtype=torch.float32)
        self.o_buf = ws.buffer("retention_o", self.v_size, dtype=torch.float32)

    def forward(self, x, batch, cache: CacheView):
        T = batch.num_tokens
        self.proj.forward(x, self.proj_buf, T, scratch=True)
        self.core(self.proj_buf, 0, self.gated_buf, 0, batch, cache)
        return self.o.forward(self.gated_buf, self.out_buf, T, scratch=True)

    def core(self, proj_buf, col, gated_buf, out_col, batch, cache: CacheView):
        """Everything between the two products: this mixer's columns start at `col` of proj_buf, the operand of the
        output product goes to column `out_col` of gated_buf."""
        T, qk = batch.num_tokens, self.qk_size
        pos = self.position
        ops.rot_widen(proj_buf, T, q_off=col, k_off=col + qk, v_off=col + 2 * qk, positions=batch.positions,
                      cos_sin=pos.table(), rotary_dim=pos.rotary_dim, k_scale=self.dim ** -0.5, work=self.work,
                      heads=self.heads, dim=self.dim, vdim=self.vdim)
        w = self.work
        ops.decay_recurrence(w[:, :qk], w[:, qk:2 * qk], w[:, 2 * qk:], self.decay_vec, None, cache.state, self.o_buf,
                             state_slots=batch.state_slots, cu_seqlens=batch.cu_seqlens, seq_lens=batch.seq_lens,
                             num_reqs=batch.num_reqs, groups=self.heads, heads=self.heads, dim=self.dim, vdim=self.vdim)
        ops.gated_group_norm(self.o_buf, proj_buf, col + self.g_off, gated_buf, T, groups=self.heads, group=self.vdim,
                             eps=self.norm_eps, col_off=out_col, out_scale=self.out_scale, gate_first=False)
