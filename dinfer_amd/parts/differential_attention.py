"""Differential attention: every head runs two softmax attentions ("maps") over the same values, and the second,
times one learned number, is taken off the first.

With h the mixer's input, H heads, G key/value heads (head i reads key/value head i // (H / G)), D the size of a
map's queries and keys, V the value size:

    q = Wq h + bq  (H x [map 1 (D) | map 2 (D)])     k = Wk h + bk  (G x [map 1 | map 2])     v = Wv h + bv  (G x V)
    a_m = softmax_j( scale * q_m . k_m,j ) v_j       j <= i, and j > i - window where a window is given   (m = 1, 2)
    lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff  (one number a layer; lq*, lk* are tensors of D entries)
    o = a_1 - lambda a_2;   o <- o / sqrt(mean(o^2) + eps) * (1 - diff)         (the mean over a head's V values)
    y = Wo concat_h(o_h)

No positions enter the scores. The cache holds, a token and key/value head, the two keys side by side (a key head of
2 D entries in the key pages) and the value. The plain kernel walks the keys once for both maps
(csrc/attention_ref.hip); prompt portions and single rows run the same kernel.

On the matrix cores (bfloat16, V = 2 D, sizes the flash kernel takes): a map is a query head of its own, 2 D wide, whose
other map's half is zero, [q_1 | 0] and [0 | q_2]; against the key head [k_1 | k_2] it scores q_m . k_m, and the 2 H
such heads over G key/value heads are grouped-query attention as the flash kernel with options runs it (the zeros come
out of the projection: the rows of Wq and bq are spread at bind). A small kernel then takes lambda times the second
map off the first and norms (csrc/attention_ref.hip, diff_combine). The products with the zeros are a third more
arithmetic than the maps need and run an order of magnitude faster than the plain kernel's.
"""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from .base import CacheView, Mixer
from .linear import Linear
from .registry import MIXERS
from .spec import KVSpec, TensorSpec


@MIXERS.register("differential_attention")
class DifferentialAttention(Mixer):
    capturable = True            # every kernel reads tokens, positions, slots, tables and lengths from the batch's device buffers
    capturable_portions = True   # one kernel for every step

    NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
             "lq1": "lq1", "lk1": "lk1", "lq2": "lq2", "lk2": "lk2"}

    def __init__(self, hidden: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, diff: float,
                 norm_eps: float, window: int | None = None, bias: bool = True, names: dict | None = None):
        if heads % kv_heads:
            raise ValueError(f"heads {heads} not divisible by kv_heads {kv_heads}")
        if not (0 < 2 * dim <= ops.MAX_HEAD_DIM and 0 < vdim <= ops.MAX_HEAD_DIM):
            raise ValueError(f"differential attention: dim {dim} or vdim {vdim} has no kernel (2 dim and vdim up to "
                             f"{ops.MAX_HEAD_DIM})")
        self.hidden, self.heads, self.kv_heads, self.dim, self.vdim = hidden, heads, kv_heads, dim, vdim
        self.scale, self.diff, self.norm_eps, self.window, self.bias = float(scale), float(diff), float(norm_eps), window, bool(bias)
        self.names = dict(self.NAMES, **(names or {}))
        self.q_size, self.k_size, self.v_size = heads * 2 * dim, kv_heads * 2 * dim, kv_heads * vdim
        self.qkv = Linear(hidden, self.q_size + self.k_size + self.v_size)
        self.o = Linear(heads * vdim, hidden)
        self.bias_vec = None
        self.lam = 0.0
        self.mfma = False      # decided in bind

    def cache_spec(self):
        return KVSpec(self.kv_heads, 2 * self.dim, self.window, v_dim=self.vdim)

    def tensors(self):
        n, Hd = self.names, self.hidden
        t = {n["q"]: TensorSpec((self.q_size, Hd)), n["k"]: TensorSpec((self.k_size, Hd)),
             n["v"]: TensorSpec((self.v_size, Hd)), n["o"]: TensorSpec((Hd, self.heads * self.vdim))}
        if self.bias:
            t[n["q_bias"]] = TensorSpec((self.q_size,), init="zeros")
            t[n["k_bias"]] = TensorSpec((self.k_size,), init="zeros")
            t[n["v_bias"]] = TensorSpec((self.v_size,), init="zeros")
        for k in ("lq1", "lk1", "lq2", "lk2"):
            t[n[k]] = TensorSpec((self.dim,))
        return t

    def _spread(self, q: torch.Tensor) -> torch.Tensor:
        """Rows (or entries) of the queries [H, 2, D, ...] -> [H, 2, 2 D, ...]: map m keeps its place in a head of 2 D,
        the other map's half is zero."""
        H, D = self.heads, self.dim
        q = q.view(H, 2, D, *q.shape[1:])
        out = q.new_zeros((H, 2, 2 * D, *q.shape[3:]))
        out[:, 0, :D] = q[:, 0]
        out[:, 1, D:] = q[:, 1]
        return out.view(H * 4 * D, *q.shape[3:])

    def load(self, get):
        n = self.names
        self.qkv.set_weight(torch.cat([get(n[k], compute=True) for k in ("q", "k", "v")], dim=0))
        self.o.set_weight(get(n["o"], compute=True))
        if self.bias:     # small parameters in 32 bits (exact for a bfloat16 file): q heads | k heads | v heads
            self.bias_vec = torch.cat([get(n[k]).float() for k in ("q_bias", "k_bias", "v_bias")]).contiguous()
        l = {k: get(n[k]).double().cpu() for k in ("lq1", "lk1", "lq2", "lk2")}     # one number a layer, made once
        self.lam = math.exp(float((l["lq1"] * l["lk1"]).sum())) - math.exp(float((l["lq2"] * l["lk2"]).sum())) + self.diff

    def bind(self, ctx):
        ws = ctx.workspace
        self.page_size = ctx.page_size
        self.mfma = bool(ctx.dtype == torch.bfloat16 and self.vdim == 2 * self.dim
                         and ops.attn_mfma_supports(2 * self.dim, ctx.page_size, 2 * self.heads, self.kv_heads))
        if self.mfma and self.qkv.out_features == self.q_size + self.k_size + self.v_size:
            # every map a query head of its own (see the top): the projection makes the zeros
            w, q = self.qkv.weight, self.q_size
            self.qkv = Linear(self.hidden, 2 * q + self.k_size + self.v_size)
            self.qkv.set_weight(torch.cat([self._spread(w[:q]), w[q:]], dim=0))
            if self.bias_vec is not None:
                self.bias_vec = torch.cat([self._spread(self.bias_vec[:q]), self.bias_vec[q:]]).contiguous()
            self.pair_buf = ws.buffer("diff_pairs", 2 * self.heads * self.vdim)
        self.qkv_buf = ws.buffer("qkv", self.qkv.out_features)
        self.attn_buf = ws.buffer("attn", self.heads * self.vdim)
        self.out_buf = ws.buffer("mixer_out", self.hidden)

    def forward(self, x, batch, cache: CacheView):
        T, g = batch.num_tokens, cache.group
        D2 = 2 * self.dim
        heads = 2 * self.heads if self.mfma else self.heads       # on the matrix cores a map is a head
        q_size = heads * D2
        self.qkv.forward(x, self.qkv_buf, T, scratch=True)
        # biases, and the keys and values into their pages: no norm, no rotation
        ops.qkv_post(self.qkv_buf, T, heads=heads, kv_heads=self.kv_heads, head_dim=D2, q_off=0, k_off=q_size,
                     v_off=q_size + self.k_size, positions=batch.positions, page_size=self.page_size, q_gain=None,
                     k_gain=None, eps=0.0, gain_offset=0.0, cos_sin=None, rotary_dim=0, rope_style=0, k_cache=cache.k,
                     v_cache=cache.v, slot_mapping=batch.slot_mapping[g] if cache.owner else None, token_runs=False,
                     v_dim=self.vdim, bias=self.bias_vec)
        if self.mfma:
            ops.attn_flash_ext(self.qkv_buf, self.pair_buf, cache.k, cache.v, batch.block_table[g], batch.cu_seqlens,
                               batch.seq_lens, batch.num_reqs, batch.max_q_len, scale=self.scale, window=self.window or 0,
                               heads=heads, kv_heads=self.kv_heads, head_dim=D2, page_size=self.page_size, keep_first=0,
                               sinks=None, slope_exp=0.0, out_scale=1.0)
            ops.diff_combine(self.pair_buf, self.attn_buf, T, heads=self.heads, v_dim=self.vdim, lam=self.lam,
                             eps=self.norm_eps, post=1.0 - self.diff)
            return self.o.forward(self.attn_buf, self.out_buf, T, scratch=True)
        ops.attn_paged_diff(self.qkv_buf, self.attn_buf, cache.k, cache.v, batch.block_table[g], batch.cu_seqlens,
                            batch.seq_lens, batch.num_reqs, T, scale=self.scale, window=self.window or 0,
                            heads=self.heads, kv_heads=self.kv_heads, head_dim=self.dim, v_dim=self.vdim,
                            page_size=self.page_size, lam=self.lam, eps=self.norm_eps, post=1.0 - self.diff)
        return self.o.forward(self.attn_buf, self.out_buf, T, scratch=True)
