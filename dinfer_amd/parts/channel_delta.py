"""Delta rule with a decay and a removal rate of its own for every key channel: a recurrent mixer with one float32
matrix S [dim, dim] a head and request as its state.

With h the mixer's input, H heads of `dim` entries:

    r, k, v = Wr h, Wk h, Wv h                                                        (H x dim each)
    w = exp(-rate * sigmoid(Ww2 tanh(Ww1 h) + w0))        a decay in (exp(-rate), 1)  (H x dim; Ww1 has `low` rows)
    a = sigmoid(Wa h + ab)                                a removal rate              (H x dim)
    u = k / sqrt(sum k^2 + unit_eps)                      the unit key                (per head)
    S <- diag(w) S - (a * u) (u^T S) + k v^T              (both terms read the state before);     o = S^T r
    y = Wo ( concat_h( o_h / rms(o_h) ) * g * sigmoid(Wg h) )                          (g: a gain of H dim entries)

One product makes r | k | v | gate | removal logits | Ww1 h; what follows up to the operand of Wo is float
(csrc/delta.hip). The small product with Ww2 rides in the kernel that prepares the recurrence in steps of few rows;
in steps of many it is a matrix product of its own (tanh in the engine's dtype, the result float32). The state lives in the request's state slot (DeltaStateSpec without a convolution); a request's
first step (position 0) starts from zeros. Prompt portions of any size and single rows run the same recurrence, every
token the same arithmetic in the same order; only the decay's inner product is summed in another order in steps of
many rows.
"""
from __future__ import annotations

import math

import torch

from ..kernels import gemm, ops
from .base import CacheView, Mixer
from .linear import Linear
from .registry import MIXERS
from .spec import DeltaStateSpec, TensorSpec

DEFAULT_RATE = math.exp(-0.5)
# Up to this many rows the product with Ww2 rides in the preparing kernel (a wave a (token, head) reads the head's rows
# of Ww2: two launches fewer); beyond, every wave reading them again costs more than a matrix product (2,048 rows of 32
# heads of 64 with 64 inside: 147 us against 20 for the act and the product)
LOW_IN_KERNEL_ROWS = 64


@MIXERS.register("channel_delta_rule")
class ChannelDeltaRule(Mixer):
    capturable = True            # every kernel reads slots, lengths and row counts from the batch's device buffers
    capturable_portions = True

    NAMES = {"r": "r", "k": "k", "v": "v", "g": "g", "a": "a", "a_bias": "a.b", "w1": "w1", "w2": "w2", "w0": "w0",
             "norm": "norm", "o": "o"}

    def __init__(self, hidden: int, heads: int, dim: int, low: int, norm_eps: float, rate: float = DEFAULT_RATE,
                 unit_eps: float = 1e-6, out_scale: float = 1.0, names: dict | None = None):
        if not (0 < dim <= ops.DELTA_MAX_DIM and 0 < low <= ops.CHANNEL_DELTA_MAX_LOW):
            raise ValueError(f"channel delta rule: dim {dim} or an inner decay size of {low} has no kernel (dim up to "
                             f"{ops.DELTA_MAX_DIM}, inner size up to {ops.CHANNEL_DELTA_MAX_LOW})")
        self.hidden, self.heads, self.dim, self.low = hidden, heads, dim, low
        self.norm_eps, self.rate, self.unit_eps, self.out_scale = float(norm_eps), float(rate), float(unit_eps), float(out_scale)
        self.names = dict(self.NAMES, **(names or {}))
        self.size = heads * dim
        # columns of the fused product: r | k | v | gate | removal logits | inner decay projection, padded to 8
        self.k_off, self.v_off, self.g_off, self.a_off, self.l_off = (i * self.size for i in range(1, 6))
        self.used = self.l_off + low
        self.proj = Linear(hidden, -(-self.used // 8) * 8)
        self.o = Linear(self.size, hidden)

    def cache_spec(self):
        return DeltaStateSpec(self.heads, self.dim, self.dim, 0, 1)

    def tensors(self):
        n, Hd, s = self.names, self.hidden, self.size
        return {n["r"]: TensorSpec((s, Hd)), n["k"]: TensorSpec((s, Hd)), n["v"]: TensorSpec((s, Hd)),
                n["g"]: TensorSpec((s, Hd)), n["a"]: TensorSpec((s, Hd)), n["a_bias"]: TensorSpec((s,), init="zeros"),
                n["w1"]: TensorSpec((self.low, Hd)), n["w2"]: TensorSpec((s, self.low)), n["w0"]: TensorSpec((s,), init="zeros"),
                n["norm"]: TensorSpec((s,), init="gain"), n["o"]: TensorSpec((Hd, s))}

    # ---- the middle part alone, for a mixer that joins several (parts/joined.py) ------------------
    @property
    def in_columns(self) -> int:
        return self.proj.out_features

    @property
    def out_columns(self) -> int:
        return self.size

    def out_weight(self, get) -> torch.Tensor:
        return get(self.names["o"], compute=True)

    def weight_rows(self, get) -> torch.Tensor:
        """The rows of the fused product, in the order of its columns (padding included)."""
        n = self.names
        w = torch.cat([get(n[k], compute=True) for k in ("r", "k", "v", "g", "a", "w1")], dim=0)
        if w.shape[0] < self.proj.out_features:
            w = torch.cat([w, w.new_zeros(self.proj.out_features - w.shape[0], self.hidden)], dim=0)
        return w

    def load_small(self, get) -> None:
        n = self.names
        # small parameters in 32 bits (exact for a bfloat16 file): they enter the recurrence
        self.a_bias = get(n["a_bias"]).float().contiguous()
        self.w2 = get(n["w2"]).float().contiguous()
        self.w2_operand = get(n["w2"], compute=True).contiguous()
        self.w0 = get(n["w0"]).float().contiguous()
        self.norm_weight = get(n["norm"]).float().contiguous()

    def load(self, get):
        self.proj.set_weight(self.weight_rows(get))
        self.load_small(get)
        self.o.set_weight(self.out_weight(get))

    def bind(self, ctx):
        ws = ctx.workspace
        self.proj_buf = ws.buffer("channel_delta_proj", self.proj.out_features)
        self.gated_buf = ws.buffer("channel_delta_gated", self.size)
        self.out_buf = ws.buffer("mixer_out", self.hidden)
        self.bind_core(ctx)

    def bind_core(self, ctx):
        ws = ctx.workspace
        self.work = ws.buffer("channel_delta_work", ops.channel_delta_work_columns(self.heads, self.dim), dtype=torch.float32)
        self.o_buf = ws.buffer("channel_delta_o", self.size, dtype=torch.float32)
        self.tanh_buf = ws.buffer("channel_delta_tanh", self.low)
        self.z_buf = ws.buffer("channel_delta_z", self.size, dtype=torch.float32)

    def forward(self, x, batch, cache: CacheView):
        T = batch.num_tokens
        self.proj.forward(x, self.proj_buf, T, scratch=True)
        self.core(self.proj_buf, 0, self.gated_buf, 0, batch, cache)
        return self.o.forward(self.gated_buf, self.out_buf, T, scratch=True)

    def core(self, proj_buf, col, gated_buf, out_col, batch, cache: CacheView):
        """Everything between the two products: this mixer's columns start at `col` of proj_buf, the operand of the
        output product goes to column `out_col` of gated_buf."""
        T = batch.num_tokens
        if not cache.owner:
            raise NotImplementedError("a recurrent mixer keeps a state a request: an entry that borrows a cache has none")
        z = None
        if T > LOW_IN_KERNEL_ROWS:
            lo = col + self.l_off
            ops.act(proj_buf[:, lo:lo + self.low], self.tanh_buf, T, "tanh")
            z = gemm.matmul_nt(self.tanh_buf, self.w2_operand, self.z_buf, T, may_pad=True)
        ops.channel_delta_prep(proj_buf, T, r_off=col, k_off=col + self.k_off, v_off=col + self.v_off,
                               a_off=col + self.a_off, low_off=col + self.l_off, a_bias=self.a_bias, w2=self.w2,
                               w0=self.w0, work=self.work, heads=self.heads, dim=self.dim, eps=self.unit_eps,
                               rate=self.rate, z=z)
        ops.channel_delta_recurrence(self.work, cache.state, self.o_buf, state_slots=batch.state_slots,
                                     cu_seqlens=batch.cu_seqlens, seq_lens=batch.seq_lens, num_reqs=batch.num_reqs,
                                     heads=self.heads, dim=self.dim)
        ops.delta_out(self.o_buf, proj_buf, col + self.g_off, self.norm_weight, gated_buf, T, heads=self.heads,
                      vdim=self.dim, eps=self.norm_eps, col_off=out_col, out_scale=self.out_scale, gate="sigmoid")
