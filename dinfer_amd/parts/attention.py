"""Grouped-query attention over the paged cache, with optional per-head q/k
norm, a position encoding and an optional sliding window.

Order of operations (models/qwen3/src/model.rs:199-315): fused q|k|v projection ->
per-head norm of q and k -> rotation -> k, v into the cache pages -> causal
attention over the pages (scale given, default head_dim^-0.5) -> output projection.

Options, each a constructor parameter that is off by default: values of a size of their own (`v_dim`); the first
`keep_first` keys staying visible behind the window; a learned sink a head in the softmax's denominator (`sink`, a
tensor [heads]); a bias that takes 2^(-slope_exp (h + 1) / heads) times the distance off the scores (`slope_exp`);
values that are the keys (`values_are_keys`: no value projection, no value pages); the output multiplied by
`out_scale`; tensor names (`names`). Further: biases on the q, k and v projections (`bias`); q and k divided by their
root mean square a head without a gain (`qk_unit_eps`); a query that grows with its position, times
1 + coef ln(floor((p + 1) / every) + 1) (`q_temp = (coef, every)`); a sink of a fixed score instead of a learned one
(`sink_value`: 0.0 adds one to the softmax's denominator); the concatenated heads multiplied by an activation of one
more projection of the mixer's input before the output projection (`gate`: "sigmoid" or "silu"; with `gate_heads` the
projection gives one number a head, which multiplies all of the head's values); a learned temperature a head that
multiplies the head's scores (`head_temp`, a tensor [heads]; it rides on the query, in the per-head norm). A layer that uses any
option runs the flash kernel with options on the matrix cores where its sizes allow, else the plain kernel with options
(csrc/attention_ref.hip), for prompt portions and single rows alike; the matrix-core kernels serve the others.
"""
from __future__ import annotations

import torch

from ..kernels import attention as attn_kernels
from ..kernels import ops
from .base import CacheView, Mixer
from .linear import Linear
from .registry import MIXERS, NORMS, POSITION_ENCODINGS
from .spec import KVSpec, PartSpec, TensorSpec


@MIXERS.register("attention")
class Attention(Mixer):
    carries_norms = True   # the q/k/v product takes a Carried, the output product an Into
    capturable = True      # every kernel reads tokens, positions, slots, tables and lengths from the batch's device buffers
    capturable_portions = True   # the choice of kernels follows the step's counts alone

    NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
             "q_norm": "q_norm.", "k_norm": "k_norm.", "sink": "sinks", "q_bias": "q_proj.bias", "k_bias": "k_proj.bias",
             "v_bias": "v_proj.bias", "g": "g_proj.weight", "temp": "temp"}

    def __init__(self, hidden: int, heads: int, kv_heads: int, head_dim: int, position: PartSpec,
                 qk_norm: PartSpec | None = None, window: int | None = None, scale: float | None = None,
                 v_dim: int | None = None, keep_first: int = 0, sink: bool = False, slope_exp: float = 0.0,
                 values_are_keys: bool = False, out_scale: float = 1.0, names: dict | None = None, bias: bool = False,
                 qk_unit_eps: float | None = None, q_temp: tuple | None = None, sink_value: float | None = None,
                 gate: str | None = None, gate_heads: bool = False, head_temp: bool = False):
        if heads % kv_heads:
            raise ValueError(f"heads {heads} not divisible by kv_heads {kv_heads}")
        if head_dim <= 0 or head_dim > ops.MAX_HEAD_DIM:   # said at build, not at the first step
            raise ValueError(f"attention: head_dim {head_dim} has no kernel (up to {ops.MAX_HEAD_DIM})")
        self.hidden, self.heads, self.kv_heads, self.head_dim = hidden, heads, kv_heads, head_dim
        self.window = window
        self.scale = float(scale) if scale is not None else head_dim ** -0.5
        self.v_dim = head_dim if v_dim is None else int(v_dim)
        self.keep_first, self.sink, self.slope_exp = int(keep_first), bool(sink), float(slope_exp)
        self.values_are_keys, self.out_scale = bool(values_are_keys), float(out_scale)
        if self.values_are_keys and self.v_dim != head_dim:
            raise ValueError("attention: values that are the keys have the keys' size")
        if self.keep_first < 0 or self.v_dim <= 0 or self.v_dim > ops.MAX_HEAD_DIM:
            raise ValueError(f"attention: keep_first {keep_first} or v_dim {v_dim} out of range")
        if self.keep_first and not window:
            self.keep_first = 0     # without a window every key stays visible anyway
        self.names = dict(self.NAMES, **(names or {}))
        self.bias, self.qk_unit_eps, self.gate = bool(bias), qk_unit_eps, gate
        self.q_temp = None if q_temp is None else (float(q_temp[0]), int(q_temp[1]))
        self.sink_value = None if sink_value is None else float(sink_value)
        if self.sink and self.sink_value is not None:
            raise ValueError("attention: a sink is learned (`sink`) or of a fixed score (`sink_value`), not both")
        if qk_unit_eps is not None and qk_norm is not None:
            raise ValueError("attention: q and k are normed with gains (`qk_norm`) or without (`qk_unit_eps`), not both")
        if self.q_temp is not None and (self.q_temp[1] <= 0 or (qk_norm is None and qk_unit_eps is None)):
            raise ValueError("attention: a query temperature needs every > 0 and a per-head norm of q (it rides in it)")
        if gate is not None and gate not in ("sigmoid", "silu"):
            raise ValueError(f"attention: gate {gate!r} unknown (known: 'sigmoid', 'silu')")
        self.gate_heads, self.head_temp = bool(gate_heads) and gate is not None, bool(head_temp)
        if self.head_temp and qk_norm is None and qk_unit_eps is None:
            raise ValueError("attention: a temperature a head needs a per-head norm of q (it rides in it)")
        if self.bias and self.values_are_keys:
            raise ValueError("attention: biases with values that are the keys are not built")
        # what the matrix-core kernels do not do runs through the plain kernel with options
        self.extended = bool(self.v_dim != head_dim or self.keep_first or self.sink or self.slope_exp
                             or self.values_are_keys or self.out_scale != 1.0 or self.bias or qk_unit_eps is not None
                             or self.q_temp is not None or self.sink_value is not None or gate is not None
                             or self.head_temp)
        self.q_size, self.kv_size = heads * head_dim, kv_heads * head_dim
        self.v_size = 0 if self.values_are_keys else kv_heads * self.v_dim
        self.g_size = (heads if self.gate_heads else heads * self.v_dim) if gate is not None else 0
        self.temps = None
        self.g_off = self.q_size + self.kv_size + self.v_size
        self.qkv = Linear(hidden, self.q_size + self.kv_size + self.v_size + self.g_size)
        self.bias_vec = self.unit_gain = None
        self.o = Linear(heads * self.v_dim, hidden)
        self.sinks = None
        # decided in bind: the matrix-core flash kernel with options serves bfloat16 layers whose values have the keys'
        # size; it reads values from transposed pages, so a layer whose values are its keys keeps them there as well
        self.mfma_ext = False
        self.stores_values = not self.values_are_keys
        self.position = POSITION_ENCODINGS.get(position.kind)(head_dim=head_dim, **position.params)
        self.q_norm = self.k_norm = None
        if qk_norm is not None:
            cls = NORMS.get(qk_norm.kind)
            self.q_norm, self.k_norm = cls(head_dim, **qk_norm.params), cls(head_dim, **qk_norm.params)

    def cache_spec(self):
        # (asked after bind, which settles whether values that are the keys are stored a second time)
        return KVSpec(self.kv_heads, self.head_dim, self.window, v_dim=self.v_dim, keep_first=self.keep_first,
                      values=self.stores_values)

    def tensors(self):
        D, Hd, nm = self.head_dim, self.hidden, self.names
        t = {
            nm["q"]: TensorSpec((self.q_size, Hd)),
            nm["k"]: TensorSpec((self.kv_size, Hd)),
            nm["o"]: TensorSpec((Hd, self.heads * self.v_dim)),
        }
        if not self.values_are_keys:
            t[nm["v"]] = TensorSpec((self.v_size, Hd))
        if self.q_norm is not None:
            for which, norm in (("q_norm", self.q_norm), ("k_norm", self.k_norm)):
                for n, spec in norm.tensors().items():
                    t[nm[which] + n] = spec
        if self.sink:
            t[nm["sink"]] = TensorSpec((self.heads,))
        if self.bias:
            t[nm["q_bias"]] = TensorSpec((self.q_size,), init="zeros")
            t[nm["k_bias"]] = TensorSpec((self.kv_size,), init="zeros")
            t[nm["v_bias"]] = TensorSpec((self.v_size,), init="zeros")
        if self.gate is not None:
            t[nm["g"]] = TensorSpec((self.g_size, Hd))
        if self.head_temp:
            t[nm["temp"]] = TensorSpec((self.heads,), init="gain")
        for n, spec in self.position.tensors().items():   # an encoding with parameters of its own (rotations have none)
            t["position." + n] = spec
        return t

    # ---- the middle part alone, for a mixer that joins several (parts/joined.py) ------------------
    @property
    def in_columns(self) -> int:
        return self.q_size + self.kv_size + self.v_size + self.g_size

    @property
    def out_columns(self) -> int:
        return self.heads * self.v_dim

    def weight_rows(self, get) -> torch.Tensor:
        # q, k, v rows concatenated into one [(H + 2 Hkv) D, hidden] operand (model.rs:141-165)
        nm = self.names
        rows = [get(nm["q"], compute=True), get(nm["k"], compute=True)]
        if not self.values_are_keys:
            rows.append(get(nm["v"], compute=True))
        if self.gate is not None:
            rows.append(get(nm["g"], compute=True))
        return torch.cat(rows, dim=0)

    def out_weight(self, get) -> torch.Tensor:
        return get(self.names["o"], compute=True)

    def load(self, get):
        self.qkv.set_weight(self.weight_rows(get))
        self.o.set_weight(self.out_weight(get))
        self.load_small(get)

    def load_small(self, get):
        nm = self.names
        if self.q_norm is not None:
            self.q_norm.load(lambda n, **kw: get(nm["q_norm"] + n, **kw))
            self.k_norm.load(lambda n, **kw: get(nm["k_norm"] + n, **kw))
        if self.sink:
            self.sinks = get(nm["sink"]).float().contiguous()
        some = get(nm["q"], compute=True)
        if self.sink_value is not None:
            self.sinks = torch.full((self.heads,), self.sink_value, dtype=torch.float32, device=some.device)
        if self.bias:     # small parameters in 32 bits (exact for a bfloat16 file): q heads | k heads | v heads
            self.bias_vec = torch.cat([get(nm[k]).float() for k in ("q_bias", "k_bias", "v_bias")]).contiguous()
        if self.head_temp:
            self.temps = get(nm["temp"]).float().contiguous()
        if self.qk_unit_eps is not None:
            self.unit_gain = torch.ones(self.head_dim, dtype=torch.float32, device=some.device)
        self.position.load(lambda n, **kw: get("position." + n, **kw))

    def bind_core(self, ctx):
        self.page_size = ctx.page_size
        self.position.bind(ctx)
        self.mfma_ext = bool(ctx.dtype == torch.bfloat16 and self.v_dim == self.head_dim
                             and ops.attn_mfma_supports(self.head_dim, ctx.page_size, self.heads, self.kv_heads))
        self.stores_values = not self.values_are_keys or self.mfma_ext

    def bind(self, ctx):
        ws = ctx.workspace
        self.bind_core(ctx)
        self.qkv_buf = ws.buffer("qkv", self.qkv.out_features)
        self.attn_buf = ws.buffer("attn", self.heads * self.v_dim)
        self.out_buf = ws.buffer("mixer_out", self.hidden)
        self.attn_ws = attn_kernels.Workspace(ctx, self.heads, self.kv_heads, self.head_dim)

    def forward(self, x, batch, cache: CacheView, into=None):
        T = batch.num_tokens
        g = cache.group
        self.qkv.forward(x, self.qkv_buf, T, scratch=True)
        self.core(self.qkv_buf, 0, self.attn_buf, 0, batch, cache)
        return self._project_out(T, into)

    def core(self, qkv_buf, col, attn_buf, out_col, batch, cache: CacheView):
        """Everything between the two products: q | k | v are read from column `col` of qkv_buf on, the heads'
        outputs go to column `out_col` of attn_buf (a mixer that joins several shares one product on each side)."""
        T = batch.num_tokens
        g = cache.group
        if self.extended or col or out_col:
            return self._core_ext(qkv_buf, col, attn_buf, out_col, batch, cache)
        qn, pos = self.q_norm, self.position
        geometry = dict(heads=self.heads, kv_heads=self.kv_heads, head_dim=self.head_dim, q_off=0, k_off=self.q_size,
                        v_off=self.q_size + self.kv_size, positions=batch.positions, page_size=self.page_size)
        norm = dict(q_gain=qn.weight if qn else None, k_gain=self.k_norm.weight if qn else None,
                    eps=qn.eps if qn else 0.0, gain_offset=qn.weight_offset if qn else 0.0)
        no_norm = dict(q_gain=None, k_gain=None, eps=0.0, gain_offset=0.0)
        write = dict(k_cache=cache.k, v_cache=cache.v, slot_mapping=batch.slot_mapping[g] if cache.owner else None,
                     token_runs=batch.max_q_len >= 8)
        if (pos.fused and batch.all_decode and self.attn_ws.decode_takes_post and pos.style == 0
                and pos.rotary_dim == self.head_dim and (qn is None or qn.weight.dtype == torch.bfloat16)):
            # only single rows: norm, rotation and cache write ride in the attention kernel, one launch fewer a layer
            attn_kernels.decode_with_post(
                self.qkv_buf, self.attn_buf, cache.k, cache.v, batch, g, self.attn_ws, write=cache.owner,
                scale=self.scale, window=self.window or 0, heads=self.heads, kv_heads=self.kv_heads,
                head_dim=self.head_dim, page_size=self.page_size, q_off=0, k_off=self.q_size,
                v_off=self.q_size + self.kv_size, positions=batch.positions, cos_sin=pos.table(), **norm)
            return
        if pos.fused:
            # per-head norm, rotation by the encoding's table and the cache write in one kernel
            ops.qkv_post(self.qkv_buf, T, **geometry, **norm, cos_sin=pos.table(), rotary_dim=pos.rotary_dim,
                         rope_style=pos.style, **write)
        else:
            # an encoding that is no rotation by a table works on q and k itself, between the norm and the cache write
            if qn:
                ops.qkv_post(self.qkv_buf, T, **geometry, **norm, cos_sin=None, rotary_dim=0, rope_style=0, k_cache=None,
                             v_cache=None, slot_mapping=None, token_runs=False)
            q = self.qkv_buf[:T, :self.q_size].view(T, self.heads, self.head_dim)
            k = self.qkv_buf[:T, self.q_size:self.q_size + self.kv_size].view(T, self.kv_heads, self.head_dim)
            pos.transform(q, k, batch.positions[:T])
            if cache.owner:
                ops.qkv_post(self.qkv_buf, T, **geometry, **no_norm, cos_sin=None, rotary_dim=0, rope_style=0, **write)
        attn_kernels.paged_attention(
            self.qkv_buf, self.attn_buf, cache.k, cache.v, batch, g, self.attn_ws, scale=self.scale,
            window=self.window or 0, heads=self.heads, kv_heads=self.kv_heads, head_dim=self.head_dim,
            page_size=self.page_size)

    def _core_ext(self, qkv_buf, col, attn_buf, out_col, batch, cache: CacheView):
        """Per-head norm, rotation and cache write, then the flash kernel with this layer's options on the matrix
        cores, or the plain kernel with them (32-bit, sizes the matrix-core kernel does not take)."""
        T, g = batch.num_tokens, cache.group
        qn, pos = self.q_norm, self.position
        if not pos.fused:
            raise NotImplementedError("attention with options takes a rotation by a table, or none")
        vd = self.v_dim
        q_gain, k_gain = (qn.weight, self.k_norm.weight) if qn else (self.unit_gain, self.unit_gain)
        eps = qn.eps if qn else (self.qk_unit_eps or 0.0)
        ops.qkv_post(qkv_buf, T, heads=self.heads, kv_heads=self.kv_heads, head_dim=self.head_dim, q_off=col,
                     k_off=col + self.q_size,     # (values that are the keys: the key columns as the product left them)
                     v_off=col + self.q_size + (0 if self.values_are_keys else self.kv_size),
                     positions=batch.positions, page_size=self.page_size,
                     q_gain=q_gain, k_gain=k_gain, eps=eps, gain_offset=qn.weight_offset if qn else 0.0,
                     cos_sin=pos.table(), rotary_dim=pos.rotary_dim, rope_style=pos.style,
                     k_cache=cache.k, v_cache=cache.v, slot_mapping=batch.slot_mapping[g] if cache.owner else None,
                     token_runs=False, v_dim=vd, bias=self.bias_vec, q_temp=self.q_temp, q_head_scale=self.temps)
        self._attend_ext(qkv_buf, col, attn_buf, out_col, batch, cache)
        if self.gate is not None:
            n = self.heads * vd
            ops.gate(attn_buf[:, out_col:out_col + n], qkv_buf[:, col + self.g_off:col + self.g_off + self.g_size], T,
                     self.gate, group=vd if self.gate_heads else 1)

    def _attend_ext(self, qkv_buf, col, attn_buf, out_col, batch, cache: CacheView):
        T, g, vd = batch.num_tokens, cache.group, self.v_dim
        if self.mfma_ext:
            ops.attn_flash_ext(qkv_buf[:, col:], attn_buf[:, out_col:], cache.k, cache.v, batch.block_table[g],
                               batch.cu_seqlens, batch.seq_lens, batch.num_reqs, batch.max_q_len, scale=self.scale,
                               window=self.window or 0, heads=self.heads, kv_heads=self.kv_heads, head_dim=self.head_dim,
                               page_size=self.page_size, keep_first=self.keep_first, sinks=self.sinks,
                               slope_exp=self.slope_exp, out_scale=self.out_scale)
            return
        ops.attn_paged_ext(qkv_buf[:, col:], attn_buf[:, out_col:], cache.k, cache.v, batch.block_table[g],
                           batch.cu_seqlens, batch.seq_lens, batch.num_reqs, T, scale=self.scale,
                           window=self.window or 0, heads=self.heads, kv_heads=self.kv_heads, head_dim=self.head_dim,
                           page_size=self.page_size, v_dim=vd, keep_first=self.keep_first, sinks=self.sinks,
                           slope_exp=self.slope_exp, out_scale=self.out_scale)

    def _project_out(self, T, into):
        if into is not None:
            done = self.o.forward_into(self.attn_buf, into, T)
            if done is not None:
                return done
        return self.o.forward(self.attn_buf, self.out_buf, T, scratch=True)
