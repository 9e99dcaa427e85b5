"""Latent attention: keys and values of all heads are made from one latent vector a token, and only that vector and
one rotated key part shared by the heads are cached.

With h the mixer's input, H heads, per head dn unrotated and dr rotated query/key entries, dv value entries, R the
latent size:

    q_h = Wq_h h = [qn_h (dn) | qr_h (dr)]          [c' (R) | kr' (dr)] = Wdkv h
    c = rmsnorm(c') * w                              kr = rot(kr'),  qr_h <- rot(qr_h)
    kn_h = Wuk_h c,   v_h = Wuv_h c
    s_ij = scale * (qn_h,i . kn_h,j + qr_h,i . kr_j),   j <= i  (j > i - window where a window is given)
    y = Wo concat_h( sigmoid(Wg h)_h * sum_j softmax(s)_ij v_h,j )        (the gate only with `gated`)

The cache holds [c | kr] per token (LatentSpec). The products with Wuk and Wuv are done on the query side:
qa_h = Wuk_h^T qn_h, s = scale * <[qa_h | qr_h], [c | kr]>, and the attention's output in latent space is multiplied
by Wuv_h afterwards, so no key or value is ever expanded and prompt portions and single decoded tokens run through
the same kernels. A layer with `shares_cache` has no down projection: it reads the cache of the run entry it is
given (written by a layer whose latent sizes and rotation equal its own) with heads, Wuk and Wuv of its own.

With `q_rank` the queries go through a latent of their own: cq = rmsnorm(Wdq h) * wq (the latent norm's kind and eps),
q = Wuq cq; the first product then makes [cq' | c' | kr'] and a second one the queries (names "dq", "dq.norm", "uq").
The rotation pairs entries (2i, 2i+1) or (i, i + rot/2), as the position encoding says.
"""
from __future__ import annotations

import torch

from ..kernels import latent as latent_kernels
from ..kernels import ops
from .base import CacheView, Mixer
from .linear import Linear
from .registry import MIXERS, NORMS, POSITION_ENCODINGS
from .spec import LatentSpec, PartSpec, TensorSpec


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    capturable = True            # every kernel reads tokens, positions, slots, tables and lengths from the batch's device buffers
    capturable_portions = True   # the choice of kernels follows the step's counts alone

    def __init__(self, hidden: int, heads: int, dim: int, rot_dim: int, vdim: int, rank: int, scale: float,
                 position: PartSpec, latent_norm: PartSpec, gated: bool = True, shares_cache: bool = False,
                 window: int | None = None,
                 names: tuple = ("q", "dkv", "dkv.norm", "uk", "uv", "g", "o"), q_rank: int | None = None,
                 q_names: tuple = ("dq", "dq.norm", "uq")):
        if rank <= 0 or rank > ops.LATENT_MAX_RANK or rank + rot_dim > ops.LATENT_MAX_KEY:
            raise ValueError(f"latent attention: rank {rank} with rot_dim {rot_dim} has no kernel (rank up to "
                             f"{ops.LATENT_MAX_RANK}, rank + rot_dim up to {ops.LATENT_MAX_KEY})")
        self.hidden, self.heads, self.dim, self.rot_dim, self.vdim, self.rank = hidden, heads, dim, rot_dim, vdim, rank
        self.scale, self.gated, self.shares_cache, self.window = float(scale), gated, shares_cache, window
        self.names = dict(zip(("q", "dkv", "norm", "uk", "uv", "g", "o"), names))
        self.q_size = heads * (dim + rot_dim)
        self.q_rank = int(q_rank) if q_rank else 0
        self.q_names = dict(zip(("dq", "norm", "uq"), q_names))
        first = self.q_rank or self.q_size           # what the first product makes of the queries
        self.c_off = None if shares_cache else first
        self.g_off = first + (0 if shares_cache else rank + rot_dim)
        used = self.g_off + (heads if gated else 0)
        self.proj = Linear(hidden, -(-used // 8) * 8)      # q | down projection | gate in one product (rows padded to 8)
        self.used = used
        self.o = Linear(heads * vdim, hidden)
        self.position = POSITION_ENCODINGS.get(position.kind)(head_dim=rot_dim, **position.params)
        if not self.position.fused:
            raise ValueError("latent attention rotates by a table: a position encoding of another kind has no kernel here")
        self.latent_norm = None if shares_cache else NORMS.get(latent_norm.kind)(rank, **latent_norm.params)
        self.q_norm = self.uq = None
        if self.q_rank:
            self.q_norm = NORMS.get(latent_norm.kind)(self.q_rank, **latent_norm.params)
            self.uq = Linear(self.q_rank, self.q_size)
            if self.q_norm.carried() is None or self.q_norm.carried()[1] != 0.0:
                raise ValueError("latent attention norms its query latent by root mean square with a plain gain")
        if self.latent_norm is not None and (self.latent_norm.carried() is None or self.latent_norm.carried()[1] != 0.0):
            raise ValueError("latent attention norms its latent by root mean square with a plain gain")

    def cache_spec(self):
        # (asked after bind: the matrix-core kernel wants the latents a second time, transposed)
        return LatentSpec(self.rank, self.rot_dim, self.window, transposed=self.attn_ws.mfma)

    def tensors(self):
        n, H = self.names, self.heads
        t = {n["uk"]: TensorSpec((H * self.dim, self.rank)),
             n["uv"]: TensorSpec((H * self.vdim, self.rank)),
             n["o"]: TensorSpec((self.hidden, H * self.vdim))}
        if self.q_rank:
            qn = self.q_names
            t[qn["dq"]] = TensorSpec((self.q_rank, self.hidden))
            t[qn["uq"]] = TensorSpec((self.q_size, self.q_rank))
            for name, spec in self.q_norm.tensors().items():
                t[qn["norm"] + name] = spec
        else:
            t[n["q"]] = TensorSpec((self.q_size, self.hidden))
        if not self.shares_cache:
            t[n["dkv"]] = TensorSpec((self.rank + self.rot_dim, self.hidden))
            for name, spec in self.latent_norm.tensors().items():
                t[n["norm"] + name] = spec
        if self.gated:
            t[n["g"]] = TensorSpec((H, self.hidden))
        return t

    def load(self, get):
        n, H = self.names, self.heads
        if self.q_rank:
            qn = self.q_names
            rows = [get(qn["dq"], compute=True)]
            self.q_norm.load(lambda name, **kw: get(qn["norm"] + name, **kw))
            self.uq.set_weight(get(qn["uq"], compute=True))
        else:
            rows = [get(n["q"], compute=True)]
        if not self.shares_cache:
            rows.append(get(n["dkv"], compute=True))
            self.latent_norm.load(lambda name, **kw: get(n["norm"] + name, **kw))
        if self.gated:
            rows.append(get(n["g"], compute=True))
        w = torch.cat(rows, dim=0)
        if w.shape[0] < self.proj.out_features:
            w = torch.cat([w, w.new_zeros(self.proj.out_features - w.shape[0], self.hidden)], dim=0)
        self.proj.set_weight(w)
        # Wuk_h^T [R, dn] per head: the query side of the key expansion; Wuv_h [dv, R] as stored
        self.uk_t = get(n["uk"], compute=True).view(H, self.dim, self.rank).transpose(1, 2).contiguous()
        self.uv = get(n["uv"], compute=True).view(H, self.vdim, self.rank).contiguous()
        self.o.set_weight(get(n["o"], compute=True))

    def bind(self, ctx):
        ws = ctx.workspace
        self.page_size = ctx.page_size
        self.position.bind(ctx)
        H = self.heads
        self.proj_buf = ws.buffer("latent_proj", self.proj.out_features)
        if self.q_rank:
            self.cq_buf = ws.buffer("latent_cq", self.q_rank)
            self.q_buf = ws.buffer("latent_q", self.q_size)
        self.qa_buf = ws.buffer("latent_qa", H * (self.rank + self.rot_dim))
        self.ol_buf = ws.buffer("latent_ol", H * self.rank)
        self.attn_buf = ws.buffer("latent_heads", H * self.vdim)
        self.out_buf = ws.buffer("mixer_out", self.hidden)
        self.attn_ws = latent_kernels.Workspace(ctx, H, self.rank, self.rot_dim)

    def forward(self, x, batch, cache: CacheView):
        T, g = batch.num_tokens, cache.group
        H, dn, dr, R = self.heads, self.dim, self.rot_dim, self.rank
        self.proj.forward(x, self.proj_buf, T, scratch=True)
        write = cache.owner and not self.shares_cache
        gain = self.latent_norm.weight if write else None
        q_src = None
        if self.q_rank:      # the queries' own latent: norm, then the product that makes the queries
            self.q_norm.forward(self.proj_buf[:, :self.q_rank], self.cq_buf, T)
            q_src = self.uq.forward(self.cq_buf, self.q_buf, T, scratch=True)
        ops.latent_post(self.proj_buf, T, heads=H, dim=dn, rot_dim=dr, rank=R, q_off=0, c_off=self.c_off if write else None,
                        gain=gain, eps=self.latent_norm.eps if write else 0.0, positions=batch.positions,
                        cos_sin=self.position.table(), rotary_dim=self.position.rotary_dim, qa=self.qa_buf,
                        cache=cache.latent if write else None, slot_mapping=batch.slot_mapping[g] if write else None,
                        cache_t=cache.tensors.get("latent_t") if write else None, style=self.position.style, q_src=q_src)
        ops.heads_nt(self.proj_buf if q_src is None else q_src, 0, dn + dr, self.uk_t, self.qa_buf, 0, R + dr, T)
        latent_kernels.paged_attention(self.qa_buf, self.ol_buf, cache.latent, cache.tensors.get("latent_t"), batch, g,
                                       self.attn_ws, scale=self.scale,
                                       window=self.window or 0, heads=H, rank=R, rot_dim=dr, page_size=self.page_size)
        ops.heads_nt(self.ol_buf, 0, R, self.uv, self.attn_buf, 0, self.vdim, T,
                     gate=self.proj_buf if self.gated else None, gate_off=self.g_off)
        return self.o.forward(self.attn_buf, self.out_buf, T, scratch=True)
