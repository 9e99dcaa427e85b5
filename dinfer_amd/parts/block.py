"""Block arrangements.

"prenorm":  h += mixer(norm_in(h));  h += ff(norm_post(h))
(models/qwen3/src/model.rs:708-813). The feed-forward's add is deferred into the
next block's input norm kernel, and the mixer's add into this block's second
norm kernel, so each add costs no pass of its own (model.rs:700-701,722-731,772-781).
In steps of a few tokens the norms have no kernel at all: the product before a norm adds
into the stream and leaves what the norm needs, the product after it applies it (Carried).
In steps of many tokens the product before a norm adds into the stream as well (the library's
beta = 1), and the norm's kernel reads the stream alone.
"""
from __future__ import annotations

import torch

from ..kernels import gemm, ops
from .base import Block, CacheView, Carried, Into
from .registry import BLOCKS, FEED_FORWARDS, MIXERS, NORMS
from .spec import LayerSpec

# A norm is carried by the products around it in steps of up to this many tokens (one token tile of the few-row
# kernel). Measured at the 8B sizes: a step of 1 token 3.82 -> 3.68 ms, of 8 4.07 -> 4.00, of 16 4.65 -> 4.62; at 32
# tokens (two token tiles) the longer ends of four kernels cost more than the two norm kernels did (5.93 -> 6.11 ms);
# carrying only the norm after the mixer there (the down projection has another kernel at those rows) 5.39 -> 5.44 ms,
# and with the kernel for wide weights as the gate/up product that applies it 5.22 -> 5.28 (4.88 -> 4.92 at 24 tokens).
CARRY_ROWS = 16


def _sub(get, prefix):
    return lambda name, **kw: get(prefix + name, **kw)


@BLOCKS.register("prenorm")
class PreNormBlock(Block):
    """params: mixer_prefix, ff_prefix, norm_in_name, norm_post_name (weight-name pieces)."""
    carries_norms = True

    def __init__(self, hidden: int, layer: LayerSpec, mixer_prefix: str = "self_attn.", ff_prefix: str = "mlp.",
                 norm_in: str = "input_layernorm.", norm_post: str = "post_attention_layernorm."):
        self.hidden = hidden
        self.prefixes = (mixer_prefix, ff_prefix, norm_in, norm_post)
        self.mixer = MIXERS.get(layer.mixer.kind)(hidden=hidden, **layer.mixer.params)
        self.ff = FEED_FORWARDS.get(layer.feed_forward.kind)(hidden=hidden, **layer.feed_forward.params)
        ncls = NORMS.get(layer.norm.kind)
        self.norm_in, self.norm_post = ncls(hidden, **layer.norm.params), ncls(hidden, **layer.norm.params)
        if getattr(self.ff, "absent", False):      # a layer that is its mixer alone: h += mixer(norm_in(h))
            self.ff = self.norm_post = None

    def _parts(self):
        return [(p, part) for p, part in zip(self.prefixes, (self.mixer, self.ff, self.norm_in, self.norm_post))
                if part is not None]

    @property
    def capturable(self):
        return all(part.capturable for _, part in self._parts())

    @property
    def capturable_portions(self):
        return all(part.capturable and part.capturable_portions for _, part in self._parts())

    def tensors(self):
        return {p + n: s for p, part in self._parts() for n, s in part.tensors().items()}

    def load(self, get):
        for p, part in self._parts():
            part.load(_sub(get, p))

    def bind(self, ctx):
        for _, part in self._parts():
            part.bind(ctx)
        ws = ctx.workspace
        self.normed = ws.buffer("normed", self.hidden)
        # for norms carried by the products around them (steps of up to CARRY_ROWS tokens)
        self.xg = ws.buffer("carried_xg", self.hidden, rows=CARRY_ROWS)
        self.stats = ws.buffer("carried_stats", -(-self.hidden // gemm.STATS_COLUMNS), dtype=torch.float32,
                               rows=CARRY_ROWS)

    def input_norm(self):
        return self.norm_in if self.mixer.carries_norms else None

    def _into(self, hidden, norm, part, T):
        if norm is None or not part.carries_norms:
            return {}
        return {"into": Into(hidden, norm, self.xg, self.stats, self.normed)}

    def forward(self, hidden, pending, batch, cache: CacheView, next_norm=None):
        T = batch.num_tokens
        if isinstance(pending, Carried):
            x = pending if self.mixer.carries_norms else pending.materialise()
        elif pending is None:
            x = self.norm_in.forward(hidden, self.normed, T)
        else:
            x = self.norm_in.forward(pending, self.normed, T, residual=hidden)
        if self.ff is None:
            return self.mixer.forward(x, batch, cache, **self._into(hidden, next_norm, self.mixer, T))
        a = self.mixer.forward(x, batch, cache, **self._into(hidden, self.norm_post, self.mixer, T))
        if isinstance(a, Carried):
            x = a if self.ff.carries_norms else a.materialise()
        else:
            x = self.norm_post.forward(a, self.normed, T, residual=hidden)
        return self.ff.forward(x, batch, **self._into(hidden, next_norm, self.ff, T))


@BLOCKS.register("sandwich")
class SandwichBlock(Block):
    """A norm before and after each sublayer, and a multiplier on what is added:

        h += mult * norm_a_out(mixer(norm_a(h)));   h += mult * norm_b_out(ff(norm_b(h)))

    One kernel a sublayer's end norms the branch, adds it into the stream (in the stream's own dtype, 32 bits where
    the model says so) and norms the stream for what reads it next: this block's feed-forward, or the next block's
    mixer (handed over as a Carried that is ready). params: mult, mixer_prefix, ff_prefix and the four norms' names.
    All four norms are of the layer's norm kind, which must be a root-mean-square norm (`carried()` gives its gain).

    shift (a tensor's name, [hidden]): token shift. What the mixer reads, x = norm_a(h), becomes x + (x' - x) * shift,
    x' the x of the token before in its request as the norm gave it (zeros before the first token). The last x of a
    request is state of its own, one row a request and run entry, kept beside the mixer's cache: the entry's cache
    is then the mixer's under "mixer" joined with that row under "shift"."""
    carries_norms = True

    def __init__(self, hidden: int, layer: LayerSpec, mult: float = 1.0, mixer_prefix: str = "mix.", ff_prefix: str = "mlp.",
                 norm_a: str = "norm1", norm_a_out: str = "norm1b", norm_b: str = "norm2", norm_b_out: str = "norm2b",
                 shift: str | None = None):
        self.hidden, self.mult = hidden, float(mult)
        self.shift_name, self.shift = shift, None
        self.mixer = MIXERS.get(layer.mixer.kind)(hidden=hidden, **layer.mixer.params)
        self.ff = FEED_FORWARDS.get(layer.feed_forward.kind)(hidden=hidden, **layer.feed_forward.params)
        if getattr(self.ff, "absent", False):
            self.ff = None
        ncls = NORMS.get(layer.norm.kind)
        names = [norm_a, norm_a_out] + ([norm_b, norm_b_out] if self.ff is not None else [])
        self.norms = [(n, ncls(hidden, **layer.norm.params)) for n in names]
        if any(n.carried() is None for _, n in self.norms):
            raise ValueError("the sandwich arrangement takes root-mean-square norms")
        self.prefixes = (mixer_prefix, ff_prefix)

    def _parts(self):
        out = [(self.prefixes[0], self.mixer)] + list(self.norms)
        if self.ff is not None:
            out.append((self.prefixes[1], self.ff))
        return out

    @property
    def capturable(self):
        return all(part.capturable for _, part in self._parts())

    @property
    def capturable_portions(self):
        return all(part.capturable and part.capturable_portions for _, part in self._parts())

    def tensors(self):
        t = {p + n: s for p, part in self._parts() for n, s in part.tensors().items()}
        if self.shift_name is not None:
            from .spec import TensorSpec
            t[self.shift_name] = TensorSpec((self.hidden,), init="shares")
        return t

    def load(self, get):
        for p, part in self._parts():
            part.load(_sub(get, p))
        for _, n in self.norms:
            n.weight = n.weight.float().contiguous()     # (exact for a bfloat16 file) one type for all gains of a kernel
        if self.shift_name is not None:
            self.shift = get(self.shift_name).float().contiguous()

    def bind(self, ctx):
        for _, part in self._parts():
            part.bind(ctx)
        self.normed = ctx.workspace.buffer("normed", self.hidden)
        if self.shift_name is not None:
            self.shifted = ctx.workspace.buffer("shifted", self.hidden)

    def cache_spec(self):
        if self.shift_name is None:
            return self.mixer.cache_spec()
        from .spec import JoinedSpec, StateSpec
        return JoinedSpec({"mixer": self.mixer.cache_spec(), "shift": StateSpec((self.hidden,), dtype="engine")})

    def input_norm(self):
        return self.norms[0][1]

    def _close(self, hidden, branch, norm_out, T, then):
        """stream += mult * norm_out(branch); then the stream normed by `then` (a norm or None) into self.normed."""
        g, off, eps = norm_out.carried()
        kw = {}
        if then is not None:
            w2, off2, eps2 = then.carried()
            kw = dict(out=self.normed, weight=w2, eps=eps2, offset=off2)
        return ops.rmsnorm_stream(hidden, T, branch=branch, branch_weight=g, branch_eps=eps, branch_offset=off,
                                  mult=self.mult, **kw)

    def forward(self, hidden, pending, batch, cache: CacheView, next_norm=None):
        T = batch.num_tokens
        if isinstance(pending, Carried):
            x = pending.materialise()
        else:
            if pending is not None:      # a block of another kind left its last branch to be added
                ops.add_rows(hidden, T, a=pending)
            x = self.norms[0][1].forward(hidden, self.normed, T)
        if self.shift is not None:
            if not cache.owner:
                raise NotImplementedError("token shift keeps a row a request: an entry that borrows a cache has none")
            x = ops.token_shift(x, self.shifted, cache.child("shift").state, self.shift, cu_seqlens=batch.cu_seqlens,
                                seq_lens=batch.seq_lens, state_slots=batch.state_slots, num_reqs=batch.num_reqs,
                                max_rows=batch.max_q_len)
            cache = cache.child("mixer")
        a = self.mixer.forward(x, batch, cache)
        if next_norm is not None:     # handed on only where the kernel can apply it: a gain of the type of this block's
            params = next_norm.carried()
            if params is None or params[0] is None or params[0].dtype != self.norms[0][1].weight.dtype:
                next_norm = None
        if self.ff is None:
            self._close(hidden, a, self.norms[1][1], T, next_norm)
        else:
            x = self._close(hidden, a, self.norms[1][1], T, self.norms[2][1])
            f = self.ff.forward(x, batch)
            self._close(hidden, f, self.norms[3][1], T, next_norm)
        if next_norm is None:
            return None
        return Carried(None, None, 0, 0.0, self.hidden, next_norm, hidden, self.normed, T, ready=True)


class StreamsWrite:
    """A sublayer's output that is still to be written into the residual streams (x_t <- sum_s mix[s, t] x_s +
    out[t] y): left pending by a `streams` block so that the kernel which reads the streams next does the write in the
    same pass. `settle(rows)` does it alone, for whoever needs the streams whole (the model's end, something added
    between layers)."""
    __slots__ = ("streams", "n", "branch", "mix", "out")

    def __init__(self, streams, n, branch, mix, out):
        self.streams, self.n, self.branch, self.mix, self.out = streams, n, branch, mix, out

    def settle(self, rows: int) -> None:
        ops.streams_step(self.streams, rows, self.n, dtype=self.branch.dtype, branch=self.branch, mix=self.mix,
                         out_weights=self.out)


@BLOCKS.register("streams")
class StreamsBlock(Block):
    """Pre-norm sublayers around `streams` residual streams a token instead of one ("hyper-connections"). For each
    sublayer (the mixer, then the feed-forward) with its tensors in (streams), mix (streams x streams, [from, to]) and
    out (streams):

        u = sum_s in[s] x_s;   y = sublayer(norm(u));   x_t <- sum_s mix[s, t] x_s + out[t] y   (all t from the old x)

    `hidden` is [T, streams * width] float32, the streams side by side. One kernel a sublayer boundary does the write
    of the sublayer before, the read for the next and its norm (a layer norm with gain and bias); the write of a block's
    last sublayer is left pending for the next block's first kernel. params: streams, the prefixes and names."""

    def __init__(self, hidden: int, layer: LayerSpec, streams: int, mixer_prefix: str = "mix.", ff_prefix: str = "mlp.",
                 norm_a: str = "norm1", norm_b: str = "norm2", hc_a: str = "hc1.", hc_b: str = "hc2."):
        if not 0 < streams <= ops.STREAMS_MAX or hidden > ops.STREAMS_MAX_WIDTH:
            raise ValueError(f"streams block: {streams} streams of width {hidden} have no kernel (up to "
                             f"{ops.STREAMS_MAX} of {ops.STREAMS_MAX_WIDTH})")
        self.hidden, self.n = hidden, streams
        self.mixer = MIXERS.get(layer.mixer.kind)(hidden=hidden, **layer.mixer.params)
        self.ff = FEED_FORWARDS.get(layer.feed_forward.kind)(hidden=hidden, **layer.feed_forward.params)
        if getattr(self.ff, "absent", False):
            self.ff = None
        ncls = NORMS.get(layer.norm.kind)
        self.norms = [(norm_a, ncls(hidden, **layer.norm.params))]
        self.hc_names = [hc_a]
        if self.ff is not None:
            self.norms.append((norm_b, ncls(hidden, **layer.norm.params)))
            self.hc_names.append(hc_b)
        for _, nm in self.norms:
            if not hasattr(nm, "has_bias"):
                raise ValueError("the streams arrangement takes layer norms (gain and optional bias)")
        self.prefixes = (mixer_prefix, ff_prefix)
        self.hc = []

    def _parts(self):
        out = [(self.prefixes[0], self.mixer)] + list(self.norms)
        if self.ff is not None:
            out.append((self.prefixes[1], self.ff))
        return out

    @property
    def capturable(self):
        return all(part.capturable for _, part in self._parts())

    @property
    def capturable_portions(self):
        return all(part.capturable and part.capturable_portions for _, part in self._parts())

    def tensors(self):
        from .spec import TensorSpec
        t = {p + n: s for p, part in self._parts() for n, s in part.tensors().items()}
        for hc in self.hc_names:
            t[hc + "in"] = TensorSpec((self.n,), init="ones")
            t[hc + "out"] = TensorSpec((self.n,), init="ones")
            t[hc + "mix"] = TensorSpec((self.n, self.n), init="eye")
        return t

    def load(self, get):
        for p, part in self._parts():
            part.load(_sub(get, p))
        # small parameters in 32 bits (exact for a bfloat16 file): they act on the residual streams
        self.hc = [tuple(get(hc + k).float().contiguous() for k in ("in", "mix", "out")) for hc in self.hc_names]

    def bind(self, ctx):
        for _, part in self._parts():
            part.bind(ctx)
        self.normed = ctx.workspace.buffer("normed", self.hidden)

    def _boundary(self, hidden, pending, which, T):
        """The write that is pending (if any), then the read and the norm of sublayer `which`; returns the normed input."""
        if pending is not None and not isinstance(pending, StreamsWrite):
            raise TypeError("a streams block follows blocks of its own kind only")
        norm = self.norms[which][1]
        kw = {}
        if pending is not None:
            kw = dict(branch=pending.branch, mix=pending.mix, out_weights=pending.out)
        return ops.streams_step(hidden, T, self.n, dtype=self.normed.dtype, read=self.hc[which][0], gain=norm.weight,
                                bias=norm.bias, eps=norm.eps, out=self.normed, **kw)

    def forward(self, hidden, pending, batch, cache: CacheView):
        T = batch.num_tokens
        if isinstance(pending, Carried):
            pending = None
        x = self._boundary(hidden, pending, 0, T)
        a = self.mixer.forward(x, batch, cache)
        pending = StreamsWrite(hidden, self.n, a, self.hc[0][1], self.hc[0][2])
        if self.ff is not None:
            x = self._boundary(hidden, pending, 1, T)
            f = self.ff.forward(x, batch)
            pending = StreamsWrite(hidden, self.n, f, self.hc[1][1], self.hc[1][2])
        return pending
