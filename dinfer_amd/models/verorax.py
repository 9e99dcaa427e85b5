"""Verorax: configuration -> ModelSpec.

embed -> run list of sandwich blocks( token shift, mixer | feed-forward or none ) -> norm -> head.
A block: x = shift(norm1(h)); h += norm1b(mixer(x)); h += norm2b(ff(norm2(h))), root-mean-square norms with plain
gains, a 32-bit residual stream. Mixers: `latent_attention` (queries through a normed latent, keys and values from one
normed latent a token plus a rotated key part shared by the heads, causal), `attention` (differential attention: two
windowed softmax maps a head over the same values, biases, no positions) or `parallel` (a windowed attention with
per-head q/k norm, a rotation of part of each head, a temperature a head and one sigmoid gate a head, beside a delta
rule with a decay and a removal rate a key channel; the two scaled and summed). Rotations pair entry i with
i + dims/2. Feed-forwards: gated with the tanh form of gelu, or routed experts (silu) chosen by softmax score plus a
correction, weighted by the scores as they are, the last router outputs standing for experts that hand their input
on. A layer with `weights_of` is a second run entry of the layer it names, with a cache of its own (where its entry
differs from that layer's in a constant, it is a layer of its own that reads the same tensors).
Tensor names: embed, l<i>.norm{1,1b,2,2b}, l<i>.shift, l<i>.mix.{dq, dq.norm, uq, dkv, dkv.norm, uk, uv, o} or
l<i>.mix.{q, k, v}(.b), l<i>.mix.{lq1, lk1, lq2, lk2, o} or l<i>.mix.left.{q, k, v, q.norm, k.norm, temp, g, o} and
l<i>.mix.right.{r, k, v, g, a, a.b, w1, w2, w0, norm, o}; l<i>.mlp.{gate, up, down} or
l<i>.mlp.{router, correction, e<j>.{gate, up, down}}; final.norm, head.
"""
from __future__ import annotations

import math

from ..config.registry import register_architecture
from ..config.verorax import VeroraxConfig
from ..parts.spec import LayerSpec, ModelSpec, RunEntry, part

DECAY_RATE = math.exp(-0.5)    # a channel's decay is exp(-DECAY_RATE * sigmoid(.)): never below 0.545 a token
UNIT_EPS = 1e-6                # under the root of the delta rule's unit key


def _rotary(cfg: VeroraxConfig, rot):
    return part("rotary", theta=rot.base, max_positions=cfg.MAX_POSITIONS, rotary_dim=rot.dims, style="neox")


def _mixer(cfg: VeroraxConfig, l):
    m, eps = l.mixer, cfg.norm_eps
    plain_norm = part("rmsnorm", eps=eps, weight_name="")
    if l.type == "latent_attention":
        return part("latent_attention", heads=m.heads, dim=m.dim, rot_dim=m.rot_dim, vdim=m.vdim, rank=m.kv_rank,
                    q_rank=m.q_rank, scale=m.scale, position=_rotary(cfg, m.rot), latent_norm=plain_norm, gated=False)
    if l.type == "attention":
        return part("differential_attention", heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale,
                    diff=m.diff, norm_eps=eps, window=m.window, bias=True)
    a, r = m.left, m.right
    left = part("attention", heads=a.heads, kv_heads=a.kv_heads, head_dim=a.dim, v_dim=a.vdim, position=_rotary(cfg, a.rot),
                qk_norm=plain_norm, window=a.window, scale=a.scale, head_temp=True, gate="sigmoid", gate_heads=True,
                names={"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "g": "g",
                       "temp": "temp"})
    right = part("channel_delta_rule", heads=r.heads, dim=r.dim, low=r.decay_rank, norm_eps=eps, rate=DECAY_RATE,
                 unit_eps=UNIT_EPS)
    return part("joined", members=[("left", left, m.left_scale), ("right", right, m.right_scale)])


def _feed_forward(f):
    if f is None:
        return part("none")
    if f.kind == "dense":
        return part("gated_mlp", intermediate=f.ff, act="gelu_tanh", names=("gate", "up", "down"))
    return part("moe", experts=f.experts, top=f.top, intermediate=f.ff, act="silu", scores="all", correction=True,
                identity=f.identity)


def build_spec(cfg: VeroraxConfig) -> ModelSpec:
    norm = part("rmsnorm", eps=cfg.norm_eps, weight_name="")
    layers, place, run = [], {}, []
    for i, l in enumerate(cfg.layers):
        if l.weights_of is None:      # a layer with tensors of its own
            place[i] = len(layers)
            layers.append(LayerSpec(block=part("sandwich", shift="shift"), mixer=_mixer(cfg, l),
                                    feed_forward=_feed_forward(l.mlp), norm=norm, prefix=f"l{i}."))
    for i, l in enumerate(cfg.layers):
        src = i if l.weights_of is None else l.weights_of
        if src != i and (l.mixer, l.mlp) != (cfg.layers[src].mixer, cfg.layers[src].mlp):
            # the same tensors under constants of its own (a window, a scale): a layer of its own that reads them again
            place[i] = len(layers)
            layers.append(LayerSpec(block=part("sandwich", shift="shift"), mixer=_mixer(cfg, l),
                                    feed_forward=_feed_forward(l.mlp), norm=norm, prefix=f"l{src}."))
            src = i
        run.append(RunEntry(place[src]))
    return ModelSpec(
        architecture=cfg.ARCHITECTURE, vocab_size=cfg.vocab, hidden_size=cfg.width, max_positions=cfg.MAX_POSITIONS,
        layers=layers, run=run, final_norm=norm, final_norm_name="final.norm", embed_name="embed", head_name="head",
        tie_embeddings=False, eos_token_ids=(), stream_dtype="float32")


register_architecture(VeroraxConfig.ARCHITECTURE, VeroraxConfig, build_spec)
