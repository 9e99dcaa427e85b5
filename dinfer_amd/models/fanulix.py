"""Fanulix: configuration -> ModelSpec.

embed -> N x streams block( mixer | routed feed-forward or none ) -> sum of the streams -> layer norm -> the embedding
table as head -> logits * logit_scale. `streams` residual streams a token, read and written by learned weights around
every sublayer (without `streams`: one stream and the plain pre-norm residual). Layer norms with bias. Mixers:
`parallel`: a softmax attention (biases on q, k, v; q and k divided by their root mean square a head; a query that
grows with its position; a sink of score zero; an output gate) beside a retention (rotation of pairs (i, i + rot/2),
a fixed decay a head), the two scaled and summed; `mamba2`: a state-space mixer with a scalar decay a head and token.
Feed-forward: routed experts of the form down(gelu(up x)), the chosen softmax scores divided by their sum, plus a
shared expert. Tensor names: embed, l<i>.norm{1,2}(.b), l<i>.hc{1,2}.{in, out, mix}, l<i>.mix.left.{q, k, v}(.b),
l<i>.mix.left.{g, o}, l<i>.mix.right.{q, k, v, g, o}, or l<i>.mix.{in, conv, conv.b, dt_bias, A_log, D, norm, o};
l<i>.mlp.{router, e<j>.{up, down}, shared.{up, down}}, final.norm(.b).
"""
from __future__ import annotations

from ..config.fanulix import FanulixConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, RunEntry, part

SINK_SCORE = 0.0     # the softmax's denominator holds exp(0) = 1 beside the keys' terms


def _parallel(cfg: FanulixConfig, m):
    a, r = m.left, m.right
    left = part("attention", heads=a.heads, kv_heads=a.kv_heads, head_dim=a.dim, v_dim=a.vdim, position=part("none"),
                scale=a.scale, bias=True, qk_unit_eps=cfg.norm_eps, q_temp=(a.temp_coef, a.temp_every),
                sink_value=SINK_SCORE, gate="sigmoid",
                names={"q": "q", "k": "k", "v": "v", "o": "o", "g": "g", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b"})
    position = part("none") if r.rot_dims == 0 else part("rotary", theta=r.rot_base, max_positions=cfg.MAX_POSITIONS,
                                                        rotary_dim=r.rot_dims, style="neox")
    right = part("retention", heads=r.heads, dim=r.dim, vdim=r.vdim, decay=r.decay, position=position, norm_eps=cfg.norm_eps)
    return part("joined", members=[("left", left, m.left_scale), ("right", right, m.right_scale)])


def build_spec(cfg: FanulixConfig) -> ModelSpec:
    norm = part("layernorm", eps=cfg.norm_eps, bias=True, weight_name="", bias_name=".b")
    if cfg.streams is None:
        block = part("prenorm", mixer_prefix="mix.", ff_prefix="mlp.", norm_in="norm1", norm_post="norm2")
    else:
        block = part("streams", streams=cfg.streams)
    layers = []
    for i, l in enumerate(cfg.layers):
        if l.type == "parallel":
            mixer = _parallel(cfg, l.mixer)
        else:
            m = l.mixer
            mixer = part("state_space", heads=m.heads, vdim=m.vdim, state=m.state, groups=m.groups, taps=m.conv,
                         norm_groups=m.norm_groups, norm_eps=cfg.norm_eps)
        f = l.mlp
        ff = part("none") if f is None else part("moe", experts=f.experts, top=f.top, intermediate=f.ff,
                                                 shared_intermediate=f.shared_ff, act="gelu", gated=False, shared_gate=False)
        layers.append(LayerSpec(block=block, mixer=mixer, feed_forward=ff, norm=norm, prefix=f"l{i}."))
    return ModelSpec(
        architecture=cfg.ARCHITECTURE, vocab_size=cfg.vocab, hidden_size=cfg.width, max_positions=cfg.MAX_POSITIONS,
        layers=layers, run=[RunEntry(i) for i in range(len(layers))], final_norm=norm, final_norm_name="final.norm",
        embed_name="embed", head_name="head", tie_embeddings=True, eos_token_ids=(), stream_dtype="float32",
        streams=cfg.streams or 1,
        logits_post=None if cfg.logit_scale == 1.0 else part("scale_softcap", scale=cfg.logit_scale))


register_architecture(FanulixConfig.ARCHITECTURE, FanulixConfig, build_spec)
