"""Configuration of the Fanulix architecture: a decoder whose layers hold either a softmax attention with a sink
beside a retention (linear attention with a fixed decay a head), or a state-space mixer with a scalar decay a head and
token; routed feed-forwards with a shared expert; several residual streams mixed by learned weights.

config.json is nested; every size and every constant that may differ between models of the design is read from it:

    architecture    "Fanulix"
    vocab, width, logit_scale
    streams         number of residual streams; absent or null: one stream with the plain residual sum
    norm.eps
    layers[i].type  "parallel" | "mamba2"
    layers[i].mixer parallel: left{heads, kv_heads, dim, vdim, scale, q_temp{coef, every}},
                              right{heads, dim, vdim, decay[heads], rot{base, dims}}, left_scale, right_scale
                    mamba2:   heads, vdim, state, groups, conv, norm_groups
    layers[i].mlp   null | {kind: "moe", router{experts, top}, expert{ff}, shared{ff} or null}
"""
from __future__ import annotations

from dataclasses import dataclass, field

from .base import ConfigError, ModelConfig, coerce, key
from .kudurax import _num, _section


@dataclass(frozen=True)
class SinkAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    temp_coef: float
    temp_every: int


@dataclass(frozen=True)
class RetentionConfig:
    heads: int
    dim: int
    vdim: int
    decay: tuple
    rot_base: float
    rot_dims: int


@dataclass(frozen=True)
class SideBySideConfig:
    left: SinkAttentionConfig
    right: RetentionConfig
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class StateSpaceConfig:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int


@dataclass(frozen=True)
class RoutedConfig:
    experts: int
    top: int
    ff: int
    shared_ff: int | None


@dataclass(frozen=True)
class FanulixLayer:
    type: str                    # "parallel" | "mamba2"
    mixer: object                # SideBySideConfig | StateSpaceConfig
    mlp: RoutedConfig | None


def _left(m: dict, where: str) -> SinkAttentionConfig:
    temp = _section(m, "q_temp", where)
    out = SinkAttentionConfig(heads=_num(m, "heads", int, where), kv_heads=_num(m, "kv_heads", int, where),
                              dim=_num(m, "dim", int, where), vdim=_num(m, "vdim", int, where),
                              scale=_num(m, "scale", float, where),
                              temp_coef=_num(temp, "coef", float, where + "q_temp.", positive=False),
                              temp_every=_num(temp, "every", int, where + "q_temp."))
    if out.heads % out.kv_heads:
        raise ConfigError(f"config key {where}'heads' {out.heads} is no multiple of 'kv_heads' {out.kv_heads}")
    return out


def _right(m: dict, where: str) -> RetentionConfig:
    rot = _section(m, "rot", where)
    decay = m.get("decay")
    heads = _num(m, "heads", int, where)
    if not isinstance(decay, list) or len(decay) != heads:
        raise ConfigError(f"config key {where}'decay' must list one decay a head ({heads}), got {decay!r}")
    decay = tuple(coerce(f"{where}decay[{i}]", v, float) for i, v in enumerate(decay))
    out = RetentionConfig(heads=heads, dim=_num(m, "dim", int, where), vdim=_num(m, "vdim", int, where), decay=decay,
                          rot_base=_num(rot, "base", float, where + "rot."),
                          rot_dims=_num(rot, "dims", int, where + "rot.", positive=False))
    if out.rot_dims < 0 or out.rot_dims > out.dim or out.rot_dims % 2:
        raise ConfigError(f"config key {where}'rot.dims' must be even and at most dim {out.dim}, got {out.rot_dims}")
    return out


def _state_space(m: dict, where: str) -> StateSpaceConfig:
    out = StateSpaceConfig(*(_num(m, k, int, where) for k in ("heads", "vdim", "state", "groups", "conv", "norm_groups")))
    if out.heads % out.groups:
        raise ConfigError(f"config key {where}'heads' {out.heads} is no multiple of 'groups' {out.groups}")
    if (out.heads * out.vdim) % out.norm_groups:
        raise ConfigError(f"config key {where}'norm_groups' {out.norm_groups} does not divide heads * vdim "
                          f"{out.heads * out.vdim}")
    return out


def _routed(f: dict, where: str) -> RoutedConfig:
    if f.get("kind") != "moe":
        raise ConfigError(f"config key {where}'kind': unknown feed-forward {f.get('kind')!r} (known: 'moe')")
    router = _section(f, "router", where)
    shared = f.get("shared")
    if shared is not None and not isinstance(shared, dict):
        raise ConfigError(f"config key {where}'shared' must be an object or null, got {shared!r}")
    out = RoutedConfig(experts=_num(router, "experts", int, where + "router."), top=_num(router, "top", int, where + "router."),
                       ff=_num(_section(f, "expert", where), "ff", int, where + "expert."),
                       shared_ff=None if shared is None else _num(shared, "ff", int, where + "shared."))
    if out.top > out.experts:
        raise ConfigError(f"config key {where}'router.top' {out.top} exceeds 'router.experts' {out.experts}")
    return out


@dataclass(frozen=True)
class FanulixConfig(ModelConfig):
    vocab: int = key(int)
    width: int = key(int)
    logit_scale: float = key(float, 1.0)
    streams: int | None = key(int, None, nullable=True)
    norm_eps: float = field(default=1e-5)
    layers: tuple = field(default=())

    ARCHITECTURE = "Fanulix"
    MAX_POSITIONS = (1 << 31) - 1     # the design sets no limit; positions are 32-bit in the batch

    @classmethod
    def extra_from_dict(cls, d: dict) -> dict:
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config key 'layers' must be a non-empty list")
        out = []
        for i, l in enumerate(layers):
            where = f"layers[{i}]."
            if not isinstance(l, dict):
                raise ConfigError(f"config key 'layers[{i}]' must be an object")
            typ, m = l.get("type"), _section(l, "mixer", where)
            if typ == "parallel":
                mixer = SideBySideConfig(_left(_section(m, "left", where + "mixer."), where + "mixer.left."),
                                         _right(_section(m, "right", where + "mixer."), where + "mixer.right."),
                                         _num(m, "left_scale", float, where + "mixer.", positive=False),
                                         _num(m, "right_scale", float, where + "mixer.", positive=False))
            elif typ == "mamba2":
                mixer = _state_space(m, where + "mixer.")
            else:
                raise ConfigError(f"config key {where}'type': unknown mixer {typ!r} (known: 'parallel', 'mamba2')")
            f = l.get("mlp")
            if f is not None and not isinstance(f, dict):
                raise ConfigError(f"config key {where}'mlp' must be an object or null, got {f!r}")
            out.append(FanulixLayer(typ, mixer, None if f is None else _routed(f, where + "mlp.")))
        return {"norm_eps": _num(_section(d, "norm", ""), "eps", float, "norm."), "layers": tuple(out)}

    def check(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError(f"config keys 'vocab' and 'width' must be positive, got {self.vocab} and {self.width}")
        if self.streams is not None and self.streams <= 0:
            raise ConfigError(f"config key 'streams' must be positive or null, got {self.streams}")

    def extra_to_dict(self) -> dict:
        def mixer(l: FanulixLayer):
            m = l.mixer
            if l.type == "mamba2":
                return {"heads": m.heads, "vdim": m.vdim, "state": m.state, "groups": m.groups, "conv": m.conv,
                        "norm_groups": m.norm_groups}
            a, r = m.left, m.right
            return {"left": {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale,
                             "q_temp": {"coef": a.temp_coef, "every": a.temp_every}},
                    "right": {"heads": r.heads, "dim": r.dim, "vdim": r.vdim, "decay": list(r.decay),
                              "rot": {"base": r.rot_base, "dims": r.rot_dims}},
                    "left_scale": m.left_scale, "right_scale": m.right_scale}

        def mlp(f: RoutedConfig | None):
            if f is None:
                return None
            return {"kind": "moe", "router": {"experts": f.experts, "top": f.top}, "expert": {"ff": f.ff},
                    "shared": None if f.shared_ff is None else {"ff": f.shared_ff}}

        return {"architecture": self.ARCHITECTURE, "norm": {"eps": self.norm_eps},
                "layers": [{"type": l.type, "mixer": mixer(l), "mlp": mlp(l.mlp)} for l in self.layers]}

    def to_dict(self) -> dict:
        out = {"vocab": self.vocab, "width": self.width, "logit_scale": self.logit_scale, "streams": self.streams}
        out.update(self.extra_to_dict())
        return out

    # what programs that know no architecture ask a configuration
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def max_position_embeddings(self) -> int:
        return self.MAX_POSITIONS

    @property
    def eos_token_ids(self) -> tuple:
        return ()
