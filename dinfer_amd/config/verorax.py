"""Configuration of the Verorax architecture: a decoder whose layers mix by latent attention (queries through a latent
of their own), by a windowed differential attention, or by a windowed, gated attention beside a delta rule with
per-channel decay; every mixer reads a token-shifted input; a norm before and after every sublayer; dense or routed
feed-forwards; layers that run on another layer's weights.

config.json is nested; every size and every constant that may differ between models of the design is read from it:

    architecture    "Verorax"
    vocab, width
    norm.eps
    layers[i].type  "latent_attention" | "attention" | "parallel"
    layers[i].mixer latent_attention: heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, rot{base, dims}
                    attention:        heads, kv_heads, dim, vdim, scale, diff, mask{size}
                    parallel:         left{heads, kv_heads, dim, vdim, scale, mask{size}, rot{base, dims}},
                                      right{heads, dim}, left_scale, right_scale
    layers[i].mlp   null | {kind: "dense", ff} | {kind: "moe", expert{ff}, router{experts, identity, top}}
    layers[i].weights_of   (optional) j: the layer has no tensors and runs on layer j's, with a cache of its own (its entry
                    is expected to equal layer j's; where a constant differs, a window say, the entry's own counts, and
                    a size that does not fit layer j's tensors is refused when the weights are checked)

One size is in no key: the inner size of the decay projection of a parallel layer's right half is the row count of the
tensor l<i>.mix.right.w1. `sizes_from_tensors` puts it into the parsed file as right.decay_rank before the
configuration is made (a file that holds the key itself is taken at its word).
"""
from __future__ import annotations

from dataclasses import dataclass, field

from .base import ConfigError, ModelConfig, key
from .kudurax import _num, _section


@dataclass(frozen=True)
class Rotation:
    base: float
    dims: int


@dataclass(frozen=True)
class LatentConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: Rotation


@dataclass(frozen=True)
class DifferentialConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    window: int


@dataclass(frozen=True)
class GatedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    rot: Rotation


@dataclass(frozen=True)
class ChannelDeltaConfig:
    heads: int
    dim: int
    decay_rank: int


@dataclass(frozen=True)
class ParallelConfig:
    left: GatedAttentionConfig
    right: ChannelDeltaConfig
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str              # "dense" | "moe"
    ff: int                # the inner size (of an expert, where routed)
    experts: int = 0
    identity: int = 0
    top: int = 0


@dataclass(frozen=True)
class VeroraxLayer:
    type: str              # "latent_attention" | "attention" | "parallel"
    mixer: object
    mlp: FeedForwardConfig | None
    weights_of: int | None = None


def _rotation(m: dict, where: str, most: int) -> Rotation:
    rot = _section(m, "rot", where)
    out = Rotation(_num(rot, "base", float, where + "rot."), _num(rot, "dims", int, where + "rot."))
    if out.dims % 2 or out.dims > most:
        raise ConfigError(f"config key {where}'rot.dims' must be even and at most {most}, got {out.dims}")
    return out


def _heads(m: dict, where: str) -> tuple:
    heads, kv = _num(m, "heads", int, where), _num(m, "kv_heads", int, where)
    if heads % kv:
        raise ConfigError(f"config key {where}'heads' {heads} is no multiple of 'kv_heads' {kv}")
    return heads, kv


def _mixer(typ: str, m: dict, where: str):
    if typ == "latent_attention":
        rot_dim = _num(m, "rot_dim", int, where)
        rot = _rotation(m, where, rot_dim)       # (the design turns the rotated part whole; fewer entries are taken too)
        return LatentConfig(_num(m, "heads", int, where), _num(m, "dim", int, where), rot_dim, _num(m, "vdim", int, where),
                            _num(m, "kv_rank", int, where), _num(m, "q_rank", int, where), _num(m, "scale", float, where), rot)
    if typ == "attention":
        heads, kv = _heads(m, where)
        return DifferentialConfig(heads, kv, _num(m, "dim", int, where), _num(m, "vdim", int, where),
                                  _num(m, "scale", float, where), _num(m, "diff", float, where, positive=False),
                                  _num(_section(m, "mask", where), "size", int, where + "mask."))
    if typ == "parallel":
        l, lw = _section(m, "left", where), where + "left."
        r, rw = _section(m, "right", where), where + "right."
        heads, kv = _heads(l, lw)
        dim = _num(l, "dim", int, lw)
        left = GatedAttentionConfig(heads, kv, dim, _num(l, "vdim", int, lw), _num(l, "scale", float, lw),
                                    _num(_section(l, "mask", lw), "size", int, lw + "mask."), _rotation(l, lw, dim))
        if "decay_rank" not in r:
            raise ConfigError(f"config key {rw}'decay_rank' is neither in the file nor known from the tensor "
                              "'mix.right.w1' (a configuration made without its weights must name it)")
        right = ChannelDeltaConfig(_num(r, "heads", int, rw), _num(r, "dim", int, rw), _num(r, "decay_rank", int, rw))
        return ParallelConfig(left, right, _num(m, "left_scale", float, where, positive=False),
                              _num(m, "right_scale", float, where, positive=False))
    raise ConfigError(f"config key {where[:-6]}'type': unknown mixer {typ!r} (known: 'latent_attention', 'attention', "
                      "'parallel')")


def _feed_forward(f, where: str) -> FeedForwardConfig | None:
    if f is None:
        return None
    if not isinstance(f, dict) or f.get("kind") not in ("dense", "moe"):
        raise ConfigError(f"config key {where}'mlp' must be null or an object of kind 'dense' or 'moe', got {f!r}")
    if f["kind"] == "dense":
        return FeedForwardConfig("dense", _num(f, "ff", int, where + "mlp."))
    r = _section(f, "router", where + "mlp.")
    rw = where + "mlp.router."
    out = FeedForwardConfig("moe", _num(_section(f, "expert", where + "mlp."), "ff", int, where + "mlp.expert."),
                            experts=_num(r, "experts", int, rw), top=_num(r, "top", int, rw),
                            identity=_num(r, "identity", int, rw, positive=False) if r.get("identity") is not None else 0)
    if out.identity < 0 or out.top > out.experts + out.identity:
        raise ConfigError(f"config key {rw}: {out.top} of {out.experts} + {out.identity} experts cannot be chosen")
    return out


@dataclass(frozen=True)
class VeroraxConfig(ModelConfig):
    vocab: int = key(int)
    width: int = key(int)
    norm_eps: float = field(default=1e-6)
    layers: tuple = field(default=())

    ARCHITECTURE = "Verorax"
    MAX_POSITIONS = (1 << 31) - 1     # the design sets no limit; positions are 32-bit in the batch

    @staticmethod
    def sizes_from_tensors(d: dict, shapes: dict) -> dict:
        """d: the parsed config.json; shapes: tensor name -> shape of the model's weight files. Returns d with the
        sizes that only a tensor's shape gives filled in."""
        layers = d.get("layers")
        if not isinstance(layers, list):
            return d
        out = []
        for i, l in enumerate(layers):
            right = l.get("mixer", {}).get("right") if isinstance(l, dict) and isinstance(l.get("mixer"), dict) else None
            src = l.get("weights_of", i) if isinstance(l, dict) else i
            shape = shapes.get(f"l{src}.mix.right.w1")
            if isinstance(right, dict) and "decay_rank" not in right and shape:
                l = dict(l, mixer=dict(l["mixer"], right=dict(right, decay_rank=int(shape[0]))))
            out.append(l)
        return dict(d, layers=out)

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
            typ = l.get("type")
            src = l.get("weights_of")
            if src is not None:
                src = _num(l, "weights_of", int, where, positive=False)
                if not (0 <= src < len(layers)) or src == i or layers[src].get("weights_of") is not None:
                    raise ConfigError(f"config key {where}'weights_of' {src} must name another layer that has weights of its own")
                if layers[src].get("type") != typ:
                    raise ConfigError(f"config key {where}'weights_of' {src} names a layer of another type")
            out.append(VeroraxLayer(typ, _mixer(typ, _section(l, "mixer", where), where + "mixer."),
                                    _feed_forward(l.get("mlp"), where), src))
        for i, l in enumerate(out):
            if l.weights_of is not None and (l.mlp is None) != (out[l.weights_of].mlp is None):
                raise ConfigError(f"config key layers[{i}]: a layer with 'weights_of' has a feed-forward if and only if the "
                                  "layer it names has one")
        return {"norm_eps": _num(_section(d, "norm", ""), "eps", float, "norm."), "layers": tuple(out)}

    def check(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError(f"config keys 'vocab' and 'width' must be positive, got {self.vocab} and {self.width}")

    def extra_to_dict(self) -> dict:
        def rot(r: Rotation):
            return {"base": r.base, "dims": r.dims}

        def mixer(l: VeroraxLayer):
            m = l.mixer
            if l.type == "latent_attention":
                return {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                        "q_rank": m.q_rank, "scale": m.scale, "rot": rot(m.rot)}
            if l.type == "attention":
                return {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                        "diff": m.diff, "mask": {"size": m.window}}
            a, r = m.left, m.right
            return {"left": {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale,
                             "mask": {"size": a.window}, "rot": rot(a.rot)},
                    "right": {"heads": r.heads, "dim": r.dim, "decay_rank": r.decay_rank},
                    "left_scale": m.left_scale, "right_scale": m.right_scale}

        def mlp(f: FeedForwardConfig | None):
            if f is None:
                return None
            if f.kind == "dense":
                return {"kind": "dense", "ff": f.ff}
            return {"kind": "moe", "expert": {"ff": f.ff}, "router": {"experts": f.experts, "identity": f.identity, "top": f.top}}

        layers = []
        for l in self.layers:
            e = {"type": l.type, "mixer": mixer(l), "mlp": mlp(l.mlp)}
            if l.weights_of is not None:
                e["weights_of"] = l.weights_of
            layers.append(e)
        return {"architecture": self.ARCHITECTURE, "norm": {"eps": self.norm_eps}, "layers": layers}

    def to_dict(self) -> dict:
        out = {"vocab": self.vocab, "width": self.width}
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
