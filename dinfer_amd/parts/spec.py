"""Descriptions from which a model is put together.

An architecture turns its configuration into a ``ModelSpec``: per layer the
kind and parameters of its mixer, feed-forward, norms and block arrangement,
plus the order in which layers run. Nothing here names a model; sizes and
constants arrive as parameters.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any


@dataclass(frozen=True)
class PartSpec:
    """Kind (a name in the matching registry) and constructor parameters of one part."""
    kind: str
    params: dict = field(default_factory=dict)

    def __hash__(self):
        return hash((self.kind, repr(sorted(self.params.items(), key=lambda kv: kv[0]))))


def part(kind: str, **params: Any) -> PartSpec:
    return PartSpec(kind, dict(params))


@dataclass(frozen=True)
class TensorSpec:
    """One tensor a part expects from the weight file.

    init: how the random-weights mode draws it: "linear" N(0, 0.02), "gain"
    1 + N(0, 0.1), "shares" uniform in [0, 1), "zeros", "ones", "eye" (the unit matrix). keep_f32: stays 32-bit even in a bfloat16
    engine when the file stores it so.
    """
    shape: tuple
    init: str = "linear"
    integer: bool = False


class CacheSpec:
    """What one run entry keeps between steps, and how its memory is made. The engine sizes, groups and allocates
    every cache through these methods only, so a mixer with another kind of cache (one vector a token, unequal key
    and value widths, a layout of its own) brings a subclass and nothing in the engine changes.

    Paged memory: entries whose `group_key()` is equal share a pool of pages and one block table a request; a page id
    is valid in the tensors of every entry of the group. `page_bytes` says what one page of this entry takes, and
    `allocate` makes the tensors for `num_blocks` pages. Per-request memory of fixed size: `slot_bytes` a request,
    `allocate` makes room for `num_slots` requests (one of them is a spare that padded rows of a replayed graph use),
    `reset_slots` clears the slots of requests that have just been admitted.
    """
    window: int | None = None      # W: pages whose keys all lie more than W before the next token are given back
    keep_first: int = 0            # with a window: the pages of the first keep_first keys are never given back
    recomputable: bool = True      # the contents follow from the request's tokens alone (pages may be shared and refilled)
    chunk_alignment: int = 1       # prompt portions that do not end the request must end at a multiple of this

    def group_key(self) -> tuple | None:
        """Hashable name of the page group; None if nothing here is paged."""
        return None

    def page_bytes(self, page_size: int, dtype) -> int:
        return 0

    def slot_bytes(self, dtype) -> int:
        return 0

    def allocate(self, num_blocks: int, page_size: int, num_slots: int, dtype, device) -> dict:
        """name -> tensor; the mixer finds them as attributes of its CacheView."""
        return {}

    def reset_slots(self, tensors: dict, slots) -> None:
        """slots: int64 tensor of request slots that start from nothing."""


def _element_size(dtype) -> int:
    import torch
    return torch.empty((), dtype=dtype).element_size()


@dataclass(frozen=True)
class KVSpec(CacheSpec):
    """Cache need of a mixer that stores a key and a value per token and kv head.

    window: None keeps every key of the request; W keeps the last W keys, so
    pages that the window has passed are given back while the request lives
    (but for the pages of the first keep_first keys, which stay visible).
    v_dim: the size of a value head where it differs from head_dim. values False:
    the values are the keys and only key pages are kept.
    """
    kv_heads: int
    head_dim: int
    window: int | None = None
    v_dim: int | None = None
    keep_first: int = 0
    values: bool = True

    def group_key(self) -> tuple:
        # Layers of equal page geometry and equal window share block tables.
        key = ("kv", self.kv_heads, self.head_dim, self.window)
        if self.v_dim not in (None, self.head_dim) or self.keep_first or not self.values:
            key += (self.v_dim, self.keep_first, self.values)
        return key

    def page_bytes(self, page_size, dtype):
        per_key = self.head_dim + ((self.v_dim or self.head_dim) if self.values else 0)
        return self.kv_heads * per_key * page_size * _element_size(dtype)

    def allocate(self, num_blocks, page_size, num_slots, dtype, device):
        import torch
        from ..kernels import ops
        out = {"k": torch.empty(ops.k_cache_shape(num_blocks, self.kv_heads, page_size, self.head_dim), dtype=dtype,
                                device=device)}
        if self.values:
            out["v"] = torch.empty(ops.v_cache_shape(num_blocks, self.kv_heads, page_size, self.v_dim or self.head_dim),
                                   dtype=dtype, device=device)
        return out


@dataclass(frozen=True)
class LatentSpec(CacheSpec):
    """Cache need of a mixer that stores one row a token which all its heads share: `rank` numbers of a latent from
    which keys and values are made, and `rot_dim` numbers of a rotated key part. Pages [blocks, page, rank + rot_dim];
    transposed: the latents once more as [blocks, rank, page], which the matrix-core kernel's product with the values
    reads (the contraction runs over the keys there)."""
    rank: int
    rot_dim: int
    window: int | None = None
    transposed: bool = False

    def group_key(self) -> tuple:
        return ("latent", self.rank, self.rot_dim, self.window, self.transposed)

    def page_bytes(self, page_size, dtype):
        return ((2 if self.transposed else 1) * self.rank + self.rot_dim) * page_size * _element_size(dtype)

    def allocate(self, num_blocks, page_size, num_slots, dtype, device):
        import torch
        from ..kernels import ops
        shape = ops.latent_cache_shape(num_blocks, page_size, self.rank, self.rot_dim)
        out = {"latent": torch.zeros(shape, dtype=dtype, device=device)}
        if self.transposed:
            out["latent_t"] = torch.zeros((num_blocks, self.rank, page_size), dtype=dtype, device=device)
        return out


@dataclass(frozen=True)
class StateSpec(CacheSpec):
    """Cache need of a mixer with per-request state of fixed size (shape per request). The state cannot be rebuilt
    from pages, so a model that has one gets no prefix cache. dtype: a torch dtype's name, or "engine" for the dtype
    the engine computes in."""
    shape: tuple
    dtype: str = "float32"
    recomputable = False

    def _dtype(self, engine_dtype):
        import torch
        return engine_dtype if self.dtype == "engine" else getattr(torch, self.dtype)

    def slot_bytes(self, dtype):
        n = 1
        for s in self.shape:
            n *= s
        return n * _element_size(self._dtype(dtype))

    def allocate(self, num_blocks, page_size, num_slots, dtype, device):
        import torch
        return {"state": torch.zeros((num_slots, *self.shape), dtype=self._dtype(dtype), device=device)}

    def reset_slots(self, tensors, slots):
        tensors["state"].index_fill_(0, slots, 0)


@dataclass(frozen=True)
class DeltaStateSpec(CacheSpec):
    """Cache need of a mixer whose state is one float32 matrix a head and request, kept transposed [heads, vdim, dim]
    (the delta rule, a retention, a state-space mixer), and, where it has a short convolution, the last taps - 1 inputs
    of every channel of it, in the engine's dtype (channels 0 and taps 1: none)."""
    heads: int
    dim: int
    vdim: int
    channels: int
    taps: int
    recomputable = False

    def slot_bytes(self, dtype):
        return self.heads * self.dim * self.vdim * 4 + self.channels * (self.taps - 1) * _element_size(dtype)

    def allocate(self, num_blocks, page_size, num_slots, dtype, device):
        import torch
        return {"state": torch.zeros((num_slots, self.heads, self.vdim, self.dim), dtype=torch.float32, device=device),
                "conv": torch.zeros((num_slots, self.channels, self.taps - 1), dtype=dtype, device=device)}

    def reset_slots(self, tensors, slots):
        tensors["state"].index_fill_(0, slots, 0)
        tensors["conv"].index_fill_(0, slots, 0)


class JoinedSpec(CacheSpec):
    """The cache needs of a mixer made of several mixers, by name: member `left`'s tensor `k` becomes `left.k`
    (CacheView.child("left") shows it as `k` again). At most one member may be paged: a run entry has one block table
    a request."""

    def __init__(self, members: dict):
        self.members = {n: m for n, m in members.items() if m is not None}
        paged = [m for m in self.members.values() if m.group_key() is not None]
        if len(paged) > 1:
            raise ValueError("a joined cache may have one paged member: a run entry has one block table a request")
        self.paged = paged[0] if paged else None
        self.window = self.paged.window if self.paged else None
        self.keep_first = self.paged.keep_first if self.paged else 0
        self.recomputable = all(m.recomputable for m in self.members.values())
        import math
        self.chunk_alignment = math.lcm(*(m.chunk_alignment for m in self.members.values())) if self.members else 1

    def group_key(self):
        return self.paged.group_key() if self.paged else None

    def page_bytes(self, page_size, dtype):
        return sum(m.page_bytes(page_size, dtype) for m in self.members.values())

    def slot_bytes(self, dtype):
        return sum(m.slot_bytes(dtype) for m in self.members.values())

    def allocate(self, num_blocks, page_size, num_slots, dtype, device):
        return {f"{n}.{k}": t for n, m in self.members.items()
                for k, t in m.allocate(num_blocks, page_size, num_slots, dtype, device).items()}

    def reset_slots(self, tensors, slots):
        for n, m in self.members.items():
            m.reset_slots({k[len(n) + 1:]: t for k, t in tensors.items() if k.startswith(n + ".")}, slots)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: which block arrangement holds which mixer, feed-forward and norm.

    prefix: the layer's weight-name prefix; each part adds its own sub-prefix and
    local tensor names.
    """
    block: PartSpec
    mixer: PartSpec
    feed_forward: PartSpec
    norm: PartSpec
    prefix: str


@dataclass(frozen=True)
class RunEntry:
    """One position in the execution order.

    layer: index into ModelSpec.layers (a layer may appear more than once: its
    weights are shared). cache: index of the run entry whose cache this entry
    uses; its own index by default. An entry that names another entry's cache
    reads it and writes nothing. before: a PartSpec of STREAM_OPS applied to the
    residual stream right before this entry's layer (a model that runs some of
    its layers several times may add something at the start of each pass); its
    tensors are read under the names it gives, without a prefix.
    """
    layer: int
    cache: int | None = None
    before: PartSpec | None = None


@dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    layers: list  # [LayerSpec]
    run: list  # [RunEntry]
    final_norm: PartSpec
    final_norm_name: str
    embed_name: str
    head_name: str
    tie_embeddings: bool
    eos_token_ids: tuple = ()
    # optional, each a PartSpec of STREAM_OPS: applied in place to the embeddings before the first layer (tensors of
    # its own under embed_name + "post.") and to the logits after the head (under head_name + "post.")
    embed_post: PartSpec | None = None
    logits_post: PartSpec | None = None
    # the embeddings are multiplied by this on their way into the stream (inside the gather)
    embed_scale: float = 1.0
    # "float32": the residual stream is kept in 32 bits whatever the engine's dtype (the blocks' norms read it and write
    # the engine's dtype); None: the engine's dtype
    stream_dtype: str | None = None
    # residual streams a token: with n > 1 the blocks are handed [T, n * hidden] (float32), the streams side by side,
    # every one starting as the embedding; the final norm reads their sum
    streams: int = 1
