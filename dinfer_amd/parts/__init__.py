from . import (attention, block, channel_delta, delta_rule, differential_attention, joined, latent_attention, mlp, moe, norm, position, retention, state_space,  # noqa: F401
               stream_ops)  # noqa: F401  (register the built-in parts)
from .base import Block, BuildContext, CacheView, Carried, FeedForward, Into, Mixer, Norm, Part, PositionEncoding, Workspace
from .model import DecoderModel, expected_tensors
from .registry import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, STREAM_OPS, Registry
from .spec import CacheSpec, DeltaStateSpec, JoinedSpec, KVSpec, LatentSpec, LayerSpec, ModelSpec, PartSpec, RunEntry, StateSpec, TensorSpec, part
