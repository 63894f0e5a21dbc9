from . import attention, block, mlp, norm, position, stream_ops  # noqa: F401  (register the built-in parts)
from .base import Block, BuildContext, CacheView, Carried, FeedForward, Into, Mixer, Norm, Part, PositionEncoding, Workspace
from .model import DecoderModel, expected_tensors
from .registry import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, STREAM_OPS, Registry
from .spec import CacheSpec, KVSpec, LayerSpec, ModelSpec, PartSpec, RunEntry, StateSpec, TensorSpec, part
