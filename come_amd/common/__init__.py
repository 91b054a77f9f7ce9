"""Host-side helpers of the attention path (mirror of the reference's ``src/accelerate/common``)."""

from .qkv import RotaryPositionEmbedding2D, prepare_packed_self_attention_qkv  # noqa: F401
