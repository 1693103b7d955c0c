"""pkh3-attn: gfx950 (MI355X) attention engine for the Pika H3 Flex video+audio DiT.

Python host side over the C-ABI library ``libpkh3attn.so`` (hand-written HIP kernels).  There is
no fallback implementation: using any op without the built library raises.
"""
from . import _lib
from ._lib import Pkh3Error, ROPE_HALF, ROPE_INTERLEAVED, ROPE_NONE
from .layout import (
    audio_position_ids,
    local_window_tile_map,
    video_position_ids,
)
from . import packing
from . import projections
from .ops import BlockMask, PreparedKV, attention, attention_prepared, prepare_kv, rope_tables, time_attention_kernel
from .processor import PikaH3AttnProcessor

__all__ = [
    "BlockMask", "PikaH3AttnProcessor", "Pkh3Error", "ROPE_HALF", "ROPE_INTERLEAVED", "ROPE_NONE",
    "PreparedKV", "attention", "attention_prepared", "audio_position_ids", "local_window_tile_map", "packing", "prepare_kv", "projections", "rope_tables", "time_attention_kernel",
    "video_position_ids",
]
