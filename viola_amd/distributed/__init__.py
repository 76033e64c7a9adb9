"""FP8 gradient wire codec (single GPU: pack / unpack only, no collectives)."""

from .fp8 import FP8Communication, packet_bytes

__all__ = ["FP8Communication", "packet_bytes"]
