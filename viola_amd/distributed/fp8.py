"""Scaled FP8 on the wire (viola/distributed/fp8.py:9-85), one GPU: the codec and its packet
geometry. The reference's collectives (all_to_all + all_gather, gather to owner) sit between pack and
unpack; with one process they are the identity, which is what `roundtrip` exercises."""

import math

import torch

from . import _fp8_kernels as codec


def packet_bytes(groups, tile_size):
    """Bytes of one packet row: codes + fp32 scales, rounded up to 16."""
    return (groups * (tile_size + 4) + 15) // 16 * 16


class FP8Communication:
    """Single-process stand-in with the reference's constructor: world size 1, so all_reduce / reduce
    return at once (fp8.py:50-51,69-70). `roundtrip` runs encode -> decode on a bucket."""

    def __init__(self, capacity, mesh=None, device=None, *, mode="all_reduce", fp8_format="e4m3", tile_size=256):
        assert tile_size >= 32 and tile_size & (tile_size - 1) == 0
        self.fp8_dtype = {"e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2}[fp8_format]
        self.tile_size, self.mode, self.device = tile_size, mode, device
        self.rank, self.world = 0, 1
        groups = math.ceil(capacity / tile_size)
        self.send = torch.empty((1, packet_bytes(groups, tile_size)), device=device, dtype=torch.uint8)

    @property
    def workspace_bytes(self):
        return self.send.numel()

    def all_reduce(self, value):
        return

    def reduce(self, value, owner):
        return

    @torch.no_grad()
    def roundtrip(self, value):
        """value (fp32, in place) <- decode(encode(value)): what one hop of the wire does to a bucket."""
        groups = math.ceil(value.numel() / self.tile_size)
        packet = self.send.view(-1)[:packet_bytes(groups, self.tile_size)].view(1, -1)
        codec.pack(value, packet, self.tile_size, self.fp8_dtype)
        codec.unpack(packet, value, self.tile_size, self.fp8_dtype)
        return value
