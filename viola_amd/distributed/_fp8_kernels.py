"""FP8 gradient wire codec operators (operator seam of viola/distributed/_fp8_kernels.py:
views :10, pack :84, unpack :90). A packet is [rows, stride] uint8; each row holds groups*tile
FP8 codes, then `groups` fp32 scales, padded to a multiple of 16 bytes."""

import torch

from .. import _lib


def views(packet, tile_size, fp8_dtype):
    groups = packet.shape[1] // (tile_size + 4)
    width = groups * tile_size
    return packet[:, :width].view(fp8_dtype), packet[:, width:width + groups * 4].view(torch.float32)


def _geometry(packet, tile_size):
    assert packet.is_cuda and packet.dtype == torch.uint8 and packet.dim() == 2 and packet.is_contiguous()
    groups = packet.shape[1] // (tile_size + 4)
    assert packet.shape[1] == (groups * (tile_size + 4) + 15) // 16 * 16, "packet row is not packet_bytes(groups, tile)"
    return packet.shape[0], groups


def pack(source, packet, tile_size, fp8_dtype):
    """fp32 vector -> packet rows; element index = row*groups*tile + group*tile + i, zero past the end."""
    rows, groups = _geometry(packet, tile_size)
    assert source.dtype == torch.float32 and source.is_contiguous()
    _lib.call("viola_comm_pack", _lib.ptr(source), source.numel(), _lib.ptr(packet), rows, groups, tile_size,
              _lib.code(fp8_dtype))


def unpack(packet, out, tile_size, fp8_dtype, *, reduce=False):
    """packet rows -> fp32 vector; reduce=True sums the rows (one per sending rank) in rank order."""
    rows, groups = _geometry(packet, tile_size)
    assert out.dtype == torch.float32 and out.is_contiguous()
    _lib.call("viola_comm_unpack", _lib.ptr(packet), _lib.ptr(out), out.numel(), rows, groups, tile_size,
              _lib.code(fp8_dtype), int(reduce))
