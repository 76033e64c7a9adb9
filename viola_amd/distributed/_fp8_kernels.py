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


def _table(rows, device, cache):
    from ..optim._kernels import _device_table
    return _device_table(rows, device, cache)


def pack_many(sources, packets, tile_size, fp8_dtype, *, cache=None):
    """pack() for a list of buckets in ONE launch (the reference drains its buckets one launch at a time,
    viola/distributed/gradients.py:101-125); same bytes as bucket-by-bucket calls, which is also what shapes
    the table kernel does not take fall back to. cache: a dict that keeps the device-side table between calls."""
    geometry = [_geometry(packet, tile_size) for packet in packets]
    assert len(sources) == len(packets) and all(s.dtype == torch.float32 and s.is_contiguous() for s in sources)
    together = tile_size == 256 and len(packets) > 1 and all(s.data_ptr() % 16 == 0 for s in sources)
    if together:
        rows = [(s.data_ptr(), s.numel(), p.data_ptr(), r, g, 0, 0, 0) for s, p, (r, g) in zip(sources, packets, geometry)]
        table = _table(rows, packets[0].device, cache)
        status = _lib.call("viola_comm_pack_table", _lib.ptr(table), len(rows), max(r * g for r, g in geometry), tile_size,
                           _lib.code(fp8_dtype), unsupported_ok=True)
        together = status == 0
    if not together:
        for source, packet in zip(sources, packets):
            pack(source, packet, tile_size, fp8_dtype)


def unpack_many(packets, outs, tile_size, fp8_dtype, *, reduce=False, cache=None):
    """unpack() for a list of buckets in ONE launch; same values as bucket-by-bucket calls."""
    geometry = [_geometry(packet, tile_size) for packet in packets]
    assert len(outs) == len(packets) and all(o.dtype == torch.float32 and o.is_contiguous() for o in outs)
    capacity = [(1 if reduce else r) * g * tile_size for r, g in geometry]
    assert all(o.numel() <= c for o, c in zip(outs, capacity))
    if len(packets) > 1 and all(o.data_ptr() % 16 == 0 for o in outs):
        rows = [(p.data_ptr(), o.numel(), o.data_ptr(), r, g, 0, 0, 0) for p, o, (r, g) in zip(packets, outs, geometry)]
        table = _table(rows, packets[0].device, cache)
        _lib.call("viola_comm_unpack_table", _lib.ptr(table), len(rows), max(capacity), tile_size, _lib.code(fp8_dtype), int(reduce))
        return
    for packet, out in zip(packets, outs):
        unpack(packet, out, tile_size, fp8_dtype, reduce=reduce)
