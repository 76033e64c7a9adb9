"""FP8 gradient wire codec on CPU. TEST INFRASTRUCTURE ONLY.

Packet layout (viola/distributed/_fp8_kernels.py:10-15, fp8.py:9-11): `rows` rows of
`stride = ceil16(groups*(tile+4))` bytes; a row holds groups*tile FP8 codes, then
`groups` fp32 scales, then zero padding.
"""

import torch
import torch.nn.functional as F


def packet_bytes(groups, tile_size):
    """viola/distributed/fp8.py:9-11."""
    return (groups * (tile_size + 4) + 15) // 16 * 16


def views(packet, tile_size, fp8_dtype):
    """Code and scale views of a [rows, stride] uint8 packet (_fp8_kernels.py:10-15)."""
    groups = packet.shape[1] // (tile_size + 4)
    width = groups * tile_size
    return packet[:, :width].view(fp8_dtype), packet[:, width:width + groups * 4].view(torch.float32)


def pack(source, rows, groups, tile_size, fp8_dtype):
    """fp32 vector -> packet (viola/distributed/_fp8_kernels.py:18-43).

    element index = row*width + group*tile + i (0 past n); amax treats NaN as +inf;
    scale = max(amax, 1e-30)/fmax; code = fp8(v/scale) with no clamp.
    """
    width = groups * tile_size
    fmax = torch.finfo(fp8_dtype).max
    x = F.pad(source.reshape(-1).float(), (0, rows * width - source.numel())).view(rows, groups, tile_size)
    magnitude = torch.where(x.isnan(), torch.full_like(x, float("inf")), x.abs())
    scales = magnitude.amax(2).clamp_min(1e-30) / fmax
    codes = (x / scales[..., None]).to(fp8_dtype)
    packet = torch.zeros(rows, packet_bytes(groups, tile_size), dtype=torch.uint8)
    q, s = views(packet, tile_size, fp8_dtype)
    q.copy_(codes.view(rows, width))
    s.copy_(scales)
    return packet


def unpack(packet, n, tile_size, fp8_dtype, *, reduce=False):
    """packet -> fp32 vector (viola/distributed/_fp8_kernels.py:46-69); reduce sums rows in order."""
    q, s = views(packet, tile_size, fp8_dtype)
    rows, groups = s.shape
    values = q.float().view(rows, groups, tile_size) * s[..., None]
    if reduce:
        total = torch.zeros(groups, tile_size)
        for rank in range(rows):
            total = total + values[rank]
        return total.flatten()[:n]
    return values.flatten()[:n]


def roundtrip(x, tile_size, fp8_dtype):
    """pad -> per-tile amax -> cast -> multiply back (checks/fp8_communication.py:32-38)."""
    count = x.numel()
    x = F.pad(x, (0, -count % tile_size)).view(-1, tile_size)
    scale = x.abs().amax(1, keepdim=True).clamp_min(1e-30) / torch.finfo(fp8_dtype).max
    return ((x / scale).to(fp8_dtype).float() * scale).flatten()[:count]
