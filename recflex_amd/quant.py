"""Row-wise 8-bit table format of the fused embedding kernel.

A row of ``dim`` values is stored as ``dim`` unsigned 8-bit codes followed by an fp16 scale and
an fp16 bias, and rows are ``row_stride = round_up(dim + 4, 16)`` bytes apart (the unused tail
bytes are zero).  ``value = code * scale + bias`` with ``scale = (max - min) / 255`` and
``bias = min`` of the row, both rounded to fp16 before the codes are computed, so that the
stored triple is self-consistent.  The reference has fp32 tables only; this is the int8 format
that ``MetaData(data_type="int8")`` refers to.
"""

import torch


def int8_row_stride(dim: int) -> int:
    return (dim + 4 + 15) // 16 * 16


def quantize_rowwise_int8(weights: torch.Tensor) -> torch.Tensor:
    """fp32 ``[rows, dim]`` -> uint8 ``[rows, int8_row_stride(dim)]`` on the same device."""
    assert weights.dim() == 2
    rows, dim = weights.shape
    w = weights.float()
    lo = w.min(dim=1, keepdim=True).values if dim > 0 else w.new_zeros(rows, 1)
    hi = w.max(dim=1, keepdim=True).values if dim > 0 else w.new_zeros(rows, 1)
    bias16 = lo.half()
    scale16 = ((hi - lo) / 255.0).half()
    scale = scale16.float()
    safe = torch.where(scale > 0, scale, torch.ones_like(scale))
    codes = torch.round((w - bias16.float()) / safe).clamp_(0, 255).to(torch.uint8)
    out = torch.zeros(rows, int8_row_stride(dim), dtype=torch.uint8, device=weights.device)
    out[:, :dim] = codes
    sb = torch.cat([scale16, bias16], dim=1).contiguous()          # [rows, 2] fp16
    out[:, dim:dim + 4] = sb.view(torch.uint8).view(rows, 4)
    return out


def random_int8_table(rows: int, dim: int, device, generator: torch.Generator = None,
                      std: float = 1.0, chunk_rows: int = 1 << 20) -> torch.Tensor:
    """Quantised N(0, std) table built chunk by chunk so that no fp32 copy of the whole table
    is ever resident."""
    out = torch.empty(rows, int8_row_stride(dim), dtype=torch.uint8, device=device)
    for r0 in range(0, rows, chunk_rows):
        r1 = min(rows, r0 + chunk_rows)
        w = torch.randn(r1 - r0, dim, dtype=torch.float32, device=device, generator=generator) * std
        out[r0:r1] = quantize_rowwise_int8(w)
    return out
