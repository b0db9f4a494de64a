"""TEST INFRASTRUCTURE, NOT PRODUCT CODE -- the reference's CPU code path as it actually
executes: a Python loop over rows and row segments issuing a handful of tiny torch ops
per segment.  This is the form whose wall-clock time bench.py reports as the CPU
baseline (kind "port"), and a third cross-check of the C and numpy restatements.

Reference lines followed (relative to the reference checkout):
  qtensor/functional.py:526-615   per-segment quantize loop     -> quantize_loop
  qtensor/functional.py:618-688   per-segment dequantize loop   -> dequantize_loop
  qtensor/functional.py:703-746   nearest rule, nibble packing
Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this.
"""
from __future__ import annotations

import math

import torch


def _nearest(vals: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    n = table.numel()
    pos = torch.searchsorted(table, vals, right=True).clamp(max=n)
    below = (pos - 1).clamp(min=0)
    above = pos.clamp(max=n - 1)
    take_above = (vals - table[below]).abs() > (table[above] - vals).abs()
    return torch.where(take_above, above, below)


def _pack(idx: torch.Tensor, bits: int) -> torch.Tensor:
    if bits == 8:
        return idx.to(torch.uint8)
    if idx.numel() % 2:
        idx = torch.cat([idx, idx.new_zeros(1)])
    two = idx.view(-1, 2)
    return ((two[:, 0] << 4) + (two[:, 1] & 15)).to(torch.uint8)


def _unpack(packed: torch.Tensor, numel: int, bits: int) -> torch.Tensor:
    wide = packed.to(torch.int64)
    if bits == 8:
        return wide[:numel]
    return torch.stack([wide >> 4, wide & 15], dim=1).reshape(-1)[:numel]


@torch.no_grad()
def quantize_loop(A: torch.Tensor, code: torch.Tensor, order: int, blocksize: int, bits: int,
                  store_diag: bool = False, max_rows: int | None = None):
    """Returns (out, absmax[, diag]).  max_rows limits the loop to the first rows (used by
    the benchmark to time a bounded sample); the remaining rows are then left at index 0."""
    if bits not in (4, 8):
        raise ValueError(f"unsupported bit width {bits}")
    table = code.to(torch.float32)
    order_map = None
    if bool(torch.any(table[1:] < table[:-1])):
        table, order_map = torch.sort(table, stable=True)
    tmin, tmax = table[0].item(), table[-1].item()
    nb = math.ceil(order / blocksize)
    flat = A.to(torch.float32).contiguous().view(-1).clone()
    if flat.numel() != order * order:
        raise ValueError(f"expected {order * order} elements, found {flat.numel()}")
    absmax = torch.zeros(order * nb, dtype=torch.float32)
    diag = None
    if store_diag:
        diag = torch.diagonal(A.view(order, order)).to(torch.float32).clone()
        flat[torch.arange(order) * (order + 1)] = 0.0
    idx = torch.zeros(order * order, dtype=torch.int64)
    rows = order if max_rows is None else min(order, max_rows)
    for r in range(rows):
        for b in range(nb):
            s = r * order + b * blocksize
            e = r * order + min((b + 1) * blocksize, order)
            seg = flat[s:e]
            top = float(seg.abs().max())
            absmax[r * nb + b] = top
            if top == 0.0:
                continue
            picked = _nearest((seg / top).clamp(min=tmin, max=tmax), table)
            idx[s:e] = picked if order_map is None else order_map[picked]
    out = _pack(idx, bits)
    if store_diag:
        return out, absmax, diag
    return out, absmax


@torch.no_grad()
def dequantize_loop(q: torch.Tensor, code: torch.Tensor, order: int, absmax: torch.Tensor,
                    blocksize: int, bits: int, outdtype=torch.float32, diag=None,
                    max_rows: int | None = None) -> torch.Tensor:
    nb = math.ceil(order / blocksize)
    if absmax.numel() != order * nb:
        raise ValueError(f"absmax has {absmax.numel()} entries, expected {order * nb}")
    table = code.to(torch.float32)
    idx = _unpack(q, order * order, bits)
    vals = torch.zeros(order * order, dtype=torch.float32)
    rows = order if max_rows is None else min(order, max_rows)
    for r in range(rows):
        for b in range(nb):
            s = r * order + b * blocksize
            e = r * order + min((b + 1) * blocksize, order)
            top = float(absmax[r * nb + b])
            if top == 0.0:
                continue
            vals[s:e] = table[idx[s:e]] * top
    res = vals.view(order, order).to(outdtype)
    if diag is not None:
        if diag.numel() != order:
            raise ValueError(f"diag must have length {order}")
        res.diagonal().copy_(diag.to(outdtype))
    return res
