"""Small host-side helpers."""

import torch


def ceil_divide(a: int, b: int) -> int:
    return (a + b - 1) // b


def ensure_contiguous(t: torch.Tensor | None) -> torch.Tensor | None:
    return None if t is None else t.contiguous()


def expert_major_strides(w: torch.Tensor, name: str) -> tuple[int, int]:
    """(expert stride, row stride) in elements of a weight handed over as the reference does it: a (rows, cols, E)
    permuted view of the (E, rows, cols) parameter (sonicmoe/moe.py:223-225).  The innermost dimension of the
    parameter (cols) must be contiguous."""
    if w.dim() != 3:
        raise ValueError(f"{name}: expected a (rows, cols, E) view, got shape {tuple(w.shape)}")
    s_row, s_col, s_e = w.stride()
    if s_col != 1:
        raise ValueError(f"{name}: the column dimension must be contiguous (strides {w.stride()})")
    return s_e, s_row
