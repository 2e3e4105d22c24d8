"""Expert histogram + inclusive prefix sum (interface of sonicmoe/count_cumsum/__init__.py:11-29)."""

import torch

from .. import _lib
from ..enums import LIBRARY_NAME


@torch.library.custom_op(f"{LIBRARY_NAME}::count_cumsum_cuda", mutates_args={"count_output", "cumsum_output"})
def count_cumsum_cuda(x: torch.Tensor, count_output: torch.Tensor, cumsum_output: torch.Tensor | None) -> None:
    _lib.require_device(x, count_output, cumsum_output)
    x = x.contiguous()
    rc = _lib.lib().smoe_count_cumsum(
        _lib.ptr(x),
        1 if x.dtype == torch.int64 else 0,
        x.numel(),
        count_output.numel(),
        _lib.ptr(count_output),
        _lib.ptr(cumsum_output),
        _lib.current_stream_handle(),
    )
    _lib.check(rc, "count_cumsum")


@torch.no_grad()
def count_cumsum(x: torch.Tensor, E: int, do_cumsum: bool = True):
    """count (E,) int32 and, with do_cumsum, the INCLUSIVE cumulative sum (E,) int32 of the values of the 1-D
    int32/int64 tensor `x`, all in [0, E)."""
    assert x.dim() == 1, "x should be 1-dimensional"
    assert x.dtype in [torch.int32, torch.long]

    count_output = torch.empty(E, dtype=torch.int32, device=x.device)
    cumsum_output = torch.empty(E, dtype=torch.int32, device=x.device) if do_cumsum else None
    count_cumsum_cuda(x=x, count_output=count_output, cumsum_output=cumsum_output)
    if do_cumsum:
        return count_output, cumsum_output
    return count_output
