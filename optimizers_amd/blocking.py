"""Parameter blocking: merge small dimensions, then cut into blocks of at most
`max_preconditioner_dim` per dimension.

Integer-only host logic that reproduces, index for index, what the reference gets from
`merge_small_dims` + `multi_dim_split` (utils/shampoo_utils.py:38-174) applied to
`param.view(merged_shape)` (distributor/shampoo_distributor.py:173-219): the same merged
shapes, the same blocks in the same order, described as (offset, shape, row stride)
instead of tensor views so they can go straight into the native descriptor table.
"""

from __future__ import annotations

import itertools
import math
from dataclasses import dataclass
from functools import lru_cache
from typing import Sequence


@lru_cache(maxsize=None)
def merge_small_dims(
    tensor_shape: tuple[int, ...], threshold: int | float, target_tensor_dimensionality: int | float = 1
) -> tuple[int, ...]:
    """Squeeze 1-dims, then fold dims right-to-left into their right neighbour while more dims
    remain than the target and the product does not exceed the threshold."""
    tensor_shape = tuple(int(s) for s in tensor_shape)
    if 0 in tensor_shape:
        return (0,)
    if isinstance(target_tensor_dimensionality, float):
        assert target_tensor_dimensionality == math.inf, (
            f"{target_tensor_dimensionality=} has to be an integer or math.inf."
        )
        return tensor_shape
    dims = [s for s in tensor_shape[::-1] if s != 1]
    if not dims:
        return (1,)
    merged = [dims[0]]
    for consumed in range(1, len(dims)):
        size = dims[consumed]
        dims_if_nothing_more_merges = len(merged) + len(dims) - consumed
        if dims_if_nothing_more_merges > target_tensor_dimensionality and merged[-1] * size <= threshold:
            merged[-1] *= size
        else:
            merged.append(size)
    return tuple(merged[::-1])


def chunk_bounds(extent: int, size: int | float) -> list[tuple[int, int]]:
    """[lo, hi) pieces torch.split would produce along one dim."""
    if isinstance(size, float):
        assert size == math.inf, f"{size=} has to be an integer or math.inf."
        return [(0, extent)]
    if extent == 0:
        return [(0, 0)]
    return [(lo, min(extent, lo + size)) for lo in range(0, extent, size)]


@dataclass(frozen=True)
class BlockSpec:
    """One block of one parameter, as plain integers."""

    param_index: int
    block_index: int            # index within the parameter: state key "block_<k>"
    merged_shape: tuple[int, ...]
    ranges: tuple[tuple[int, int], ...]  # [lo, hi) per merged dim
    shape: tuple[int, ...]
    offset: int                 # elements from the start of the (contiguous) parameter
    strides: tuple[int, ...]    # element strides of the block view

    @property
    def numel(self) -> int:
        return math.prod(self.shape)

    @property
    def order(self) -> int:
        return len(self.shape)

    @property
    def block_key(self) -> str:
        return f"block_{self.block_index}"


def partition_parameter(
    param_index: int,
    shape: Sequence[int],
    max_preconditioner_dim: int | float,
    target_parameter_dimensionality: int | float = 1,
) -> list[BlockSpec]:
    """All blocks of a parameter, in the reference's order (dim 0 slowest)."""
    merged = merge_small_dims(tuple(shape), max_preconditioner_dim, target_parameter_dimensionality)
    strides = [1] * len(merged)
    for d in range(len(merged) - 2, -1, -1):
        strides[d] = strides[d + 1] * merged[d + 1]
    out = []
    per_dim = [chunk_bounds(e, max_preconditioner_dim) for e in merged]
    for k, ranges in enumerate(itertools.product(*per_dim)):
        out.append(
            BlockSpec(
                param_index=param_index,
                block_index=k,
                merged_shape=merged,
                ranges=tuple(ranges),
                shape=tuple(hi - lo for lo, hi in ranges),
                offset=sum(lo * st for (lo, _), st in zip(ranges, strides)),
                strides=tuple(strides),
            )
        )
    return out
