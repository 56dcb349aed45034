"""The reference's distributor seam on the MI355X: `DistributorInterface` and the default single-device
`Distributor` (distributor/shampoo_distributor.py:34-430), the class `_select_distributor_class`
(distributed_shampoo.py:595-644) returns for `SingleDeviceDistributedConfig`.

Same constructor (`param_group`, `runtime_config`), same properties (`local_grad_selector`,
`local_blocked_params`, `local_masked_blocked_params`, `local_block_info_list`), same
`merge_and_block_gradients()` / `update_params()`.  Blocks are views of the parameters and gradients (no copies),
cut by the integer partition of `optimizers_amd.blocking`; the parameter update is one native call
(`sa_add_to_views`) on the current HIP stream.  There is no CPU path for `update_params`.
"""

from __future__ import annotations

from abc import ABC, abstractmethod
from typing import Any, Iterable

import torch
from torch import Tensor

from . import native
from .blocking import BlockSpec, partition_parameter
from .preconditioner_list import BlockInfo
from .shampoo_types import DISTRIBUTED_CONFIG, MAX_PRECONDITIONER_DIM, PARAMS, ShampooRuntimeConfig


def _block_views(tensor: Tensor, specs: list[BlockSpec]) -> list[Tensor]:
    """The blocks of `tensor.view(merged_shape)` the reference obtains with `multi_dim_split`
    (utils/shampoo_utils.py:124-174), as views."""
    merged = tensor.detach().view(specs[0].merged_shape)
    strides = merged.stride()
    return [
        torch.as_strided(
            merged,
            spec.shape,
            strides,
            merged.storage_offset() + sum(lo * st for (lo, _), st in zip(spec.ranges, strides)),
        )
        for spec in specs
    ]


class DistributorInterface(ABC):
    """distributor/shampoo_distributor.py:34-299."""

    def __init__(self, param_group: dict[str, Any], runtime_config: ShampooRuntimeConfig | None = None) -> None:
        self._param_group = param_group
        self._runtime_config: ShampooRuntimeConfig = runtime_config if runtime_config is not None else ShampooRuntimeConfig()
        self._merge_and_block_parameters()
        self._global_grad_selector: tuple[bool, ...] = (True,) * len(self._global_blocked_params)
        self._previous_global_grad_selector: tuple[bool, ...] | None = None
        self._distributor_selector: tuple[bool, ...]
        self._local_grad_selector: tuple[bool, ...]
        self._local_blocked_params: tuple[Tensor, ...]
        self._local_masked_blocked_params: tuple[Tensor, ...]
        self._local_block_info_list: tuple[BlockInfo, ...]

    @abstractmethod
    def update_params(self, blocked_search_directions: tuple[Tensor, ...], use_masked_tensors: bool = True) -> None: ...

    @abstractmethod
    def merge_and_block_gradients(self) -> tuple[Tensor, ...]: ...

    @property
    def local_grad_selector(self) -> tuple[bool, ...]:
        return self._local_grad_selector

    @property
    def local_blocked_params(self) -> tuple[Tensor, ...]:
        return self._local_blocked_params

    @property
    def local_masked_blocked_params(self) -> tuple[Tensor, ...]:
        return self._local_masked_blocked_params

    @property
    def local_block_info_list(self) -> tuple[BlockInfo, ...]:
        return self._local_block_info_list

    def _construct_composable_block_ids(self, param_index: int, block_index: int, rank: int | None = None) -> tuple[int, str]:
        """(param_index, "block_k"), or (param_index, "rank_r-block_k") when a rank is given (:93-135)."""
        name = f"block_{block_index}"
        return (param_index, name if rank is None else f"rank_{rank}-{name}")

    def _get_params_or_grads(self, get_grad: bool = False) -> Iterable[Tensor | None]:
        params = self._param_group[PARAMS]
        return (p.grad for p in params) if get_grad else params

    def _partition(self, param_index: int, shape: torch.Size) -> list[BlockSpec]:
        return partition_parameter(
            param_index,
            tuple(shape),
            self._param_group[MAX_PRECONDITIONER_DIM],
            self._param_group[DISTRIBUTED_CONFIG].target_parameter_dimensionality,
        )

    @torch.no_grad()
    def _merge_and_block_parameters(self) -> None:
        self._specs_per_param: list[list[BlockSpec]] = []
        blocked: list[Tensor] = []
        for index, param in enumerate(self._get_params_or_grads()):
            specs = self._partition(index, param.size())
            self._specs_per_param.append(specs)
            blocked.extend(_block_views(param, specs))
        self._global_blocked_params: tuple[Tensor, ...] = tuple(blocked)
        self._global_num_blocks_per_param: tuple[int, ...] = tuple(len(s) for s in self._specs_per_param)

    @torch.no_grad()
    def _merge_and_block_gradients(self) -> tuple[Tensor, ...]:
        """Blocks of every gradient that exists; None and empty gradients keep their blocks but are masked out
        of every update (:229-299)."""
        blocks: list[Tensor] = []
        selector: list[bool] = []
        first = 0
        for grad, specs in zip(self._get_params_or_grads(get_grad=True), self._specs_per_param, strict=True):
            mine = self._distributor_selector[first : first + len(specs)]
            first += len(specs)
            invalid = grad is None or grad.numel() == 0
            selector.extend([not invalid] * len(specs))
            if invalid or not any(mine):
                continue
            if self._runtime_config.eager_nan_check:
                assert torch.isfinite(grad).all(), (
                    f"Encountered gradient containing NaN/Inf in parameter with shape {grad.shape}. "
                    "Check your model for numerical instability or consider gradient clipping."
                )
            blocks.extend(view for view, keep in zip(_block_views(grad, specs), mine) if keep)
        self._global_grad_selector = tuple(selector)
        return tuple(blocks)


class Distributor(DistributorInterface):
    """Default distributor: every block is local, nothing is communicated (:302-430)."""

    def __init__(self, param_group: dict[str, Any], runtime_config: ShampooRuntimeConfig | None = None) -> None:
        super().__init__(param_group, runtime_config)
        self._local_grad_selector = (True,) * len(self._global_blocked_params)
        self._distributor_selector = self._local_grad_selector
        self._local_blocked_params = self._global_blocked_params
        self._local_masked_blocked_params = self._local_blocked_params
        self._local_block_info_list = tuple(
            BlockInfo(param=param, composable_block_ids=self._construct_composable_block_ids(spec.param_index, spec.block_index))
            for param, specs in zip(self._get_params_or_grads(), self._specs_per_param, strict=True)
            for spec in specs
        )

    @torch.no_grad()
    def update_params(self, blocked_search_directions: tuple[Tensor, ...], use_masked_tensors: bool = True) -> None:
        targets = self._local_masked_blocked_params if use_masked_tensors else self._local_blocked_params
        assert len(blocked_search_directions) == len(targets), (
            f"Expected {len(blocked_search_directions)=} to be equal to {len(targets)=}."
        )
        if not blocked_search_directions:
            return
        device = targets[0].device
        n = len(targets)
        dst, src = (native.View * n)(), (native.View * n)()
        for i, (target, direction) in enumerate(zip(targets, blocked_search_directions, strict=True)):
            if target.device.type != "cuda" or direction.device != target.device or target.device != device:
                raise ValueError(f"update_params: block {i} must live on one HIP device, got {target.device} and {direction.device}")
            if target.dtype != torch.float32 or direction.dtype != torch.float32:
                raise ValueError(f"update_params: block {i} must be float32, got {target.dtype} and {direction.dtype}")
            if target.shape != direction.shape:
                raise ValueError(f"update_params: block {i} has shape {tuple(target.shape)}, its direction {tuple(direction.shape)}")
            native.fill_view(dst[i], target)
            native.fill_view(src[i], direction)
        with torch.cuda.device(device):
            native.check(native.load().sa_add_to_views(dst, src, n, native.current_stream_ptr(device)), "sa_add_to_views")

    def merge_and_block_gradients(self) -> tuple[Tensor, ...]:
        """Must be called in the step after the gradients have been written; refreshes the selectors when the
        set of parameters with a gradient changed (:404-430)."""
        local_masked_blocked_grads = self._merge_and_block_gradients()
        if self._previous_global_grad_selector != self._global_grad_selector:
            self._previous_global_grad_selector = self._global_grad_selector
            self._local_grad_selector = tuple(
                g for g, mine in zip(self._global_grad_selector, self._distributor_selector) if mine
            )
            self._local_masked_blocked_params = tuple(
                p for p, keep in zip(self._local_blocked_params, self._local_grad_selector) if keep
            )
        return local_masked_blocked_grads
