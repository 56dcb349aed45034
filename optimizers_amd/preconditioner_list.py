"""The reference's `PreconditionerList` seam on one MI355X.

`RootInvShampooPreconditionerList` and `EigenvalueCorrectedShampooPreconditionerList` take the constructor
arguments of the reference's classes (preconditioner/shampoo_preconditioner_list.py:1240-1249, selected in
distributed_shampoo.py:659-759) and expose its three operations (preconditioner/preconditioner_list.py:49-102):

    update_preconditioners(masked_grad_list, step, perform_amortized_computation)
    precondition(masked_grad_list) -> tuple of new tensors
    compress_preconditioner_list(local_grad_selector)

Everything numerical runs in libshampoo_amd.so on the blocks' device; torch only allocates.  Limits of the native
step apply: fp32, blocks of order 0..3, packed factor matrices, integer roots for the coupled iterations.
"""

from __future__ import annotations

import ctypes
from abc import ABC, abstractmethod
from dataclasses import dataclass, field
from fractions import Fraction
from functools import partial
from typing import Any, Callable, Hashable, Mapping

import torch
from torch import Tensor

from optimizers_amd import native
from optimizers_amd.distributed_shampoo import _AmortizedComputation
from optimizers_amd.matrix_functions_types import (
    CoupledHigherOrderConfig,
    EigenConfig,
)
from optimizers_amd.shampoo_types import (
    EPSILON,
    EigendecomposedKLShampooPreconditionerConfig,
    EigendecomposedShampooPreconditionerConfig,
    EigenvalueCorrectedShampooPreconditionerConfig,
    RootInvKLShampooPreconditionerConfig,
    RootInvShampooPreconditionerConfig,
)

SHAMPOO = "shampoo"


@dataclass
class BlockInfo:
    """distributor/shampoo_block_info.py:18-65."""

    param: Tensor
    composable_block_ids: tuple[int, str]
    allocate_zeros_tensor: Callable[..., Tensor] = partial(torch.zeros)
    allocate_ones_tensor: Callable[..., Tensor] = field(init=False, default_factory=lambda: torch.ones)
    allocate_eye_tensor: Callable[..., Tensor] = field(init=False, default_factory=lambda: torch.eye)
    get_tensor: Callable[..., Tensor] = field(init=False, default_factory=lambda: lambda input_tensor: input_tensor)


class PreconditionerList(ABC):
    """preconditioner/preconditioner_list.py:49-102."""

    def __init__(self, block_list: tuple[Tensor, ...]) -> None:
        super().__init__()
        self._numel_list: tuple[int, ...] = (0,) * len(block_list)
        self._dims_list: tuple[torch.Size, ...] = tuple(block.size() for block in block_list)
        self._num_bytes_list: tuple[int, ...] = (0,) * len(block_list)

    @abstractmethod
    def update_preconditioners(self, masked_grad_list: tuple[Tensor, ...], step: Tensor, perform_amortized_computation: bool) -> None: ...

    @abstractmethod
    def precondition(self, masked_grad_list: tuple[Tensor, ...]) -> tuple[Tensor, ...]: ...

    @abstractmethod
    def compress_preconditioner_list(self, local_grad_selector: tuple[bool, ...]) -> None: ...

    @property
    def numel_list(self) -> tuple[int, ...]:
        return self._numel_list

    @property
    def dims_list(self) -> tuple[torch.Size, ...]:
        return self._dims_list

    @property
    def num_bytes_list(self) -> tuple[int, ...]:
        return self._num_bytes_list

    def numel(self) -> int:
        return sum(self._numel_list)

    def num_bytes(self) -> int:
        return sum(self._num_bytes_list)


@dataclass
class RootInvShampooKroneckerFactorsState:
    """What the reference keeps under state[param][block]["shampoo"] (shampoo_preconditioner_list.py:446-560):
    packed upper-triangular factor matrices and inverse roots."""

    factor_matrices: tuple[Tensor, ...]
    inv_factor_matrices: tuple[Tensor, ...]
    factor_matrix_indices: tuple[str, ...]
    roots: tuple[float, ...]


@dataclass
class EigenvalueCorrectedShampooKroneckerFactorsState:
    """shampoo_preconditioner_list.py:942-1055: packed factor matrices, dense eigenbases, rotated second moment."""

    factor_matrices: tuple[Tensor, ...]
    factor_matrices_eigenvectors: tuple[Tensor, ...]
    corrected_eigenvalues: Tensor
    factor_matrix_indices: tuple[str, ...]
    roots: tuple[float, ...]


@dataclass
class EigendecomposedShampooKroneckerFactorsState:
    """shampoo_preconditioner_list.py:692-760: packed factor matrices, their eigenvectors (identity at the start)
    and eigenvalues (ones at the start)."""

    factor_matrices: tuple[Tensor, ...]
    factor_matrices_eigenvectors: tuple[Tensor, ...]
    factor_matrices_eigenvalues: tuple[Tensor, ...]
    factor_matrix_indices: tuple[str, ...]
    roots: tuple[float, ...]


class _NativeShampooPreconditionerList(PreconditionerList, _AmortizedComputation):
    soap = False
    eigendecomposed = False
    kl = False

    def __init__(
        self,
        block_list: tuple[Tensor, ...],
        state: Mapping[Tensor, Any],
        block_info_list: tuple[BlockInfo, ...],
        preconditioner_config: RootInvShampooPreconditionerConfig | EigenvalueCorrectedShampooPreconditionerConfig,
        beta2: float = 1.0,
        weighting_factor: float = 1.0,
        epsilon: float = 1e-12,
        use_bias_correction: bool = True,
    ) -> None:
        super().__init__(block_list)
        self.lib = native.load()
        self.preconditioner_config = preconditioner_config
        self._beta2 = beta2
        self._weighting_factor = weighting_factor
        self._epsilon = epsilon
        self._use_bias_correction = use_bias_correction
        self._bias_correction2: Tensor = torch.tensor(1.0)
        self._check_config()
        self._blocks = tuple(block_list)
        for b in self._blocks:
            if b.device.type != "cuda" or b.dtype != torch.float32:
                raise RuntimeError(f"the native preconditioner list runs on an MI355X only: fp32 blocks on a HIP device, got {b.dtype} on {b.device}")
            if b.dim() > 3:
                raise NotImplementedError(f"blocks of order {b.dim()} are not built natively")
        self.device = self._blocks[0].device if self._blocks else torch.device("cuda:0")
        acc = preconditioner_config.amortized_computation_config
        self.use_eigh = isinstance(acc, EigenConfig) or self.eigendecomposed
        self.eigenvalue_tensors: list[Tensor] = []
        self._private_inverses: list[tuple[Tensor, ...]] = []
        self.use_higher_order = isinstance(acc, CoupledHigherOrderConfig)
        self.max_jacobi_sweeps = 30
        self.bad_root_blocks: dict[int, str] = {}
        self.failed_counter: dict[int, int] = {}
        self.factor_names: list[str] = []
        self.factor_block: list[int] = []
        self.factor_roots: list[float] = []
        self._selectors = tuple(self._create_preconditioned_dims_selector(dims) for dims in self._dims_list)
        self._local = tuple(True for _ in self._blocks)  # blocks that the next masked lists hold
        self._states: list[Any] = []
        numel, nbytes = [], []
        for k, (block, info, selector) in enumerate(zip(self._blocks, block_info_list, self._selectors, strict=True)):
            param_index, block_index = info.composable_block_ids
            assert block_index in state[info.param], f"{block_index=} not found in {state[info.param]=}."
            block_state = state[info.param][block_index]
            roots = tuple(
                1 / self._get_inverse_exponent(dimension=d, order=len(selector)) for d, on in enumerate(selector) if on
            )
            dims = tuple(n for n, on in zip(block.shape, selector) if on)
            names = tuple(f"{param_index}.{block_index}.{j}" for j in range(len(dims)))
            zeros = partial(info.allocate_zeros_tensor, dtype=torch.float32, device=block.device)
            factors = tuple(info.get_tensor(zeros(size=(n * (n + 1) // 2,))) for n in dims)
            if self.soap and not dims:
                raise NotImplementedError(
                    f"block {names or (param_index, block_index)} has no preconditioned dim: the eigenvalue-corrected "
                    "list would precondition it in the standard basis, which this seam does not build "
                    "(optimizers_amd.DistributedShampoo does)"
                )
            if self.soap:
                bases = tuple(info.get_tensor(zeros(size=(n, n))) for n in dims)
                for q in bases:
                    q.copy_(torch.eye(q.shape[0], device=q.device))
                corrected = info.get_tensor(zeros(size=tuple(block.shape)))
                st = EigenvalueCorrectedShampooKroneckerFactorsState(factors, bases, corrected, names, roots)
                count = sum(f.numel() for f in factors) + sum(q.numel() for q in bases) + corrected.numel()
            elif self.eigendecomposed:
                bases = tuple(info.get_tensor(zeros(size=(n, n))) for n in dims)
                for q in bases:
                    q.copy_(torch.eye(q.shape[0], device=q.device))
                values = tuple(info.get_tensor(zeros(size=(n,))).fill_(1.0) for n in dims)
                self.eigenvalue_tensors.extend(values)
                # Q diag(w) Q^T, a function of the state, kept outside of it
                inverses = tuple(torch.zeros(n * (n + 1) // 2, dtype=torch.float32, device=block.device) for n in dims)
                for inv, n in zip(inverses, dims):
                    idx = torch.arange(n, device=inv.device)
                    inv[idx * n - idx * (idx - 1) // 2] = 1.0
                self._private_inverses.append(inverses)
                st = EigendecomposedShampooKroneckerFactorsState(factors, bases, values, names, roots)
                count = sum(f.numel() for f in factors) + sum(q.numel() for q in bases) + sum(v.numel() for v in values)
            else:
                inverses = tuple(info.get_tensor(zeros(size=(n * (n + 1) // 2,))) for n in dims)
                for inv, n in zip(inverses, dims):
                    idx = torch.arange(n, device=inv.device)
                    inv[idx * n - idx * (idx - 1) // 2] = 1.0  # packed identity
                st = RootInvShampooKroneckerFactorsState(factors, inverses, names, roots)
                count = sum(f.numel() for f in factors) + sum(f.numel() for f in inverses)
            if not self.eigendecomposed:
                self._private_inverses.append(())
            block_state[SHAMPOO] = st
            self._states.append(st)
            numel.append(count)
            nbytes.append(4 * count)
            for j, r in enumerate(roots):
                self.factor_names.append(names[j])
                self.factor_block.append(k)
                self.factor_roots.append(float(r))
                if not (self.use_eigh or self.soap) and Fraction(r).denominator != 1:
                    if self.use_higher_order:
                        raise NotImplementedError(f"CoupledHigherOrderConfig with a fractional root ({Fraction(r)}) is not built natively")
                    self.bad_root_blocks[k] = f"{Fraction(r).denominator=} must be equal to 1 to use coupled inverse Newton iteration!"
        self._numel_list = tuple(numel)
        self._num_bytes_list = tuple(nbytes)
        self.n_factors = len(self.factor_names)
        self.iterations = (ctypes.c_int32 * max(self.n_factors, 1))()
        self.status = (ctypes.c_int32 * max(self.n_factors, 1))()
        self.eigenvalue_ptrs = (ctypes.c_void_p * max(self.n_factors, 1))(*(t.data_ptr() for t in self.eigenvalue_tensors))
        self.plan = ctypes.c_void_p()
        self._plan_strides: tuple[int, ...] | None = None
        self._workspace: Tensor | None = None
        self._scalars = native.StepScalars()
        self._scalars.bias_correction1 = 1.0
        self._scalars.graft_type = native.SA_GRAFT_NONE
        self._scalars.graft_bias_correction2 = 1.0

    # ---- configuration --------------------------------------------------------------------------------------
    @abstractmethod
    def _check_config(self) -> None: ...

    @abstractmethod
    def _get_inverse_exponent(self, dimension: int, order: int) -> float: ...

    def _create_preconditioned_dims_selector(self, dims: torch.Size) -> tuple[bool, ...]:
        return tuple(self._get_inverse_exponent(dimension=d, order=len(dims)) != 0.0 for d in range(len(dims)))

    # ---- plan -----------------------------------------------------------------------------------------------
    def _destroy_plan(self) -> None:
        if getattr(self, "plan", None):
            self.lib.sa_plan_destroy(self.plan)
            self.plan = ctypes.c_void_p()

    def __del__(self) -> None:
        self._destroy_plan()

    @staticmethod
    def _row_stride(t: Tensor) -> tuple[int, ...]:
        """Strides the plan needs: (row stride,) of a matrix, (dim-0 stride, dim-1 stride) of an order-3 block."""
        if t.dim() < 2:
            return (1,)
        if t.dim() == 2:
            return (max(int(t.stride(0)), int(t.shape[1])),)
        inner = max(int(t.stride(1)), int(t.shape[2]))
        return (max(int(t.stride(0)), inner * int(t.shape[1])), inner)

    def _ensure_plan(self, strides: tuple[tuple[int, ...], ...]) -> None:
        """(Re)creates the plan when the row strides of the gradient blocks differ from the ones it was built for."""
        if self.plan and strides == self._plan_strides:
            return
        self._destroy_plan()
        nb = len(self._blocks)
        if nb == 0:
            return
        descs = (native.BlockDesc * nb)()
        for k, (block, st, selector) in enumerate(zip(self._blocks, self._states, self._selectors)):
            d = descs[k]
            if block.dim() == 3:
                d.rows, d.cols, d.ld = block.shape[0] * block.shape[1], block.shape[2], strides[k][1]
                d.mid, d.ld_outer = block.shape[1], strides[k][0]
            elif block.dim() == 2:
                d.rows, d.cols, d.ld = block.shape[0], block.shape[1], strides[k][0]
            else:
                d.rows, d.cols, d.ld = max(block.numel(), 1), 1, 1
            d.param = block.data_ptr()  # never written: only the factor update and the preconditioning run on this plan
            slot = 0
            for dim, on in enumerate(selector):
                if not on:
                    continue
                d.factor[dim] = st.factor_matrices[slot].data_ptr()
                root = Fraction(st.roots[slot])
                d.root[dim] = int(root.numerator) if root.denominator == 1 else max(int(round(st.roots[slot])), 1)
                if self.soap or self.eigendecomposed:
                    d.eigenvectors[dim] = st.factor_matrices_eigenvectors[slot].data_ptr()
                if self.eigendecomposed:
                    d.inv_factor[dim] = self._private_inverses[k][slot].data_ptr()
                elif not self.soap:
                    d.inv_factor[dim] = st.inv_factor_matrices[slot].data_ptr()
                slot += 1
            if self.soap:
                d.corrected_eigenvalues = st.corrected_eigenvalues.data_ptr()
        self._descs = descs
        native.check(self.lib.sa_plan_create(descs, nb, ctypes.byref(self.plan)), "sa_plan_create")
        need = int(self.lib.sa_plan_workspace_bytes(self.plan))
        if self._workspace is None or self._workspace.numel() < need:
            self._workspace = torch.empty(need, dtype=torch.uint8, device=self.device)
        native.check(self.lib.sa_plan_bind_workspace(self.plan, self._workspace.data_ptr(), need), "sa_plan_bind_workspace")
        assert int(self.lib.sa_plan_num_factors(self.plan)) == self.n_factors
        pc = self.preconditioner_config
        if pc.use_trace_scaling:
            native.check(self.lib.sa_plan_set_trace_scaling(self.plan, 1, pc.trace_scaling_exponent, self._epsilon), "sa_plan_set_trace_scaling")
        if self.kl:
            native.check(self.lib.sa_plan_set_kl_shampoo(self.plan, 1), "sa_plan_set_kl_shampoo")
        self._plan_strides = strides

    def _bind(self, masked_grad_list: tuple[Tensor, ...]) -> int:
        selected = [k for k, on in enumerate(self._local) if on]
        if len(masked_grad_list) != len(selected):
            raise ValueError(f"expected {len(selected)} gradient blocks after compress_preconditioner_list, got {len(masked_grad_list)}")
        strides = list(self._plan_strides) if self._plan_strides else [self._row_stride(b) for b in self._blocks]
        for k, g in zip(selected, masked_grad_list):
            if g.shape != self._blocks[k].shape:
                raise ValueError(f"gradient block {k} has shape {tuple(g.shape)}, the parameter block {tuple(self._blocks[k].shape)}")
            if g.dtype != torch.float32 or g.device != self.device:
                raise NotImplementedError("gradients must be fp32 on the blocks' device")
            if g.dim() >= 2 and g.stride(-1) != 1 and g.shape[-1] > 1:
                raise NotImplementedError("gradient blocks must have unit stride in their last dim")
            strides[k] = self._row_stride(g)
        self._ensure_plan(tuple(strides))
        ptrs = (ctypes.c_void_p * max(len(self._blocks), 1))()
        for k, g in zip(selected, masked_grad_list):
            ptrs[k] = g.data_ptr()
        self._grads_alive = masked_grad_list
        stream = native.current_stream_ptr(self.device)
        native.check(self.lib.sa_plan_bind_gradients(self.plan, ptrs, stream), "sa_plan_bind_gradients")
        return stream

    # ---- the three operations -------------------------------------------------------------------------------
    def update_preconditioners(self, masked_grad_list: tuple[Tensor, ...], step: Tensor, perform_amortized_computation: bool) -> None:
        """shampoo_preconditioner_list.py:1392-1430 (+ :1891-1912 for the eigenvalue-corrected list)."""
        if not self._blocks:
            return
        stream = self._bind(masked_grad_list)
        pc = self.preconditioner_config
        native.check(self.lib.sa_update_factor_matrices(self.plan, self._beta2, self._weighting_factor, stream), "sa_update_factor_matrices")
        if self._use_bias_correction and self._beta2 < 1.0 and not pc.drop_weighting_factor_on_gsquare:
            self._bias_correction2 = torch.tensor(1.0) - self._beta2**step
        if perform_amortized_computation:
            self._amortized_computation({EPSILON: self._epsilon}, float(self._bias_correction2), stream)
        if self.soap:
            native.check(
                self.lib.sa_update_corrected_eigenvalues(self.plan, self._beta2, self._weighting_factor, stream),
                "sa_update_corrected_eigenvalues",
            )
        self._grads_alive = None

    def precondition(self, masked_grad_list: tuple[Tensor, ...]) -> tuple[Tensor, ...]:
        """shampoo_preconditioner_list.py:1672-1695 / :1914-1942: new tensors, shapes of the inputs."""
        if not self._blocks:
            return ()
        stream = self._bind(masked_grad_list)
        if self.soap:
            native.check(
                self.lib.sa_precondition_eigenvalue_corrected(
                    self.plan, ctypes.byref(self._scalars), float(self._bias_correction2), self._epsilon, self._soap_root, stream
                ),
                "sa_precondition_eigenvalue_corrected",
            )
        else:
            native.check(self.lib.sa_precondition(self.plan, ctypes.byref(self._scalars), stream), "sa_precondition")
        out = []
        for k, g in zip((k for k, on in enumerate(self._local) if on), masked_grad_list):
            p = torch.empty(g.shape, dtype=torch.float32, device=self.device)
            native.check(self.lib.sa_plan_read_preconditioned(self.plan, k, p.data_ptr(), stream), "sa_plan_read_preconditioned")
            out.append(p)
        self._grads_alive = None
        return tuple(out)

    def compress_preconditioner_list(self, local_grad_selector: tuple[bool, ...]) -> None:
        """shampoo_preconditioner_list.py:1580-1620: the next masked lists hold the selected blocks only."""
        if len(local_grad_selector) != len(self._blocks):
            raise ValueError(f"selector of {len(local_grad_selector)} entries for {len(self._blocks)} blocks")
        self._local = tuple(bool(x) for x in local_grad_selector)


class RootInvShampooPreconditionerList(_NativeShampooPreconditionerList):
    """Root-inverse Shampoo (shampoo_preconditioner_list.py:1697-1790)."""

    soap = False

    def _check_config(self) -> None:
        from optimizers_amd.distributed_shampoo import _NativeGroup

        if not isinstance(self.preconditioner_config, RootInvShampooPreconditionerConfig):
            raise NotImplementedError(f"{self.preconditioner_config=} not supported!")
        _NativeGroup._check_supported({"distributed_config": _single_device(), "iterate_averaging_config": None}, self.preconditioner_config)

    def _get_inverse_exponent(self, dimension: int, order: int) -> float:
        override = self.preconditioner_config.inverse_exponent_override.get(order, {})
        if isinstance(override, dict):
            return override.get(dimension, 1 / (2 * max(order, 1)))
        return override


class EigenvalueCorrectedShampooPreconditionerList(_NativeShampooPreconditionerList):
    """Eigenvalue-corrected Shampoo / SOAP (shampoo_preconditioner_list.py:1793-1990)."""

    soap = True

    def _check_config(self) -> None:
        from optimizers_amd.distributed_shampoo import _NativeGroup

        pc = self.preconditioner_config
        if not isinstance(pc, EigenvalueCorrectedShampooPreconditionerConfig):
            raise NotImplementedError(f"{pc=} not supported!")
        _NativeGroup._check_supported({"distributed_config": _single_device(), "iterate_averaging_config": None}, pc)
        orders = {len(d) for d in self._dims_list if len(d) > 0}
        roots = {1 / pc.inverse_exponent_override.get(o, 1 / 2) for o in orders} or {2.0}
        if len(roots) > 1:
            raise NotImplementedError("different eigenvalue exponents per tensor order are not built natively")
        self._soap_root = float(roots.pop())

    def _get_inverse_exponent(self, dimension: int, order: int) -> float:
        return self.preconditioner_config.inverse_exponent_override.get(order, 1 / 2)

    def _create_preconditioned_dims_selector(self, dims: torch.Size) -> tuple[bool, ...]:
        ignored = self.preconditioner_config.ignored_basis_change_dims.get(len(dims), [])
        return tuple(d not in ignored for d in range(len(dims)))


class EigendecomposedShampooPreconditionerList(_NativeShampooPreconditionerList):
    """Eigendecomposed Shampoo (shampoo_preconditioner_list.py:1793-1832): Q diag(lambda^(-1/root)) Q^T from the stored
    eigendecomposition of every factor."""

    eigendecomposed = True

    def _check_config(self) -> None:
        from optimizers_amd.distributed_shampoo import _NativeGroup

        if not isinstance(self.preconditioner_config, EigendecomposedShampooPreconditionerConfig):
            raise NotImplementedError(f"{self.preconditioner_config=} not supported!")
        _NativeGroup._check_supported({"distributed_config": _single_device(), "iterate_averaging_config": None}, self.preconditioner_config)

    _get_inverse_exponent = RootInvShampooPreconditionerList._get_inverse_exponent


class RootInvKLShampooPreconditionerList(RootInvShampooPreconditionerList):
    """Root-inverse KL-Shampoo (shampoo_preconditioner_list.py:1945-1987)."""

    kl = True

    def _check_config(self) -> None:
        if not isinstance(self.preconditioner_config, RootInvKLShampooPreconditionerConfig):
            raise NotImplementedError(f"{self.preconditioner_config=} not supported!")
        super()._check_config()


class EigendecomposedKLShampooPreconditionerList(EigendecomposedShampooPreconditionerList):
    """Eigendecomposed KL-Shampoo (shampoo_preconditioner_list.py:1989-2046)."""

    kl = True

    def _check_config(self) -> None:
        if not isinstance(self.preconditioner_config, EigendecomposedKLShampooPreconditionerConfig):
            raise NotImplementedError(f"{self.preconditioner_config=} not supported!")
        super()._check_config()


def _single_device():
    from optimizers_amd.shampoo_types import DefaultSingleDeviceDistributedConfig

    return DefaultSingleDeviceDistributedConfig
