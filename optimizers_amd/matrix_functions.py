"""`matrix_inverse_root` and `matrix_eigendecomposition` on one MI355X.

Same names, arguments, defaults and error behaviour as the reference's module-level functions
(distributed_shampoo/preconditioner/matrix_functions.py:282-304 / :663-695 and :698-908), which its
preconditioner lists look up by name.  Each call runs the library's batched solver on a plan that holds
the one matrix as the single factor of a 1-D block; plans are cached per (order, kind, root, device).

Differences from the reference, all at rounding level or documented limits:
 * input and output are fp32 tensors on a HIP device (there is no CPU path);
 * `matrix_inverse_root` returns the mirrored upper triangle of the solver's result, which is what the
   optimizer stores (shampoo_preconditioner_list.py:678);
 * `CoupledNewtonConfig` / `CoupledHigherOrderConfig` take integer roots whose power chain has at most five
   products (every root up to 14, and 16), the higher-order iteration no fractional roots;
 * `eigendecomposition_offload_device` must be "" and `retry_double_precision` is not needed (the solvers
   do not fail on finite input);
 * a non-finite input or result comes back as a matrix of NaN, where the reference's LAPACK call would raise.
"""

from __future__ import annotations

import ctypes
import logging
from collections import OrderedDict
from fractions import Fraction

import torch
from torch import Tensor

from optimizers_amd import native
from optimizers_amd.matrix_functions_types import (
    CoupledHigherOrderConfig,
    CoupledNewtonConfig,
    DefaultEigenConfig,
    DefaultEigendecompositionConfig,
    EigenConfig,
    EigendecompositionConfig,
    EighEigendecompositionConfig,
    PerturbationConfig,
    PseudoInverseConfig,
    QREigendecompositionConfig,
    RootInvConfig,
)

logger: logging.Logger = logging.getLogger(__name__)

_MAX_SWEEPS = 30
_PLAN_CACHE_SIZE = 8
_plans: "OrderedDict[tuple, _FactorPlan]" = OrderedDict()


class _FactorPlan:
    """One factor matrix of order d as the only factor of a 1-D block of d elements."""

    def __init__(self, d: int, device: torch.device, eigenbasis: bool, root: int) -> None:
        self.lib = native.load()
        self.d = d
        self.param = torch.zeros(d, device=device)
        self.grad = torch.zeros(d, device=device)
        self.factor = torch.zeros(d * (d + 1) // 2, device=device)
        self.triu = torch.triu_indices(d, d, device=device)
        self.descs = (native.BlockDesc * 1)()
        b = self.descs[0]
        b.rows, b.cols, b.ld = d, 1, 1
        b.param = self.param.data_ptr()
        b.factor[0] = self.factor.data_ptr()
        if eigenbasis:
            self.basis = torch.eye(d, device=device)
            self.corrected = torch.zeros(d, device=device)
            self.eigenvalues = torch.zeros(d, device=device)
            b.eigenvectors[0] = self.basis.data_ptr()
            b.corrected_eigenvalues = self.corrected.data_ptr()
            b.root[0] = 1
        else:
            self.inverse = torch.zeros(d * (d + 1) // 2, device=device)
            b.inv_factor[0] = self.inverse.data_ptr()
            b.root[0] = root
        self.plan = ctypes.c_void_p()
        native.check(self.lib.sa_plan_create(self.descs, 1, ctypes.byref(self.plan)), "sa_plan_create")
        need = int(self.lib.sa_plan_workspace_bytes(self.plan))
        self.workspace = torch.empty(need, dtype=torch.uint8, device=device)
        native.check(self.lib.sa_plan_bind_workspace(self.plan, self.workspace.data_ptr(), need), "sa_plan_bind_workspace")
        self.grad_ptrs = (ctypes.c_void_p * 1)(self.grad.data_ptr())
        self.iterations = (ctypes.c_int32 * 1)()
        self.status = (ctypes.c_int32 * 1)()

    def load(self, A: Tensor, stream: int) -> None:
        self.factor.copy_(A[self.triu[0], self.triu[1]])
        native.check(self.lib.sa_plan_bind_gradients(self.plan, self.grad_ptrs, stream), "sa_plan_bind_gradients")

    def unpacked_inverse(self) -> Tensor:
        out = torch.empty(self.d, self.d, device=self.inverse.device)
        out[self.triu[0], self.triu[1]] = self.inverse
        out[self.triu[1], self.triu[0]] = self.inverse
        return out

    def __del__(self) -> None:
        if getattr(self, "plan", None):
            self.lib.sa_plan_destroy(self.plan)
            self.plan = ctypes.c_void_p()


def _plan_for(A: Tensor, eigenbasis: bool, root: int) -> _FactorPlan:
    key = (A.shape[0], eigenbasis, root, A.device)
    plan = _plans.pop(key, None)
    if plan is None:
        plan = _FactorPlan(A.shape[0], A.device, eigenbasis, root)
    _plans[key] = plan
    while len(_plans) > _PLAN_CACHE_SIZE:
        _plans.popitem(last=False)
    return plan


def _check_square_matrix(A: Tensor) -> None:
    """matrix_functions.py:89-139."""
    if len(A.shape) != 2:
        raise ValueError(f"Matrix is not 2-dimensional! {A.shape=}")
    if A.shape[0] != A.shape[1]:
        raise ValueError(f"Matrix is not square! {A.shape=}")


def _check_device(A: Tensor) -> None:
    if A.device.type != "cuda" or A.dtype != torch.float32:
        raise RuntimeError(
            f"optimizers_amd.matrix_functions runs on an MI355X only: fp32 tensors on a HIP device, got {A.dtype} on {A.device}."
        )


def _nan_like(A: Tensor) -> Tensor:
    return torch.full_like(A, float("nan"))


def matrix_inverse_root(
    A: Tensor,
    root: Fraction,
    root_inv_config: RootInvConfig = DefaultEigenConfig,
    epsilon: float = 0.0,
) -> Tensor:
    """Inverse root A^(-1/root) of a symmetric positive (semi-)definite matrix (matrix_functions.py:282-304,
    :663-695)."""
    _check_square_matrix(A)
    if not isinstance(root_inv_config, (EigenConfig, CoupledNewtonConfig, CoupledHigherOrderConfig)):
        raise NotImplementedError(
            f"Root inverse config is not implemented! Specified root inverse config is {root_inv_config=}."
        )
    _check_device(A)
    stream = native.current_stream_ptr(A.device)
    lib = native.load()
    if isinstance(root_inv_config, EigenConfig):
        if root <= 0:
            raise ValueError(f"Root {root} should be positive!")
        stability = root_inv_config.rank_deficient_stability_config
        if isinstance(stability, PseudoInverseConfig):
            if epsilon != 0.0:
                raise ValueError(f"{epsilon=} should be 0.0 when using pseudo-inverse!")
            mode, rtol, atol = 2, (-1.0 if stability.rank_rtol is None else float(stability.rank_rtol)), float(stability.rank_atol)
        elif isinstance(stability, PerturbationConfig):
            mode, rtol, atol = int(stability.perturb_before_computation), 0.0, 0.0
        else:
            raise NotImplementedError(f"rank_deficient_stability_config={stability} is not supported.")
        if root_inv_config.eigendecomposition_offload_device != "":
            raise NotImplementedError("eigendecomposition_offload_device: the decomposition runs on the MI355X")
        plan = _plan_for(A, False, 1)
        plan.load(A, stream)
        roots = (ctypes.c_float * 1)(float(root))
        native.check(
            lib.sa_compute_root_inverses_eigh(
                plan.plan, 1.0, epsilon, roots, mode, rtol, atol, _MAX_SWEEPS, plan.iterations, plan.status, stream
            ),
            "sa_compute_root_inverses_eigh",
        )
    elif isinstance(root_inv_config, CoupledNewtonConfig):
        if root.denominator != 1:
            raise ValueError(f"{root.denominator=} must be equal to 1 to use coupled inverse Newton iteration!")
        plan = _plan_for(A, False, int(root.numerator))
        plan.load(A, stream)
        native.check(
            lib.sa_compute_root_inverses_newton(
                plan.plan, 1.0, epsilon, root_inv_config.max_iterations, root_inv_config.tolerance,
                plan.iterations, plan.status, stream,
            ),
            "sa_compute_root_inverses_newton",
        )
        if int(plan.status[0]) == native.SA_FACTOR_NOT_CONVERGED:
            logger.warning("Newton did not converge and reached maximum number of iterations!")
    else:
        if root.denominator != 1:
            raise NotImplementedError(f"CoupledHigherOrderConfig with a fractional root ({root}) is not built natively")
        plan = _plan_for(A, False, int(root.numerator))
        plan.load(A, stream)
        native.check(
            lib.sa_compute_root_inverses_higher_order(
                plan.plan, 1.0, root_inv_config.rel_epsilon, root_inv_config.abs_epsilon, root_inv_config.max_iterations,
                root_inv_config.tolerance, root_inv_config.order, plan.iterations, plan.status, stream,
            ),
            "sa_compute_root_inverses_higher_order",
        )
        if int(plan.status[0]) == native.SA_FACTOR_SOLVER_FAILED:
            raise ArithmeticError(
                "Error in matrix inverse root exceeds threshold 1e-1 or the result holds NaN/Inf, raising an exception!"
            )
        if int(plan.status[0]) == native.SA_FACTOR_NOT_CONVERGED:
            logger.warning("Higher order method did not converge and reached maximum number of iterations!")
    if int(plan.status[0]) in (native.SA_FACTOR_INPUT_NONFINITE, native.SA_FACTOR_RESULT_NONFINITE):
        return _nan_like(A)
    return plan.unpacked_inverse()


def matrix_eigendecomposition(
    A: Tensor,
    epsilon: float = 0.0,
    eigendecomposition_config: EigendecompositionConfig = DefaultEigendecompositionConfig,
    eigenvectors_estimate: Tensor | None = None,
) -> tuple[Tensor, Tensor]:
    """Eigenvalues (ascending for a fresh decomposition) and eigenvectors (columns) of a symmetric matrix
    (matrix_functions.py:698-908)."""
    _check_square_matrix(A)
    stability = eigendecomposition_config.rank_deficient_stability_config
    if isinstance(stability, PseudoInverseConfig) and epsilon != 0.0:
        raise ValueError(f"{epsilon=} should be 0.0 when using pseudo-inverse!")
    ridge = epsilon * float(getattr(stability, "perturb_before_computation", 0))
    if isinstance(eigendecomposition_config, EighEigendecompositionConfig):
        if eigendecomposition_config.tolerance != 0.0 and eigenvectors_estimate is None:
            raise ValueError(
                "eigenvectors_estimate should be passed to matrix_eigendecomposition when using tolerance != 0.0."
            )
        if eigendecomposition_config.eigendecomposition_offload_device != "":
            raise NotImplementedError("eigendecomposition_offload_device: the decomposition runs on the MI355X")
    elif isinstance(eigendecomposition_config, QREigendecompositionConfig):
        assert eigenvectors_estimate is not None, "eigenvectors_estimate should not be None when QR algorithm is used."
    else:
        raise NotImplementedError(
            f"Eigendecomposition config is not implemented! Specified eigendecomposition config is {type(eigendecomposition_config).__name__}."
        )
    _check_device(A)
    stream = native.current_stream_ptr(A.device)
    lib = native.load()
    plan = _plan_for(A, True, 1)
    plan.load(A, stream)
    if eigenvectors_estimate is not None:
        plan.basis.copy_(eigenvectors_estimate)
    if isinstance(eigendecomposition_config, EighEigendecompositionConfig):
        native.check(
            lib.sa_refresh_eigenbases_eigh(
                plan.plan, 1.0, ridge, eigendecomposition_config.tolerance, _MAX_SWEEPS, plan.iterations, plan.status, stream
            ),
            "sa_refresh_eigenbases_eigh",
        )
    else:
        native.check(
            lib.sa_refresh_eigenbases_qr(
                plan.plan, 1.0, ridge, eigendecomposition_config.max_iterations, eigendecomposition_config.tolerance,
                plan.iterations, plan.status, stream,
            ),
            "sa_refresh_eigenbases_qr",
        )
    if int(plan.status[0]) in (native.SA_FACTOR_INPUT_NONFINITE, native.SA_FACTOR_RESULT_NONFINITE):
        return torch.full((A.shape[0],), float("nan"), device=A.device), _nan_like(A)
    native.check(lib.sa_plan_read_eigenvalues(plan.plan, 0, plan.eigenvalues.data_ptr(), stream), "sa_plan_read_eigenvalues")
    return plan.eigenvalues.clone(), plan.basis.clone()
