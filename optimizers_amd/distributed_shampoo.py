"""DistributedShampoo for one MI355X: the reference's constructor and `step()` surface over
the native gfx950 kernels.

Drop-in for `distributed_shampoo.DistributedShampoo` (reference
distributed_shampoo/distributed_shampoo.py:361-382 ctor, :1677-1711 step) on the
single-device distributor.  The Python here is host logic only: hyper-parameter checks,
block partition, state allocation, the step schedule and error mapping.  Every tensor
operation of the step runs in libshampoo_amd.so (hand-written HIP); there is no torch or
CPU fallback for it, and construction fails if the library or a GPU is missing.
"""

from __future__ import annotations

import ctypes
import logging
import math
import os
from contextlib import nullcontext
from fractions import Fraction
from typing import Any, Callable

import torch

from optimizers_amd import native
from optimizers_amd.blocking import BlockSpec, partition_parameter
from optimizers_amd.matrix_functions_types import (
    CoupledHigherOrderConfig,
    CoupledNewtonConfig,
    EigenConfig,
    EigendecompositionConfig,
    EighEigendecompositionConfig,
    PerturbationConfig,
    PseudoInverseConfig,
    QREigendecompositionConfig,
)
from optimizers_amd.shampoo_types import (
    ADAGRAD,
    BETA3,
    BETAS,
    DISTRIBUTED_CONFIG,
    EPSILON,
    FILTERED_GRAD,
    GRAFTING_CONFIG,
    ITERATE_AVERAGING_CONFIG,
    LR,
    MAX_PRECONDITIONER_DIM,
    MOMENTUM_BUFFER,
    PARAMS,
    PEAK_LR,
    PRECONDITION_FREQUENCY,
    PRECONDITIONER_CONFIG,
    SHAMPOO,
    START_PRECONDITIONING_STEP,
    STEP,
    USE_BIAS_CORRECTION,
    USE_PIN_MEMORY,
    WEIGHT_DECAY,
    WEIGHT_DECAY_TYPE,
    AdaGradPreconditionerConfig,
    AdamPreconditionerConfig,
    BaseShampooPreconditionerConfig,
    ClassicMomentumConfig,
    GeneralizedPrimalAveragingConfig,
    LR_SUM,
    ScheduleFreeConfig,
    TRAIN_MODE,
    WEIGHT_BUFFER,
    ConcurrencyConfig,
    DefaultConcurrencyConfig,
    DefaultShampooConfig,
    DefaultShampooRuntimeConfig,
    DefaultSingleDeviceDistributedConfig,
    DistributedConfig,
    EigendecomposedKLShampooPreconditionerConfig,
    EigendecomposedShampooPreconditionerConfig,
    EigenvalueCorrectedShampooPreconditionerConfig,
    IterateAveragingConfig,
    PreconditionerConfig,
    PreconditionerValueError,
    RMSpropPreconditionerConfig,
    RootInvKLShampooPreconditionerConfig,
    RootInvShampooPreconditionerConfig,
    SGDPreconditionerConfig,
    ShampooRuntimeConfig,
    SingleDeviceDistributedConfig,
    WeightDecayType,
)

logger: logging.Logger = logging.getLogger(__name__)

_ALIGN = 64  # floats: every state tensor starts on a 256-byte boundary of its arena


def _round_up(x: int, a: int) -> int:
    return (x + a - 1) // a * a


class _Arena:
    """One flat device buffer (fp32 unless stated) handing out aligned views (state tensors stay ordinary torch
    tensors, so checkpoints see the same objects the kernels update)."""

    def __init__(self, sizes: list[int], device: torch.device, dtype: torch.dtype = torch.float32) -> None:
        self.offsets = []
        total = 0
        for n in sizes:
            self.offsets.append(total)
            total += _round_up(max(n, 1), _ALIGN)
        self.buffer = torch.zeros(max(total, _ALIGN), dtype=dtype, device=device)

    def view(self, i: int, shape: tuple[int, ...]) -> torch.Tensor:
        n = math.prod(shape)
        return self.buffer[self.offsets[i] : self.offsets[i] + n].view(shape)


def _save_matrix_for_debugging(name: str, factor: torch.Tensor, bc2: float) -> None:
    """The reference keeps the bias-corrected factor matrix of a failed computation in /tmp/<index>.pt
    (shampoo_preconditioner_list.py:1596-1646); `factor` is the stored factor, a packed upper triangle or d x d."""
    from pathlib import Path

    try:
        m = factor.detach()
        if m.dim() == 1:
            n = int((math.isqrt(8 * m.numel() + 1) - 1) // 2)
            iu = torch.triu_indices(n, n, device=m.device)
            full = torch.zeros(n, n, dtype=m.dtype, device=m.device)
            full[iu[0], iu[1]] = m
            m = full + torch.triu(full, 1).T
        file_path = Path("/tmp").resolve() / f"{name.replace('.', '_')}.pt"
        torch.save((m / bc2).cpu(), file_path)
        logger.info(f"Matrix has been saved to {file_path} for debugging.")
    except Exception as e:  # the dump is a debugging aid; it must not hide the error it accompanies
        logger.warning(f"Failed to save matrix of factor {name}: {e}")


class _AmortizedComputation:
    """Batched amortized computation of one plan with the reference's error semantics.  Needs the attributes
    lib, plan, preconditioner_config, soap, use_eigh, use_higher_order, n_factors, factor_names, factor_block,
    factor_roots, iterations, status, max_jacobi_sweeps, bad_root_blocks, failed_counter."""

    def _amortized_computation(self, group: dict[str, Any], bc2: float, stream: int) -> None:
        """Batched inverse roots + the reference's error semantics
        (shampoo_preconditioner_list.py:314-443)."""
        pc = self.preconditioner_config
        cfg = pc.amortized_computation_config
        refreshes_basis = self.soap or getattr(self, "eigendecomposed", False)
        if getattr(self, "factor_f64", False) and isinstance(cfg, CoupledNewtonConfig):
            # float64 factor matrices: the reference's coupled Newton iteration on a float64 matrix
            native.check(
                self.lib.sa_compute_root_inverses_newton_f64(
                    self.plan, bc2, group[EPSILON], cfg.max_iterations, cfg.tolerance, 0, self.iterations, self.status, stream
                ),
                "sa_compute_root_inverses_newton_f64",
            )
        elif getattr(self, "factor_f64", False) and not refreshes_basis:
            # float64 factor matrices with EigenConfig: eigendecomposition and inverse root in double precision
            roots = (ctypes.c_float * max(self.n_factors, 1))(*self.factor_roots)
            stab = cfg.rank_deficient_stability_config
            if isinstance(stab, PseudoInverseConfig):
                mode, rtol, atol = 2, (-1.0 if stab.rank_rtol is None else float(stab.rank_rtol)), float(stab.rank_atol)
            else:
                mode, rtol, atol = int(stab.perturb_before_computation), 0.0, 0.0
            native.check(
                self.lib.sa_compute_root_inverses_eigh_f64(
                    self.plan, bc2, group[EPSILON], roots, mode, rtol, atol, self.max_jacobi_sweeps, self.iterations,
                    self.status, stream,
                ),
                "sa_compute_root_inverses_eigh_f64",
            )
        elif refreshes_basis and isinstance(cfg, EighEigendecompositionConfig):
            # epsilon * I is added only when the config perturbs before the computation (matrix_functions.py:869-882)
            ridge = group[EPSILON] * float(cfg.rank_deficient_stability_config.perturb_before_computation)
            native.check(
                self.lib.sa_refresh_eigenbases_eigh(
                    self.plan, bc2, ridge, cfg.tolerance, self.max_jacobi_sweeps, self.iterations, self.status, stream
                ),
                "sa_refresh_eigenbases_eigh",
            )
        elif refreshes_basis:
            ridge = group[EPSILON] * float(getattr(cfg.rank_deficient_stability_config, "perturb_before_computation", False))
            native.check(
                self.lib.sa_refresh_eigenbases_qr(
                    self.plan, bc2, ridge, cfg.max_iterations, cfg.tolerance, self.iterations, self.status, stream
                ),
                "sa_refresh_eigenbases_qr",
            )
        elif self.use_eigh:
            roots = (ctypes.c_float * max(self.n_factors, 1))(*self.factor_roots)
            stab = cfg.rank_deficient_stability_config
            if isinstance(stab, PseudoInverseConfig):
                # rank_rtol=None is the reference's "order * machine epsilon" (matrix_functions.py:226-229)
                mode, rtol, atol = 2, (-1.0 if stab.rank_rtol is None else float(stab.rank_rtol)), float(stab.rank_atol)
            else:
                mode, rtol, atol = int(stab.perturb_before_computation), 0.0, 0.0
            native.check(
                self.lib.sa_compute_root_inverses_eigh(
                    self.plan, bc2, group[EPSILON], roots, mode, rtol, atol, self.max_jacobi_sweeps,
                    self.iterations, self.status, stream,
                ),
                "sa_compute_root_inverses_eigh",
            )
        elif self.use_higher_order:
            native.check(
                self.lib.sa_compute_root_inverses_higher_order(
                    self.plan, bc2, cfg.rel_epsilon, cfg.abs_epsilon, cfg.max_iterations, cfg.tolerance, cfg.order,
                    self.iterations, self.status, stream,
                ),
                "sa_compute_root_inverses_higher_order",
            )
        else:
            native.check(
                self.lib.sa_compute_root_inverses_newton(
                    self.plan, bc2, group[EPSILON], cfg.max_iterations, cfg.tolerance, self.iterations, self.status, stream
                ),
                "sa_compute_root_inverses_newton",
            )
        self.last_newton_iterations = [int(self.iterations[i]) for i in range(self.n_factors)]
        for i in range(self.n_factors):
            st = int(self.status[i])
            name = self.factor_names[i]
            if st == native.SA_FACTOR_INPUT_NONFINITE:
                raise PreconditionerValueError(
                    f"Encountered nan/inf values in factor matrix {name}! "
                    "To mitigate, check if nan inputs are being passed into the network or nan gradients are being passed to the optimizer. "
                    "Otherwise, in some cases, this may be due to divergence of the algorithm. To mitigate, try decreasing the learning rate or increasing grafting epsilon."
                )
            if st == native.SA_FACTOR_RESULT_NONFINITE:
                self._dump_factor(i, bc2)
                raise PreconditionerValueError(
                    f"Encountered nan or inf values in name of factor matrix {name}! "
                    "To mitigate, check factor matrix before the matrix computation."
                )
            if st == native.SA_FACTOR_NOT_CONVERGED:
                if refreshes_basis:
                    pass
                elif self.use_higher_order:
                    logger.warning("Higher order method did not converge and reached maximum number of iterations!")
                elif self.use_eigh:
                    logger.warning(f"Eigensolver did not converge for factor matrix {name} ({self.max_jacobi_sweeps} Jacobi sweeps, or 30 QL sweeps per eigenvalue).")
                else:
                    logger.warning("Newton did not converge and reached maximum number of iterations!")
        # a solver failure keeps the block's previous inverse and is tolerated a limited number of consecutive times
        # (shampoo_preconditioner_list.py:388-443)
        failed_now = {self.factor_block[i] for i in range(self.n_factors) if int(self.status[i]) == native.SA_FACTOR_SOLVER_FAILED}
        computed_now = {self.factor_block[i] for i in range(self.n_factors) if int(self.status[i]) != native.SA_FACTOR_SKIPPED}
        for k in computed_now - failed_now - set(self.bad_root_blocks):
            self.failed_counter[k] = 0
        for k in sorted(failed_now):
            count = self.failed_counter.get(k, 0) + 1
            self.failed_counter[k] = count
            names = tuple(n for n, b in zip(self.factor_names, self.factor_block) if b == k)
            for i in range(self.n_factors):
                if self.factor_block[i] == k and int(self.status[i]) == native.SA_FACTOR_SOLVER_FAILED:
                    self._dump_factor(i, bc2)
            logger.warning(f"Matrix computation failed for factor matrices {names}. Using previous preconditioner and continuing...")
            if count > pc.num_tolerated_failed_amortized_computations:
                raise ValueError(
                    f"The number of failed amortized computations for factors {names} exceeded the allowed tolerance. "
                    "The last seen exception was an ArithmeticError of the coupled higher-order iteration."
                )
        if getattr(self, "eigendecomposed", False):
            # the eigenvalues of every factor that was decomposed go into the state; the inverse roots
            # Q diag(w) Q^T follow from the stored (Q, lambda) of all active factors
            for i in range(self.n_factors):
                if int(self.status[i]) in (native.SA_FACTOR_OK, native.SA_FACTOR_NOT_CONVERGED):
                    native.check(
                        self.lib.sa_plan_read_eigenvalues(self.plan, i, self.eigenvalue_tensors[i].data_ptr(), stream),
                        "sa_plan_read_eigenvalues",
                    )
            self._inverse_roots_from_eigendecomposition(group, stream)
        # blocks whose root cannot be used by the coupled Newton iteration fail every time
        for k, message in self.bad_root_blocks.items():
            count = self.failed_counter.get(k, 0) + 1
            self.failed_counter[k] = count
            logger.warning(f"Matrix computation failed with exception={message!r}. Using previous preconditioner and continuing...")
            if count > pc.num_tolerated_failed_amortized_computations:
                names = tuple(n for n, b in zip(self.factor_names, self.factor_block) if b == k)
                raise ValueError(
                    f"The number of failed amortized computations for factors {names} exceeded the allowed tolerance. "
                    f"The last seen exception was {message}."
                )


    def _dump_factor(self, i: int, bc2: float) -> None:
        tensors = getattr(self, "factor_tensors", None)
        if tensors is not None and i < len(tensors):
            _save_matrix_for_debugging(self.factor_names[i], tensors[i], bc2)

    def _inverse_roots_from_eigendecomposition(self, group: dict[str, Any], stream: int) -> None:
        """Eigendecomposed Shampoo: X = Q diag(w(lambda)) Q^T of every active factor
        (matrix_functions.py:179-279 as called from shampoo_preconditioner_list.py:1793-1832)."""
        stab = self.preconditioner_config.amortized_computation_config.rank_deficient_stability_config
        if isinstance(stab, PseudoInverseConfig):
            mode, rtol, atol = 2, (-1.0 if stab.rank_rtol is None else float(stab.rank_rtol)), float(stab.rank_atol)
        else:
            mode, rtol, atol = int(stab.perturb_before_computation), 0.0, 0.0
        roots = (ctypes.c_float * max(self.n_factors, 1))(*self.factor_roots)
        status = (ctypes.c_int32 * max(self.n_factors, 1))()
        native.check(
            self.lib.sa_compute_root_inverses_from_eigendecomposition(
                self.plan, self.eigenvalue_ptrs, group[EPSILON], roots, mode, rtol, atol, status, stream
            ),
            "sa_compute_root_inverses_from_eigendecomposition",
        )
        for i in range(self.n_factors):
            if int(status[i]) == native.SA_FACTOR_RESULT_NONFINITE:
                raise PreconditionerValueError(
                    f"Encountered nan or inf values in the inverse root formed from the eigendecomposition of factor matrix "
                    f"{self.factor_names[i]}! To mitigate, check the stored eigenvalues (non-positive after the epsilon shift?)."
                )


class _NativeGroup(_AmortizedComputation):
    """Native state and schedule of one parameter group (reference: the per-group state lists
    built in distributed_shampoo.py:563-975 plus `_group_step_body` :1562-1667)."""

    # Eigenvalue-corrected Shampoo: one library call updates the second moment in the eigenbasis and preconditions, reusing
    # the rotated gradient for both.  False = the two separate calls of the reference's order (same results up to rounding).
    fuse_eigenbasis_rotations = True

    # Upper bound, in bytes, of the scratch region of the amortized computations (root inverses, eigenbasis refreshes):
    # the factors of a group are solved in waves that fit it together (sa_plan_set_scratch_budget), so the workspace of
    # a group with many factors stays bounded; results do not depend on it.  One Llama-3-8B layer with blocks of 2048
    # needs 14.6 GB for all its 112 factors at once and stays one wave.  None = no limit.  The environment variable
    # SHAMPOO_AMD_SCRATCH_BYTES overrides it.
    scratch_budget_bytes: int | None = 32 << 30

    # Coupled Newton: a batch whose stages are launches of fewer 128 x 128 tiles than this iterates as two halves side by
    # side on two streams (sa_plan_set_newton_split_tiles; same bits either way).  None = the library's default (0 = never;
    # the halves measured slower than the whole batch on the GPT-2 parameter set).  The environment variable SHAMPOO_AMD_NEWTON_SPLIT_TILES overrides it.
    newton_split_tiles: int | None = None

    def __init__(self, optimizer: "DistributedShampoo", group: dict[str, Any], group_index: int) -> None:
        self.lib = native.load()
        self.group_index = group_index
        params: list[torch.Tensor] = group[PARAMS]
        if not params:
            raise ValueError(f"Shampoo got an empty parameter {group=}")
        self.params = params
        self.device = params[0].device
        if self.device.type != "cuda":
            raise RuntimeError(
                "optimizers_amd.DistributedShampoo runs on an MI355X only: parameters must live on a "
                f"HIP device, got {self.device}. There is no CPU path."
            )
        for p in params:
            if p.device != self.device:
                raise ValueError("all parameters of a group must live on the same device")
            if p.dtype != torch.float32:
                raise NotImplementedError(f"only fp32 parameters are supported, got {p.dtype}")
            if not p.is_contiguous():
                raise ValueError("parameters must be contiguous (the reference views them with merged shapes)")

        pc = group[PRECONDITIONER_CONFIG]
        # An element-wise method as the preconditioner itself (SGD / AdaGrad / RMSprop / Adam configs,
        # distributed_shampoo.py:673-714: the reference then runs its AdagradPreconditionerList, or nothing for SGD, in
        # place of a Shampoo list): the same arithmetic as grafting with that method before
        # start_preconditioning_step, so every step takes the fused grafting-only kernel and no block has factors.
        self.elementwise_only = isinstance(
            pc, (SGDPreconditionerConfig, AdaGradPreconditionerConfig, RMSpropPreconditionerConfig, AdamPreconditionerConfig)
        )
        self.elementwise_config = pc if self.elementwise_only else None
        if self.elementwise_only:
            if group[GRAFTING_CONFIG] is not None:
                raise NotImplementedError("grafting on top of an element-wise preconditioner_config is not built natively")
            pc = RootInvShampooPreconditionerConfig(inverse_exponent_override={1: 0.0, 2: 0.0, 3: 0.0})
        self._check_supported(group, pc)
        self.preconditioner_config = pc
        dist: DistributedConfig = group[DISTRIBUTED_CONFIG]
        self.block_specs: list[BlockSpec] = []
        self.num_blocks_per_param: list[int] = []
        for i, p in enumerate(params):
            specs = partition_parameter(
                i, tuple(p.shape), group[MAX_PRECONDITIONER_DIM], dist.target_parameter_dimensionality
            )
            self.num_blocks_per_param.append(len(specs))
            self.block_specs.extend(specs)
        for s in self.block_specs:
            if s.order > 3:
                raise NotImplementedError(
                    f"block of order {s.order} (shape {s.shape}): the native step covers blocks of order 1 to 3"
                )

        # native blocks = blocks with at least one element
        self.native_index = [i for i, s in enumerate(self.block_specs) if s.numel > 0]
        nb = len(self.native_index)
        beta1 = group[BETAS][0]
        graft = self.elementwise_config if self.elementwise_only else group[GRAFTING_CONFIG]
        self.graft_type, self.graft_beta2, self.graft_weight, self.graft_bias, self.graft_eps = self._graft_setup(graft)
        momentum_cfg = group[ITERATE_AVERAGING_CONFIG]

        # which dims carry a Kronecker factor, and with which root
        self.selectors: list[tuple[bool, ...]] = []
        self.roots: list[tuple[float, ...]] = []
        self.soap = isinstance(pc, EigenvalueCorrectedShampooPreconditionerConfig)
        self.eigendecomposed = isinstance(pc, EigendecomposedShampooPreconditionerConfig)
        self.kl = isinstance(pc, (RootInvKLShampooPreconditionerConfig, EigendecomposedKLShampooPreconditionerConfig))
        for i in self.native_index:
            order = self.block_specs[i].order
            if self.soap:
                # shampoo_preconditioner_list.py:1843-1865: one root for the corrected eigenvalues
                ignored = pc.ignored_basis_change_dims.get(order, [])
                sel = tuple(d not in ignored for d in range(order))
                self.selectors.append(sel)
                self.roots.append((1 / pc.inverse_exponent_override.get(order, 1 / 2),) * sum(sel))
            else:
                exps = [self._inverse_exponent(pc, d, order) for d in range(order)]
                self.selectors.append(tuple(e != 0.0 for e in exps))
                self.roots.append(tuple(1 / e for e in exps if e != 0.0))
        if self.soap:
            distinct = {1 / pc.inverse_exponent_override.get(self.block_specs[i].order, 1 / 2) for i in self.native_index}
            if len(distinct) > 1:
                raise NotImplementedError("different eigenvalue exponents per tensor order are not built natively")
            self.soap_root = distinct.pop() if distinct else 2.0

        numels = [self.block_specs[i].numel for i in self.native_index]
        fdims: list[int] = []
        for k, i in enumerate(self.native_index):
            s = self.block_specs[i]
            fdims.extend(s.shape[d] for d in range(s.order) if self.selectors[k][d])
        packed = [d * (d + 1) // 2 for d in fdims]
        self.factor_f64 = pc.factor_matrix_dtype == torch.float64
        self.factor_arena = _Arena(packed, self.device, pc.factor_matrix_dtype)
        self.inv_arena = _Arena(packed, self.device) if not self.soap else None
        # use_symmetric_packing=False (shampoo_preconditioner_list.py:139-156): the state shows dense d x d matrices; the
        # kernels keep working on the packed triangles above, which then are private, and the dense tensors are
        # rewritten from them after every factor update / amortized computation (sa_plan_export_dense_state)
        self.dense_state = not pc.use_symmetric_packing
        self.dense_factor_arena = _Arena([d * d for d in fdims], self.device, pc.factor_matrix_dtype) if self.dense_state else None
        self.dense_inv_arena = (
            _Arena([d * d for d in fdims], self.device) if (self.dense_state and not self.soap and not self.eigendecomposed) else None
        )
        self.dense_factor_ptrs = (ctypes.c_void_p * max(len(fdims), 1))()
        self.dense_inv_ptrs = (ctypes.c_void_p * max(len(fdims), 1))()
        self.eigvec_arena = _Arena([d * d for d in fdims], self.device) if (self.soap or self.eigendecomposed) else None
        self.eigenvalue_arena = _Arena(list(fdims), self.device) if self.eigendecomposed else None
        self.eigenvalue_tensors: list[torch.Tensor] = []
        self.corrected_arena = _Arena(numels, self.device) if self.soap else None
        self.filtered_arena = _Arena(numels, self.device) if beta1 != 0.0 else None
        self.adagrad_arena = _Arena(numels, self.device) if self.graft_type == native.SA_GRAFT_ADAGRAD else None
        self.momentum_arena = _Arena(numels, self.device) if isinstance(momentum_cfg, ClassicMomentumConfig) else None
        self.primal_averaging = isinstance(momentum_cfg, (GeneralizedPrimalAveragingConfig, ScheduleFreeConfig))
        self.weight_arena = _Arena(numels, self.device) if self.primal_averaging else None

        # optimizer.state layout (reference golden: tests/distributed_shampoo_test.py:516-622)
        descs = (native.BlockDesc * max(nb, 1))()
        self.factor_names: list[str] = []
        self.factor_block: list[int] = []
        self.factor_roots: list[float] = []
        self.factor_tensors: list[torch.Tensor] = []  # the state's factor matrices, in plan order
        self.use_eigh = isinstance(pc.amortized_computation_config, EigenConfig) or self.eigendecomposed
        self.use_higher_order = isinstance(pc.amortized_computation_config, CoupledHigherOrderConfig)
        self._slots: list[tuple[torch.Tensor, str, tuple, torch.Tensor]] = []
        self.bad_root_blocks: dict[int, str] = {}
        self.failed_counter: dict[int, int] = {}
        fi = 0
        for k, i in enumerate(self.native_index):
            s = self.block_specs[i]
            p = params[s.param_index]
            block_state: dict[str, Any] = optimizer.state[p].setdefault(s.block_key, {})
            d = descs[k]
            if s.order == 1:
                d.rows, d.cols, d.ld = s.shape[0], 1, 1
            elif s.order == 2:
                d.rows, d.cols, d.ld = s.shape[0], s.shape[1], s.strides[0]
            else:  # d0 x d1 x d2 flattened to (d0 d1) x d2
                d.rows, d.cols, d.ld = s.shape[0] * s.shape[1], s.shape[2], s.strides[1]
                d.mid, d.ld_outer = s.shape[1], s.strides[0]
            d.param = p.data_ptr() + 4 * s.offset
            shampoo_state: dict[str, Any] = (
                {"factor_matrices": {}, "factor_matrices_eigenvectors": {}}
                if self.soap
                else {"factor_matrices": {}, "factor_matrices_eigenvectors": {}, "factor_matrices_eigenvalues": {}}
                if self.eigendecomposed
                else {"factor_matrices": {}, "inv_factor_matrices": {}}
            )
            if self.soap:
                shampoo_state["corrected_eigenvalues"] = self.corrected_arena.view(k, s.shape)
                d.corrected_eigenvalues = shampoo_state["corrected_eigenvalues"].data_ptr()
                self._slots.append((p, s.block_key, (SHAMPOO, "corrected_eigenvalues"), shampoo_state["corrected_eigenvalues"]))
            if self.soap and not any(self.selectors[k]):
                # every basis change ignored: the block is preconditioned in the standard basis (this is Adam /
                # RMSprop on the block, shampoo_eigenvalue_correction_test.py:60-272); the native step rotates
                # by one identity matrix on the smaller dim, which is exact
                dim = min(range(s.order), key=lambda t: s.shape[t])
                d.eigenvectors[dim] = self._identity(s.shape[dim]).data_ptr()
            slot = 0
            for dim in range(s.order):
                if not self.selectors[k][dim]:
                    continue
                n = s.shape[dim]
                f = self.factor_arena.view(fi, (n * (n + 1) // 2,))
                d.factor[dim] = f.data_ptr()
                if self.dense_state:
                    f = self.dense_factor_arena.view(fi, (n, n))
                    self.dense_factor_ptrs[fi] = f.data_ptr()
                shampoo_state["factor_matrices"][slot] = f
                self.factor_tensors.append(f)
                self._slots.append((p, s.block_key, (SHAMPOO, "factor_matrices", slot), f))
                if self.soap or self.eigendecomposed:
                    q = self.eigvec_arena.view(fi, (n, n))
                    q.copy_(torch.eye(n, device=self.device))
                    shampoo_state["factor_matrices_eigenvectors"][slot] = q
                    d.eigenvectors[dim] = q.data_ptr()
                    self._slots.append((p, s.block_key, (SHAMPOO, "factor_matrices_eigenvectors", slot), q))
                if self.eigendecomposed:
                    # eigenvalues start at one, eigenvectors at the identity (shampoo_preconditioner_list.py:730-750)
                    lam = self.eigenvalue_arena.view(fi, (n,))
                    lam.fill_(1.0)
                    shampoo_state["factor_matrices_eigenvalues"][slot] = lam
                    self.eigenvalue_tensors.append(lam)
                    self._slots.append((p, s.block_key, (SHAMPOO, "factor_matrices_eigenvalues", slot), lam))
                if not self.soap:
                    inv = self.inv_arena.view(fi, (n * (n + 1) // 2,))
                    idx = torch.arange(n, device=self.device)
                    inv[idx * n - idx * (idx - 1) // 2] = 1.0  # packed identity
                    d.inv_factor[dim] = inv.data_ptr()
                    if self.dense_inv_arena is not None:
                        inv = self.dense_inv_arena.view(fi, (n, n))
                        inv.copy_(torch.eye(n, device=self.device))
                        self.dense_inv_ptrs[fi] = inv.data_ptr()
                    if not self.eigendecomposed:  # eigendecomposed Shampoo keeps Q diag(w) Q^T as a private cache
                        shampoo_state["inv_factor_matrices"][slot] = inv
                        self._slots.append((p, s.block_key, (SHAMPOO, "inv_factor_matrices", slot), inv))
                root = Fraction(self.roots[k][slot])
                self.factor_roots.append(float(self.roots[k][slot]))
                if self.factor_f64 and root.denominator != 1 and not self.use_eigh:
                    raise NotImplementedError(
                        f"factor_matrix_dtype=float64 with a fractional root ({root}) needs EigenConfig"
                    )
                if self.use_eigh or self.soap:
                    d.root[dim] = max(int(round(self.roots[k][slot])), 1)  # unused by the eigh paths
                elif root.denominator != 1 and self.use_higher_order:
                    raise NotImplementedError(
                        f"CoupledHigherOrderConfig with a fractional root ({root}) is not built natively"
                    )
                elif root.denominator != 1:
                    # the reference raises inside matrix_inverse_root at every amortized step and
                    # tolerates it num_tolerated_failed_amortized_computations times
                    self.bad_root_blocks[k] = (
                        f"{root.denominator=} must be equal to 1 to use coupled inverse Newton iteration!"
                    )
                    d.root[dim] = 1
                else:
                    d.root[dim] = int(root.numerator)
                self.factor_names.append(f"{s.param_index}.{s.block_key}.{slot}")
                self.factor_block.append(k)
                slot += 1
                fi += 1
            block_state[SHAMPOO] = shampoo_state
            if self.adagrad_arena is not None:
                block_state[ADAGRAD] = self.adagrad_arena.view(k, s.shape)
                d.adagrad = block_state[ADAGRAD].data_ptr()
                self._slots.append((p, s.block_key, (ADAGRAD,), block_state[ADAGRAD]))
            if self.filtered_arena is not None:
                block_state[FILTERED_GRAD] = self.filtered_arena.view(k, s.shape)
                d.filtered_grad = block_state[FILTERED_GRAD].data_ptr()
                self._slots.append((p, s.block_key, (FILTERED_GRAD,), block_state[FILTERED_GRAD]))
            if self.momentum_arena is not None:
                block_state[MOMENTUM_BUFFER] = self.momentum_arena.view(k, s.shape)
                d.momentum_buffer = block_state[MOMENTUM_BUFFER].data_ptr()
                self._slots.append((p, s.block_key, (MOMENTUM_BUFFER,), block_state[MOMENTUM_BUFFER]))
            if self.weight_arena is not None:
                # the "z" sequence starts at the current parameters (distributed_shampoo.py:909-922)
                z = self.weight_arena.view(k, s.shape)
                z.copy_(torch.as_strided(p.detach(), s.shape, s.strides, p.storage_offset() + s.offset))
                block_state[WEIGHT_BUFFER] = z
                d.weight_buffer = z.data_ptr()
                self._slots.append((p, s.block_key, (WEIGHT_BUFFER,), z))
            logger.info(
                f"Instantiated Shampoo Preconditioner {s.param_index}.{s.block_key} for Parameter {s.param_index} "
                f"({tuple(p.shape)}), Block {s.block_key} ({s.shape})."
            )
        # empty blocks still own a (state-less) entry, as in the reference
        for i, s in enumerate(self.block_specs):
            optimizer.state[params[s.param_index]].setdefault(s.block_key, {})

        self.descs = descs
        self.n_native = nb
        self._param_ptrs = [p.data_ptr() for p in params]
        self.plan = ctypes.c_void_p()
        self.workspace = None
        if nb:
            native.check(self.lib.sa_plan_create(descs, nb, ctypes.byref(self.plan)), "sa_plan_create")
            if self.factor_f64:
                native.check(self.lib.sa_plan_set_factor_dtype(self.plan, 64), "sa_plan_set_factor_dtype")
            budget = os.environ.get("SHAMPOO_AMD_SCRATCH_BYTES", self.scratch_budget_bytes)
            if budget is not None and int(budget) > 0:
                native.check(self.lib.sa_plan_set_scratch_budget(self.plan, int(budget)), "sa_plan_set_scratch_budget")
            need = int(self.lib.sa_plan_workspace_bytes(self.plan))
            self.workspace = torch.empty(need, dtype=torch.uint8, device=self.device)
            native.check(
                self.lib.sa_plan_bind_workspace(self.plan, self.workspace.data_ptr(), need), "sa_plan_bind_workspace"
            )
            self.n_factors = int(self.lib.sa_plan_num_factors(self.plan))
            assert self.n_factors == len(self.factor_names)
            if pc.use_trace_scaling:
                native.check(
                    self.lib.sa_plan_set_trace_scaling(self.plan, 1, pc.trace_scaling_exponent, group[EPSILON]),
                    "sa_plan_set_trace_scaling",
                )
            lanes = os.environ.get("SHAMPOO_AMD_TRIDIAGONAL_LANES")
            if lanes is not None:
                native.check(self.lib.sa_plan_set_tridiagonal_lanes(self.plan, int(lanes)), "sa_plan_set_tridiagonal_lanes")
            split = os.environ.get("SHAMPOO_AMD_NEWTON_SPLIT_TILES", self.newton_split_tiles)
            if split is not None:
                native.check(self.lib.sa_plan_set_newton_split_tiles(self.plan, int(split)), "sa_plan_set_newton_split_tiles")
            if self.kl:
                try:
                    native.check(self.lib.sa_plan_set_kl_shampoo(self.plan, 1), "sa_plan_set_kl_shampoo")
                except native.NativeError as e:
                    raise NotImplementedError(f"KL-Shampoo: {e}") from e
        else:
            self.n_factors = 0
        self.iterations = (ctypes.c_int32 * max(self.n_factors, 1))()
        self.status = (ctypes.c_int32 * max(self.n_factors, 1))()
        self.eigenvalue_ptrs = (ctypes.c_void_p * max(self.n_factors, 1))(*(t.data_ptr() for t in self.eigenvalue_tensors))
        self.inverse_roots_stale = False  # set when (Q, lambda) were written from outside (checkpoint load)
        self.grad_ptrs = (ctypes.c_void_p * max(nb, 1))()
        self.last_newton_iterations: list[int] = []
        self.max_jacobi_sweeps = 30

        # one CPU step counter per group, aliased under every parameter (distributed_shampoo.py:790-815)
        self.step_tensor = torch.tensor(0, dtype=torch.int64, device="cpu")
        for p in params:
            optimizer.state[p][STEP] = self.step_tensor
        if self.primal_averaging:
            # per-group scalars aliased under every parameter (distributed_shampoo.py:924-937)
            self.lr_sum = torch.tensor(0.0, dtype=torch.float, device=self.device)
            self._lr_sum_host = torch.tensor(0.0, dtype=torch.float)
            self.train_mode = torch.tensor(True, dtype=torch.bool, device="cpu")
            for p in params:
                optimizer.state[p][TRAIN_MODE] = self.train_mode
                optimizer.state[p][LR_SUM] = self.lr_sum
        self.stream: torch.cuda.Stream | None = None

    def _identity(self, n: int) -> torch.Tensor:
        cache = self.__dict__.setdefault("_identities", {})
        if n not in cache:
            cache[n] = torch.eye(n, device=self.device, dtype=torch.float32)
        return cache[n]

    def close(self) -> None:
        if self.plan:
            self.lib.sa_plan_destroy(self.plan)
            self.plan = ctypes.c_void_p()

    # -- configuration helpers ---------------------------------------------------------------

    @staticmethod
    def _check_supported(group: dict[str, Any], pc: PreconditionerConfig) -> None:
        if not isinstance(group[DISTRIBUTED_CONFIG], SingleDeviceDistributedConfig):
            raise NotImplementedError(f"{group[DISTRIBUTED_CONFIG]=} not supported!")
        if not isinstance(
            pc,
            (RootInvShampooPreconditionerConfig, EigenvalueCorrectedShampooPreconditionerConfig, EigendecomposedShampooPreconditionerConfig),
        ):
            raise NotImplementedError(f"{pc=} not supported!")
        acc = pc.amortized_computation_config
        if isinstance(pc, EigendecomposedShampooPreconditionerConfig):
            if not isinstance(acc, (QREigendecompositionConfig, EighEigendecompositionConfig)):
                raise NotImplementedError(
                    f"Eigendecomposition config is not implemented! Specified eigendecomposition config is {type(acc).__name__}."
                )
            if not isinstance(acc.rank_deficient_stability_config, (PerturbationConfig, PseudoInverseConfig)):
                raise NotImplementedError(f"{acc.rank_deficient_stability_config=} is not supported.")
            if isinstance(acc, EighEigendecompositionConfig) and acc.eigendecomposition_offload_device != "":
                raise NotImplementedError("eigendecomposition_offload_device: the decomposition runs on the MI355X")
            if pc.factor_matrix_eigenvectors_dtype != torch.float32 or pc.factor_matrix_eigenvalues_dtype != torch.float32:
                raise NotImplementedError("eigenvectors and eigenvalues are fp32 in the native step")
        elif isinstance(pc, EigenvalueCorrectedShampooPreconditionerConfig):
            if not isinstance(acc, (QREigendecompositionConfig, EighEigendecompositionConfig)):
                raise NotImplementedError(
                    f"Eigendecomposition config is not implemented! Specified eigendecomposition config is {type(acc).__name__}."
                )
            if not isinstance(acc.rank_deficient_stability_config, PerturbationConfig):
                raise NotImplementedError(f"{acc.rank_deficient_stability_config=} is not supported.")
            if isinstance(acc, EighEigendecompositionConfig) and acc.eigendecomposition_offload_device != "":
                raise NotImplementedError("eigendecomposition_offload_device: the decomposition runs on the MI355X")
            if pc.factor_matrix_eigenvectors_dtype != torch.float32 or pc.corrected_eigenvalues_dtype != torch.float32:
                raise NotImplementedError("eigenvectors and corrected eigenvalues are fp32 in the native step")
        elif isinstance(acc, EigenConfig):
            if not isinstance(acc.rank_deficient_stability_config, (PerturbationConfig, PseudoInverseConfig)):
                raise NotImplementedError(f"{acc.rank_deficient_stability_config=} is not supported.")
            if acc.eigendecomposition_offload_device != "":
                raise NotImplementedError("eigendecomposition_offload_device: the decomposition runs on the MI355X")
        elif isinstance(acc, CoupledHigherOrderConfig):
            if not 2 <= acc.order <= 8:
                raise NotImplementedError(f"CoupledHigherOrderConfig: orders 2..8 are built, got {acc.order=}")
        elif not isinstance(acc, CoupledNewtonConfig):
            raise NotImplementedError(
                f"Root inverse config is not implemented! Specified root inverse config is {acc=}."
            )
        if getattr(pc, "inv_factor_matrix_dtype", torch.float32) != torch.float32:
            raise NotImplementedError("inverse factor matrices are fp32 in the native step")
        if pc.factor_matrix_dtype == torch.float64:
            root_inverse = type(pc) is RootInvShampooPreconditionerConfig and isinstance(acc, (CoupledNewtonConfig, EigenConfig))
            keeps_eigenvectors = type(pc) in (EigenvalueCorrectedShampooPreconditionerConfig, EigendecomposedShampooPreconditionerConfig)
            if not (root_inverse or keeps_eigenvectors) or pc.use_trace_scaling:
                raise NotImplementedError(
                    "factor_matrix_dtype=float64 is built for RootInvShampooPreconditionerConfig with CoupledNewtonConfig or "
                    "EigenConfig and for the eigenvalue-corrected and eigendecomposed lists, without trace scaling"
                )
        elif pc.factor_matrix_dtype != torch.float32:
            raise NotImplementedError(f"factor matrices are fp32 or fp64 in the native step, got {pc.factor_matrix_dtype}")
        if group[ITERATE_AVERAGING_CONFIG] is not None and not isinstance(
            group[ITERATE_AVERAGING_CONFIG], (ClassicMomentumConfig, GeneralizedPrimalAveragingConfig, ScheduleFreeConfig)
        ):
            raise NotImplementedError(
                f"{group[ITERATE_AVERAGING_CONFIG]=} is not supported! "
                "Supported configs: ClassicMomentumConfig, GeneralizedPrimalAveragingConfig, ScheduleFreeConfig."
            )

    @staticmethod
    def _inverse_exponent(pc: RootInvShampooPreconditionerConfig, dimension: int, order: int) -> float:
        """shampoo_preconditioner_list.py:1726-1747."""
        override = pc.inverse_exponent_override.get(order, {})
        if isinstance(override, dict):
            return override.get(dimension, 1 / (2 * max(order, 1)))
        return override

    @staticmethod
    def _graft_setup(graft: PreconditionerConfig | None) -> tuple[int, float, float, bool, float]:
        """(type, beta2, weighting factor, bias correction, epsilon), distributed_shampoo.py:673-714."""
        if graft is None:
            return native.SA_GRAFT_NONE, 1.0, 1.0, False, 0.0
        if isinstance(graft, SGDPreconditionerConfig):
            return native.SA_GRAFT_SGD, 1.0, 1.0, False, 0.0
        if isinstance(graft, RMSpropPreconditionerConfig) and graft.drop_weighting_factor_on_gsquare:
            return native.SA_GRAFT_ADAGRAD, graft.beta2, 1.0, False, graft.epsilon
        if isinstance(graft, AdamPreconditionerConfig):
            return native.SA_GRAFT_ADAGRAD, graft.beta2, 1 - graft.beta2, True, graft.epsilon
        if isinstance(graft, RMSpropPreconditionerConfig):
            return native.SA_GRAFT_ADAGRAD, graft.beta2, 1 - graft.beta2, False, graft.epsilon
        if isinstance(graft, AdaGradPreconditionerConfig):
            return native.SA_GRAFT_ADAGRAD, 1.0, 1.0, False, graft.epsilon
        raise NotImplementedError(f"{graft=} not supported!")

    # -- one step ----------------------------------------------------------------------------

    def _bind_gradients(self, eager_nan_check: bool) -> int:
        """Per-block gradient pointers; a parameter without a (non-empty) gradient masks its blocks
        (shampoo_distributor.py:259-299).  Returns the number of active blocks."""
        grads: list[torch.Tensor | None] = []
        for p in self.params:
            g = p.grad
            if g is None or g.numel() == 0:
                grads.append(None)
                continue
            if g.dtype != torch.float32 or g.device != p.device:
                raise NotImplementedError("gradients must be fp32 on the parameter's device")
            if not g.is_contiguous():
                raise ValueError("gradients must be contiguous (the reference views them with merged shapes)")
            if eager_nan_check:
                assert torch.isfinite(g).all(), (
                    f"Encountered gradient containing NaN/Inf in parameter with shape {g.shape}. "
                    "Check your model for numerical instability or consider gradient clipping."
                )
            grads.append(g)
        self._follow_parameter_storage()
        active = 0
        for k, i in enumerate(self.native_index):
            s = self.block_specs[i]
            g = grads[s.param_index]
            if g is None:
                self.grad_ptrs[k] = None
            else:
                self.grad_ptrs[k] = g.data_ptr() + 4 * s.offset
                active += 1
        self._grads_alive = grads  # keep the tensors alive until the step has been enqueued
        return active

    def _follow_parameter_storage(self) -> None:
        """The plan holds raw pointers into the parameters.  When a parameter's storage is replaced after the optimizer
        was built (`p.data = ...`, weight swaps, some checkpoint loaders) the pointers of the step differ from the ones
        the plan has, and the plan is re-pointed.  This is a deliberate deviation from the reference, which blocks
        detached views of the storage that existed at construction (shampoo_distributor.py:202-216) and keeps updating
        that old storage, so that the parameter no longer moves."""
        ptrs = [p.data_ptr() for p in self.params]
        if ptrs == self._param_ptrs:
            return
        for p in self.params:
            if p.device != self.device or p.dtype != torch.float32:
                raise NotImplementedError("parameters must stay fp32 on the device the optimizer was built for")
            if not p.is_contiguous():
                raise ValueError("parameters must be contiguous (the reference views them with merged shapes)")
        table = (ctypes.c_void_p * max(self.n_native, 1))()
        for k, i in enumerate(self.native_index):
            s = self.block_specs[i]
            table[k] = ptrs[s.param_index] + 4 * s.offset
            self.descs[k].param = table[k]
        native.check(self.lib.sa_plan_rebind_params(self.plan, table), "sa_plan_rebind_params")
        self._param_ptrs = ptrs

    def _interp_coeffs(self, cfg: Any, lr: torch.Tensor | None) -> tuple[torch.Tensor, torch.Tensor]:
        """(mu_y, mu_x) as fp32 tensors, distributed_shampoo.py:1296-1340.  Schedule-Free accumulates lr^power in
        `lr_sum` (state) and uses mu_x = 1 - lr^power / lr_sum; without an lr (train / eval switch) mu_x is 0."""
        train = torch.tensor(cfg.train_interp_coeff, dtype=torch.float32)
        if isinstance(cfg, GeneralizedPrimalAveragingConfig):
            return train, torch.tensor(cfg.eval_interp_coeff, dtype=torch.float32)
        if lr is None:
            logger.warning("lr or lr_sum not provided to _get_train_and_eval_interp_coeffs; returning eval_interp_coeff = 0.0!")
            return train, torch.tensor(0.0, dtype=torch.float32)
        lr_power = torch.pow(lr, cfg.eval_coeff_lr_power)
        # the sum is kept on the host and mirrored into the state tensor, so that no step waits for the device
        self._lr_sum_host = self._lr_sum_host + lr_power
        self.lr_sum.copy_(self._lr_sum_host, non_blocking=True)
        return train, 1.0 - lr_power / self._lr_sum_host

    def switch_mode(self, group: dict[str, Any], train: bool) -> None:
        """train(): y = x + (1 - mu_y)(z - x); eval(): x = y + (1 - 1/mu_y)(z - y), on every block
        (distributed_shampoo.py:1729-1797)."""
        if not self.primal_averaging or bool(self.train_mode) == train:
            return
        mu_y, _ = self._interp_coeffs(group[ITERATE_AVERAGING_CONFIG], None)
        coeff = float(1 - mu_y) if train else float(1 - torch.reciprocal(mu_y))
        if self.n_native:
            with torch.cuda.device(self.device):
                native.check(
                    self.lib.sa_move_params_towards_weight_buffer(self.plan, coeff, native.current_stream_ptr(self.device)),
                    "sa_move_params_towards_weight_buffer",
                )
        self.train_mode.fill_(train)

    def step(self, group: dict[str, Any], runtime: ShampooRuntimeConfig) -> None:
        lib = self.lib
        active = self._bind_gradients(runtime.eager_nan_check) if self.n_native else 0
        step = self.step_tensor.add_(1)
        step_val = int(step.item())
        if not active:
            self._grads_alive = None
            return
        stream = native.current_stream_ptr(self.device)
        native.check(lib.sa_plan_bind_gradients(self.plan, self.grad_ptrs, stream), "sa_plan_bind_gradients")

        beta1, beta2 = group[BETAS]
        beta3 = group[BETA3]
        lr = torch.tensor(group[LR], dtype=torch.float32).item()
        weight_decay = group[WEIGHT_DECAY]
        wd_type = group[WEIGHT_DECAY_TYPE]
        start = group[START_PRECONDITIONING_STEP]
        freq = group[PRECONDITION_FREQUENCY]
        use_bc = group[USE_BIAS_CORRECTION]
        pc = self.preconditioner_config
        amortize = (step_val % freq == 0 and step_val > start) or step_val == start
        graft_only = (step_val < start and group[GRAFTING_CONFIG] is not None) or self.elementwise_only

        if weight_decay != 0.0 and wd_type == WeightDecayType.L2:
            native.check(lib.sa_add_l2_regularization(self.plan, weight_decay, stream), "sa_add_l2_regularization")

        if self.eigendecomposed and self.inverse_roots_stale:
            # (Q, lambda) were restored from a checkpoint: the inverse roots they define are needed by the preconditioning
            # and, for KL-Shampoo, by the factor update
            self._inverse_roots_from_eigendecomposition(group, stream)
            self.inverse_roots_stale = False
        drop = pc.drop_weighting_factor_on_gsquare
        weighting = 1.0 if (drop or beta2 == 1.0) else 1 - beta2
        if self.factor_f64:
            native.check(lib.sa_update_factor_matrices_f64(self.plan, beta2, weighting, stream), "sa_update_factor_matrices_f64")
        else:
            native.check(lib.sa_update_factor_matrices(self.plan, beta2, weighting, stream), "sa_update_factor_matrices")
        if self.dense_state:
            native.check(lib.sa_plan_export_dense_state(self.plan, self.dense_factor_ptrs, None, stream), "sa_plan_export_dense_state")

        # fp32 scalars evaluated with the very torch expressions the reference uses
        bc2 = 1.0
        if use_bc and beta2 < 1.0 and not drop:
            bc2 = float(torch.tensor(1.0) - beta2**step)
        if amortize:
            self._amortized_computation(group, bc2, stream)
            self.inverse_roots_stale = False
            if self.dense_inv_arena is not None:
                native.check(
                    lib.sa_plan_export_dense_state(self.plan, None, self.dense_inv_ptrs, stream), "sa_plan_export_dense_state"
                )
        # one call updates the second moment in the eigenbasis and preconditions (the rotated gradient serves both);
        # with beta3 != beta1, or while only the grafting method steps, the statistic is updated on its own
        fuse_soap = self.soap and self.fuse_eigenbasis_rotations and not graft_only and (beta1 == 0.0 or beta3 == beta1)
        if self.soap and not fuse_soap:
            native.check(
                lib.sa_update_corrected_eigenvalues(self.plan, beta2, weighting, stream), "sa_update_corrected_eigenvalues"
            )

        s = native.StepScalars()
        s.lr = lr
        s.beta1 = beta1
        s.beta3 = beta3 if beta1 != 0.0 else 0.0
        # the lerp weights reach fp32 the way the reference's Python scalars do: 1 - beta in double, rounded once
        s.lerp_weight1 = 1 - beta1
        s.lerp_weight3 = 1 - beta3
        s.filtered_grad_mode = 0 if beta1 == 0.0 else (1 if beta3 == beta1 else 2)
        s.bias_correction1 = float(1.0 - beta3 * beta1 ** (step - 1)) if (use_bc and beta1 != 0.0) else 1.0
        s.graft_type = self.graft_type
        s.graft_beta2 = self.graft_beta2
        s.graft_weight = self.graft_weight
        s.graft_bias_correction2 = (
            float(torch.tensor(1.0) - self.graft_beta2**step) if (self.graft_bias and self.graft_beta2 < 1.0) else 1.0
        )
        s.graft_epsilon = self.graft_eps
        alpha = 0.0
        if weight_decay != 0.0 and wd_type != WeightDecayType.L2:
            if wd_type == WeightDecayType.DECOUPLED:
                alpha = weight_decay
            elif wd_type == WeightDecayType.CORRECTED:
                alpha = weight_decay * lr / group[PEAK_LR]
            elif wd_type == WeightDecayType.INDEPENDENT:
                alpha = weight_decay / group[PEAK_LR]
            else:
                raise ValueError(f"Invalid weight decay type: {wd_type=}!")
        s.weight_decay_alpha = alpha
        mom = group[ITERATE_AVERAGING_CONFIG]
        if isinstance(mom, ClassicMomentumConfig):
            s.momentum, s.dampening, s.use_nesterov = mom.momentum, mom.dampening, int(mom.use_nesterov)
        else:
            s.momentum, s.dampening, s.use_nesterov = 0.0, 0.0, 0
        if self.primal_averaging:
            if not bool(self.train_mode):
                raise RuntimeError(
                    "Called _apply_in_place_primal_averaging when not in train mode. Call optimizer.train() before calling optimizer.step()!"
                )
            train_coeff, eval_coeff = self._interp_coeffs(mom, torch.tensor(group[LR], dtype=torch.float32))
            s.use_primal_averaging = 1
            s.averaging_direction_coeff = float(1 - train_coeff * eval_coeff)
            s.averaging_buffer_coeff = float(1 - eval_coeff)

        ref = ctypes.byref(s)
        if graft_only:
            native.check(lib.sa_grafting_only_step(self.plan, ref, stream), "sa_grafting_only_step")
        else:
            native.check(
                lib.sa_update_grafting_and_filtered_grad(self.plan, ref, stream),
                "sa_update_grafting_and_filtered_grad",
            )
            if fuse_soap:
                native.check(
                    lib.sa_update_and_precondition_eigenvalue_corrected(
                        self.plan, ref, beta2, weighting, bc2, group[EPSILON], self.soap_root, stream),
                    "sa_update_and_precondition_eigenvalue_corrected",
                )
            elif self.soap:
                native.check(
                    lib.sa_precondition_eigenvalue_corrected(self.plan, ref, bc2, group[EPSILON], self.soap_root, stream),
                    "sa_precondition_eigenvalue_corrected",
                )
            else:
                # With grafting the search direction only enters through P / ||P|| (distributed_shampoo.py:1110-1122), which
                # does not change when P is scaled: the product is then formed from the filtered gradient as it is
                # stored, without its bias correction, and the GEMM's loader has no division to do per element and
                # slab.  (The reference divides first; the results differ by fp32 rounding.)
                if self.graft_type != native.SA_GRAFT_NONE and s.bias_correction1 != 1.0:
                    unscaled = native.StepScalars.from_buffer_copy(s)
                    unscaled.bias_correction1 = 1.0
                    native.check(lib.sa_precondition(self.plan, ctypes.byref(unscaled), stream), "sa_precondition")
                else:
                    native.check(lib.sa_precondition(self.plan, ref, stream), "sa_precondition")
            native.check(lib.sa_apply_update(self.plan, ref, stream), "sa_apply_update")
        # drop the references so param.grad can be freed (distributed_shampoo.py:1666-1667)
        self._grads_alive = None


class DistributedShampoo(torch.optim.Optimizer):
    """Distributed Shampoo on one MI355X.

    Arguments, defaults and validation follow the reference constructor
    (distributed_shampoo/distributed_shampoo.py:361-535).  Built natively:
    `RootInvShampooPreconditionerConfig` with `CoupledNewtonConfig`, `CoupledHigherOrderConfig` (orders 2..8) or
    `EigenConfig` (`PerturbationConfig` and `PseudoInverseConfig`), `use_trace_scaling`,
    `RootInvKLShampooPreconditionerConfig` / `EigendecomposedKLShampooPreconditionerConfig` (blocks of order 1 and 2),
    `EigenvalueCorrectedShampooPreconditionerConfig` and `EigendecomposedShampooPreconditionerConfig` with
    `QREigendecompositionConfig` or `EighEigendecompositionConfig` (including `ignored_basis_change_dims`), grafting with SGD / AdaGrad / RMSprop /
    Adam or none, every `WeightDecayType`, `ClassicMomentumConfig`, `GeneralizedPrimalAveragingConfig`, `ScheduleFreeConfig`, `inverse_exponent_override`,
    an SGD / AdaGrad / RMSprop / Adam config as `preconditioner_config` itself,
    `SingleDeviceDistributedConfig`, fp32 state with packed factor matrices (`factor_matrix_dtype=torch.float64` for
    root-inverse Shampoo: fp64 factor averages and an fp64 coupled Newton root inverse), blocks of order 1 to 3 (order 3: what is left of
    convolution weights).
    Anything else raises NotImplementedError at construction.
    """

    def __init__(
        self,
        params,
        lr: float = 1e-2,
        betas: tuple[float, float] = (0.9, 1.0),
        beta3: float = -1.0,
        epsilon: float = 1e-12,
        weight_decay: float = 0.0,
        weight_decay_type: WeightDecayType = WeightDecayType.DECOUPLED,
        max_preconditioner_dim: int | float = 1024,
        precondition_frequency: int = 1,
        start_preconditioning_step: int = -1,
        use_bias_correction: bool = True,
        iterate_averaging_config: IterateAveragingConfig | None = None,
        grafting_config: PreconditionerConfig | None = None,
        use_pin_memory: bool = False,
        shampoo_pt2_compile_config: object | None = None,
        distributed_config: DistributedConfig = DefaultSingleDeviceDistributedConfig,
        preconditioner_config: PreconditionerConfig = DefaultShampooConfig,
        shampoo_runtime_config: ShampooRuntimeConfig = DefaultShampooRuntimeConfig,
        concurrency_config: ConcurrencyConfig = DefaultConcurrencyConfig,
    ) -> None:
        super().__init__(
            params,
            {
                LR: lr,
                BETAS: betas,
                BETA3: beta3,
                EPSILON: epsilon,
                WEIGHT_DECAY: weight_decay,
                PEAK_LR: lr,
                WEIGHT_DECAY_TYPE: weight_decay_type,
                MAX_PRECONDITIONER_DIM: max_preconditioner_dim,
                PRECONDITION_FREQUENCY: precondition_frequency,
                START_PRECONDITIONING_STEP: start_preconditioning_step,
                USE_BIAS_CORRECTION: use_bias_correction,
                ITERATE_AVERAGING_CONFIG: iterate_averaging_config,
                GRAFTING_CONFIG: grafting_config,
                USE_PIN_MEMORY: use_pin_memory,
                DISTRIBUTED_CONFIG: distributed_config,
                PRECONDITIONER_CONFIG: preconditioner_config,
            },
        )
        if shampoo_pt2_compile_config is not None:
            raise NotImplementedError("shampoo_pt2_compile_config: the native step is not traced by torch.compile")
        for i, group in enumerate(self.param_groups):
            logger.info(f"Checking param_group {i} hyperparameters...")
            self._check_group(group)
        self._runtime_config = shampoo_runtime_config
        self._concurrency_config = concurrency_config
        self._groups: list[_NativeGroup] = [_NativeGroup(self, g, i) for i, g in enumerate(self.param_groups)]
        all_cuda = all(g[PARAMS][0].device.type == "cuda" for g in self.param_groups)
        self._use_streams = bool(concurrency_config.enable_cuda_stream_for_param_groups and all_cuda)
        if self._use_streams:
            for ng in self._groups:
                ng.stream = torch.cuda.Stream(device=ng.device)
        self.register_load_state_dict_post_hook(DistributedShampoo._after_load_state_dict)

    def __del__(self) -> None:
        for ng in getattr(self, "_groups", []):
            try:
                ng.close()
            except Exception:  # noqa: BLE001 - interpreter shutdown
                pass

    @staticmethod
    def _check_group(param_group: dict[str, Any]) -> None:
        """distributed_shampoo.py:411-530, same conditions and messages."""
        if not param_group[LR] >= 0.0:
            raise ValueError(f"Invalid {param_group[LR]=}. Must be >= 0.0.")
        if not 0.0 <= param_group[BETAS][0] < 1.0:
            raise ValueError(f"Invalid {param_group[BETAS][0]=}. Must be in [0.0, 1.0).")
        if not 0.0 <= param_group[BETAS][1] <= 1.0:
            raise ValueError(f"Invalid {param_group[BETAS][1]=}. Must be in [0.0, 1.0].")
        if param_group[BETA3] == -1.0:
            param_group[BETA3] = param_group[BETAS][0]
        elif not 0.0 <= param_group[BETA3] < 1.0:
            raise ValueError(f"Invalid {param_group[BETA3]=}. Must be in [0.0, 1.0).")
        pc = param_group[PRECONDITIONER_CONFIG]
        if (
            isinstance(pc, BaseShampooPreconditionerConfig)
            and isinstance(pc.amortized_computation_config, EigendecompositionConfig)
            and isinstance(pc.amortized_computation_config.rank_deficient_stability_config, PseudoInverseConfig)
        ):
            if param_group[EPSILON] != 0.0:
                raise ValueError(f"Invalid {param_group[EPSILON]=}. Must be == 0.0 when PseudoInverseConfig is used.")
        elif not param_group[EPSILON] > 0.0:
            raise ValueError(f"Invalid {param_group[EPSILON]=}. Must be > 0.0.")
        if not param_group[WEIGHT_DECAY] >= 0.0:
            raise ValueError(f"Invalid {param_group[WEIGHT_DECAY]=}. Must be >= 0.0.")
        if (
            param_group[WEIGHT_DECAY_TYPE] in (WeightDecayType.CORRECTED, WeightDecayType.INDEPENDENT)
            and not param_group[PEAK_LR] > 0.0
        ):
            raise ValueError(
                f"Invalid {param_group[PEAK_LR]=}. Must be > 0.0 when using WeightDecayType.CORRECTED or WeightDecayType.INDEPENDENT."
            )
        if isinstance(param_group[MAX_PRECONDITIONER_DIM], float) and param_group[MAX_PRECONDITIONER_DIM] != math.inf:
            raise ValueError(f"Invalid {param_group[MAX_PRECONDITIONER_DIM]=}. Must be an integer or math.inf.")
        if not param_group[MAX_PRECONDITIONER_DIM] >= 1:
            raise ValueError(f"Invalid {param_group[MAX_PRECONDITIONER_DIM]=}. Must be >= 1.")
        if not param_group[PRECONDITION_FREQUENCY] >= 1:
            raise ValueError(f"Invalid {param_group[PRECONDITION_FREQUENCY]=}. Must be >= 1.")
        if not param_group[START_PRECONDITIONING_STEP] >= -1:
            raise ValueError(f"Invalid {param_group[START_PRECONDITIONING_STEP]=}. Must be >= -1.")
        if param_group[START_PRECONDITIONING_STEP] == -1:
            param_group[START_PRECONDITIONING_STEP] = param_group[PRECONDITION_FREQUENCY]
            logger.warning(
                f"start_preconditioning_step set to -1. Setting start_preconditioning_step equal to {param_group[PRECONDITION_FREQUENCY]=} by default."
            )
        if param_group[START_PRECONDITIONING_STEP] < param_group[PRECONDITION_FREQUENCY]:
            raise ValueError(
                f"Invalid {param_group[START_PRECONDITIONING_STEP]=}. Must be >= {param_group[PRECONDITION_FREQUENCY]=}."
            )

    @torch.no_grad()
    def train(self) -> None:
        """distributed_shampoo.py:1729-1761: groups with primal averaging / Schedule-Free move back to the training
        sequence."""
        logger.info("Enabling train mode in Distributed Shampoo!")
        for ng, group in zip(self._groups, self.param_groups, strict=True):
            ng.switch_mode(group, train=True)

    @torch.no_grad()
    def eval(self) -> None:
        """distributed_shampoo.py:1763-1797: groups with primal averaging / Schedule-Free move to the evaluation
        sequence."""
        logger.info("Enabling eval mode in Distributed Shampoo!")
        for ng, group in zip(self._groups, self.param_groups, strict=True):
            ng.switch_mode(group, train=False)

    @torch.no_grad()
    def step(self, closure: Callable[[], float] | None = None) -> float | None:
        """One optimization step (distributed_shampoo.py:1677-1711)."""
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for ng, group in zip(self._groups, self.param_groups, strict=True):
            if self._use_streams:
                ng.stream.wait_stream(torch.cuda.current_stream(ng.device))
                ctx = torch.cuda.stream(ng.stream)
            else:
                ctx = nullcontext()
            with ctx:
                ng.step(group, self._runtime_config)
        if self._use_streams:
            for ng in self._groups:
                torch.cuda.current_stream(ng.device).wait_stream(ng.stream)
        return loss

    # -- checkpointing ----------------------------------------------------------------------

    @staticmethod
    def _after_load_state_dict(optimizer: "DistributedShampoo") -> None:
        """torch's load_state_dict replaces the state tensors with copies; move the loaded values
        back into the arenas the kernels own and re-alias the state (the reference copies in place
        too, distributed_shampoo.py:1803-1889)."""
        for ng in optimizer._groups:
            ng.restore_state(optimizer)


def _restore_state(self: _NativeGroup, optimizer: DistributedShampoo) -> None:
    for param, block_key, path, mine in self._slots:
        node = optimizer.state[param].setdefault(block_key, {})
        for key in path[:-1]:
            nxt = node.get(key, node.get(str(key))) if isinstance(node, dict) else None
            if nxt is None:
                nxt = {}
                node[key] = nxt
            node = nxt
        last = path[-1]
        src = node.get(last, node.get(str(last)))
        if src is not None and src.data_ptr() != mine.data_ptr():
            mine.copy_(src.to(device=mine.device, dtype=mine.dtype).reshape(mine.shape))
        node.pop(str(last), None)
        node[last] = mine
    loaded_steps = [int(optimizer.state[p][STEP]) for p in self.params if STEP in optimizer.state[p]]
    if loaded_steps:
        assert len(set(loaded_steps)) == 1, f"parameters of one group disagree on step: {sorted(set(loaded_steps))}"
        self.step_tensor.fill_(loaded_steps[0])
    for p in self.params:
        optimizer.state[p][STEP] = self.step_tensor
    if self.primal_averaging:
        # per-group scalars of primal averaging / Schedule-Free, re-aliased under every parameter
        for key, mine in ((LR_SUM, self.lr_sum), (TRAIN_MODE, self.train_mode)):
            loaded = [optimizer.state[p][key] for p in self.params if key in optimizer.state[p]]
            if loaded:
                mine.copy_(torch.as_tensor(loaded[0]).to(device=mine.device, dtype=mine.dtype))
            for p in self.params:
                optimizer.state[p][key] = mine
        self._lr_sum_host = self.lr_sum.detach().cpu().clone()
    if self.plan and self.dense_state:
        # the loaded dense matrices are the state; the kernels' packed triangles follow them
        with torch.cuda.device(self.device):
            native.check(
                self.lib.sa_plan_import_dense_state(
                    self.plan, self.dense_factor_ptrs, self.dense_inv_ptrs if self.dense_inv_arena is not None else None,
                    native.current_stream_ptr(self.device)),
                "sa_plan_import_dense_state",
            )
    if self.plan:
        native.check(self.lib.sa_plan_invalidate_inverse_cache(self.plan), "sa_plan_invalidate_inverse_cache")
    # eigendecomposed Shampoo: the inverse roots are a function of the restored (Q, lambda)
    self.inverse_roots_stale = self.eigendecomposed


_NativeGroup.restore_state = _restore_state  # type: ignore[attr-defined]
