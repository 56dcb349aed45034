"""CPU oracle for the Distributed Shampoo per-step preconditioner hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this file:
only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may
use it, and there only as the checker / the timed CPU baseline.

It is a plain-torch restatement (no reference import) of the algorithm that
`DistributedShampoo.step()` executes on the single-device distributor.  Every
function names the reference file:line it follows (paths relative to the
reference checkout).  Floating point follows the reference's own op order where
that is observable: fp32 bias-correction scalars, `factor / bc2` before the root
inverse, upper-triangle storage of the inverse root, the 1e-16 grafting guard.

Pinning status (which independent check fixes which function) is recorded per
function below; anything that only the reference's own trajectory can fix is
pinned by the committed fixtures under tests/golden/ (written once by
tests/golden/make_fixtures.py from the real reference, CPU, fp32).
"""

from __future__ import annotations

import itertools
import math
from dataclasses import dataclass, field
from fractions import Fraction
from typing import Any, Sequence

import torch
from torch import Tensor


class OraclePreconditionerValueError(ValueError):
    """Mirror of PreconditionerValueError (shampoo_types.py:87-88)."""


# --------------------------------------------------------------------------- #
# Block partition (integer work, must be bit-exact)
# --------------------------------------------------------------------------- #


def merge_small_dims(
    shape: Sequence[int], threshold: int | float, target_dimensionality: int | float = 1
) -> tuple[int, ...]:
    """utils/shampoo_utils.py:38-121.

    Drop size-1 dims, then walk the dims right-to-left greedily multiplying a
    dim into its right neighbour while (a) more dims remain than the target and
    (b) the product stays <= threshold.
    Pinned by the reference's vectors (utils/tests/shampoo_utils_test.py:64-169).
    """
    shape = tuple(int(s) for s in shape)
    if 0 in shape:
        return (0,)
    if isinstance(target_dimensionality, float):
        assert target_dimensionality == math.inf
        return shape
    rev = [s for s in reversed(shape) if s != 1] or [1]
    out = [rev[0]]
    total = len(rev)
    for seen, nxt in enumerate(rev[1:], start=1):
        could_still_have = len(out) + (total - seen)
        if could_still_have > target_dimensionality and out[-1] * nxt <= threshold:
            out[-1] *= nxt
        else:
            out.append(nxt)
    return tuple(reversed(out))


def split_bounds(extent: int, size: int | float) -> list[tuple[int, int]]:
    """Chunk boundaries of torch.split(extent, size): full chunks then a remainder."""
    if isinstance(size, float):
        assert size == math.inf
        return [(0, extent)]
    if extent == 0:
        return [(0, 0)]
    return [(lo, min(lo + size, extent)) for lo in range(0, extent, size)]


def block_slices(
    shape: Sequence[int], block_size: int | float
) -> list[tuple[tuple[int, int], ...]]:
    """utils/shampoo_utils.py:124-174 (multi_dim_split) as index ranges.

    Splitting dim 0 first and then each piece along dim 1 ... enumerates the
    block grid in row-major (lexicographic) order.
    Pinned by utils/tests/shampoo_utils_test.py:172-211 and brute force vs torch.split.
    """
    per_dim = [split_bounds(int(e), block_size) for e in shape]
    return list(itertools.product(*per_dim))


def multi_dim_split(t: Tensor, block_size: int | float) -> tuple[Tensor, ...]:
    out = []
    for ranges in block_slices(t.shape, block_size):
        v = t
        for d, (lo, hi) in enumerate(ranges):
            v = v.narrow(d, lo, hi - lo)
        out.append(v)
    return tuple(out)


def blocks_of(
    t: Tensor, max_preconditioner_dim: int | float, target_dimensionality: int | float = 1
) -> tuple[Tensor, ...]:
    """distributor/shampoo_distributor.py:173-219: view(merged shape) then split."""
    merged = merge_small_dims(tuple(t.shape), max_preconditioner_dim, target_dimensionality)
    return multi_dim_split(t.view(merged), max_preconditioner_dim)


# --------------------------------------------------------------------------- #
# Symmetric packing
# --------------------------------------------------------------------------- #


def pack_triu(m: Tensor) -> Tensor:
    """utils/shampoo_utils.py:1217-1231: row-major upper triangle incl. diagonal."""
    d = m.shape[0]
    r, c = torch.triu_indices(d, d, device=m.device)
    return m[r, c].contiguous()


def unpack_triu(p: Tensor, d: int) -> Tensor:
    """utils/shampoo_utils.py:1234-1249: mirror the upper triangle into the lower."""
    out = torch.zeros(d, d, dtype=p.dtype, device=p.device)
    r, c = torch.triu_indices(d, d, device=p.device)
    out[r, c] = p
    out[c, r] = p
    return out


def packed_dim(numel: int) -> int:
    """shampoo_preconditioner_list.py:269-282."""
    return (-1 + math.isqrt(1 + 8 * numel)) // 2


def packed_eye(d: int, dtype=torch.float32, device="cpu") -> Tensor:
    """shampoo_preconditioner_list.py:67-103: diagonal (i,i) sits at i*d - i*(i-1)/2."""
    p = torch.zeros(d * (d + 1) // 2, dtype=dtype, device=device)
    i = torch.arange(d, device=device)
    p[i * d - i * (i - 1) // 2] = 1.0
    return p


# --------------------------------------------------------------------------- #
# Matrix functions
# --------------------------------------------------------------------------- #


def ridge(a: Tensor, eps: float) -> Tensor:
    """preconditioner/matrix_functions.py:145-176 (dense-matrix branch)."""
    if eps == 0:
        return a
    return a.add(torch.eye(a.shape[0], dtype=a.dtype, device=a.device), alpha=eps)


def newton_inverse_root(
    a: Tensor, root: int, eps: float = 0.0, max_iterations: int = 100, tolerance: float = 1e-6
) -> tuple[Tensor, Tensor, bool, int, Tensor]:
    """preconditioner/matrix_functions.py:368-437 (coupled inverse Newton).

    Returns (X, M, converged, iterations, error).  The loop condition is written
    exactly as `error > tol and it < max`, so a NaN error ends the loop.
    Pinned by: known answers matrix_functions_test.py:216-273, residual invariant
    :599-661, fp64 eigh truth, and the fixture trajectories (iteration counts).
    """
    d = a.shape[0]
    alpha = -1 / root
    eye = torch.eye(d, dtype=a.dtype, device=a.device)
    a_r = ridge(a, eps)
    nrm = torch.linalg.norm(a_r)
    z = (root + 1) / (2 * nrm)
    x = z ** (-alpha) * eye
    m = z * a_r
    err = torch.dist(m, eye, p=torch.inf)
    it = 0
    while err > tolerance and it < max_iterations:
        it += 1
        m_p = m.mul(alpha).add_(eye, alpha=(1 - alpha))
        x = x @ m_p
        m = torch.linalg.matrix_power(m_p, root) @ m
        err = torch.dist(m, eye, p=torch.inf)
    return x, m, bool(err <= tolerance), it, err



class OracleArithmeticError(ArithmeticError):
    """The failures matrix_functions.py:543-546, :629-632, :655-658 raise as ArithmeticError."""


def higher_order_coefficients(p: int, order: int) -> list[float]:
    """matrix_functions.py:520-526: Taylor coefficients of (1 - x)^(-1/p),
    b_0 = 1, b_i = b_{i-1} * (1 + (i - 1) p) / (i p), kept as exact integer
    numerator / denominator products and divided once per entry.
    Pinned by the binomial series (-1)^i binom(-1/p, i) in the tests.
    """
    b = [1.0]
    num, den = 1, 1
    for i in range(1, order):
        num *= 1 + (i - 1) * p
        den *= i * p
        b.append(num / den)
    return b


def higher_order_inverse_root(
    a: Tensor,
    root: Fraction,
    rel_epsilon: float = 0.0,
    abs_epsilon: float = 0.0,
    max_iterations: int = 100,
    tolerance: float = 1e-8,
    order: int = 3,
) -> tuple[Tensor, Tensor, str, int, Tensor]:
    """preconditioner/matrix_functions.py:439-661 (coupled higher-order iteration).

    A_r = A + max(rel_eps * |A|_inf, abs_eps) I; z = 1 / trace(A_r); X = z^(1/p) I, M = z A_r;
    one unconditional Newton step; then while error > tol and it < max: M_p = sum_i b_i (I - M)^i
    by Horner, X <- X M_p, M <- M_p^p M; stop early when the new error exceeds 1.2 x the previous
    one or repeats it below 1e-3 (X and M keep the last update, the error does not).  Afterwards
    |A_r X^p - I|_max > 0.1 and a non-finite X^q raise.
    Returns (X^q, M, flag, iterations, true_error), flag in {"converged", "max_iters", "early_stop"}.
    Pinned by: the reference's known answers matrix_functions_test.py:216-273 (orders 2..6, roots
    2 and 2/2), its failure cases :275-287, :337-370, fp64 eigh truth, order 2 against
    newton_inverse_root on the same start, and fixture trajectories (iteration counts, flags).
    """
    p, q = root.numerator, root.denominator
    b = higher_order_coefficients(p, order)
    d = a.shape[0]
    s = -1 / p
    lam_max = torch.linalg.matrix_norm(a, torch.inf)
    if not math.isfinite(lam_max.item()):
        raise OracleArithmeticError("Input matrix has entries close to inf, exiting root inverse")
    eps = torch.clamp(lam_max * rel_epsilon, min=abs_epsilon)
    eye = torch.eye(d, dtype=a.dtype, device=a.device)
    a_r = a + eps * eye  # _matrix_perturbation with a tensor epsilon, matrix_functions.py:145-176
    z = torch.reciprocal(torch.trace(a_r))
    x = torch.pow(z, -s) * eye
    m = z * a_r
    err = torch.linalg.vector_norm(m - eye, torch.inf)
    # one plain Newton step first (:565-572)
    m_p = m.mul(s).add_(eye, alpha=(1 - s))
    x = x @ m_p
    m = torch.linalg.matrix_power(m_p, p) @ m
    err = torch.linalg.vector_norm(m - eye, torch.inf)
    it = 1
    flag = None
    while err > tolerance and it < max_iterations:
        it += 1
        base = eye - m
        m_p = base.mul(b[order - 1]).add_(eye, alpha=b[order - 2])
        for i in reversed(range(order - 2)):
            m_p = torch.addmm(eye, m_p, base, beta=b[i])
        x = x @ m_p
        m = torch.linalg.matrix_power(m_p, p) @ m
        new_err = torch.linalg.vector_norm(m - eye, torch.inf)
        if new_err > err * 1.2 or (new_err == err and err < 1e-3):
            flag = "early_stop"
            break
        err = new_err
    if flag is None:
        flag = "max_iters" if err > tolerance else "converged"
    true_err = torch.linalg.vector_norm(a_r @ torch.linalg.matrix_power(x, p) - eye, torch.inf)
    if true_err > 1e-1:
        raise OracleArithmeticError(
            f"Error in matrix inverse root (before powering for fractions) {true_err} exceeds threshold 1e-1, raising an exception!"
        )
    if q > 1:
        x = torch.linalg.matrix_power(x, q)
    if not torch.isfinite(x).all():
        raise OracleArithmeticError(
            "NaN/Inf in matrix inverse root (after powering for fractions), raising an exception!"
        )
    return x, m, flag, it, true_err


def eigh_inverse_root(a: Tensor, root: float, eps: float = 0.0) -> Tensor:
    """matrix_functions.py:306-366 + :698-770 + :179-279 with the default
    PerturbationConfig(perturb_before_computation=True): ridge first, eigh,
    shift the spectrum to >= eps only if its minimum fell below eps.
    Pinned by library identity Q diag(l^-1/r) Q^T (torch.linalg.eigh) and the
    perturbation cases matrix_functions_test.py:116-151.
    """
    lam, q = torch.linalg.eigh(ridge(a, eps))
    lmin = torch.min(lam).item()
    if lmin < eps:
        lam = lam + (-lmin)
        lam = lam + eps
    return q * lam.pow(-1.0 / root).unsqueeze(0) @ q.T


def inverse_root_from_eigendecomposition(lam: Tensor, q: Tensor, root: float, eps: float = 0.0) -> Tensor:
    """matrix_functions.py:179-279 with the default PerturbationConfig(perturb_before_computation=True):
    the eigenvalues are used as they are unless their minimum is below eps, in which case they are
    shifted to start at eps (two rounded additions); X = Q diag(lam^(-1/root)) Q^T.
    Pinned by the same identity as eigh_inverse_root (which is this function applied to torch.linalg.eigh)
    and by the eigendecomposed-Shampoo fixtures written from the reference."""
    lmin = torch.min(lam).item()
    if lmin < eps:
        lam = lam + (-lmin)
        lam = lam + eps
    return q * lam.pow(-1.0 / root).unsqueeze(0) @ q.T


def eigh_pseudo_inverse_root(
    a: Tensor, root: float, rank_rtol: float | None = None, rank_atol: float = 0.0
) -> Tensor:
    """matrix_functions.py:206-249 (PseudoInverseConfig, epsilon = 0): eigenvalues at or
    below max(rank_atol, rtol * relu(lambda_max)) get weight zero, rtol = rank_rtol or
    n * machine epsilon; the others lambda^(-1/root).
    Pinned by numpy.linalg.pinv (root 1, same cutoff) and closed forms on projectors.
    """
    lam, q = torch.linalg.eigh(a)
    rtol = lam.numel() * torch.finfo(lam.dtype).eps if rank_rtol is None else rank_rtol
    cutoff = torch.clamp(rtol * lam.max().relu(), min=rank_atol)
    w = torch.where(lam <= cutoff, torch.zeros_like(lam), lam.pow(-1.0 / root))
    return q * w.unsqueeze(0) @ q.T


def qr_refresh(
    a: Tensor, q_prev: Tensor, eps: float = 0.0, max_iterations: int = 1, tolerance: float = 0.0
) -> tuple[Tensor, Tensor]:
    """matrix_functions.py:799-852 via :865-904: one (or more) unshifted QR
    iteration(s) started from the previous eigenbasis, then a stable ascending
    sort of the Rayleigh diagonal that permutes Q's columns.
    Pinned by matrix_functions_test.py:776-839 (3x3 vectors) and fixtures.
    """
    a_r = ridge(a, eps)
    q_est = q_prev
    b = q_est.T @ a_r @ q_est
    it = 0

    def small_enough(bm: Tensor) -> bool:
        n = torch.linalg.norm(bm)
        dn = torch.linalg.norm(bm.diag())
        return bool(torch.sqrt(n**2 - dn**2) <= tolerance * n)

    while it < max_iterations and not small_enough(b):
        qq, rr = torch.linalg.qr(b)
        b = rr @ qq
        q_est = q_est @ qq
        it += 1
    vals, idx = b.diag().sort(stable=True)
    return vals, q_est[:, idx]


# --------------------------------------------------------------------------- #
# The optimizer step
# --------------------------------------------------------------------------- #


@dataclass
class OracleConfig:
    """Hyper-parameters with the reference's names (distributed_shampoo.py:361-382).

    preconditioner: "newton" | "higher_order" | "eigh" (RootInvShampooPreconditionerConfig with
    CoupledNewtonConfig / CoupledHigherOrderConfig / EigenConfig) or "soap_qr" | "soap_eigh"
    (EigenvalueCorrectedShampooPreconditionerConfig) or "eigendecomposed_eigh" | "eigendecomposed_qr"
    (EigendecomposedShampooPreconditionerConfig).
    grafting: None | "adam" | "rmsprop" | "adagrad" | "sgd".
    """

    lr: float = 1e-2
    betas: tuple[float, float] = (0.9, 1.0)
    beta3: float = -1.0
    epsilon: float = 1e-12
    weight_decay: float = 0.0
    weight_decay_type: str = "DECOUPLED"  # L2 | DECOUPLED | CORRECTED | INDEPENDENT
    max_preconditioner_dim: int | float = 1024
    precondition_frequency: int = 1
    start_preconditioning_step: int = -1
    use_bias_correction: bool = True
    preconditioner: str = "eigh"
    newton_max_iterations: int = 100
    newton_tolerance: float = 1e-6
    higher_order: int = 3  # CoupledHigherOrderConfig fields (matrix_functions_types.py:217-240)
    higher_order_rel_epsilon: float = 0.0
    higher_order_abs_epsilon: float = 0.0
    higher_order_max_iterations: int = 100
    higher_order_tolerance: float = 1e-8
    qr_max_iterations: int = 1
    qr_tolerance: float = 0.0
    inverse_exponent_override: dict = field(default_factory=dict)
    ignored_basis_change_dims: dict = field(default_factory=dict)
    grafting: str | None = None
    grafting_beta2: float = 0.999
    grafting_epsilon: float = 1e-10
    averaging: str | None = None  # "gpa" (GeneralizedPrimalAveragingConfig) | "schedule_free" (ScheduleFreeConfig)
    eval_interp_coeff: float = 0.9
    train_interp_coeff: float = 0.8
    eval_coeff_lr_power: int = 2
    momentum: float = 0.0  # ClassicMomentumConfig.momentum (0 = disabled)
    dampening: float = 0.0
    use_nesterov: bool = False
    use_symmetric_packing: bool = True
    num_tolerated_failed_amortized_computations: int = 3
    factor_matrix_dtype: str = "float32"  # "float64": factor matrices and their root inverse in double (shampoo_types.py:184)
    kl: bool = False  # RootInvKLShampooPreconditionerConfig / EigendecomposedKLShampooPreconditionerConfig
    use_trace_scaling: bool = False  # shampoo_types.py:187-188
    trace_scaling_exponent: float = 0.5


class ShampooOracle:
    """Restatement of DistributedShampoo for one parameter group on one device.

    step() follows distributed_shampoo.py:1562-1667 (_group_step_body) ->
    :1384-1501 (_compute_search_directions) -> shampoo_distributor.py:335-365.
    """

    def __init__(self, params: Sequence[Tensor], cfg: OracleConfig) -> None:
        self.cfg = cfg
        self.params = list(params)
        self.peak_lr = cfg.lr
        self.beta3 = cfg.betas[0] if cfg.beta3 == -1.0 else cfg.beta3
        # distributed_shampoo.py:517-530
        self.start = (
            cfg.precondition_frequency
            if cfg.start_preconditioning_step == -1
            else cfg.start_preconditioning_step
        )
        if self.start < cfg.precondition_frequency:
            raise ValueError("start_preconditioning_step must be >= precondition_frequency")
        self.step_t = torch.tensor(0, dtype=torch.int64)
        self.lr_sum = torch.tensor(0.0, dtype=torch.float32)
        self.train_mode = True
        self.soap = cfg.preconditioner.startswith("soap")
        self.eigendecomposed = cfg.preconditioner.startswith("eigendecomposed")
        self.blocks: list[Tensor] = []
        self.block_ids: list[tuple[int, str]] = []
        self.num_blocks_per_param: list[int] = []
        for pi, p in enumerate(self.params):
            bl = blocks_of(p.detach(), cfg.max_preconditioner_dim)
            self.num_blocks_per_param.append(len(bl))
            for bi, b in enumerate(bl):
                self.blocks.append(b)
                self.block_ids.append((pi, f"block_{bi}"))
        self.state: list[dict[str, Any]] = [self._init_block(b) for b in self.blocks]
        self.bc2_shampoo = torch.tensor(1.0)
        self.bc2_graft = torch.tensor(1.0)
        self.last_newton_iterations: list[list[int]] = []
        # Test hook, called with the oracle right after every amortized computation and before anything uses its result
        # (a test that compares runs on two hosts uses it to give columns of a refreshed eigenbasis whose eigenvalue
        # estimates are tied within rounding the order they had in the other run).
        self.after_amortized: Any = None

    # -- construction ------------------------------------------------------- #

    def _exponent(self, order: int, dim: int) -> float:
        """shampoo_preconditioner_list.py:1726-1747."""
        ov = self.cfg.inverse_exponent_override.get(order, {})
        if isinstance(ov, dict):
            return ov.get(dim, 1 / (2 * max(order, 1)))
        return ov

    def _init_block(self, b: Tensor) -> dict[str, Any]:
        cfg = self.cfg
        order = b.dim()
        dev, dt = b.device, b.dtype
        st: dict[str, Any] = {}
        if self.soap:
            # shampoo_preconditioner_list.py:1843-1865
            ignored = cfg.ignored_basis_change_dims.get(order, [])
            sel = tuple(d not in ignored for d in range(order))
            st["roots"] = (1 / cfg.inverse_exponent_override.get(order, 1 / 2),)
        else:
            sel = tuple(self._exponent(order, d) != 0.0 for d in range(order))
            st["roots"] = tuple(1 / self._exponent(order, d) for d in range(order) if sel[d])
        st["selector"] = sel
        dims = [b.shape[d] for d in range(order) if sel[d]]
        st["dims"] = dims
        fdt = torch.float64 if cfg.factor_matrix_dtype == "float64" else dt
        if cfg.use_symmetric_packing:
            st["factors"] = [torch.zeros(d * (d + 1) // 2, dtype=fdt, device=dev) for d in dims]
        else:
            st["factors"] = [torch.zeros(d, d, dtype=fdt, device=dev) for d in dims]
        if self.soap:
            st["eigvecs"] = [torch.eye(d, dtype=dt, device=dev) for d in dims]
            st["corrected"] = torch.zeros(b.shape, dtype=dt, device=dev)
        elif self.eigendecomposed:
            # shampoo_preconditioner_list.py:730-750: identity eigenvectors, unit eigenvalues
            st["eigvecs"] = [torch.eye(d, dtype=dt, device=dev) for d in dims]
            st["eigvals"] = [torch.ones(d, dtype=dt, device=dev) for d in dims]
        else:
            if cfg.use_symmetric_packing:
                st["inv"] = [packed_eye(d, dt, dev) for d in dims]
            else:
                st["inv"] = [torch.eye(d, dtype=dt, device=dev) for d in dims]
        st["failed"] = 0
        if cfg.grafting in ("adam", "rmsprop", "adagrad"):
            st["adagrad"] = torch.zeros(b.shape, dtype=dt, device=dev)
        if cfg.betas[0] != 0.0:
            st["filtered_grad"] = torch.zeros(b.shape, dtype=dt, device=dev)
        if cfg.momentum != 0.0:
            st["momentum_buffer"] = torch.zeros(b.shape, dtype=dt, device=dev)
        if cfg.averaging is not None:  # the z sequence starts at the parameters (distributed_shampoo.py:909-922)
            st["weight_buffer"] = b.detach().clone()
        return st

    # -- helpers ------------------------------------------------------------ #

    def _pack(self, m: Tensor) -> Tensor:
        return pack_triu(m) if self.cfg.use_symmetric_packing else m

    def _unpack(self, p: Tensor) -> Tensor:
        return unpack_triu(p, packed_dim(p.numel())) if self.cfg.use_symmetric_packing else p

    @staticmethod
    def _contract(g: Tensor, sel: Sequence[bool], mats: Sequence[Tensor], dims=([0], [0])) -> Tensor:
        """shampoo_preconditioner_list.py:1541-1578: every dim, in order, is either
        contracted against its matrix (result axis moves to the back) or rotated
        to the back untouched."""
        it = iter(mats)
        out = g
        for s in sel:
            out = torch.tensordot(out, next(it), dims=dims) if s else out.permute(*range(1, out.ndim), 0)
        return out

    # -- step --------------------------------------------------------------- #

    def _update_factors(self, grads: Sequence[Tensor]) -> None:
        """shampoo_preconditioner_list.py:1490-1539."""
        cfg = self.cfg
        beta2 = cfg.betas[1]
        w = 1.0 if beta2 == 1.0 else 1 - beta2
        for g, st in zip(grads, self.state):
            if not st["factors"]:
                continue
            order = g.dim()
            ks = [k for k in range(order) if st["selector"][k]]
            outer = []
            mats = self._inverse_roots(st) if cfg.kl else None
            for idx_of_k, k in enumerate(ks):
                rest = [d for d in range(order) if d != k]
                src = g
                if cfg.kl:
                    # shampoo_preconditioner_list.py:1945-2046: the gradient preconditioned along every other
                    # preconditioned dim with the stored inverse roots
                    local = list(st["selector"])
                    local[k] = False
                    src = self._contract(g, local, [m for i, m in enumerate(mats) if i != idx_of_k])
                outer.append(self._pack(torch.tensordot(src, src, dims=[rest, rest])))
            for f, o in zip(st["factors"], outer):
                if beta2 != 1.0:
                    f.mul_(beta2)
                f.add_(o, alpha=w)

    def _amortized(self, st: dict[str, Any], bi: int) -> list[int]:
        """shampoo_preconditioner_list.py:314-443 (+ :631-680 / :1137-1198)."""
        cfg = self.cfg
        iters: list[int] = []
        last_exc: Exception | None = None
        for k, f in enumerate(st["factors"]):
            a = self._unpack(f / self.bc2_shampoo)
            if cfg.use_trace_scaling:  # shampoo_preconditioner_list.py:366-371
                safe_trace = torch.clamp(torch.trace(a), min=cfg.epsilon)
                a = a * torch.pow(safe_trace, -cfg.trace_scaling_exponent)
            name = f"{self.block_ids[bi][0]}.{self.block_ids[bi][1]}.{k}"
            if not torch.isfinite(a).all():
                raise OraclePreconditionerValueError(
                    f"Encountered nan/inf values in factor matrix {name}! "
                )
            try:
                if self.eigendecomposed:
                    # shampoo_preconditioner_list.py:868-940: matrix_eigendecomposition started from the stored basis
                    if cfg.preconditioner == "eigendecomposed_qr":
                        # the previous eigenvectors enter with the dtype of the factor (:1160-1166)
                        vals, res = qr_refresh(a, st["eigvecs"][k].to(a.dtype), cfg.epsilon, cfg.qr_max_iterations, cfg.qr_tolerance)
                    else:
                        vals, res = torch.linalg.eigh(ridge(a, cfg.epsilon))
                    eigenvalues = vals
                    key, packed = "eigvecs", res
                elif self.soap:
                    if cfg.preconditioner == "soap_qr":
                        _, res = qr_refresh(
                            a, st["eigvecs"][k].to(a.dtype), cfg.epsilon, cfg.qr_max_iterations, cfg.qr_tolerance
                        )
                    else:
                        _, res = torch.linalg.eigh(ridge(a, cfg.epsilon))
                    key, packed = "eigvecs", res
                else:
                    root = Fraction(st["roots"][k])
                    if cfg.preconditioner == "newton":
                        if root.denominator != 1:
                            raise ValueError(
                                f"{root.denominator=} must be equal to 1 to use coupled inverse Newton iteration!"
                            )
                        res, _, _, it, _ = newton_inverse_root(
                            a, root.numerator, cfg.epsilon, cfg.newton_max_iterations, cfg.newton_tolerance
                        )
                        iters.append(it)
                    elif cfg.preconditioner == "higher_order":  # matrix_functions.py:682-689: epsilon is not passed on
                        res, _, _, it, _ = higher_order_inverse_root(
                            a, root, cfg.higher_order_rel_epsilon, cfg.higher_order_abs_epsilon,
                            cfg.higher_order_max_iterations, cfg.higher_order_tolerance, cfg.higher_order,
                        )
                        iters.append(it)
                    else:
                        res = eigh_inverse_root(a, root, cfg.epsilon)
                    key, packed = "inv", self._pack(res)
            except Exception as exc:  # keep the previous result, count the failure
                last_exc = exc
                continue
            if self.eigendecomposed:  # both computed quantities are checked, eigenvalues first (:401-426)
                if not torch.isfinite(eigenvalues).all():
                    raise OraclePreconditionerValueError(
                        f"Encountered nan or inf values in eigenvalues of factor matrix {name}! "
                    )
                st["eigvals"][k].copy_(eigenvalues)
            if not torch.isfinite(packed).all():
                raise OraclePreconditionerValueError(
                    f"Encountered nan or inf values in {'eigenvectors' if (self.soap or self.eigendecomposed) else 'matrices'} of factor matrix {name}! "
                )
            st[key][k].copy_(packed)
        if last_exc is None:
            st["failed"] = 0
        else:
            st["failed"] += 1
            if st["failed"] > cfg.num_tolerated_failed_amortized_computations:
                raise ValueError(
                    "The number of failed amortized computations for factors exceeded the allowed tolerance."
                ) from last_exc
        return iters

    def _graft_direction(self, st: dict[str, Any], ghat: Tensor) -> Tensor:
        """adagrad_preconditioner_list.py:143-162 (SGD grafting is the identity)."""
        if self.cfg.grafting == "sgd":
            return ghat
        den = (st["adagrad"] / self.bc2_graft).sqrt_().add_(self.cfg.grafting_epsilon)
        return ghat / den

    def _inverse_roots(self, st: dict[str, Any]) -> list[Tensor]:
        if self.eigendecomposed:
            # shampoo_preconditioner_list.py:1800-1832: the inverse roots are formed from (lambda, Q) in every step
            return [
                inverse_root_from_eigendecomposition(lam, q, Fraction(r), self.cfg.epsilon)
                for lam, q, r in zip(st["eigvals"], st["eigvecs"], st["roots"])
            ]
        return [self._unpack(p) for p in st["inv"]]

    def _shampoo_direction(self, st: dict[str, Any], ghat: Tensor) -> Tensor:
        cfg = self.cfg
        sel = st["selector"]
        if not self.soap:
            return self._contract(ghat, sel, self._inverse_roots(st))
        # shampoo_preconditioner_list.py:1914-1942
        rot = self._contract(ghat.clone(), sel, st["eigvecs"])
        rot.div_((st["corrected"] / self.bc2_shampoo).pow_(1 / st["roots"][0]).add_(cfg.epsilon))
        return self._contract(rot, sel, st["eigvecs"], dims=([0], [1]))

    def step(self, grads: Sequence[Tensor | None]) -> None:
        cfg = self.cfg
        beta1, beta2 = cfg.betas
        # blocked gradients + selector (shampoo_distributor.py:237-299)
        gblocks: list[Tensor | None] = []
        for g, nb in zip(grads, self.num_blocks_per_param):
            if g is None or g.numel() == 0:
                gblocks.extend([None] * nb)
            else:
                gblocks.extend(blocks_of(g, cfg.max_preconditioner_dim))
        active = [i for i, g in enumerate(gblocks) if g is not None]
        if not active:
            self.step_t.add_(1)
            return
        step = self.step_t.add_(1)
        s = int(step.item())
        lr = torch.tensor(cfg.lr, dtype=torch.float32, device=self.blocks[0].device)
        amortize = (s % cfg.precondition_frequency == 0 and s > self.start) or s == self.start
        graft_only = s < self.start and cfg.grafting is not None

        G = [gblocks[i] for i in active]
        W = [self.blocks[i] for i in active]
        S = [self.state[i] for i in active]

        # 1. L2 regularisation (distributed_shampoo.py:1127-1139) -- in place on the grad
        if cfg.weight_decay != 0.0 and cfg.weight_decay_type == "L2":
            for g, w in zip(G, W):
                g.add_(w, alpha=cfg.weight_decay)

        # 2. preconditioner updates (:1142-1159)
        saved = self.state
        self.state = S
        self._update_factors(G)
        self.state = saved
        if cfg.use_bias_correction and beta2 < 1.0:
            self.bc2_shampoo = torch.tensor(1.0) - beta2**step
        self.last_newton_iterations = []
        if amortize:
            for i, st in zip(active, S):
                self.last_newton_iterations.append(self._amortized(st, i))
            if self.after_amortized is not None:
                self.after_amortized(self)
        if self.soap:
            # shampoo_preconditioner_list.py:1891-1912
            w2 = 1.0 if beta2 == 1.0 else 1 - beta2
            for g, st in zip(G, S):
                rot = self._contract(g, st["selector"], st["eigvecs"])
                if beta2 != 1.0:
                    st["corrected"].mul_(beta2)
                st["corrected"].addcmul_(rot, rot, value=w2)
        if cfg.grafting in ("adam", "rmsprop", "adagrad"):
            gb2 = 1.0 if cfg.grafting == "adagrad" else cfg.grafting_beta2
            gw = 1.0 if cfg.grafting == "adagrad" else 1 - gb2
            for g, st in zip(G, S):
                if gb2 != 1.0:
                    st["adagrad"].mul_(gb2)
                st["adagrad"].addcmul_(g, g, value=gw)
            if cfg.grafting == "adam" and gb2 < 1.0:
                self.bc2_graft = torch.tensor(1.0) - gb2**step

        # 3. filtered gradient (:1162-1199)
        if beta1 != 0.0:
            if self.beta3 != beta1:
                ghat = [torch.lerp(st["filtered_grad"], g, 1 - self.beta3) for g, st in zip(G, S)]
            for g, st in zip(G, S):
                st["filtered_grad"].lerp_(g, 1 - beta1)
            if self.beta3 == beta1:
                ghat = [st["filtered_grad"] for st in S]
            if cfg.use_bias_correction:
                bc1 = 1.0 - self.beta3 * beta1 ** (step - 1)
                ghat = [x / bc1 for x in ghat]
        else:
            ghat = list(G)

        # 4. precondition + graft (:1081-1124)
        if graft_only:
            P = [self._graft_direction(st, x) for st, x in zip(S, ghat)]
            # the reference hands back fresh tensors; SGD grafting returns its input
            P = [p.clone() if p is x else p for p, x in zip(P, ghat)]
        else:
            P = [self._shampoo_direction(st, x) for st, x in zip(S, ghat)]
            P = [p.clone() if p.data_ptr() == x.data_ptr() else p for p, x in zip(P, ghat)]
            if cfg.grafting is not None:
                for p, st, x in zip(P, S, ghat):
                    gn = torch.linalg.vector_norm(self._graft_direction(st, x))
                    sn = torch.linalg.vector_norm(p) + 1e-16
                    p.mul_(gn / sn)

        # 5. weight decay folded into the direction (:1202-1254)
        if cfg.weight_decay != 0.0 and cfg.weight_decay_type != "L2":
            if cfg.weight_decay_type == "DECOUPLED":
                a = cfg.weight_decay
            elif cfg.weight_decay_type == "CORRECTED":
                a = cfg.weight_decay * torch.tensor(cfg.lr, dtype=torch.float32).item() / self.peak_lr
            else:
                a = cfg.weight_decay / self.peak_lr
            if cfg.averaging is not None:  # the decay shrinks z instead of entering the direction
                for st in S:
                    st["weight_buffer"].mul_((1 - lr * a).to(st["weight_buffer"].dtype))
            else:
                for p, w in zip(P, W):
                    p.add_(w, alpha=a)

        # 6. classic momentum (:1257-1293)
        if cfg.momentum != 0.0:
            for p, st in zip(P, S):
                mb = st["momentum_buffer"]
                mb.mul_(cfg.momentum).add_(p, alpha=1 - cfg.dampening)
                if cfg.use_nesterov:
                    p.mul_(1 - cfg.dampening).add_(mb, alpha=cfg.momentum)
                else:
                    p.copy_(mb)

        # 7. learning rate, primal averaging (:1343-1382) and apply (:1484, shampoo_distributor.py:362-365)
        if cfg.averaging is not None:
            if not self.train_mode:
                raise RuntimeError(
                    "Called _apply_in_place_primal_averaging when not in train mode. Call optimizer.train() before calling optimizer.step()!"
                )
            mu_y, mu_x = self._interp_coeffs(lr)
        for p, w, st in zip(P, W, S):
            p.mul_(-lr)
            if cfg.averaging is not None:
                z = st["weight_buffer"]
                z_minus_y = z - w
                z.add_(p)
                p.mul_((1 - mu_y * mu_x).to(p.dtype))
                p.add_(z_minus_y, alpha=float(1 - mu_x))
            w.add_(p)

    def _interp_coeffs(self, lr: Tensor | None) -> tuple[Tensor, Tensor]:
        """distributed_shampoo.py:1296-1340: (mu_y, mu_x) as fp32 tensors; Schedule-Free accumulates lr^power."""
        cfg = self.cfg
        mu_y = torch.tensor(cfg.train_interp_coeff, dtype=torch.float32)
        if cfg.averaging == "gpa":
            return mu_y, torch.tensor(cfg.eval_interp_coeff, dtype=torch.float32)
        if lr is None:
            return mu_y, torch.tensor(0.0, dtype=torch.float32)
        lr_power = torch.pow(lr.to(torch.float32).cpu(), cfg.eval_coeff_lr_power)
        self.lr_sum = self.lr_sum + lr_power
        return mu_y, 1.0 - lr_power / self.lr_sum

    def train(self) -> None:
        """distributed_shampoo.py:1729-1761: y = x + (1 - mu_y)(z - x) on every block."""
        if self.cfg.averaging is None or self.train_mode:
            return
        mu_y, _ = self._interp_coeffs(None)
        for w, st in zip(self.blocks, self.state):
            w.add_((st["weight_buffer"] - w) * float(1 - mu_y))
        self.train_mode = True

    def eval(self) -> None:
        """distributed_shampoo.py:1763-1797: x = y + (1 - 1/mu_y)(z - y) on every block."""
        if self.cfg.averaging is None or not self.train_mode:
            return
        mu_y, _ = self._interp_coeffs(None)
        for w, st in zip(self.blocks, self.state):
            w.add_((st["weight_buffer"] - w) * float(1 - torch.reciprocal(mu_y)))
        self.train_mode = False
