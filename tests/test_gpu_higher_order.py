"""CoupledHigherOrderConfig on the MI355X (through the C ABI): the batched higher-order iteration against the
oracle, the fixtures the real reference wrote, and fp64 truth; failure and iteration-limit semantics."""

import logging
from fractions import Fraction

import pytest
import torch

from tests.golden_cases import load_npz, rel_err

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _pack(a: torch.Tensor) -> torch.Tensor:
    r, c = torch.triu_indices(a.shape[0], a.shape[0])
    return a[r, c]


def _unpack(v: torch.Tensor, d: int) -> torch.Tensor:
    out = torch.zeros(d, d, dtype=v.dtype)
    r, c = torch.triu_indices(d, d)
    out[r, c] = v
    out[c, r] = v
    return out


def solve_native(A: torch.Tensor, root: int, cfg, tolerated: int = 3):
    """Runs the native amortized computation on a d x d block whose two factor matrices are set to A."""
    import optimizers_amd as oa

    d = A.shape[0]
    p = torch.nn.Parameter(torch.zeros(d, d, device=DEV))
    opt = oa.DistributedShampoo(
        [p], lr=0.0, betas=(0.0, 1.0), epsilon=1e-12, max_preconditioner_dim=d, precondition_frequency=1,
        start_preconditioning_step=1000, use_bias_correction=False,
        preconditioner_config=oa.RootInvShampooPreconditionerConfig(
            amortized_computation_config=cfg, inverse_exponent_override={2: 1.0 / root},
            num_tolerated_failed_amortized_computations=tolerated),
        grafting_config=oa.SGDPreconditionerConfig(),
    )
    p.grad = torch.zeros(d, d, device=DEV)
    opt.step()  # binds the block; factors stay zero
    st = opt.state[p]["block_0"]["shampoo"]
    for j in range(2):
        st["factor_matrices"][j].copy_(_pack(A).to(DEV))
    ng = opt._groups[0]

    def run():
        ng._amortized_computation(opt.param_groups[0], 1.0, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        return _unpack(st["inv_factor_matrices"][0].cpu(), d), int(ng.iterations[0]), int(ng.status[0])

    return run


def test_reference_trajectories():
    """Every stored input of the reference (tests/golden/higher_order_trajectories.npz): same X, or the same refusal."""
    import optimizers_amd as oa
    from optimizers_amd import native

    z = load_npz("higher_order_trajectories")
    names = sorted({k[: -len("_meta")] for k in z if k.endswith("_meta")})
    for n in names:
        root, order, maxit, iters, raised = (int(v) for v in z[n + "_meta"])
        rel, ab, tol = (float(v) for v in z[n + "_eps"])
        print(f"case {n} root={root} order={order}", flush=True)
        A = torch.from_numpy(z[n + "_A"])
        cfg = oa.CoupledHigherOrderConfig(rel_epsilon=rel, abs_epsilon=ab, max_iterations=maxit, tolerance=tol, order=order)
        X, it, status = solve_native(A, root, cfg)()
        if raised:
            assert status == native.SA_FACTOR_SOLVER_FAILED, n
            assert torch.equal(X, torch.eye(A.shape[0])), n  # the stored inverse is untouched
            continue
        assert status in (native.SA_FACTOR_OK, native.SA_FACTOR_NOT_CONVERGED), (n, status)
        # the loop ends on a rounding-level event (the error stops shrinking): allow a few iterations either way
        assert abs(it - iters) <= 3, (n, it, iters)
        want = torch.from_numpy(z[n + "_X"])
        want = _unpack(_pack(want), A.shape[0])  # the stored inverse is the mirrored upper triangle
        lam = torch.linalg.eigvalsh(A.double())
        ridge = max(rel * float(A.abs().sum(1).max()), ab)
        cond = float((lam.max() + ridge) / (lam.min().clamp_min(0.0) + ridge))
        # both fp32 results sit ~3e-9 x cond away from exact arithmetic
        assert rel_err(X, want) < 1e-3 + 1e-8 * cond, (n, rel_err(X, want), cond)


@pytest.mark.parametrize("order", [2, 3, 4, 8])
@pytest.mark.parametrize("d, root", [(200, 4), (384, 2), (130, 1), (520, 4), (96, 8)])
def test_matches_oracle_and_fp64_truth(d, root, order):
    import optimizers_amd as oa
    from oracle.shampoo_oracle import higher_order_inverse_root

    print(f"case d={d} root={root} order={order}", flush=True)
    g = torch.Generator().manual_seed(d + root + order)
    a = torch.randn(d, 3 * d, generator=g)
    A = a @ a.T / (3 * d)
    cfg = oa.CoupledHigherOrderConfig(rel_epsilon=1e-7, abs_epsilon=1e-12, order=order)
    X, it, status = solve_native(A, root, cfg)()
    want, _, flag, it_ref, _ = higher_order_inverse_root(A, Fraction(root), 1e-7, 1e-12, 100, 1e-8, order)
    lam, q = torch.linalg.eigh(A.double())
    truth = q * lam.pow(-1.0 / root) @ q.T
    assert status == 0
    assert rel_err(X, _unpack(_pack(want), d)) < 1e-3
    assert rel_err(X, truth) < 1e-3
    assert abs(it - it_ref) <= 3, (it, it_ref)


def test_failure_keeps_previous_inverse_and_is_tolerated_three_times():
    """A rank-deficient factor without any ridge fails the residual gate (matrix_functions.py:622-632): the reference
    swallows the ArithmeticError, keeps the old inverse and gives up after num_tolerated + 1 consecutive failures."""
    import optimizers_amd as oa
    from optimizers_amd import native

    g = torch.Generator().manual_seed(5)
    a = torch.randn(40, 24, generator=g)
    A = a @ a.T
    run = solve_native(A, 4, oa.CoupledHigherOrderConfig(rel_epsilon=0.0, abs_epsilon=0.0), tolerated=2)
    for _ in range(2):
        X, _, status = run()
        assert status == native.SA_FACTOR_SOLVER_FAILED
        assert torch.equal(X, torch.eye(40))
    with pytest.raises(ValueError, match="exceeded the allowed tolerance"):
        run()


def test_iteration_limit_warns_and_keeps_the_result(caplog):
    import optimizers_amd as oa
    from optimizers_amd import native

    g = torch.Generator().manual_seed(6)
    a = torch.randn(128, 512, generator=g)
    A = a @ a.T / 512
    X, it, status = solve_native(A, 4, oa.CoupledHigherOrderConfig(rel_epsilon=0.0, abs_epsilon=0.0))()
    assert status == native.SA_FACTOR_OK and it >= 4
    with caplog.at_level(logging.WARNING):
        X2, it2, status2 = solve_native(
            A, 4, oa.CoupledHigherOrderConfig(rel_epsilon=0.0, abs_epsilon=0.0, max_iterations=it - 2))()
    assert it2 == it - 2 and status2 == native.SA_FACTOR_NOT_CONVERGED
    assert any("Higher order method did not converge" in r.message for r in caplog.records)
    assert rel_err(X2, X) < 1e-2  # two iterations short of the end: already close


def test_fractional_root_and_order_limits_are_rejected():
    import optimizers_amd as oa

    p = torch.nn.Parameter(torch.zeros(8, 8, device=DEV))
    with pytest.raises(NotImplementedError, match="fractional root"):
        oa.DistributedShampoo([p], max_preconditioner_dim=8, preconditioner_config=oa.RootInvShampooPreconditionerConfig(
            amortized_computation_config=oa.CoupledHigherOrderConfig(rel_epsilon=0.0, abs_epsilon=0.0),
            inverse_exponent_override={2: 0.4}))
    with pytest.raises(NotImplementedError, match="orders 2..8"):
        oa.DistributedShampoo([p], preconditioner_config=oa.RootInvShampooPreconditionerConfig(
            amortized_computation_config=oa.CoupledHigherOrderConfig(rel_epsilon=0.0, abs_epsilon=0.0, order=9)))
