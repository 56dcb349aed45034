"""`optimizers_amd.matrix_functions` (the module-level seam of the reference: matrix_inverse_root and
matrix_eigendecomposition) against the reference's own known answers (preconditioner/tests/matrix_functions_test.py),
its error behaviour, the oracle and fp64 truth."""

import logging
import re
from dataclasses import dataclass
from fractions import Fraction

import pytest
import torch

from tests.golden_cases import rel_err

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")

DIAG = (torch.tensor([[1.0, 0.0], [0.0, 4.0]]), torch.tensor([[1.0, 0.0], [0.0, 0.5]]))
DENSE = (
    torch.tensor([[1195.0, -944.0, -224.0], [-944.0, 746.0, 177.0], [-224.0, 177.0, 42.0]]),
    torch.tensor([[1.0, 1.0, 1.0], [1.0, 2.0, -3.0], [1.0, -3.0, 18.0]]),
)
DENSE_EIGENVALUES = torch.tensor([2.9008677229e-03, 1.7424316704e-01, 1.9828229980e03])
DENSE_EIGENVECTORS = torch.tensor(
    [
        [0.0460073575, -0.6286827326, 0.7762997746],
        [-0.1751257628, -0.7701635957, -0.6133345366],
        [0.9834705591, -0.1077321917, -0.1455317289],
    ]
)


def _configs():
    import optimizers_amd as oa

    return [
        oa.EigenConfig(),
        oa.CoupledNewtonConfig(),
        oa.EigenConfig(rank_deficient_stability_config=oa.PerturbationConfig(perturb_before_computation=False)),
        oa.EigenConfig(rank_deficient_stability_config=oa.PseudoInverseConfig(rank_rtol=None)),
        *(oa.CoupledHigherOrderConfig(rel_epsilon=0.0, abs_epsilon=0.0, order=order) for order in range(2, 7)),
    ]


@pytest.mark.parametrize("which", range(9))
@pytest.mark.parametrize("exp", (1, 2))
@pytest.mark.parametrize("case", (DIAG, DENSE), ids=("diagonal", "dense"))
def test_matrix_inverse_root_known_answers(case, exp, which):
    """matrix_functions_test.py:216-273: A^(-exp/2) for every root-inverse config, atol 0.05, rtol 1e-2."""
    from optimizers_amd.matrix_functions import matrix_inverse_root

    A, root_mat = case
    cfg = _configs()[which]
    X = matrix_inverse_root(A=A.to(DEV), root=Fraction(2, exp), root_inv_config=cfg)
    torch.testing.assert_close(torch.linalg.matrix_power(root_mat, exp), X.cpu(), atol=0.05, rtol=1e-2)


def test_matrix_inverse_root_error_behaviour(caplog):
    """matrix_functions_test.py:62-110, 287-300, 337-395."""
    import optimizers_amd as oa
    from optimizers_amd.matrix_functions import matrix_eigendecomposition, matrix_inverse_root

    A = torch.tensor([[1.0, 0.0], [0.0, 4.0]], device=DEV)
    with pytest.raises(ValueError, match=re.escape("Matrix is not 2-dimensional!")):
        matrix_inverse_root(A=torch.zeros(1, 2, 3, device=DEV), root=Fraction(2))
    with pytest.raises(ValueError, match=re.escape("Matrix is not square!")):
        matrix_inverse_root(A=torch.zeros(2, 3, device=DEV), root=Fraction(2))
    with pytest.raises(ValueError, match=re.escape("root.denominator=3 must be equal to 1 to use coupled inverse Newton iteration!")):
        matrix_inverse_root(A=A, root=Fraction(2, 3), root_inv_config=oa.CoupledNewtonConfig())
    with pytest.raises(ValueError, match=re.escape("Root -1 should be positive!")):
        matrix_inverse_root(A=A, root=Fraction(-1))
    with pytest.raises(ValueError, match=re.escape("epsilon=1e-08 should be 0.0 when using pseudo-inverse!")):
        matrix_inverse_root(A=A, root=Fraction(2), epsilon=1e-8, root_inv_config=oa.EigenConfig(
            rank_deficient_stability_config=oa.PseudoInverseConfig(rank_rtol=None)))

    @dataclass
    class NotSupportedRootInvConfig(oa.RootInvConfig):
        unsupported_root: int = -1

    with pytest.raises(NotImplementedError, match=r"Root inverse config is not implemented! Specified root inverse config is root_inv_config=.*NotSupportedRootInvConfig\(.*\)\."):
        matrix_inverse_root(A=A, root=Fraction(4), root_inv_config=NotSupportedRootInvConfig())
    # ill-conditioned input, no iterations allowed: the residual gate of the higher-order method raises
    B = torch.tensor([[1.0, 0.0], [0.0, 1e-4]], device=DEV)
    with pytest.raises(ArithmeticError):
        matrix_inverse_root(A=B, root=Fraction(2), root_inv_config=oa.CoupledHigherOrderConfig(
            rel_epsilon=0.0, abs_epsilon=0.0, max_iterations=0))
    with caplog.at_level(logging.WARNING):
        matrix_inverse_root(A=A, root=Fraction(4), root_inv_config=oa.CoupledNewtonConfig(max_iterations=1))
    assert any("Newton did not converge and reached maximum number of iterations!" in r.message for r in caplog.records)

    @dataclass
    class NotSupportedEigendecompositionConfig(oa.EigendecompositionConfig):
        unsupported_field: int = 0

    with pytest.raises(NotImplementedError, match=re.escape(
            "Eigendecomposition config is not implemented! Specified eigendecomposition config is NotSupportedEigendecompositionConfig.")):
        matrix_eigendecomposition(A=A, eigendecomposition_config=NotSupportedEigendecompositionConfig())
    with pytest.raises(ValueError, match=re.escape(
            "eigenvectors_estimate should be passed to matrix_eigendecomposition when using tolerance != 0.0.")):
        matrix_eigendecomposition(A=A, eigendecomposition_config=oa.EighEigendecompositionConfig(tolerance=0.01))
    with pytest.raises(ValueError, match=re.escape("epsilon=1e-08 should be 0.0 when using pseudo-inverse!")):
        matrix_eigendecomposition(A=torch.ones(2, 2, device=DEV), epsilon=1e-8, eigendecomposition_config=oa.EighEigendecompositionConfig(
            rank_deficient_stability_config=oa.PseudoInverseConfig(rank_rtol=None)))
    with pytest.raises(RuntimeError, match="MI355X only"):
        matrix_inverse_root(A=A.cpu(), root=Fraction(2))


def _align_signs(vectors, expected):
    vectors = vectors.clone()
    vectors[:, expected[0, :] / vectors[0, :] < 0] *= -1
    return vectors


@pytest.mark.parametrize("perturb_before_computation", (False, True))
def test_matrix_eigendecomposition_with_eigh_known_answers(perturb_before_computation):
    """matrix_functions_test.py:700-755 (eigenvector signs aligned: a sign is not defined).  Eigenvectors to the
    reference's atol 1e-4; eigenvalues to 2.5e-4 = fp32 machine epsilon x |A|_2 (1983), which is all a backward
    stable fp32 solver guarantees: the middle eigenvalue 0.17424 comes out 1.2e-4 off (LAPACK's own fp32 result
    happens to land inside the reference's 1e-4 on this matrix)."""
    import optimizers_amd as oa
    from optimizers_amd.matrix_functions import matrix_eigendecomposition

    cfg = oa.EighEigendecompositionConfig(
        rank_deficient_stability_config=oa.PerturbationConfig(perturb_before_computation=perturb_before_computation))
    L, Q = matrix_eigendecomposition(A=DIAG[0].to(DEV), eigendecomposition_config=cfg)
    torch.testing.assert_close((torch.tensor([1.0, 4.0]), torch.eye(2)), (L.cpu(), _align_signs(Q.cpu(), torch.eye(2) + 1e-9)), atol=1e-4, rtol=1e-5)
    L, Q = matrix_eigendecomposition(A=DENSE[0].to(DEV), eigendecomposition_config=cfg)
    torch.testing.assert_close(DENSE_EIGENVALUES, L.cpu(), atol=2.5e-4, rtol=1e-5)
    torch.testing.assert_close(DENSE_EIGENVECTORS, _align_signs(Q.cpu(), DENSE_EIGENVECTORS), atol=1e-4, rtol=1e-5)


def test_matrix_eigendecomposition_keeps_a_good_estimate():
    """matrix_functions_test.py:757-775: tolerance criterion met, the estimate and diag(Q^T A Q) come back."""
    import optimizers_amd as oa
    from optimizers_amd.matrix_functions import matrix_eigendecomposition

    L, Q = matrix_eigendecomposition(
        A=DIAG[0].to(DEV), eigendecomposition_config=oa.EighEigendecompositionConfig(tolerance=0.01),
        eigenvectors_estimate=torch.eye(2, device=DEV))
    torch.testing.assert_close((torch.tensor([1.0, 4.0]), torch.eye(2)), (L.cpu(), Q.cpu()))
    # a permuted identity is an exact eigenbasis too: it is kept, with its eigenvalues in its own order
    P = torch.tensor([[0.0, 1.0], [1.0, 0.0]], device=DEV)
    L, Q = matrix_eigendecomposition(
        A=DIAG[0].to(DEV), eigendecomposition_config=oa.EighEigendecompositionConfig(tolerance=0.01), eigenvectors_estimate=P)
    torch.testing.assert_close((torch.tensor([4.0, 1.0]), P.cpu()), (L.cpu(), Q.cpu()))


@pytest.mark.parametrize("start", ("identity", "eigh"))
@pytest.mark.parametrize("case", ("diagonal", "dense"))
def test_matrix_eigendecomposition_with_qr_known_answers(case, start):
    """matrix_functions_test.py:777-839: QR iterations to convergence, atol 2e-3, rtol 1e-5."""
    import optimizers_amd as oa
    from optimizers_amd.matrix_functions import matrix_eigendecomposition

    A, want_l, want_q = (
        (DIAG[0], torch.tensor([1.0, 4.0]), torch.eye(2)) if case == "diagonal" else (DENSE[0], DENSE_EIGENVALUES, DENSE_EIGENVECTORS)
    )
    A = A.to(DEV)
    init = torch.eye(A.shape[0], device=DEV) if start == "identity" else matrix_eigendecomposition(A)[1]
    L, Q = matrix_eigendecomposition(
        A=A, eigenvectors_estimate=init, eigendecomposition_config=oa.QREigendecompositionConfig(max_iterations=10_000))
    Q = _align_signs(Q.cpu(), want_q + 1e-9)
    torch.testing.assert_close((want_l, want_q), (L.cpu(), Q), atol=2e-3, rtol=1e-5)


@pytest.mark.parametrize("d", (64, 300, 700))
def test_larger_matrices_against_fp64(d):
    import optimizers_amd as oa
    from optimizers_amd.matrix_functions import matrix_eigendecomposition, matrix_inverse_root

    g = torch.Generator().manual_seed(d)
    a = torch.randn(d, 3 * d, generator=g)
    A = a @ a.T / (3 * d)
    lam, q = torch.linalg.eigh(A.double())
    for cfg, root in ((oa.EigenConfig(), Fraction(4)), (oa.CoupledNewtonConfig(), Fraction(4)), (oa.EigenConfig(), Fraction(3, 2)),
                      (oa.CoupledHigherOrderConfig(rel_epsilon=0.0, abs_epsilon=0.0), Fraction(2))):
        X = matrix_inverse_root(A.to(DEV), root, cfg, 0.0 if isinstance(cfg, oa.CoupledHigherOrderConfig) else 1e-12)
        truth = q * lam.pow(-1.0 / float(root)) @ q.T
        assert rel_err(X.cpu(), truth) < 1e-3, (type(cfg).__name__, root)
    L, Q = matrix_eigendecomposition(A.to(DEV))
    assert rel_err(L.cpu(), lam) < 1e-5
    Qd = Q.cpu().double()
    assert (Qd.T @ Qd - torch.eye(d, dtype=torch.float64)).abs().max() < 1e-5
    assert rel_err(Qd * L.cpu().double() @ Qd.T, A.double()) < 1e-5


@pytest.mark.parametrize("d", (200, 768, 1024))
def test_symmetric_products_converge_like_full_products(d, caplog):
    """Product policy 1 (every Newton product computed on the upper-triangle tiles and mirrored, operands read
    through their transpose) must converge in the iterations the reference's full products need (+-1 where the error
    hovers at the tolerance) and give the same inverse root to well below the 1e-3 bar: every symmetric product has to
    leave an exactly mirrored matrix, diagonal tiles included."""
    import optimizers_amd as oa
    from optimizers_amd import native
    from optimizers_amd.matrix_functions import _plan_for, matrix_inverse_root

    gen = torch.Generator().manual_seed(d)
    G = torch.randn(d, 3 * d // 2, generator=gen, dtype=torch.float64)
    A = (G @ G.T / G.shape[1]).float().to(DEV)
    lib = native.load()
    results, counts = [], []
    try:
        for policy in (0, 1):
            lib.sa_set_symmetric_newton(policy)
            with caplog.at_level(logging.WARNING):
                caplog.clear()
                X = matrix_inverse_root(A=A, root=Fraction(4), root_inv_config=oa.CoupledNewtonConfig(), epsilon=1e-12)
            assert not any("did not converge" in r.message for r in caplog.records), f"policy {policy} did not converge"
            results.append(X)
            counts.append(int(_plan_for(A, False, 4).iterations[0]))
    finally:
        lib.sa_set_symmetric_newton(2)
    assert abs(counts[0] - counts[1]) <= 1, counts
    assert rel_err(results[1], results[0]) <= 1e-4
    lam, Q = torch.linalg.eigh(A.double().cpu())
    truth = (Q * lam.pow(-0.25)) @ Q.T
    assert rel_err(results[1].double().cpu(), truth) <= 1e-3


@pytest.mark.parametrize("d", (512, 700, 1000))
def test_qr_refresh_of_large_matrices_against_fp64(d):
    """One QR iteration from a perturbed eigenbasis at orders where the Householder panels are gathered into outer blocks
    (block reflectors merged, one trailing update per block; 700 and 1000 end in ragged blocks): the new basis must be
    the oracle's in fp64 (matrix_functions.py:799-852) up to column signs, and orthonormal to fp32 rounding."""
    import optimizers_amd as oa
    from optimizers_amd.matrix_functions import matrix_eigendecomposition
    from oracle.shampoo_oracle import qr_refresh
    from tests.golden_cases import assert_reordering_is_between_ties

    g = torch.Generator().manual_seed(d)
    a = torch.randn(d, 2 * d, generator=g, dtype=torch.float64)
    A = a @ a.T / (2 * d) + 0.5 * torch.eye(d, dtype=torch.float64)  # condition number ~ 7: the factorization is well posed
    q0 = torch.linalg.qr(torch.linalg.eigh(A)[1] + 0.02 * torch.randn(d, d, generator=g, dtype=torch.float64))[0]
    want_l, want_q = qr_refresh(A, q0, max_iterations=1)
    L, Q = matrix_eigendecomposition(
        A=A.float().to(DEV), eigenvectors_estimate=q0.float().to(DEV),
        eigendecomposition_config=oa.QREigendecompositionConfig(max_iterations=1))
    Qd = Q.cpu().double()
    assert (Qd.T @ Qd - torch.eye(d, dtype=torch.float64)).abs().max() < 2e-5
    # The refresh ends with a stable sort of the eigenvalue estimates (matrix_functions.py:848-850): two estimates that
    # agree to fp32 rounding may come out in either order, so the columns are matched by direction first, and any that
    # sit elsewhere than in the fp64 run must be such ties (Rayleigh quotients in float64).
    match = (want_q.T @ Qd).abs().argmax(dim=1)
    assert sorted(match.tolist()) == list(range(d)), "the columns are not a permutation of the oracle's"
    moved, gap = assert_reordering_is_between_ties(match, Qd, A, f"order {d}")
    print(f"order {d}: {moved} columns in another position than in the fp64 run, estimates {gap:.1e} apart", flush=True)
    Qm = Qd[:, match]
    signs = torch.sign((Qm * want_q).sum(0))
    assert rel_err(Qm * signs, want_q) < 1e-4
    assert rel_err(L.cpu().double()[match], want_l) < 1e-5
