"""Pins the oracle without the reference: vectors transcribed (as data) from the
reference's own tests, library equivalences and what the mathematics fixes."""

import math

import pytest
import torch

from oracle import shampoo_oracle as O


# utils/tests/shampoo_utils_test.py:64-169 (expected shapes are the reference's)
@pytest.mark.parametrize(
    "shape, threshold, target, expected",
    [
        ((1, 2, 5, 1), 10, 1, (10,)),
        ((1, 2, 5, 1), 1, 1, (2, 5)),
        ((2,), 10, 1, (2,)),
        ((1, 1, 1, 1), 10, 1, (1,)),
        ((1, 1, 1, 1), 1, 1, (1,)),
        ((0,), 10, 1, (0,)),
        ((0, 1, 5, 10, 20), 10, 1, (0,)),
        ((1, 5, 0, 10, 20), 10, 1, (0,)),
        ((1, 5, 10, 20, 0), 10, 1, (0,)),
        ((), 10, 1, (1,)),
        ((), 1, 1, (1,)),
        ((1, 2, 5, 1), 10, math.inf, (1, 2, 5, 1)),
        ((32, 3, 64, 64), 10, 1, (32, 3, 64, 64)),
        ((32, 3, 64, 64), 200, 1, (32, 192, 64)),
        ((32, 3, 64, 64), 8192, 1, (96, 4096)),
        ((32, 3, 64, 64), 1_000_000, 1, (96 * 4096,)),
        ((32, 3, 64, 64), 10, 2, (32, 3, 64, 64)),
        ((32, 3, 64, 64), 200, 2, (32, 192, 64)),
        ((32, 3, 64, 64), 8192, 2, (96, 4096)),
        ((32, 3, 64, 64), 1_000_000, 2, (32, 3 * 4096)),
        ((32, 3, 64, 64), 8192, 3, (32, 3, 4096)),
        ((32, 3, 64, 64), 8192, 4, (32, 3, 64, 64)),
        ((32, 3, 64, 64), 8192, math.inf, (32, 3, 64, 64)),
    ],
)
def test_merge_small_dims_reference_vectors(shape, threshold, target, expected):
    assert O.merge_small_dims(shape, threshold, target) == expected


def test_multi_dim_split_reference_vectors():
    # utils/tests/shampoo_utils_test.py:172-211
    g = torch.arange(10).reshape(5, 2)
    out = O.multi_dim_split(g, 3)
    assert [o.tolist() for o in out] == [[[0, 1], [2, 3], [4, 5]], [[6, 7], [8, 9]]]
    g = torch.arange(15).reshape(5, 3)
    out = O.multi_dim_split(g, 2)
    assert [o.tolist() for o in out] == [
        [[0, 1], [3, 4]], [[2], [5]], [[6, 7], [9, 10]], [[8], [11]], [[12, 13]], [[14]],
    ]
    assert len(O.multi_dim_split(g, 5)) == 1 and len(O.multi_dim_split(g, math.inf)) == 1


@pytest.mark.parametrize("shape, b", [((7, 5), 3), ((4, 9, 2), 4), ((10,), 4), ((6, 6), 6), ((5, 3), 7)])
def test_block_order_equals_torch_split_brute_force(shape, b):
    t = torch.arange(math.prod(shape)).reshape(shape)
    want = (t,)
    for d in range(t.dim()):
        want = tuple(s for x in want for s in torch.split(x, b, dim=d))
    got = O.multi_dim_split(t, b)
    assert len(got) == len(want)
    for a, w in zip(got, want):
        assert a.shape == w.shape and torch.equal(a, w) and a.data_ptr() == w.data_ptr()


def test_pack_unpack_reference_vectors():
    # utils/tests/shampoo_utils_test.py:468-540
    assert O.pack_triu(torch.tensor([[1.0, 2.0], [3.0, 4.0]])).tolist() == [1.0, 2.0, 4.0]
    m = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0], [7.0, 8.0, 9.0]])
    assert O.pack_triu(m).tolist() == [1.0, 2.0, 3.0, 5.0, 6.0, 9.0]
    assert O.unpack_triu(torch.tensor([1.0, 2.0, 4.0]), 2).tolist() == [[1.0, 2.0], [2.0, 4.0]]
    u = O.unpack_triu(torch.tensor([1.0, 2.0, 3.0, 5.0, 6.0, 9.0]), 3)
    assert u.tolist() == [[1.0, 2.0, 3.0], [2.0, 5.0, 6.0], [3.0, 6.0, 9.0]]
    for d in (1, 2, 3, 5, 8):
        a = torch.randn(d, d)
        s = a + a.T
        assert torch.equal(O.unpack_triu(O.pack_triu(s), d), s)
        assert O.packed_dim(d * (d + 1) // 2) == d
        assert torch.equal(O.unpack_triu(O.packed_eye(d), d), torch.eye(d))


# preconditioner/tests/matrix_functions_test.py:216-273
_KNOWN = [
    (torch.tensor([[1.0, 0.0], [0.0, 4.0]]), torch.tensor([[1.0, 0.0], [0.0, 0.5]])),
    (
        torch.tensor([[1195.0, -944.0, -224.0], [-944.0, 746.0, 177.0], [-224.0, 177.0, 42.0]]),
        torch.tensor([[1.0, 1.0, 1.0], [1.0, 2.0, -3.0], [1.0, -3.0, 18.0]]),
    ),
]


@pytest.mark.parametrize("A, root_mat", _KNOWN)
def test_inverse_root_known_answers(A, root_mat):
    # root 2: A^(-1/2); root 1: A^(-1) = (A^(-1/2))^2
    x2, *_ = O.newton_inverse_root(A, 2)
    torch.testing.assert_close(x2, root_mat, atol=0.05, rtol=1e-2)
    x1, *_ = O.newton_inverse_root(A, 1)
    torch.testing.assert_close(x1, root_mat @ root_mat, atol=0.05, rtol=1e-2)
    torch.testing.assert_close(O.eigh_inverse_root(A, 2), root_mat, atol=0.05, rtol=1e-2)
    torch.testing.assert_close(O.eigh_inverse_root(A, 1), root_mat @ root_mat, atol=0.05, rtol=1e-2)


@pytest.mark.parametrize("n", [10, 100])
@pytest.mark.parametrize("root", [2, 4, 8])
def test_inverse_root_residual_on_tridiagonal_family(n, root):
    # matrix_functions_test.py:575-661: ||X^-p - A||_inf / max(1, ||A||_inf) <= 1e-4
    for alpha, beta in [(1e-3, 1e-2), (1e-2, 1e-1), (1e-1, 1.0)]:
        A = torch.zeros(n, n, dtype=torch.float64)
        i = torch.arange(n)
        A[i, i] = alpha
        A[i[:-1], i[:-1] + 1] = beta
        A[i[:-1] + 1, i[:-1]] = beta
        A = A @ A.T  # SPD by construction
        for fn in (lambda a: O.newton_inverse_root(a, root)[0], lambda a: O.eigh_inverse_root(a, root)):
            X = fn(A)
            back = torch.linalg.matrix_power(torch.linalg.inv(X), root)
            res = (back - A).abs().max() / max(1.0, A.abs().max())
            assert res <= 1e-4


def test_newton_matches_fp64_eigh_truth_and_has_no_transposed_operand():
    torch.manual_seed(3)
    g = torch.randn(40, 160, dtype=torch.float64)
    A = g @ g.T / 160
    lam, q = torch.linalg.eigh(A)
    for root in (2, 4):
        truth = (q * lam.pow(-1 / root)) @ q.T
        X, M, conv, it, err = O.newton_inverse_root(A, root, 0.0, tolerance=1e-13)
        assert conv and it < 30
        assert ((X - truth).norm() / truth.norm()) < 1e-11
        # coupled invariant: M = X^p A stays near I at convergence
        assert (torch.linalg.matrix_power(X, root) @ A - torch.eye(40, dtype=torch.float64)).abs().max() < 1e-10


def test_qr_refresh_is_one_orthogonal_iteration():
    # textbook: with Q0=I, one step gives Q1 from qr(A), B1 = R Q = Q1^T A Q1, columns sorted by diag(B1)
    torch.manual_seed(0)
    g = torch.randn(12, 30, dtype=torch.float64)
    A = g @ g.T
    vals, Q = O.qr_refresh(A, torch.eye(12, dtype=torch.float64))
    assert torch.allclose(Q.T @ Q, torch.eye(12, dtype=torch.float64), atol=1e-12)
    assert torch.all(vals[1:] >= vals[:-1])
    assert torch.allclose((Q.T @ A @ Q).diag(), vals, atol=1e-9)
    q1, _ = torch.linalg.qr(A)
    # same column space up to the permutation
    assert torch.allclose((Q.T @ q1).abs().sum(0), torch.ones(12, dtype=torch.float64), atol=1e-9)
    # reference 3x3 (matrix_functions_test.py:700-839): many iterations converge to the eigenpairs
    A3 = torch.tensor([[1.0, 0.0], [0.0, 4.0]])
    v, q = O.qr_refresh(A3, torch.eye(2), max_iterations=1, tolerance=0.0)
    torch.testing.assert_close(v, torch.tensor([1.0, 4.0]))


@pytest.mark.parametrize("wd_type", ["DECOUPLED", "L2"])
def test_grafting_only_equals_torch_adam(wd_type):
    """gpu_tests/shampoo_grafting_test.py:68-266: with preconditioning never starting,
    Shampoo + Adam grafting is Adam (L2) / AdamW (decoupled)."""
    torch.manual_seed(5)
    shapes = [(9, 7), (7,)]
    init = [torch.randn(*s) for s in shapes]
    lr, betas, eps, wd = 0.01, (0.9, 0.999), 1e-8, 0.05
    ref_p = [torch.nn.Parameter(t.clone()) for t in init]
    cls = torch.optim.AdamW if wd_type == "DECOUPLED" else torch.optim.Adam
    ref = cls(ref_p, lr=lr, betas=betas, eps=eps, weight_decay=wd)
    mine = [t.clone() for t in init]
    cfg = O.OracleConfig(
        lr=lr, betas=betas, epsilon=1e-12, weight_decay=wd, weight_decay_type=wd_type,
        max_preconditioner_dim=4, precondition_frequency=1, start_preconditioning_step=10**9,
        preconditioner="newton", grafting="adam", grafting_beta2=betas[1], grafting_epsilon=eps,
    )
    opt = O.ShampooOracle(mine, cfg)
    for _ in range(5):
        grads = [torch.randn(*s) for s in shapes]
        for p, g in zip(ref_p, grads):
            p.grad = g.clone()
        ref.step()
        opt.step([g.clone() for g in grads])
    for a, b in zip(mine, ref_p):
        torch.testing.assert_close(a, b.detach(), rtol=2e-5, atol=2e-6)


def test_closed_form_scaled_identity_factors():
    """shampoo_preconditioner_list_test.py:684-926 idea: gradients chosen so that the
    factors are c*I make the preconditioned gradient analytic.  G = a*I (n x n), beta2=1:
    L = R = a^2 I, so P = L^-1/4 G R^-1/4 = a * (a^2)^-1/2 * I = I."""
    n, a = 6, 3.0
    W = [torch.zeros(n, n)]
    cfg = O.OracleConfig(lr=1.0, betas=(0.0, 1.0), epsilon=0.0 + 1e-30, max_preconditioner_dim=8,
                         precondition_frequency=1, start_preconditioning_step=1, preconditioner="eigh",
                         use_bias_correction=False)
    opt = O.ShampooOracle(W, cfg)
    opt.step([a * torch.eye(n)])
    torch.testing.assert_close(W[0], -torch.eye(n), atol=1e-5, rtol=1e-5)
    # second step accumulates: L = R = 2 a^2 I  ->  P = a / (sqrt(2) a) I
    opt.step([a * torch.eye(n)])
    torch.testing.assert_close(W[0], -(1 + 1 / math.sqrt(2)) * torch.eye(n), atol=1e-5, rtol=1e-5)


def test_ema_factor_is_gram_ema_and_uses_raw_gradient():
    torch.manual_seed(1)
    W = [torch.randn(5, 4)]
    cfg = O.OracleConfig(lr=0.1, betas=(0.9, 0.99), epsilon=1e-6, max_preconditioner_dim=8,
                         precondition_frequency=1, start_preconditioning_step=100, preconditioner="eigh",
                         grafting="adam", use_symmetric_packing=False)
    opt = O.ShampooOracle(W, cfg)
    L = torch.zeros(5, 5)
    R = torch.zeros(4, 4)
    for _ in range(3):
        g = torch.randn(5, 4)
        L = 0.99 * L + 0.01 * g @ g.T
        R = 0.99 * R + 0.01 * g.T @ g
        opt.step([g])
    torch.testing.assert_close(opt.state[0]["factors"][0], L, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(opt.state[0]["factors"][1], R, rtol=1e-5, atol=1e-7)


def test_pseudo_inverse_root_matches_numpy_pinv_and_projector_closed_form():
    """PseudoInverseConfig branch (matrix_functions.py:206-249).  Root 1 is the Moore-Penrose inverse: numpy's
    pinv with the same relative cutoff must agree; for a scaled projector c P the root-r result is c^(-1/r) P."""
    import numpy as np

    g = torch.Generator().manual_seed(5)
    B = torch.randn(12, 5, generator=g, dtype=torch.float64)
    A = B @ B.T  # rank 5 of 12
    X = O.eigh_pseudo_inverse_root(A, 1)
    want = torch.from_numpy(np.linalg.pinv(A.numpy(), rcond=12 * torch.finfo(torch.float64).eps, hermitian=True))
    torch.testing.assert_close(X, want, atol=1e-10, rtol=1e-8)
    # the null space stays a null space for every root
    lam, q = torch.linalg.eigh(A)
    null = q[:, :7]
    for root in (2, 4):
        Xr = O.eigh_pseudo_inverse_root(A, root)
        assert float((Xr @ null).abs().max()) < 1e-10
    Q, _ = torch.linalg.qr(torch.randn(9, 3, generator=g, dtype=torch.float64))
    P = Q @ Q.T
    torch.testing.assert_close(O.eigh_pseudo_inverse_root(16.0 * P, 4), 0.5 * P, atol=1e-12, rtol=1e-10)
    # absolute tolerance: everything at or below rank_atol is dropped
    D = torch.diag(torch.tensor([4.0, 1.0, 0.25], dtype=torch.float64))
    torch.testing.assert_close(O.eigh_pseudo_inverse_root(D, 2, rank_rtol=0.0, rank_atol=0.25),
                               torch.diag(torch.tensor([0.5, 1.0, 0.0], dtype=torch.float64)))


# --- coupled higher-order iteration ------------------------------------------------------------------------


@pytest.mark.parametrize("order", range(2, 7))
@pytest.mark.parametrize("exp", (1, 2))
def test_higher_order_known_answers(order, exp):
    """The reference's own vectors (matrix_functions_test.py:216-273): A^(-exp/2) for a diagonal and a dense 3x3."""
    from fractions import Fraction

    cases = (
        (torch.tensor([[1.0, 0.0], [0.0, 4.0]]), torch.tensor([[1.0, 0.0], [0.0, 0.5]])),
        (
            torch.tensor([[1195.0, -944.0, -224.0], [-944.0, 746.0, 177.0], [-224.0, 177.0, 42.0]]),
            torch.tensor([[1.0, 1.0, 1.0], [1.0, 2.0, -3.0], [1.0, -3.0, 18.0]]),
        ),
    )
    for A, root_mat in cases:
        X, _, _, _, _ = O.higher_order_inverse_root(A, Fraction(2, exp), order=order)
        torch.testing.assert_close(torch.linalg.matrix_power(root_mat, exp), X, atol=0.05, rtol=1e-2)


def test_higher_order_coefficients_are_the_binomial_series():
    """b_i = (-1)^i binom(-1/p, i): the Taylor coefficients of (1 - x)^(-1/p)."""
    for p in (1, 2, 3, 4, 8):
        want, c = [], 1.0
        for i in range(7):
            want.append(c)
            c *= (1.0 / p + i) / (i + 1)
        assert O.higher_order_coefficients(p, 7) == pytest.approx(want, rel=1e-14)
        # and the polynomial approximates (1 - x)^(-1/p)
        x = 0.05
        assert sum(b * x**i for i, b in enumerate(want)) == pytest.approx((1 - x) ** (-1.0 / p), rel=1e-8)


@pytest.mark.parametrize("order", (2, 3, 5))
@pytest.mark.parametrize("root", (1, 2, 4))
def test_higher_order_matches_fp64_eigh_truth(order, root):
    from fractions import Fraction

    g = torch.Generator().manual_seed(3)
    a = torch.randn(24, 80, generator=g, dtype=torch.float64)
    A = a @ a.T / 80
    lam, q = torch.linalg.eigh(A)
    truth = q * lam.pow(-1.0 / root) @ q.T
    X, M, flag, it, res = O.higher_order_inverse_root(A, Fraction(root), order=order, tolerance=1e-13)
    assert flag in ("converged", "early_stop") and it < 30
    assert float((X - truth).norm() / truth.norm()) < 1e-10
    assert float((M - torch.eye(24, dtype=torch.float64)).abs().max()) < 1e-10
    # a transposed or swapped operand in X <- X M_p would break symmetry of X on this non-commuting test:
    B = A.clone()
    B[0, 1] += 0.05  # slightly non-symmetric input: X must still invert B^(1/root) to first order
    Xb, *_ = O.higher_order_inverse_root(B, Fraction(root), order=order, tolerance=1e-13)
    assert float((torch.linalg.matrix_power(Xb, root) @ B - torch.eye(24, dtype=torch.float64)).abs().max()) < 1e-8


def test_higher_order_order_two_is_newton_from_the_trace_start():
    """order 2 has M_p = I + (I - M) / p, the Newton map: from a common start both give the same iterates."""
    from fractions import Fraction

    g = torch.Generator().manual_seed(4)
    a = torch.randn(16, 40, generator=g, dtype=torch.float64)
    A = a @ a.T / 40
    X2, *_ = O.higher_order_inverse_root(A, Fraction(4), order=2, tolerance=1e-13)
    # Newton started at z = (p + 1) / (2 |A|_F) converges to the same matrix
    Xn, *_ = O.newton_inverse_root(A, 4, 0.0, 100, 1e-13)
    assert float((X2 - Xn).norm() / Xn.norm()) < 1e-10


def test_higher_order_failure_cases_of_the_reference():
    """matrix_functions_test.py:275-287, 337-370: blow-up after powering, inf input, residual gate."""
    from fractions import Fraction

    A = torch.tensor([[1.0, 0.0], [0.0, 1e-4]])
    with pytest.raises(O.OracleArithmeticError, match="after powering for fractions"):
        O.higher_order_inverse_root(A, Fraction(1, 20))
    with pytest.raises(O.OracleArithmeticError, match="close to inf"):
        O.higher_order_inverse_root(torch.tensor([[1.0, 0.0], [0.0, float("inf")]]), Fraction(2))
    with pytest.raises(O.OracleArithmeticError, match=r"exceeds threshold 1e-1"):
        O.higher_order_inverse_root(A, Fraction(2), max_iterations=0)


def test_trace_scaling_closed_form():
    """Factor c I_d scaled by trace^(-1/2) is sqrt(c / d) I: without grafting the first preconditioned
    update of a block whose factors are multiples of the identity has a closed form."""
    d, c = 8, 3.0
    A = c * torch.eye(d, dtype=torch.float64)
    scaled = A * torch.pow(torch.clamp(torch.trace(A), min=1e-12), -0.5)
    assert torch.allclose(scaled, math.sqrt(c / d) * torch.eye(d, dtype=torch.float64))
    # through the optimizer: one parameter (d x d), gradient sqrt(c) * Q with Q orthogonal gives L = R = c I
    q, _ = torch.linalg.qr(torch.randn(d, d, generator=torch.Generator().manual_seed(0), dtype=torch.float64))
    G = math.sqrt(c) * q
    W = torch.zeros(d, d, dtype=torch.float64)
    cfg = O.OracleConfig(lr=1.0, betas=(0.0, 1.0), epsilon=1e-30, max_preconditioner_dim=8, precondition_frequency=1,
                         start_preconditioning_step=1, preconditioner="eigh", use_trace_scaling=True,
                         trace_scaling_exponent=0.5)
    opt = O.ShampooOracle([W], cfg)
    opt.step([G.clone()])
    # P = L'^(-1/4) G R'^(-1/4) with L' = R' = sqrt(c / d) I  =>  W = -(c / d)^(-1/4) G
    assert torch.allclose(W, -((c / d) ** -0.25) * G, rtol=1e-9, atol=1e-12)
