"""The `PreconditionerList` seam (optimizers_amd/preconditioner_list.py) driven the way the reference's own tests
drive its classes (preconditioner/tests/shampoo_preconditioner_list_test.py, preconditioner_list_test_utils.py):
same block lists, same gradients, same closed-form expectations; every solver the native path has."""

import math
import re
from dataclasses import replace

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
SOLVERS = ("eigh", "newton", "higher_order", "eigendecomposed_eigh", "eigendecomposed_qr", "kl_eigh", "kl_eigendecomposed_qr")


def _config(solver):
    import optimizers_amd as oa

    if solver.startswith("kl_"):
        # RootInvKLShampooPreconditionerListTest / EigendecomposedKLShampooPreconditionerListTest (:1514-1554) inherit the
        # abstract tests: the inverse roots are the identity until the one amortized computation at the last step
        base = _config(solver[3:])
        kl = oa.EigendecomposedKLShampooPreconditionerConfig if "eigendecomposed" in solver else oa.RootInvKLShampooPreconditionerConfig
        return kl(amortized_computation_config=base.amortized_computation_config)
    if solver.startswith("eigendecomposed"):
        # EigendecomposedShampooPreconditionerList: the same abstract tests apply (shampoo_preconditioner_list_test.py:1185-1262)
        acc = oa.QREigendecompositionConfig() if solver.endswith("qr") else oa.EighEigendecompositionConfig()
        return oa.EigendecomposedShampooPreconditionerConfig(amortized_computation_config=acc)
    acc = {
        "eigh": oa.EigenConfig(),
        "newton": oa.CoupledNewtonConfig(),
        "higher_order": oa.CoupledHigherOrderConfig(rel_epsilon=0.0, abs_epsilon=0.0),
    }[solver]
    return oa.RootInvShampooPreconditionerConfig(amortized_computation_config=acc)


class Harness:
    """setUp of AbstractTest.BaseShampooPreconditionerListTest (shampoo_preconditioner_list_test.py:207-259)."""

    def __init__(self):
        from optimizers_amd.preconditioner_list import BlockInfo

        self.params = (
            torch.tensor([1.0, 2.0], device=DEV),
            torch.arange(6, dtype=torch.float, device=DEV).reshape(3, 2),
            torch.tensor(1.0, device=DEV),  # a 0D tensor
        )
        self.state = {
            self.params[0]: {"block_0": {}},
            self.params[1]: {"block_0": {}, "block_1": {}},
            self.params[2]: {"block_0": {}},
        }
        self.block_info_list = (
            BlockInfo(param=self.params[0], composable_block_ids=(0, "block_0")),
            BlockInfo(param=self.params[1], composable_block_ids=(1, "block_0")),
            BlockInfo(param=self.params[1], composable_block_ids=(1, "block_1")),
            BlockInfo(param=self.params[2], composable_block_ids=(2, "block_0")),
        )
        # maximum_preconditioner_dim = 2: params[0] is one block, params[1] splits in two
        self.block_list = (self.params[0], *torch.split(self.params[1], 2, dim=0), self.params[2])

    def instantiate(self, factory=None, **kwargs):
        import optimizers_amd as oa
        from optimizers_amd.preconditioner_list import EigendecomposedShampooPreconditionerList, RootInvShampooPreconditionerList

        from optimizers_amd.preconditioner_list import EigendecomposedKLShampooPreconditionerList, RootInvKLShampooPreconditionerList

        cfg = kwargs.get("preconditioner_config")
        if factory is None:
            for cls, lst in ((oa.EigendecomposedKLShampooPreconditionerConfig, EigendecomposedKLShampooPreconditionerList),
                             (oa.RootInvKLShampooPreconditionerConfig, RootInvKLShampooPreconditionerList),
                             (oa.EigendecomposedShampooPreconditionerConfig, EigendecomposedShampooPreconditionerList)):
                if isinstance(cfg, cls):
                    factory = lst
                    break
        return (factory or RootInvShampooPreconditionerList)(
            block_list=self.block_list, state=self.state, block_info_list=self.block_info_list, **kwargs)


def _dev(ts):
    return tuple(t.to(DEV) for t in ts)


def verify(preconditioner_list, masked_grad_lists, expected, rtol=1e-4, atol=1e-6):
    """preconditioner_list_test_utils.py:133-171."""
    for step, grads in enumerate(masked_grad_lists, start=1):
        preconditioner_list.update_preconditioners(
            masked_grad_list=_dev(grads), step=torch.tensor(step), perform_amortized_computation=step == len(masked_grad_lists))
    actual = preconditioner_list.precondition(masked_grad_list=_dev(masked_grad_lists[-1]))
    assert len(actual) == len(expected)
    for a, e in zip(actual, expected):
        assert a.shape == e.shape and a.device.type == "cuda"
        torch.testing.assert_close(a.cpu(), e, rtol=rtol, atol=atol)


GRADS1 = (torch.tensor([1.0, 0.0]), torch.eye(2) / math.sqrt(2.0), torch.tensor([[1.0, 0.0]]), torch.tensor(3.0))
GRADS2 = (torch.tensor([0.0, 1.0]), torch.eye(2) / math.sqrt(2.0), torch.tensor([[0.0, 1.0]]), torch.tensor(2.0))


@pytest.mark.parametrize("solver", SOLVERS)
def test_update_preconditioners_and_precondition(solver):
    """shampoo_preconditioner_list_test.py:684-926: factors that are multiples of the identity."""
    cfg = _config(solver)
    expected = [g.clone() for g in GRADS2]
    expected[2] /= 2.0 ** (1 / 4)
    verify(Harness().instantiate(preconditioner_config=cfg, beta2=1.0, weighting_factor=1.0, use_bias_correction=True),
           [GRADS1, GRADS2], expected)

    beta2 = 0.9
    w = 1 - beta2
    g1 = tuple(g / math.sqrt(beta2 * w) for g in GRADS1)
    g2 = tuple(g / math.sqrt(w) for g in GRADS2)
    expected = [g.clone() for g in g2]
    expected[2] /= 2.0 ** (1 / 4)
    verify(Harness().instantiate(preconditioner_config=cfg, beta2=beta2, weighting_factor=w, use_bias_correction=False),
           [g1, g2], expected)

    b1 = tuple(g * math.sqrt(1 - beta2**2) for g in g1)
    b2 = tuple(g * math.sqrt(1 - beta2**2) for g in g2)
    expected = [g.clone() for g in b2]
    expected[2] /= 2.0 ** (1 / 4)
    verify(Harness().instantiate(preconditioner_config=cfg, beta2=beta2, weighting_factor=w, use_bias_correction=True),
           [b1, b2], expected)

    # trace scaling, exponent 1/2 and 1 (:838-926)
    expected = [GRADS2[0] * 2.0 ** (1 / 4), GRADS2[1] * 2.0 ** (1 / 4), GRADS2[2], GRADS2[3]]
    verify(Harness().instantiate(preconditioner_config=replace(cfg, use_trace_scaling=True), beta2=1.0, weighting_factor=1.0),
           [GRADS1, GRADS2], expected)
    expected = [GRADS2[0] * 2.0 ** (1 / 2), GRADS2[1] * 2.0 ** (1 / 2), GRADS2[2] * 2.0 ** (1 / 4), GRADS2[3]]
    verify(Harness().instantiate(preconditioner_config=replace(cfg, use_trace_scaling=True, trace_scaling_exponent=1.0),
                                 beta2=1.0, weighting_factor=1.0), [GRADS1, GRADS2], expected)


@pytest.mark.parametrize("solver", ("eigh", "newton"))
def test_update_preconditioners_and_precondition_with_epsilon(solver):
    """:928-1020, epsilon = 80 (the higher-order iteration ignores the optimizer's epsilon, as in the reference)."""
    g1 = (torch.tensor([1.0, 0.0]), torch.eye(2) / math.sqrt(2), torch.tensor([[1.0, 0.0]]), torch.tensor(1.0))
    g2 = (torch.tensor([0.0, 1.0]), torch.eye(2) / math.sqrt(2), torch.tensor([[0.0, 1.0]]), torch.tensor(1.0))
    expected = (torch.tensor([0.0, 1.0 / 9.0]), torch.eye(2) / (9 * math.sqrt(2)),
                torch.tensor([[0.0, 1.0 / 3.0 * 82.0 ** (-1 / 4)]]), torch.tensor(1.0))
    verify(Harness().instantiate(preconditioner_config=_config(solver), beta2=1.0, weighting_factor=1.0,
                                 use_bias_correction=True, epsilon=80.0), [g1, g2], expected)


@pytest.mark.parametrize("solver", SOLVERS)
def test_update_preconditioners_and_precondition_with_dims_ignored(solver):
    """:1022-1105."""
    cfg = _config(solver)
    g1 = (torch.tensor([4.0, 0.0]), torch.eye(2) * 3, torch.tensor([[2.0, 0.0]]), torch.tensor(3.0))
    g2 = (torch.tensor([0.0, 4.0]), torch.eye(2) * 4, torch.tensor([[0.0, 2.0]]), torch.tensor(2.0))
    expected = [torch.tensor([0.0, 1.0]), g2[1] / 5, g2[2] / math.sqrt(2 * math.sqrt(8)), torch.tensor(2.0)]
    verify(Harness().instantiate(preconditioner_config=cfg, beta2=1.0, weighting_factor=1.0), [g1, g2], expected)
    ignored = replace(cfg, inverse_exponent_override={0: {0: 0.0}, 1: {0: 0.0}, 2: 0.0})
    verify(Harness().instantiate(preconditioner_config=ignored, beta2=1.0, weighting_factor=1.0), [g1, g2], g2)


@pytest.mark.parametrize("solver", SOLVERS)
def test_inverse_exponent_override(solver):
    """:1107-1182: every root is 1."""
    cfg = replace(_config(solver), inverse_exponent_override={0: {0: 1.0}, 1: {0: 1.0}, 2: 1.0})
    g1 = (torch.tensor([1.0, 0.0]), torch.eye(2) / math.sqrt(2.0), torch.tensor([[1.0, 0.0]]), torch.tensor(3.0))
    g2 = (torch.tensor([0.0, 2.0]), torch.eye(2) / math.sqrt(2.0), torch.tensor([[0.0, 2.0]]), torch.tensor(2.0))
    expected = (torch.tensor([0, 0.5]), torch.eye(2) / math.sqrt(2.0), torch.tensor([[0, 0.1]]), torch.tensor(2.0))
    verify(Harness().instantiate(preconditioner_config=cfg, beta2=1.0, weighting_factor=1.0, use_bias_correction=True),
           [g1, g2], expected)


def test_lists_sizes_and_state_layout():
    """numel / dims / bytes lists and what lands in the optimizer state (packed triangles, packed identity)."""
    h = Harness()
    pl = h.instantiate(preconditioner_config=_config("eigh"))
    assert pl.dims_list == (torch.Size([2]), torch.Size([2, 2]), torch.Size([1, 2]), torch.Size([]))
    assert pl.numel_list == (6, 12, 8, 0)  # packed factor + packed inverse per preconditioned dim
    assert pl.num_bytes_list == (24, 48, 32, 0)
    assert pl.numel() == 26 and pl.num_bytes() == 104
    st = h.state[h.params[1]]["block_0"]["shampoo"]
    assert st.factor_matrix_indices == ("1.block_0.0", "1.block_0.1") and st.roots == (4.0, 4.0)
    assert torch.equal(st.inv_factor_matrices[0].cpu(), torch.tensor([1.0, 0.0, 1.0]))
    assert torch.equal(st.factor_matrices[0].cpu(), torch.zeros(3))


@pytest.mark.parametrize("invalid_value", (float("nan"), float("inf")))
def test_raise_invalid_value_in_factor_matrix(invalid_value):
    """:261-277."""
    from optimizers_amd import PreconditionerValueError

    pl = Harness().instantiate(preconditioner_config=_config("eigh"))
    grads = (torch.tensor([invalid_value, invalid_value]), torch.eye(2) / math.sqrt(2.0),
             torch.tensor([[invalid_value, invalid_value]]), torch.tensor(invalid_value))
    with pytest.raises(PreconditionerValueError, match=re.escape("Encountered nan/inf values in factor matrix")):
        pl.update_preconditioners(masked_grad_list=_dev(grads), step=torch.tensor(1), perform_amortized_computation=True)


def test_compress_preconditioner_list():
    """Only the selected blocks are passed afterwards; the others keep their state (:1580-1620)."""
    h = Harness()
    pl = h.instantiate(preconditioner_config=_config("eigh"), beta2=1.0, weighting_factor=1.0)
    pl.compress_preconditioner_list(local_grad_selector=(True, False, True, False))
    sel1 = (GRADS1[0], GRADS1[2])
    sel2 = (GRADS2[0], GRADS2[2])
    expected = (GRADS2[0], GRADS2[2] / 2.0 ** (1 / 4))
    verify(pl, [sel1, sel2], expected)
    untouched = h.state[h.params[1]]["block_0"]["shampoo"]
    assert torch.equal(untouched.factor_matrices[0].cpu(), torch.zeros(3))
    assert torch.equal(untouched.inv_factor_matrices[1].cpu(), torch.tensor([1.0, 0.0, 1.0]))
    with pytest.raises(ValueError, match="expected 2 gradient blocks"):
        pl.precondition(masked_grad_list=_dev(GRADS2))


def test_strided_gradient_views_and_larger_blocks():
    """Column-split blocks (row stride of the parent) against the oracle's formulas in fp64."""
    from optimizers_amd.preconditioner_list import BlockInfo, RootInvShampooPreconditionerList

    g = torch.Generator().manual_seed(0)
    param = torch.randn(96, 200, generator=g).to(DEV)
    blocks = torch.split(param, 128, dim=1)  # 96 x 128 and 96 x 72, row stride 200
    state = {param: {"block_0": {}, "block_1": {}}}
    infos = tuple(BlockInfo(param=param, composable_block_ids=(0, f"block_{k}")) for k in range(2))
    pl = RootInvShampooPreconditionerList(block_list=blocks, state=state, block_info_list=infos,
                                          preconditioner_config=_config("newton"), beta2=0.99, weighting_factor=0.01,
                                          epsilon=1e-8, use_bias_correction=True)
    grads_all = [torch.randn(96, 200, generator=g) for _ in range(4)]
    for step, G in enumerate(grads_all, start=1):
        pl.update_preconditioners(masked_grad_list=torch.split(G.to(DEV), 128, dim=1), step=torch.tensor(step),
                                  perform_amortized_computation=step == 4)
    out = pl.precondition(masked_grad_list=torch.split(grads_all[-1].to(DEV), 128, dim=1))
    bc2 = 1 - 0.99**4
    for k, cols in enumerate((slice(0, 128), slice(128, 200))):
        Gs = [G[:, cols].double() for G in grads_all]
        L = sum(0.99 ** (3 - t) * 0.01 * (x @ x.T) for t, x in enumerate(Gs)) / bc2
        R = sum(0.99 ** (3 - t) * 0.01 * (x.T @ x) for t, x in enumerate(Gs)) / bc2

        def inv_root(A):
            lam, q = torch.linalg.eigh(A + 1e-8 * torch.eye(A.shape[0], dtype=torch.float64))
            return q * lam.pow(-0.25) @ q.T

        want = inv_root(L) @ Gs[-1] @ inv_root(R)
        # L (96 x 96 from at most 4 x 72..128 columns) is well conditioned; R of rank <= 384 vs order 128 / 72 too
        assert float((out[k].cpu().double() - want).norm() / want.norm()) < 1e-3


@pytest.mark.parametrize("kind", ("qr", "eigh"))
def test_eigenvalue_corrected_list_matches_oracle_formulas(kind):
    """shampoo_preconditioner_list.py:1891-1942 rebuilt in fp64 from the list's own state."""
    import optimizers_amd as oa
    from optimizers_amd.preconditioner_list import BlockInfo, EigenvalueCorrectedShampooPreconditionerList

    g = torch.Generator().manual_seed(1)
    param = torch.randn(40, 24, generator=g).to(DEV)
    state = {param: {"block_0": {}}}
    cfg = oa.DefaultSOAPConfig if kind == "qr" else oa.DefaultEigenvalueCorrectedShampooConfig
    pl = EigenvalueCorrectedShampooPreconditionerList(
        block_list=(param,), state=state, block_info_list=(BlockInfo(param=param, composable_block_ids=(0, "block_0")),),
        preconditioner_config=cfg, beta2=0.95, weighting_factor=0.05, epsilon=1e-8, use_bias_correction=True)
    grads = [torch.randn(40, 24, generator=g) for _ in range(3)]
    v = torch.zeros(40, 24, dtype=torch.float64)
    st = state[param]["block_0"]["shampoo"]
    for step, G in enumerate(grads, start=1):
        pl.update_preconditioners(masked_grad_list=(G.to(DEV),), step=torch.tensor(step), perform_amortized_computation=True)
        Q = [q.cpu().double() for q in st.factor_matrices_eigenvectors]
        v = 0.95 * v + 0.05 * (Q[0].T @ G.double() @ Q[1]) ** 2
    out = pl.precondition(masked_grad_list=(grads[-1].to(DEV),))[0]
    assert float((st.corrected_eigenvalues.cpu().double() - v).norm() / v.norm()) < 1e-5
    for q in Q:
        assert (q.T @ q - torch.eye(q.shape[0], dtype=torch.float64)).abs().max() < 1e-5
    rot = Q[0].T @ grads[-1].double() @ Q[1]
    rot = rot / ((v / (1 - 0.95**3)).sqrt() + 1e-8)
    want = Q[0] @ rot @ Q[1].T
    assert float((out.cpu().double() - want).norm() / want.norm()) < 1e-4


def test_order_three_blocks():
    """tensordot semantics of the reference for a conv-like block and a middle-dim split view of it
    (shampoo_preconditioner_list.py:1490-1578), rebuilt in fp64."""
    from optimizers_amd.preconditioner_list import BlockInfo, RootInvShampooPreconditionerList

    g = torch.Generator().manual_seed(2)
    param = torch.randn(12, 40, 9, generator=g).to(DEV)
    blocks = torch.split(param, 32, dim=1)  # 12 x 32 x 9 and 12 x 8 x 9: the middle dim is split
    state = {param: {"block_0": {}, "block_1": {}}}
    infos = tuple(BlockInfo(param=param, composable_block_ids=(0, f"block_{k}")) for k in range(2))
    pl = RootInvShampooPreconditionerList(block_list=blocks, state=state, block_info_list=infos,
                                          preconditioner_config=_config("eigh"), beta2=1.0, weighting_factor=1.0, epsilon=1e-6)
    assert state[param]["block_0"]["shampoo"].roots == (6.0, 6.0, 6.0)
    grads = [torch.randn(12, 40, 9, generator=g) for _ in range(3)]
    for step, G in enumerate(grads, start=1):
        pl.update_preconditioners(masked_grad_list=torch.split(G.to(DEV), 32, dim=1), step=torch.tensor(step),
                                  perform_amortized_computation=step == 3)
    out = pl.precondition(masked_grad_list=torch.split(grads[-1].to(DEV), 32, dim=1))
    for k, sl in enumerate((slice(0, 32), slice(32, 40))):
        Gs = [G[:, sl, :].double() for G in grads]
        want = Gs[-1]
        for dim in range(3):
            rest = [d for d in range(3) if d != dim]
            F = sum(torch.tensordot(x, x, dims=[rest, rest]) for x in Gs)
            lam, q = torch.linalg.eigh(F + 1e-6 * torch.eye(F.shape[0], dtype=torch.float64))
            X = q * lam.pow(-1.0 / 6.0) @ q.T
            want = torch.tensordot(want, X, dims=([0], [0]))  # contracts dim 0, appends the result: rotates the dims
        assert out[k].shape == want.shape
        assert float((out[k].cpu().double() - want).norm() / want.norm()) < 1e-3
