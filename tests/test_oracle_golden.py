"""Pins the oracle against the fixtures the real reference wrote (CPU fp32), and
against what the reference's own tests and the mathematics fix."""

import json
import os

import numpy as np
import pytest
import torch

from oracle import shampoo_oracle as O
from tests.golden_cases import GOLDEN, align_oracle_to_fixture, grad_stream, initial_params, load_cases, load_npz, oracle_config, rel_err

CASES = load_cases()


HORIZON_CASES = [n for n in CASES if n.startswith("horizon_")]


@pytest.mark.parametrize("name", [n for n in CASES if n != "cfg1_override" and n not in HORIZON_CASES])
def test_multi_step_matches_reference(name):
    c = CASES[name]
    z = load_npz(name)
    params = [p.clone() for p in initial_params(c)]
    opt = O.ShampooOracle(params, oracle_config(c))
    its = []
    for s, grads in grad_stream(c):
        if "lr_schedule" in c:
            opt.cfg.lr = c["lr_schedule"][s - 1]
        opt.step(grads)
        if c.get("toggle_eval_at") == s:
            opt.eval()
            for i, p in enumerate(params):
                assert rel_err(p.reshape(-1), z[f"eval_p{i}"]) < 5e-6
            opt.train()
        its.append([i for blk in opt.last_newton_iterations for i in blk])
        for i, p in enumerate(params):
            assert p.double().norm().item() == pytest.approx(float(z[f"norm_s{s}_p{i}"]), rel=2e-6)
    for i, p in enumerate(params):
        assert rel_err(p.reshape(-1), z[f"final_p{i}"]) < 5e-6
    if c["preconditioner"] in ("newton", "higher_order"):
        ref_it = z["newton_iterations"]
        for r, row in enumerate(its):
            assert row == [int(v) for v in ref_it[r] if v >= 0]
    # state tensors
    bi = 0
    for pi, nb in enumerate(opt.num_blocks_per_param):
        for k in range(nb):
            st = opt.state[bi]
            pre = f"state_p{pi}_block_{k}_"
            for j, f in enumerate(st["factors"]):
                assert rel_err(f, z[pre + f"factor_matrices_{j}"]) < 2e-6
            for j, f in enumerate(st.get("inv", [])):
                assert rel_err(f, z[pre + f"inv_factor_matrices_{j}"]) < 2e-5
            for j, f in enumerate(st.get("eigvecs", [])):
                assert rel_err(f, z[pre + f"factor_matrices_eigenvectors_{j}"]) < 2e-5
            for j, f in enumerate(st.get("eigvals", [])):
                assert rel_err(f, z[pre + f"factor_matrices_eigenvalues_{j}"]) < 2e-5
            if "corrected" in st:
                assert rel_err(st["corrected"], z[pre + "corrected_eigenvalues"]) < 2e-5
            if "adagrad" in st:
                assert rel_err(st["adagrad"], z[pre + "adagrad"]) < 2e-6
            if "filtered_grad" in st:
                assert rel_err(st["filtered_grad"], z[pre + "filtered_grad"]) < 2e-6
            if "weight_buffer" in st:
                assert rel_err(st["weight_buffer"], z[pre + "weight_buffer"]) < 5e-6
            if "momentum_buffer" in st:
                assert rel_err(st["momentum_buffer"], z[pre + "momentum_buffer"]) < 2e-5
            bi += 1


@pytest.mark.parametrize("name", HORIZON_CASES)
def test_benchmark_horizons_match_reference(name):
    """The mid-size cases that run the benchmark configurations' step counts and cadences (20 steps of Newton on a ragged
    GPT-2 slice and on a Llama slice, 50 steps of SOAP with a QR refresh every 10, 100 steps with an eigendecomposition
    every 50): subsampled parameters after every step, final parameters and Newton iteration counts."""
    c = CASES[name]
    z = load_npz(name)
    params = [p.clone() for p in initial_params(c)]
    opt = O.ShampooOracle(params, oracle_config(c))
    reordered = []
    if c.get("basis_signature"):
        # The QR refresh ends with a stable sort of eigenvalue estimates (matrix_functions.py:848-850); estimates tied
        # within their rounding error come out in either order depending on the host's BLAS kernels and thread count
        # (the run of this very oracle on another machine differs from the fixture by 4e-3 after 50 steps for that
        # reason alone).  The fixture records the order of the reference's run; ties, and only ties, follow it.
        align_oracle_to_fixture(opt, z, reordered)
    worst = 0.0
    for s, grads in grad_stream(c):
        opt.step(grads)
        for i, p in enumerate(params):
            worst = max(worst, rel_err(p.reshape(-1)[:: c["trace_stride"]], z[f"trace_s{s}_p{i}"]))
        if c["preconditioner"] == "newton":
            got = [i for blk in opt.last_newton_iterations for i in blk]
            assert got == [int(v) for v in z["newton_iterations"][s - 1] if v >= 0], s
    final = max(rel_err(p.reshape(-1)[::37], z[f"final_p{i}"]) for i, p in enumerate(params))
    print(f"{name}: oracle vs reference, worst per-step {worst:.2e}, final {final:.2e}; tied columns put in the "
          f"reference run's order: {sum(m for *_, m, _ in reordered)}")
    assert worst < 1e-5 and final < 1e-5


def test_config1_with_override_matches_reference():
    c = CASES["cfg1_override"]
    z = load_npz("cfg1_override")
    params = [p.clone() for p in initial_params(c)]
    opt = O.ShampooOracle(params, oracle_config(c))
    for s, grads in grad_stream(c):
        opt.step(grads)
        got = [i for blk in opt.last_newton_iterations for i in blk]
        assert got == [int(v) for v in z["newton_iterations"][s - 1] if v >= 0]
        for i, p in enumerate(params):
            assert p.double().norm().item() == pytest.approx(float(z[f"norm_s{s}_p{i}"]), rel=1e-5)
    for i, p in enumerate(params):
        assert rel_err(p.reshape(-1)[::37], z[f"final_p{i}"]) < 1e-5


def test_config1_as_stated_raises_like_reference():
    """benchmark configuration 1 verbatim makes the reference raise PreconditionerValueError at
    step 1 on the bias block's rank-1 factor; the oracle must fail the same way."""
    with open(os.path.join(GOLDEN, "cfg1_as_stated.json")) as f:
        rec = json.load(f)
    assert rec["raised"] and rec["step"] == 1 and rec["type"] == "PreconditionerValueError"
    c = dict(CASES["cfg1_override"], override_1d=False)
    params = [p.clone() for p in initial_params(c)]
    opt = O.ShampooOracle(params, oracle_config(c))
    _, grads = next(iter(grad_stream(c)))
    with pytest.raises(O.OraclePreconditionerValueError) as e:
        opt.step(grads)
    assert str(e.value).startswith("Encountered nan or inf values in")
    assert "1.block_0.0" in str(e.value) and "1.block_0.0" in rec["message_prefix"]


def test_newton_trajectories():
    z = load_npz("newton_trajectories")
    names = sorted({k[: -len("_meta")] for k in z if k.endswith("_meta")})
    assert len(names) == 7
    for n in names:
        root, iters, finite = (int(v) for v in z[n + "_meta"])
        A = torch.from_numpy(z[n + "_A"])
        X, _, _, it, _ = O.newton_inverse_root(A, root, float(z[n + "_eps"]))
        assert it == iters, n
        assert bool(torch.isfinite(X).all()) == bool(finite), n
        if finite:
            assert rel_err(X, z[n + "_X"]) < 1e-5, n


def test_higher_order_trajectories():
    """CoupledHigherOrderConfig on stored inputs: the reference's X, iteration count, or the fact that it raised."""
    from fractions import Fraction

    z = load_npz("higher_order_trajectories")
    names = sorted({k[: -len("_meta")] for k in z if k.endswith("_meta")})
    assert len(names) == 13
    for n in names:
        root, order, maxit, iters, raised = (int(v) for v in z[n + "_meta"])
        rel, ab, tol = (float(v) for v in z[n + "_eps"])
        A = torch.from_numpy(z[n + "_A"])
        try:
            X, _, _, it, _ = O.higher_order_inverse_root(A, Fraction(root), rel, ab, maxit, tol, order)
        except O.OracleArithmeticError:
            assert raised, n
            continue
        assert not raised, n
        assert it == iters, n
        assert rel_err(X, z[n + "_X"]) < 1e-5, n


def test_eigh_and_qr_cases():
    z = load_npz("eig_cases")
    A = torch.from_numpy(z["eigh_A"])
    assert rel_err(O.eigh_inverse_root(A, 4, 1e-12), z["eigh_X_r4"]) < 1e-5
    A2 = torch.from_numpy(z["eigh_def_A"])
    assert rel_err(O.eigh_inverse_root(A2, 2, 1e-3), z["eigh_def_X_r2_eps1e-3"]) < 1e-5
    A = torch.from_numpy(z["qr_A"])
    A3 = torch.from_numpy(z["qr_A3"])
    l1, Q1 = O.qr_refresh(A, torch.eye(40), 1e-12)
    assert rel_err(l1, z["qr_l1"]) < 1e-5 and rel_err(Q1, z["qr_Q1"]) < 1e-5
    l2, Q2 = O.qr_refresh(A3, Q1, 1e-12)
    assert rel_err(l2, z["qr_l2"]) < 1e-5 and rel_err(Q2, z["qr_Q2"]) < 1e-5
    l3, Q3 = O.qr_refresh(A3, Q2, 1e-12, max_iterations=5, tolerance=0.05)
    assert rel_err(l3, z["qr_l3"]) < 1e-5 and rel_err(Q3, z["qr_Q3"]) < 1e-5
