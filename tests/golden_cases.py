"""Helpers shared by the golden tests: rebuild a fixture case for the oracle or the
native optimizer from the plain-data description in tests/golden/cases.json."""

from __future__ import annotations

import json
import math
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load_cases() -> dict:
    with open(os.path.join(GOLDEN, "cases.json")) as f:
        return json.load(f)


def load_npz(name: str) -> dict:
    with np.load(os.path.join(GOLDEN, f"{name}.npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def case_params(shapes, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(*s, generator=g) for s in shapes]


def case_grads(shapes, seed, step, scale):
    g = torch.Generator().manual_seed(seed * 1000 + step)
    return [scale * torch.randn(*s, generator=g) for s in shapes]


def horizon_grads(c, step):
    """Gradients of the mid-size cases that run the benchmark configurations' horizons and cadences (kept apart from
    case_grads so that the older fixtures stay bit-identical).  CPU generator, so every run sees the same bits.
      gauss:          grad_scale * N(0, 1)
      gauss_lowrank:  the same plus lowrank_scale * (a @ c) with one seeded rank-r pair (a, c) per matrix, the same
                      at every step: r outlier directions above the noise bulk (a skewed spectrum)
      graded:         grad_scale * N(0, 1) with column j scaled by 10^(-grade_decades * j / (cols - 1))
      spectrum:       U diag(s) V^T with Haar U, V (QR of Gaussians) and s log-uniform in [lo, hi], drawn anew per
                      step; vectors get N(0, 1) * grad_scale"""
    shapes = [tuple(s) for s in c["shapes"]]
    g = torch.Generator().manual_seed(c["seed"] * 1000 + step)
    kind = c["grad_kind"]
    out = []
    for i, sh in enumerate(shapes):
        if kind == "spectrum" and len(sh) == 2:
            lo, hi = c["spectrum"]
            m, n = sh
            k = min(m, n)
            u, _ = torch.linalg.qr(torch.randn(m, k, generator=g))
            v, _ = torch.linalg.qr(torch.randn(n, k, generator=g))
            sv = torch.exp(torch.empty(k).uniform_(math.log(lo), math.log(hi), generator=g))
            out.append(((u * sv) @ v.T).contiguous())
            continue
        t = c["grad_scale"] * torch.randn(*sh, generator=g)
        if kind == "graded" and len(sh) == 2:
            # columns scaled over grade_decades decades: R = G^T G is a graded matrix D M D whose small eigenvalues are
            # well determined (to high relative accuracy) but far below what fp32 resolves next to the large ones
            t = t * torch.pow(10.0, -torch.linspace(0.0, float(c["grade_decades"]), sh[1]))
        if kind == "gauss_lowrank" and len(sh) == 2:
            r = c["lowrank_rank"]
            gl = torch.Generator().manual_seed(c["seed"] * 7919 + i)
            a = torch.randn(sh[0], r, generator=gl)
            b = torch.randn(r, sh[1], generator=gl)
            t = t + c["lowrank_scale"] * (a @ b)
        out.append(t)
    return out


def initial_params(c) -> list[torch.Tensor]:
    shapes = [tuple(s) for s in c["shapes"]]
    if c.get("zero_init"):
        return [torch.zeros(*s) for s in shapes]
    return case_params(shapes, c["seed"])


def grad_stream(c):
    """Yields (step, grads) exactly as the fixture generator drew them."""
    shapes = [tuple(s) for s in c["shapes"]]
    if c.get("torch_seed_grads"):
        torch.manual_seed(c["seed"])
    for s in range(1, c["steps"] + 1):
        if c.get("torch_seed_grads"):
            yield s, [torch.randn(*sh) for sh in shapes]
        elif "grad_kind" in c:
            yield s, horizon_grads(c, s)
        else:
            yield s, case_grads(shapes, c["seed"], s, c["grad_scale"])


def oracle_config(c):
    from oracle.shampoo_oracle import OracleConfig

    return OracleConfig(
        lr=c["lr"], betas=tuple(c["betas"]), beta3=c.get("beta3", -1.0), epsilon=c["epsilon"],
        weight_decay=c["weight_decay"], weight_decay_type=c["weight_decay_type"],
        max_preconditioner_dim=c["max_preconditioner_dim"],
        precondition_frequency=c["precondition_frequency"],
        start_preconditioning_step=c["start_preconditioning_step"],
        preconditioner=c["preconditioner"],
        inverse_exponent_override={1: {0: 0.0}} if c.get("override_1d") else {},
        grafting=c["grafting"], grafting_beta2=c.get("grafting_beta2", 0.999),
        grafting_epsilon=c.get("grafting_epsilon", 1e-10),
        momentum=c.get("momentum", 0.0), dampening=c.get("dampening", 0.0),
        use_nesterov=c.get("use_nesterov", False),
        averaging=c.get("averaging"), eval_interp_coeff=c.get("eval_interp_coeff", 0.9),
        train_interp_coeff=c.get("train_interp_coeff", 0.8), eval_coeff_lr_power=c.get("eval_coeff_lr_power", 2),
        kl=c.get("kl", False), factor_matrix_dtype=c.get("factor_matrix_dtype", "float32"),
        use_trace_scaling=c.get("use_trace_scaling", False),
        trace_scaling_exponent=c.get("trace_scaling_exponent", 0.5),
        higher_order=c.get("ho_order", 3), higher_order_rel_epsilon=c.get("ho_rel_epsilon", 0.0),
        higher_order_abs_epsilon=c.get("ho_abs_epsilon", 0.0),
        use_symmetric_packing=c.get("use_symmetric_packing", True),
    )


def basis_signature(q: torch.Tensor, k: int) -> torch.Tensor:
    """|P^T q_j| for k seeded Gaussian probes P (n x k) and every column q_j of an eigenbasis: a (k, n) array that
    names each column whatever its sign.  The fixtures of the eigenvalue-corrected cases hold it for every refresh
    of the reference's run, so that a test can tell in which order that run's stable sort left columns whose
    eigenvalue estimates were tied within rounding."""
    n = q.shape[0]
    g = torch.Generator().manual_seed(7_000_003 + n)
    probes = torch.randn(n, k, generator=g, dtype=torch.float64)
    return (probes.T @ q.detach().cpu().double()).abs().float()


def match_columns(signature: torch.Tensor, want: torch.Tensor) -> tuple[torch.Tensor, float]:
    """For every column of `want` (k, n) the column of `signature` that is closest in the maximum norm, and the largest
    such distance.  Raises if the assignment is not a permutation."""
    d = (signature.double().T[:, None, :] - want.double().T[None, :, :]).abs().amax(dim=2)  # [have, want]
    dist, match = d.min(dim=0)
    assert sorted(match.tolist()) == list(range(want.shape[1])), "columns do not match one to one"
    return match, float(dist.max())


def dense_symmetric(factor: torch.Tensor, n: int) -> torch.Tensor:
    """A factor matrix as a dense float64 matrix, whether it is kept dense or as its packed upper triangle."""
    if factor.dim() == 2:
        return factor.detach().cpu().double()
    iu = torch.triu_indices(n, n)
    full = torch.zeros(n, n, dtype=torch.float64)
    full[iu[0], iu[1]] = factor.detach().cpu().double()
    return full + torch.triu(full, 1).T


def tie_tolerance(n: int) -> float:
    """How far apart, relative to the largest one, two eigenvalue estimates of an order-n factor may be and still count
    as tied: the estimates are the diagonal of an fp32 product R Q of that order, whose entries carry a rounding error
    of about sqrt(n) units in the last place of the largest (6 sqrt(n) 2^-24: 5.7e-6 at order 256, 1.1e-5 at 1024;
    measured largest gap between reordered columns 1.8e-6 at order 256 and 7.3e-6 at order 768)."""
    return 6.0 * math.sqrt(n) * 2.0**-24


def assert_reordering_is_between_ties(match: torch.Tensor, q: torch.Tensor, factor: torch.Tensor, where: str) -> tuple[int, float]:
    """`match[c]` is the column of the native basis q that the reference run holds at position c.  Every column that
    sits elsewhere must have moved between positions whose Rayleigh quotients q_j^T A q_j (float64, A = the factor
    matrix) differ by less than tie_tolerance of the largest.  Returns (columns out of place, largest gap among them)."""
    n = q.shape[0]
    qd = q.detach().cpu().double()
    rayleigh = torch.einsum("ij,ik,kj->j", qd, dense_symmetric(factor, n), qd)
    moved = [(c, int(r)) for c, r in enumerate(match.tolist()) if r != c]
    worst = 0.0
    for c, r in moved:
        gap = float((rayleigh[r] - rayleigh[c]).abs() / rayleigh.abs().max())
        worst = max(worst, gap)
        assert gap < tie_tolerance(n), f"{where}: column {r} sits at {c} in the reference run, Rayleigh quotients {gap:.2e} apart"
    return len(moved), worst


def is_refresh_step(c, s: int) -> bool:
    start, freq = c["start_preconditioning_step"], c["precondition_frequency"]
    return s == start or (s > start and s % freq == 0)


def align_oracle_to_fixture(oracle, z, log: list | None = None) -> None:
    """Installs the oracle's after_amortized hook for an eigenvalue-corrected case whose fixture holds the reference
    run's basis signatures: after every refresh each eigenbasis must consist of the reference run's columns (signatures
    equal to 1e-3), and columns in another position must be ties (assert_reordering_is_between_ties); they are then put
    in the reference run's order, before the step preconditions with them.  On the host that wrote the fixture this
    changes nothing."""

    def hook(o):
        s = int(o.step_t)
        for bi, st in enumerate(o.state):
            pi, key = o.block_ids[bi]
            for k, q in enumerate(st.get("eigvecs", [])):
                name = f"sig_s{s}_p{pi}_{key}_{k}"
                if name not in z:
                    continue
                want = torch.as_tensor(z[name])
                match, dist = match_columns(basis_signature(q, want.shape[0]), want)
                assert dist < 1e-3, (name, dist)
                moved, gap = assert_reordering_is_between_ties(match, q, st["factors"][k], name)
                if moved:
                    q.copy_(q[:, match])
                if log is not None:
                    log.append((s, bi, k, moved, gap))

    oracle.after_amortized = hook


def rel_err(a, b) -> float:
    a = torch.as_tensor(a, dtype=torch.float64)
    b = torch.as_tensor(b, dtype=torch.float64)
    return float((a - b).norm() / b.norm().clamp_min(1e-300))
