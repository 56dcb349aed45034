"""The benchmark configurations' horizons and cadences against fixtures the real reference wrote: 20 steps of coupled
Newton on a ragged GPT-2 slice (81 x 768 tail block) and on a Llama slice, 50 steps of eigenvalue-corrected Shampoo with
a QR refresh every 10 on 256-blocks and 30 steps on one 1024 x 768 block, 100 steps with an eigendecomposition root
inverse every 50 on log-uniform spectra.  The initial parameters are zero, so the parameters compared ARE the accumulated
updates.  The native step (through the C ABI) is compared with the reference's stored fp32 run, step by step on a
subsample and at the end, and the float64 run stored beside it shows how far two correct fp32 evaluations can be apart.

Bound: 1e-3 relative Frobenius error on the accumulated update at every step (the stated tolerance), for every case.

The eigenvalue-corrected cases need one thing said about the reference first.  A QR refresh ends with a stable sort of
the eigenvalue estimates, and the second moment kept in the eigenbasis is not re-indexed
(shampoo_preconditioner_list.py:1867-1912, matrix_functions.py:848-850).  The estimates are the diagonal of an fp32
product and carry a rounding error of a few 1e-6 of the largest; with hundreds of neighbouring pairs per factor some are
always closer than that, and in which order such a pair leaves the sort depends on the last bits: the reference's own
run differs between two hosts (other BLAS kernels, another thread count) by 4e-3 after 50 steps for this reason alone,
and by 4.4e-3 from its float64 run.  A swapped pair meets each other's second moment until the next refresh.  The
fixtures therefore record, for every refresh of the reference's run, a signature of every column of every eigenbasis
(tests/golden_cases.py: basis_signature).  The tests read the native bases right after each native refresh, before the
step uses them; every column must be one of the reference run's columns, a column in another position must have moved
between positions whose Rayleigh quotients (float64) are tied within the estimates' rounding error (tie_tolerance), and
such columns are then put in the reference run's order, the documented route for outside writes to the state
(sa_plan_invalidate_inverse_cache).  Anything that is not a reordering of ties fails.  With that, the run meets the
plain 1e-3 on every step (measured 1e-6).  The same is done beside the fp32 oracle for all five refreshes with the
columns compared directly (|cosine| > 0.999), and a run without any alignment is held to 1e-3 before the first refresh
and to 3e-2 (a few swapped pairs' worth) afterwards, with the error's path printed."""

import pytest
import torch

from tests.golden_cases import (
    assert_reordering_is_between_ties, basis_signature, grad_stream, initial_params, load_cases, load_npz, match_columns,
    oracle_config, rel_err,
)
from tests.test_gpu_step_parity import native_optimizer

pytestmark = pytest.mark.gpu

CASES = load_cases()
HORIZON_CASES = [n for n in CASES if n.startswith("horizon_")]
SOAP_CASES = [n for n in HORIZON_CASES if CASES[n].get("basis_signature")]


def _native(c, params):
    import optimizers_amd as oa

    if c["preconditioner"] == "soap_qr":
        return oa.DistributedShampoo(
            params, lr=c["lr"], betas=tuple(c["betas"]), epsilon=c["epsilon"], max_preconditioner_dim=c["max_preconditioner_dim"],
            precondition_frequency=c["precondition_frequency"], start_preconditioning_step=c["start_preconditioning_step"],
            grafting_config=None, preconditioner_config=oa.DefaultSOAPConfig)
    return native_optimizer(c, params)


def order_ties_like(opt, params, wanted_signature, log, compare=None, tolerance=1e-3):
    """Wraps the amortized computation of the optimizer's (only) group: right after every native eigenbasis refresh, and
    before the step uses the bases, every basis is matched column by column against `wanted_signature(step, block index,
    block spec, factor)` (a (k, n) basis signature of the run to follow, or None).  Every column must be found there
    (signatures equal to `tolerance`); a column found at another position must be a tie (assert_reordering_is_between_ties);
    the columns are then put in the followed run's order and the plan is told that its state was written from outside.
    `compare(step, block index, factor, reordered native basis)` may check more.  log collects
    (step, block index, factor, columns moved, largest relative gap of their Rayleigh quotients)."""
    from optimizers_amd import native

    group = opt._groups[0]
    inner = group._amortized_computation

    def amortized_then_ordered(g, bc2, stream):
        inner(g, bc2, stream)
        s = int(group.step_tensor)
        for bi in group.native_index:
            spec = group.block_specs[bi]
            st = opt.state[params[spec.param_index]][spec.block_key]["shampoo"]
            for k, q in sorted(st["factor_matrices_eigenvectors"].items()):
                want = wanted_signature(s, bi, spec, k)
                if want is None:
                    continue
                where = f"step {s} block {bi} factor {k}"
                match, dist = match_columns(basis_signature(q, want.shape[0]), want)
                assert dist < tolerance, (where, dist)
                moved, gap = assert_reordering_is_between_ties(match, q, st["factor_matrices"][k], where)
                if moved:
                    q.copy_(q[:, match.to(q.device)])
                if compare is not None:
                    compare(s, bi, k, q)
                log.append((s, bi, k, moved, gap))
        native.check(group.lib.sa_plan_invalidate_inverse_cache(group.plan), "sa_plan_invalidate_inverse_cache")

    group._amortized_computation = amortized_then_ordered


def _summary(log):
    per_step = {}
    for s, _, _, moved, gap in log:
        n, g = per_step.get(s, (0, 0.0))
        per_step[s] = (n + moved, max(g, gap))
    return {s: (n, float(f"{g:.1e}")) for s, (n, g) in per_step.items()}


def _run(name, align):
    c = CASES[name]
    z = load_npz(name)
    dev = torch.device("cuda:0")
    params = [torch.nn.Parameter(t.clone().to(dev)) for t in initial_params(c)]
    opt = _native(c, params)
    log = []
    if align:
        def from_fixture(s, bi, spec, k):
            key = f"sig_s{s}_p{spec.param_index}_{spec.block_key}_{k}"
            return torch.as_tensor(z[key]) if key in z else None

        order_ties_like(opt, params, from_fixture, log)
    stride = c["trace_stride"]
    freq, start = c["precondition_frequency"], c["start_preconditioning_step"]
    worst = floor = worst64 = 0.0
    errs = []
    iteration_mismatch = 0
    for s, grads in grad_stream(c):
        for p, g in zip(params, grads):
            p.grad = g.to(dev)
        opt.step()
        err = 0.0
        for i, p in enumerate(params):
            got = p.detach().reshape(-1)[::stride].cpu()
            err = max(err, rel_err(got, z[f"trace_s{s}_p{i}"]))
            worst64 = max(worst64, rel_err(got, z[f"o64_trace_s{s}_p{i}"]))
            floor = max(floor, rel_err(z[f"trace_s{s}_p{i}"], z[f"o64_trace_s{s}_p{i}"]))
        errs.append(err)
        worst = max(worst, err)
        if c["preconditioner"] == "newton":
            want = [int(v) for v in z["newton_iterations"][s - 1] if v >= 0]
            got_it = opt._groups[0].last_newton_iterations if want else []
            if want:
                assert len(got_it) == len(want)
                iteration_mismatch = max(iteration_mismatch, max(abs(a - b) for a, b in zip(got_it, want)))
    final = max(rel_err(p.detach().reshape(-1)[::37].cpu(), z[f"final_p{i}"]) for i, p in enumerate(params))
    final64 = max(rel_err(p.detach().reshape(-1)[::37].cpu(), z[f"o64_final_p{i}"]) for i, p in enumerate(params))
    refresh = [s for s in range(1, c["steps"] + 1) if s == start or (s > start and s % freq == 0)]
    jumps = {s: errs[s - 1] - errs[s - 2] for s in refresh if s >= 2}
    growth_between = 0.0  # what the error gains outside of refresh steps, summed over the stretches between them
    for s in range(2, c["steps"] + 1):
        if s not in refresh:
            growth_between += max(errs[s - 1] - errs[s - 2], 0.0)
    print(
        f"  {name}: native vs reference fp32: worst step {worst:.2e}, final {final:.2e} (bound 1e-3, no allowance); native vs "
        f"float64: worst step {worst64:.2e}, final {final64:.2e}; reference fp32 vs float64 (its own rounding floor): "
        f"{floor:.2e}; Newton iteration counts differ by at most {iteration_mismatch}; error before the first refresh "
        f"{max(errs[: start - 1], default=0.0):.2e}, jumps at refresh steps {({s: float(f'{j:.1e}') for s, j in jumps.items()})}, "
        f"growth outside of refresh steps {growth_between:.2e}"
        + (f"; tied columns put in the reference run's order per refresh (count, largest relative gap): {_summary(log)}" if align else ""),
        flush=True,
    )
    return errs, worst, final, iteration_mismatch


@pytest.mark.parametrize("name", HORIZON_CASES)
def test_benchmark_horizon_matches_reference_fixture(name):
    print(f"case {name}", flush=True)
    _, worst, final, iteration_mismatch = _run(name, align=name in SOAP_CASES)
    assert worst < 1e-3 and final < 1e-3, (worst, final)
    assert iteration_mismatch <= 1


@pytest.mark.parametrize("name", SOAP_CASES)
def test_soap_horizon_left_to_its_own_tie_order_stays_within_a_few_swapped_pairs(name):
    """No alignment: what a user's run shows against the reference's run on another machine."""
    print(f"case {name}", flush=True)
    c = CASES[name]
    errs, worst, final, _ = _run(name, align=False)
    assert max(errs[: c["start_preconditioning_step"] - 1], default=0.0) < 1e-3
    assert worst < 3e-2 and final < 3e-2, (worst, final)


@pytest.mark.parametrize("name", SOAP_CASES)
def test_soap_horizon_beside_the_oracle_differs_only_by_the_order_of_tied_estimates(name):
    """The fp32 oracle steps beside the native optimizer over the whole horizon.  After every refresh each native basis is
    compared with the oracle's, column by column: |cosine| > 0.999 once ties are in the oracle's order, and nothing but
    ties may be out of order.  The parameters then agree to the stated 1e-3 at every step (measured 1e-6)."""
    from oracle.shampoo_oracle import ShampooOracle

    print(f"case {name}", flush=True)
    c = CASES[name]
    dev = torch.device("cuda:0")
    init = initial_params(c)
    params = [torch.nn.Parameter(t.clone().to(dev)) for t in init]
    opt = _native(c, params)
    ref_params = [t.clone() for t in init]
    ref = ShampooOracle(ref_params, oracle_config(c))
    log = []
    lowest = [1.0]

    def from_oracle(s, bi, spec, k):
        return basis_signature(ref.state[bi]["eigvecs"][k], 3)

    def cosines(s, bi, k, q):
        cos = (q.detach().cpu().double() * ref.state[bi]["eigvecs"][k].double()).sum(0).abs()
        lowest[0] = min(lowest[0], float(cos.min()))
        assert cos.min() > 0.999, (s, bi, k, float(cos.min()))

    order_ties_like(opt, params, from_oracle, log, cosines)
    worst = 0.0
    for s, grads in grad_stream(c):
        ref.step([g.clone() for g in grads])  # the oracle first: its refreshed bases are what the native ones follow
        for p, g in zip(params, grads):
            p.grad = g.to(dev)
        opt.step()
        err = max(rel_err(p.detach().cpu(), r) for p, r in zip(params, ref_params))
        worst = max(worst, err)
        assert err < 1e-3, (s, err)
    refreshes = sorted({s for s, *_ in log})
    assert len(refreshes) == (c["steps"] - c["start_preconditioning_step"]) // c["precondition_frequency"] + 1
    print(
        f"  {name}: {len(refreshes)} refreshes beside the oracle; tied columns in the other order per refresh (count, largest "
        f"relative gap of their Rayleigh quotients): {_summary(log)}; lowest |cosine| between matched columns "
        f"{lowest[0]:.6f}; parameters differ by at most {worst:.1e} over {c['steps']} steps",
        flush=True,
    )
