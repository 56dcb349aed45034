"""Eigenvalue-corrected Shampoo (SOAP, QR eigenbasis refresh) through the C ABI against the CPU oracle and the
fixture written by the real reference."""

import pytest
import torch

from tests.golden_cases import grad_stream, initial_params, load_cases, load_npz, oracle_config, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
CASES = load_cases()


def _aligned_up_to_sign(q_native, q_ref):
    """Eigenvector matrices may differ by column signs only (squares / two-sided products cancel them)."""
    signs = torch.sign((q_native * q_ref).sum(0))
    signs[signs == 0] = 1
    return q_native * signs


@pytest.mark.parametrize("name", ["soap_qr", "f64_soap_qr", "conv_like_soap_qr", "conv_like_soap_eigh"])
def test_soap_fixture_case_matches_reference(name):
    """soap_qr: matrices and vectors; conv_like_*: blocks of order 3 split along every dim."""
    import optimizers_amd as oa
    from oracle.shampoo_oracle import ShampooOracle

    print(f"case {name}", flush=True)
    c = CASES[name]
    z = load_npz(name)
    init = initial_params(c)
    params = [torch.nn.Parameter(t.clone().to(DEV)) for t in init]
    graft = None
    if c["grafting"] == "adam":
        graft = oa.AdamPreconditionerConfig(beta2=c["grafting_beta2"], epsilon=c["grafting_epsilon"])
    pc = oa.DefaultSOAPConfig if c["preconditioner"] == "soap_qr" else oa.DefaultEigenvalueCorrectedShampooConfig
    if c.get("factor_matrix_dtype") == "float64":  # factors averaged in double, eigenvectors still fp32
        from dataclasses import replace

        pc = replace(pc, factor_matrix_dtype=torch.float64)
    opt = oa.DistributedShampoo(
        params, lr=c["lr"], betas=tuple(c["betas"]), epsilon=c["epsilon"], max_preconditioner_dim=c["max_preconditioner_dim"],
        precondition_frequency=c["precondition_frequency"], start_preconditioning_step=c["start_preconditioning_step"],
        grafting_config=graft,
        preconditioner_config=pc)
    ref_p = [t.clone() for t in init]
    ref = ShampooOracle(ref_p, oracle_config(c))
    ref64_p = [t.clone().double() for t in init]
    ref64 = ShampooOracle(ref64_p, oracle_config(c))
    # The 1-D blocks and the 8-column blocks of this case own rank-deficient factors for the first steps: the
    # basis the QR refresh returns for their null space is decided by rounding, in the reference as well.  The
    # bound is therefore 1e-3 plus twice the reference algorithm's own fp32-vs-fp64 gap.
    worst_allow = 0.0
    for s, grads in grad_stream(c):
        for p, g in zip(params, grads):
            p.grad = g.to(DEV)
        opt.step()
        ref.step([g.clone() for g in grads])
        ref64.step([g.double() for g in grads])
        for p, r, r64 in zip(params, ref_p, ref64_p):
            allow = 1e-3 + 2.0 * rel_err(r, r64)
            worst_allow = max(worst_allow, allow)
            assert rel_err(p.detach().cpu(), r) < allow, s
    for i, p in enumerate(params):
        assert rel_err(p.detach().cpu().reshape(-1), z[f"final_p{i}"]) < worst_allow
    ng = opt._groups[0]
    for k, bi in enumerate(ng.native_index):
        spec = ng.block_specs[bi]
        st = opt.state[params[spec.param_index]][spec.block_key]["shampoo"]
        ost = ref.state[bi]
        for j, f in enumerate(ost["factors"]):
            assert rel_err(st["factor_matrices"][j].cpu(), f) < 1e-5
        for j, q in enumerate(ost["eigvecs"]):
            got = st["factor_matrices_eigenvectors"][j].cpu()
            assert rel_err(got.T @ got, torch.eye(got.shape[0])) < 1e-5
            if name.endswith("soap_qr") and not name.startswith("conv") and spec.order == 2 and min(spec.shape) >= 16:  # full-rank factors: the basis is well defined
                assert rel_err(_aligned_up_to_sign(got, q), q) < 1e-3
        if name.endswith("soap_qr") and not name.startswith("conv") and spec.order == 2 and min(spec.shape) >= 16:
            assert rel_err(st["corrected_eigenvalues"].cpu(), ost["corrected"]) < 1e-3
        if spec.order == 3:
            # the rotated second moment belongs to the native bases: rebuild it from them (fp64) for the last gradient
            pass


# shapes whose factors all have full rank by the first refresh, so that the eigenbases are well defined
@pytest.mark.parametrize("kind", ["soap_qr", "soap_eigh"])
@pytest.mark.parametrize("shapes, b, graft", [([(256, 256)], 128, "adam"), ([(1024, 768)], 1024, None)])
def test_soap_medium_blocks_match_oracle(shapes, b, graft, kind):
    """Two refreshes (steps 3 and 6 of 7) beside the fp32 and the float64 oracle; (1024, 768) with b = 1024 takes the
    outer-block QR that benchmark configuration 4 runs.

    QR refresh: held to the plain 1e-3 on the accumulated update against the fp32 oracle at every step.  The refreshed
    bases are read right after each native refresh; their columns must be the oracle's (|cosine| > 0.999), columns in
    another position must be ties of the sorted estimates within their rounding error, and those are put in the oracle's
    order before the step uses them (tests/test_gpu_horizons.py: order_ties_like) - the noise bulk of this spectrum holds
    hundreds of such ties at order 1024.

    Eigendecomposition refresh: no such statement exists.  Inside the noise bulk neighbouring eigenvalues are closer
    than fp32 resolves next to the leading ones, so the eigenvectors there - not just their order - are decided by
    rounding: two correct fp32 eigensolvers (LAPACK on two hosts, or LAPACK and the native solver) return bases that
    differ by rotations inside the bulk, and the reference's own fp32 and float64 runs differ by about 1e-2 here.  Against
    the reference's eigh the result is pinned only through what is invariant (orthogonality, the leading invariant
    subspace) and through the distance to the float64 run: the native run must stay as close to it as the fp32 oracle
    does, up to a factor of 2.5 (measured 2.1 to 2.3)."""
    import optimizers_amd as oa
    from oracle.shampoo_oracle import OracleConfig, ShampooOracle
    from tests.golden_cases import basis_signature
    from tests.test_gpu_horizons import _summary, order_ties_like

    print(f"case {shapes} b={b} graft={graft} {kind}", flush=True)
    g = torch.Generator().manual_seed(17)
    init = [0.1 * torch.randn(*s, generator=g) for s in shapes]
    kw = dict(lr=1e-2, betas=(0.9, 0.99), epsilon=1e-12, max_preconditioner_dim=b, precondition_frequency=3,
              start_preconditioning_step=3)
    params = [torch.nn.Parameter(t.clone().to(DEV)) for t in init]
    opt = oa.DistributedShampoo(
        params, preconditioner_config=oa.DefaultSOAPConfig if kind == "soap_qr" else oa.DefaultEigenvalueCorrectedShampooConfig,
        grafting_config=oa.AdamPreconditionerConfig(beta2=0.99, epsilon=1e-8) if graft else None, **kw)
    ref_p = [t.clone() for t in init]
    ocfg = OracleConfig(preconditioner=kind, grafting=graft, grafting_beta2=0.99, grafting_epsilon=1e-8, **kw)
    ref = ShampooOracle(ref_p, ocfg)
    ref64_p = [t.clone().double() for t in init]
    ref64 = ShampooOracle(ref64_p, ocfg)
    qr = kind == "soap_qr"
    log = []
    if qr:
        def cosines(s, bi, k, q):
            cos = (q.detach().cpu().double() * ref.state[bi]["eigvecs"][k].double()).sum(0).abs()
            assert cos.min() > 0.999, (s, bi, k, float(cos.min()))

        # eight probes per column and a looser match than for the horizon fixtures: at the first refresh the factors have
        # seen three gradients, and one QR step on such a matrix returns columns that differ by some 1e-3 between two fp32
        # evaluations (the cosines are checked right after)
        order_ties_like(opt, params, lambda s, bi, spec, k: basis_signature(ref.state[bi]["eigvecs"][k], 8), log, cosines,
                        tolerance=1e-2)
    # low-rank + noise gradients give a skewed, well separated leading spectrum
    lows = [(torch.randn(s[0], 8, generator=g), torch.randn(8, s[1], generator=g)) if len(s) == 2 else None for s in shapes]
    worst = 0.0
    for step in range(7):
        grads = []
        for s, lr_ in zip(shapes, lows):
            n = 0.05 * torch.randn(*s, generator=g)
            if lr_ is not None:
                n = n + (lr_[0] * torch.rand(8, generator=g)) @ lr_[1] / 8
            grads.append(n)
        ref.step([x.clone() for x in grads])
        ref64.step([x.double() for x in grads])
        for p, gr in zip(params, grads):
            p.grad = gr.to(DEV)
        opt.step()
        for p, r, r64, w0 in zip(params, ref_p, ref64_p, init):
            if qr:
                err = rel_err(p.detach().cpu().double() - w0.double(), r.double() - w0.double())
                worst = max(worst, err)
                assert err < 1e-3, (step, err)
            else:
                assert rel_err(p.detach().cpu().double(), r64) < 1e-3 + 2.5 * rel_err(r, r64), step
    if qr:
        print(f"  accumulated update vs the fp32 oracle: at most {worst:.1e} (bound 1e-3, no allowance); tied columns put in "
              f"the oracle's order per refresh (count, largest relative gap): {_summary(log)}", flush=True)
    ng = opt._groups[0]
    for k, bi in enumerate(ng.native_index):
        spec = ng.block_specs[bi]
        st = opt.state[params[spec.param_index]][spec.block_key]["shampoo"]
        for j, q in enumerate(ref.state[bi]["eigvecs"]):
            got = st["factor_matrices_eigenvectors"][j].cpu()
            assert rel_err(got.T @ got, torch.eye(got.shape[0])) < 1e-4
            # the leading (well separated) part of the spectrum spans the same subspace
            lead = slice(got.shape[0] - 8, got.shape[0])
            assert rel_err(got[:, lead] @ got[:, lead].T, q[:, lead] @ q[:, lead].T) < 1e-3


def test_eigh_refresh_tolerance_keeps_a_good_enough_basis():
    """EighEigendecompositionConfig.tolerance (matrix_functions.py:885-897): a stored basis Q with
    ||B - diag B||_F <= tolerance ||B||_F, B = Q^T A Q, is kept; tolerance 0 always decomposes."""
    import optimizers_amd as oa

    g = torch.Generator().manual_seed(3)
    grad = torch.randn(64, 48, generator=g)
    out = {}
    for tol in (1.0, 0.0):
        p = torch.nn.Parameter(torch.zeros(64, 48, device=DEV))
        cfg = oa.EigenvalueCorrectedShampooPreconditionerConfig(
            amortized_computation_config=oa.EighEigendecompositionConfig(tolerance=tol))
        opt = oa.DistributedShampoo([p], lr=1e-2, betas=(0.9, 0.99), epsilon=1e-12, max_preconditioner_dim=64,
                                    precondition_frequency=1, start_preconditioning_step=1, preconditioner_config=cfg)
        p.grad = grad.to(DEV)
        opt.step()
        basis = opt.state[p]["block_0"]["shampoo"]["factor_matrices_eigenvectors"]
        out[tol] = [basis[j].cpu() for j in range(2)]
    for q in out[1.0]:  # the criterion holds trivially: the identity stays
        assert torch.equal(q, torch.eye(q.shape[0]))
    for q, a in zip(out[0.0], (grad @ grad.T, grad.T @ grad)):
        assert rel_err(q.T @ q, torch.eye(q.shape[0])) < 1e-5
        lam = torch.diagonal(q.T @ a @ q)
        assert bool((lam[1:] >= lam[:-1] - 1e-4 * lam.abs().max()).all())  # ascending, like torch.linalg.eigh
        assert rel_err(q @ torch.diag(lam) @ q.T, a) < 1e-4


@pytest.mark.parametrize("weight_decay", [0.0, 0.1])
def test_all_basis_changes_ignored_is_adam(weight_decay):
    """shampoo_eigenvalue_correction_test.py:60-272: eigenvalue-corrected Shampoo whose basis changes are all
    ignored preconditions in the standard basis, i.e. it is Adam (AdamW with decoupled weight decay)."""
    import optimizers_amd as oa

    g = torch.Generator().manual_seed(11)
    shapes = [(24, 16), (16,), (5, 40)]
    init = [torch.randn(s, generator=g) for s in shapes]
    params = [torch.nn.Parameter(t.clone().to(DEV)) for t in init]
    cfg = oa.EigenvalueCorrectedShampooPreconditionerConfig(ignored_basis_change_dims={1: [0], 2: [0, 1]})
    opt = oa.DistributedShampoo(params, lr=1e-2, betas=(0.9, 0.999), epsilon=1e-8, weight_decay=weight_decay,
                                max_preconditioner_dim=16, precondition_frequency=1, start_preconditioning_step=1,
                                use_bias_correction=True, preconditioner_config=cfg, grafting_config=None)
    ref_p = [torch.nn.Parameter(t.clone()) for t in init]
    ref = (torch.optim.AdamW(ref_p, lr=1e-2, betas=(0.9, 0.999), eps=1e-8, weight_decay=weight_decay)
           if weight_decay else torch.optim.Adam(ref_p, lr=1e-2, betas=(0.9, 0.999), eps=1e-8))
    for _ in range(5):
        grads = [torch.randn(s, generator=g) for s in shapes]
        for p, r, gr in zip(params, ref_p, grads):
            p.grad = gr.to(DEV)
            r.grad = gr.clone()
        opt.step()
        ref.step()
    for p, r in zip(params, ref_p):
        assert rel_err(p.detach().cpu(), r.detach()) < 1e-5
    # no Kronecker factors and no eigenbases are kept for ignored dims
    st = opt.state[params[0]]["block_0"]["shampoo"]
    assert len(st["factor_matrices"]) == 0 and len(st["factor_matrices_eigenvectors"]) == 0


@pytest.mark.parametrize("kind", ["soap_qr", "soap_eigh"])
def test_order_three_blocks_rebuilt_from_the_stored_state(kind):
    """A convolution weight (48, 40, 3, 3) with max_preconditioner_dim = 32: four order-3 blocks, two of them views
    with a split middle dim.  The rotated second moment and the applied update are recomputed in fp64 from the
    eigenbases the optimizer stores (shampoo_preconditioner_list.py:1891-1942 with tensordot over three dims)."""
    import optimizers_amd as oa

    g = torch.Generator().manual_seed(41)
    shape = (48, 40, 3, 3)
    w0 = 0.1 * torch.randn(*shape, generator=g)
    p = torch.nn.Parameter(w0.clone().to(DEV))
    lr, beta1, beta2, eps = 1e-2, 0.9, 0.95, 1e-9
    opt = oa.DistributedShampoo(
        [p], lr=lr, betas=(beta1, beta2), epsilon=eps, max_preconditioner_dim=32, precondition_frequency=2,
        start_preconditioning_step=2,
        preconditioner_config=oa.DefaultSOAPConfig if kind == "soap_qr" else oa.DefaultEigenvalueCorrectedShampooConfig)
    ng = opt._groups[0]
    specs = [ng.block_specs[i] for i in ng.native_index]
    assert [s.shape for s in specs] == [(32, 32, 9), (32, 8, 9), (16, 32, 9), (16, 8, 9)]

    def block(t, s):
        return torch.as_strided(t.reshape(-1), s.shape, s.strides, s.offset)

    def rotate(x, qs, back=False):
        for q in qs:  # every tensordot contracts dim 0 and appends the result: after three the dims are back in order
            x = torch.tensordot(x, q, dims=([0], [1] if back else [0]))
        return x

    v = [torch.zeros(s.shape, dtype=torch.float64) for s in specs]
    m = [torch.zeros(s.shape, dtype=torch.float64) for s in specs]
    steps = 5
    for step in range(1, steps + 1):
        G = torch.randn(*shape, generator=g)
        before = p.detach().cpu().clone()
        p.grad = G.to(DEV)
        opt.step()
        after = p.detach().cpu()
        Gm = G.reshape(48, 40, 9).double()
        for k, s in enumerate(specs):
            st = opt.state[p][s.block_key]["shampoo"]
            Q = [st["factor_matrices_eigenvectors"][j].cpu().double() for j in range(3)]
            gb = block(Gm, s)
            v[k] = beta2 * v[k] + (1 - beta2) * rotate(gb, Q) ** 2
            m[k] = beta1 * m[k] + (1 - beta1) * gb
            if step == steps:
                for q in Q:
                    assert (q.T @ q - torch.eye(q.shape[0], dtype=torch.float64)).abs().max() < 1e-5
                assert rel_err(st["corrected_eigenvalues"].cpu(), v[k]) < 1e-4
                ghat = m[k] / (1 - beta1**step)
                rot = rotate(ghat, Q) / ((v[k] / (1 - beta2**step)).sqrt() + eps)
                want = -lr * rotate(rot, Q, back=True)
                delta = (block(after.reshape(48, 40, 9), s) - block(before.reshape(48, 40, 9), s)).double()
                assert rel_err(delta, want) < 1e-3


@pytest.mark.parametrize("beta1, graft", [(0.9, None), (0.0, None), (0.9, "adam")])
@pytest.mark.parametrize("kind", ["soap_qr", "soap_eigh"])
def test_shared_rotation_step_equals_the_two_separate_calls(kind, beta1, graft):
    """The step updates the second moment in the eigenbasis and preconditions in one library call that rotates the gradient
    once and carries Q_L^T m Q_R along by m's moving average between refreshes.  It must give what
    sa_update_corrected_eigenvalues + sa_precondition_eigenvalue_corrected give (rotation of m itself on every step), over
    refreshes, a masked parameter, ragged tiles, one-sided and order-3 blocks and a state reload."""
    import optimizers_amd as oa
    from optimizers_amd.distributed_shampoo import _NativeGroup

    shapes = [(200, 136), (64, 300), (520,), (6, 40, 24), (128, 128)]
    torch.manual_seed(3)
    init = [0.1 * torch.randn(s) for s in shapes]
    grads = [[0.05 * torch.randn(s) for s in shapes] for _ in range(13)]

    def run(fused):
        params = [torch.nn.Parameter(t.clone().to(DEV)) for t in init]

        def make(ps):
            return oa.DistributedShampoo(
                ps, lr=0.02, betas=(beta1, 0.95), epsilon=1e-8, weight_decay=0.01, max_preconditioner_dim=128,
                precondition_frequency=4, start_preconditioning_step=4,
                grafting_config=oa.AdamPreconditionerConfig(beta2=0.95, epsilon=1e-8) if graft else None,
                preconditioner_config=oa.DefaultSOAPConfig if kind == "soap_qr" else oa.DefaultEigenvalueCorrectedShampooConfig)

        opt = make(params)
        shared = 0
        count = lambda o: o._groups[0].lib.sa_plan_shared_rotation_steps(o._groups[0].plan)
        old = _NativeGroup.fuse_eigenbasis_rotations
        _NativeGroup.fuse_eigenbasis_rotations = fused
        try:
            for s, gs in enumerate(grads, start=1):
                for i, (p, g) in enumerate(zip(params, gs)):
                    p.grad = None if (i == 1 and s in (7, 8)) else g.to(DEV)  # a parameter without gradient for two steps
                opt.step()
                if s == 10:  # rebuild from the checkpoint: nothing derived from the old plan may survive
                    sd = opt.state_dict()
                    shared += count(opt)
                    params = [torch.nn.Parameter(p.detach().clone()) for p in params]
                    opt = make(params)
                    opt.load_state_dict(sd)
                if s == 11:  # and a reload into the live optimizer, whose plan holds a rotated copy of the old state
                    opt.load_state_dict(opt.state_dict())
        finally:
            _NativeGroup.fuse_eigenbasis_rotations = old
        return [p.detach().cpu() for p in params], shared + count(opt)

    (want, n_separate), (got, n_shared) = run(False), run(True)
    # Without grafting every step preconditions (identity bases before step 4), with it steps 4..13.  With a filtered
    # gradient the copy is rebuilt on the first step, after the refreshes (4, 8, 12), the mask changes (7, 9) and the
    # reloads (11, 12): steps 2, 3, 5, 6, 10 and 13 are left, 5, 6, 10 and 13 with grafting.
    assert n_separate == 0 and n_shared == (13 if beta1 == 0.0 else (4 if graft else 6))
    for w, g in zip(want, got):
        assert torch.isfinite(g).all()
        assert rel_err(g, w) < 2e-5
