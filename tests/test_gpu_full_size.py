"""The benchmark configurations at their full sizes, checked through properties that do not depend on size
(the CPU oracle would need minutes per step there): every quantity the native step stores or applies is
recomputed for sampled blocks in fp64 with plain torch from the same inputs.

 * Kronecker factors = the EMA of the Gram matrices of the gradients that were fed       (<= 1e-5)
 * inverse roots X of the Newton path: X^4 (L / bc2 + eps I) = I                          (<= 1e-3, max norm)
 * inverse roots of the eigh path on the resolved part of the spectrum                    (<= 2e-3)
 * eigenbases of the eigenvalue-corrected path are orthogonal                             (<= 1e-5)
 * the applied update equals -lr * |graft| / |P| * P with P rebuilt from the stored state (<= 1e-4; 5e-4 with
   the ill-conditioned inverse roots of the 4096-block configuration)
 * every block's update has the norm of its grafting direction                            (<= 1e-4)
"""

import pytest
import torch

import bench
from tests.golden_cases import rel_err

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _unpack64(v: torch.Tensor, d: int) -> torch.Tensor:
    out = torch.zeros(d, d, dtype=torch.float64, device=v.device)
    r, c = torch.triu_indices(d, d, device=v.device)
    out[r, c] = v.double()
    out[c, r] = v.double()
    return out


def _block_view(t: torch.Tensor, spec) -> torch.Tensor:
    return torch.as_strided(t.detach().reshape(-1), spec.shape, spec.strides, spec.offset)


def _run(workload: dict, steps: int):
    """Steps the native optimizer; returns what the checks need: gradients fed, parameters before the last step."""
    params, opt = bench.build(workload, DEV)
    grads_seen, before = [], None
    for s in range(1, steps + 1):
        grads = bench.make_grads(workload, params, s, DEV)
        grads_seen.append([g.clone() for g in grads])
        if s == steps:
            before = [p.detach().clone() for p in params]
        for p, g in zip(params, grads):
            p.grad = g
        opt.step()
    torch.cuda.synchronize()
    return params, opt, grads_seen, before


def _sample_blocks(ng, count: int):
    two_d = [k for k, bi in enumerate(ng.native_index) if ng.block_specs[bi].order == 2]
    stride = max(len(two_d) // count, 1)
    return two_d[::stride][:count]


def test_llama_layer_blocks_2048_newton():
    """Benchmark configuration 3 at full size (58 blocks, 112 factors of order 2048 / 1024), three steps."""
    w = bench.WORKLOADS["llama3_8b_layer"]
    beta1, beta2 = w["betas"]
    steps = 3
    params, opt, grads_seen, before = _run(w, steps)
    ng = opt._groups[0]
    assert len(ng.native_index) == 58 and ng.n_factors == 108
    bc2 = 1.0 - beta2**steps
    bc1 = 1.0 - beta1**steps
    for k in _sample_blocks(ng, 5):
        spec = ng.block_specs[ng.native_index[k]]
        print(f"block {k} of parameter {spec.param_index} shape {spec.shape}", flush=True)
        st = opt.state[params[spec.param_index]][spec.block_key]
        G = [_block_view(gs[spec.param_index], spec).double() for gs in grads_seen]
        # Kronecker factors
        L = sum((beta2 ** (steps - 1 - t)) * (1 - beta2) * (g @ g.T) for t, g in enumerate(G))
        R = sum((beta2 ** (steps - 1 - t)) * (1 - beta2) * (g.T @ g) for t, g in enumerate(G))
        X = []
        for j, F in enumerate((L, R)):
            d = F.shape[0]
            got = _unpack64(st["shampoo"]["factor_matrices"][j], d)
            assert rel_err(got.cpu(), F.cpu()) < 1e-5
            Xj = _unpack64(st["shampoo"]["inv_factor_matrices"][j], d)
            A = F / bc2 + w["epsilon"] * torch.eye(d, dtype=torch.float64, device=DEV)
            res = (torch.linalg.matrix_power(Xj, 4) @ A - torch.eye(d, dtype=torch.float64, device=DEV)).abs().max().item()
            assert res < 1e-3, (j, res)
            X.append(Xj)
        # the update that was applied
        m = st["filtered_grad"].double()
        ghat = m / bc1
        v = st["adagrad"].double()
        graft = ghat / ((v / bc2).sqrt() + w["graft_eps"])
        P = X[0] @ ghat @ X[1]
        want = -w["lr"] * (graft.norm() / (P.norm() + 1e-16)) * P
        delta = (_block_view(params[spec.param_index], spec) - _block_view(before[spec.param_index], spec)).double()
        assert rel_err(delta.cpu(), want.cpu()) < 1e-4
    # norm of every block's update = lr * norm of its grafting direction
    for k, bi in enumerate(ng.native_index):
        spec = ng.block_specs[bi]
        st = opt.state[params[spec.param_index]][spec.block_key]
        graft = (st["filtered_grad"].double() / bc1) / ((st["adagrad"].double() / bc2).sqrt() + w["graft_eps"])
        delta = (_block_view(params[spec.param_index], spec) - _block_view(before[spec.param_index], spec)).double()
        assert delta.norm().item() == pytest.approx(w["lr"] * graft.norm().item(), rel=1e-4)


def test_large_blocks_4096_eigh():
    """Benchmark configuration 5 at full size (16 blocks of 4096 x 4096, spectrum over twelve decades), with the
    eigendecomposition at step 2 instead of 50."""
    w = dict(bench.WORKLOADS["large_block_eigh"], precondition_frequency=1, start_preconditioning_step=2)
    beta1, beta2 = w["betas"]
    steps = 2
    params, opt, grads_seen, before = _run(w, steps)
    ng = opt._groups[0]
    assert len(ng.native_index) == 16 and ng.n_factors == 32
    bc2 = 1.0 - beta2**steps
    bc1 = 1.0 - beta1**steps
    for k in (0, 9):
        spec = ng.block_specs[ng.native_index[k]]
        print(f"block {k} shape {spec.shape}", flush=True)
        st = opt.state[params[spec.param_index]][spec.block_key]
        G = [_block_view(gs[spec.param_index], spec).double() for gs in grads_seen]
        X = []
        for j in range(2):
            F = sum((beta2 ** (steps - 1 - t)) * (1 - beta2) * ((g @ g.T) if j == 0 else (g.T @ g)) for t, g in enumerate(G))
            d = F.shape[0]
            assert rel_err(_unpack64(st["shampoo"]["factor_matrices"][j], d).cpu(), F.cpu()) < 1e-5
            Xj = _unpack64(st["shampoo"]["inv_factor_matrices"][j], d)
            lam, q = torch.linalg.eigh(F / bc2)
            keep = lam > 1e-4 * lam.max()  # the part of the spectrum fp32 resolves
            qk = q[:, keep]
            proj = qk.T @ Xj @ qk
            assert rel_err(proj.cpu(), torch.diag(lam[keep].pow(-0.25)).cpu()) < 2e-3
            X.append(Xj)
        ghat = st["filtered_grad"].double() / bc1
        graft = ghat / ((st["adagrad"].double() / bc2).sqrt() + w["graft_eps"])
        P = X[0] @ ghat @ X[1]
        want = -w["lr"] * (graft.norm() / (P.norm() + 1e-16)) * P
        delta = (_block_view(params[spec.param_index], spec) - _block_view(before[spec.param_index], spec)).double()
        # the inverse roots' eigenvalues span three decades here (1 .. 1e3), so the fp32 products cancel more
        assert rel_err(delta.cpu(), want.cpu()) < 5e-4


def test_large_blocks_4096_eigh_at_the_stated_cadence():
    """Benchmark configuration 5 at full size AND with its own schedule: 49 grafting-only steps, the eigendecomposition
    of all 32 factors at step 50, one more step that uses it.  Two gradient sets alternate (as in the benchmark), so the
    factors have a closed form: c_1 G_1 G_1^T + c_2 G_2 G_2^T with the two sums of EMA weights."""
    w = bench.WORKLOADS["large_block_eigh"]
    assert w["precondition_frequency"] == 50 and w["start_preconditioning_step"] == 50
    beta1, beta2 = w["betas"]
    steps = 51
    params, opt = bench.build(w, DEV)
    sets = [bench.make_grads(w, params, s, DEV) for s in (1, 2)]
    before = None
    for s in range(1, steps + 1):
        if s == steps:
            before = [p.detach().clone() for p in params]
        for p, g in zip(params, sets[s % 2]):
            p.grad = g.clone()
        opt.step()
    torch.cuda.synchronize()
    ng = opt._groups[0]
    assert len(ng.native_index) == 16 and ng.n_factors == 32
    # the factors the root inverse saw are those of step 50; the update of step 51 uses the moments of step 51
    weight = {50: [0.0, 0.0], 51: [0.0, 0.0]}
    for upto in (50, 51):
        for t in range(1, upto + 1):
            weight[upto][t % 2] += (beta2 ** (upto - t)) * (1 - beta2)
    bc1 = 1.0 - beta1**steps
    bc2 = 1.0 - beta2**steps
    for k in (3, 12):
        spec = ng.block_specs[ng.native_index[k]]
        print(f"block {k} shape {spec.shape}", flush=True)
        st = opt.state[params[spec.param_index]][spec.block_key]
        G = [_block_view(sets[i][spec.param_index], spec).double() for i in range(2)]
        X = []
        for j in range(2):
            gram = [(g @ g.T) if j == 0 else (g.T @ g) for g in G]
            d = gram[0].shape[0]
            F51 = weight[51][0] * gram[0] + weight[51][1] * gram[1]
            assert rel_err(_unpack64(st["shampoo"]["factor_matrices"][j], d).cpu(), F51.cpu()) < 1e-5
            F50 = weight[50][0] * gram[0] + weight[50][1] * gram[1]
            Xj = _unpack64(st["shampoo"]["inv_factor_matrices"][j], d)
            lam, q = torch.linalg.eigh(F50 / (1.0 - beta2**50))
            keep = lam > 1e-4 * lam.max()  # the part of the spectrum fp32 resolves
            qk = q[:, keep]
            assert rel_err((qk.T @ Xj @ qk).cpu(), torch.diag(lam[keep].pow(-0.25)).cpu()) < 2e-3
            X.append(Xj)
        ghat = st["filtered_grad"].double() / bc1
        graft = ghat / ((st["adagrad"].double() / bc2).sqrt() + w["graft_eps"])
        P = X[0] @ ghat @ X[1]
        want = -w["lr"] * (graft.norm() / (P.norm() + 1e-16)) * P
        delta = (_block_view(params[spec.param_index], spec) - _block_view(before[spec.param_index], spec)).double()
        assert rel_err(delta.cpu(), want.cpu()) < 5e-4


def test_llama_layer_blocks_1024_eigenvalue_corrected():
    """Benchmark configuration 4 at full size (216 blocks, 424 eigenbases of order 1024), QR refresh at steps 2 and 3."""
    w = dict(bench.WORKLOADS["llama3_8b_layer_soap"], precondition_frequency=1, start_preconditioning_step=2)
    beta1, beta2 = w["betas"]
    steps = 3
    params, opt, grads_seen, before = _run(w, steps)
    ng = opt._groups[0]
    assert len(ng.native_index) == 216 and ng.n_factors == 424
    bc2 = 1.0 - beta2**steps
    bc1 = 1.0 - beta1**steps
    for k in _sample_blocks(ng, 4):
        spec = ng.block_specs[ng.native_index[k]]
        print(f"block {k} shape {spec.shape}", flush=True)
        st = opt.state[params[spec.param_index]][spec.block_key]
        Q = [st["shampoo"]["factor_matrices_eigenvectors"][j].double() for j in range(2)]
        for q in Q:
            d = q.shape[0]
            assert (q.T @ q - torch.eye(d, dtype=torch.float64, device=DEV)).abs().max().item() < 1e-5
        ghat = st["filtered_grad"].double() / bc1
        rot = Q[0].T @ ghat @ Q[1]
        rot = rot / ((st["shampoo"]["corrected_eigenvalues"].double() / bc2).sqrt() + w["epsilon"])
        want = -w["lr"] * (Q[0] @ rot @ Q[1].T)
        delta = (_block_view(params[spec.param_index], spec) - _block_view(before[spec.param_index], spec)).double()
        assert rel_err(delta.cpu(), want.cpu()) < 1e-4


def test_llama_layer_blocks_1024_eigenvalue_corrected_at_the_stated_cadence():
    """Benchmark configuration 4 at full size AND with its own schedule: first eigenbases at step 10, QR refreshes at
    steps 20 and 30, one more step on the bases of step 30.  Sampled blocks: the Kronecker factors are the EMA of the 31
    Gram matrices, the bases are orthogonal, and the update is the one rebuilt from the stored state."""
    w = bench.WORKLOADS["llama3_8b_layer_soap"]
    assert w["precondition_frequency"] == 10 and w["start_preconditioning_step"] == 10
    beta1, beta2 = w["betas"]
    steps = 31
    params, opt = bench.build(w, DEV)
    ng = opt._groups[0]
    assert len(ng.native_index) == 216 and ng.n_factors == 424
    sampled = _sample_blocks(ng, 4)
    seen = {k: [] for k in sampled}
    before = None
    for s in range(1, steps + 1):
        grads = bench.make_grads(w, params, s, DEV)
        for k in sampled:
            spec = ng.block_specs[ng.native_index[k]]
            seen[k].append(_block_view(grads[spec.param_index], spec).clone())
        if s == steps:
            before = [p.detach().clone() for p in params]
        for p, g in zip(params, grads):
            p.grad = g
        opt.step()
    torch.cuda.synchronize()
    bc2 = 1.0 - beta2**steps
    bc1 = 1.0 - beta1**steps
    for k in sampled:
        spec = ng.block_specs[ng.native_index[k]]
        print(f"block {k} shape {spec.shape}", flush=True)
        st = opt.state[params[spec.param_index]][spec.block_key]
        Q = [st["shampoo"]["factor_matrices_eigenvectors"][j].double() for j in range(2)]
        for j, q in enumerate(Q):
            d = q.shape[0]
            # each column passes through up to 1024 fp32 reflections: the bound is d * 2^-24 = 6e-5, measured 1.0e-5
            departure = (q.T @ q - torch.eye(d, dtype=torch.float64, device=DEV)).abs().max().item()
            print(f"  basis {j}: max |Q^T Q - I| = {departure:.2e}", flush=True)
            assert departure < 3e-5
            grams = [(g.double() @ g.double().T) if j == 0 else (g.double().T @ g.double()) for g in seen[k]]
            F31 = sum((beta2 ** (steps - 1 - t)) * (1 - beta2) * gm for t, gm in enumerate(grams))
            assert rel_err(_unpack64(st["shampoo"]["factor_matrices"][j], d).cpu(), F31.cpu()) < 1e-5
        ghat = st["filtered_grad"].double() / bc1
        rot = Q[0].T @ ghat @ Q[1]
        rot = rot / ((st["shampoo"]["corrected_eigenvalues"].double() / bc2).sqrt() + w["epsilon"])
        want = -w["lr"] * (Q[0] @ rot @ Q[1].T)
        delta = (_block_view(params[spec.param_index], spec) - _block_view(before[spec.param_index], spec)).double()
        assert rel_err(delta.cpu(), want.cpu()) < 1e-4


def test_gpt2_small_ragged_blocks():
    """Benchmark configuration 2 at full size: 194 blocks (ragged 256 x 768 and 81 x 768 among them), the first
    preconditioned step at 11 as in the benchmark; factors of the ragged tail block and the update norms."""
    w = bench.WORKLOADS["gpt2_small"]
    beta1, beta2 = w["betas"]
    steps = 11
    params, opt, grads_seen, before = _run(w, steps)
    ng = opt._groups[0]
    assert len(ng.native_index) == 194
    bc2 = 1.0 - beta2**steps
    bc1 = 1.0 - beta1**steps
    tail = max(k for k, bi in enumerate(ng.native_index) if ng.block_specs[bi].shape == (81, 768))
    for k in (tail, tail - 1, 0):
        spec = ng.block_specs[ng.native_index[k]]
        st = opt.state[params[spec.param_index]][spec.block_key]
        G = [_block_view(gs[spec.param_index], spec).double() for gs in grads_seen]
        for j in range(2):
            F = sum((beta2 ** (steps - 1 - t)) * (1 - beta2) * ((g @ g.T) if j == 0 else (g.T @ g)) for t, g in enumerate(G))
            assert rel_err(_unpack64(st["shampoo"]["factor_matrices"][j], F.shape[0]).cpu(), F.cpu()) < 1e-5
    for k, bi in enumerate(ng.native_index):
        spec = ng.block_specs[bi]
        st = opt.state[params[spec.param_index]][spec.block_key]
        graft = (st["filtered_grad"].double() / bc1) / ((st["adagrad"].double() / bc2).sqrt() + w["graft_eps"])
        delta = (_block_view(params[spec.param_index], spec) - _block_view(before[spec.param_index], spec)).double()
        assert delta.norm().item() == pytest.approx(w["lr"] * graft.norm().item(), rel=1e-4)


def test_four_llama_layers_in_one_group_under_a_scratch_budget():
    """Four Llama-3-8B layers in ONE parameter group (432 factors): with the scratch of the amortized computation capped
    at 24 GB the factors are solved in waves; parameters and Newton iteration counts must equal, bit for bit, those of a
    run that solves all factors at once (58 GB of scratch)."""
    import os

    from optimizers_amd.distributed_shampoo import _NativeGroup

    if "SHAMPOO_AMD_SCRATCH_BYTES" in os.environ:
        pytest.skip("the environment overrides the scratch budget this test sets")
    w = dict(bench.WORKLOADS["llama3_8b_layer"])
    w["shapes"] = list(w["shapes"]) * 4
    saved = _NativeGroup.scratch_budget_bytes
    runs = []
    try:
        for budget in (24 << 30, None):
            print(f"scratch budget {budget}", flush=True)
            _NativeGroup.scratch_budget_bytes = budget
            params, opt = bench.build(w, DEV)
            ng = opt._groups[0]
            waves = int(ng.lib.sa_plan_num_waves(ng.plan))
            workspace = ng.workspace.numel()
            iterations = []
            for s in range(1, 5):
                for p, g in zip(params, bench.make_grads(w, params, s, DEV)):
                    p.grad = g
                opt.step()
                iterations.append(list(ng.last_newton_iterations))
            torch.cuda.synchronize()
            runs.append((waves, workspace, iterations, [p.detach().clone() for p in params]))
            del params, opt, ng
            torch.cuda.empty_cache()
    finally:
        _NativeGroup.scratch_budget_bytes = saved
    (waves_c, ws_c, it_c, p_c), (waves_u, ws_u, it_u, p_u) = runs
    print(f"capped: {waves_c} waves, workspace {ws_c / 2**30:.1f} GiB; uncapped: {waves_u} wave, {ws_u / 2**30:.1f} GiB", flush=True)
    assert waves_u == 1 and waves_c == 3
    assert ws_c < (24 << 30) + (9 << 30) < ws_u
    assert it_c == it_u and any(any(r) for r in it_c)
    for a, b in zip(p_c, p_u):
        assert torch.equal(a, b)


def test_symmetric_product_policy_against_full_products_at_full_size():
    """The Llama layer at full size, four steps, once with the reference's full products in every coupled Newton iteration
    (policy 0) and once with the library's default policy 2 (symmetric products for factors whose previous solve converged
    within 14 iterations) -- two plans with different policies in one process.  Inverse roots and parameters of the two
    runs must agree far inside the 1e-3 bar."""
    w = bench.WORKLOADS["llama3_8b_layer"]
    runs = []
    for policy in (0, 2):
        params, opt = bench.build(w, DEV)
        ng = opt._groups[0]
        assert ng.lib.sa_plan_set_symmetric_newton(ng.plan, policy) == 0
        for s in range(1, 5):
            for p, g in zip(params, bench.make_grads(w, params, s, DEV)):
                p.grad = g
            opt.step()
        torch.cuda.synchronize()
        runs.append(([p.detach().clone() for p in params], ng.inv_arena.buffer.clone(), list(ng.last_newton_iterations)))
        del params, opt, ng
        torch.cuda.empty_cache()
    (p0, inv0, it0), (p2, inv2, it2) = runs
    inv_err = rel_err(inv2.cpu(), inv0.cpu())
    upd_err = max(rel_err(a.cpu(), b.cpu()) for a, b in zip(p2, p0))
    print(f"policy 2 vs policy 0: inverse roots {inv_err:.2e}, parameters {upd_err:.2e}; iterations {max(it0)} / {max(it2)}", flush=True)
    assert inv_err < 1e-4 and upd_err < 1e-4
    assert max(abs(a - b) for a, b in zip(it0, it2)) <= 1
