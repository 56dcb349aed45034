"""Host-visible behaviour of the native optimizer on the GPU: library equivalences, masking,
weight-decay flavours, checkpoint round trip, failure semantics."""

import copy
import math

import pytest
import torch

from tests.golden_cases import rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _newton(**kw):
    import optimizers_amd as oa

    return oa.RootInvShampooPreconditionerConfig(amortized_computation_config=oa.CoupledNewtonConfig(), **kw)


def _oracle(params, **kw):
    from oracle.shampoo_oracle import OracleConfig, ShampooOracle

    return ShampooOracle(params, OracleConfig(preconditioner="newton", **kw))


@pytest.mark.parametrize("decoupled", [True, False])
def test_grafting_only_equals_torch_adam(decoupled):
    """gpu_tests/shampoo_grafting_test.py:68-266 idea: preconditioning never starts."""
    import optimizers_amd as oa

    torch.manual_seed(0)
    shapes = [(70, 33), (33,), (5, 1, 7)]
    init = [torch.randn(*s) for s in shapes]
    lr, betas, eps, wd = 0.01, (0.9, 0.999), 1e-8, 0.05
    ref_p = [torch.nn.Parameter(t.clone()) for t in init]
    ref = (torch.optim.AdamW if decoupled else torch.optim.Adam)(ref_p, lr=lr, betas=betas, eps=eps, weight_decay=wd)
    params = [torch.nn.Parameter(t.clone().to(DEV)) for t in init]
    opt = oa.DistributedShampoo(
        params, lr=lr, betas=betas, epsilon=1e-12, weight_decay=wd,
        weight_decay_type=oa.WeightDecayType.DECOUPLED if decoupled else oa.WeightDecayType.L2,
        max_preconditioner_dim=32, precondition_frequency=1, start_preconditioning_step=10**9,
        preconditioner_config=_newton(), grafting_config=oa.AdamPreconditionerConfig(beta2=betas[1], epsilon=eps),
    )
    for _ in range(6):
        grads = [torch.randn(*s) for s in shapes]
        for p, q, g in zip(ref_p, params, grads):
            p.grad = g.clone()
            q.grad = g.to(DEV)
        ref.step()
        opt.step()
    for q, p in zip(params, ref_p):
        torch.testing.assert_close(q.detach().cpu(), p.detach(), rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("wd_type", ["DECOUPLED", "CORRECTED", "INDEPENDENT", "L2"])
@pytest.mark.parametrize("graft", ["adam", "rmsprop", "adagrad", "sgd", None])
def test_weight_decay_and_grafting_flavours_match_oracle(wd_type, graft):
    import optimizers_amd as oa

    g = torch.Generator().manual_seed(11)
    shapes = [(40, 24), (24,)]
    init = [torch.randn(*s, generator=g) for s in shapes]
    kw = dict(lr=0.02, betas=(0.9, 0.99), epsilon=1e-8, weight_decay=0.01, max_preconditioner_dim=16,
              precondition_frequency=2, start_preconditioning_step=4)
    gcfg = {"adam": oa.AdamPreconditionerConfig(beta2=0.95, epsilon=1e-7), "rmsprop": oa.RMSpropPreconditionerConfig(beta2=0.95, epsilon=1e-7),
            "adagrad": oa.AdaGradPreconditionerConfig(epsilon=1e-7), "sgd": oa.SGDPreconditionerConfig(), None: None}[graft]
    params = [torch.nn.Parameter(t.clone().to(DEV)) for t in init]
    opt = oa.DistributedShampoo(params, weight_decay_type=oa.WeightDecayType[wd_type],
                                preconditioner_config=_newton(inverse_exponent_override={1: {0: 0.0}}), grafting_config=gcfg, **kw)
    ref_p = [t.clone() for t in init]
    ref = _oracle(ref_p, weight_decay_type=wd_type, inverse_exponent_override={1: {0: 0.0}}, grafting=graft,
                  grafting_beta2=0.95, grafting_epsilon=1e-7, **kw)
    for step in range(8):
        grads = [torch.randn(*s, generator=g) for s in shapes]
        if step == 3:
            opt.param_groups[0]["lr"] = 0.01  # exercises CORRECTED (lr / peak_lr)
            ref.cfg.lr = 0.01
        for q, gr in zip(params, grads):
            q.grad = gr.to(DEV)
        opt.step()
        ref.step([x.clone() for x in grads])
    for q, r in zip(params, ref_p):
        assert rel_err(q.detach().cpu(), r) < 1e-4


def test_none_and_empty_gradients_mask_their_blocks():
    """shampoo_distributor.py:269-277 / tests/distributed_shampoo_test.py:1533-1579."""
    import optimizers_amd as oa

    g = torch.Generator().manual_seed(3)
    shapes = [(20, 12), (12,), (9, 9)]
    init = [torch.randn(*s, generator=g) for s in shapes]
    # epsilon is large enough that the few-gradient factors of the small blocks are well posed
    kw = dict(lr=0.01, betas=(0.9, 0.99), epsilon=1e-2, max_preconditioner_dim=8, precondition_frequency=1,
              start_preconditioning_step=2)
    params = [torch.nn.Parameter(t.clone().to(DEV)) for t in init]
    opt = oa.DistributedShampoo(params, preconditioner_config=_newton(inverse_exponent_override={1: {0: 0.0}}),
                                grafting_config=oa.AdaGradPreconditionerConfig(epsilon=1e-8), **kw)
    ref_p = [t.clone() for t in init]
    ref = _oracle(ref_p, inverse_exponent_override={1: {0: 0.0}}, grafting="adagrad", grafting_epsilon=1e-8, **kw)
    masks = [(1, 1, 1), (1, 0, 1), (0, 1, 1), (1, 1, 0), (1, 1, 1), (0, 0, 0), (1, 1, 1)]
    for m in masks:
        grads = [torch.randn(*s, generator=g) if keep else None for s, keep in zip(shapes, m)]
        for q, gr in zip(params, grads):
            q.grad = None if gr is None else gr.to(DEV)
        before = [q.detach().clone() for q in params]
        opt.step()
        ref.step([None if x is None else x.clone() for x in grads])
        for q, b, keep in zip(params, before, m):
            if not keep:
                assert torch.equal(q.detach(), b)
    for q, r in zip(params, ref_p):
        assert rel_err(q.detach().cpu(), r) < 1e-4
    assert int(opt.state[params[0]]["step"]) == len(masks) == int(ref.step_t)


def test_state_dict_layout_and_round_trip():
    """Golden layout tests/distributed_shampoo_test.py:516-622; resume must continue bit-identically."""
    import optimizers_amd as oa

    def make(init):
        ps = [torch.nn.Parameter(t.clone().to(DEV)) for t in init]
        o = oa.DistributedShampoo(ps, lr=0.01, betas=(0.9, 0.99), epsilon=1e-6, max_preconditioner_dim=5,
                                  precondition_frequency=1, start_preconditioning_step=1,
                                  preconditioner_config=_newton(), grafting_config=oa.AdaGradPreconditionerConfig(epsilon=1e-3))
        return ps, o

    g = torch.Generator().manual_seed(5)
    init = [torch.randn(5, 10, generator=g)]
    params, opt = make(init)
    sd = opt.state_dict()
    blk = sd["state"][0]["block_0"]
    assert set(sd["state"][0]) == {"block_0", "block_1", "step"}
    assert set(blk) == {"shampoo", "adagrad", "filtered_grad"}
    assert set(blk["shampoo"]) == {"factor_matrices", "inv_factor_matrices"}
    assert blk["shampoo"]["factor_matrices"][0].shape == (15,) and blk["adagrad"].shape == (5, 5)
    eye = torch.zeros(15)
    eye[[0, 5, 9, 12, 14]] = 1
    assert torch.equal(blk["shampoo"]["inv_factor_matrices"][1].cpu(), eye)
    assert sd["param_groups"][0]["beta3"] == 0.9 and sd["param_groups"][0]["start_preconditioning_step"] == 1
    grads = [torch.randn(5, 10, generator=g) for _ in range(6)]
    for gr in grads[:3]:
        params[0].grad = gr.to(DEV)
        opt.step()
    saved = copy.deepcopy(opt.state_dict())
    saved_w = params[0].detach().clone()
    for gr in grads[3:]:
        params[0].grad = gr.to(DEV)
        opt.step()
    # resume in a fresh optimizer
    params2, opt2 = make([saved_w.cpu()])
    opt2.load_state_dict(saved)
    assert int(opt2.state[params2[0]]["step"]) == 3
    for gr in grads[3:]:
        params2[0].grad = gr.to(DEV)
        opt2.step()
    assert torch.equal(params2[0].detach(), params[0].detach())


def test_two_param_groups_and_streams():
    import optimizers_amd as oa

    g = torch.Generator().manual_seed(8)
    a0, b0 = torch.randn(24, 16, generator=g), torch.randn(16, 40, generator=g)
    pa, pb = torch.nn.Parameter(a0.clone().to(DEV)), torch.nn.Parameter(b0.clone().to(DEV))
    opt = oa.DistributedShampoo(
        [{"params": [pa], "lr": 0.01}, {"params": [pb], "lr": 0.03, "max_preconditioner_dim": 8}],
        betas=(0.9, 0.99), epsilon=1e-6, max_preconditioner_dim=16, precondition_frequency=1,
        start_preconditioning_step=2, preconditioner_config=_newton(), grafting_config=oa.AdamPreconditionerConfig(beta2=0.99, epsilon=1e-8))
    ra, rb = [a0.clone()], [b0.clone()]
    common = dict(betas=(0.9, 0.99), epsilon=1e-6, precondition_frequency=1, start_preconditioning_step=2,
                  grafting="adam", grafting_beta2=0.99, grafting_epsilon=1e-8)
    oa_ = _oracle(ra, lr=0.01, max_preconditioner_dim=16, **common)
    ob_ = _oracle(rb, lr=0.03, max_preconditioner_dim=8, **common)
    for _ in range(5):
        ga, gb = torch.randn(24, 16, generator=g), torch.randn(16, 40, generator=g)
        pa.grad, pb.grad = ga.to(DEV), gb.to(DEV)
        opt.step()
        oa_.step([ga.clone()])
        ob_.step([gb.clone()])
    assert rel_err(pa.detach().cpu(), ra[0]) < 1e-4 and rel_err(pb.detach().cpu(), rb[0]) < 1e-4


def test_non_integer_root_fails_like_reference_after_tolerance():
    """matrix_functions.py:670-673 raises inside the tolerated region of shampoo_preconditioner_list.py:430-443."""
    import optimizers_amd as oa

    p = torch.nn.Parameter(torch.randn(6, 6).to(DEV))
    opt = oa.DistributedShampoo([p], lr=0.01, betas=(0.0, 1.0), epsilon=1e-6, max_preconditioner_dim=8,
                                precondition_frequency=1, start_preconditioning_step=1,
                                preconditioner_config=_newton(inverse_exponent_override={2: 0.3}))
    for i in range(3):
        p.grad = torch.randn(6, 6).to(DEV)
        opt.step()  # tolerated: 3 failures
    p.grad = torch.randn(6, 6).to(DEV)
    with pytest.raises(ValueError, match="exceeded the allowed tolerance"):
        opt.step()


def test_nonfinite_gradient_raises_preconditioner_value_error():
    import optimizers_amd as oa

    p = torch.nn.Parameter(torch.randn(8, 8).to(DEV))
    opt = oa.DistributedShampoo([p], lr=0.01, betas=(0.9, 0.99), epsilon=1e-6, max_preconditioner_dim=8,
                                precondition_frequency=1, start_preconditioning_step=1, preconditioner_config=_newton())
    g = torch.randn(8, 8)
    g[2, 3] = float("nan")
    p.grad = g.to(DEV)
    with pytest.raises(oa.PreconditionerValueError, match="Encountered nan/inf values in factor matrix 0.block_0.0"):
        opt.step()
    opt2 = oa.DistributedShampoo([p], lr=0.01, epsilon=1e-6, preconditioner_config=_newton(),
                                 shampoo_runtime_config=oa.ShampooRuntimeConfig(eager_nan_check=True))
    with pytest.raises(AssertionError, match="Encountered gradient containing NaN/Inf"):
        opt2.step()


def test_large_ragged_kronecker_update_and_precondition():
    """GPT-2-like ragged blocks (81x768, 256x768, 1024x768) for two steps against the oracle."""
    import optimizers_amd as oa

    g = torch.Generator().manual_seed(21)
    shapes = [(1105, 768), (768, 1300), (768,)]
    init = [0.02 * torch.randn(*s, generator=g) for s in shapes]
    # epsilon = 1e-3 keeps the rank-deficient factors (81 or 337 rows feeding a 768 x 768 factor) well posed;
    # with 1e-12 the reference's Newton iteration returns rounding noise or raises on them
    kw = dict(lr=1e-3, betas=(0.9, 0.999), epsilon=1e-3, max_preconditioner_dim=1024, precondition_frequency=1,
              start_preconditioning_step=2)
    params = [torch.nn.Parameter(t.clone().to(DEV)) for t in init]
    opt = oa.DistributedShampoo(params, preconditioner_config=_newton(inverse_exponent_override={1: {0: 0.0}}),
                                grafting_config=oa.AdamPreconditionerConfig(beta2=0.999, epsilon=1e-8), **kw)
    ref_p = [t.clone() for t in init]
    ref = _oracle(ref_p, inverse_exponent_override={1: {0: 0.0}}, grafting="adam", grafting_beta2=0.999, grafting_epsilon=1e-8, **kw)
    for _ in range(3):
        grads = [0.02 * torch.randn(*s, generator=g) for s in shapes]
        for q, gr in zip(params, grads):
            q.grad = gr.to(DEV)
        opt.step()
        ref.step([x.clone() for x in grads])
    ng = opt._groups[0]
    for k, bi in enumerate(ng.native_index):
        spec = ng.block_specs[bi]
        st = opt.state[params[spec.param_index]][spec.block_key]
        for j, f in enumerate(ref.state[bi]["factors"]):
            assert rel_err(st["shampoo"]["factor_matrices"][j].cpu(), f) < 1e-5
        for j, f in enumerate(ref.state[bi]["inv"]):
            assert rel_err(st["shampoo"]["inv_factor_matrices"][j].cpu(), f) < 1e-3
    for q, r in zip(params, ref_p):
        assert rel_err(q.detach().cpu(), r) < 1e-4


@pytest.mark.parametrize("kind", ["newton", "eigh", "soap_qr"])
def test_zero_dimensional_empty_and_tiny_parameters(kind):
    """The reference's distributor fixture (shampoo_distributor_test.py:24-341): 0-D, empty, 1-D and tiny 2-D
    parameters in one group go through the same step."""
    import optimizers_amd as oa
    from oracle.shampoo_oracle import OracleConfig, ShampooOracle

    g = torch.Generator().manual_seed(0)
    shapes = [(), (0, 5), (7,), (6, 4), (1, 3)]
    init = [torch.randn(s, generator=g) for s in shapes]
    pc = {"newton": oa.RootInvShampooPreconditionerConfig(amortized_computation_config=oa.CoupledNewtonConfig()),
          "eigh": oa.DefaultShampooConfig, "soap_qr": oa.DefaultSOAPConfig}[kind]
    kw = dict(lr=1e-2, betas=(0.9, 0.99), epsilon=1e-4, max_preconditioner_dim=8, precondition_frequency=1,
              start_preconditioning_step=2)
    params = [torch.nn.Parameter(t.clone().to(DEV)) for t in init]
    opt = oa.DistributedShampoo(params, preconditioner_config=pc,
                                grafting_config=oa.AdamPreconditionerConfig(beta2=0.99, epsilon=1e-8), **kw)
    ref_p = [t.clone() for t in init]
    ref = ShampooOracle(ref_p, OracleConfig(preconditioner=kind, grafting="adam", grafting_beta2=0.99,
                                            grafting_epsilon=1e-8, **kw))
    for _ in range(4):
        grads = [torch.randn(s, generator=g) for s in shapes]
        for p, gr in zip(params, grads):
            p.grad = gr.to(DEV)
        opt.step()
        ref.step([x.clone() for x in grads])
    assert float(params[0].detach().cpu()) != float(init[0])  # the 0-D parameter is stepped
    assert rel_err(params[0].detach().cpu().reshape(1), ref_p[0].reshape(1)) < 1e-6
    assert params[1].numel() == 0
    # the 1-D block's factor has rank one with epsilon = 1e-4: loose bound, the others are well conditioned
    for p, r, tol in zip(params[2:], ref_p[2:], (5e-3, 1e-5, 1e-5)):
        assert rel_err(p.detach().cpu(), r) < tol


@pytest.mark.parametrize("kind", ["newton", "eigh"])
def test_order_three_blocks_with_every_kind_of_split(kind):
    """A conv weight whose merged shape 192 x 160 x 9 splits (max_preconditioner_dim = 128) into four order-3
    blocks, two of them views with a split middle dim, against the oracle for three steps."""
    import optimizers_amd as oa
    from oracle.shampoo_oracle import OracleConfig, ShampooOracle

    g = torch.Generator().manual_seed(33)
    shapes = [(192, 160, 3, 3), (40,)]
    init = [0.1 * torch.randn(*s, generator=g) for s in shapes]
    kw = dict(lr=1e-2, betas=(0.9, 0.99), epsilon=1e-6, max_preconditioner_dim=128, precondition_frequency=1,
              start_preconditioning_step=2, weight_decay=1e-3)
    acc = oa.CoupledNewtonConfig() if kind == "newton" else oa.EigenConfig()
    params = [torch.nn.Parameter(t.clone().to(DEV)) for t in init]
    opt = oa.DistributedShampoo(
        params, preconditioner_config=oa.RootInvShampooPreconditionerConfig(
            amortized_computation_config=acc, inverse_exponent_override={1: {0: 0.0}}),  # the rank-3 factor of the vector is left out
        grafting_config=oa.AdamPreconditionerConfig(beta2=0.99, epsilon=1e-8), **kw)
    assert [opt._groups[0].block_specs[i].shape for i in range(4)] == [(128, 128, 9), (128, 32, 9), (64, 128, 9), (64, 32, 9)]
    ref_p = [t.clone() for t in init]
    ref = ShampooOracle(ref_p, OracleConfig(preconditioner=kind, grafting="adam", grafting_beta2=0.99,
                                            grafting_epsilon=1e-8, inverse_exponent_override={1: {0: 0.0}}, **kw))
    for _ in range(3):
        grads = [torch.randn(*s, generator=g) for s in shapes]
        for q, gr in zip(params, grads):
            q.grad = gr.to(DEV)
        opt.step()
        ref.step([x.clone() for x in grads])
    ng = opt._groups[0]
    for k, bi in enumerate(ng.native_index):
        spec = ng.block_specs[bi]
        st = opt.state[params[spec.param_index]][spec.block_key]
        for j, f in enumerate(ref.state[bi]["factors"]):
            assert rel_err(st["shampoo"]["factor_matrices"][j].cpu(), f) < 1e-5
        for j, f in enumerate(ref.state[bi]["inv"]):
            assert rel_err(st["shampoo"]["inv_factor_matrices"][j].cpu(), f) < 1e-3
    for q, r in zip(params, ref_p):
        assert rel_err(q.detach().cpu(), r) < 1e-4


def test_parameter_storage_replaced_between_steps_is_followed():
    """`p.data = ...` after the optimizer was built: the native plan holds raw pointers and is re-pointed, so the new
    storage is what gets updated.  Not parity but a deliberate deviation: the reference's blocks are detached views of the
    storage that existed at construction (shampoo_distributor.py:202-216), and it would keep updating (and reading) the
    old allocation."""
    import optimizers_amd as oa

    def run(swap: bool):
        g = torch.Generator().manual_seed(3)
        params = [torch.nn.Parameter(torch.randn(96, 80, generator=g).cuda()), torch.nn.Parameter(torch.randn(80, generator=g).cuda())]
        opt = oa.DistributedShampoo(
            params, lr=1e-2, betas=(0.9, 0.99), epsilon=1e-8, weight_decay=1e-2, max_preconditioner_dim=64,
            precondition_frequency=1, start_preconditioning_step=2,
            preconditioner_config=oa.RootInvShampooPreconditionerConfig(
                amortized_computation_config=oa.CoupledNewtonConfig(), inverse_exponent_override={1: {0: 0.0}}),
            grafting_config=oa.AdamPreconditionerConfig(beta2=0.99, epsilon=1e-8))
        old = None
        for step in range(6):
            if swap and step == 3:
                old = [p.data for p in params]
                frozen = [t.clone() for t in old]
                for p in params:
                    p.data = p.data.clone()  # new storage, same values
            for p in params:
                p.grad = torch.randn(p.shape, generator=g).cuda()
            opt.step()
        torch.cuda.synchronize()
        if swap:
            for t, f in zip(old, frozen):
                assert torch.equal(t, f)  # nothing wrote to the abandoned storage
        return [p.detach().clone() for p in params]

    for a, b in zip(run(False), run(True)):
        assert torch.equal(a, b)


def test_checkpoint_written_by_the_reference_is_loaded_and_resumed():
    """tests/distributed_shampoo_test.py:395-431 across implementations: `tests/golden/state_dict_resume.npz` holds the
    `state_dict()["state"]` the REFERENCE wrote after 7 steps (its own nesting: state / param / block / shampoo / ...), the
    parameters at that moment and the parameters 5 steps later.  The native optimizer loads it with load_state_dict and
    must arrive where the reference arrived."""
    import json
    import os

    import optimizers_amd as oa
    from tests.golden_cases import GOLDEN, case_grads, load_npz

    z = load_npz("state_dict_resume")
    with open(os.path.join(GOLDEN, "state_dict_resume.json")) as f:
        meta = json.load(f)
    c = meta["case"]
    shapes = [tuple(s) for s in c["shapes"]]
    params = [torch.nn.Parameter(torch.from_numpy(z[f"params_at_save_p{i}"]).to(DEV)) for i in range(len(shapes))]
    opt = oa.DistributedShampoo(
        params, lr=c["lr"], betas=tuple(c["betas"]), epsilon=c["epsilon"], weight_decay=c["weight_decay"],
        weight_decay_type=oa.WeightDecayType[c["weight_decay_type"]], max_preconditioner_dim=c["max_preconditioner_dim"],
        precondition_frequency=c["precondition_frequency"], start_preconditioning_step=c["start_preconditioning_step"],
        preconditioner_config=oa.RootInvShampooPreconditionerConfig(
            amortized_computation_config=oa.CoupledNewtonConfig(), inverse_exponent_override={1: {0: 0.0}}),
        grafting_config=oa.AdamPreconditionerConfig(beta2=c["grafting_beta2"], epsilon=c["grafting_epsilon"]),
        iterate_averaging_config=oa.ClassicMomentumConfig(momentum=c["momentum"], dampening=c["dampening"], use_nesterov=c["use_nesterov"]))
    own = opt.state_dict()

    def leaves(prefix, node, out):
        if isinstance(node, dict):
            for k, v in node.items():
                leaves(f"{prefix}/{k}", v, out)
        else:
            out[prefix] = node
        return out

    # the reference's checkpoint has exactly the leaves the native optimizer's own state_dict has
    assert sorted(leaves("state", own["state"], {})) == meta["keys"]
    state = {}
    for key in meta["keys"]:
        node = state
        parts = key.split("/")[1:]
        for part in parts[:-1]:
            node = node.setdefault(int(part) if part.isdigit() else part, {})
        leaf = parts[-1]
        node[int(leaf) if leaf.isdigit() else leaf] = torch.from_numpy(z[key])
    opt.load_state_dict({"state": state, "param_groups": own["param_groups"]})
    assert int(opt.state[params[0]]["step"]) == meta["saved_after_step"]
    for s in range(meta["saved_after_step"] + 1, meta["steps"] + 1):
        for p, g in zip(params, case_grads(shapes, c["seed"], s, c["grad_scale"])):
            p.grad = g.to(DEV)
        opt.step()
    torch.cuda.synchronize()
    for i, p in enumerate(params):
        err = rel_err(p.detach().cpu(), z[f"final_p{i}"])
        print(f"parameter {i}: resumed from the reference's checkpoint, rel. error to the reference's run {err:.2e}", flush=True)
        assert err < 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["newton", "eigh", "soap", "newton_f64"])
def test_state_without_symmetric_packing_is_dense_and_changes_nothing_else(kind):
    """use_symmetric_packing=False (shampoo_types.py:170-186, shampoo_preconditioner_list.py:139-156, 283-301): the state
    holds d x d factor matrices and inverse roots instead of packed triangles.  Same seeds with and without packing:
    identical parameters, dense state = mirror of the packed state bit for bit, and a checkpoint taken in the dense layout
    resumes where the uninterrupted run goes.  (Shapes and values against the reference itself: fixture `dense_state_newton`, checked by
    test_step_matches_oracle_and_reference_fixture.)"""
    import optimizers_amd as oa

    def config(packing):
        if kind == "soap":
            return oa.EigenvalueCorrectedShampooPreconditionerConfig(
                amortized_computation_config=oa.QREigendecompositionConfig(), use_symmetric_packing=packing)
        extra = {"factor_matrix_dtype": torch.float64} if kind == "newton_f64" else {}
        return oa.RootInvShampooPreconditionerConfig(
            amortized_computation_config=oa.EigenConfig() if kind == "eigh" else oa.CoupledNewtonConfig(),
            inverse_exponent_override={1: {0: 0.0}}, use_symmetric_packing=packing, **extra)

    def make(init, packing):
        ps = [torch.nn.Parameter(t.clone().to(DEV)) for t in init]
        o = oa.DistributedShampoo(ps, lr=0.01, betas=(0.9, 0.99), epsilon=1e-4, max_preconditioner_dim=96,
                                  precondition_frequency=2, start_preconditioning_step=2, preconditioner_config=config(packing),
                                  grafting_config=None if kind == "soap" else oa.AdamPreconditionerConfig(beta2=0.99, epsilon=1e-8))
        return ps, o

    g = torch.Generator().manual_seed(11)
    init = [torch.randn(130, 200, generator=g) * 0.1, torch.randn(70, generator=g) * 0.1]
    grads = [[torch.randn(130, 200, generator=g), torch.randn(70, generator=g)] for _ in range(7)]
    packed_p, packed_o = make(init, True)
    dense_p, dense_o = make(init, False)
    saved = saved_w = None
    for s, gs in enumerate(grads):
        for ps, o in ((packed_p, packed_o), (dense_p, dense_o)):
            for p, gr in zip(ps, gs):
                p.grad = gr.to(DEV)
            o.step()
        if s == 3:
            saved = copy.deepcopy(dense_o.state_dict())
            saved_w = [p.detach().clone().cpu() for p in dense_p]
    for a, b in zip(packed_p, dense_p):
        assert torch.equal(a.detach(), b.detach())

    def unpack(t, n):
        m = torch.zeros(n, n, dtype=t.dtype, device=t.device)
        iu = torch.triu_indices(n, n, device=t.device)
        m[iu[0], iu[1]] = t
        return torch.triu(m) + torch.triu(m, 1).T

    checked = 0
    for pp, dp in zip(packed_p, dense_p):
        for key, blk in packed_o.state[pp].items():
            if not isinstance(blk, dict) or "shampoo" not in blk:
                continue
            dblk = dense_o.state[dp][key]["shampoo"]
            for name in ("factor_matrices", "inv_factor_matrices"):
                for j, t in blk["shampoo"].get(name, {}).items():
                    d = dblk[name][j]
                    assert d.dim() == 2 and d.shape[0] == d.shape[1] and t.numel() == d.shape[0] * (d.shape[0] + 1) // 2
                    assert d.dtype == t.dtype and torch.equal(d, unpack(t, d.shape[0])), (name, key, j)
                    checked += 1
    assert checked >= (4 if kind == "soap" else 8)

    # a checkpoint in the dense layout: resume in a fresh optimizer, arrive at the same parameters
    ps2, o2 = make(saved_w, False)
    o2.load_state_dict(saved)
    for gs in grads[4:]:
        for p, gr in zip(ps2, gs):
            p.grad = gr.to(DEV)
        o2.step()
    # (not bit for bit: which Newton products run in their symmetric form depends on the previous solve of the same
    # optimizer object, which a fresh one has not had)
    for a, b in zip(ps2, dense_p):
        assert rel_err(a.detach().cpu(), b.detach().cpu()) < 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["newton", "soap"])
def test_small_launches_give_the_same_bits_with_either_tile_size(kind):
    """Launches of fewer than 256 large tiles run as 64 x 64 tiles (sa_set_small_launch_tiles).  Every output element sees
    the same sequence of matrix-core instructions and the same epilogue arithmetic either way, so parameters and factor
    matrices must agree bit for bit -- which they only do with floating-point contraction off in the kernel: the
    compiler fused a different product of the factor average in each instantiation."""
    import optimizers_amd as oa
    from optimizers_amd import native

    lib = native.load()

    def run(tiles):
        native.check(lib.sa_set_small_launch_tiles(tiles), "sa_set_small_launch_tiles")
        g = torch.Generator().manual_seed(3)
        ps = [torch.nn.Parameter((torch.randn(256, 512, generator=g) * 0.1).to(DEV))]
        if kind == "soap":
            pc = oa.EigenvalueCorrectedShampooPreconditionerConfig(amortized_computation_config=oa.QREigendecompositionConfig())
            graft = None
        else:
            pc = oa.RootInvShampooPreconditionerConfig(amortized_computation_config=oa.CoupledNewtonConfig())
            graft = oa.AdamPreconditionerConfig(beta2=0.99, epsilon=1e-8)
        o = oa.DistributedShampoo(ps, lr=0.01, betas=(0.9, 0.99), epsilon=1e-6, max_preconditioner_dim=256,
                                  precondition_frequency=2, start_preconditioning_step=2, preconditioner_config=pc,
                                  grafting_config=graft)
        out = []
        for _ in range(4):
            ps[0].grad = torch.randn(256, 512, generator=g).to(DEV)
            o.step()
            st = o.state[ps[0]]
            out.append([st[k]["shampoo"]["factor_matrices"][j].clone() for k in ("block_0", "block_1") for j in (0, 1)]
                       + [ps[0].detach().clone()])
        return out

    try:
        large, small = run(0), run(256)
    finally:
        native.check(lib.sa_set_small_launch_tiles(256), "sa_set_small_launch_tiles")
    for a, b in zip(large, small):
        for x, y in zip(a, b):
            assert torch.equal(x, y)


@pytest.mark.gpu
def test_late_newton_iterations_in_small_tiles_give_the_same_bits():
    """A coupled Newton batch whose launches are large (here 32 factors of order 512: 512 large tiles per full product, 320
    per symmetric one) ends with a few badly conditioned factors still iterating; from the
    second solve on the host knows from the previous one which, and runs those late stages in 64 x 64 tiles.  Parameters
    and inverse roots must equal, bit for bit, those of a run that keeps the large tiles throughout."""
    import optimizers_amd as oa
    from optimizers_amd import native

    lib = native.load()

    def run(tiles):
        native.check(lib.sa_set_small_launch_tiles(tiles), "sa_set_small_launch_tiles")
        g = torch.Generator().manual_seed(11)
        ps = [torch.nn.Parameter((torch.randn(512, 512, generator=g) * 0.1).to(DEV)) for _ in range(16)]
        # spectra from flat to steep: the Newton iteration counts of the factors spread over a wide range
        decay = [10.0 ** (-0.05 * i * torch.linspace(0, 1, 512)) for i in range(16)]
        o = oa.DistributedShampoo(ps, lr=0.01, betas=(0.9, 0.99), epsilon=1e-8, max_preconditioner_dim=512,
                                  precondition_frequency=1, start_preconditioning_step=1,
                                  preconditioner_config=oa.RootInvShampooPreconditionerConfig(
                                      amortized_computation_config=oa.CoupledNewtonConfig()),
                                  grafting_config=oa.AdamPreconditionerConfig(beta2=0.99, epsilon=1e-8))
        out = []
        for _ in range(4):
            for p, w in zip(ps, decay):
                p.grad = (torch.randn(512, 512, generator=g) * w[None, :] * w[:, None]).to(DEV)
            o.step()
            out.append([o.state[p]["block_0"]["shampoo"]["inv_factor_matrices"][j].clone() for p in ps for j in (0, 1)]
                       + [p.detach().clone() for p in ps])
        return out

    try:
        large, small = run(0), run(256)
    finally:
        native.check(lib.sa_set_small_launch_tiles(256), "sa_set_small_launch_tiles")
    for a, b in zip(large, small):
        for x, y in zip(a, b):
            assert torch.equal(x, y)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["newton", "higher_order", "eigh", "newton_f64", "eigh_f64", "soap_qr", "soap_eigh", "eigendecomposed"])
def test_every_amortized_computation_gives_the_same_bits_in_waves(kind):
    """sa_plan_set_scratch_budget cuts the factors of an amortized computation into consecutive waves that share one
    scratch region.  Every entry point runs wave by wave through the same wrapper; a budget that holds two factors at a
    time must leave the same parameters and the same state, bit for bit, as the default (everything at once)."""
    import os

    import optimizers_amd as oa
    from optimizers_amd.distributed_shampoo import _NativeGroup

    if "SHAMPOO_AMD_SCRATCH_BYTES" in os.environ:
        pytest.skip("the environment overrides the scratch budget this test sets")
    f64 = {"factor_matrix_dtype": torch.float64} if kind.endswith("_f64") else {}
    if kind in ("newton", "newton_f64"):
        pc = oa.RootInvShampooPreconditionerConfig(amortized_computation_config=oa.CoupledNewtonConfig(), **f64)
    elif kind == "higher_order":
        pc = oa.RootInvShampooPreconditionerConfig(amortized_computation_config=oa.CoupledHigherOrderConfig(rel_epsilon=1e-6, abs_epsilon=0.0))
    elif kind in ("eigh", "eigh_f64"):
        pc = oa.RootInvShampooPreconditionerConfig(amortized_computation_config=oa.EigenConfig(), **f64)
    elif kind == "soap_qr":
        pc = oa.EigenvalueCorrectedShampooPreconditionerConfig(amortized_computation_config=oa.QREigendecompositionConfig())
    elif kind == "soap_eigh":
        pc = oa.EigenvalueCorrectedShampooPreconditionerConfig(amortized_computation_config=oa.EighEigendecompositionConfig())
    else:
        pc = oa.EigendecomposedShampooPreconditionerConfig(amortized_computation_config=oa.EighEigendecompositionConfig())
    g = torch.Generator().manual_seed(17)
    init = [torch.randn(128, 256, generator=g) * 0.1, torch.randn(100, 64, generator=g) * 0.1]
    grads = [[torch.randn(128, 256, generator=g), torch.randn(100, 64, generator=g)] for _ in range(6)]
    saved = _NativeGroup.scratch_budget_bytes
    runs = []
    try:
        # 64-blocks: 2 x 4 + 2 x 1 = 10 blocks, 20 factors of order <= 64 (dpad 128: 512 KB of scratch each, 1 MB in double)
        for budget in ((2 << 20) + 4096 if f64 else (1 << 20) + 4096, None):
            _NativeGroup.scratch_budget_bytes = budget
            ps = [torch.nn.Parameter(t.clone().to(DEV)) for t in init]
            o = oa.DistributedShampoo(ps, lr=0.01, betas=(0.9, 0.99), epsilon=1e-3, max_preconditioner_dim=64,
                                      precondition_frequency=2, start_preconditioning_step=3, preconditioner_config=pc,
                                      grafting_config=None if kind.startswith("soap") else oa.AdamPreconditionerConfig(beta2=0.99, epsilon=1e-8))
            ng = o._groups[0]
            waves = int(ng.lib.sa_plan_num_waves(ng.plan))
            for gs in grads:
                for p, gr in zip(ps, gs):
                    p.grad = gr.to(DEV)
                o.step()
            torch.cuda.synchronize()
            state = [t.clone() for _, _, _, t in ng._slots]
            runs.append((waves, [p.detach().clone() for p in ps], state))
    finally:
        _NativeGroup.scratch_budget_bytes = saved
    (waves_c, p_c, s_c), (waves_u, p_u, s_u) = runs
    print(f"{kind}: {waves_c} waves under the budget, {waves_u} without", flush=True)
    assert waves_u == 1 and waves_c >= 3
    for a, b in zip(p_c, p_u):
        assert torch.equal(a, b)
    for a, b in zip(s_c, s_u):
        assert torch.equal(a, b)


def test_newton_batch_in_two_halves_side_by_side_gives_the_bits_of_the_whole_batch():
    """sa_plan_set_newton_split_tiles: a batch of coupled Newton iterations whose stages are short launches iterates as
    two halves on two streams.  Factors are independent of each other, so parameters, every state tensor and the
    per-factor iteration counts must equal those of the unsplit run bit for bit; factors of five orders (1024, 768, 512,
    384, 256), some of which converge earlier than others, and a second amortized computation that predicts its iteration
    count from the first."""
    import optimizers_amd as oa

    g = torch.Generator().manual_seed(23)
    from optimizers_amd import native

    # 36 factors, 574 tiles per stage with symmetric products (a batch splits from 512 tiles and 8 factors on)
    shapes = [(768, 512), (512, 384), (384, 256), (256, 768), (512, 512), (768, 768)] + [(1024, 1024)] * 6
    init = [torch.randn(s, generator=g) * 0.1 for s in shapes]
    # a few low-rank directions on top of the noise give the factors different condition numbers
    lows = [(torch.randn(s[0], 4, generator=g), torch.randn(4, s[1], generator=g)) for s in shapes]
    grads = [[0.1 * torch.randn(s, generator=g) + 0.05 * k * (a @ b) for k, (s, (a, b)) in enumerate(zip(shapes, lows))]
             for _ in range(6)]
    runs = []
    for split_tiles in (1 << 20, 0):
        ps = [torch.nn.Parameter(t.clone().to(DEV)) for t in init]
        o = oa.DistributedShampoo(
            ps, lr=0.01, betas=(0.9, 0.99), epsilon=1e-8, max_preconditioner_dim=1024, precondition_frequency=1,
            start_preconditioning_step=4,
            preconditioner_config=oa.RootInvShampooPreconditionerConfig(amortized_computation_config=oa.CoupledNewtonConfig()),
            grafting_config=oa.AdamPreconditionerConfig(beta2=0.99, epsilon=1e-8))
        ng = o._groups[0]
        native.check(ng.lib.sa_plan_set_newton_split_tiles(ng.plan, split_tiles), "sa_plan_set_newton_split_tiles")
        counts = []
        for gs in grads:
            for p, gr in zip(ps, gs):
                p.grad = gr.to(DEV)
            o.step()
            counts.append(list(ng.last_newton_iterations))
        torch.cuda.synchronize()
        runs.append(([p.detach().clone() for p in ps], [t.clone() for _, _, _, t in ng._slots], counts))
    (p_s, s_s, c_s), (p_u, s_u, c_u) = runs
    print(f"iteration counts per amortized computation: {[c for c in c_u if c]}", flush=True)
    assert c_s == c_u and any(len(set(c)) > 1 for c in c_u if c)
    for a, b in zip(p_s, p_u):
        assert torch.isfinite(a).all() and torch.equal(a, b)
    for a, b in zip(s_s, s_u):
        assert torch.equal(a, b)
