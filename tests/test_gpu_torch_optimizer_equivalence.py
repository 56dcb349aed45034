"""The reference's equivalence suites on the MI355X (gpu_tests/shampoo_grafting_test.py:68-266,
gpu_tests/weight_decay_test.py): with start_preconditioning_step = inf, Distributed Shampoo with a grafting
method is that method, so five steps on the reference's toy problem (tests/shampoo_test_utils.py: seed 42,
unit-norm inputs, a learnable 0-D scalar plus linear layers (10, 1, 1) filled with ones, MSE against zero) must give
the weights and the loss of torch.optim.{Adagrad, Adam, AdamW, RMSprop, SGD} run on the same device."""

import math
from functools import partial
from itertools import pairwise

import pytest
import torch
from torch import nn
from torch.optim import SGD, Adagrad, Adam, AdamW, RMSprop

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


class _Model(nn.Module):
    def __init__(self, dims):
        super().__init__()
        self.scalar = nn.Parameter(torch.zeros(()))
        self.linear_layers = nn.Sequential(*(nn.Linear(a, b, bias=False) for a, b in pairwise(dims)))

    def forward(self, x):
        return self.linear_layers(x) + self.scalar


def _train(optim_factory, dims, steps=5):
    torch.manual_seed(42)
    data = torch.randn(dims[0], dtype=torch.float)
    data /= torch.linalg.norm(data)
    model = _Model(dims).to(DEV)
    for m in model.linear_layers:
        nn.init.constant_(m.weight, 1.0)
    loss = nn.MSELoss()
    target = torch.tensor([[0.0] * dims[-1]], device=DEV)
    opt = optim_factory(model.parameters())
    torch.manual_seed(42)
    train = torch.randn(steps, dims[0], dtype=torch.float)
    train /= torch.linalg.norm(train, dim=-1, keepdim=True)
    train = train.to(DEV)
    for s in range(steps):
        opt.zero_grad()
        loss(model(train[s]), target).backward()
        opt.step()
    final = loss(model(data.to(DEV).unsqueeze(0)), target)
    return [p.detach().clone() for p in model.parameters()], final.detach()


def _compare(control, experimental, dims=(10, 1, 1)):
    want_p, want_l = _train(control, dims)
    got_p, got_l = _train(experimental, dims)
    torch.testing.assert_close(got_l, want_l)
    torch.testing.assert_close(got_p, want_p)


def _configs():
    import optimizers_amd as oa

    return (oa.DefaultShampooConfig, oa.DefaultEigenvalueCorrectedShampooConfig, oa.DefaultSOAPConfig,
            oa.EigendecomposedShampooPreconditionerConfig())


def _shampoo(params, **kw):
    import optimizers_amd as oa

    kw["weight_decay_type"] = getattr(oa.WeightDecayType, kw["weight_decay_type"])
    return oa.DistributedShampoo(params, max_preconditioner_dim=10, precondition_frequency=1,
                                 start_preconditioning_step=math.inf, **kw)


@pytest.mark.parametrize("which", range(4))
@pytest.mark.parametrize("weight_decay", (0.0, 0.3))
def test_adagrad_grafting(weight_decay, which):
    import optimizers_amd as oa

    _compare(partial(Adagrad, lr=0.01, weight_decay=weight_decay, eps=1e-10),
             partial(_shampoo, lr=0.01, weight_decay=weight_decay, betas=(0.0, 1.0), epsilon=1e-10, weight_decay_type="L2",
                     grafting_config=oa.AdaGradPreconditionerConfig(epsilon=1e-10), preconditioner_config=_configs()[which]))


@pytest.mark.parametrize("which", range(4))
@pytest.mark.parametrize("weight_decay", (0.0, 0.3))
def test_adam_grafting(weight_decay, which):
    import optimizers_amd as oa

    _compare(partial(Adam, lr=0.001, betas=(0.9, 0.999), weight_decay=weight_decay, eps=1e-8),
             partial(_shampoo, lr=0.001, betas=(0.9, 0.999), weight_decay=weight_decay, epsilon=1e-8, weight_decay_type="L2",
                     grafting_config=oa.AdamPreconditionerConfig(beta2=0.999, epsilon=1e-8),
                     preconditioner_config=_configs()[which]))


@pytest.mark.parametrize("which", range(4))
@pytest.mark.parametrize("weight_decay", (0.0, 0.3))
def test_adamw_grafting(weight_decay, which):
    import optimizers_amd as oa

    _compare(partial(AdamW, lr=0.001, betas=(0.9, 0.999), weight_decay=weight_decay, eps=1e-8),
             partial(_shampoo, lr=0.001, betas=(0.9, 0.999), weight_decay=weight_decay, epsilon=1e-8,
                     weight_decay_type="DECOUPLED", grafting_config=oa.AdamPreconditionerConfig(beta2=0.999, epsilon=1e-8),
                     preconditioner_config=_configs()[which]))


@pytest.mark.parametrize("which", range(4))
@pytest.mark.parametrize("weight_decay", (0.0, 0.3))
def test_rmsprop_grafting(weight_decay, which):
    import optimizers_amd as oa

    _compare(partial(RMSprop, lr=0.01, weight_decay=weight_decay, alpha=0.99, eps=1e-8),
             partial(_shampoo, lr=0.01, weight_decay=weight_decay, betas=(0.0, 0.99), epsilon=1e-8, use_bias_correction=False,
                     weight_decay_type="L2", grafting_config=oa.RMSpropPreconditionerConfig(beta2=0.99, epsilon=1e-8),
                     preconditioner_config=_configs()[which]))


@pytest.mark.parametrize("which", range(4))
@pytest.mark.parametrize("weight_decay", (0.0, 0.3))
def test_sgd_grafting(weight_decay, which):
    import optimizers_amd as oa

    _compare(partial(SGD, lr=0.1, weight_decay=weight_decay),
             partial(_shampoo, lr=0.1, weight_decay=weight_decay, betas=(0.0, 1.0), epsilon=1e-10, weight_decay_type="L2",
                     grafting_config=oa.SGDPreconditionerConfig(), preconditioner_config=_configs()[which]),
             dims=(10, 10))


@pytest.mark.parametrize("nesterov", (False, True))
def test_sgd_momentum_through_classic_momentum(nesterov):
    """gpu_tests/iterate_averaging_test.py: ClassicMomentumConfig on top of SGD grafting is torch's SGD momentum."""
    import optimizers_amd as oa

    _compare(partial(SGD, lr=0.1, momentum=0.5, nesterov=nesterov),
             partial(_shampoo, lr=0.1, weight_decay=0.0, betas=(0.0, 1.0), epsilon=1e-10, weight_decay_type="L2",
                     grafting_config=oa.SGDPreconditionerConfig(),
                     iterate_averaging_config=oa.ClassicMomentumConfig(momentum=0.5, use_nesterov=nesterov),
                     preconditioner_config=oa.DefaultShampooConfig),
             dims=(10, 10))


@pytest.mark.parametrize("which", range(4))
@pytest.mark.parametrize("weight_decay", (0.0, 0.3))
def test_corrected_weight_decay(weight_decay, which):
    """gpu_tests/weight_decay_test.py:170-217: at a constant learning rate (lr == peak_lr) the corrected decay
    params *= 1 - lr * (lr / peak_lr) * weight_decay is AdamW's."""
    import optimizers_amd as oa

    _compare(partial(AdamW, lr=0.001, betas=(0.9, 0.999), weight_decay=weight_decay, eps=1e-8),
             partial(_shampoo, lr=0.001, betas=(0.9, 0.999), weight_decay=weight_decay, epsilon=1e-8,
                     weight_decay_type="CORRECTED", grafting_config=oa.AdamPreconditionerConfig(beta2=0.999, epsilon=1e-8),
                     preconditioner_config=_configs()[which]))


@pytest.mark.parametrize("which", range(4))
@pytest.mark.parametrize("weight_decay", (0.0, 0.3))
def test_independent_weight_decay(weight_decay, which):
    """gpu_tests/weight_decay_test.py:219-270: the independent decay params *= 1 - (lr / peak_lr) * weight_decay is,
    at a constant learning rate, AdamW with weight_decay / lr."""
    import optimizers_amd as oa

    lr = 0.001
    _compare(partial(AdamW, lr=lr, betas=(0.9, 0.999), weight_decay=weight_decay / lr, eps=1e-8),
             partial(_shampoo, lr=lr, betas=(0.9, 0.999), weight_decay=weight_decay, epsilon=1e-8,
                     weight_decay_type="INDEPENDENT", grafting_config=oa.AdamPreconditionerConfig(beta2=0.999, epsilon=1e-8),
                     preconditioner_config=_configs()[which]))


def test_generalized_primal_averaging_is_heavy_ball_momentum():
    """gpu_tests/iterate_averaging_test.py:80-144: with the gradient taken at the averaged iterate itself
    (train_interp_coeff = 1) and eval_interp_coeff = momentum, primal averaging over plain SGD at lr / (1 - momentum)
    is torch's SGD with heavy-ball momentum."""
    import optimizers_amd as oa

    lr, momentum = 0.1, 0.9
    _compare(partial(SGD, lr=lr, momentum=momentum, weight_decay=0.0),
             lambda ps: oa.DistributedShampoo(
                 ps, lr=lr / (1 - momentum), betas=(0.0, 1.0), epsilon=1e-10, weight_decay=0.0, max_preconditioner_dim=10,
                 precondition_frequency=1, start_preconditioning_step=-1, weight_decay_type=oa.WeightDecayType.L2,
                 preconditioner_config=oa.SGDPreconditionerConfig(), grafting_config=None,
                 iterate_averaging_config=oa.GeneralizedPrimalAveragingConfig(eval_interp_coeff=momentum,
                                                                              train_interp_coeff=1.0)),
             dims=(10, 10))


@pytest.mark.parametrize("nesterov", (False, True))
def test_classic_momentum_over_the_sgd_preconditioner(nesterov):
    """gpu_tests/iterate_averaging_test.py:265-305: ClassicMomentumConfig with dampening 0 over
    `preconditioner_config=SGDPreconditionerConfig()` is torch's SGD momentum."""
    import optimizers_amd as oa

    _compare(partial(SGD, lr=0.01, weight_decay=0.0, momentum=0.9, dampening=0.0, nesterov=nesterov),
             lambda ps: oa.DistributedShampoo(
                 ps, lr=0.01, betas=(0.0, 1.0), epsilon=1e-10, weight_decay=0.0, max_preconditioner_dim=10,
                 precondition_frequency=1, start_preconditioning_step=-1, weight_decay_type=oa.WeightDecayType.L2,
                 preconditioner_config=oa.SGDPreconditionerConfig(), grafting_config=None,
                 iterate_averaging_config=oa.ClassicMomentumConfig(momentum=0.9, dampening=0.0, use_nesterov=nesterov)),
             dims=(10, 10))


@pytest.mark.parametrize("weight_decay", (0.0, 0.3))
def test_elementwise_methods_as_the_preconditioner_itself(weight_decay):
    """`preconditioner_config=AdamPreconditionerConfig(...)` etc. without grafting (distributed_shampoo.py:673-714: the
    reference then runs its Adagrad list in place of a Shampoo list) is the torch optimizer of that name."""
    import optimizers_amd as oa

    common = dict(max_preconditioner_dim=10, precondition_frequency=1, start_preconditioning_step=1, weight_decay=weight_decay)
    _compare(partial(Adam, lr=0.001, betas=(0.9, 0.999), weight_decay=weight_decay, eps=1e-8),
             lambda ps: oa.DistributedShampoo(ps, lr=0.001, betas=(0.9, 0.999), epsilon=1e-8, weight_decay_type=oa.WeightDecayType.L2,
                                              preconditioner_config=oa.AdamPreconditionerConfig(beta2=0.999, epsilon=1e-8), **common))
    _compare(partial(AdamW, lr=0.001, betas=(0.9, 0.999), weight_decay=weight_decay, eps=1e-8),
             lambda ps: oa.DistributedShampoo(ps, lr=0.001, betas=(0.9, 0.999), epsilon=1e-8, weight_decay_type=oa.WeightDecayType.DECOUPLED,
                                              preconditioner_config=oa.AdamPreconditionerConfig(beta2=0.999, epsilon=1e-8), **common))
    _compare(partial(Adagrad, lr=0.01, weight_decay=weight_decay, eps=1e-10),
             lambda ps: oa.DistributedShampoo(ps, lr=0.01, betas=(0.0, 1.0), epsilon=1e-10, weight_decay_type=oa.WeightDecayType.L2,
                                              preconditioner_config=oa.AdaGradPreconditionerConfig(epsilon=1e-10), **common))
    _compare(partial(RMSprop, lr=0.01, weight_decay=weight_decay, alpha=0.99, eps=1e-8),
             lambda ps: oa.DistributedShampoo(ps, lr=0.01, betas=(0.0, 0.99), epsilon=1e-8, use_bias_correction=False,
                                              weight_decay_type=oa.WeightDecayType.L2,
                                              preconditioner_config=oa.RMSpropPreconditionerConfig(beta2=0.99, epsilon=1e-8), **common))
    _compare(partial(SGD, lr=0.1, weight_decay=weight_decay),
             lambda ps: oa.DistributedShampoo(ps, lr=0.1, betas=(0.0, 1.0), epsilon=1e-10, weight_decay_type=oa.WeightDecayType.L2,
                                              preconditioner_config=oa.SGDPreconditionerConfig(), **common),
             dims=(10, 10))


def test_grafting_on_an_elementwise_preconditioner_is_rejected():
    import optimizers_amd as oa

    p = torch.nn.Parameter(torch.zeros(4, 4, device=DEV))
    with pytest.raises(NotImplementedError, match="element-wise preconditioner_config"):
        oa.DistributedShampoo([p], preconditioner_config=oa.AdamPreconditionerConfig(),
                              grafting_config=oa.SGDPreconditionerConfig())
