"""The default distributor on the MI355X, driven like the reference's own tests
(distributor/tests/shampoo_distributor_test.py:20-330: model = 0-D scalar + Linear(10, 5) with bias, zero filled,
max_preconditioner_dim 5 -> blocks scalar, two 5x5 weight blocks, bias), plus the native strided update on ragged,
column-split and order-3 views against torch's own addition (bit-exact: one fp32 add per element)."""

from unittest import mock

import pytest
import torch
from torch import nn

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
D = 5


class _Model(nn.Module):
    def __init__(self, dims, bias):
        super().__init__()
        self.scalar = nn.Parameter(torch.zeros(()))
        self.linear_layers = nn.ModuleList([nn.Linear(a, b, bias=bias) for a, b in zip(dims[:-1], dims[1:])])
        for layer in self.linear_layers:
            nn.init.zeros_(layer.weight)
            if bias:
                nn.init.zeros_(layer.bias)


def _distributor(model, runtime_config=None, max_dim=D):
    import optimizers_amd as oa
    from optimizers_amd.distributor import Distributor

    opt = oa.DistributedShampoo(model.parameters(), max_preconditioner_dim=max_dim)
    return Distributor(param_group=opt.param_groups[0], runtime_config=runtime_config)


@pytest.fixture
def setup():
    model = _Model((2 * D, D), bias=True).to(DEV)
    return model, _distributor(model)


def _mask_scalar_and_bias(model):
    model.scalar.grad = None
    w = model.linear_layers[0].weight
    w.grad = torch.ones_like(w)
    model.linear_layers[0].bias.grad = None


def test_update_params(setup):
    model, dist = setup
    _mask_scalar_and_bias(model)
    dist.merge_and_block_gradients()
    directions = (
        torch.arange(D * D, dtype=torch.float, device=DEV).reshape(D, D),
        torch.arange(D * D, 2 * D * D, dtype=torch.float, device=DEV).reshape(D, D),
    )
    dist.update_params(blocked_search_directions=directions)
    torch.testing.assert_close(dist.local_masked_blocked_params, directions, rtol=0, atol=0)
    # the blocks are views: the parameter itself moved (columns 0-4 and 5-9 of the 5 x 10 weight)
    torch.testing.assert_close(model.linear_layers[0].weight.detach(), torch.cat(directions, dim=1), rtol=0, atol=0)
    assert float(model.scalar.detach()) == 0.0 and float(model.linear_layers[0].bias.detach().abs().sum()) == 0.0


def test_local_grad_selector(setup):
    model, dist = setup
    _mask_scalar_and_bias(model)
    dist.merge_and_block_gradients()
    assert dist.local_grad_selector == (False, True, True, False)


def test_local_blocked_params(setup):
    _, dist = setup
    expected = (torch.zeros((1,)), torch.zeros(D, D), torch.zeros(D, D), torch.zeros(D))
    assert [tuple(p.shape) for p in dist.local_blocked_params] == [tuple(e.shape) for e in expected]
    torch.testing.assert_close(tuple(p.cpu() for p in dist.local_blocked_params), expected)


def test_local_block_info_list(setup):
    model, dist = setup
    w, b = model.linear_layers[0].weight, model.linear_layers[0].bias
    expected = ((model.scalar, (0, "block_0")), (w, (1, "block_0")), (w, (1, "block_1")), (b, (2, "block_0")))
    assert len(dist.local_block_info_list) == len(expected)
    for info, (param, ids) in zip(dist.local_block_info_list, expected):
        assert info.param is param
        assert info.composable_block_ids == ids


def test_merge_and_block_gradients(setup):
    model, dist = setup
    model.scalar.grad = torch.ones_like(model.scalar)
    w = model.linear_layers[0].weight
    w.grad = torch.arange(w.numel(), dtype=torch.float, device=DEV).reshape(w.shape)
    model.linear_layers[0].bias.grad = None
    got = dist.merge_and_block_gradients()
    want = (torch.ones((1,), device=DEV),) + torch.split(w.grad, D, dim=1)
    assert len(got) == 3
    for g, e in zip(got, want):
        torch.testing.assert_close(g, e, rtol=0, atol=0)
    # views, not copies
    assert got[1].data_ptr() == w.grad.data_ptr() and got[2].data_ptr() == w.grad.data_ptr() + 4 * D


@pytest.mark.parametrize("enabled, calls", ((True, 2), (False, 0)))
def test_eager_nan_check(enabled, calls):
    import optimizers_amd as oa

    model = _Model((2 * D, D), bias=True).to(DEV)
    dist = _distributor(model, runtime_config=oa.ShampooRuntimeConfig(eager_nan_check=enabled))
    model.scalar.grad = torch.tensor(1.0, device=DEV)
    w = model.linear_layers[0].weight
    w.grad = torch.ones_like(w)
    model.linear_layers[0].bias.grad = None
    with mock.patch.object(torch, "isfinite") as isfinite:
        dist.merge_and_block_gradients()
    assert isfinite.call_count == calls


def test_empty_parameter():
    """DistributorOnEmptyParamTest: a (0 x 5) weight keeps a block of shape (0,) that every update masks out."""
    model = _Model((D, 0), bias=False).to(DEV)
    dist = _distributor(model)
    model.scalar.grad = torch.ones_like(model.scalar)
    w = model.linear_layers[0].weight
    assert w.numel() == 0
    w.grad = torch.ones_like(w)
    grads = dist.merge_and_block_gradients()
    assert [tuple(g.shape) for g in grads] == [(1,)]
    assert dist.local_grad_selector == (True, False)
    assert [tuple(p.shape) for p in dist.local_blocked_params] == [(1,), (0,)]
    assert [i.composable_block_ids for i in dist.local_block_info_list] == [(0, "block_0"), (1, "block_0")]
    dist.update_params(blocked_search_directions=(torch.ones((1,), device=DEV),))
    torch.testing.assert_close(dist.local_masked_blocked_params, (torch.ones((1,), device=DEV),), rtol=0, atol=0)
    # all blocks, masked or not
    dist.update_params((torch.ones((1,), device=DEV), torch.zeros((0,), device=DEV)), use_masked_tensors=False)
    assert float(model.scalar.detach()) == 2.0


def test_update_params_rejects_a_wrong_count(setup):
    model, dist = setup
    _mask_scalar_and_bias(model)
    dist.merge_and_block_gradients()
    with pytest.raises(AssertionError, match="to be equal to"):
        dist.update_params(blocked_search_directions=(torch.zeros(D, D, device=DEV),))


def test_strided_update_on_ragged_and_order_three_blocks():
    """More blocks than one launch carries (24), column splits (row stride != width), widths that are not a
    multiple of 4, a convolution weight left as order-3 blocks, and transposed (non-dense) directions."""
    import optimizers_amd as oa
    from optimizers_amd.distributor import Distributor

    torch.manual_seed(3)
    params = [
        nn.Parameter(torch.randn(70, 45, device=DEV)),      # 5 x 3 blocks of at most 16 x 16, ragged tails 6 and 13
        nn.Parameter(torch.randn(33, device=DEV)),
        nn.Parameter(torch.randn(()).to(DEV)),
        nn.Parameter(torch.randn(20, 18, 3, 3, device=DEV)),  # merges to (20, 18, 9): order-3 blocks
        nn.Parameter(torch.randn(64, 64, device=DEV)),      # aligned: the 16-byte path
    ]
    opt = oa.DistributedShampoo(params, max_preconditioner_dim=16)
    dist = Distributor(param_group=opt.param_groups[0])
    blocks = dist.local_blocked_params
    assert len(blocks) > 24 and sum(b.dim() == 3 for b in blocks) == 4
    before = [p.detach().clone() for p in params]
    directions = []
    for i, b in enumerate(blocks):
        d = torch.randn(b.shape, device=DEV)
        if b.dim() == 2 and i % 2:
            d = torch.randn(b.shape[::-1], device=DEV).t()  # column-major direction
        directions.append(d)
    expected_blocks = [b.clone() + d for b, d in zip(blocks, directions)]
    dist.update_params(tuple(directions), use_masked_tensors=False)
    torch.cuda.synchronize()
    for b, e in zip(blocks, expected_blocks):
        torch.testing.assert_close(b, e, rtol=0, atol=0)
    # every element of every parameter moved exactly once
    for p, old in zip(params, before):
        assert bool((p.detach() != old).all())
