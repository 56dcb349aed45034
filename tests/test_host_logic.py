"""CPU tests of the host side: C ABI exports, config validation, block partition."""

import math
import os
import re

import pytest
import torch

import optimizers_amd as oa
from optimizers_amd import native
from optimizers_amd.blocking import merge_small_dims, partition_parameter
from oracle import shampoo_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_loads_and_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "shampoo_amd.h")).read()
    declared = set(re.findall(r"\b(sa_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 20
    lib = native.load()
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in include/shampoo_amd.h but not exported"
    assert set(native.EXPORTS) <= declared
    assert lib.sa_abi_version() == 3


def test_struct_layouts_match_the_header():
    import ctypes

    # sa_block_desc: 2*int32, int64, 4 pointers, 3+3 pointers, 3*int32 (+4 pad), 3+1 pointers, int32 (+4 pad), int64,
    # 1 pointer -> 168 bytes on LP64
    assert ctypes.sizeof(native.BlockDesc) == 168
    assert native.BlockDesc.ld.offset == 8 and native.BlockDesc.factor.offset == 48
    assert native.BlockDesc.inv_factor.offset == 72 and native.BlockDesc.root.offset == 96
    assert native.BlockDesc.eigenvectors.offset == 112 and native.BlockDesc.corrected_eigenvalues.offset == 136
    assert native.BlockDesc.mid.offset == 144 and native.BlockDesc.ld_outer.offset == 152
    assert native.BlockDesc.weight_buffer.offset == 160
    assert ctypes.sizeof(native.StepScalars) == 64 and native.StepScalars.use_primal_averaging.offset == 52


def test_no_gpu_means_loud_failure_not_fallback():
    p = torch.nn.Parameter(torch.zeros(4, 4))
    with pytest.raises(RuntimeError, match="no CPU path"):
        oa.DistributedShampoo(
            [p], preconditioner_config=oa.RootInvShampooPreconditionerConfig(
                amortized_computation_config=oa.CoupledNewtonConfig()))


@pytest.mark.parametrize(
    "kwargs, message",
    [
        (dict(lr=-0.1), "Invalid param_group[LR]=-0.1. Must be >= 0.0."),
        (dict(betas=(-0.1, 1.0)), "Invalid param_group[BETAS][0]=-0.1. Must be in [0.0, 1.0)."),
        (dict(betas=(0.9, 1.1)), "Invalid param_group[BETAS][1]=1.1. Must be in [0.0, 1.0]."),
        (dict(beta3=1.0), "Invalid param_group[BETA3]=1.0. Must be in [0.0, 1.0)."),
        (dict(epsilon=0.0), "Invalid param_group[EPSILON]=0.0. Must be > 0.0."),
        (dict(weight_decay=-0.1), "Invalid param_group[WEIGHT_DECAY]=-0.1. Must be >= 0.0."),
        (dict(max_preconditioner_dim=3.14), "Must be an integer or math.inf."),
        (dict(max_preconditioner_dim=0), "Must be >= 1."),
        (dict(precondition_frequency=0), "Must be >= 1."),
        (dict(start_preconditioning_step=-2), "Must be >= -1."),
        (dict(start_preconditioning_step=5, precondition_frequency=10), "Must be >= param_group[PRECONDITION_FREQUENCY]=10."),
    ],
)
def test_constructor_validation_like_reference(kwargs, message):
    # conditions of distributed_shampoo.py:411-530; messages pinned by tests/distributed_shampoo_test.py:96-154
    p = torch.nn.Parameter(torch.zeros(4, 4))
    with pytest.raises(ValueError) as e:
        oa.DistributedShampoo([p], **kwargs)
    assert message in str(e.value)


def test_config_dataclass_validation():
    with pytest.raises(ValueError, match="Invalid epsilon value"):
        oa.AdaGradPreconditionerConfig(epsilon=0.0)
    with pytest.raises(ValueError, match="Invalid grafting beta2 parameter"):
        oa.AdamPreconditionerConfig(beta2=0.0)
    with pytest.raises(ValueError, match="Invalid tolerance value"):
        oa.EigenConfig(tolerance=0.5)
    with pytest.raises(ValueError, match="All orders must be >= 0"):
        oa.RootInvShampooPreconditionerConfig(inverse_exponent_override={-1: 0.5})
    with pytest.raises(ValueError, match="All dimensions must be within"):
        oa.RootInvShampooPreconditionerConfig(inverse_exponent_override={2: {2: 0.5}})
    with pytest.raises(ValueError, match="All overrides must be >= 0"):
        oa.RootInvShampooPreconditionerConfig(inverse_exponent_override={2: {0: -0.5}})
    with pytest.raises(ValueError, match="Must be within"):
        oa.ClassicMomentumConfig(momentum=1.0)
    with pytest.raises(TypeError):
        oa.PreconditionerConfig()  # abstract
    assert oa.DefaultSOAPConfig.amortized_computation_config == oa.QREigendecompositionConfig()
    assert oa.CoupledNewtonConfig().max_iterations == 100 and oa.CoupledNewtonConfig().tolerance == 1e-6
    assert oa.DefaultShampooConfig.amortized_computation_config == oa.EigenConfig()


@pytest.mark.parametrize(
    "shape, b",
    [((512, 512), 512), ((2304, 768), 1024), ((50257, 768), 1024), ((768,), 1024), ((4096, 14336), 2048),
     ((3, 5, 7), 4), ((1, 9, 1), 4), ((6, 1, 6), 36), ((0, 3), 8), ((), 8)],
)
def test_partition_equals_oracle_blocks(shape, b):
    t = torch.zeros(shape)
    want = O.blocks_of(t, b)
    got = partition_parameter(0, shape, b)
    assert merge_small_dims(tuple(shape), b, 1) == O.merge_small_dims(shape, b, 1)
    assert [s.shape for s in got] == [tuple(w.shape) for w in want]
    if t.numel():
        assert [s.offset for s in got] == [w.storage_offset() for w in want]
        assert [s.strides for s in got] == [tuple(w.stride()) for w in want]


def test_baseline_block_tables():
    """Block and factor counts of the five benchmark configurations."""
    gpt2 = sum(([(2304, 768), (768, 768), (3072, 768), (768, 3072), (768,), (768,)] for _ in range(12)), []) + [(50257, 768)]
    blocks = [s for i, sh in enumerate(gpt2) for s in partition_parameter(i, sh, 1024)]
    assert len(blocks) == 194
    from collections import Counter

    dims = Counter(d for s in blocks for d in s.shape)
    assert dims == Counter({81: 1, 256: 12, 768: 206, 1024: 145})
    llama = [(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096), (14336, 4096), (14336, 4096), (4096, 14336), (4096,), (4096,)]
    blocks = [s for i, sh in enumerate(llama) for s in partition_parameter(i, sh, 2048)]
    assert len(blocks) == 58
    assert Counter(s.shape for s in blocks) == Counter({(2048, 2048): 50, (1024, 2048): 4, (2048,): 4})
    assert sum(math.prod(s.shape) for s in blocks) == 218_112_000
