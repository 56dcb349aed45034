"""Writes the golden fixtures under tests/golden/ from the REAL reference.

Run once, in the build container only (the reference checkout does not travel):

    python tests/golden/make_fixtures.py [/root/reference] [--only name,name,...]

(`--only` rewrites just the named multi-step cases / groups and leaves the other files alone.)

It imports `distributed_shampoo` from the reference checkout, runs it on CPU in
fp32 on tiny seeded cases and stores inputs/outputs as .npz (data only, no
pickles).  It is used only for what nothing else pins: the multi-step
composition of `DistributedShampoo.step()`, the coupled-Newton trajectory
(iteration counts, behaviour on rank-deficient input) and the QR-refresh column
ordering.  Every case is described by plain hyper-parameters so that
tests/test_oracle_golden.py can rebuild it for the oracle without the reference.
"""

from __future__ import annotations

import json
import os
import sys
from fractions import Fraction
from unittest import mock

import numpy as np
import torch

_args = [a for a in sys.argv[1:]]
ONLY = None
if "--only" in _args:
    k = _args.index("--only")
    ONLY = set(_args[k + 1].split(","))
    del _args[k : k + 2]
REF = _args[0] if _args else "/root/reference"
sys.path.insert(0, REF)

from distributed_shampoo import (  # noqa: E402
    AdaGradPreconditionerConfig,
    AdamPreconditionerConfig,
    CoupledHigherOrderConfig,
    CoupledNewtonConfig,
    DefaultSOAPConfig,
    DistributedShampoo,
    EigenConfig,
    EigendecomposedKLShampooPreconditionerConfig,
    EigendecomposedShampooPreconditionerConfig,
    EigenvalueCorrectedShampooPreconditionerConfig,
    EighEigendecompositionConfig,
    QREigendecompositionConfig,
    RootInvKLShampooPreconditionerConfig,
    RootInvShampooPreconditionerConfig,
    WeightDecayType,
)
from distributed_shampoo.preconditioner.matrix_functions import (  # noqa: E402
    matrix_eigendecomposition,
    matrix_inverse_root,
)
from distributed_shampoo.shampoo_types import (  # noqa: E402
    ClassicMomentumConfig,
    GeneralizedPrimalAveragingConfig,
    ScheduleFreeConfig,
)

OUT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(OUT)))
from tests.golden_cases import basis_signature, horizon_grads, oracle_config  # noqa: E402  (shared with the tests)


def case_params(shapes, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(*s, generator=g) for s in shapes]


def case_grads(shapes, seed, step, scale):
    g = torch.Generator().manual_seed(seed * 1000 + step)
    return [scale * torch.randn(*s, generator=g) for s in shapes]


# Plain-data descriptions; tests rebuild the oracle from the same dicts.
CASES = {
    "ragged_newton": dict(
        shapes=[[48, 40], [40]], seed=1, grad_scale=1.0, steps=12,
        lr=1e-2, betas=[0.9, 0.999], epsilon=1e-12, weight_decay=1e-2, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=32, precondition_frequency=2, start_preconditioning_step=6,
        preconditioner="newton", override_1d=True, grafting="adam", grafting_beta2=0.999, grafting_epsilon=1e-8,
    ),
    "ragged_newton_1d": dict(  # 1-D blocks preconditioned, large epsilon keeps rank-1 factors well posed
        shapes=[[20, 12], [12]], seed=2, grad_scale=1.0, steps=6,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-2, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=8, precondition_frequency=1, start_preconditioning_step=2,
        preconditioner="newton", override_1d=False, grafting="adam", grafting_beta2=0.99, grafting_epsilon=1e-8,
    ),
    "momentum_l2_beta3": dict(
        shapes=[[24, 36]], seed=3, grad_scale=0.1, steps=8,
        lr=5e-3, betas=[0.8, 0.95], beta3=0.7, epsilon=1e-10, weight_decay=1e-3, weight_decay_type="L2",
        max_preconditioner_dim=16, precondition_frequency=1, start_preconditioning_step=4,
        preconditioner="newton", override_1d=True, grafting="adagrad", grafting_epsilon=1e-8,
        momentum=0.5, dampening=0.1, use_nesterov=True,
    ),
    "dense_state_newton": dict(  # use_symmetric_packing=False: the state holds d x d factor matrices and inverse roots
        shapes=[[48, 40], [40]], seed=21, grad_scale=1.0, steps=10,
        lr=1e-2, betas=[0.9, 0.999], epsilon=1e-10, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=32, precondition_frequency=2, start_preconditioning_step=4,
        preconditioner="newton", override_1d=True, grafting="adam", grafting_beta2=0.999, grafting_epsilon=1e-8,
        use_symmetric_packing=False,
    ),
    "eigh_rootinv": dict(
        shapes=[[24, 20], [20]], seed=4, grad_scale=1.0, steps=6,
        lr=1e-2, betas=[0.9, 1.0], epsilon=1e-12, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=3, start_preconditioning_step=3,
        preconditioner="eigh", override_1d=False, grafting="adam", grafting_beta2=0.999, grafting_epsilon=1e-8,
    ),
    "soap_qr": dict(
        shapes=[[24, 20], [20]], seed=5, grad_scale=1.0, steps=9,
        lr=1e-2, betas=[0.9, 0.999], epsilon=1e-12, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=3, start_preconditioning_step=3,
        preconditioner="soap_qr", override_1d=False, grafting=None,
    ),
    "trace_scaled_newton": dict(  # use_trace_scaling without grafting: the scale of the inverse roots matters
        shapes=[[24, 20], [20]], seed=6, grad_scale=1.0, steps=8,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-6, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=2, start_preconditioning_step=4,
        preconditioner="newton", override_1d=True, grafting=None,
        use_trace_scaling=True, trace_scaling_exponent=0.5,
    ),
    "trace_scaled_eigh": dict(
        shapes=[[24, 20], [20]], seed=7, grad_scale=0.5, steps=8,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-4, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=2, start_preconditioning_step=4,
        preconditioner="eigh", override_1d=False, grafting="adagrad", grafting_epsilon=1e-8,
        use_trace_scaling=True, trace_scaling_exponent=1.0,
    ),
    "higher_order": dict(  # CoupledHigherOrderConfig, default order 3
        shapes=[[24, 20], [20]], seed=8, grad_scale=1.0, steps=8,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-12, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=2, start_preconditioning_step=4,
        preconditioner="higher_order", override_1d=True, grafting="adam", grafting_beta2=0.99, grafting_epsilon=1e-8,
        ho_order=3, ho_rel_epsilon=1e-6, ho_abs_epsilon=1e-10,
    ),
    "higher_order_o5": dict(  # order 5, 1-D blocks preconditioned too, no grafting
        shapes=[[20, 12], [12]], seed=9, grad_scale=1.0, steps=6,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-12, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=8, precondition_frequency=1, start_preconditioning_step=3,
        preconditioner="higher_order", override_1d=False, grafting=None,
        ho_order=5, ho_rel_epsilon=1e-3, ho_abs_epsilon=0.0,
    ),
    "conv_like_eigh": dict(  # order-3 blocks (conv weights): splits along dim 0, the middle dim and the last dim
        shapes=[[20, 6, 3, 3], [6, 20, 3, 3], [5, 4, 20], [7]], seed=10, grad_scale=1.0, steps=8,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-8, weight_decay=1e-3, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=2, start_preconditioning_step=4,
        preconditioner="eigh", override_1d=True, grafting="adam", grafting_beta2=0.99, grafting_epsilon=1e-8,
    ),
    "conv_like_newton": dict(  # the same with the coupled Newton iteration (root 6) and no filtered gradient
        shapes=[[20, 6, 3, 3], [6, 20, 3, 3], [5, 4, 20], [7]], seed=11, grad_scale=1.0, steps=8,
        lr=1e-2, betas=[0.0, 0.99], epsilon=1e-6, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=2, start_preconditioning_step=4,
        preconditioner="newton", override_1d=True, grafting="adagrad", grafting_epsilon=1e-8,
    ),
    "conv_like_soap_qr": dict(  # eigenvalue-corrected Shampoo on order-3 blocks, QR refresh, no grafting
        shapes=[[20, 6, 3, 3], [6, 20, 3, 3], [5, 4, 20], [7]], seed=12, grad_scale=1.0, steps=9,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-10, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=3, start_preconditioning_step=3,
        preconditioner="soap_qr", override_1d=False, grafting=None,
    ),
    "conv_like_soap_eigh": dict(  # the same with the eigh refresh, Adam grafting and no filtered gradient
        shapes=[[20, 6, 3, 3], [6, 20, 3, 3], [5, 4, 20]], seed=13, grad_scale=1.0, steps=8,
        lr=1e-2, betas=[0.0, 0.99], epsilon=1e-10, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=2, start_preconditioning_step=2,
        preconditioner="soap_eigh", override_1d=False, grafting="adam", grafting_beta2=0.99, grafting_epsilon=1e-8,
    ),
    # EigendecomposedShampooPreconditionerConfig, default eigh, 1-D blocks preconditioned too (their rank-deficient
    # factors are well posed only with an epsilon above the fp32 resolution of the spectrum)
    "eigendecomposed_eigh": dict(
        shapes=[[24, 20], [20]], seed=14, grad_scale=1.0, steps=8,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-4, weight_decay=1e-3, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=2, start_preconditioning_step=4,
        preconditioner="eigendecomposed_eigh", override_1d=False, grafting="adam", grafting_beta2=0.99, grafting_epsilon=1e-8,
    ),
    # the same family with the QR algorithm started from the stored eigenvectors; the first refresh comes when the
    # order-16 factor of the 16 x 4 block has seen five gradients (rank 20), so no null space makes the basis arbitrary
    "eigendecomposed_qr": dict(
        shapes=[[24, 20], [20]], seed=15, grad_scale=1.0, steps=10,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-6, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=1, start_preconditioning_step=5,
        preconditioner="eigendecomposed_qr", override_1d=True, grafting="adagrad", grafting_epsilon=1e-8,
    ),
    "kl_rootinv_eigh": dict(  # RootInvKLShampooPreconditionerConfig, default eigh root inverse
        shapes=[[24, 20], [20]], seed=16, grad_scale=1.0, steps=8,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-6, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=1, start_preconditioning_step=5,
        preconditioner="eigh", kl=True, override_1d=True, grafting="adam", grafting_beta2=0.99, grafting_epsilon=1e-8,
    ),
    "kl_rootinv_newton": dict(  # the same with the coupled Newton iteration, amortized every second step
        shapes=[[24, 20], [20]], seed=17, grad_scale=1.0, steps=9,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-6, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=2, start_preconditioning_step=5,
        preconditioner="newton", kl=True, override_1d=True, grafting="adagrad", grafting_epsilon=1e-8,
    ),
    "kl_eigendecomposed_eigh": dict(  # EigendecomposedKLShampooPreconditionerConfig
        shapes=[[24, 20], [20]], seed=18, grad_scale=1.0, steps=8,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-6, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=1, start_preconditioning_step=5,
        preconditioner="eigendecomposed_eigh", kl=True, override_1d=True, grafting="adam", grafting_beta2=0.99,
        grafting_epsilon=1e-8,
    ),
    # factor_matrix_dtype=float64: factors averaged and inverted in double, inverse roots stored in fp32; epsilon small
    # enough that fp32 factors would not resolve it; the first root inverse comes when every factor has full rank (the
    # Gram matrices are fp32 products, so a rank-deficient factor is indefinite at the 1e-7 level and its root inverse
    # is decided by rounding noise)
    "f64_factors_eigh": dict(
        shapes=[[24, 20], [20]], seed=19, grad_scale=1.0, steps=8,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-10, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=2, start_preconditioning_step=6,
        preconditioner="eigh", factor_matrix_dtype="float64", override_1d=True, grafting="adam", grafting_beta2=0.99,
        grafting_epsilon=1e-8,
    ),
    # float64 factors whose small eigenvalues only double precision resolves: gradient columns graded over three decades
    # (R = G^T G has eigenvalues over six decades, epsilon = 1e-14), eigendecomposition root inverse
    "f64_graded_eigh": dict(
        shapes=[[24, 20]], seed=23, grad_kind="graded", grade_decades=3, grad_scale=1.0, steps=8,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-14, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=32, precondition_frequency=2, start_preconditioning_step=4,
        preconditioner="eigh", factor_matrix_dtype="float64", override_1d=True, grafting="adam", grafting_beta2=0.99,
        grafting_epsilon=1e-8,
    ),
    # float64 factor matrices under the lists that keep eigenvectors (stored in fp32 by the reference too): the factor is
    # averaged in double, decomposed in double and the basis cast to fp32 (shampoo_preconditioner_list.py:1160-1166)
    "f64_soap_qr": dict(
        shapes=[[24, 20], [20]], seed=24, grad_scale=1.0, steps=9,
        lr=1e-2, betas=[0.9, 0.999], epsilon=1e-12, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=3, start_preconditioning_step=3,
        preconditioner="soap_qr", factor_matrix_dtype="float64", override_1d=False, grafting=None,
    ),
    "f64_eigendecomposed_eigh": dict(
        shapes=[[24, 20], [20]], seed=25, grad_scale=1.0, steps=8,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-4, weight_decay=1e-3, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=2, start_preconditioning_step=4,
        preconditioner="eigendecomposed_eigh", factor_matrix_dtype="float64", override_1d=False, grafting="adam",
        grafting_beta2=0.99, grafting_epsilon=1e-8,
    ),
    "f64_factors_newton": dict(
        shapes=[[24, 20], [20]], seed=20, grad_scale=1.0, steps=8,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-10, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=2, start_preconditioning_step=4,
        preconditioner="newton", factor_matrix_dtype="float64", override_1d=True, grafting="adagrad", grafting_epsilon=1e-8,
    ),
    # iterate averaging: generalized primal averaging, with a round trip through eval() / train() after step 7; the first
    # root inverse comes when the order-16 factor of the 16 x 4 block has seen six gradients (rank 24)
    "gpa_newton": dict(
        shapes=[[24, 20], [20]], seed=21, grad_scale=1.0, steps=9,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-6, weight_decay=1e-3, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=2, start_preconditioning_step=6,
        preconditioner="newton", override_1d=True, grafting="adam", grafting_beta2=0.99, grafting_epsilon=1e-8,
        averaging="gpa", eval_interp_coeff=0.9, train_interp_coeff=0.8, toggle_eval_at=7,
    ),
    # Schedule-Free with a learning rate that changes every step (mu_x follows lr^2 / sum of lr^2)
    "schedule_free_eigh": dict(
        shapes=[[24, 20], [20]], seed=22, grad_scale=1.0, steps=9,
        lr=1e-2, betas=[0.9, 0.99], epsilon=1e-6, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=16, precondition_frequency=2, start_preconditioning_step=6,
        preconditioner="eigh", override_1d=True, grafting="adagrad", grafting_epsilon=1e-8,
        averaging="schedule_free", train_interp_coeff=0.7, eval_coeff_lr_power=2, toggle_eval_at=7,
        lr_schedule=[1e-2, 2e-2, 3e-2, 3e-2, 2.5e-2, 2e-2, 1e-2, 5e-3, 2e-3],
    ),
    # ---- mid-size cases that run the benchmark configurations' horizons and cadences (zero initial parameters, so the
    # final parameters ARE the accumulated update; per-step subsamples of the parameters are stored with stride
    # trace_stride, and the same run of the oracle in float64 is stored beside the reference's fp32 run) ----
    # configuration 2: a 1105 x 768 slice of the embedding with blocks <= 1024 gives the ragged 81 x 768 tail block
    # (its order-768 factor has full rank once it has seen ten gradients), plus one LayerNorm vector; 20 steps
    "horizon_gpt2_slice": dict(
        shapes=[[1105, 768], [768]], seed=31, grad_kind="gauss", grad_scale=0.02, steps=20, zero_init=True,
        trace_stride=997, lr=1e-3, betas=[0.9, 0.999], epsilon=1e-12, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=1024, precondition_frequency=1, start_preconditioning_step=11,
        preconditioner="newton", override_1d=True, grafting="adam", grafting_beta2=0.999, grafting_epsilon=1e-8,
    ),
    # configuration 3: 512 x 1024 in blocks of 512 plus a vector, gradients N(0, 1e-4), Newton every step; 20 steps
    "horizon_llama_slice": dict(
        shapes=[[512, 1024], [1024]], seed=32, grad_kind="gauss", grad_scale=1e-2, steps=20, zero_init=True,
        trace_stride=997, lr=1e-3, betas=[0.9, 0.999], epsilon=1e-12, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=512, precondition_frequency=1, start_preconditioning_step=2,
        preconditioner="newton", override_1d=True, grafting="adam", grafting_beta2=0.999, grafting_epsilon=1e-8,
    ),
    # configuration 4: eigenvalue-corrected Shampoo (DefaultSOAPConfig), 256-blocks, a fixed rank-32 component above the
    # noise bulk, QR refresh every 10 steps; 50 steps
    "horizon_soap": dict(
        shapes=[[512, 768]], seed=33, grad_kind="gauss_lowrank", grad_scale=1e-2, lowrank_rank=32, lowrank_scale=1e-3,
        steps=50, zero_init=True, trace_stride=997, lr=1e-3, betas=[0.9, 0.999], epsilon=1e-12, weight_decay=0.0,
        weight_decay_type="DECOUPLED", max_preconditioner_dim=256, precondition_frequency=10,
        start_preconditioning_step=10, preconditioner="soap_qr", override_1d=False, grafting=None, basis_signature=3,
    ),
    # configuration 4 at its real block order: one 1024 x 768 block (factors of order 1024 and 768), same gradients'
    # recipe and cadence; 30 steps, three refreshes
    "horizon_soap_1024": dict(
        shapes=[[1024, 768]], seed=35, grad_kind="gauss_lowrank", grad_scale=1e-2, lowrank_rank=32, lowrank_scale=1e-3,
        steps=30, zero_init=True, trace_stride=997, lr=1e-3, betas=[0.9, 0.999], epsilon=1e-12, weight_decay=0.0,
        weight_decay_type="DECOUPLED", max_preconditioner_dim=1024, precondition_frequency=10,
        start_preconditioning_step=10, preconditioner="soap_qr", override_1d=False, grafting=None, basis_signature=3,
    ),
    # configuration 5: 512-blocks, G = U diag(s) V^T with s log-uniform in [1e-6, 1], eigendecomposition root inverse
    # every 50 steps (EigenConfig); 100 steps
    "horizon_eigh": dict(
        shapes=[[512, 512], [1024, 512]], seed=34, grad_kind="spectrum", spectrum=[1e-6, 1.0], grad_scale=1.0, steps=100,
        zero_init=True, trace_stride=997, lr=1e-3, betas=[0.9, 0.999], epsilon=1e-12, weight_decay=0.0,
        weight_decay_type="DECOUPLED", max_preconditioner_dim=512, precondition_frequency=50,
        start_preconditioning_step=50, preconditioner="eigh", override_1d=True, grafting="adam", grafting_beta2=0.999,
        grafting_epsilon=1e-8,
    ),
    "cfg1_override": dict(  # benchmark configuration 1 with 1-D blocks left to grafting
        shapes=[[512, 512], [512]], seed=0, grad_scale=1.0, steps=10, zero_init=True, torch_seed_grads=True,
        lr=1e-3, betas=[0.9, 0.999], epsilon=1e-12, weight_decay=0.0, weight_decay_type="DECOUPLED",
        max_preconditioner_dim=512, precondition_frequency=1, start_preconditioning_step=1,
        preconditioner="newton", override_1d=True, grafting="adam", grafting_beta2=0.999, grafting_epsilon=1e-8,
    ),
}


def build_reference(c, params):
    trace = dict(
        use_trace_scaling=c.get("use_trace_scaling", False), trace_scaling_exponent=c.get("trace_scaling_exponent", 0.5)
    )
    if c.get("factor_matrix_dtype") == "float64":
        trace["factor_matrix_dtype"] = torch.float64
    if c.get("use_symmetric_packing") is False:
        trace["use_symmetric_packing"] = False
    RootInv = RootInvKLShampooPreconditionerConfig if c.get("kl") else RootInvShampooPreconditionerConfig
    Eigendecomposed = EigendecomposedKLShampooPreconditionerConfig if c.get("kl") else EigendecomposedShampooPreconditionerConfig
    if c["preconditioner"] == "newton":
        pc = RootInv(
            amortized_computation_config=CoupledNewtonConfig(),
            inverse_exponent_override={1: {0: 0.0}} if c["override_1d"] else {}, **trace,
        )
    elif c["preconditioner"] == "higher_order":
        pc = RootInv(
            amortized_computation_config=CoupledHigherOrderConfig(
                rel_epsilon=c["ho_rel_epsilon"], abs_epsilon=c["ho_abs_epsilon"], order=c["ho_order"]
            ),
            inverse_exponent_override={1: {0: 0.0}} if c["override_1d"] else {}, **trace,
        )
    elif c["preconditioner"] == "eigh":
        pc = RootInv(
            amortized_computation_config=EigenConfig(),
            inverse_exponent_override={1: {0: 0.0}} if c["override_1d"] else {}, **trace,
        )
    elif c["preconditioner"] == "soap_qr":
        pc = EigenvalueCorrectedShampooPreconditionerConfig(
            amortized_computation_config=QREigendecompositionConfig(),
            **({"factor_matrix_dtype": torch.float64} if c.get("factor_matrix_dtype") == "float64" else {}),
        )
        assert c.get("factor_matrix_dtype") == "float64" or pc == DefaultSOAPConfig
    elif c["preconditioner"] == "soap_eigh":
        pc = EigenvalueCorrectedShampooPreconditionerConfig()
    elif c["preconditioner"] in ("eigendecomposed_eigh", "eigendecomposed_qr"):
        pc = Eigendecomposed(
            amortized_computation_config=(
                QREigendecompositionConfig() if c["preconditioner"].endswith("qr") else EighEigendecompositionConfig()
            ),
            inverse_exponent_override={1: {0: 0.0}} if c["override_1d"] else {},
            **({"factor_matrix_dtype": torch.float64} if c.get("factor_matrix_dtype") == "float64" else {}),
        )
    else:
        raise ValueError(c["preconditioner"])
    graft = {
        None: None,
        "adam": AdamPreconditionerConfig(beta2=c.get("grafting_beta2", 0.999), epsilon=c.get("grafting_epsilon", 1e-10)),
        "adagrad": AdaGradPreconditionerConfig(epsilon=c.get("grafting_epsilon", 1e-10)),
    }[c["grafting"]]
    mom = (
        ClassicMomentumConfig(momentum=c["momentum"], dampening=c["dampening"], use_nesterov=c["use_nesterov"])
        if c.get("momentum", 0.0) != 0.0
        else None
    )
    if c.get("averaging") == "gpa":
        mom = GeneralizedPrimalAveragingConfig(
            eval_interp_coeff=c["eval_interp_coeff"], train_interp_coeff=c["train_interp_coeff"]
        )
    elif c.get("averaging") == "schedule_free":
        mom = ScheduleFreeConfig(train_interp_coeff=c["train_interp_coeff"], eval_coeff_lr_power=c["eval_coeff_lr_power"])
    return DistributedShampoo(
        params, lr=c["lr"], betas=tuple(c["betas"]), beta3=c.get("beta3", -1.0), epsilon=c["epsilon"],
        weight_decay=c["weight_decay"], weight_decay_type=WeightDecayType[c["weight_decay_type"]],
        max_preconditioner_dim=c["max_preconditioner_dim"], precondition_frequency=c["precondition_frequency"],
        start_preconditioning_step=c["start_preconditioning_step"], preconditioner_config=pc, grafting_config=graft,
        iterate_averaging_config=mom,
    )


def run_case(name, c):
    shapes = [tuple(s) for s in c["shapes"]]
    if c.get("zero_init"):
        init = [torch.zeros(*s) for s in shapes]
    else:
        init = case_params(shapes, c["seed"])
    params = [torch.nn.Parameter(t.clone()) for t in init]
    opt = build_reference(c, params)
    out = {}
    dist_calls = []
    real_dist = torch.dist

    def counting_dist(*a, **k):
        dist_calls[-1] += 1
        return real_dist(*a, **k)

    real_mir = matrix_inverse_root

    def counting_mir(*a, **k):
        dist_calls.append(0)
        return real_mir(*a, **k)

    # the higher-order iteration evaluates torch.linalg.vector_norm once at the start, once per iteration and
    # once for the final residual
    real_vn = torch.linalg.vector_norm

    def counting_vn(*a, **k):
        if dist_calls:
            dist_calls[-1] += 1
        return real_vn(*a, **k)

    higher = c["preconditioner"] == "higher_order"
    iters_per_step = []
    if c.get("torch_seed_grads"):
        torch.manual_seed(c["seed"])
    with mock.patch.object(torch, "dist", counting_dist), mock.patch.object(
        torch.linalg, "vector_norm", counting_vn if higher else real_vn
    ), mock.patch(
        "distributed_shampoo.preconditioner.shampoo_preconditioner_list.matrix_inverse_root", counting_mir
    ):
        for s in range(1, c["steps"] + 1):
            if c.get("torch_seed_grads"):
                grads = [torch.randn_like(p) for p in params]
            elif "grad_kind" in c:
                grads = horizon_grads(c, s)
            else:
                grads = case_grads(shapes, c["seed"], s, c["grad_scale"])
            for p, g in zip(params, grads):
                p.grad = g
            dist_calls.clear()
            if "lr_schedule" in c:
                opt.param_groups[0]["lr"] = c["lr_schedule"][s - 1]
            opt.step()
            if c.get("toggle_eval_at") == s:
                # the evaluation sequence, then back to the training sequence
                opt.eval()
                for i, p in enumerate(params):
                    out[f"eval_p{i}"] = p.detach().reshape(-1).numpy().copy()
                opt.train()
            # torch.dist is called once before the loop and once per iteration
            iters_per_step.append([n - (2 if higher else 1) for n in dist_calls])
            for i, p in enumerate(params):
                out[f"norm_s{s}_p{i}"] = np.float64(p.detach().double().norm().item())
                if "trace_stride" in c:
                    out[f"trace_s{s}_p{i}"] = p.detach().reshape(-1)[:: c["trace_stride"]].numpy().copy()
            start, freq = c["start_preconditioning_step"], c["precondition_frequency"]
            if c.get("basis_signature") and (s == start or (s > start and s % freq == 0)):
                # The order in which THIS run's stable sort left the columns of every refreshed eigenbasis
                # (matrix_functions.py:848-850), as a few seeded projections per column: estimates that agree to
                # within their rounding error come out in either order from one correct fp32 evaluation to the next.
                for pi, p in enumerate(params):
                    for key, val in opt.state[p].items():
                        if isinstance(val, dict) and "shampoo" in val:
                            for k, q in enumerate(val["shampoo"].factor_matrices_eigenvectors):
                                out[f"sig_s{s}_p{pi}_{key}_{k}"] = basis_signature(q, c["basis_signature"]).numpy().copy()
            if "trace_stride" in c:
                print(f"  {name}: reference step {s} done", flush=True)
    big = max(p.numel() for p in params) > 100_000
    for i, p in enumerate(params):
        flat = p.detach().reshape(-1)
        out[f"final_p{i}"] = (flat[::37] if big else flat).numpy().copy()
    # optimizer state (only for the small cases)
    if not big:
        for pi, p in enumerate(params):
            st = opt.state[p]
            for key, val in st.items():
                if not isinstance(val, dict):
                    continue
                for sk, sv in val.items():
                    if isinstance(sv, torch.Tensor):
                        out[f"state_p{pi}_{key}_{sk}"] = sv.numpy().copy()
                    elif sk == "shampoo":
                        for fname in ("factor_matrices", "inv_factor_matrices", "factor_matrices_eigenvectors",
                                      "factor_matrices_eigenvalues"):
                            for k, t in enumerate(getattr(sv, fname, ())):
                                out[f"state_p{pi}_{key}_{fname}_{k}"] = t.numpy().copy()
                        if hasattr(sv, "corrected_eigenvalues"):
                            out[f"state_p{pi}_{key}_corrected_eigenvalues"] = sv.corrected_eigenvalues.numpy().copy()
    if "trace_stride" in c:
        # the same run in exact-ish arithmetic: the oracle (pinned to the reference by the other fixtures) on float64
        # parameters and gradients; |reference fp32 - this| is the reference algorithm's own rounding-noise floor
        from oracle.shampoo_oracle import ShampooOracle

        o64 = [t.clone().double() for t in init]
        oracle = ShampooOracle(o64, oracle_config(c))
        for s in range(1, c["steps"] + 1):
            oracle.step([g.double() for g in horizon_grads(c, s)])
            for i, p in enumerate(o64):
                out[f"o64_trace_s{s}_p{i}"] = p.reshape(-1)[:: c["trace_stride"]].float().numpy().copy()
        for i, p in enumerate(o64):
            out[f"o64_final_p{i}"] = p.reshape(-1)[::37].float().numpy().copy()
    maxlen = max((len(x) for x in iters_per_step), default=0)
    it = np.full((len(iters_per_step), max(maxlen, 1)), -1, dtype=np.int64)
    for r, row in enumerate(iters_per_step):
        it[r, : len(row)] = row
    out["newton_iterations"] = it
    np.savez_compressed(os.path.join(OUT, f"{name}.npz"), **out)
    print(name, "ok; iterations per amortized step:", [r for r in iters_per_step if r][:3])


def cfg1_as_stated():
    """benchmark configuration 1 verbatim: what does the reference do?"""
    torch.manual_seed(0)
    w = torch.nn.Parameter(torch.zeros(512, 512))
    b = torch.nn.Parameter(torch.zeros(512))
    opt = DistributedShampoo(
        [w, b], lr=1e-3, betas=(0.9, 0.999), epsilon=1e-12, max_preconditioner_dim=512,
        precondition_frequency=1, start_preconditioning_step=1,
        preconditioner_config=RootInvShampooPreconditionerConfig(amortized_computation_config=CoupledNewtonConfig()),
        grafting_config=AdamPreconditionerConfig(beta2=0.999, epsilon=1e-8),
    )
    rec = {"raised": False}
    for s in range(1, 11):
        w.grad = torch.randn_like(w)
        b.grad = torch.randn_like(b)
        try:
            opt.step()
        except Exception as e:  # noqa: BLE001
            rec = {"raised": True, "step": s, "type": type(e).__name__, "mro": [k.__name__ for k in type(e).__mro__],
                   "message_prefix": str(e)[:80]}
            break
    with open(os.path.join(OUT, "cfg1_as_stated.json"), "w") as f:
        json.dump(rec, f, indent=1)
    print("cfg1_as_stated", rec)


def newton_trajectories():
    """matrix_inverse_root (coupled Newton) on stored inputs: X, iteration count, finiteness."""
    g = torch.Generator().manual_seed(7)
    mats = {}
    a = torch.randn(64, 256, generator=g)
    mats["wellcond64_r4"] = (a @ a.T / 256, 4, 1e-12)
    a = torch.randn(48, 100, generator=g)
    mats["wellcond48_r2"] = (a @ a.T / 100, 2, 1e-12)
    a = torch.randn(128, 128, generator=g)
    mats["square128_r4"] = (a @ a.T, 4, 1e-12)
    a = torch.randn(96, 1, generator=g)
    mats["rank1_96_r2_bigeps"] = (a @ a.T, 2, 1e-1)
    a = torch.randn(32, 1, generator=g)
    mats["rank1_32_r2"] = (a @ a.T, 2, 1e-12)
    a = torch.randn(40, 24, generator=g)
    mats["rank24_40_r4"] = (a @ a.T, 4, 1e-12)
    mats["scaled_identity_r4"] = (3.0 * torch.eye(20), 4, 0.0)
    out = {}
    for name, (A, root, eps) in mats.items():
        calls = [0]
        real = torch.dist

        def cd(*aa, **kk):
            calls[0] += 1
            return real(*aa, **kk)

        with mock.patch.object(torch, "dist", cd):
            X = matrix_inverse_root(A, Fraction(root), CoupledNewtonConfig(), eps)
        out[f"{name}_A"] = A.numpy()
        out[f"{name}_X"] = X.numpy()
        out[f"{name}_meta"] = np.array([root, calls[0] - 1, int(torch.isfinite(X).all())], dtype=np.int64)
        out[f"{name}_eps"] = np.float64(eps)
        print("newton", name, "iters", calls[0] - 1, "finite", bool(torch.isfinite(X).all()))
    np.savez_compressed(os.path.join(OUT, "newton_trajectories.npz"), **out)


def eig_cases():
    """eigh root inverse and one QR refresh on stored inputs."""
    g = torch.Generator().manual_seed(11)
    out = {}
    a = torch.randn(40, 64, generator=g)
    A = a @ a.T / 64
    out["eigh_A"] = A.numpy()
    out["eigh_X_r4"] = matrix_inverse_root(A, Fraction(4), EigenConfig(), 1e-12).numpy()
    a = torch.randn(30, 10, generator=g)
    A2 = a @ a.T
    out["eigh_def_A"] = A2.numpy()
    out["eigh_def_X_r2_eps1e-3"] = matrix_inverse_root(A2, Fraction(2), EigenConfig(), 1e-3).numpy()
    # QR refresh from identity and from a previous basis, incl. sort permutation
    Q0 = torch.eye(40)
    l1, Q1 = matrix_eigendecomposition(A, 1e-12, QREigendecompositionConfig(), Q0)
    a = torch.randn(40, 64, generator=g)
    A3 = 0.9 * A + 0.1 * (a @ a.T / 64)
    l2, Q2 = matrix_eigendecomposition(A3, 1e-12, QREigendecompositionConfig(), Q1)
    l3, Q3 = matrix_eigendecomposition(A3, 1e-12, QREigendecompositionConfig(max_iterations=5, tolerance=0.05), Q2)
    for k, v in dict(qr_A=A, qr_A3=A3, qr_l1=l1, qr_Q1=Q1, qr_l2=l2, qr_Q2=Q2, qr_l3=l3, qr_Q3=Q3).items():
        out[k] = v.numpy()
    np.savez_compressed(os.path.join(OUT, "eig_cases.npz"), **out)
    print("eig cases ok")


def higher_order_trajectories():
    """matrix_inverse_root with CoupledHigherOrderConfig on stored inputs: X, iteration count, or the error raised."""
    g = torch.Generator().manual_seed(13)
    mats = {}
    a = torch.randn(64, 256, generator=g)
    well64 = a @ a.T / 256
    a = torch.randn(48, 100, generator=g)
    well48 = a @ a.T / 100
    a = torch.randn(40, 24, generator=g)
    rank24 = a @ a.T
    a = torch.randn(96, 96, generator=g)
    square96 = a @ a.T
    for order in (2, 3, 4, 6):
        mats[f"well64_r4_o{order}"] = (well64, 4, order, 0.0, 0.0, 100, 1e-8)
    mats["well48_r2_o3"] = (well48, 2, 3, 0.0, 0.0, 100, 1e-8)
    mats["well48_r3_o3"] = (well48, 3, 3, 0.0, 0.0, 100, 1e-8)
    mats["well48_r1_o4"] = (well48, 1, 4, 0.0, 0.0, 100, 1e-8)
    mats["well48_r8_o3_loose"] = (well48, 8, 3, 0.0, 0.0, 100, 1e-4)
    mats["square96_r4_o3_rel"] = (square96, 4, 3, 1e-5, 0.0, 100, 1e-8)
    mats["square96_r4_o3_maxit4"] = (square96, 4, 3, 1e-5, 0.0, 4, 1e-8)
    mats["rank24_r4_o3_abs"] = (rank24, 4, 3, 0.0, 1e-3, 100, 1e-8)
    mats["rank24_r4_o3_noeps"] = (rank24, 4, 3, 0.0, 0.0, 100, 1e-8)
    mats["rank24_r2_o5_rel"] = (rank24, 2, 5, 1e-6, 1e-12, 100, 1e-8)
    out = {}
    for name, (A, root, order, rel, ab, maxit, tol) in mats.items():
        calls = [0]
        real = torch.linalg.vector_norm

        def cv(*aa, **kk):
            calls[0] += 1
            return real(*aa, **kk)

        cfg = CoupledHigherOrderConfig(rel_epsilon=rel, abs_epsilon=ab, max_iterations=maxit, tolerance=tol, order=order)
        raised = ""
        X = torch.full_like(A, float("nan"))
        with mock.patch.object(torch.linalg, "vector_norm", cv):
            try:
                X = matrix_inverse_root(A, Fraction(root), cfg, 0.0)
            except ArithmeticError as e:
                raised = str(e)[:60]
        out[f"{name}_A"] = A.numpy()
        out[f"{name}_X"] = X.numpy()
        out[f"{name}_meta"] = np.array([root, order, maxit, calls[0] - 2, int(bool(raised))], dtype=np.int64)
        out[f"{name}_eps"] = np.array([rel, ab, tol], dtype=np.float64)
        print("higher order", name, "iters", calls[0] - 2, "raised", raised)
    np.savez_compressed(os.path.join(OUT, "higher_order_trajectories.npz"), **out)


def state_dict_resume():
    """A state_dict written by the reference in mid-run (7 steps of the ragged Newton case with momentum and weight
    decay), the parameters at that moment and the parameters after 5 more steps: what an optimizer that loads the
    checkpoint and goes on with the same gradients has to reproduce.  The nested dict is stored flat, one array per
    leaf, under keys "state/<param>/<block>/.../<leaf>" (the reference's own nesting, tests/distributed_shampoo_test.py:516-622)."""
    c = dict(CASES["ragged_newton"], momentum=0.5, dampening=0.0, use_nesterov=False)
    shapes = [tuple(s) for s in c["shapes"]]
    params = [torch.nn.Parameter(t.clone()) for t in case_params(shapes, c["seed"])]
    opt = build_reference(c, params)
    out = {}

    def flatten(prefix, node):
        if isinstance(node, dict):
            for k, v in node.items():
                flatten(f"{prefix}/{k}", v)
        elif isinstance(node, torch.Tensor):
            out[prefix] = node.detach().cpu().numpy().copy()
        else:
            raise TypeError(f"{prefix}: {type(node)}")

    for s in range(1, 13):
        for p, g in zip(params, case_grads(shapes, c["seed"], s, c["grad_scale"])):
            p.grad = g
        opt.step()
        if s == 7:
            flatten("state", opt.state_dict()["state"])
            for i, p in enumerate(params):
                out[f"params_at_save_p{i}"] = p.detach().numpy().copy()
    for i, p in enumerate(params):
        out[f"final_p{i}"] = p.detach().numpy().copy()
    np.savez_compressed(os.path.join(OUT, "state_dict_resume.npz"), **out)
    with open(os.path.join(OUT, "state_dict_resume.json"), "w") as f:
        json.dump({"case": c, "saved_after_step": 7, "steps": 12, "keys": sorted(k for k in out if k.startswith("state/"))}, f, indent=1)
    print("state_dict_resume ok:", len([k for k in out if k.startswith("state/")]), "state leaves")


if __name__ == "__main__":
    torch.set_num_threads(8)
    with open(os.path.join(OUT, "cases.json"), "w") as f:
        json.dump(CASES, f, indent=1)
    groups = {
        "newton_trajectories": newton_trajectories, "higher_order_trajectories": higher_order_trajectories,
        "eig_cases": eig_cases, "cfg1_as_stated": cfg1_as_stated, "state_dict_resume": state_dict_resume,
    }
    for gname, fn in groups.items():
        if ONLY is None or gname in ONLY:
            fn()
    for n, c in CASES.items():
        if ONLY is None or n in ONLY:
            run_case(n, c)
