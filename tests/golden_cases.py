"""Helpers shared by the golden tests: rebuild a fixture case for the oracle or the
native optimizer from the plain-data description in tests/golden/cases.json."""

from __future__ import annotations

import json
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
    )


def rel_err(a, b) -> float:
    a = torch.as_tensor(a, dtype=torch.float64)
    b = torch.as_tensor(b, dtype=torch.float64)
    return float((a - b).norm() / b.norm().clamp_min(1e-300))
