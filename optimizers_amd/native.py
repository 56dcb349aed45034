"""ctypes binding of libshampoo_amd.so (C ABI declared in include/shampoo_amd.h).

There is no CPU fallback: if the library is missing or a call fails, an exception is raised.
torch must be imported before the library is loaded so that both share one HIP runtime.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_double, c_float, c_int32, c_int64, c_void_p

import torch  # noqa: F401  (loads the HIP runtime the library binds to)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libshampoo_amd.so")

SA_OK = 0
SA_FACTOR_OK = 0
SA_FACTOR_INPUT_NONFINITE = 1
SA_FACTOR_RESULT_NONFINITE = 2
SA_FACTOR_NOT_CONVERGED = 3
SA_FACTOR_SKIPPED = 4
SA_FACTOR_SOLVER_FAILED = 5
SA_GRAFT_NONE = 0
SA_GRAFT_SGD = 1
SA_GRAFT_ADAGRAD = 2

EXPORTS = (
    "sa_last_error", "sa_abi_version", "sa_plan_create", "sa_plan_destroy", "sa_plan_workspace_bytes",
    "sa_plan_bind_workspace", "sa_plan_num_factors", "sa_plan_invalidate_inverse_cache", "sa_plan_set_newton_split_tiles", "sa_plan_set_tridiagonal_lanes",
    "sa_plan_bind_gradients", "sa_add_l2_regularization", "sa_update_factor_matrices",
    "sa_compute_root_inverses_newton", "sa_compute_root_inverses_eigh", "sa_refresh_eigenbases_qr", "sa_refresh_eigenbases_eigh", "sa_update_corrected_eigenvalues",
    "sa_precondition_eigenvalue_corrected", "sa_update_and_precondition_eigenvalue_corrected", "sa_plan_shared_rotation_steps", "sa_update_grafting_and_filtered_grad", "sa_precondition",
    "sa_apply_update", "sa_grafting_only_step", "sa_plan_read_norms", "sa_plan_read_preconditioned",
    "sa_gemm_f32", "sa_gemm_f32_static", "sa_copy_f32", "sa_set_profiling", "sa_phase_ms", "sa_phase_flops", "sa_phase_launches", "sa_phase_executed_flops", "sa_set_symmetric_newton", "sa_set_eigh_solver",
    "sa_plan_set_trace_scaling", "sa_compute_root_inverses_higher_order", "sa_plan_read_eigenvalues", "sa_add_to_views",
    "sa_compute_root_inverses_from_eigendecomposition", "sa_plan_set_kl_shampoo",
    "sa_move_params_towards_weight_buffer", "sa_plan_set_factor_dtype", "sa_update_factor_matrices_f64", "sa_compute_root_inverses_newton_f64",
    "sa_plan_set_scratch_budget", "sa_plan_num_waves", "sa_plan_set_symmetric_newton", "sa_plan_set_eigh_solver",
    "sa_plan_rebind_params", "sa_compute_root_inverses_eigh_f64",
    "sa_plan_export_dense_state", "sa_plan_import_dense_state", "sa_set_small_launch_tiles",
)


SA_MAX_ORDER = 3


class BlockDesc(ctypes.Structure):
    _fields_ = [
        ("rows", c_int32),
        ("cols", c_int32),
        ("ld", c_int64),
        ("param", c_void_p),
        ("filtered_grad", c_void_p),
        ("adagrad", c_void_p),
        ("momentum_buffer", c_void_p),
        ("factor", c_void_p * SA_MAX_ORDER),
        ("inv_factor", c_void_p * SA_MAX_ORDER),
        ("root", c_int32 * SA_MAX_ORDER),
        ("eigenvectors", c_void_p * SA_MAX_ORDER),
        ("corrected_eigenvalues", c_void_p),
        ("mid", c_int32),
        ("ld_outer", c_int64),
        ("weight_buffer", c_void_p),
    ]


class StepScalars(ctypes.Structure):
    _fields_ = [
        ("lr", c_float),
        ("beta1", c_float),
        ("beta3", c_float),
        ("bias_correction1", c_float),
        ("graft_type", c_int32),
        ("graft_beta2", c_float),
        ("graft_weight", c_float),
        ("graft_bias_correction2", c_float),
        ("graft_epsilon", c_float),
        ("weight_decay_alpha", c_float),
        ("momentum", c_float),
        ("dampening", c_float),
        ("use_nesterov", c_int32),
        ("use_primal_averaging", c_int32),
        ("averaging_direction_coeff", c_float),
        ("averaging_buffer_coeff", c_float),
        ("lerp_weight1", c_float),
        ("lerp_weight3", c_float),
        ("filtered_grad_mode", c_int32),
    ]


class View(ctypes.Structure):
    """sa_view: a strided fp32 view of device memory (sizes and element strides, outermost dim first)."""

    _fields_ = [
        ("data", c_void_p),
        ("order", c_int32),
        ("size", c_int64 * SA_MAX_ORDER),
        ("stride", c_int64 * SA_MAX_ORDER),
    ]


def fill_view(view: View, t: torch.Tensor) -> None:
    view.data = t.data_ptr()
    view.order = t.dim()
    for k in range(t.dim()):
        view.size[k] = t.size(k)
        view.stride[k] = t.stride(k)


class NativeError(RuntimeError):
    """A call into libshampoo_amd.so failed."""


_lib = None


def load() -> ctypes.CDLL:
    """Loads the library once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise NativeError(
            f"{LIB_PATH} is missing: build it with `python optimizers_amd/csrc/build.py` "
            "(hipcc, gfx950). There is no CPU fallback."
        )
    lib = ctypes.CDLL(LIB_PATH)
    lib.sa_last_error.restype = c_char_p
    lib.sa_abi_version.restype = c_int32
    lib.sa_plan_create.argtypes = [POINTER(BlockDesc), c_int32, POINTER(c_void_p)]
    lib.sa_plan_destroy.argtypes = [c_void_p]
    lib.sa_plan_destroy.restype = None
    lib.sa_plan_workspace_bytes.argtypes = [c_void_p]
    lib.sa_plan_workspace_bytes.restype = c_int64
    lib.sa_plan_bind_workspace.argtypes = [c_void_p, c_void_p, c_int64]
    lib.sa_plan_num_factors.argtypes = [c_void_p]
    lib.sa_plan_invalidate_inverse_cache.argtypes = [c_void_p]
    lib.sa_plan_set_newton_split_tiles.argtypes = [c_void_p, c_int32]
    lib.sa_plan_set_tridiagonal_lanes.argtypes = [c_void_p, c_int32]
    lib.sa_plan_bind_gradients.argtypes = [c_void_p, POINTER(c_void_p), c_void_p]
    lib.sa_add_l2_regularization.argtypes = [c_void_p, c_float, c_void_p]
    lib.sa_update_factor_matrices.argtypes = [c_void_p, c_float, c_float, c_void_p]
    lib.sa_compute_root_inverses_newton.argtypes = [
        c_void_p, c_float, c_float, c_int32, c_float, POINTER(c_int32), POINTER(c_int32), c_void_p,
    ]
    lib.sa_compute_root_inverses_higher_order.argtypes = [
        c_void_p, c_float, c_float, c_float, c_int32, c_float, c_int32, POINTER(c_int32), POINTER(c_int32), c_void_p,
    ]
    lib.sa_compute_root_inverses_eigh.argtypes = [
        c_void_p, c_float, c_float, POINTER(c_float), c_int32, c_float, c_float, c_int32, POINTER(c_int32), POINTER(c_int32),
        c_void_p,
    ]
    lib.sa_refresh_eigenbases_qr.argtypes = [
        c_void_p, c_float, c_float, c_int32, c_float, POINTER(c_int32), POINTER(c_int32), c_void_p,
    ]
    lib.sa_refresh_eigenbases_eigh.argtypes = [
        c_void_p, c_float, c_float, c_float, c_int32, POINTER(c_int32), POINTER(c_int32), c_void_p,
    ]
    lib.sa_update_corrected_eigenvalues.argtypes = [c_void_p, c_float, c_float, c_void_p]
    lib.sa_precondition_eigenvalue_corrected.argtypes = [c_void_p, POINTER(StepScalars), c_float, c_float, c_float, c_void_p]
    lib.sa_plan_shared_rotation_steps.argtypes = [c_void_p]
    lib.sa_plan_shared_rotation_steps.restype = c_int64
    lib.sa_update_and_precondition_eigenvalue_corrected.argtypes = [
        c_void_p, POINTER(StepScalars), c_float, c_float, c_float, c_float, c_float, c_void_p]
    for name in ("sa_update_grafting_and_filtered_grad", "sa_precondition", "sa_apply_update", "sa_grafting_only_step"):
        getattr(lib, name).argtypes = [c_void_p, POINTER(StepScalars), c_void_p]
    lib.sa_plan_read_norms.argtypes = [c_void_p, POINTER(c_float), POINTER(c_float), c_void_p]
    lib.sa_plan_read_preconditioned.argtypes = [c_void_p, c_int32, c_void_p, c_void_p]
    lib.sa_gemm_f32.argtypes = [
        c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int64, c_int64, c_int64, c_int32, c_int32,
        c_int32, c_int64, c_int64, c_int64, c_void_p,
    ]
    lib.sa_gemm_f32_static.argtypes = lib.sa_gemm_f32.argtypes
    lib.sa_copy_f32.argtypes = [c_void_p, c_void_p, c_int64, c_void_p]
    lib.sa_compute_root_inverses_from_eigendecomposition.argtypes = [
        c_void_p, POINTER(c_void_p), c_float, POINTER(c_float), c_int32, c_float, c_float, POINTER(c_int32), c_void_p,
    ]
    lib.sa_plan_set_kl_shampoo.argtypes = [c_void_p, c_int32]
    lib.sa_move_params_towards_weight_buffer.argtypes = [c_void_p, c_float, c_void_p]
    lib.sa_plan_set_factor_dtype.argtypes = [c_void_p, c_int32]
    lib.sa_plan_set_scratch_budget.argtypes = [c_void_p, c_int64]
    lib.sa_plan_num_waves.argtypes = [c_void_p]
    lib.sa_plan_set_symmetric_newton.argtypes = [c_void_p, c_int32]
    lib.sa_plan_set_eigh_solver.argtypes = [c_void_p, c_int32]
    lib.sa_plan_rebind_params.argtypes = [c_void_p, POINTER(c_void_p)]
    lib.sa_set_small_launch_tiles.argtypes = [c_int32]
    lib.sa_plan_export_dense_state.argtypes = [c_void_p, POINTER(c_void_p), POINTER(c_void_p), c_void_p]
    lib.sa_plan_import_dense_state.argtypes = [c_void_p, POINTER(c_void_p), POINTER(c_void_p), c_void_p]
    lib.sa_update_factor_matrices_f64.argtypes = [c_void_p, c_double, c_double, c_void_p]
    lib.sa_compute_root_inverses_newton_f64.argtypes = [
        c_void_p, c_float, c_double, c_int32, c_double, c_int32, POINTER(c_int32), POINTER(c_int32), c_void_p,
    ]
    lib.sa_compute_root_inverses_eigh_f64.argtypes = [
        c_void_p, c_float, c_double, POINTER(c_float), c_int32, c_double, c_double, c_int32, POINTER(c_int32), POINTER(c_int32),
        c_void_p,
    ]
    lib.sa_add_to_views.argtypes = [POINTER(View), POINTER(View), c_int32, c_void_p]
    lib.sa_set_profiling.argtypes = [c_int32]
    lib.sa_phase_ms.argtypes = [c_char_p]
    lib.sa_phase_ms.restype = c_double
    lib.sa_phase_flops.argtypes = [c_char_p]
    lib.sa_phase_flops.restype = c_double
    lib.sa_phase_executed_flops.argtypes = [c_char_p]
    lib.sa_phase_executed_flops.restype = c_double
    lib.sa_set_symmetric_newton.argtypes = [c_int32]
    lib.sa_set_eigh_solver.argtypes = [c_int32]
    lib.sa_plan_read_eigenvalues.argtypes = [c_void_p, c_int32, c_void_p, c_void_p]
    lib.sa_plan_set_trace_scaling.argtypes = [c_void_p, c_int32, c_float, c_float]
    lib.sa_phase_launches.argtypes = [c_char_p]
    lib.sa_phase_launches.restype = c_int32
    for name in EXPORTS:
        fn = getattr(lib, name)
        if fn.restype is ctypes.c_int:
            fn.restype = c_int32
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    if status != SA_OK:
        msg = load().sa_last_error().decode(errors="replace")
        raise NativeError(f"{what} failed with status {status}: {msg}")


def current_stream_ptr(device: torch.device) -> int:
    """hipStream_t of torch's current stream on `device` (never assumes stream 0)."""
    return int(torch.cuda.current_stream(device).cuda_stream)
