/*
 * C ABI of the MI355X-native Distributed Shampoo step (libshampoo_amd.so).
 *
 * The reference (facebookresearch/optimizers) is pure Python over torch ops and has no FFI
 * of its own; the seam this library plugs into is the `PreconditionerList` interface
 * (distributed_shampoo/preconditioner/preconditioner_list.py:49-102) together with the
 * default `Distributor` (distributed_shampoo/distributor/shampoo_distributor.py:302-430)
 * and the elementwise part of `DistributedShampoo._compute_search_directions`
 * (distributed_shampoo/distributed_shampoo.py:1384-1501).  Each entry point names the
 * reference routine it replaces.
 *
 * Conventions: every pointer inside a descriptor is a DEVICE pointer borrowed from the
 * caller (who keeps it alive until the stream work has finished); `stream` is a
 * hipStream_t passed as void*; every call returns SA_OK or an error code and leaves a
 * message for sa_last_error().  No exceptions cross the boundary.  All arithmetic is fp32, except the factor
 * averages and the coupled Newton iteration of a plan switched to fp64 factors (sa_plan_set_factor_dtype).
 * One plan describes the blocks of one parameter group on one GPU; calls on one plan must
 * not overlap.
 */
#ifndef SHAMPOO_AMD_H
#define SHAMPOO_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SA_OK 0
#define SA_ERR_INVALID 1     /* bad argument */
#define SA_ERR_HIP 2         /* a HIP runtime call failed */
#define SA_ERR_WORKSPACE 3   /* workspace missing or too small */
#define SA_ERR_UNSUPPORTED 4 /* valid in the reference, not built here */
#define SA_ERR_STATE 5       /* call order violated (e.g. gradients not bound) */

/* Per-factor status written by sa_compute_root_inverses_newton. */
#define SA_FACTOR_OK 0
#define SA_FACTOR_INPUT_NONFINITE 1  /* bias-corrected factor holds nan/inf (shampoo_preconditioner_list.py:374) */
#define SA_FACTOR_RESULT_NONFINITE 2 /* inverse root holds nan/inf        (shampoo_preconditioner_list.py:405) */
#define SA_FACTOR_NOT_CONVERGED 3    /* max_iterations reached; result kept (matrix_functions.py:678-681) */
#define SA_FACTOR_SKIPPED 4          /* follows a non-finite factor; not computed, state untouched */
#define SA_FACTOR_SOLVER_FAILED 5    /* the solver gave up where the reference raises inside matrix_inverse_root
                                        (matrix_functions.py:543, 629, 655); the stored inverse is untouched and the
                                        caller counts the failure (shampoo_preconditioner_list.py:388-443) */

/* Grafting flavours (distributed_shampoo.py:673-714). */
#define SA_GRAFT_NONE 0
#define SA_GRAFT_SGD 1
#define SA_GRAFT_ADAGRAD 2 /* AdaGrad / RMSprop / Adam: second moment + optional bias correction */

typedef struct sa_plan sa_plan;

#define SA_MAX_ORDER 3

/*
 * One block of a (merged) parameter, produced by merge_small_dims + multi_dim_split
 * (utils/shampoo_utils.py:38-174): an fp32 strided view of order 1, 2 or 3.
 *   order 2:  rows x cols, row stride ld.                       mid = 0.
 *   order 1:  length d as rows = d, cols = 1, ld = 1.           mid = 0.
 *   order 3:  d0 x d1 x d2 with element strides (ld_outer, ld, 1) as rows = d0 * d1, cols = d2, mid = d1:
 *             row r = i0 * d1 + i1 of the flattened block starts at i0 * ld_outer + i1 * ld.
 * State buffers are contiguous (rows * cols, the block's own row-major order).  Kronecker factor k belongs to
 * dim k of the block: for order <= 2 dim 0 = rows, dim 1 = cols; for order 3 dims (d0, d1, d2).
 * Mirrors what BlockInfo + the per-block optimizer state hold
 * (distributor/shampoo_block_info.py:18-65; state keys shampoo_types.py:35-41).
 */
typedef struct sa_block_desc {
  int32_t rows, cols;
  int64_t ld;             /* row stride, in elements, of the block inside its parameter and gradient */
  float* param;           /* block of the parameter (updated in place) */
  float* filtered_grad;   /* EMA of the gradient, or NULL when beta1 == 0 */
  float* adagrad;         /* grafting second moment, or NULL */
  float* momentum_buffer; /* classic momentum buffer, or NULL */
  float* factor[SA_MAX_ORDER];     /* packed upper-triangular Kronecker factor per dim; NULL = dim not preconditioned */
  float* inv_factor[SA_MAX_ORDER]; /* packed upper-triangular inverse root of that factor (root-inverse Shampoo), or NULL */
  int32_t root[SA_MAX_ORDER];      /* integer inverse root (2 * order by default: 2 for vectors, 4 for matrices, 6 for order 3) */
  /* eigenvalue-corrected Shampoo / SOAP (shampoo_preconditioner_list.py:942-1007): dense
   * d x d eigenbasis of each factor (row-major, columns are eigenvectors) and the second moment kept in the rotated
   * basis (rows x cols, contiguous).  NULL for root-inverse Shampoo.  eigenvectors[k] with factor[k] == NULL is a
   * fixed basis: it rotates the block but has no statistics and is never refreshed (a block whose basis
   * changes are all ignored, ignored_basis_change_dims, passes one identity matrix). */
  float* eigenvectors[SA_MAX_ORDER];
  float* corrected_eigenvalues;
  int32_t mid;            /* d1 of an order-3 block, else 0 */
  int64_t ld_outer;       /* stride of dim 0 of an order-3 block */
  float* weight_buffer;   /* the "z" sequence of generalized primal averaging / Schedule-Free (rows * cols, contiguous), or NULL */
} sa_block_desc;

/* Scalars of one step, already evaluated by the host exactly as the reference evaluates
 * them (fp32 bias corrections: distributed_shampoo.py:1190-1195,
 * adagrad_preconditioner_list.py:139-141). */
typedef struct sa_step_scalars {
  float lr;
  float beta1;             /* 0 disables the filtered gradient */
  float beta3;             /* == beta1 unless set */
  float bias_correction1;  /* divisor of the filtered gradient, 1.0f when off */
  int32_t graft_type;      /* SA_GRAFT_* */
  float graft_beta2;
  float graft_weight;      /* weighting factor of g*g */
  float graft_bias_correction2; /* divisor of the second moment, 1.0f when off */
  float graft_epsilon;
  float weight_decay_alpha; /* added to the direction as alpha*W (decoupled / corrected / independent); 0 = none */
  float momentum;           /* 0 = classic momentum off */
  float dampening;
  int32_t use_nesterov;
  /* Generalized primal averaging / Schedule-Free (distributed_shampoo.py:1343-1382), applied to the scaled direction
   * D = -lr P: T = Z - W; Z += D; D <- D * averaging_direction_coeff + averaging_buffer_coeff * T; W += D, with
   * averaging_direction_coeff = 1 - mu_y mu_x and averaging_buffer_coeff = 1 - mu_x evaluated by the host in fp32. */
  int32_t use_primal_averaging;
  float averaging_direction_coeff;
  float averaging_buffer_coeff;
  /* Weights of the two lerps of the filtered gradient, rounded to fp32 once from the host's double 1 - beta1 and
   * 1 - beta3 like the Python scalars the reference hands to torch._foreach_lerp_ (distributed_shampoo.py:1173-1188;
   * 1.0f - (float)beta differs from (float)(1.0 - beta) in the last bit for most betas). */
  float lerp_weight1;
  float lerp_weight3;
  /* Where the bias-corrected filtered gradient comes from, decided by the host on its double betas:
   * 0 = the gradient itself (beta1 == 0), 1 = the filtered gradient (beta3 == beta1), 2 = a separate lerp with beta3. */
  int32_t filtered_grad_mode;
} sa_step_scalars;

const char* sa_last_error(void);
int32_t sa_abi_version(void);

/* Builds the ragged batched descriptor table for a parameter group (replaces the per-step
 * Python list building of shampoo_distributor.py:237-299 and the per-block loops of
 * shampoo_preconditioner_list.py:1509-1539, 1672-1695). */
int32_t sa_plan_create(const sa_block_desc* blocks, int32_t n_blocks, sa_plan** plan_out);
void sa_plan_destroy(sa_plan* plan);

/* Scratch + dense-inverse cache the caller must provide (device memory, 256-byte aligned). */
int64_t sa_plan_workspace_bytes(const sa_plan* plan);
int32_t sa_plan_bind_workspace(sa_plan* plan, void* workspace, int64_t bytes);

/* Bounds the scratch region of the amortized computations (sa_compute_root_inverses_*, sa_refresh_eigenbases_*): every
 * factor in flight needs 8 dense dpad x dpad fp32 arrays (16 with fp64 factors; dpad = order rounded up to 128), which
 * for all factors of a large parameter group at once is 8 x the dense inverse roots.  With a budget the factors are cut
 * into waves of consecutive factors whose arrays fit `bytes` together (one factor at least), and the calls above work
 * through the waves one after the other in the same region; results do not depend on the budget.  0 (the default) = no
 * limit, one wave.  Must be called before sa_plan_workspace_bytes / sa_plan_bind_workspace.  No counterpart in the
 * reference, which allocates per factor. */
int32_t sa_plan_set_scratch_budget(sa_plan* plan, int64_t bytes);
int32_t sa_plan_num_waves(const sa_plan* plan);

/* Number of factor matrices, in block order then dim order (the order of every per-factor array). */
int32_t sa_plan_num_factors(const sa_plan* plan);

/* Marks what the plan derives from the optimizer state stale: the dense inverse cache and the filtered gradient kept
 * in the eigenbasis (after the caller wrote inv_factor, eigenvectors or filtered_grad itself, e.g. load_state_dict). */
int32_t sa_plan_invalidate_inverse_cache(sa_plan* plan);

/* How sa_compute_root_inverses_newton schedules a batch (no counterpart in the reference, whose loop runs factor by
 * factor): a batch whose stages are launches of fewer than `tiles` 128 x 128 tiles is cut into two halves that iterate
 * side by side, the second on a stream the plan owns (joined with the caller's stream before the call's result pass).
 * Every stage of an iteration waits for the one before it, so a short launch alone leaves the chip idle while it ramps
 * up and drains; the other half's launch fills that.  The factors are independent: results and iteration counts are the
 * bits of the unsplit run.  Default 0 = never split: on the GPT-2 parameter set the two halves measured slower than the
 * whole batch (73.8 against 69.6 ms per step), so the switch is kept for experiments only. */
int32_t sa_plan_set_newton_split_tiles(sa_plan* plan, int32_t tiles);

/* Lanes of the Householder tridiagonalisation behind sa_compute_root_inverses_eigh / sa_refresh_eigenbases_eigh for
 * orders from 512 on (no counterpart in the reference, which calls torch.linalg.eigh factor by factor): a batch of
 * factors is reduced in `lanes` parts (1..4, default 3; at least two factors per part), the parts after the first on
 * streams the plan owns, joined with the caller's stream when the reduction ends.  Per column the reduction is one
 * latency-bound workgroup per factor and one bandwidth-bound product, each waiting for the other; parts side by side fill
 * each other's gaps (32 factors of order 4096: 415 / 376 / 361 / 527 ms with 1 / 2 / 3 / 4 lanes).  Same bits for every
 * number of lanes. */
int32_t sa_plan_set_tridiagonal_lanes(sa_plan* plan, int32_t lanes);

/* Gradients of this step, one device pointer per block (same rows/cols/ld as the block); NULL
 * masks a block out of every following call (shampoo_distributor.py:269-277). */
int32_t sa_plan_bind_gradients(sa_plan* plan, float* const* grads, void* stream);

/* G += weight_decay * W, in place on the gradient (distributed_shampoo.py:1127-1139). */
int32_t sa_add_l2_regularization(sa_plan* plan, float weight_decay, void* stream);

/* L <- beta2 L + w G G^T, R <- beta2 R + w G^T G on packed storage
 * (shampoo_preconditioner_list.py:1490-1539). */
int32_t sa_update_factor_matrices(sa_plan* plan, float beta2, float weighting_factor, void* stream);

/* Batched coupled inverse Newton iteration on every factor, A = unpack(factor / bias_correction2)
 * (matrix_functions.py:368-437 via shampoo_preconditioner_list.py:314-443, 631-680).
 * iterations_out / status_out: host arrays of sa_plan_num_factors() entries.  Inverse roots of
 * factors that precede the first non-finite one are stored into inv_factor (upper triangle);
 * the call synchronises the stream before it returns.  M_p^root is a square-and-multiply chain of at most
 * five products: every integer root up to 14, and 16 (SA_ERR_UNSUPPORTED beyond). */
int32_t sa_compute_root_inverses_newton(sa_plan* plan, float bias_correction2, float epsilon,
                                        int32_t max_iterations, float tolerance,
                                        int32_t* iterations_out, int32_t* status_out, void* stream);

/* Factor matrices in fp64 (`factor_matrix_dtype=torch.float64`, shampoo_types.py:184 of the reference): with 64,
 * every `factor[]` pointer of the plan's descriptors addresses a packed triangle of doubles, the Gram matrices (fp32
 * products, like the reference's tensordot of fp32 gradients) are averaged in double, and the root inverse runs in
 * double precision; `inv_factor[]` stays fp32 (`inv_factor_matrix_dtype`).  Plans that keep eigenvectors
 * (eigenvalue-corrected and eigendecomposed Shampoo) average their factors in double as well; their eigenbasis refreshes
 * (sa_refresh_eigenbases_*) run in fp32 on the rounded average, the eigenvectors being fp32 state in the reference too
 * (factor_matrix_eigenvectors_dtype; the reference decomposes in double and casts, shampoo_preconditioner_list.py:1160-1166).
 * Must be called before sa_plan_workspace_bytes / sa_plan_bind_workspace (the scratch doubles). */
int32_t sa_plan_set_factor_dtype(sa_plan* plan, int32_t bits);

/* sa_update_factor_matrices for an fp64 plan: L <- beta2 L + w G G^T with beta2 and w in double, as
 * `factor.mul_(beta2)`, `factor.add_(outer_product, alpha=w)` act on a float64 factor
 * (shampoo_preconditioner_list.py:1524-1539). */
int32_t sa_update_factor_matrices_f64(sa_plan* plan, double beta2, double weighting_factor, void* stream);

/* sa_compute_root_inverses_newton for an fp64 plan: the coupled Newton iteration of matrix_functions.py:368-437 on
 * A = unpack(factor / bias_correction2) + epsilon I in double precision (fp64 MFMA GEMMs), the result cast to the fp32
 * inverse-root state (shampoo_preconditioner_list.py:672-678).  bias_correction2 is the reference's fp32 scalar, widened
 * exactly.  iterations_out / status_out as in the fp32 call.  widen_ridge_on_failure = 0 is the reference's CoupledNewtonConfig
 * on a float64 factor.  With 1 the call stands in for the reference's float64 eigendecomposition root inverse
 * (EigenConfig, matrix_functions.py:306-366): a factor on which the iteration does not converge (not positive
 * definite above epsilon) is solved again with the ridge epsilon + 2^-21 ||A||_F, where the eigendecomposition would
 * shift the spectrum by its smallest eigenvalue. */
int32_t sa_compute_root_inverses_newton_f64(sa_plan* plan, float bias_correction2, double epsilon, int32_t max_iterations,
                                            double tolerance, int32_t widen_ridge_on_failure, int32_t* iterations_out,
                                            int32_t* status_out, void* stream);

/* sa_compute_root_inverses_eigh for an fp64 plan (sa_plan_set_factor_dtype(plan, 64)): the reference's eigendecomposition
 * root inverse on a float64 factor (matrix_functions.py:306-366 with torch.linalg.eigh in float64, :725-770).
 * A = unpack(factor / bias_correction2) (+ epsilon I for stability 1) in double; its eigendecomposition to double
 * precision (the fp32 solvers on the rounded matrix give eigenvectors good to 1e-6, two Newton-Schulz steps make them
 * orthogonal to rounding, cyclic Jacobi in fp64 on X^T A X finishes); the weights of
 * matrix_inverse_root_from_eigendecomposition (`stability`, `rank_rtol`, `rank_atol`, `roots` as in
 * sa_compute_root_inverses_eigh) and X = Q diag(w) Q^T in double; the result cast to the fp32 inverse-root state
 * (shampoo_preconditioner_list.py:672-678).  sweeps_out: Jacobi sweeps in fp64 (at most max_sweeps, which also bounds the fp32 solver's
 * sweeps; SA_FACTOR_NOT_CONVERGED beyond; two to three are usual, the fp32 eigenvectors leave X^T A X diagonal to 1e-6). */
int32_t sa_compute_root_inverses_eigh_f64(sa_plan* plan, float bias_correction2, double epsilon, const float* roots,
                                          int32_t stability, double rank_rtol, double rank_atol, int32_t max_sweeps,
                                          int32_t* sweeps_out, int32_t* status_out, void* stream);

/* Batched coupled higher-order iteration on every factor (CoupledHigherOrderConfig; matrix_functions.py:439-661 via
 * :682-689): A = unpack(factor / bias_correction2), A_r = A + max(rel_epsilon * |A|_inf, abs_epsilon) I,
 * z = 1 / trace(A_r); one plain Newton step, then steps with M_p = sum_{i < order} b_i (I - M)^i until the error
 * max|M - I| is at most `tolerance`, max_iterations is reached, or the error grows by more than 1.2 x or repeats
 * itself below 1e-3 (the update of that step stays).  A factor whose result has |A_r X^p - I|_max > 0.1 or holds
 * nan/inf gets SA_FACTOR_SOLVER_FAILED and keeps its stored inverse; the optimizer's epsilon plays no part, as in
 * the reference.  Orders 2..8; roots as for the Newton call (the root's denominator must be 1).
 * iterations_out / status_out as for the Newton call; the call synchronises the stream before it returns. */
int32_t sa_compute_root_inverses_higher_order(sa_plan* plan, float bias_correction2, float rel_epsilon,
                                              float abs_epsilon, int32_t max_iterations, float tolerance,
                                              int32_t order, int32_t* iterations_out, int32_t* status_out,
                                              void* stream);

/* Batched symmetric eigendecomposition root inverse on every factor (solver: see sa_set_eigh_solver):
 * A = unpack(factor / bias_correction2), (lambda, Q) = eigh(A), X = Q diag(w) Q^T
 * (matrix_functions.py:179-279, 306-366, 698-770 via shampoo_preconditioner_list.py:314-443, 631-680).
 * stability selects the reference's rank_deficient_stability_config:
 *   0  PerturbationConfig(perturb_before_computation=False): lambda <- lambda - min(lambda_min, 0) + epsilon;
 *   1  PerturbationConfig(perturb_before_computation=True): A + epsilon I is decomposed, and the spectrum is
 *      shifted by -lambda_min + epsilon only if lambda_min < epsilon;
 *   2  PseudoInverseConfig(rank_rtol, rank_atol): epsilon must be 0; w = 0 where
 *      lambda <= max(rank_atol, rtol * max(lambda_max, 0)), rtol = rank_rtol or, for rank_rtol < 0 (the
 *      reference's None), order * 2^-23.
 * Otherwise w = lambda^(-1/root).  roots: host array, one (possibly fractional) root per factor.
 * sweeps_out / status_out as for the Newton call; SA_FACTOR_NOT_CONVERGED means the solver gave up
 * (Jacobi rotations still being applied in sweep max_sweeps, or the QL sweep budget of 30 per eigenvalue). */
int32_t sa_compute_root_inverses_eigh(sa_plan* plan, float bias_correction2, float epsilon, const float* roots,
                                      int32_t stability, float rank_rtol, float rank_atol, int32_t max_sweeps,
                                      int32_t* sweeps_out, int32_t* status_out, void* stream);

/* Eigenbasis refresh through a full symmetric eigendecomposition: the `EighEigendecompositionConfig` branch of
 * matrix_eigendecomposition (matrix_functions.py:725-770, :885-900) inside the eigenvalue-corrected list's
 * amortized computation (shampoo_preconditioner_list.py:1793-1990).  A = factor / bias_correction2 + epsilon I
 * (pass epsilon = 0 when the config does not perturb before the computation); the eigenvectors, in ascending
 * order of their eigenvalues, replace `eigenvectors[]` of every active block.  tolerance != 0: a factor whose
 * stored basis Q already satisfies ||B - diag B||_F <= tolerance ||B||_F, B = Q^T A Q, keeps it
 * (matrix_functions.py:772-797).  status / sweeps arrays as in sa_compute_root_inverses_eigh. */
int32_t sa_refresh_eigenbases_eigh(sa_plan* plan, float bias_correction2, float epsilon, float tolerance, int32_t max_sweeps,
                                   int32_t* sweeps_out, int32_t* status_out, void* stream);

/* Eigenbasis refresh of eigenvalue-corrected Shampoo with the QR algorithm: B = Q^T A Q with
 * A = unpack(factor / bias_correction2) + epsilon I; while ||B - diag(B)||_F > tolerance ||B||_F and fewer than
 * max_iterations were done: (Q', R) = qr(B) (blocked Householder), Q <- Q Q', B <- Q^T A Q; finally the columns
 * of Q are ordered by ascending diag(B) with a stable sort (matrix_functions.py:799-852 via
 * shampoo_preconditioner_list.py:314-443, 1137-1198).  iterations_out / status_out as for the Newton call. */
int32_t sa_refresh_eigenbases_qr(sa_plan* plan, float bias_correction2, float epsilon, int32_t max_iterations,
                                 float tolerance, int32_t* iterations_out, int32_t* status_out, void* stream);

/* Eigendecomposed Shampoo (EigendecomposedShampooPreconditionerConfig): a block descriptor gives `factor`,
 * `eigenvectors` AND `inv_factor` for each preconditioned dim and no `corrected_eigenvalues`.  The amortized
 * computation (shampoo_preconditioner_list.py:763-940: matrix_eigendecomposition of the bias-corrected factor, started
 * from the stored eigenvectors for the QR algorithm) is sa_refresh_eigenbases_eigh / sa_refresh_eigenbases_qr followed
 * by sa_plan_read_eigenvalues into the caller's eigenvalue state; this call then forms
 * X = Q diag(w) Q^T, w from matrix_inverse_root_from_eigendecomposition (matrix_functions.py:179-279; `stability`,
 * `rank_rtol`, `rank_atol` and `roots` as in sa_compute_root_inverses_eigh), and stores it in `inv_factor`, which
 * sa_precondition uses.  The reference forms the same product in every step (:1793-1832); it only changes with
 * (Q, lambda).  `eigenvalues[i]`: device pointer to the d eigenvalues of factor i (plan order).  Call it again after
 * writing eigenvectors / eigenvalues from outside (checkpoint load).  status_out: SA_FACTOR_OK, _SKIPPED or
 * _RESULT_NONFINITE. */
int32_t sa_compute_root_inverses_from_eigendecomposition(sa_plan* plan, const float* const* eigenvalues, float epsilon,
                                                         const float* roots, int32_t stability, float rank_rtol,
                                                         float rank_atol, int32_t* status_out, void* stream);

/* corrected_eigenvalues <- beta2 * corrected_eigenvalues + w * (Q_L^T G Q_R)^2 with the raw gradient
 * (shampoo_preconditioner_list.py:1891-1912). */
int32_t sa_update_corrected_eigenvalues(sa_plan* plan, float beta2, float weighting_factor, void* stream);

/* P = Q_L [ (Q_L^T Ghat Q_R) / ((corrected_eigenvalues / bias_correction2)^(1/root) + epsilon) ] Q_R^T into the
 * workspace plus its squared norm per block (shampoo_preconditioner_list.py:1914-1942). */
int32_t sa_precondition_eigenvalue_corrected(sa_plan* plan, const sa_step_scalars* s, float bias_correction2,
                                             float epsilon, float root, void* stream);

/* sa_update_corrected_eigenvalues followed by sa_precondition_eigenvalue_corrected on the bound gradients, for the
 * step as the reference runs it (shampoo_preconditioner_list.py:1891-1942 within distributed_shampoo.py:1162-1270:
 * the eigenbases do not change between the two).  Call it after sa_update_grafting_and_filtered_grad of the same step.
 * The rotation is linear, so Q_L^T Ghat Q_R need not be formed by two more products: with beta1 = 0 it is the
 * rotated gradient of the statistic, and otherwise the plan keeps Q_L^T m Q_R and advances it by m's own moving
 * average inside the statistic's launch (blocks of order 2 with both eigenbases; the copy is rebuilt by the next
 * full preconditioning after a refresh, a workspace bind, sa_plan_invalidate_inverse_cache or a change of the masked
 * blocks).  Results equal the two separate calls up to fp32 rounding of the reordered sums.  beta3 != beta1 is
 * rejected with SA_ERR_UNSUPPORTED: make the two separate calls, the first one before the prologue. */
int32_t sa_update_and_precondition_eigenvalue_corrected(sa_plan* plan, const sa_step_scalars* s, float beta2,
                                                        float weighting_factor, float bias_correction2, float epsilon,
                                                        float root, void* stream);

/* How many calls of sa_update_and_precondition_eigenvalue_corrected shared the rotation (the others fell back to the
 * two separate routines and rebuilt the rotated copy).  No counterpart in the reference; for tests and tuning. */
int64_t sa_plan_shared_rotation_steps(const sa_plan* plan);

/* Grafting second moment, filtered gradient and the grafted direction's squared norm per block
 * (adagrad_preconditioner_list.py:122-162, distributed_shampoo.py:1162-1199, 1110-1114). */
int32_t sa_update_grafting_and_filtered_grad(sa_plan* plan, const sa_step_scalars* s, void* stream);

/* P = L^-1/r0 * Ghat * R^-1/r1 into the workspace plus its squared norm per block
 * (shampoo_preconditioner_list.py:1541-1578, 1672-1695, 1780-1790). */
int32_t sa_precondition(sa_plan* plan, const sa_step_scalars* s, void* stream);

/* Grafting rescale, weight decay, momentum, learning rate and W += P
 * (distributed_shampoo.py:1115-1122, 1202-1293, 1484; shampoo_distributor.py:335-365). */
int32_t sa_apply_update(sa_plan* plan, const sa_step_scalars* s, void* stream);

/* W += coeff * (Z - W) for every block that has a weight buffer, masked or not: the switch between the training
 * sequence y and the evaluation sequence x of generalized primal averaging / Schedule-Free,
 * `DistributedShampoo.train()` (coeff = 1 - mu_y) and `eval()` (coeff = 1 - 1 / mu_y), distributed_shampoo.py:1729-1793. */
int32_t sa_move_params_towards_weight_buffer(sa_plan* plan, float coeff, void* stream);

/* Whole step before preconditioning starts: the grafted direction is the update
 * (distributed_shampoo.py:1093-1098 followed by :1202-1293, 1484). */
int32_t sa_grafting_only_step(sa_plan* plan, const sa_step_scalars* s, void* stream);

/* Test / measurement aids. */

/* Eigenvalue estimates that belong to the eigenbasis the last sa_refresh_eigenbases_eigh / _qr call on this plan
 * left for factor `factor` (index in plan order), in the order of the basis' columns: the ascending eigenvalues
 * of a fresh decomposition, diag(Q^T A Q) of a basis kept by the tolerance criterion, the sorted Rayleigh
 * quotients of a QR refresh -- the first return value of matrix_eigendecomposition (matrix_functions.py:698-908).
 * out: device array of that factor's order.  Must directly follow the refresh call; SA_ERR_STATE otherwise. */
int32_t sa_plan_read_eigenvalues(sa_plan* plan, int32_t factor, float* out, void* stream);

/* Per-block squared norms of the last step: graft_sq[i], precond_sq[i] (host arrays of n_blocks). */
int32_t sa_plan_read_norms(sa_plan* plan, float* graft_sq, float* precond_sq, void* stream);

/* Copies the preconditioned (unscaled) direction of block i into out (device, contiguous rows*cols). */
int32_t sa_plan_read_preconditioned(sa_plan* plan, int32_t block, float* out, void* stream);

/* C = op(A) op(B) with the grouped MFMA kernel, one problem, `batch` copies strided by the given
 * element strides.  a_layout: 0 = A[m*lda+k], 1 = A[k*lda+m]; b_layout: 0 = B[k*ldb+n], 1 = B[n*ldb+k]. */
int32_t sa_gemm_f32(const float* A, const float* B, float* C, int32_t M, int32_t N, int32_t K,
                    int64_t lda, int64_t ldb, int64_t ldc, int32_t a_layout, int32_t b_layout,
                    int32_t batch, int64_t stride_a, int64_t stride_b, int64_t stride_c, void* stream);

/* State tensors without symmetric packing (reference: use_symmetric_packing = False, shampoo_types.py:170-186; the
 * state then holds d x d matrices, shampoo_preconditioner_list.py:139-156, and _pack / _unpack are the identity,
 * :283-301).  The plan's factor[] / inv_factor[] stay packed triangles owned by the caller as before; these two calls
 * move them to and from dense tensors (row-major, row stride d, both triangles) that the caller shows in its state.
 * dense_factor / dense_inv: one pointer per factor matrix, in the order of the descriptors' non-NULL factor[] entries
 * (block by block, dim by dim); a NULL array or a NULL entry is skipped.  dense_factor holds floats, or doubles on a
 * plan whose factor matrices are doubles (sa_plan_set_factor_dtype); dense_inv always holds floats.
 * sa_plan_export_dense_state: dense = mirror(packed).  sa_plan_import_dense_state: packed = upper triangle of dense
 * (after a checkpoint load; call sa_plan_invalidate_inverse_cache afterwards as for any outside write). */
int32_t sa_plan_export_dense_state(sa_plan* plan, void* const* dense_factor, void* const* dense_inv, void* stream);
int32_t sa_plan_import_dense_state(sa_plan* plan, void* const* dense_factor, void* const* dense_inv, void* stream);

/* sa_gemm_f32 for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments, same kernels and
 * bit-identical results; the problem table that sa_gemm_f32 keeps in a device buffer it allocates and uploads lives in
 * a file-scope device array of SA_GEMM_STATIC_MAX_BATCH entries (128 KB, held by every GPU the library runs on until
 * the process ends) and is written by a small kernel from the call's arguments.  The call issues kernel launches only:
 * no hipMalloc / hipFree, no copy, no allocating library routine.  batch > SA_GEMM_STATIC_MAX_BATCH is rejected with
 * SA_ERR_INVALID.  Every call on a GPU shares that GPU's table: calls that overlap on one GPU (two streams, two
 * threads) race; calls on one stream are ordered. */
#define SA_GEMM_STATIC_MAX_BATCH 1024
int32_t sa_gemm_f32_static(const float* A, const float* B, float* C, int32_t M, int32_t N, int32_t K,
                           int64_t lda, int64_t ldb, int64_t ldc, int32_t a_layout, int32_t b_layout,
                           int32_t batch, int64_t stride_a, int64_t stride_b, int64_t stride_c, void* stream);

/* A strided fp32 view of device memory of at most SA_MAX_ORDER dims: what a torch view of a parameter block
 * is (sizes and element strides, outermost dim first; order 0 = one element). */
typedef struct sa_view {
  void* data;
  int32_t order;
  int64_t size[SA_MAX_ORDER];
  int64_t stride[SA_MAX_ORDER];
} sa_view;

/* dst[i] += src[i] for n pairs of views of equal sizes: `Distributor.update_params`
 * (distributor/shampoo_distributor.py:335-365, one `torch._foreach_add_` over the masked blocked parameters and
 * their search directions).  The tables are host arrays read during the call; no device memory is allocated (the
 * jobs travel as kernel arguments, 24 pairs per launch).  All pairs are validated before the first launch.
 * Destination views must not alias each other. */
int32_t sa_add_to_views(const sa_view* dst, const sa_view* src, int32_t n, void* stream);

/* dst[i] = src[i] for n floats with a plain float4 copy kernel (n % 4 == 0, 16-byte aligned): the
 * known-traffic kernel that hardware HBM counters are calibrated against. */
int32_t sa_copy_f32(const float* src, float* dst, int64_t n, void* stream);

/* Averaged duration (milliseconds, HIP events on `stream`) of the kernels of the named phase during
 * the most recent call that ran it: "newton_gemm", "syrk", "precondition_gemm", "grafting", "apply".
 * Timing is off unless sa_set_profiling(1) was called; switching it on (from off) forgets every recorded phase.
 * Returns a negative value if unavailable.
 * Independently of the timing, SHAMPOO_AMD_ROCTX=1 in the environment brackets the same phases on the host with
 * roctxRangePush / roctxRangePop (looked up at run time, nothing links against the marker library): the ranges a tracer
 * shows under the Python ranges of the optimizer, as the reference's record_function ranges do
 * (preconditioner/preconditioner_list.py:23-46). */
int32_t sa_set_profiling(int32_t enabled);
double sa_phase_ms(const char* phase);
double sa_phase_flops(const char* phase); /* algorithmic flops (or bytes for HBM-bound phases) of that call */
int32_t sa_phase_launches(const char* phase);
double sa_phase_executed_flops(const char* phase); /* flops actually issued by "newton_gemm" (symmetric products are halved) */

/* Coupled Newton products are symmetric in exact arithmetic (every operand is a polynomial in the
 * factor).  A symmetric product computes only the tiles on or above the diagonal and mirrors them
 * (1.9x fewer MFMA flops at d = 2048); the reference's `@` (matrix_functions.py:426-427) is a full GEMM.
 * Both variants deviate from exact arithmetic by about 3e-9 x condition number (the symmetric one by about
 * twice as much), so they agree to < 1e-4 while the factor's condition number is below 1e4, which shows
 * as a solve of at most 14 iterations.  Policy (the default of plans created afterwards):
 *   0  every product is a full GEMM, the reference's arithmetic;
 *   1  every product is symmetric;
 *   2  (default) per factor: symmetric only if the factor's previous solve converged within 14 iterations;
 *      a symmetric solve that then needs more than 17 iterations or does not converge is repeated with
 *      full products, so failure semantics are those of policy 0.
 * No counterpart in the reference. */
int32_t sa_set_symmetric_newton(int32_t policy);
/* No counterpart in the reference.  Launches of the coupled Newton loop, the factor update and the first
 * preconditioning product that hold fewer than `tiles` 128 x 128 output tiles run with 64 x 64 tiles instead (four times
 * the workgroups for a launch that cannot fill the chip); the results are bit-identical either way.  Default 256 (one
 * large tile per CU); 0 switches the small tiles off.  The late iterations of a coupled Newton batch, in which the factors
 * that the host expects to be still iterating (from their previous solve) hold fewer than 1.25 x `tiles` large tiles per
 * product, take the small tiles too.  Process-wide. */
int32_t sa_set_small_launch_tiles(int32_t tiles);
/* The same choice for one plan (sa_set_symmetric_newton sets the default that plans created afterwards start with). */
int32_t sa_plan_set_symmetric_newton(sa_plan* plan, int32_t policy);

/* Solver behind sa_compute_root_inverses_eigh (stands in for torch.linalg.eigh, matrix_functions.py:233-366):
 *   0  (default) by order: two-sided block Jacobi below 512; from 512 up to 8192 blocked Householder
 *      tridiagonalisation, then bisection + inverse iteration on the tridiagonal matrix (one thread per eigenpair; a
 *      factor whose vectors fail the residual / orthogonality check is redone with the implicit QL iteration);
 *   1  block Jacobi for every factor;
 *   2  tridiagonalisation for every factor whose padded order is at least 256;
 *   3  like 2, with the implicit QL iteration (batched rotation application) for every factor.
 * The default of plans created afterwards.  No counterpart in the reference. */
int32_t sa_set_eigh_solver(int32_t solver);
/* The same choice for one plan (sa_set_eigh_solver sets the default that plans created afterwards start with). */
int32_t sa_plan_set_eigh_solver(sa_plan* plan, int32_t solver);

/* New parameter pointers for the blocks of a plan, one per block in plan order (same shapes and strides): for callers
 * whose parameter storage moved after the plan was built (`p.data = ...`, weight swaps, some checkpoint loaders).
 * A deliberate deviation, not parity: the reference blocks detached views of the storage the parameters had when the
 * optimizer was built (shampoo_distributor.py:202-216) and goes on updating that old storage after such a change, so the
 * parameter stops moving; following the new storage is what the caller of `p.data = ...` means. */
int32_t sa_plan_rebind_params(sa_plan* plan, float* const* params);

/* KL-Shampoo (RootInvKLShampooPreconditionerConfig / EigendecomposedKLShampooPreconditionerConfig,
 * shampoo_preconditioner_list.py:1945-2046): with `enabled`, sa_update_factor_matrices takes the Gram matrices of a
 * block with two Kronecker factors from the gradient preconditioned along the other dim with the stored inverse
 * root, L <- beta2 L + w (G X_R)(G X_R)^T and R <- beta2 R + w (X_L G)^T (X_L G); blocks with one factor are
 * unchanged.  Order-3 blocks with more than one factor are rejected. */
int32_t sa_plan_set_kl_shampoo(sa_plan* plan, int32_t enabled);

/* Trace scaling (use_trace_scaling / trace_scaling_exponent, shampoo_preconditioner_list.py:366-371): when
 * enabled, every root-inverse and eigenbasis computation of this plan works on
 *   (factor / bias_correction2) * max(trace(factor / bias_correction2), floor) ^ (-exponent)
 * instead of factor / bias_correction2; `floor` is the optimizer's epsilon.  The multiplier is evaluated on the
 * device, one per factor, in front of the finiteness check of the input.  Off by default. */
int32_t sa_plan_set_trace_scaling(sa_plan* plan, int32_t enabled, float exponent, float floor);

#ifdef __cplusplus
}
#endif
#endif /* SHAMPOO_AMD_H */
