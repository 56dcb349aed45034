// Batched symmetric eigendecomposition for gfx950: two-sided block Jacobi.
//
// A factor matrix (dense, mirrored, zero padded to dpad = multiple of 128) is cut into
// column/row blocks of 32.  One sweep visits every pair of blocks (I, J) once, in the
// nb-1 rounds of a round-robin tournament; the nb/2 pairs of a round are disjoint, so a
// round is three launches over all factors and all pairs at once:
//   1. jacobi_pivot_kernel: the 64x64 pivot [A_II A_IJ; A_JI A_JJ] goes to LDS and gets one
//      cyclic Jacobi sweep (parallel ordering, 63 rounds of 32 independent rotations);
//      the accumulated 64x64 rotation U is written out.
//   2. jacobi_cols_kernel:  A[:, I u J] <- A[:, I u J] U and V[:, I u J] <- V[:, I u J] U
//   3. jacobi_rows_kernel:  A[I u J, :] <- U^T A[I u J, :]
// Steps 2 and 3 are 64-deep fp32 MFMA products on 128-row (128-column) slabs read and
// written in place, i.e. HBM-bound: 24 d^2 bytes per round.  After convergence diag(A)
// holds the eigenvalues and V the eigenvectors; padded rows/columns never rotate (their
// off-diagonal entries are exactly zero), so they stay decoupled unit vectors.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm.h"

namespace sa {

constexpr int JB = 32;        // Jacobi block size
constexpr int JP = 2 * JB;    // pivot size

struct JacobiFactor {
  float* A;            // dpad x dpad, ld = dpad
  float* V;            // dpad x dpad eigenvector accumulator
  float* U;            // (nb/2) x 64 x 64 rotations of the current round
  const int2* sched;   // (nb-1) x (nb/2) block pairs (I < J)
  int* rotations;      // number of rotations applied in the current sweep
  float* rot_mass;     // sum of 2 a_pq^2 over those rotations = decrease of the off-diagonal norm^2
  const int* active;   // skip the factor when *active == 0
  float thr_abs;       // |a_pq| below this is treated as zero
  float thr_diag;      // a pair whose two diagonal entries are both below this (in magnitude) lies in the
                       // part of the spectrum fp32 cannot resolve and is left alone
  int d, dpad, nb;
  int pair_begin;      // first global pair id of this factor
};

__device__ __forceinline__ int jacobi_locate(const JacobiFactor* __restrict__ f, int n, int id) {
  int lo = 0, hi = n - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (f[mid].pair_begin <= id) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// pair k of round r in a round-robin tournament of n (even) players
__device__ __forceinline__ void circle_pair(int n, int r, int k, int& p, int& q) {
  const int m = n - 1;
  int a, b;
  if (k == 0) { a = 0; b = (r % m) + 1; }
  else { a = ((r + k) % m) + 1; b = ((r - k + m) % m) + 1; }
  p = min(a, b);
  q = max(a, b);
}

__global__ __launch_bounds__(256) void jacobi_pivot_kernel(const JacobiFactor* __restrict__ factors, int n_factors,
                                                          int round) {
  __shared__ float G[JP][JP + 1];
  __shared__ float U[JP][JP + 1];
  __shared__ float cs[2][JB];
  __shared__ int pq[2][JB];
  __shared__ int nrot;
  __shared__ float nmass;
  const int fi = jacobi_locate(factors, n_factors, blockIdx.x);
  const JacobiFactor& F = factors[fi];
  if (*F.active == 0 || round >= F.nb - 1) return;
  const int pair = blockIdx.x - F.pair_begin;
  const int2 ij = F.sched[round * (F.nb / 2) + pair];
  const int tid = threadIdx.x;
  const long long ld = F.dpad;
  if (tid == 0) { nrot = 0; nmass = 0.0f; }
  for (int e = tid; e < JP * JP; e += 256) {
    const int i = e >> 6, j = e & 63;
    const int gi = (i < JB ? ij.x * JB + i : ij.y * JB + i - JB);
    const int gj = (j < JB ? ij.x * JB + j : ij.y * JB + j - JB);
    G[i][j] = F.A[gi * ld + gj];
    U[i][j] = (i == j) ? 1.0f : 0.0f;
  }
  __syncthreads();
  const float thr_abs = F.thr_abs;
  for (int ir = 0; ir < JP - 1; ++ir) {
    if (tid < JB) {
      int p, q;
      circle_pair(JP, ir, tid, p, q);
      const float app = G[p][p], aqq = G[q][q], apq = 0.5f * (G[p][q] + G[q][p]);
      float c = 1.0f, s = 0.0f;
      const float thr = fmaxf(5.9604645e-8f * sqrtf(fabsf(app * aqq)), thr_abs);
      const bool unresolvable = fabsf(app) < F.thr_diag && fabsf(aqq) < F.thr_diag;
      if (fabsf(apq) > thr && !unresolvable) {
        const float tau = (aqq - app) / (2.0f * apq);
        const float t = (tau >= 0.0f) ? 1.0f / (tau + sqrtf(1.0f + tau * tau)) : 1.0f / (tau - sqrtf(1.0f + tau * tau));
        c = 1.0f / sqrtf(1.0f + t * t);
        s = t * c;
        atomicAdd(&nrot, 1);
        atomicAdd(&nmass, 2.0f * apq * apq);
      }
      // Rutishauser's form: x' = x - s (y + tq x), y' = y + s (x - tq y) with tq = tan(theta/2) = s / (1 + c).
      // It adds the small term (1 - c) x to the other small term before touching x, so tiny rotations do not
      // bias the column norms (c alone rounds to 1 for |t| < 2.4e-4).
      cs[0][tid] = s / (1.0f + c);
      cs[1][tid] = s;
      pq[0][tid] = p;
      pq[1][tid] = q;
    }
    __syncthreads();
    {  // columns of G and U: row i, 8 pairs per thread
      const int i = tid >> 2, k0 = (tid & 3) * 8;
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) {
        const int k = k0 + kk, p = pq[0][k], q = pq[1][k];
        const float tq = cs[0][k], s = cs[1][k];
        const float gp = G[i][p], gq = G[i][q];
        G[i][p] = gp - s * (gq + tq * gp);
        G[i][q] = gq + s * (gp - tq * gq);
        const float up = U[i][p], uq = U[i][q];
        U[i][p] = up - s * (uq + tq * up);
        U[i][q] = uq + s * (up - tq * uq);
      }
    }
    __syncthreads();
    {  // rows of G: column j, 8 pairs per thread
      const int j = tid & 63, k0 = (tid >> 6) * 8;
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) {
        const int k = k0 + kk, p = pq[0][k], q = pq[1][k];
        const float tq = cs[0][k], s = cs[1][k];
        const float gp = G[p][j], gq = G[q][j];
        G[p][j] = gp - s * (gq + tq * gp);
        G[q][j] = gq + s * (gp - tq * gq);
      }
    }
    __syncthreads();
  }
  float* Uout = F.U + (long long)pair * JP * JP;
  for (int e = tid; e < JP * JP; e += 256) Uout[e] = U[e >> 6][e & 63];
  if (tid == 0 && nrot) {
    atomicAdd(F.rotations, nrot);
    atomicAdd(F.rot_mass, nmass);
  }
}

// which: 0 -> A, 1 -> V.  Grid: (pairs of all factors, dpad_max/128 row slabs, 2)
__global__ __launch_bounds__(256) void jacobi_cols_kernel(const JacobiFactor* __restrict__ factors, int n_factors,
                                                         int round) {
  __shared__ __attribute__((aligned(16))) float Ps[JP][132];
  __shared__ __attribute__((aligned(16))) float Us[JP][JP + 4];
  const int fi = jacobi_locate(factors, n_factors, blockIdx.x);
  const JacobiFactor& F = factors[fi];
  if (*F.active == 0 || round >= F.nb - 1) return;
  const int r0 = blockIdx.y * 128;
  if (r0 >= F.dpad) return;
  float* __restrict__ Mx = blockIdx.z == 0 ? F.A : F.V;
  const int pair = blockIdx.x - F.pair_begin;
  const int2 ij = F.sched[round * (F.nb / 2) + pair];
  const float* __restrict__ Uin = F.U + (long long)pair * JP * JP;
  const int tid = threadIdx.x;
  const long long ld = F.dpad;
  for (int e = tid; e < JP * JP / 4; e += 256) {
    const int k = e >> 4, n4 = (e & 15) << 2;
    *reinterpret_cast<float4*>(&Us[k][n4]) = *reinterpret_cast<const float4*>(Uin + k * JP + n4);
  }
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int idx = tid + it * 256;
    const int row = idx >> 4, k = (idx & 15) << 2;
    const int gc = (k < JB ? ij.x * JB + k : ij.y * JB + k - JB);
    const float4 v = *reinterpret_cast<const float4*>(Mx + (long long)(r0 + row) * ld + gc);
    Ps[k + 0][row] = v.x;
    Ps[k + 1][row] = v.y;
    Ps[k + 2][row] = v.z;
    Ps[k + 3][row] = v.w;
  }
  __syncthreads();
  const int lane = tid & 63, w = tid >> 6, l32 = lane & 31, h = lane >> 5;
  floatx16 acc[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
#pragma unroll 8
  for (int ks = 0; ks < JP / 2; ++ks) {
    const int kr = 2 * ks + h;
    const float a = Ps[kr][32 * w + l32];
    acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, Us[kr][l32], acc[0], 0, 0, 0);
    acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, Us[kr][32 + l32], acc[1], 0, 0, 0);
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int gc = (j == 0 ? ij.x : ij.y) * JB + l32;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int row = r0 + 32 * w + 8 * (e >> 2) + 4 * h + (e & 3);
      Mx[(long long)row * ld + gc] = acc[j][e];
    }
  }
}

// A[I u J, c0:c0+128] <- U^T A[I u J, c0:c0+128].  Grid: (pairs, dpad_max/128 column slabs)
__global__ __launch_bounds__(256) void jacobi_rows_kernel(const JacobiFactor* __restrict__ factors, int n_factors,
                                                         int round) {
  __shared__ __attribute__((aligned(16))) float Ps[JP][132];
  __shared__ __attribute__((aligned(16))) float Us[JP][JP + 4];
  const int fi = jacobi_locate(factors, n_factors, blockIdx.x);
  const JacobiFactor& F = factors[fi];
  if (*F.active == 0 || round >= F.nb - 1) return;
  const int c0 = blockIdx.y * 128;
  if (c0 >= F.dpad) return;
  const int pair = blockIdx.x - F.pair_begin;
  const int2 ij = F.sched[round * (F.nb / 2) + pair];
  const float* __restrict__ Uin = F.U + (long long)pair * JP * JP;
  const int tid = threadIdx.x;
  const long long ld = F.dpad;
  for (int e = tid; e < JP * JP / 4; e += 256) {
    const int k = e >> 4, n4 = (e & 15) << 2;
    *reinterpret_cast<float4*>(&Us[k][n4]) = *reinterpret_cast<const float4*>(Uin + k * JP + n4);
  }
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int idx = tid + it * 256;
    const int k = idx >> 5, n4 = (idx & 31) << 2;
    const int gr = (k < JB ? ij.x * JB + k : ij.y * JB + k - JB);
    *reinterpret_cast<float4*>(&Ps[k][n4]) = *reinterpret_cast<const float4*>(F.A + (long long)gr * ld + c0 + n4);
  }
  __syncthreads();
  const int lane = tid & 63, w = tid >> 6, l32 = lane & 31, h = lane >> 5;
  floatx16 acc[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
#pragma unroll 8
  for (int ks = 0; ks < JP / 2; ++ks) {
    const int kr = 2 * ks + h;
    const float b = Ps[kr][32 * w + l32];
    acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(Us[kr][l32], b, acc[0], 0, 0, 0);
    acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(Us[kr][32 + l32], b, acc[1], 0, 0, 0);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int li = 8 * (e >> 2) + 4 * h + (e & 3);
      const int gr = (i == 0 ? ij.x : ij.y) * JB + li;
      F.A[(long long)gr * ld + c0 + 32 * w + l32] = acc[i][e];
    }
  }
}

// Eigenvalue post-processing of the reference's eigh root inverse, one workgroup per factor:
// lambda as left by the solver; if min(lambda) < eps: lambda <- (lambda - min) + eps (matrix_functions.py:256-264,
// two rounded additions); w = lambda^exponent.  Padded entries get weight 0.
struct EigFinal {
  const float* lambda_in;  // eigenvalue i at lambda_in[i * lambda_stride] (the diagonal of the diagonalised matrix, or a vector)
  long long lambda_stride;
  const float* V;      // eigenvectors (columns)
  float* Vs;           // V with column c scaled by w[c]
  float* lambda_out;   // dpad floats
  float* weight_out;   // dpad floats
  int d, dpad;
  float exponent;      // -1 / root
  int row_begin;       // first global 8-row slab of this factor (eig_scale_cols_kernel)
  int enabled;
  int scale_cols;      // eigenvectors are the columns of V: produce Vs (otherwise the caller scales rows)
};

// stability 1: epsilon was already added to the diagonal before the decomposition and the spectrum is shifted
// only if its minimum is still below epsilon; stability 0 (matrix_functions.py:265-271):
// lambda <- (lambda - min(lambda_min, 0)) + epsilon unconditionally; stability 2 (PseudoInverseConfig,
// matrix_functions.py:206-249): eigenvalues at or below max(rank_atol, rtol * max(lambda_max, 0)) get weight 0,
// rtol = rank_rtol, or d * 2^-23 when rank_rtol < 0 (the reference's None).
__global__ __launch_bounds__(256) void eig_weights_kernel(const EigFinal* __restrict__ jobs, float eps, int stability,
                                                         float rank_rtol, float rank_atol) {
  __shared__ float red[4], redmax[4];
  const EigFinal& J = jobs[blockIdx.x];
  if (!J.enabled) return;
  const int d = J.d, dpad = J.dpad;
  float m = 3.4028234663852886e38f, mx = -3.4028234663852886e38f;
  for (int i = threadIdx.x; i < d; i += 256) {
    const float l = J.lambda_in[i * J.lambda_stride];
    m = fminf(m, l);
    mx = fmaxf(mx, l);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    m = fminf(m, __shfl_xor(m, o, 64));
    mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) { red[wave] = m; redmax[wave] = mx; }
  __syncthreads();
  const float lam_min = fminf(fminf(red[0], red[1]), fminf(red[2], red[3]));
  const float lam_max = fmaxf(fmaxf(redmax[0], redmax[1]), fmaxf(redmax[2], redmax[3]));
  const bool pinv = stability == 2;
  const bool shift = pinv ? false : (stability == 1 ? (lam_min < eps) : true);
  const float first = (stability == 1) ? -lam_min : -fminf(lam_min, 0.0f);
  const float rtol = (rank_rtol < 0.0f) ? (float)d * 1.1920929e-7f : rank_rtol;
  const float cutoff = fmaxf(rtol * fmaxf(lam_max, 0.0f), rank_atol);
  for (int i = threadIdx.x; i < dpad; i += 256) {
    float lam = 0.0f, wgt = 0.0f;
    if (i < d) {
      lam = J.lambda_in[i * J.lambda_stride];
      if (shift) {
        if (first != 0.0f) lam = lam + first;
        if (eps != 0.0f) lam = lam + eps;
      }
      wgt = (pinv && lam <= cutoff) ? 0.0f : powf(lam, J.exponent);
    }
    J.lambda_out[i] = lam;
    J.weight_out[i] = wgt;
  }
}

// Vs[r][c] = V[r][c] * w[c]; one workgroup per 8 rows of one factor.
__global__ __launch_bounds__(256) void eig_scale_cols_kernel(const EigFinal* __restrict__ jobs, int n_jobs) {
  int lo = 0, hi = n_jobs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (jobs[mid].row_begin <= (int)blockIdx.x) lo = mid; else hi = mid - 1;
  }
  const EigFinal& J = jobs[lo];
  if (!J.enabled || !J.scale_cols) return;
  const int dpad = J.dpad;
  const int r0 = (blockIdx.x - J.row_begin) * 8;
  for (int e = threadIdx.x * 4; e < 8 * dpad; e += 256 * 4) {
    const int r = r0 + e / dpad, c = e % dpad;
    const float4 v = *reinterpret_cast<const float4*>(J.V + (long long)r * dpad + c);
    const float4 w = *reinterpret_cast<const float4*>(J.weight_out + c);
    *reinterpret_cast<float4*>(J.Vs + (long long)r * dpad + c) = make_float4(v.x * w.x, v.y * w.y, v.z * w.z, v.w * w.w);
  }
}

// Stable ascending order of the eigenvalues of one factor (ties keep their index order, like
// torch.linalg.eigh's ascending output up to degenerate pairs): order[k] = index of the k-th smallest.
// One workgroup per factor.
struct RankJob {
  const float* lambda_in;
  long long lambda_stride;
  int* order;
  int d;
};
__global__ __launch_bounds__(256) void eig_rank_kernel(const RankJob* __restrict__ jobs) {
  const RankJob& J = jobs[blockIdx.x];
  const int d = J.d;
  for (int i = threadIdx.x; i < d; i += 256) {
    const float x = J.lambda_in[i * J.lambda_stride];
    int rank = 0;
    for (int j = 0; j < d; ++j) {
      const float y = J.lambda_in[j * J.lambda_stride];
      rank += (y < x || (y == x && j < i)) ? 1 : 0;
    }
    J.order[rank] = i;
  }
}

// out[k] = base[(order ? order[k] : k) * stride]
__global__ __launch_bounds__(256) void gather_strided_kernel(const float* __restrict__ base, long long stride,
                                                            const int* __restrict__ order, float* __restrict__ out, int n) {
  const int k = blockIdx.x * 256 + threadIdx.x;
  if (k < n) out[k] = base[(long long)(order ? order[k] : k) * stride];
}

// dst[r][k] = src[order[k]][r]: eigenvectors held as rows become sorted columns.  32 x 32 tiles through LDS,
// grid (ceil(d / 32), ceil(d / 32), factors).
struct RowsToCols {
  const float* src;
  float* dst;
  const int* order;
  long long lds_, ldd;
  int d;
};
__global__ __launch_bounds__(256) void rows_to_sorted_cols_kernel(const RowsToCols* __restrict__ jobs) {
  __shared__ float tile[32][33];
  const RowsToCols& J = jobs[blockIdx.z];
  const int d = J.d;
  const int k0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
  if (k0 >= d || r0 >= d) return;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  for (int kk = ty; kk < 32; kk += 8) {
    const int k = k0 + kk, r = r0 + tx;
    float v = 0.f;
    if (k < d && r < d) {
      const int row = min(max(J.order[k], 0), d - 1);  // clamp: a NaN spectrum leaves ranks undefined
      v = J.src[row * J.lds_ + r];
    }
    tile[kk][tx] = v;
  }
  __syncthreads();
  for (int rr = ty; rr < 32; rr += 8) {
    const int r = r0 + rr, k = k0 + tx;
    if (r < d && k < d) J.dst[r * J.ldd + k] = tile[tx][rr];
  }
}

// dense <- packed / bc2 (+ eps on the diagonal), V <- I : start of an eigendecomposition.
struct EigInit {
  const float* packed;
  const float* scale;  // optional per-factor multiplier applied after the division by bc2 (trace scaling)
  float* A;
  float* V;  // optional
  int d, dpad;
  int tile_begin;  // first 64 x 64 tile id of this factor (full grid, not triangular)
  int tiles;       // dpad / 64
  int enabled;
};

__global__ __launch_bounds__(256) void eig_init_kernel(const EigInit* __restrict__ jobs, int n_jobs, float bc2, float eps) {
  int lo = 0, hi = n_jobs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (jobs[mid].tile_begin <= (int)blockIdx.x) lo = mid; else hi = mid - 1;
  }
  const EigInit& J = jobs[lo];
  if (!J.enabled) return;
  const int t = blockIdx.x - J.tile_begin;
  const int bi = t / J.tiles, bj = t % J.tiles;
  const int d = J.d, dpad = J.dpad;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  // the packed rows are read along themselves: a tile below the diagonal reads its mirror image and turns it in LDS
  __shared__ float tile[64][65];
  const int r0 = 64 * min(bi, bj), c0 = 64 * max(bi, bj);
  for (int rr = ty; rr < 64; rr += 4) {
    const int r = r0 + rr, c = c0 + tx;
    float v = 0.0f;
    if (r < d && c < d && c >= r) {
      v = J.packed[(long long)r * d - ((long long)r * (r - 1)) / 2 + (c - r)] / bc2;
      if (J.scale != nullptr) v = v * J.scale[0];
      if (r == c && eps != 0.0f) v = v + eps;
    }
    tile[rr][tx] = v;
  }
  __syncthreads();
  for (int rr = ty; rr < 64; rr += 4) {
    const int r = bi * 64 + rr, c = bj * 64 + tx;
    const bool as_read = bi < bj || (bi == bj && tx >= rr);
    J.A[(long long)r * dpad + c] = as_read ? tile[rr][tx] : tile[tx][rr];
    if (J.V != nullptr) J.V[(long long)r * dpad + c] = (r == c) ? 1.0f : 0.0f;
  }
}

}  // namespace sa
