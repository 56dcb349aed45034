// Batched blocked Householder QR for the eigenbasis refresh of eigenvalue-corrected Shampoo.
//
// One refresh factors B = Q^T A Q (d x d) for every factor at once.  Columns are processed in panels;
// a panel (all rows below the diagonal x up to 32 columns) is factored by ONE workgroup entirely in LDS
// (up to 135 KB of the 160 KB a CU has), producing the Householder vectors V (unit lower trapezoid) and
// the triangular factor T of the compact WY form H_1...H_k = I - V T V^T.  Panels are gathered into outer
// blocks of up to QR_OUTER columns: a panel's reflectors are applied at once only to the rest of its outer block,
// its (V, T) is merged into the block's (T12 = -T1 (V1^T V2) T2), and the trailing matrix and the accumulated
// eigenbasis are updated once per outer block with the grouped MFMA GEMM (EPI_SUB), k = block width.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm.h"

namespace sa {

constexpr int QR_MAX_PANEL = 32;
constexpr int QR_OUTER = 128;
constexpr int QR_THREADS = 1024;

struct QrPanel {
  const float* B;   // matrix being factored, row stride ldb
  float* V;         // this panel's column block of the outer block's V (row stride ldv): `top` rows of zeros, then
                    // rows x pcols Householder vectors (unit diagonal, zeros above)
  float* T;         // this panel's column block of the outer block's T (row stride ldt, t_rows rows): the pcols x pcols
                    // upper triangular factor at rows [top, top + pcols), zeros elsewhere
  long long ldb;
  int d;            // matrix dimension
  int j0;           // first column / row of the panel
  int pcols;        // columns in this panel
  int ldv, ldt;
  int top;          // columns of the outer block before this panel
  int t_rows;       // width of the outer block
  const int* active;
};

// dynamic LDS: rows * (pcols + 1) floats for the panel.  1024 threads: a panel of 1024 rows is one row per thread, and four
// waves per SIMD hide the LDS latency of the column-by-column sweeps.
__global__ __launch_bounds__(QR_THREADS) void qr_panel_kernel(const QrPanel* __restrict__ jobs) {
  extern __shared__ float lds[];
  constexpr int NW = QR_THREADS / 64;
  __shared__ float wred[NW][QR_MAX_PANEL];
  __shared__ float wfin[QR_MAX_PANEL];
  __shared__ float tau_s[QR_MAX_PANEL];
  __shared__ float S[QR_MAX_PANEL][QR_MAX_PANEL + 1];
  __shared__ float Tm[QR_MAX_PANEL][QR_MAX_PANEL + 1];
  __shared__ float bcast[2];
  const QrPanel& J = jobs[blockIdx.x];
  if (J.active != nullptr && *J.active == 0) return;
  const int rows = J.d - J.j0, pc = J.pcols, st = pc + 1;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float* P = lds;
  for (int e = tid; e < rows * pc; e += QR_THREADS) {
    const int r = e / pc, c = e - r * pc;
    P[r * st + c] = J.B[(long long)(J.j0 + r) * J.ldb + J.j0 + c];
  }
  __syncthreads();
  for (int c = 0; c < pc; ++c) {
    // --- Householder vector of column c (LAPACK slarfg): rows c..rows-1
    float part = 0.f;
    for (int r = c + 1 + tid; r < rows; r += QR_THREADS) { const float x = P[r * st + c]; part += x * x; }
    part = wave_sum(part);
    if (lane == 0) wred[wave][0] = part;
    __syncthreads();
    if (tid == 0) {
      float sigma2 = 0.f;
      for (int w = 0; w < NW; ++w) sigma2 += wred[w][0];
      const float alpha = (c < rows) ? P[c * st + c] : 0.f;
      float tau = 0.f, scale = 0.f, beta = alpha;
      if (sigma2 != 0.f && c < rows) {
        beta = -copysignf(sqrtf(alpha * alpha + sigma2), alpha);
        tau = (beta - alpha) / beta;
        scale = 1.0f / (alpha - beta);
      }
      tau_s[c] = tau;
      bcast[0] = scale;
      bcast[1] = beta;
    }
    __syncthreads();
    const float scale = bcast[0], tau = tau_s[c];
    for (int r = c + 1 + tid; r < rows; r += QR_THREADS) P[r * st + c] *= scale;
    if (tid == 0 && c < rows) P[c * st + c] = bcast[1];
    __syncthreads();
    if (tau != 0.f) {
      // --- apply H_c to the remaining panel columns: w = v^T P[:, c'] ; P[:, c'] -= tau w v
      for (int cc = c + 1; cc < pc; ++cc) {
        float w = 0.f;
        for (int r = c + 1 + tid; r < rows; r += QR_THREADS) w += P[r * st + c] * P[r * st + cc];
        w = wave_sum(w);
        if (lane == 0) wred[wave][cc] = w;
      }
      __syncthreads();
      if (tid < pc - (c + 1)) {
        // row c itself (v[c] = 1) is this thread's alone
        const int cc = c + 1 + tid;
        float w = 0.f;
        for (int k = 0; k < NW; ++k) w += wred[k][cc];
        w = tau * (P[c * st + cc] + w);
        wfin[cc] = w;
        P[c * st + cc] -= w;
      }
      __syncthreads();
      for (int r = c + 1 + tid; r < rows; r += QR_THREADS) {
        const float v = P[r * st + c];
        for (int cc = c + 1; cc < pc; ++cc) P[r * st + cc] -= wfin[cc] * v;
      }
      __syncthreads();
    }
  }
  // --- S = V^T V (strict upper part), v_k has an implicit 1 at row k and zeros above
  for (int e = tid; e < pc * pc; e += QR_THREADS) {
    const int i = e / pc, k = e - i * pc;
    float acc = 0.f;
    if (i < k && k < rows) {
      acc = P[k * st + i];  // v_i[k] * v_k[k] with v_k[k] = 1
      for (int r = k + 1; r < rows; ++r) acc += P[r * st + i] * P[r * st + k];
    }
    S[i][k] = acc;
  }
  for (int e = tid; e < QR_MAX_PANEL * QR_MAX_PANEL; e += QR_THREADS) Tm[e / QR_MAX_PANEL][e % QR_MAX_PANEL] = 0.f;
  __syncthreads();
  // --- T (LAPACK slarft, forward columnwise): T[i][i] = tau_i, T[0:i, i] = -tau_i T[0:i,0:i] S[0:i, i]
  for (int i = 0; i < pc; ++i) {
    if (tid < i) {
      float acc = 0.f;
      for (int m = tid; m < i; ++m) acc += Tm[tid][m] * S[m][i];
      Tm[tid][i] = -tau_s[i] * acc;
    }
    if (tid == i) Tm[i][i] = tau_s[i];
    __syncthreads();
  }
  for (int e = tid; e < J.t_rows * pc; e += QR_THREADS) {
    const int r = e / pc, c = e - r * pc, i = r - J.top;
    J.T[(long long)r * J.ldt + c] = (i >= 0 && i < pc) ? Tm[i][c] : 0.f;
  }
  for (int e = tid; e < (J.top + rows) * pc; e += QR_THREADS) {
    const int rr = e / pc, c = e - rr * pc, r = rr - J.top;
    float v = 0.f;
    if (r >= 0) v = (r > c) ? P[r * st + c] : (r == c ? 1.0f : 0.0f);
    J.V[(long long)rr * J.ldv + c] = v;
  }
}

// Sums of the 32 values x q[i] over the 64 lanes of a wavefront: at every stage a lane keeps one half of its values and
// trades the other half with the lane whose index differs in one bit.  The first two stages (bits 5 and 4) are the lane
// swaps of gfx950, v_permlane32_swap and v_permlane16_swap, which exchange the upper half of one register with the lower
// half of another (of every 32 lanes, of every 16): one instruction per pair of values and no trip through LDS.  On
// return lane l holds the total of value (l >> 1).
typedef unsigned qr_uint2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float wave_sum32(const float (&q)[32], float x, int lane) {
  float a[16], b[8], c[4], d[2];
  const bool h3 = lane & 8, h2 = lane & 4, h1 = lane & 2;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    // lanes 0-31 end up with both halves' value i, lanes 32-63 with both halves' value i + 16
    const qr_uint2 t = __builtin_amdgcn_permlane32_swap(__float_as_uint(x * q[i]), __float_as_uint(x * q[i + 16]), false, false);
    a[i] = __uint_as_float(t.x) + __uint_as_float(t.y);
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    // even rows of 16 lanes end up with value i of both rows, odd rows with value i + 8
    const qr_uint2 t = __builtin_amdgcn_permlane16_swap(__float_as_uint(a[i]), __float_as_uint(a[i + 8]), false, false);
    b[i] = __uint_as_float(t.x) + __uint_as_float(t.y);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) c[i] = (h3 ? b[i + 4] : b[i]) + __shfl_xor(h3 ? b[i] : b[i + 4], 8);
#pragma unroll
  for (int i = 0; i < 2; ++i) d[i] = (h2 ? c[i + 2] : c[i]) + __shfl_xor(h2 ? c[i] : c[i + 2], 4);
  float e = (h1 ? d[1] : d[0]) + __shfl_xor(h1 ? d[0] : d[1], 2);
  return e + __shfl_xor(e, 1);
}

// The same factorisation with the panel in registers: thread t holds row t of the panel, 32 columns, so the panel has at
// most 1024 rows, and j0 is a multiple of 32.  Column k needs the products of column k below the diagonal with EVERY
// column of the panel: with the columns to its right they give the update of the panel, with itself the norm, with the
// columns to its left (Householder vectors by then) the entries of V^T V that the triangular factor is built from.  None
// of them needs the scaling of the vector, so one reduction of 32 values and two barriers do a column.  The registers of a
// row form a ring that turns by one column per step: the current column is always ring[0], so the loop stays rolled (its
// unrolled form, 100 KB of straight-line code run once, is bound by instruction fetches) and after 32 steps every column
// is back in its place.  Writes V and T like qr_panel_kernel.
__global__ __launch_bounds__(QR_THREADS, 8) void qr_panel_rows_kernel(const QrPanel* __restrict__ jobs) {
  constexpr int NW = QR_THREADS / 64, PW = QR_MAX_PANEL;
  __shared__ float wred[NW][PW];
  __shared__ float rowk[PW];
  __shared__ __align__(16) float wfin[PW];
  __shared__ float tau_s[PW];
  __shared__ float S[PW][PW + 1];
  __shared__ float Tm[PW][PW + 1];
  __shared__ float bcast[2];
  const QrPanel& J = jobs[blockIdx.x];
  if (J.active != nullptr && *J.active == 0) return;
  const int rows = J.d - J.j0, pc = J.pcols;
  const int r = threadIdx.x, lane = r & 63, wave = r >> 6;
  const int waves_with_rows = min(NW, (rows + 63) / 64);
  float ring[PW];
  if (r < rows) {
    const float4* src = reinterpret_cast<const float4*>(J.B + (long long)(J.j0 + r) * J.ldb + J.j0);
#pragma unroll
    for (int c4 = 0; c4 < PW / 4; ++c4) {
      const float4 x = src[c4];
      ring[4 * c4 + 0] = (4 * c4 + 0 < pc) ? x.x : 0.f;
      ring[4 * c4 + 1] = (4 * c4 + 1 < pc) ? x.y : 0.f;
      ring[4 * c4 + 2] = (4 * c4 + 2 < pc) ? x.z : 0.f;
      ring[4 * c4 + 3] = (4 * c4 + 3 < pc) ? x.w : 0.f;
    }
  } else {
#pragma unroll
    for (int c = 0; c < PW; ++c) ring[c] = 0.f;
  }
  if (lane < PW) wred[wave][lane] = 0.f;
  for (int e = r; e < PW * (PW + 1); e += QR_THREADS) { (&S[0][0])[e] = 0.f; (&Tm[0][0])[e] = 0.f; }
  __syncthreads();
#pragma unroll 1
  for (int k = 0; k < PW; ++k) {
    // ring[i] is column (k + i) mod 32: the current one, those to its right, then the finished ones
    if (k < pc) {  // the same for every thread
      if (wave < waves_with_rows) {
        const float x = (r > k) ? ring[0] : 0.f;  // rows beyond the panel hold zeros
        const float total = wave_sum32(ring, x, lane);
        if ((lane & 1) == 0) wred[wave][lane >> 1] = total;
      }
      if (r == k) {
#pragma unroll
        for (int i = 0; i < PW; ++i) rowk[i] = ring[i];
      }
      __syncthreads();
      if (wave == 0) {
        const int i = lane & (PW - 1), j = (k + i) & (PW - 1);  // ring position and the column it holds
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) s += wred[w][i];  // wavefronts without rows left their zeros there
        const float sigma2 = __shfl(s, 0);
        const float alpha = rowk[0], x = rowk[i];
        float tau = 0.f, scale = 0.f, beta = alpha;
        if (sigma2 != 0.f) {  // LAPACK slarfg
          beta = -copysignf(sqrtf(alpha * alpha + sigma2), alpha);
          tau = (beta - alpha) / beta;
          scale = 1.0f / (alpha - beta);
        }
        if (lane < PW) {
          wfin[i] = (j > k) ? tau * (x + scale * s) : 0.f;  // tau v^T P[:, j] with v = (1, scale x); finished columns stay
          if (j < k) S[j][k] = x + scale * s;               // v_j^T v_k
          if (j == k) { tau_s[k] = tau; bcast[0] = scale; bcast[1] = beta; }
        }
      }
      __syncthreads();
      if (r >= k) {
        const float v = (r > k) ? ring[0] * bcast[0] : 1.0f;
        ring[0] = (r > k) ? v : bcast[1];
#pragma unroll
        for (int i = 1; i < PW; ++i) ring[i] -= wfin[i] * v;
      }
    }
    const float first = ring[0];
#pragma unroll
    for (int i = 0; i < PW - 1; ++i) ring[i] = ring[i + 1];
    ring[PW - 1] = first;
  }
  // --- T (LAPACK slarft, forward columnwise): T[i][i] = tau_i, T[0:i, i] = -tau_i T[0:i,0:i] S[0:i, i]
  for (int i = 0; i < pc; ++i) {
    if (r < i) {
      float acc = 0.f;
      for (int m = r; m < i; ++m) acc += Tm[r][m] * S[m][i];
      Tm[r][i] = -tau_s[i] * acc;
    }
    if (r == i) Tm[i][i] = tau_s[i];
    __syncthreads();
  }
  for (int e = r; e < J.t_rows * pc; e += QR_THREADS) {
    const int tr = e / pc, c = e - tr * pc, i = tr - J.top;
    J.T[(long long)tr * J.ldt + c] = (i >= 0 && i < pc) ? Tm[i][c] : 0.f;
  }
  for (int e = r; e < J.top * pc; e += QR_THREADS) J.V[(long long)(e / pc) * J.ldv + e % pc] = 0.f;
  if (r < rows) {
    float* dst = J.V + (long long)(J.top + r) * J.ldv;
    float v[PW];
#pragma unroll
    for (int c = 0; c < PW; ++c) v[c] = (r > c) ? ring[c] : (r == c ? 1.0f : 0.0f);
    if (pc == PW && (J.ldv & 3) == 0 && (reinterpret_cast<uintptr_t>(J.V) & 15) == 0) {
#pragma unroll
      for (int c4 = 0; c4 < PW / 4; ++c4)
        reinterpret_cast<float4*>(dst)[c4] = make_float4(v[4 * c4], v[4 * c4 + 1], v[4 * c4 + 2], v[4 * c4 + 3]);
    } else {
#pragma unroll
      for (int c = 0; c < PW; ++c)
        if (c < pc) dst[c] = v[c];
    }
  }
}

// Generic strided 2-D copy: dst[r][c] = src[r][c]
struct Copy2D {
  const float* src;
  float* dst;
  long long lds_, ldd;
  int rows, cols;
  const int* perm;  // optional: dst[r][c] = src[r][perm[c]]
};
__global__ __launch_bounds__(256) void copy2d_kernel(const Copy2D* __restrict__ jobs) {
  const Copy2D& J = jobs[blockIdx.y];
  const long long n = (long long)J.rows * J.cols;
  for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < n; e += (long long)gridDim.x * 256) {
    const int r = (int)(e / J.cols), c = (int)(e % J.cols);
    const int sc = J.perm ? min(max(J.perm[c], 0), J.cols - 1) : c;  // clamp: a NaN spectrum leaves ranks undefined
    J.dst[r * J.ldd + c] = J.src[r * J.lds_ + sc];
  }
}

// Per factor: sum of squares of all entries and of the diagonal of a d x d matrix (criterion of
// matrix_functions.py:772-797); one workgroup per factor.
struct NormPair {
  const float* B;
  float* out_all;   // sum B^2
  float* out_diag;  // sum diag(B)^2
  long long ldb;
  int d;
};
constexpr int FACTOR_PASS_THREADS = 1024;  // one workgroup per factor: 16 waves to cover the latency of its d x d sweep
__global__ __launch_bounds__(FACTOR_PASS_THREADS) void diag_off_norm_kernel(const NormPair* __restrict__ jobs) {
  constexpr int NW = FACTOR_PASS_THREADS / 64;
  __shared__ float red[2][NW];
  const NormPair& J = jobs[blockIdx.x];
  float a = 0.f, dg = 0.f;
  const long long n = (long long)J.d * J.d;
  for (long long e = threadIdx.x; e < n; e += FACTOR_PASS_THREADS) {
    const int r = (int)(e / J.d), c = (int)(e % J.d);
    const float v = J.B[r * J.ldb + c];
    a += v * v;
    if (r == c) dg += v * v;
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  a = wave_sum(a);
  dg = wave_sum(dg);
  if (lane == 0) { red[0][wave] = a; red[1][wave] = dg; }
  __syncthreads();
  if (threadIdx.x == 0) {
    float ta = 0.f, td = 0.f;
    for (int w = 0; w < NW; ++w) { ta += red[0][w]; td += red[1][w]; }
    *J.out_all = ta;
    *J.out_diag = td;
  }
}

// Rayleigh quotients ev[i] = sum_r Q[r][i] * Y[r][i], stable ascending rank of ev, and its inverse
// permutation: order[k] = index of the k-th smallest (ties keep their original order, like
// torch.sort(stable=True), matrix_functions.py:849).  One workgroup per factor, d <= 4096.
struct SortJob {
  const float* Q;
  const float* Y;
  float* ev;     // d floats
  int* order;    // d ints
  long long ldq, ldy;
  int d;
};
__global__ __launch_bounds__(FACTOR_PASS_THREADS) void rayleigh_sort_kernel(const SortJob* __restrict__ jobs) {
  const SortJob& J = jobs[blockIdx.x];
  const int d = J.d;
  for (int i = threadIdx.x; i < d; i += FACTOR_PASS_THREADS) {
    float acc = 0.f;
    for (int r = 0; r < d; ++r) acc += J.Q[r * J.ldq + i] * J.Y[r * J.ldy + i];
    J.ev[i] = acc;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < d; i += FACTOR_PASS_THREADS) {
    const float x = J.ev[i];
    int rank = 0;
    for (int j = 0; j < d; ++j) {
      const float y = J.ev[j];
      rank += (y < x || (y == x && j < i)) ? 1 : 0;
    }
    J.order[rank] = i;
  }
}

}  // namespace sa
