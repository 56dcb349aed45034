// Batched symmetric eigendecomposition through tridiagonalisation, for factors too large for the
// block-Jacobi solver to be competitive.
//
//   1. A = Q1 T Q1^T: blocked Householder tridiagonalisation (LAPACK sytrd/latrd recurrences).  Per column
//      one single-workgroup kernel per factor (pending panel corrections, Householder vector, the w vector
//      of the previous column) and one symmetric matrix-vector product over the trailing matrix, which is
//      the HBM-bound part ((4/3) d^3 bytes per factor); per 32-column panel one rank-64 trailing update
//      A -= [V W] [W V]^T on the grouped MFMA GEMM.
//   2. Y = Q1^T by compact-WY block reflectors (grouped GEMMs).
//   3. T = Z diag(lambda) Z^T by implicit QL iteration.  One wavefront per factor runs the bulge chases, several
//      shifted sweeps at a time pipelined across its lanes, and logs the rotations of up to TQL_K sweeps; a
//      second kernel applies that chunk of sweeps to the rows of Y as a register-resident systolic pipeline
//      (one thread per column of Y, one carried row per sweep), so Y is read and written once per chunk
//      instead of once per sweep.
// On exit row i of Y is the eigenvector of eigenvalue diag[i] (not sorted).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm.h"

namespace sa {

typedef float vfloat4_t __attribute__((ext_vector_type(4)));
typedef float vfloat2_t __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(1))) vfloat2_t global_float2;

constexpr int TRD_NB = 32;               // panel width
constexpr int TRD_PW = 2 * TRD_NB;       // row length of the [V | W] and [W | V] panel buffers
constexpr int TRD_COL_THREADS = 1024;
constexpr int TRD_ROWS_PER_THREAD = 8;   // d <= 8192
constexpr int TRD_MAX_DIM = TRD_COL_THREADS * TRD_ROWS_PER_THREAD;
constexpr int TQL_K = 32;                // sweeps per chunk
constexpr int TQL_STEPS = 64;            // pipeline steps whose coefficients are staged in LDS at a time
constexpr int TQL_HDR = 4 + 2 * TQL_K;   // ints per chunk header: nsweeps, top, bot, -, l[K], m[K]

struct TrdJob {
  float* A;       // dpad x dpad, symmetric, both triangles kept current
  float* Y;       // dpad x dpad
  float* Vall;    // dpad x dpad, column j = Householder vector of column j (explicit unit entry, zeros above)
  float* P1;      // dpad x 64: [V | W] of the current panel
  float* P2;      // dpad x 64: [W | V]
  float* vbuf;    // dpad: current Householder vector, zero at and above the diagonal
  float* ybuf;    // dpad: trailing matrix times vbuf
  float* part;    // (dpad / 64)^2 x 4 x 64: transposed tile contributions of the symmetric product
  float* diag;    // dpad
  float* off;     // dpad: off[j] couples j and j + 1
  float* tau;     // dpad
  double* qd;     // dpad: diagonal of the (unit-scaled) tridiagonal matrix during the QL iteration
  double* qe;     // dpad: its off-diagonal
  float* Tmat;    // (dpad / 32) x 32 x 32 triangular factors of the block reflectors
  float2* rot;    // 2 x TQL_K x dpad rotation log (c, s)
  int* hdr;       // 2 x TQL_HDR
  int* state;     // l, -, done, failed, total sweeps, bits of the scale
  int d, dpad;
};

__device__ __forceinline__ float block_sum_1024(float v, float* red) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int k = 0; k < TRD_COL_THREADS / 64; ++k) t += red[k];
  return t;
}

// P1 and P2 are adjacent: 2 * dpad * 64 floats
__global__ __launch_bounds__(256) void trd_clear_panel_kernel(const TrdJob* __restrict__ jobs) {
  const TrdJob& J = jobs[blockIdx.y];
  const long long n4 = (long long)J.dpad * TRD_PW * 2 / 4;
  float4* dst = reinterpret_cast<float4*>(J.P1);
  for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < n4; e += (long long)gridDim.x * 256)
    dst[e] = make_float4(0.f, 0.f, 0.f, 0.f);
}

// Two dot products over the first 4 * nq4 panel columns of one row of the [V | W] buffer:
//   d1 = sum_q V[r][q] t1[q] + W[r][q] t2[q]      (correction of w)
//   d2 = sum_q V[r][q] rowW[q] + W[r][q] rowV[q]  (correction of the next column)
__device__ __forceinline__ void panel_row_dots(const float* __restrict__ row, int nq4, const float* t1, const float* t2,
                                               const float* rowV, const float* rowW, float& d1, float& d2) {
  d1 = 0.f;
  d2 = 0.f;
  for (int q4 = 0; q4 < nq4; ++q4) {
    const float4 v = *reinterpret_cast<const float4*>(row + 4 * q4);
    const float4 w = *reinterpret_cast<const float4*>(row + TRD_NB + 4 * q4);
    const int q = 4 * q4;
    d1 += (v.x * t1[q] + v.y * t1[q + 1]) + (v.z * t1[q + 2] + v.w * t1[q + 3]);
    d1 += (w.x * t2[q] + w.y * t2[q + 1]) + (w.z * t2[q + 2] + w.w * t2[q + 3]);
    d2 += (v.x * rowW[q] + v.y * rowW[q + 1]) + (v.z * rowW[q + 2] + v.w * rowW[q + 3]);
    d2 += (w.x * rowV[q] + w.y * rowV[q + 1]) + (w.z * rowV[q + 2] + w.w * rowV[q + 3]);
  }
}

// One column step of the panel reduction (LAPACK slatrd), one workgroup per factor.
// flags bit 0: finish w of column j - 1 (needs ybuf of that column); bit 1: start column j (Householder vector).
// Panel columns are p0 .. p0 + 31.  Both parts walk the same rows r >= j of the [V | W] buffer, so one pass
// yields the correction of w and the pending rank-2k correction of column j.
__global__ __launch_bounds__(TRD_COL_THREADS) void trd_column_kernel(const TrdJob* __restrict__ jobs, int j, int p0,
                                                                    int flags) {
  __shared__ float part1[32][33];
  __shared__ float part2[32][33];
  __shared__ float t1[TRD_NB], t2[TRD_NB], rowV[TRD_NB], rowW[TRD_NB];
  __shared__ float red[TRD_COL_THREADS / 64];
  __shared__ float bc[3];
  const TrdJob& J = jobs[blockIdx.x];
  const int d = J.d;
  if (j >= d) return;
  const int tid = threadIdx.x;
  const long long ld = J.dpad;
  float* __restrict__ P1 = J.P1;
  float* __restrict__ P2 = J.P2;
  const bool fin = (flags & 1) != 0, start = (flags & 2) != 0;
  const int jp = j - 1;
  const int ip = fin ? jp - p0 : j - p0;  // panel columns complete on entry
  const int nq4 = (ip + 3) / 4;
  const float tau_p = fin ? J.tau[jp] : 0.f;

  if (tid < TRD_NB) {
    t1[tid] = 0.f;
    t2[tid] = 0.f;
    rowV[tid] = (start && tid < ip) ? P1[(long long)j * TRD_PW + tid] : 0.f;
    rowW[tid] = (start && tid < ip) ? P1[(long long)j * TRD_PW + TRD_NB + tid] : 0.f;
  }
  if (fin && ip > 0) {  // t1 = W^T v, t2 = V^T v over the ip complete columns
    const int q = tid & 31, g = tid >> 5;
    float a1 = 0.f, a2 = 0.f;
    if (q < ip)
      for (int r = j + g; r < d; r += 32) {
        const float vr = J.vbuf[r];
        a1 += P1[(long long)r * TRD_PW + TRD_NB + q] * vr;
        a2 += P1[(long long)r * TRD_PW + q] * vr;
      }
    part1[g][q] = a1;
    part2[g][q] = a2;
    __syncthreads();
    if (tid < TRD_NB) {
      float s1 = 0.f, s2 = 0.f;
      for (int k = 0; k < 32; ++k) { s1 += part1[k][tid]; s2 += part2[k][tid]; }
      t1[tid] = s1;
      t2[tid] = s2;
    }
  }
  __syncthreads();

  // ---- one pass over the rows r >= j
  float wreg[TRD_ROWS_PER_THREAD], vreg[TRD_ROWS_PER_THREAD], areg[TRD_ROWS_PER_THREAD];
  float dot = 0.f;
#pragma unroll
  for (int k = 0; k < TRD_ROWS_PER_THREAD; ++k) {
    const int r = j + tid + k * TRD_COL_THREADS;
    float w = 0.f, vr = 0.f, a = 0.f;
    if (r < d) {
      float d1, d2;
      panel_row_dots(P1 + (long long)r * TRD_PW, nq4, t1, t2, rowV, rowW, d1, d2);
      if (fin) {
        vr = J.vbuf[r];
        w = tau_p * (J.ybuf[r] - d1);  // w = tau (y - V (W^T v) - W (V^T v))
        dot += w * vr;
      }
      // column j as it stands after the reflectors of this panel (row j of A is the same by symmetry)
      if (start) a = J.A[(long long)r * ld + j] - d2;
    }
    wreg[k] = w;
    vreg[k] = vr;
    areg[k] = a;
  }
  if (fin) {
    const float alpha = -0.5f * tau_p * block_sum_1024(dot, red);
#pragma unroll
    for (int k = 0; k < TRD_ROWS_PER_THREAD; ++k) {
      const int r = j + tid + k * TRD_COL_THREADS;
      if (r < d) {
        const float w = wreg[k] + alpha * vreg[k];
        wreg[k] = w;
        P1[(long long)r * TRD_PW + TRD_NB + ip] = w;
        P2[(long long)r * TRD_PW + ip] = w;
      }
    }
    if (tid == 0) bc[2] = wreg[0];  // w at row j
    __syncthreads();
    if (start) {  // the column just completed also corrects column j: V[r][ip] W[j][ip] + W[r][ip] V[j][ip]
      const float wj = bc[2], vj = 1.0f;  // the Householder vector of column j - 1 has its unit entry at row j
#pragma unroll
      for (int k = 0; k < TRD_ROWS_PER_THREAD; ++k) areg[k] -= vreg[k] * wj + wreg[k] * vj;
    }
  }

  if (start) {
    const int i = j - p0;
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < TRD_ROWS_PER_THREAD; ++k) {
      const int r = j + tid + k * TRD_COL_THREADS;
      if (r < d && r > j + 1) ss += areg[k] * areg[k];
    }
    const float sigma2 = block_sum_1024(ss, red);
    if (tid == 0) bc[0] = areg[0];
    if (tid == 1) bc[1] = areg[0];
    __syncthreads();
    const float ajj = bc[0];
    const float alpha0 = (j + 1 < d) ? bc[1] : 0.f;
    float tau = 0.f, beta = alpha0, scale = 0.f;
    if (sigma2 != 0.f) {  // LAPACK slarfg
      beta = -copysignf(sqrtf(alpha0 * alpha0 + sigma2), alpha0);
      tau = (beta - alpha0) / beta;
      scale = 1.0f / (alpha0 - beta);
    }
    if (tid == 0) {
      J.diag[j] = ajj;
      if (j + 1 < d) { J.off[j] = beta; J.tau[j] = tau; }
    }
    if (tid < 4 && j - tid >= 0) J.vbuf[j - tid] = 0.f;  // the product kernel starts at a 16-byte boundary
#pragma unroll
    for (int k = 0; k < TRD_ROWS_PER_THREAD; ++k) {
      const int r = j + tid + k * TRD_COL_THREADS;
      if (r < d && r > j) {
        const float v = (r == j + 1) ? 1.0f : areg[k] * scale;
        J.vbuf[r] = v;
        P1[(long long)r * TRD_PW + i] = v;
        P2[(long long)r * TRD_PW + TRD_NB + i] = v;
        J.Vall[(long long)r * ld + j] = v;
      }
    }
  }
}

// ybuf = (trailing matrix) x vbuf over rows and columns in (j, d), reading only the tiles on and below the
// diagonal (and only the lower triangle of those): the matrix is symmetric, so a 64 x 64 tile T = A[I][J],
// J < I, serves both y_I += T v_J and y_J += T^T v_I.  Row blocks start at `base`, the 64-aligned index at or below j + 1.  One workgroup owns the
// row blocks bx and nbk - 1 - bx (nbk + 1 tiles, the same for every workgroup).  It writes the row sums of its
// blocks to ybuf and the transposed contributions, one 64-vector per tile and wavefront, to `part`;
// trd_symv_reduce_kernel adds those to ybuf in a fixed order.  Dynamic LDS: nbk * 64 floats.
constexpr int TRD_SB = 64;

__device__ __forceinline__ void trd_symv_row_block(const TrdJob& J, const float* __restrict__ vs, int base, int nbk, int I) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rsub = lane >> 4, c4 = (lane & 15) * 4;
  const long long ld = J.dpad;
  const int row0 = I * TRD_SB + 16 * wave + rsub;  // first of this lane's four rows (stride 4), relative to base
  float vI[4], racc[4];
#pragma unroll
  for (int it = 0; it < 4; ++it) { vI[it] = vs[row0 + 4 * it]; racc[it] = 0.f; }
  const float* __restrict__ Trow = J.A + (long long)(base + row0) * ld + base + c4;
  for (int Jb = 0; Jb <= I; ++Jb) {
    vfloat4_t a[4];
#pragma unroll
    for (int it = 0; it < 4; ++it)
      a[it] = __builtin_nontemporal_load(reinterpret_cast<const vfloat4_t*>(Trow + (long long)(4 * it) * ld + Jb * TRD_SB));
    const float4 vj = *reinterpret_cast<const float4*>(vs + Jb * TRD_SB + c4);
    if (Jb == I) {
      // Diagonal tile: only its lower triangle is used, like everywhere else (the two triangles of the matrix
      // agree to rounding only, and on the numerically zero trailing blocks of a rank-deficient factor the
      // rounding is all there is).  Entries above the diagonal are dropped here and come back as the
      // transposed contribution of the strictly lower ones.
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        const int rl = 16 * wave + rsub + 4 * it;  // row inside the tile
        a[it].x = (c4 + 0 <= rl) ? a[it].x : 0.f;
        a[it].y = (c4 + 1 <= rl) ? a[it].y : 0.f;
        a[it].z = (c4 + 2 <= rl) ? a[it].z : 0.f;
        a[it].w = (c4 + 3 <= rl) ? a[it].w : 0.f;
      }
    }
#pragma unroll
    for (int it = 0; it < 4; ++it) racc[it] += (a[it].x * vj.x + a[it].y * vj.y) + (a[it].z * vj.z + a[it].w * vj.w);
    {
      if (Jb == I) {  // strictly lower part for the transposed contribution
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int rl = 16 * wave + rsub + 4 * it;
          a[it].x = (c4 + 0 < rl) ? a[it].x : 0.f;
          a[it].y = (c4 + 1 < rl) ? a[it].y : 0.f;
          a[it].z = (c4 + 2 < rl) ? a[it].z : 0.f;
          a[it].w = (c4 + 3 < rl) ? a[it].w : 0.f;
        }
      }
      float4 cs = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        cs.x += a[it].x * vI[it];
        cs.y += a[it].y * vI[it];
        cs.z += a[it].z * vI[it];
        cs.w += a[it].w * vI[it];
      }
#pragma unroll
      for (int o = 16; o <= 32; o <<= 1) {
        cs.x += __shfl_xor(cs.x, o, 64);
        cs.y += __shfl_xor(cs.y, o, 64);
        cs.z += __shfl_xor(cs.z, o, 64);
        cs.w += __shfl_xor(cs.w, o, 64);
      }
      if (lane < 16) *reinterpret_cast<float4*>(J.part + ((long long)(I * nbk + Jb) * 4 + wave) * TRD_SB + c4) = cs;
    }
  }
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    float t = racc[it];
#pragma unroll
    for (int o = 1; o <= 8; o <<= 1) t += __shfl_xor(t, o, 64);
    if ((lane & 15) == 0) J.ybuf[base + row0 + 4 * it] = t;
  }
}

__global__ __launch_bounds__(256) void trd_symv_kernel(const TrdJob* __restrict__ jobs, int j) {
  extern __shared__ float vs[];
  const TrdJob& J = jobs[blockIdx.y];
  const int d = J.d;
  const int base = (j + 1) & ~(TRD_SB - 1);
  const int nbk = (d - base + TRD_SB - 1) / TRD_SB;
  if (2 * (int)blockIdx.x >= nbk) return;
  for (int c = threadIdx.x; c < nbk * TRD_SB; c += 256) vs[c] = (base + c > j) ? J.vbuf[base + c] : 0.f;
  __syncthreads();
  const int I0 = blockIdx.x, I1 = nbk - 1 - blockIdx.x;
  trd_symv_row_block(J, vs, base, nbk, I0);
  if (I1 != I0) trd_symv_row_block(J, vs, base, nbk, I1);
}

// ybuf[J block] += sum over I >= J and the four wavefronts of part[I][J]; grid (nbk, factors).
__global__ __launch_bounds__(256) void trd_symv_reduce_kernel(const TrdJob* __restrict__ jobs, int j) {
  __shared__ float red[4][TRD_SB];
  const TrdJob& J = jobs[blockIdx.y];
  const int d = J.d;
  const int base = (j + 1) & ~(TRD_SB - 1);
  const int nbk = (d - base + TRD_SB - 1) / TRD_SB;
  const int Jb = blockIdx.x;
  const int q = threadIdx.x >> 6, r = threadIdx.x & 63;
  float acc = 0.f;
  for (int I = Jb; I < nbk; ++I) acc += J.part[((long long)(I * nbk + Jb) * 4 + q) * TRD_SB + r];
  red[q][r] = acc;
  __syncthreads();
  if (q == 0) {
    const int row = base + Jb * TRD_SB + r;
    if (row > j && row < d) J.ybuf[row] += (red[0][r] + red[1][r]) + (red[2][r] + red[3][r]);
  }
}

// Triangular factor T of the block reflector of panel blockIdx.x (LAPACK slarft, forward, columnwise):
// H_p0 ... H_p0+k-1 = I - V T V^T.  grid (panels, factors).
__global__ __launch_bounds__(256) void trd_tfactor_kernel(const TrdJob* __restrict__ jobs) {
  __shared__ float Vs[64][TRD_NB + 1];
  __shared__ float S[TRD_NB][TRD_NB + 1];
  __shared__ float Tm[TRD_NB][TRD_NB + 1];
  __shared__ float taus[TRD_NB];
  const TrdJob& J = jobs[blockIdx.y];
  const int d = J.d, p0 = blockIdx.x * TRD_NB;
  if (p0 >= d - 1) return;
  const int kcols = min(TRD_NB, d - 1 - p0);
  const int tid = threadIdx.x;
  const long long ld = J.dpad;
  const int i = tid >> 3, k0 = (tid & 7) * 4;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int rb = p0 + 1; rb < d; rb += 64) {
    for (int e = tid; e < 64 * TRD_NB; e += 256) {
      const int rr = e >> 5, c = e & 31, r = rb + rr;
      Vs[rr][c] = (r < d) ? J.Vall[(long long)r * ld + p0 + c] : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int rr = 0; rr < 64; ++rr) {
      const float vi = Vs[rr][i];
#pragma unroll
      for (int m = 0; m < 4; ++m) acc[m] += vi * Vs[rr][k0 + m];
    }
    __syncthreads();
  }
#pragma unroll
  for (int m = 0; m < 4; ++m) S[i][k0 + m] = acc[m];
  if (tid < TRD_NB) taus[tid] = (tid < kcols) ? J.tau[p0 + tid] : 0.f;
  for (int e = tid; e < TRD_NB * TRD_NB; e += 256) Tm[e >> 5][e & 31] = 0.f;
  __syncthreads();
  for (int c = 0; c < TRD_NB; ++c) {
    if (tid < c) {
      float a = 0.f;
      for (int m = tid; m < c; ++m) a += Tm[tid][m] * S[m][c];
      Tm[tid][c] = -taus[c] * a;
    }
    if (tid == c) Tm[c][c] = taus[c];
    __syncthreads();
  }
  float* out = J.Tmat + (long long)blockIdx.x * TRD_NB * TRD_NB;
  for (int e = tid; e < TRD_NB * TRD_NB; e += 256) out[e] = Tm[e >> 5][e & 31];
}

// Scale T to unit maximum entry and reset the QL state.  One workgroup per factor.
__global__ __launch_bounds__(256) void tql_init_kernel(const TrdJob* __restrict__ jobs) {
  __shared__ float red[4];
  const TrdJob& J = jobs[blockIdx.x];
  const int d = J.d;
  float m = 0.f;
  for (int i = threadIdx.x; i < d; i += 256) {
    m = fmaxf(m, fabsf(J.diag[i]));
    if (i < d - 1) m = fmaxf(m, fabsf(J.off[i]));
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  const float tn = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const double inv = (tn > 0.f) ? 1.0 / (double)tn : 1.0;
  for (int i = threadIdx.x; i < d; i += 256) {
    J.qd[i] = (double)J.diag[i] * inv;
    J.qe[i] = (i < d - 1) ? (double)J.off[i] * inv : 0.0;
  }
  if (threadIdx.x == 0) {
    J.state[0] = 0; J.state[1] = 0; J.state[2] = 0; J.state[3] = 0; J.state[4] = 0;
    J.state[5] = __float_as_int((tn > 0.f) ? tn : 1.0f);
    J.hdr[0] = 0;
    J.hdr[TQL_HDR] = 0;
  }
}

__global__ __launch_bounds__(256) void tql_finish_kernel(const TrdJob* __restrict__ jobs) {
  const TrdJob& J = jobs[blockIdx.x];
  const float tn = __int_as_float(J.state[5]);
  for (int i = threadIdx.x; i < J.d; i += 256) J.diag[i] = (float)(J.qd[i] * (double)tn);
}

// Implicit QL iteration (EISPACK tql2 recurrences) on the tridiagonal matrix of one factor per wavefront, up to
// TQL_K sweeps per launch, the rotations logged for tql_apply_kernel.
//
// A single chase is a chain of ~12 dependent operations per rotation, i.e. latency bound, so sweeps are
// pipelined across the lanes of the wavefront: a batch of p <= TQL_P sweeps with fixed shifts (the eigenvalues
// of the leading p x p block of the unreduced block, found by bisection, one per lane; the Wilkinson shift when
// p = 1) runs with lane j working TQL_LAG indices behind lane j - 1.  Lane j reads the entries lane j - 1 left
// behind at least two steps earlier (LDS operations of one wavefront execute in order), which is exactly the
// sequential order of the sweeps, so the batch equals p consecutive shifted QL steps.
//
// The recurrences run in fp64 (same issue rate as fp32 on this GPU): in fp32 the rounding of the O(1) entries at
// the far end of an unreduced block leaves a noise floor of ~1e-7 on the small entries at the deflating end,
// which both stalls convergence and costs absolute accuracy on small eigenvalues.  The logged rotations are fp32.
// Dynamic LDS: 2 * dpad doubles.
constexpr int TQL_P = 8;
constexpr int TQL_LAG = 4;  // even: all lanes use the same operand register set in a given step

__global__ __launch_bounds__(64) void tql_sweeps_kernel(const TrdJob* __restrict__ jobs, int buf, int max_sweeps) {
  extern __shared__ double lds64[];
  const TrdJob& J = jobs[blockIdx.x];
  const int n = J.d, dpad = J.dpad, lane = threadIdx.x;
  int* __restrict__ st = J.state;
  int* __restrict__ hdr = J.hdr + buf * TQL_HDR;
  float2* __restrict__ rot = J.rot + (long long)buf * TQL_K * dpad;
  if (st[2] || st[3]) {
    if (lane == 0) hdr[0] = 0;
    return;
  }
  double* dd = lds64;
  double* ee = lds64 + dpad;
  for (int i = lane; i < n; i += 64) { dd[i] = J.qd[i]; ee[i] = J.qe[i]; }
  int l = st[0];
  const int done_before = st[4];
  int sweeps = 0;
  bool failed = false;
  int top = -1, bot = 0x7fffffff;
  __syncthreads();
  const double eps = 1.1920929e-7;      // fp32 resolution is all the caller can use
  const double abs_tol = 1.4901161e-8;  // 2^-26 of the (unit) largest entry
  // every control variable below is computed identically by all lanes (uniform)
  while (l < n) {
    // smallest m >= l whose off-diagonal entry is negligible (ee[n - 1] = 0 ends every search)
    int m = l;
    for (;;) {
      const int idx = m + lane;
      bool small = true;
      if (idx < n - 1) {
        const double av = fabs(ee[idx]);
        small = (av <= eps * (fabs(dd[idx]) + fabs(dd[idx + 1]))) || (av <= abs_tol);
      }
      const unsigned long long mask = __ballot(small);
      if (mask) { m += __ffsll((long long)mask) - 1; break; }
      m += 64;
    }
    m = min(m, n - 1);
    if (m == l) { ++l; continue; }
    const int p = min(TQL_P, max(1, (m - l + 1) / 2));
    if (sweeps + p > TQL_K) break;
    if (done_before + sweeps + p > max_sweeps) { failed = true; break; }  // total budget (LAPACK steqr: 30 n)
    if (lane == 0) ee[m] = 0.0;

    // ---- shifts
    double sigma;
    if (p == 1) {
      const double dl = dd[l], el = ee[l];
      const double gw = (dd[l + 1] - dl) / (2.0 * el);
      const double rw = sqrt(gw * gw + 1.0);
      sigma = dl - el / (gw + copysign(rw, gw));
    } else {
      // lane j: j-th eigenvalue of the leading p x p block by bisection on Sturm counts.  fp64 with a refined
      // fp32 reciprocal: the block is graded, and a shift is only useful if it resolves the small eigenvalues.
      double db[TQL_P], e2[TQL_P];
      double lo = 1.0e300, hi = -1.0e300;
#pragma unroll
      for (int k = 0; k < TQL_P; ++k) {
        const bool in = k < p;
        db[k] = in ? dd[l + k] : 0.0;
        const double ek = (in && k < p - 1) ? ee[l + k] : 0.0;
        e2[k] = ek * ek;
      }
#pragma unroll
      for (int k = 0; k < TQL_P; ++k) {
        if (k < p) {
          const double rad = sqrt(e2[k]) + (k > 0 ? sqrt(e2[k - 1]) : 0.0);
          lo = fmin(lo, db[k] - rad);
          hi = fmax(hi, db[k] + rad);
        }
      }
      for (int it = 0; it < 44; ++it) {
        const double mid = 0.5 * (lo + hi);
        int cnt = 0;
        double q = 1.0;
#pragma unroll
        for (int k = 0; k < TQL_P; ++k) {
          if (k < p) {
            double qi = (double)__builtin_amdgcn_rcpf((float)q);
            qi = qi * (2.0 - q * qi);
            q = db[k] - mid - (k > 0 ? e2[k - 1] * qi : 0.0);
            if (fabs(q) < 1e-30) q = -1e-30;
            cnt += (q < 0.0) ? 1 : 0;
          }
        }
        if (cnt > lane) hi = mid; else lo = mid;
      }
      sigma = 0.5 * (lo + hi);
    }

    // ---- pipelined batch of p sweeps over [l, m]
    double s = 1.0, c = 1.0, pp = 0.0, g = 0.0, d_up = 0.0, r;
    double e_a = 0.0, d_a = 0.0, e_b = 0.0, d_b = 0.0;
    bool dead = false;
    int abort_i = l - 1;
    const int last_k = m - l - 1;
    const int n_iter = last_k + 1 + TQL_LAG * (p - 1);
    global_float2* out = (global_float2*)(rot + (long long)(sweeps + min(lane, p - 1)) * dpad);
    // One step of lane `lane` at pipeline time tau: index i = m - 1 - (tau - TQL_LAG * lane), operands (e_i, d_i)
    // of that index; they are reloaded for the index two below right after their use.  The matrix has unit scale
    // and entries below 2^-26 count as zero, so a bulge whose square is below 1e-30 is an exact underflow for
    // every purpose: that sweep ends there (EISPACK's recovery).  1 / sqrt(t): fp32 seed and one Newton step in
    // fp64 (~2e-14); normalising the rotation in fp32 instead was measured to bring the fp32 noise floor back.
#define TQL_STEP(tau_, e_i, d_i)                                                  \
  {                                                                               \
    const int k = (tau_) - TQL_LAG * lane;                                        \
    const int i = m - 1 - k;                                                      \
    if (lane < p && k == 0) {                                                     \
      g = dd[m] - sigma;                                                          \
      d_up = dd[m];                                                               \
      e_a = ee[m - 1];                                                            \
      d_a = dd[m - 1];                                                            \
      e_b = ee[max(m - 2, l)];                                                    \
      d_b = dd[max(m - 2, l)];                                                    \
    }                                                                             \
    if (lane < p && k >= 0 && k <= last_k && !dead) {                             \
      const double f = s * e_i, b = c * e_i;                                      \
      const double t = f * f + g * g;                                             \
      if (t < 1e-30) {                                                            \
        dd[i + 1] = d_up - pp;                                                    \
        if (k != 0) ee[i + 1] = 0.0; /* the new entry there is sqrt(t) */         \
        ee[i] = b; /* the rotations so far turned e[i] into c e[i]; the bulge s e[i] is dropped */ \
        dead = true;                                                              \
        abort_i = i;                                                              \
      } else {                                                                    \
        double rinv = (double)__builtin_amdgcn_rsqf((float)t);                    \
        rinv = rinv * (1.5 - (0.5 * t) * (rinv * rinv));                          \
        if (k != 0) ee[i + 1] = t * rinv;                                         \
        s = f * rinv;                                                             \
        c = g * rinv;                                                             \
        g = d_up - pp;                                                            \
        r = (d_i - g) * s + 2.0 * c * b;                                          \
        pp = s * r;                                                               \
        dd[i + 1] = g + pp;                                                       \
        g = c * r - b;                                                            \
        out[i] = vfloat2_t{(float)c, (float)s};                                   \
        d_up = d_i;                                                               \
        if (k == last_k) {                                                        \
          dd[l] = d_i - pp;                                                       \
          ee[l] = g;                                                              \
        }                                                                         \
        const int nx = max(i - 2, l);                                             \
        e_i = ee[nx];                                                             \
        d_i = dd[nx];                                                             \
      }                                                                           \
    }                                                                             \
    __builtin_amdgcn_wave_barrier();                                              \
    asm volatile("" ::: "memory");                                                \
  }
    for (int tau = 0; tau < n_iter; tau += 2) {
      TQL_STEP(tau, e_a, d_a)
      TQL_STEP(tau + 1, e_b, d_b)
    }
#undef TQL_STEP
    if (lane < p) {
      hdr[4 + sweeps + lane] = dead ? abort_i + 1 : l;
      hdr[4 + TQL_K + sweeps + lane] = m;
    }
    top = max(top, m);
    bot = min(bot, l);
    sweeps += p;
  }
  __syncthreads();
  for (int i = lane; i < n; i += 64) { J.qd[i] = dd[i]; J.qe[i] = ee[i]; }
  if (lane == 0) {
    st[0] = l;
    st[2] = (l >= n) ? 1 : 0;
    st[3] = failed ? 1 : 0;
    st[4] = done_before + sweeps;
    hdr[0] = sweeps;
    hdr[1] = top;
    hdr[2] = bot;
  }
}

// Apply one chunk of logged sweeps to the rows of Y.  Sequentially a sweep rotates rows (i, i + 1) for
// i = m - 1 down to l:  Y[i + 1] <- s Y[i] + c Y[i + 1],  Y[i] <- c Y[i] - s Y[i + 1].
// Pipeline: at step p stage k (sweep k) works at index i = p + k on the row handed down by stage k - 1
// (row i) and its own carried row (row i + 1); the finished row i + 1 goes to stage k + 1, row i is carried.
// grid (ceil(d / 256), factors): one thread per column of Y.
__global__ __launch_bounds__(256) void tql_apply_kernel(const TrdJob* __restrict__ jobs, int buf) {
  __shared__ float2 coef[TQL_STEPS][TQL_K];
  __shared__ int sl[TQL_K], sm[TQL_K];
  const TrdJob& J = jobs[blockIdx.y];
  const int* __restrict__ hdr = J.hdr + buf * TQL_HDR;
  const int nsweeps = hdr[0];
  if (nsweeps == 0) return;
  const int top = hdr[1], bot = hdr[2];
  const int dpad = J.dpad;
  const float2* __restrict__ rot = J.rot + (long long)buf * TQL_K * dpad;
  const int tid = threadIdx.x;
  const int col = blockIdx.x * 256 + tid;
  const bool valid = col < J.d;
  float* __restrict__ Y = J.Y + (valid ? col : 0);
  if (tid < TQL_K) {
    sl[tid] = (tid < nsweeps) ? hdr[4 + tid] : 0x7fffffff;
    sm[tid] = (tid < nsweeps) ? hdr[4 + TQL_K + tid] : -1;
  }
  float carry[TQL_K];
#pragma unroll
  for (int k = 0; k < TQL_K; ++k) carry[k] = 0.f;
  carry[0] = valid ? Y[(long long)top * dpad] : 0.f;
  const int p_last = bot - TQL_K;
  for (int p_hi = top - 1; p_hi >= p_last; p_hi -= TQL_STEPS) {
    __syncthreads();
    for (int e = tid; e < TQL_STEPS * TQL_K; e += 256) {
      const int t = e / TQL_K, k = e % TQL_K;
      const int i = p_hi - t + k;
      float2 cs = make_float2(1.0f, 0.0f);
      if (i >= sl[k] && i < sm[k]) cs = rot[(long long)k * dpad + i];
      coef[t][k] = cs;
    }
    __syncthreads();
    const int steps = min(TQL_STEPS, p_hi - p_last + 1);
    float xn = (valid && p_hi >= bot) ? Y[(long long)p_hi * dpad] : 0.f;
    for (int t = 0; t < steps; ++t) {
      const int p = p_hi - t;
      float x = xn;
      xn = (valid && t + 1 < steps && p - 1 >= bot) ? Y[(long long)(p - 1) * dpad] : 0.f;
#pragma unroll
      for (int k = 0; k < TQL_K; ++k) {
        const float2 cs = coef[t][k];
        const float f = carry[k];
        const float up = cs.y * x + cs.x * f;
        carry[k] = cs.x * x - cs.y * f;
        x = up;
      }
      const int r = p + TQL_K;
      if (valid && r >= bot && r <= top) Y[(long long)r * dpad] = x;
    }
  }
}

// Ys[r][c] = Y[r][c] * w[r]; one workgroup per 8 rows.
struct RowScale {
  const float* Y;
  float* Ys;
  const float* w;
  int dpad;
  int row_begin;
};
__global__ __launch_bounds__(256) void eig_scale_rows_kernel(const RowScale* __restrict__ jobs, int n_jobs) {
  int lo = 0, hi = n_jobs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (jobs[mid].row_begin <= (int)blockIdx.x) lo = mid; else hi = mid - 1;
  }
  const RowScale& J = jobs[lo];
  const int dpad = J.dpad;
  const int r0 = (blockIdx.x - J.row_begin) * 8;
  for (int e = threadIdx.x * 4; e < 8 * dpad; e += 256 * 4) {
    const int r = r0 + e / dpad, c = e % dpad;
    const float4 v = *reinterpret_cast<const float4*>(J.Y + (long long)r * dpad + c);
    const float w = J.w[r];
    *reinterpret_cast<float4*>(J.Ys + (long long)r * dpad + c) = make_float4(v.x * w, v.y * w, v.z * w, v.w * w);
  }
}

}  // namespace sa
