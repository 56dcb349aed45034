// Batched symmetric eigendecomposition through tridiagonalisation, for factors too large for the
// block-Jacobi solver to be competitive.
//
//   1. A = Q1 T Q1^T: blocked Householder tridiagonalisation (LAPACK sytrd/latrd recurrences).  Per column
//      one single-workgroup kernel per factor (the w vector of the previous column, the Householder vector,
//      its products with the panel) and one symmetric matrix-vector product over the trailing matrix, which is
//      the HBM-bound part ((2/3) d^3 bytes per factor: one triangle) and carries the panel's row terms of the
//      next column in extra workgroups; per 32-column panel one rank-64 trailing update
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
constexpr int TRD_SB = 64;               // tile of the symmetric matrix-vector product
constexpr int TDC_PF = 16;  // rows whose operands the inverse iteration fetches ahead of the recurrence
constexpr int TRD_PW = 2 * TRD_NB;       // columns of the [V | W] and [W | V] panels (the K of the trailing update)
constexpr int TRD_PR = 3 * TRD_NB;       // rows of the panel buffer, which keeps the panel columns as contiguous rows: V, W, V
constexpr int TRD_COL_THREADS = 1024;
constexpr int TRD_ROWS_PER_THREAD = 8;   // d <= 8192
constexpr int TRD_MAX_DIM = TRD_COL_THREADS * TRD_ROWS_PER_THREAD;
constexpr int TQL_K = 32;                // sweeps per chunk
constexpr int TQL_STEPS = 64;            // pipeline steps whose coefficients are staged in LDS at a time
constexpr int TQL_HDR = 4 + 2 * TQL_K;   // ints per chunk header: nsweeps, top, bot, -, l[K], m[K]

struct TrdJob {
  float* A;       // dpad x dpad, symmetric, both triangles kept current
  float* Y;       // dpad x dpad
  float* Vall;    // dpad x dpad, row j = Householder vector of column j (explicit unit entry, zeros in front of it)
  float* P1;      // 96 x dpad, the current panel by columns: rows 0-31 V, 32-63 W, 64-95 V again; [V | W] = rows 0-63
  float* P2;      // P1 + 32 dpad: [W | V] = rows 32-95 (every column step writes whole rows: no strided stores)
  float* vbuf;    // dpad: current Householder vector, zero at and above the diagonal
  float* ybuf;    // dpad: trailing matrix times vbuf
  float* part;    // ceil(dpad / 128) x dpad: column sums of the symmetric product, one vector per workgroup
  float* diag;    // dpad
  float* off;     // dpad: off[j] couples j and j + 1
  float* tau;     // dpad
  float* d1buf;   // dpad: row terms V (W^T v) + W (V^T v) of the column step in flight
  float* apre;    // dpad: the next column after the complete reflectors of the panel
  float* t12;     // 64: W^T v | V^T v over the complete panel columns, for the column step in flight
  double* qd;     // dpad: diagonal of the (unit-scaled) tridiagonal matrix during the QL iteration
  double* qe;     // dpad: its off-diagonal
  float* S128;    // (dpad / 128) x 128 x 128: Gram matrices of the Householder vectors, 128 at a time
  float* T128;    // (dpad / 128) x 128 x 128: triangular factors of the 128-wide block reflectors that accumulate Q1
  float2* rot;    // 2 x TQL_K x dpad rotation log (c, s)
  int* hdr;       // 2 x TQL_HDR
  int* state;     // l, -, done, failed, total sweeps, bits of the scale
  // bisection + inverse iteration on the tridiagonal matrix (tdc_* kernels)
  float* Z;       // dpad x dpad, column i = eigenvector i of the tridiagonal matrix
  double* lam;    // dpad eigenvalues of the unit-scaled matrix, ascending inside every unreduced block
  int* blk_s;     // dpad: first index of the unreduced block that holds index i
  int* blk_e;     // dpad: one past its last index
  int* fail;      // set when the vectors of this factor do not pass the checks (the caller then takes the QL path)
  double* lu_a;   // E-wide tables, entry [row][t] for the t-th eigenvalue of the chunk in flight: pivots of U,
  double* lu_b;   //   first superdiagonal of U,
  double* lu_d;   //   second superdiagonal of U (row interchanges),
  double* lu_c;   //   multipliers of L,
  double* lu_x;   //   the iteration vector
  unsigned char* lu_f;  // row interchange flags
  int chunk;      // E
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

__global__ __launch_bounds__(256) void trd_clear_panel_kernel(const TrdJob* __restrict__ jobs) {
  const TrdJob& J = jobs[blockIdx.y];
  const long long n4 = (long long)J.dpad * TRD_PR / 4;
  float4* dst = reinterpret_cast<float4*>(J.P1);
  for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < n4; e += (long long)gridDim.x * 256)
    dst[e] = make_float4(0.f, 0.f, 0.f, 0.f);
}

// One column step of the panel reduction (LAPACK slatrd) in two launches per column.  Column j needs, in this order,
//   (fin)   w of column j - 1:  w = tau (y - V (W^T v) - W (V^T v)),  w += -1/2 tau (w . v) v,   y = A_trail v of column j - 1
//   (start) column j of A as it stands after the reflectors of this panel, its Householder vector v, diag / off / tau.
// trd_col_kernel (one workgroup per factor) gathers y from the product's partial sums, finishes w, the corrected column
// and the Householder vector v_j, and then forms t1 = W^T v_j, t2 = V^T v_j over the complete panel columns while v_j is
// still in its registers.  What walks the panel row by row -- the row terms d1 = V t1 + W t2 of the NEXT column step and
// the pending rank-2k correction of column j + 1 by the complete panel columns -- needs nothing from the product of
// column j, so it rides in the product's launch as TRD_AUX_WGS extra workgroups per factor (trd_aux_rows below): one
// stream, no events, and the product hides it.
// flags bit 0: fin, bit 1: start.  Panel columns are p0 .. p0 + 31.
constexpr int TRD_AUX_WGS = 8;

__device__ __forceinline__ void trd_aux_rows_of(int d, int j, int g, int& r0, int& r1) {
  const int per = ((d - j + TRD_AUX_WGS - 1) / TRD_AUX_WGS + 31) & ~31;
  r0 = min(j + g * per, d);
  r1 = min(r0 + per, d);
}

// Row terms of column step j for the rows of aux workgroup g (256 threads); sh: 4 * TRD_NB floats of LDS.
__device__ __forceinline__ void trd_aux_rows(const TrdJob& J, int j, int p0, int flags, int g, float* sh) {
  float *t1 = sh, *t2 = sh + TRD_NB, *rowV = sh + 2 * TRD_NB, *rowW = sh + 3 * TRD_NB;
  const int d = J.d;
  if (j >= d) return;
  const int tid = threadIdx.x;
  const long long ld = J.dpad;
  const float* __restrict__ P1 = J.P1;
  const bool fin = (flags & 1) != 0, start = (flags & 2) != 0;
  const int ip = fin ? j - 1 - p0 : j - p0;  // panel columns complete on entry
  if (tid < TRD_NB) {
    const bool have = fin && tid < ip;
    t1[tid] = have ? J.t12[tid] : 0.f;
    t2[tid] = have ? J.t12[TRD_NB + tid] : 0.f;
    rowV[tid] = (start && tid < ip) ? P1[(long long)tid * ld + j] : 0.f;
    rowW[tid] = (start && tid < ip) ? P1[(long long)(TRD_NB + tid) * ld + j] : 0.f;
  }
  __syncthreads();
  int r0, r1;
  trd_aux_rows_of(d, j, g, r0, r1);
  for (int r = r0 + tid; r < r1; r += 256) {
    //   d1 = sum_q V[r][q] t1[q] + W[r][q] t2[q]      (correction of w)
    //   d2 = sum_q V[r][q] rowW[q] + W[r][q] rowV[q]  (correction of the next column)
    float d1 = 0.f, d2 = 0.f;
#pragma unroll 8
    for (int q = 0; q < ip; ++q) {
      const float v = P1[(long long)q * ld + r], w = P1[(long long)(TRD_NB + q) * ld + r];
      d1 += v * t1[q] + w * t2[q];
      d2 += v * rowW[q] + w * rowV[q];
    }
    if (fin) J.d1buf[r] = d1;
    // column j as it stands after the complete reflectors of this panel (row j of A is the same by symmetry)
    if (start) J.apre[r] = J.A[(long long)r * ld + j] - d2;
  }
}

// ROWS: rows per thread, ROWS * TRD_COL_THREADS >= d.
template <int ROWS>
__global__ __launch_bounds__(TRD_COL_THREADS) void trd_col_kernel(const TrdJob* __restrict__ jobs, int j, int p0, int flags) {
  __shared__ float red[TRD_COL_THREADS / 64];
  __shared__ float bc[3];
  __shared__ float vsh[ROWS * TRD_COL_THREADS];
  const TrdJob& J = jobs[blockIdx.x];
  const int d = J.d;
  if (j >= d) return;
  const int tid = threadIdx.x;
  const long long ld = J.dpad;
  float* __restrict__ P1 = J.P1;
  const bool fin = (flags & 1) != 0, start = (flags & 2) != 0;
  const int jp = j - 1;
  const int ip = fin ? jp - p0 : j - p0;
  const float tau_p = fin ? J.tau[jp] : 0.f;
  // where the symmetric product of column j - 1 left y: row sums in ybuf, column sums per workgroup in part
  const int ybase = j & ~(TRD_SB - 1);
  const int ynbk = (d - ybase + TRD_SB - 1) / TRD_SB;
  const int ywgs = (ynbk + 1) / 2;
  const long long ylen = (long long)ynbk * TRD_SB;

  float wreg[ROWS], vreg[ROWS], areg[ROWS];
  float dot = 0.f;
  // Rows of this thread; a row past the end is read as row d - 1 and dropped, so that no load depends on a branch and
  // the partial sums of all rows can be in flight together (one load per row and workgroup of the product: waiting for
  // each of them in turn was most of this kernel's time).
  int rr[ROWS];
  float yreg[ROWS];
#pragma unroll
  for (int k = 0; k < ROWS; ++k) {
    rr[k] = min(j + tid + k * TRD_COL_THREADS, d - 1);
    yreg[k] = 0.f;
  }
  if (fin) {
    const float* __restrict__ pp = J.part - ybase;
    int g = 0;
    for (; g + 4 <= ywgs; g += 4) {
      float t[4][ROWS];
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int k = 0; k < ROWS; ++k) t[u][k] = pp[(g + u) * ylen + rr[k]];
#pragma unroll
      for (int k = 0; k < ROWS; ++k) yreg[k] += (t[0][k] + t[1][k]) + (t[2][k] + t[3][k]);
    }
    for (; g < ywgs; ++g)
#pragma unroll
      for (int k = 0; k < ROWS; ++k) yreg[k] += pp[g * ylen + rr[k]];
  }
#pragma unroll
  for (int k = 0; k < ROWS; ++k) {
    const int r = j + tid + k * TRD_COL_THREADS;
    float w = 0.f, vr = 0.f, a = 0.f;
    if (fin) {
      vr = J.vbuf[rr[k]];
      w = tau_p * ((J.ybuf[rr[k]] + yreg[k]) - J.d1buf[rr[k]]);  // w = tau (y - V (W^T v) - W (V^T v))
    }
    if (start) a = J.apre[rr[k]];
    if (r >= d) { w = 0.f; vr = 0.f; a = 0.f; }
    dot += w * vr;
    wreg[k] = w;
    vreg[k] = vr;
    areg[k] = a;
  }
  if (fin) {
    const float alpha = -0.5f * tau_p * block_sum_1024(dot, red);
#pragma unroll
    for (int k = 0; k < ROWS; ++k) {
      const int r = j + tid + k * TRD_COL_THREADS;
      if (r < d) {
        const float w = wreg[k] + alpha * vreg[k];
        wreg[k] = w;
        P1[(long long)(TRD_NB + ip) * ld + r] = w;
      }
    }
    if (tid == 0) bc[2] = wreg[0];  // w at row j
    __syncthreads();
    if (start) {  // the column just completed also corrects column j: V[r][ip] W[j][ip] + W[r][ip] V[j][ip]
      const float wj = bc[2], vj = 1.0f;  // the Householder vector of column j - 1 has its unit entry at row j
#pragma unroll
      for (int k = 0; k < ROWS; ++k) areg[k] -= vreg[k] * wj + wreg[k] * vj;
    }
  }

  if (start) {
    const int i = j - p0;
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < ROWS; ++k) {
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
    float vnew[ROWS];
#pragma unroll
    for (int k = 0; k < ROWS; ++k) {
      const int r = j + tid + k * TRD_COL_THREADS;
      vnew[k] = 0.f;
      if (r < d && r > j) {
        const float v = (r == j + 1) ? 1.0f : areg[k] * scale;
        vnew[k] = v;
        J.vbuf[r] = v;
        P1[(long long)i * ld + r] = v;
        P1[(long long)(2 * TRD_NB + i) * ld + r] = v;
        J.Vall[(long long)j * ld + r] = v;
      }
    }
    // t1 = W^T v, t2 = V^T v over the i complete panel columns, for the next column step: v goes to LDS, and every
    // wavefront takes up to four of the 2 i columns (c, c + 16, ...), its lanes along the rows, the four sums advancing
    // together so that their loads are in flight at the same time.  (The last column of W was written above by this
    // workgroup; the barrier makes it visible.)
    if (i > 0) {
#pragma unroll
      for (int k = 0; k < ROWS; ++k) vsh[tid + k * TRD_COL_THREADS] = vnew[k];
      __syncthreads();
      const int lane = tid & 63, wave = tid >> 6;
      const int m = d - j;  // vsh[x] belongs to row j + x
      const float* col[4];
      float a[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = min(wave + 16 * u, 2 * i - 1);  // a wavefront without a column of its own repeats the last one
        col[u] = P1 + (long long)(c < i ? c : TRD_NB + (c - i)) * ld + j;
        a[u] = 0.f;
      }
      if (wave < 2 * i) {
        int x = lane;
        for (; x + 64 < m; x += 128) {
          const float v0 = vsh[x], v1 = vsh[x + 64];
#pragma unroll
          for (int u = 0; u < 4; ++u) a[u] += col[u][x] * v0 + col[u][x + 64] * v1;
        }
        if (x < m) {
          const float v0 = vsh[x];
#pragma unroll
          for (int u = 0; u < 4; ++u) a[u] += col[u][x] * v0;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const float t = wave_sum(a[u]);
          const int c = wave + 16 * u;
          if (lane == 0 && c < 2 * i) J.t12[c < i ? TRD_NB + c : c - i] = t;  // V column c -> t2[c], W column c - i -> t1[c - i]
        }
      }
    }
  }
}

// y = (trailing matrix) x vbuf over rows and columns in (j, d), reading only the tiles on and below the diagonal (and
// only the lower triangle of the diagonal tiles): the matrix is symmetric, so a 64 x 64 tile T = A[I][J], J <= I, serves
// both y_I += T v_J (row sums) and y_J += T^T v_I (column sums).  Row blocks start at `base`, the 64-aligned index at or
// below j + 1.  One workgroup owns the row blocks bx and nbk - 1 - bx (nbk + 1 tiles, the same for every workgroup); a
// wavefront takes whole tiles (column block J = wave, wave + 4, ...), all sixteen 16-byte loads of its lanes issued
// before the first use.  Row sums go to ybuf; the column sums of all tiles of the workgroup are kept in LDS (a wavefront
// only ever adds to its own column blocks, in program order, so the sums do not depend on scheduling) and leave as one
// vector per workgroup in `part`, which trd_col_kernel adds up.  Dynamic LDS: 2 * nbk * 64 floats.
__device__ __forceinline__ void trd_symv_row_block(const TrdJob& J, const float* __restrict__ vs, float* __restrict__ acc,
                                                   float (*rs)[TRD_SB], int base, int I) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rsub = lane >> 4, c4 = (lane & 15) * 4;
  const long long ld = J.dpad;
  float vI[16], racc[16];
#pragma unroll
  for (int it = 0; it < 16; ++it) { vI[it] = vs[I * TRD_SB + rsub + 4 * it]; racc[it] = 0.f; }
  const float* __restrict__ Trow = J.A + (long long)(base + I * TRD_SB + rsub) * ld + base + c4;
  for (int Jb = wave; Jb <= I; Jb += 4) {
    vfloat4_t a[16];
#pragma unroll
    for (int it = 0; it < 16; ++it)
      a[it] = __builtin_nontemporal_load(reinterpret_cast<const vfloat4_t*>(Trow + (long long)(4 * it) * ld + Jb * TRD_SB));
    const float4 vj = *reinterpret_cast<const float4*>(vs + Jb * TRD_SB + c4);
    if (Jb == I) {
      // Diagonal tile: only its lower triangle is used, like everywhere else (the two triangles of the matrix agree to
      // rounding only, and on the numerically zero trailing blocks of a rank-deficient factor the rounding is all
      // there is).  Entries above the diagonal are dropped and come back as the column sums of the strictly lower ones.
#pragma unroll
      for (int it = 0; it < 16; ++it) {
        const int rl = rsub + 4 * it;  // row inside the tile
        a[it].x = (c4 + 0 <= rl) ? a[it].x : 0.f;
        a[it].y = (c4 + 1 <= rl) ? a[it].y : 0.f;
        a[it].z = (c4 + 2 <= rl) ? a[it].z : 0.f;
        a[it].w = (c4 + 3 <= rl) ? a[it].w : 0.f;
      }
    }
#pragma unroll
    for (int it = 0; it < 16; ++it) racc[it] += (a[it].x * vj.x + a[it].y * vj.y) + (a[it].z * vj.z + a[it].w * vj.w);
    if (Jb == I) {  // strictly lower part for the column sums
#pragma unroll
      for (int it = 0; it < 16; ++it) {
        const int rl = rsub + 4 * it;
        a[it].x = (c4 + 0 < rl) ? a[it].x : 0.f;
        a[it].y = (c4 + 1 < rl) ? a[it].y : 0.f;
        a[it].z = (c4 + 2 < rl) ? a[it].z : 0.f;
        a[it].w = (c4 + 3 < rl) ? a[it].w : 0.f;
      }
    }
    float4 cs = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int it = 0; it < 16; ++it) {
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
    if (lane < 16) {
      float4* dst = reinterpret_cast<float4*>(acc + Jb * TRD_SB + c4);
      float4 old = *dst;
      old.x += cs.x; old.y += cs.y; old.z += cs.z; old.w += cs.w;
      *dst = old;
    }
  }
  // row sums of the wavefront's tiles, then of the four wavefronts
#pragma unroll
  for (int it = 0; it < 16; ++it) {
    float t = racc[it];
#pragma unroll
    for (int o = 1; o <= 8; o <<= 1) t += __shfl_xor(t, o, 64);
    if ((lane & 15) == 0) rs[wave][rsub + 4 * it] = t;
  }
  __syncthreads();
  if (threadIdx.x < TRD_SB)
    J.ybuf[base + I * TRD_SB + threadIdx.x] = (rs[0][threadIdx.x] + rs[1][threadIdx.x]) + (rs[2][threadIdx.x] + rs[3][threadIdx.x]);
  __syncthreads();
}

// The first aux_wgs workgroups of a factor do not take part in the product: they compute the row terms of column step
// aux_j (trd_aux_rows), which depend on the column step before this launch only.  j < 0: no product in this launch.
__global__ __launch_bounds__(256) void trd_symv_kernel(const TrdJob* __restrict__ jobs, int j, int aux_wgs, int aux_j,
                                                       int aux_p0, int aux_flags) {
  extern __shared__ float vs[];
  __shared__ float rs[4][TRD_SB];
  const TrdJob& J = jobs[blockIdx.y];
  if ((int)blockIdx.x < aux_wgs) {
    trd_aux_rows(J, aux_j, aux_p0, aux_flags, blockIdx.x, vs);
    return;
  }
  if (j < 0) return;
  const int bx = (int)blockIdx.x - aux_wgs;
  const int d = J.d;
  const int base = (j + 1) & ~(TRD_SB - 1);
  const int nbk = (d - base + TRD_SB - 1) / TRD_SB;
  if (2 * bx >= nbk) return;
  float* acc = vs + nbk * TRD_SB;
  for (int c = threadIdx.x; c < nbk * TRD_SB; c += 256) {
    vs[c] = (base + c > j && base + c < d) ? J.vbuf[base + c] : 0.f;
    acc[c] = 0.f;
  }
  __syncthreads();
  const int I0 = bx, I1 = nbk - 1 - bx;
  trd_symv_row_block(J, vs, acc, rs, base, I0);
  if (I1 != I0) trd_symv_row_block(J, vs, acc, rs, base, I1);
  float* __restrict__ out = J.part + (long long)bx * nbk * TRD_SB;
  for (int c = threadIdx.x; c < nbk * TRD_SB; c += 256) out[c] = acc[c];
}

// Triangular factor of a block reflector of TRD_QB = 128 Householder vectors (the width the matrix-core tiles want for
// the accumulation of Q1): H_p0 ... H_p0+127 = I - V T V^T with T from the Gram matrix S = V^T V of the vectors (computed
// beforehand by a grouped product) by the slarft recurrence T[0:c, c] = -tau_c T[0:c, 0:c] S[0:c, c], T[c][c] = tau_c.
// grid (blocks, factors); S and T of the block sit in LDS (2 x 64 KB).
constexpr int TRD_QB = 128;
__global__ __launch_bounds__(256) void trd_tfactor128_kernel(const TrdJob* __restrict__ jobs) {
  extern __shared__ float lds_t128[];
  float* S = lds_t128;                       // [128][128]
  float* Tm = lds_t128 + TRD_QB * TRD_QB;    // [128][128]
  __shared__ float taus[TRD_QB];
  const TrdJob& J = jobs[blockIdx.y];
  const int d = J.d, p0 = blockIdx.x * TRD_QB, tid = threadIdx.x;
  if (p0 >= d - 1) return;
  const float* __restrict__ Sg = J.S128 + (long long)blockIdx.x * TRD_QB * TRD_QB;
  float* __restrict__ Tg = J.T128 + (long long)blockIdx.x * TRD_QB * TRD_QB;
  for (int e = tid; e < TRD_QB * TRD_QB; e += 256) { S[e] = Sg[e]; Tm[e] = 0.f; }
  if (tid < TRD_QB) taus[tid] = (p0 + tid < d - 1) ? J.tau[p0 + tid] : 0.f;
  __syncthreads();
  for (int c = 0; c < TRD_QB; ++c) {
    if (tid < c) {
      float a = 0.f;
      for (int m = tid; m < c; ++m) a += Tm[tid * TRD_QB + m] * S[m * TRD_QB + c];
      Tm[tid * TRD_QB + c] = -taus[c] * a;
    }
    if (tid == c) Tm[c * TRD_QB + c] = taus[c];
    __syncthreads();
  }
  for (int e = tid; e < TRD_QB * TRD_QB; e += 256) Tg[e] = Tm[e];
}

// dst = src^T for the leading d x d part of two dpad-strided matrices; grid (ceil(d / 32), ceil(d / 32), factors), 256 threads.
struct TransposeJob { const float* src; float* dst; int d, ld; };
__global__ __launch_bounds__(256) void trd_transpose_kernel(const TransposeJob* __restrict__ jobs) {
  __shared__ float tile[32][33];
  const TransposeJob& J = jobs[blockIdx.z];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  for (int rr = ty; rr < 32; rr += 8) {
    const int r = blockIdx.y * 32 + rr, c = blockIdx.x * 32 + tx;
    tile[rr][tx] = (r < J.d && c < J.d) ? J.src[(long long)r * J.ld + c] : 0.f;
  }
  __syncthreads();
  for (int rr = ty; rr < 32; rr += 8) {
    const int r = blockIdx.x * 32 + rr, c = blockIdx.y * 32 + tx;
    if (r < J.d && c < J.d) J.dst[(long long)r * J.ld + c] = tile[tx][rr];
  }
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

// ---------------------------------------------------------------------------------------------------------------
// Eigendecomposition of the tridiagonal matrix by bisection and inverse iteration, every eigenpair on its own thread.
//
// The implicit QL iteration above is a chain of dependent rotations per factor (one wavefront per factor) whose
// rotations then have to be applied to d rows; with d eigenvalues per factor and tens of factors per batch there is far
// more parallelism in treating every eigenvalue separately:
//   tdc_setup_kernel    scales T to unit largest entry, cuts it where an off-diagonal entry is negligible (the QL
//                       iteration's deflation criterion) and records the unreduced block of every index;
//   tdc_bisect_kernel   eigenvalue k of a block = the point where the Sturm count passes k, by bisection in fp64 from the
//                       block's Gershgorin interval down to the last bit;
//   tdc_invit_kernel    (T - sigma I) x = b by LU with partial pivoting (LAPACK's dlagtf / dlagts recurrences), three
//                       iterations from a pseudo-random start; shifts of eigenvalues closer than 2e-15 are spread apart;
//   tdc_cluster_kernel  modified Gram-Schmidt inside runs of eigenvalues closer than TDC_CLUSTER (fp64 shifts separate
//                       everything wider apart to better than 5e-6 in orthogonality);
//   tdc_verify_kernel   residual, norm and neighbour orthogonality of every vector; a factor that fails is flagged and
//                       left to the QL iteration.
// All recurrences run in fp64 on the fp32 entries of T: what matters is that eigenvalues 1e-10 apart (the noise floor of a
// rank-deficient factor holds hundreds of them) still get distinct shifts and therefore independent, orthogonal vectors.
// ---------------------------------------------------------------------------------------------------------------
constexpr double TDC_CLUSTER = 2e-11;   // relative to the largest entry of T
constexpr int TDC_MAX_CLUSTER = 48;
constexpr double TDC_PIVMIN = 1e-30;

__global__ __launch_bounds__(256) void tdc_setup_kernel(const TrdJob* __restrict__ jobs) {
  __shared__ float red[4];
  __shared__ int last_bnd[256], first_bnd[256];
  const TrdJob& J = jobs[blockIdx.x];
  const int d = J.d, tid = threadIdx.x;
  float m = 0.f;
  for (int i = tid; i < d; i += 256) {
    m = fmaxf(m, fabsf(J.diag[i]));
    if (i < d - 1) m = fmaxf(m, fabsf(J.off[i]));
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if ((tid & 63) == 0) red[tid >> 6] = m;
  __syncthreads();
  const float tn = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const double inv = (tn > 0.f) ? 1.0 / (double)tn : 1.0;
  for (int i = tid; i < d; i += 256) {
    J.qd[i] = (double)J.diag[i] * inv;
    J.qe[i] = (i < d - 1) ? (double)J.off[i] * inv : 0.0;
  }
  if (tid == 0) {
    J.state[0] = 0; J.state[1] = 0; J.state[2] = 0; J.state[3] = 0; J.state[4] = 0;
    J.state[5] = __float_as_int((tn > 0.f) ? tn : 1.0f);
    J.hdr[0] = 0;
    J.hdr[TQL_HDR] = 0;
    *J.fail = 0;
  }
  __syncthreads();
  // index i starts a block when the entry that couples it to i - 1 is negligible; every thread owns a run of indices
  const double eps = 1.1920929e-7, abs_tol = 1.4901161e-8;
  auto starts = [&](int i) -> bool {
    if (i == 0) return true;
    const double av = fabs(J.qe[i - 1]);
    return (av <= eps * (fabs(J.qd[i - 1]) + fabs(J.qd[i]))) || (av <= abs_tol);
  };
  const int per = (d + 255) / 256;
  const int i0 = min(tid * per, d), i1 = min(i0 + per, d);
  int lastb = -1, firstb = 0x7fffffff;
  for (int i = i0; i < i1; ++i)
    if (starts(i)) { lastb = i; if (firstb == 0x7fffffff) firstb = i; }
  last_bnd[tid] = lastb;
  first_bnd[tid] = firstb;
  __syncthreads();
  int carry = -1;  // last boundary before this thread's run
  for (int t = tid - 1; t >= 0 && carry < 0; --t) carry = last_bnd[t];
  int nxt = d;     // first boundary after this thread's run
  for (int t = tid + 1; t < 256 && nxt == d; ++t)
    if (first_bnd[t] != 0x7fffffff) nxt = first_bnd[t];
  for (int i = i0; i < i1; ++i) {
    if (starts(i)) carry = i;
    J.blk_s[i] = carry;
  }
  for (int i = i1 - 1; i >= i0; --i) {
    J.blk_e[i] = nxt;
    if (starts(i)) nxt = i;
  }
}

// grid (ceil(d / 256), factors); dynamic LDS: 2 * dpad doubles (diagonal, squared off-diagonal).
__global__ __launch_bounds__(256) void tdc_bisect_kernel(const TrdJob* __restrict__ jobs) {
  extern __shared__ double lds64[];
  const TrdJob& J = jobs[blockIdx.y];
  const int d = J.d, dpad = J.dpad;
  double* dd = lds64;
  double* e2 = lds64 + dpad;
  for (int i = threadIdx.x; i < d; i += 256) {
    dd[i] = J.qd[i];
    const double e = J.qe[i];
    e2[i] = e * e;
  }
  __syncthreads();
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= d) return;
  const int s = J.blk_s[i], t = J.blk_e[i], k = i - s;
  if (t - s == 1) { J.lam[i] = dd[s]; return; }
  // Gershgorin interval of the block
  double lo = 1e300, hi = -1e300;
  for (int r = s; r < t; ++r) {
    const double rad = (r > s ? sqrt(e2[r - 1]) : 0.0) + (r < t - 1 ? sqrt(e2[r]) : 0.0);
    lo = fmin(lo, dd[r] - rad);
    hi = fmax(hi, dd[r] + rad);
  }
  const double width = hi - lo;
  lo -= 1e-14 * width + 1e-300;
  hi += 1e-14 * width + 1e-300;
  for (int it = 0; it < 64; ++it) {
    const double mid = 0.5 * (lo + hi);
    if (mid <= lo || mid >= hi) break;  // the interval is down to neighbouring numbers
    // Number of eigenvalues of the block below mid: sign changes in the sequence of leading principal minors of
    // T - mid I, p_i = (d_i - mid) p_(i-1) - e_(i-1)^2 p_(i-2) with p_(-1) = 1.  The pivots of the LDL^T factorisation are
    // the ratios p_i / p_(i-1); dividing at every row makes a chain of a reciprocal, its refinement and a product per
    // row (250 cycles), the minors themselves one fused multiply-add.  A minor that is exactly zero counts as positive,
    // and the one after it has the sign opposite to the one before it, so the pair still counts one change.  The pair is
    // scaled back to magnitude one after every TDC_PF rows: a row multiplies it by at most 4 and, inside an unreduced
    // block (|e| > 1.5e-8), by no less than 1.5e-8 on average, so TDC_PF rows stay far inside the range of a double.
    double p2 = 1.0, p1 = dd[s] - mid;
    unsigned neg = (unsigned)__double2hiint(p1) >> 31;
    int cnt = (int)neg;
    int r0 = s + 1;
    for (; r0 + TDC_PF <= t; r0 += TDC_PF) {
      // the operands of a block of rows are read from LDS before the dependent chain of the block starts
      double a[TDC_PF], b[TDC_PF];
#pragma unroll
      for (int j = 0; j < TDC_PF; ++j) {
        a[j] = dd[r0 + j] - mid;
        b[j] = e2[r0 + j - 1];
      }
      unsigned signs = neg;  // the signs of the minors, the newest in bit 0
#pragma unroll
      for (int j = 0; j < TDC_PF; ++j) {
        const double p = fma(a[j], p1, -(b[j] * p2));
        signs = __builtin_amdgcn_alignbit(signs, (unsigned)__double2hiint(p), 31);  // (signs << 1) | sign of p
        p2 = p1;
        p1 = p;
      }
      static_assert(TDC_PF == 16, "the sign word below holds the previous minor and sixteen new ones");
      cnt += __popc((signs ^ (signs >> 1)) & 0xffffu);
      neg = signs & 1u;
      const double m = fmax(fabs(p1), fabs(p2));
      if (m > 0.0) {
        const int ex = ilogb(m);
        p1 = ldexp(p1, -ex);
        p2 = ldexp(p2, -ex);
      }
    }
    for (; r0 < t; ++r0) {  // fewer than TDC_PF rows are left
      const double p = fma(dd[r0] - mid, p1, -(e2[r0 - 1] * p2));
      const unsigned n = (unsigned)__double2hiint(p) >> 31;
      cnt += (int)(n ^ neg);
      neg = n;
      p2 = p1;
      p1 = p;
    }
    if (cnt > k) hi = mid; else lo = mid;
  }
  J.lam[i] = 0.5 * (lo + hi);
}

__device__ __forceinline__ double tdc_random(unsigned int i, unsigned int k, unsigned int salt) {
  // a hash of (eigenvalue index, row, iteration) mapped to (-1, 1); any start vector with a component along the
  // wanted eigenvector will do
  unsigned int h = i * 0x9E3779B1u ^ (k + 0x7F4A7C15u) * 0x85EBCA6Bu ^ salt * 0xC2B2AE35u;
  h ^= h >> 15; h *= 0x2C1B3C6Du; h ^= h >> 12; h *= 0x297A2D39u; h ^= h >> 15;
  return ((double)(h & 0xffffffu) + 0.5) * (2.0 / 16777216.0) - 1.0;
}

// grid (ceil(chunk / 128), factors), 128 threads; `first` = eigenvalue index of the chunk's first thread.  The entries of
// T are read from memory as they are needed (one factorisation pass; the lanes of a wavefront mostly share a block and
// therefore the address).
__global__ __launch_bounds__(128) void tdc_invit_kernel(const TrdJob* __restrict__ jobs, int first) {
  const TrdJob& J = jobs[blockIdx.y];
  const int d = J.d, dpad = J.dpad, E = J.chunk;
  const double* __restrict__ dd = J.qd;
  const double* __restrict__ ee = J.qe;
  const int tl = blockIdx.x * 128 + threadIdx.x;  // position inside the chunk
  const int i = first + tl;
  if (tl >= E || i >= d) return;
  const int s = J.blk_s[i], t = J.blk_e[i];
  float* __restrict__ Zc = J.Z + i;
  const long long ld = dpad;
  if (t - s == 1) {
    for (int r = 0; r < dpad; ++r) Zc[(long long)r * ld] = (r == s) ? 1.0f : 0.0f;
    return;
  }
  // shifts of (nearly) coincident eigenvalues are spread by 2e-15 so that their vectors can differ
  const double pertol = 2e-15;
  double sigma = J.lam[i];
  for (int j = max(s, i - 31); j < i; ++j) sigma = fmax(sigma, J.lam[j] + (double)(i - j) * pertol);

  double* __restrict__ ua = J.lu_a + tl;
  double* __restrict__ ub = J.lu_b + tl;
  double* __restrict__ ud = J.lu_d + tl;
  double* __restrict__ lc = J.lu_c + tl;
  double* __restrict__ xv = J.lu_x + tl;
  unsigned char* __restrict__ fl = J.lu_f + tl;
  // Every pass below is one dependent recurrence per row whose operands do not depend on it: they are fetched a block of
  // TDC_PF rows ahead (all loads of a block in flight together), otherwise each row would cost a full memory latency.
  constexpr int PF = TDC_PF;
  // ---- LU with partial pivoting of T - sigma I over rows s .. t - 1
  {
    double ak = dd[s] - sigma, bk = ee[s];
    for (int k0 = s; k0 < t - 1; k0 += PF) {
      double dn[PF], ec[PF + 1];
#pragma unroll
      for (int j = 0; j < PF; ++j) dn[j] = dd[min(k0 + j + 1, t - 1)];
#pragma unroll
      for (int j = 0; j <= PF; ++j) ec[j] = ee[min(k0 + j, t - 1)];
#pragma unroll
      for (int j = 0; j < PF; ++j) {
        const int k = k0 + j;
        if (k < t - 1) {
          const double ck = ec[j];                 // entry below the pivot
          const double an = dn[j] - sigma;         // next row as it stands: (ck, an, ee[k + 1])
          const double en = (k + 1 < t - 1) ? ec[j + 1] : 0.0;
          const long long o = (long long)k * E;
          if (fabs(ak) >= fabs(ck)) {
            const double mult = (ak != 0.0) ? ck / ak : 0.0;
            ua[o] = ak; ub[o] = bk; ud[o] = 0.0; lc[o] = mult; fl[o] = 0;
            ak = an - mult * bk;
            bk = en;
          } else {
            const double mult = ak / ck;
            ua[o] = ck; ub[o] = an; ud[o] = en; lc[o] = mult; fl[o] = 1;
            ak = bk - mult * an;
            bk = -mult * en;
          }
        }
      }
    }
    const long long o = (long long)(t - 1) * E;
    ua[o] = ak; ub[o] = 0.0; ud[o] = 0.0; lc[o] = 0.0; fl[o] = 0;
  }
  // ---- inverse iteration
  const double tiny = 1e-18;
  double scale = 1.0, sumsq = 0.0;
  for (int it = 0; it < 3; ++it) {
    // forward substitution with the row interchanges; the first right-hand side is pseudo-random, later ones are the
    // previous iterate scaled to unit largest entry
    double prev = (it == 0) ? tdc_random((unsigned)i, (unsigned)s, 0u) : xv[(long long)s * E] * scale;
    for (int k0 = s + 1; k0 < t; k0 += PF) {
      double cu[PF], cc[PF];
      unsigned char ff[PF];
#pragma unroll
      for (int j = 0; j < PF; ++j) {
        const int k = min(k0 + j, t - 1);
        cu[j] = (it == 0) ? 0.0 : xv[(long long)k * E];
        cc[j] = lc[(long long)(k - 1) * E];
        ff[j] = fl[(long long)(k - 1) * E];
      }
#pragma unroll
      for (int j = 0; j < PF; ++j) {
        const int k = k0 + j;
        if (k < t) {
          const double cur = (it == 0) ? tdc_random((unsigned)i, (unsigned)k, 0u) : cu[j] * scale;
          const double c = cc[j];
          double keep, next;
          if (ff[j]) { keep = cur; next = prev - c * cur; } else { keep = prev; next = cur - c * prev; }
          xv[(long long)(k - 1) * E] = keep;
          prev = next;
        }
      }
    }
    xv[(long long)(t - 1) * E] = prev;
    // back substitution; pivots below `tiny` are pushed away from zero
    double x1 = 0.0, x2 = 0.0, big = 0.0;
    sumsq = 0.0;
    for (int k0 = t - 1; k0 >= s; k0 -= PF) {
      double pa[PF], pb[PF], pd[PF], px[PF];
#pragma unroll
      for (int j = 0; j < PF; ++j) {
        const long long o = (long long)max(k0 - j, s) * E;
        pa[j] = ua[o]; pb[j] = ub[o]; pd[j] = ud[o]; px[j] = xv[o];
      }
#pragma unroll
      for (int j = 0; j < PF; ++j) {
        const int k = k0 - j;
        if (k >= s) {
          double a = pa[j];
          if (fabs(a) < tiny) a = (a < 0.0) ? -tiny : tiny;
          const double x = (px[j] - pb[j] * x1 - pd[j] * x2) / a;
          xv[(long long)k * E] = x;
          x2 = x1;
          x1 = x;
          big = fmax(big, fabs(x));
          sumsq += x * x;
        }
      }
    }
    scale = (big > 0.0 && big < 1e300) ? 1.0 / big : 1.0;
  }
  const double inv = (sumsq > 0.0 && sumsq < 1e300) ? 1.0 / sqrt(sumsq) : 0.0;
  for (int r = 0; r < dpad; ++r) Zc[(long long)r * ld] = (r >= s && r < t) ? (float)(xv[(long long)r * E] * inv) : 0.0f;
}

// One wavefront per eigenvalue index; the one that starts a run of close eigenvalues orthonormalises the run.
// grid (d, factors), 64 threads.
__global__ __launch_bounds__(64) void tdc_cluster_kernel(const TrdJob* __restrict__ jobs) {
  const TrdJob& J = jobs[blockIdx.y];
  const int d = J.d, i = blockIdx.x, lane = threadIdx.x;
  if (i >= d) return;
  const int s = J.blk_s[i], t = J.blk_e[i];
  if (i > s && J.lam[i] - J.lam[i - 1] < TDC_CLUSTER) return;  // inside a run, not its start
  int last = i;
  while (last + 1 < t && J.lam[last + 1] - J.lam[last] < TDC_CLUSTER) ++last;
  if (last == i) return;
  if (last - i + 1 > TDC_MAX_CLUSTER) {
    if (lane == 0) *J.fail = 1;
    return;
  }
  const long long ld = J.dpad;
  for (int a = i; a <= last; ++a) {
    float* __restrict__ za = J.Z + a;
    for (int pass = 0; pass < 2; ++pass)  // twice is enough
      for (int b = i; b < a; ++b) {
        const float* __restrict__ zb = J.Z + b;
        double dot = 0.0;
        for (int r = s + lane; r < t; r += 64) dot += (double)za[(long long)r * ld] * (double)zb[(long long)r * ld];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) dot += __shfl_xor(dot, o, 64);
        for (int r = s + lane; r < t; r += 64) za[(long long)r * ld] = (float)((double)za[(long long)r * ld] - dot * (double)zb[(long long)r * ld]);
      }
    double nn = 0.0;
    for (int r = s + lane; r < t; r += 64) { const double v = za[(long long)r * ld]; nn += v * v; }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) nn += __shfl_xor(nn, o, 64);
    const double inv = nn > 0.0 ? 1.0 / sqrt(nn) : 0.0;
    if (!(nn > 1e-12)) { if (lane == 0) *J.fail = 1; }
    for (int r = s + lane; r < t; r += 64) za[(long long)r * ld] = (float)((double)za[(long long)r * ld] * inv);
  }
}

// Every vector: |T z - lambda z|_max, |z|^2 and z . z_next (next eigenvalue of the same block); eigenvalues to diag.
// grid (ceil(d / 256), factors).
__global__ __launch_bounds__(256) void tdc_verify_kernel(const TrdJob* __restrict__ jobs) {
  const TrdJob& J = jobs[blockIdx.y];
  const int d = J.d;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= d) return;
  const int s = J.blk_s[i], t = J.blk_e[i];
  const long long ld = J.dpad;
  const float* __restrict__ z = J.Z + i;
  const bool has_next = (i + 1 < t);
  const double lam = J.lam[i];
  double res = 0.0, nn = 0.0, dot = 0.0;
  double zm = 0.0, zc = z[(long long)s * ld];
  for (int r = s; r < t; ++r) {
    const double zn = (r + 1 < t) ? (double)z[(long long)(r + 1) * ld] : 0.0;
    const double tz = (r > s ? J.qe[r - 1] * zm : 0.0) + J.qd[r] * zc + (r + 1 < t ? J.qe[r] * zn : 0.0);
    res = fmax(res, fabs(tz - lam * zc));
    nn += zc * zc;
    if (has_next) dot += zc * (double)z[(long long)r * ld + 1];
    zm = zc;
    zc = zn;
  }
  const bool ok = (res <= 2e-5) && (fabs(nn - 1.0) <= 1e-4) && (fabs(dot) <= 2e-5);
  if (!ok) *J.fail = 1;  // also taken when a value is nan
  J.diag[i] = (float)(lam * (double)__int_as_float(J.state[5]));
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
