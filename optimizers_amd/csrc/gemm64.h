// fp64 path of the coupled Newton root inverse for factor matrices kept in double precision
// (factor_matrix_dtype = torch.float64 in the reference: the factor is accumulated and inverted in fp64, the inverse
// root is stored in fp32).  A grouped fp64 MFMA GEMM for gfx950 on square, zero padded operands, and the three small
// kernels around it: norm / finiteness of the ridged factor, start matrices, commit of the result.
//
// GEMM: a workgroup of 256 threads (4 wavefronts, 2 x 2) owns a 128 x 128 tile of C; each wavefront owns 64 x 64
// of it as 4 x 4 v_mfma_f64_16x16x4_f64 accumulators (4 doubles per lane each).  K is consumed in slabs of 8 staged
// through LDS k-major ([k][m] / [k][n], pitch 130 doubles), double buffered like the fp32 kernel (one such
// instruction keeps the matrix pipe busy for 64 cycles, so a slab is 2048 cycles of MFMA work per wavefront).
// Register layout of the instruction: A lane l = A[l % 16][l / 16], B lane l = B[l / 16][l % 16],
// D lane l, value r = D[4 r + l / 16][l % 16].
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm.h"

namespace sa {

typedef double doublex4 __attribute__((ext_vector_type(4)));

constexpr int BM64 = 128;
constexpr int BK64 = 8;
constexpr int LDS64_PITCH = 130;

enum Epilogue64 {
  EPI64_STORE = 0,     // C = acc
  EPI64_NEWTON_M = 1,  // C = acc (new M), C2 = acc * mp_scale + mp_diag * I, err = max |acc - I| over d x d
};

// C = A B with A(m,k) = A[m * n + k], B(k,j) = B[k * n + j]; all matrices n x n, n a multiple of 128.
struct GemmProblem64 {
  const double* A;
  const double* B;
  double* C;
  double* C2;
  unsigned int* err_bits;  // atomicMax target (bit pattern of a non-negative float)
  const int* active;       // optional: skip the problem when *active == 0
  int n;                   // padded order
  int d;                   // true order
  int tiles;               // n / 128
  int tile_begin;
};

template <int EPI>
__global__ __launch_bounds__(GEMM_THREADS) void grouped_gemm64_kernel(const GemmProblem64* __restrict__ problems,
                                                                     int n_problems, int total_tiles, double mp_scale,
                                                                     double mp_diag) {
  __shared__ __attribute__((aligned(16))) double As[2][BK64 * LDS64_PITCH];
  __shared__ __attribute__((aligned(16))) double Bs[2][BK64 * LDS64_PITCH];

  const int per_xcd = (total_tiles + NUM_XCD - 1) / NUM_XCD;
  const int logical = (blockIdx.x % NUM_XCD) * per_xcd + blockIdx.x / NUM_XCD;
  if (logical >= total_tiles) return;
  int lo = 0, hi = n_problems - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (problems[mid].tile_begin <= logical) lo = mid; else hi = mid - 1;
  }
  const GemmProblem64& P = problems[lo];
  if (P.active != nullptr && *P.active == 0) return;

  int tm, tn;
  {
    const int t = logical - P.tile_begin;
    const int per_group = GROUP_ROWS * P.tiles;
    const int g = t / per_group, r = t - g * per_group;
    const int first = g * GROUP_ROWS;
    const int gsz = min(P.tiles - first, GROUP_ROWS);
    tm = first + r % gsz;
    tn = r / gsz;
  }
  const int n = P.n;
  const int m0 = tm * BM64, n0 = tn * BM64;
  const double* __restrict__ A = P.A;
  const double* __restrict__ B = P.B;

  const int t = threadIdx.x;
  const int lane = t & 63, wave = t >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l16 = lane & 15, kq = lane >> 4;

  doublex4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = doublex4{0.0, 0.0, 0.0, 0.0};

  // A slab: 128 rows x 8 k, thread -> row t / 2, four consecutive k; B slab: 8 k x 128 cols, thread -> k t / 32,
  // four consecutive cols
  const int a_row = t >> 1, a_k = (t & 1) * 4;
  const int b_k = t >> 5, b_col = (t & 31) * 4;
  double2 ra[2], rb[2];
  auto load = [&](int k0) {
    const double* pa = A + (long long)(m0 + a_row) * n + k0 + a_k;
    const double* pb = B + (long long)(k0 + b_k) * n + n0 + b_col;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      ra[q] = *reinterpret_cast<const double2*>(pa + 2 * q);
      rb[q] = *reinterpret_cast<const double2*>(pb + 2 * q);
    }
  };
  auto store = [&](int buf) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      As[buf][(a_k + 2 * q) * LDS64_PITCH + a_row] = ra[q].x;
      As[buf][(a_k + 2 * q + 1) * LDS64_PITCH + a_row] = ra[q].y;
      *reinterpret_cast<double2*>(&Bs[buf][b_k * LDS64_PITCH + b_col + 2 * q]) = rb[q];
    }
  };

  const int slabs = n / BK64;
  load(0);
  store(0);
  __syncthreads();
  for (int s = 0; s < slabs; ++s) {
    const int cur = s & 1;
    const bool more = (s + 1 < slabs);
    if (more) load((s + 1) * BK64);
    const double* as = As[cur] + wm * 64 + l16;
    const double* bs = Bs[cur] + wn * 64 + l16;
#pragma unroll
    for (int ks = 0; ks < BK64 / 4; ++ks) {
      const int krow = (ks * 4 + kq) * LDS64_PITCH;
      double a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { a[i] = as[krow + 16 * i]; b[i] = bs[krow + 16 * i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (more) store(cur ^ 1);
    __syncthreads();
  }

  // accumulator value r of block (i, j): row = 16 i + 4 r + kq, col = 16 j + l16
  double local = 0.0;
  bool local_nan = false;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + wn * 64 + 16 * j + l16;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = m0 + wm * 64 + 16 * i + 4 * r + kq;
        const double v = acc[i][j][r];
        const long long o = (long long)row * n + col;
        P.C[o] = v;
        if (EPI == EPI64_NEWTON_M) {
          double mp = v * mp_scale;
          if (row == col && row < P.d) mp += mp_diag;
          P.C2[o] = mp;
          if (row < P.d && col < P.d) {
            const double dv = fabs(v - (row == col ? 1.0 : 0.0));
            if (dv != dv) local_nan = true;
            local = fmax(local, dv);
          }
        }
      }
    }
  }
  if (EPI == EPI64_NEWTON_M) {
    // the error is compared with a tolerance, not accumulated: single precision (rounded up) carries it
    float e = local_nan ? __builtin_nanf("") : __double2float_ru(local);
    e = wave_max_nan(e);
    if (lane == 0) atomicMax(P.err_bits, __float_as_uint(e != e ? __builtin_nanf("") : e));
  }
}

// ---- around the iteration ---------------------------------------------------------------------------------

struct Factor64 {
  const double* packed;  // row-major upper triangle, d (d + 1) / 2 doubles
  double* M;             // dense n x n outputs of the start kernel
  double* Mp;
  double* X;
  double* X1;            // x0 * M_p: the first X M_p (X is a multiple of the identity, the other terms are exact zeros)
  const double* result;  // dense n x n input of the commit kernel
  float* inv_packed;     // fp32 upper triangle of the result
  float* inv_dense;      // fp32 dense, mirrored from the upper triangle, n x n zero padded
  double* norm_sq;       // || factor / bc2 + ridge I ||_F^2
  int* nonfinite;
  double ridge;          // multiple of the identity added to the bias-corrected factor
  int d, n;
};

__device__ __forceinline__ long long packed_index(int r, int c, int d) {  // r <= c
  return (long long)r * d - ((long long)r * (r - 1)) / 2 + (c - r);
}

// One workgroup per factor: squared Frobenius norm of A = factor / bc2 + ridge I (fp64, fixed summation order) and a
// flag for non-finite entries of the bias-corrected factor.
__global__ __launch_bounds__(256) void f64_norm_kernel(const Factor64* __restrict__ jobs, double bc2) {
  __shared__ double red[256];
  __shared__ int bad;
  const Factor64& J = jobs[blockIdx.x];
  if (threadIdx.x == 0) bad = 0;
  __syncthreads();
  const int d = J.d;
  const double eps = J.ridge;
  double acc = 0.0;
  bool nonfinite = false;
  for (int r = 0; r < d; ++r) {
    const double* row = J.packed + packed_index(r, r, d);
    for (int c = r + threadIdx.x; c < d; c += 256) {
      const double v = row[c - r] / bc2;
      if (!(fabs(v) <= 1.7976931348623157e308)) nonfinite = true;
      const double a = (c == r) ? v + eps : v;
      acc += (c == r) ? a * a : 2.0 * a * a;
    }
  }
  if (nonfinite) bad = 1;
  red[threadIdx.x] = acc;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) red[threadIdx.x] += red[threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    *J.norm_sq = red[0];
    if (bad) *J.nonfinite = 1;
  }
}

// Start of the coupled Newton iteration (matrix_functions.py:400-414) in fp64: z = (p + 1) / (2 ||A||_F),
// X = z^(1/p) I, M = z A, M_p = alpha M + (1 - alpha) I; zero padding outside d x d.  grid (x, factors).
__global__ __launch_bounds__(256) void f64_newton_start_kernel(const Factor64* __restrict__ jobs, double bc2, int root,
                                                              double alpha, double one_minus_alpha) {
  const Factor64& J = jobs[blockIdx.y];
  const int d = J.d, n = J.n;
  const double eps = J.ridge;
  const double z = (root + 1.0) / (2.0 * sqrt(*J.norm_sq));
  const double x0 = pow(z, 1.0 / root);
  const long long total = (long long)n * n;
  for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < total; e += (long long)gridDim.x * 256) {
    const int r = (int)(e / n), c = (int)(e - (long long)r * n);
    double m = 0.0, mp = 0.0, x = 0.0;
    if (r < d && c < d) {
      double a = J.packed[r <= c ? packed_index(r, c, d) : packed_index(c, r, d)] / bc2;
      if (r == c) a += eps;
      m = z * a;
      mp = m * alpha;
      if (r == c) { mp += one_minus_alpha; x = x0; }
    }
    J.M[e] = m;
    J.Mp[e] = mp;
    J.X[e] = x;
    J.X1[e] = x0 * mp;
  }
}

// Result -> fp32: packed upper triangle (the stored inverse root) and its mirrored dense copy; flags non-finite
// values.  grid (x, factors).
__global__ __launch_bounds__(256) void f64_commit_kernel(const Factor64* __restrict__ jobs, int check_only) {
  const Factor64& J = jobs[blockIdx.y];
  const int d = J.d, n = J.n;
  const long long total = (long long)n * n;
  bool nonfinite = false;
  for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < total; e += (long long)gridDim.x * 256) {
    const int r = (int)(e / n), c = (int)(e - (long long)r * n);
    float v = 0.0f;
    if (r < d && c < d) {
      const double x = (r <= c) ? J.result[e] : J.result[(long long)c * n + r];
      v = (float)x;
      if (!(fabsf(v) <= 3.4028234663852886e38f)) nonfinite = true;
      if (!check_only && r <= c) J.inv_packed[packed_index(r, c, d)] = v;
    }
    if (!check_only) J.inv_dense[e] = v;
  }
  if (nonfinite) *J.nonfinite = 1;
}

}  // namespace sa
