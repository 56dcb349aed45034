// Grouped fp32 MFMA GEMM for gfx950 (CDNA4), the one contraction engine behind the
// Kronecker-factor update, the coupled-Newton iteration and the preconditioning pair.
//
// One launch walks a table of independent problems C = op(A) * op(B).  A workgroup of
// 256 threads (4 wavefronts of 64, arranged 2x2) owns a 128x128 tile of C; each wavefront
// owns 64x64 of it as 2x2 v_mfma_f32_32x32x2_f32 accumulators.  K is consumed in slabs of
// 16 staged through LDS, double buffered: the global loads of slab s+1 are issued before
// the MFMAs of slab s.  Both operands live in LDS k-major ([k][m] / [k][n], row stride 132
// floats), so every MFMA fragment is one conflict-free ds_read_b32 per lane.
//
// The workgroup id -> tile mapping is XCD aware: hardware deals consecutive workgroup ids
// round-robin over the 8 XCDs, so id w is remapped to (w % 8) * ceil(T/8) + w / 8, which
// gives every XCD one contiguous run of tiles; inside a problem tiles are enumerated in
// 8-row super-rows so that a run of 64 tiles is an 8x8 patch sharing A and B panels in
// that XCD's L2.  LDS rows are padded by 4 floats (132 for the 128-wide tile): rows stay 16-byte aligned, banks are skewed.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

namespace sa {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128;
constexpr int BN = 128;
constexpr int BK = 16;
constexpr int GEMM_THREADS = 256;
constexpr int NUM_XCD = 8;
constexpr int GROUP_ROWS = 8;

// Operand storage.  A_MK: A(m,k) = A[m*lda + k]   A_KM: A(m,k) = A[k*lda + m]
//                   B_KN: B(k,n) = B[k*ldb + n]   B_NK: B(k,n) = B[n*ldb + k]
enum ALayout { A_MK = 0, A_KM = 1 };
enum BLayout { B_KN = 0, B_NK = 1 };

// Epilogues.
enum Epilogue {
  EPI_STORE = 0,        // C = acc
  EPI_STORE_SQNORM = 1, // C = acc, partial[tile] = sum(acc^2) over the tile
  EPI_SYRK_EMA = 2,     // packed upper triangle: C = beta*C + alpha*acc   (tiles tn >= tm only)
  EPI_NEWTON_M = 3,     // C = acc (new M), C2 = acc*mp_scale + mp_diag*I, err = max|acc - I| over d x d
  EPI_SQ_EMA = 4,       // C = beta*C + alpha*acc^2        (second moment in the eigenbasis)
  EPI_DIVPOW = 5,       // C = acc / ((C2 / div)^pow_exp + eps)   (C2 has the layout of C)
  EPI_SUB = 6,          // C -= acc                         (block-reflector updates of the QR refresh)
  EPI_HORNER = 7,       // C = alpha*acc + beta*C2 + mp_diag*I over d x d (C2 read only; Horner step of a matrix polynomial)
  EPI_EC_FUSED = 9,     // acc = gradient in the eigenbasis: C = beta*C + alpha*acc^2 (second moment), C2 = lerp(C2, acc, mom_w)
                        // (filtered gradient in the eigenbasis, optional), C3 = (C2 / mom_div) / ((C / div)^pow_exp + eps)
  EPI_SYRK_EMA64 = 8,   // EPI_SYRK_EMA on a packed triangle of doubles: C = beta64*C + alpha64*acc (fp32 product, fp64 average)
};

struct GemmProblem {
  const float* A;
  const float* B;
  float* C;
  float* C2;               // EPI_NEWTON_M: M_p output.  EPI_STORE_SQNORM: per-tile partial sums.  EPI_HORNER: addend (read)
  float* C3;               // EPI_EC_FUSED: preconditioned output.  EPI_DIVPOW: optional copy of acc * mom_div
  unsigned int* err_bits;  // EPI_NEWTON_M: atomicMax target (bit pattern of a non-negative float)
  const int* active;       // optional: skip the problem when *active == 0
  long long lda, ldb, ldc;
  int M, N, K;
  int tiles_m, tiles_n;
  int tile_begin;          // first logical tile id of this problem
  int tiles_m_s, tiles_n_s;  // the same three for the 64 x 64 tiles of the small-launch variant (WB = 1)
  int tile_begin_s;
  int d;                   // EPI_NEWTON_M: true (unpadded) dimension
  int a_vec, b_vec;        // operand may be read with 16-byte loads (pointer and ld aligned)
};

// Scalars shared by every problem of one launch.
struct GemmScalars {
  float a_div, b_div;      // operand is divided by this on load (1.0f = as stored)
  float alpha, beta;       // EPI_SYRK_EMA: C = beta*C + alpha*acc.  EPI_HORNER: C = alpha*acc + beta*C2 + mp_diag*I
  float mp_scale, mp_diag; // EPI_NEWTON_M: M_p = M*mp_scale + mp_diag*I
  float div, pow_exp, eps; // EPI_DIVPOW, EPI_EC_FUSED
  float mom_w, mom_div;    // EPI_EC_FUSED: C2 <- lerp(C2, acc, mom_w), numerator C2 / mom_div.  EPI_DIVPOW: C3 = acc * mom_div
  double alpha64, beta64;  // EPI_SYRK_EMA64
};

// Loads through a pointer that is known to address device memory.  Pointers that come out of a job table are
// generic to the compiler, and a generic (flat) load counts against the LDS counter as well as the memory counter:
// the wait in front of the first MFMA of a slab would then also wait for the next slab's operands.
typedef float vfloat4 __attribute__((ext_vector_type(4)));
typedef unsigned int vuint4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 gload4(const float* p) {
  const vfloat4 v = *(const __attribute__((address_space(1))) vfloat4*)p;
  return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ float gload1(const float* p) { return *(const __attribute__((address_space(1))) float*)p; }

// live_begin[i] = number of tiles of the active problems in front of problem i (i = 0 .. n), for a launch that
// passes it to grouped_gemm_kernel, followed by NUM_XCD + 1 tile offsets that cut the live tiles into one run per XCD
// of equal WORK (a tile's work is its K): problems of different orders in one launch would otherwise leave the XCDs
// that drew the long tiles running after the others have drained.  No run is longer than `cap` tiles (the launch has
// cap workgroups per XCD).  One workgroup; `triangular` = the launch computes upper-triangle tiles only.  `live_begin`
// holds live_ints(n) ints: the offsets, the cuts, and behind them the running work as 64-bit integers.
__host__ __device__ inline size_t live_work_offset(int n) { return ((size_t)n + 1 + NUM_XCD + 1 + 1) & ~(size_t)1; }
__host__ __device__ inline size_t live_ints(int n) { return live_work_offset(n) + 2 * ((size_t)n + 1); }
__global__ __launch_bounds__(256) void gemm_live_tiles_kernel(const GemmProblem* __restrict__ problems, int n, int triangular,
                                                              int* __restrict__ live_begin, int cap, int small_tiles) {
  __shared__ int part[256];
  __shared__ long long wpart[256];
  __shared__ int carry;
  __shared__ long long wcarry;
  long long* __restrict__ work_begin = reinterpret_cast<long long*>(live_begin + live_work_offset(n));
  int* __restrict__ cut = live_begin + n + 1;
  if (threadIdx.x == 0) { carry = 0; wcarry = 0; }
  __syncthreads();
  for (int base = 0; base < n; base += 256) {
    const int i = base + threadIdx.x;
    int w = 0;
    long long ww = 0;
    if (i < n) {
      const GemmProblem& P = problems[i];
      const bool on = P.active == nullptr || *P.active != 0;
      const int t_m = small_tiles ? P.tiles_m_s : P.tiles_m, t_n = small_tiles ? P.tiles_n_s : P.tiles_n;
      w = !on ? 0 : (triangular ? t_n * (t_n + 1) / 2 : t_m * t_n);
      ww = (long long)w * max(P.K, 1);
    }
    part[threadIdx.x] = w;
    wpart[threadIdx.x] = ww;
    __syncthreads();
    // inclusive scans of the 256 widths and of their work
    for (int o = 1; o < 256; o <<= 1) {
      const int add = threadIdx.x >= o ? part[threadIdx.x - o] : 0;
      const long long wadd = threadIdx.x >= o ? wpart[threadIdx.x - o] : 0;
      __syncthreads();
      part[threadIdx.x] += add;
      wpart[threadIdx.x] += wadd;
      __syncthreads();
    }
    const int c = carry;
    const long long wc = wcarry;
    if (i < n) {
      live_begin[i] = c + part[threadIdx.x] - w;
      work_begin[i] = wc + wpart[threadIdx.x] - ww;
    }
    __syncthreads();
    if (threadIdx.x == 255) { carry = c + part[255]; wcarry = wc + wpart[255]; }
    __syncthreads();
  }
  const int total = carry;
  const long long total_work = wcarry;
  if (threadIdx.x == 0) { live_begin[n] = total; work_begin[n] = total_work; cut[0] = 0; cut[NUM_XCD] = total; }
  __syncthreads();  // the offsets written above are read below by other threads of this workgroup
  if (threadIdx.x >= 1 && threadIdx.x < NUM_XCD) {
    const long long target = total_work / NUM_XCD * threadIdx.x + total_work % NUM_XCD * threadIdx.x / NUM_XCD;
    int lo = 0, hi = n - 1;  // the last problem whose work begins at or before the target
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (work_begin[mid] <= target) lo = mid; else hi = mid - 1;
    }
    const int tiles_here = live_begin[lo + 1] - live_begin[lo];
    const long long into = (target - work_begin[lo]) / max(problems[lo].K, 1);
    cut[threadIdx.x] = live_begin[lo] + (int)min((long long)tiles_here, into);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int x = 0; x < NUM_XCD; ++x) cut[x + 1] = max(cut[x], min(cut[x + 1], cut[x] + cap));  // no run above the cap ...
    cut[NUM_XCD] = total;
    for (int x = NUM_XCD - 1; x >= 1; --x) cut[x] = max(cut[x], cut[x + 1] - cap);              // ... the last one included
  }
}

__device__ __forceinline__ float4 load4_guarded(const float* p, bool vec, int valid) {
  // valid = number of in-range elements starting at p (clamped to [0,4]).
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (valid >= 4 && vec) {
    v = gload4(p);
  } else {
    if (valid > 0) v.x = gload1(p);
    if (valid > 1) v.y = gload1(p + 1);
    if (valid > 2) v.z = gload1(p + 2);
    if (valid > 3) v.w = gload1(p + 3);
  }
  return v;
}

// Fetch this thread's share of one 128 x 16 operand slab into registers.
// K_CONTIG: the operand is k-contiguous in memory (A_MK or B_NK): thread reads 4 k's of one row.
// otherwise the operand is row/col-contiguous for fixed k (A_KM or B_KN): 4 m's (or n's) of one k.
template <bool K_CONTIG, bool EDGE, int WB>
__device__ __forceinline__ void slab_load(const float* __restrict__ base, long long ld, int row0,
                                          int rows, int k0, int K, bool vec, float4 (&r)[WB]) {
  const int t = threadIdx.x;
  constexpr int PER_ROW = 16 * WB;  // 16-byte pieces of one k row of the slab (64 WB floats)
#pragma unroll
  for (int i = 0; i < WB; ++i) {
    const int idx = t + i * GEMM_THREADS;
    if (K_CONTIG) {
      const int row = idx >> 2, k = k0 + ((idx & 3) << 2);
      const float* p = base + (long long)(row0 + row) * ld + k;
      if (EDGE) {
        const int valid = (row0 + row < rows) ? (K - k) : 0;
        r[i] = load4_guarded(p, vec, valid);
      } else {
        r[i] = gload4(p);
      }
    } else {
      const int k = k0 + idx / PER_ROW, row = (idx % PER_ROW) << 2;
      const float* p = base + (long long)k * ld + row0 + row;
      if (EDGE) {
        const int valid = (k < K) ? (rows - (row0 + row)) : 0;
        r[i] = load4_guarded(p, vec, valid);
      } else {
        r[i] = gload4(p);
      }
    }
  }
}

template <bool K_CONTIG, int WB>
__device__ __forceinline__ void slab_store(float* __restrict__ lds, const float4 (&r)[WB]) {
  const int t = threadIdx.x;
  constexpr int PER_ROW = 16 * WB;
  constexpr int LDS_STRIDE = 64 * WB + 4;
#pragma unroll
  for (int i = 0; i < WB; ++i) {
    const int idx = t + i * GEMM_THREADS;
    if (K_CONTIG) {
      const int row = idx >> 2, k = (idx & 3) << 2;
      lds[(k + 0) * LDS_STRIDE + row] = r[i].x;
      lds[(k + 1) * LDS_STRIDE + row] = r[i].y;
      lds[(k + 2) * LDS_STRIDE + row] = r[i].z;
      lds[(k + 3) * LDS_STRIDE + row] = r[i].w;
    } else {
      const int k = idx / PER_ROW, row = (idx % PER_ROW) << 2;
      *reinterpret_cast<float4*>(&lds[k * LDS_STRIDE + row]) = r[i];
    }
  }
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max_nan(float v) {
  // max that propagates NaN (a NaN anywhere must end the Newton loop like torch.dist does)
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    float w = __shfl_xor(v, o, 64);
    v = (v != v || w != w) ? __builtin_nanf("") : fmaxf(v, w);
  }
  return v;
}

// TRI: the product is known to be symmetric (coupled Newton: every operand is a polynomial in the
// same matrix).  Only tiles on or above the diagonal are computed; everything above the diagonal is stored
// twice, as computed and transposed, which halves the MFMA work of a square product and leaves an exactly
// mirrored matrix (so a later product may read it through its transpose).
// LOWER (without TRI): only the tiles on or below the diagonal of a square C are computed, with the ordinary epilogue and
// nothing mirrored -- for updates of a symmetric matrix whose readers use the lower triangle only.
// WB: 32 x 32 accumulator blocks per wavefront and dimension.  2 gives the 128 x 128 workgroup tile everything is tuned
// for; 1 gives 64 x 64 tiles for launches with too few problems to fill the chip (a 512 x 512 product is 16 large tiles
// on 256 CUs, each walking the whole K alone on its CU; as 64 small tiles it finishes in a third of the time).
template <int AL, int BL, int EPI, bool EDGE, bool TRI = (EPI == EPI_SYRK_EMA || EPI == EPI_SYRK_EMA64), bool LOWER = false, int WB = 2>
__global__ __launch_bounds__(GEMM_THREADS, 4) void grouped_gemm_kernel(
    const GemmProblem* __restrict__ problems, int n_problems, int total_tiles, GemmScalars sc,
    const int* __restrict__ live_begin = nullptr) {
  // No contraction in this kernel: which of two products the compiler would fuse into an fma differs from one
  // instantiation of this template to the next, and the epilogues restate the reference's elementwise arithmetic
  // rounding by rounding (the matrix products themselves are MFMA instructions).
#pragma clang fp contract(off)
  constexpr int BM = 64 * WB, BN = 64 * WB, LDS_STRIDE = 64 * WB + 4;
  // two operand buffers of two slabs each; a slab is at least 32 x 36 floats, what a wavefront of the mirror epilogue
  // stages through the same memory
  constexpr int SLAB = (BK * LDS_STRIDE > 1152) ? BK * LDS_STRIDE : 1152;
  __shared__ __attribute__((aligned(16))) float smem[4 * SLAB];
  float (*As)[SLAB] = reinterpret_cast<float (*)[SLAB]>(smem);
  float (*Bs)[SLAB] = reinterpret_cast<float (*)[SLAB]>(smem + 2 * SLAB);
  __shared__ float red[4];
  static_assert(WB == 2 || (EPI != EPI_STORE_SQNORM), "per-tile partial sums are laid out for 128 x 128 tiles");

  // XCD-aware remap of the hardware workgroup id to a logical tile id: every XCD walks one run of consecutive tiles.
  // With live_begin (n_problems + 1 ascending tile offsets and the NUM_XCD + 1 cuts between the runs, written by
  // gemm_live_tiles_kernel) the launch walks only the tiles of the problems that are still active, in runs of equal
  // work; without it the runs hold equal numbers of tiles.
  int logical;
  if (live_begin != nullptr) {
    const int* __restrict__ cut = live_begin + n_problems + 1;
    const int x = blockIdx.x % NUM_XCD;
    logical = cut[x] + blockIdx.x / NUM_XCD;
    if (logical >= cut[x + 1]) return;
  } else {
    const int per_xcd = (total_tiles + NUM_XCD - 1) / NUM_XCD;
    logical = (blockIdx.x % NUM_XCD) * per_xcd + blockIdx.x / NUM_XCD;
    if (logical >= total_tiles) return;
  }

  // Which problem owns this tile (tile offsets ascend; of several equal offsets the last one owns the tile).
  int lo = 0, hi = n_problems - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    const int begin = live_begin != nullptr ? live_begin[mid] : (WB == 2 ? problems[mid].tile_begin : problems[mid].tile_begin_s);
    if (begin <= logical) lo = mid; else hi = mid - 1;
  }
  const GemmProblem& P = problems[lo];
  if (P.active != nullptr && *P.active == 0) return;

  int tm, tn;
  {
    int t = logical - (live_begin != nullptr ? live_begin[lo] : (WB == 2 ? P.tile_begin : P.tile_begin_s));
    const int p_tiles_m = WB == 2 ? P.tiles_m : P.tiles_m_s, p_tiles_n = WB == 2 ? P.tiles_n : P.tiles_n_s;
    if (TRI || LOWER) {
      // Upper-triangular tile enumeration in super-rows of GROUP_ROWS tile rows.  Inside a super-row the
      // tiles are walked column by column (first the little triangle at the diagonal, then full columns
      // of GROUP_ROWS tiles), so concurrently running workgroups share A row panels and B column panels.
      const int T = p_tiles_n;
      int r0 = 0;
      for (;;) {
        const int gsz = min(GROUP_ROWS, T - r0);
        const int tri = gsz * (gsz + 1) / 2;
        const int cnt = tri + (T - r0 - gsz) * gsz;
        if (t < cnt) {
          if (t < tri) {
            int c = 0;
            while (t > c) { t -= c + 1; ++c; }  // column c of the triangle holds c + 1 tiles
            tm = r0 + t;
            tn = r0 + c;
          } else {
            t -= tri;
            tm = r0 + t % gsz;
            tn = r0 + gsz + t / gsz;
          }
          break;
        }
        t -= cnt;
        r0 += gsz;
      }
    } else {
      const int per_group = GROUP_ROWS * p_tiles_n;
      const int g = t / per_group, r = t - g * per_group;
      const int first = g * GROUP_ROWS;
      const int gsz = min(p_tiles_m - first, GROUP_ROWS);
      tm = first + r % gsz;
      tn = r / gsz;
    }
    if (LOWER) { const int u = tm; tm = tn; tn = u; }
  }
  const int m0 = tm * BM, n0 = tn * BN;
  const int M = P.M, N = P.N, K = P.K;
  const float* __restrict__ A = P.A;
  const float* __restrict__ B = P.B;
  const long long lda = P.lda, ldb = P.ldb;
  const bool avec = P.a_vec != 0, bvec = P.b_vec != 0;
  const float a_div = sc.a_div, b_div = sc.b_div;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, h = lane >> 5;

  floatx16 acc[WB][WB];
#pragma unroll
  for (int i = 0; i < WB; ++i)
#pragma unroll
    for (int j = 0; j < WB; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  float4 ra[WB], rb[WB];
  float4 ra2[WB], rb2[WB];
  const int slabs = (K + BK - 1) / BK;
  // In a diagonal tile of a symmetric product the wavefront below the diagonal computes nothing that is kept (its
  // quadrant is the mirror image of the one above): it takes part in the loads and barriers and leaves the matrix
  // cores of its SIMD to the other workgroups there.
  const bool idle_quadrant = TRI && tm == tn && wm > wn;

  // A launch that may hold ragged problems (EDGE) still runs the unguarded loop on every problem whose K is a whole
  // number of slab pairs and whose operands allow 16-byte loads and fit a buffer resource, ragged M and N included:
  // the threads that would fetch rows or columns past M or N are pointed past the resource and get zeros.
  bool fast_loop = true;
  if constexpr (EDGE) {
    const long long a_ext = (AL == A_MK) ? (long long)(M - 1) * lda + K : (long long)(K - 1) * lda + M;
    const long long b_ext = (BL == B_NK) ? (long long)(N - 1) * ldb + K : (long long)(K - 1) * ldb + N;
    // (16-byte loads along M or N must not straddle the end of the operand: M, N multiples of 4 there)
    fast_loop = avec && bvec && (K % (2 * BK) == 0) && a_ext < (1ll << 29) && b_ext < (1ll << 29) &&
                (AL == A_MK || M % 4 == 0) && (BL == B_NK || N % 4 == 0);
  }
  if (fast_loop) {
    // ---- unguarded main loop, written so that nothing but matrix instructions uses the vector ALU inside it: a VALU
    // instruction of any wavefront takes the issue slot the matrix pipe of that SIMD would have used.
    //  * global addresses = a buffer resource per operand + a per-thread 32-bit offset that never changes + the slab's
    //    position as the instruction's scalar offset (advanced by the scalar ALU);
    //  * LDS addresses = a per-thread base that never changes + immediate offsets (the slab loop is unrolled by two so
    //    that the buffer a slab lives in is a compile-time constant; the four fragment bases are made opaque to the
    //    compiler so that it keeps every fragment read as a single read with a 16-bit offset instead of pairing two
    //    behind a recomputed base).
    unsigned aoff[WB], boff[WB];
    int ast[WB], bst[WB];  // LDS store positions (floats)
#pragma unroll
    for (int i = 0; i < WB; ++i) {
      const int idx = threadIdx.x + i * GEMM_THREADS;
      constexpr int PER_ROW = 16 * WB;
      if (AL == A_MK) { aoff[i] = (unsigned)((idx >> 2) * (int)lda + ((idx & 3) << 2)); ast[i] = ((idx & 3) << 2) * LDS_STRIDE + (idx >> 2); }
      else { aoff[i] = (unsigned)((idx / PER_ROW) * (int)lda + ((idx % PER_ROW) << 2)); ast[i] = (idx / PER_ROW) * LDS_STRIDE + ((idx % PER_ROW) << 2); }
      if (BL == B_NK) { boff[i] = (unsigned)((idx >> 2) * (int)ldb + ((idx & 3) << 2)); bst[i] = ((idx & 3) << 2) * LDS_STRIDE + (idx >> 2); }
      else { boff[i] = (unsigned)((idx / PER_ROW) * (int)ldb + ((idx % PER_ROW) << 2)); bst[i] = (idx / PER_ROW) * LDS_STRIDE + ((idx % PER_ROW) << 2); }
      if constexpr (EDGE) {
        // a thread whose vector lies past M or N fetches from past the resource instead: zero, and no memory traffic
        constexpr unsigned NOWHERE = 0x3fffffffu;  // in floats; four times it is still a 32-bit offset
        if (m0 + ((AL == A_MK) ? (idx >> 2) : ((idx % PER_ROW) << 2)) >= M) aoff[i] = NOWHERE;
        if (n0 + ((BL == B_NK) ? (idx >> 2) : ((idx % PER_ROW) << 2)) >= N) boff[i] = NOWHERE;
      }
    }
    // buffer resources over the two operands: the per-thread offset goes into the instruction's vector offset, the slab's
    // position into its scalar offset (advanced by the scalar ALU)
    const float* abase = (AL == A_MK) ? A + (long long)m0 * lda : A + m0;
    const float* bbase = (BL == B_NK) ? B + (long long)n0 * ldb : B + n0;
    const long long a_floats = ((AL == A_MK) ? (long long)(M - 1) * lda + K : (long long)(K - 1) * lda + M) - (abase - A);
    const long long b_floats = ((BL == B_NK) ? (long long)(N - 1) * ldb + K : (long long)(K - 1) * ldb + N) - (bbase - B);
    const __amdgpu_buffer_rsrc_t ares = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(abase), 0, (int)(a_floats * 4), 0x00020000);
    const __amdgpu_buffer_rsrc_t bres = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(bbase), 0, (int)(b_floats * 4), 0x00020000);
    const int astep = ((AL == A_MK) ? BK : BK * (int)lda) * 4;
    const int bstep = ((BL == B_NK) ? BK : BK * (int)ldb) * 4;
    // the loop fetches two slabs ahead without asking whether there are any: past the last slab it fetches the last one
    // again, so every address it forms lies inside the operand whatever part the scalar offset plays in the range check
    // of a buffer load (on gfx950 it is checked together with the vector offset, on other parts it is not)
    const int a_last = (slabs - 1) * astep, b_last = (slabs - 1) * bstep;
    int apos = 0, bpos = 0;  // bytes
    auto fetch_into = [&](float4 (&xa)[WB], float4 (&xb)[WB]) {
#pragma unroll
      for (int i = 0; i < WB; ++i) {
        const vuint4 v = __builtin_amdgcn_raw_buffer_load_b128(ares, (int)(aoff[i] * 4), apos, 0);
        xa[i] = make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
      }
#pragma unroll
      for (int i = 0; i < WB; ++i) {
        const vuint4 v = __builtin_amdgcn_raw_buffer_load_b128(bres, (int)(boff[i] * 4), bpos, 0);
        xb[i] = make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
      }
      apos = min(apos + astep, a_last);
      bpos = min(bpos + bstep, b_last);
    };
    auto scale = [&](float4 (&xa)[WB], float4 (&xb)[WB]) {
      if (a_div != 1.0f) {
#pragma unroll
        for (int i = 0; i < WB; ++i) { xa[i].x /= a_div; xa[i].y /= a_div; xa[i].z /= a_div; xa[i].w /= a_div; }
      }
      if (b_div != 1.0f) {
#pragma unroll
        for (int i = 0; i < WB; ++i) { xb[i].x /= b_div; xb[i].y /= b_div; xb[i].z /= b_div; xb[i].w /= b_div; }
      }
    };
    auto stash_from = [&](auto cur_tag, float4 (&xa)[WB], float4 (&xb)[WB]) {
      constexpr int CUR = decltype(cur_tag)::value;
#pragma unroll
      for (int i = 0; i < WB; ++i) {
        if (AL == A_MK) {
          smem[CUR * SLAB + ast[i]] = xa[i].x; smem[CUR * SLAB + ast[i] + LDS_STRIDE] = xa[i].y;
          smem[CUR * SLAB + ast[i] + 2 * LDS_STRIDE] = xa[i].z; smem[CUR * SLAB + ast[i] + 3 * LDS_STRIDE] = xa[i].w;
        } else {
          *reinterpret_cast<float4*>(&smem[CUR * SLAB + ast[i]]) = xa[i];
        }
        if (BL == B_NK) {
          smem[(2 + CUR) * SLAB + bst[i]] = xb[i].x; smem[(2 + CUR) * SLAB + bst[i] + LDS_STRIDE] = xb[i].y;
          smem[(2 + CUR) * SLAB + bst[i] + 2 * LDS_STRIDE] = xb[i].z; smem[(2 + CUR) * SLAB + bst[i] + 3 * LDS_STRIDE] = xb[i].w;
        } else {
          *reinterpret_cast<float4*>(&smem[(2 + CUR) * SLAB + bst[i]]) = xb[i];
        }
      }
    };
    // four fragment bases the compiler cannot relate to each other: every read then keeps its own 16-bit immediate offset
    typedef const __attribute__((address_space(3))) float* lds_ptr;
    lds_ptr fa[WB], fb[WB];
#pragma unroll
    for (int i = 0; i < WB; ++i) {
      fa[i] = (lds_ptr)smem + (wm * 32 * WB + l32 + h * LDS_STRIDE + 32 * i);
      fb[i] = (lds_ptr)smem + (wn * 32 * WB + l32 + h * LDS_STRIDE + 32 * i);
      asm volatile("" : "+v"(fa[i]));
      asm volatile("" : "+v"(fb[i]));
    }
    auto multiply = [&](auto cur_tag) {
      constexpr int CUR = decltype(cur_tag)::value;
      if (!idle_quadrant) {
#pragma unroll
        for (int ks = 0; ks < BK / 2; ++ks) {
          float a[WB], b[WB];
#pragma unroll
          for (int i = 0; i < WB; ++i) a[i] = fa[i][CUR * SLAB + ks * 2 * LDS_STRIDE];
#pragma unroll
          for (int i = 0; i < WB; ++i) b[i] = fb[i][(2 + CUR) * SLAB + ks * 2 * LDS_STRIDE];
#pragma unroll
          for (int i = 0; i < WB; ++i)
#pragma unroll
            for (int j = 0; j < WB; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);  // the fragments of one k-step are live at a time
        }
      }
    };
    using T0 = std::integral_constant<int, 0>;
    using T1 = std::integral_constant<int, 1>;
    // slab 0 -> buffer 0; slab 1 in flight in set 2; inside the loop every slab is fetched two slabs ahead of its use
    fetch_into(ra, rb);
    scale(ra, rb);
    stash_from(T0{}, ra, rb);
    fetch_into(ra2, rb2);
    __syncthreads();
    for (int s = 0; s < slabs; s += 2) {
      fetch_into(ra, rb);           // slab s + 2
      multiply(T0{});               // slab s
      scale(ra2, rb2);
      stash_from(T1{}, ra2, rb2);   // slab s + 1
      __syncthreads();
      fetch_into(ra2, rb2);         // slab s + 3
      multiply(T1{});               // slab s + 1
      scale(ra, rb);
      stash_from(T0{}, ra, rb);     // slab s + 2
      __syncthreads();
    }
  } else {
  slab_load<AL == A_MK, EDGE, WB>(A, lda, m0, M, 0, K, avec, ra);
  slab_load<BL == B_NK, EDGE, WB>(B, ldb, n0, N, 0, K, bvec, rb);
  if (a_div != 1.0f) {
#pragma unroll
    for (int i = 0; i < WB; ++i) { ra[i].x /= a_div; ra[i].y /= a_div; ra[i].z /= a_div; ra[i].w /= a_div; }
  }
  if (b_div != 1.0f) {
#pragma unroll
    for (int i = 0; i < WB; ++i) { rb[i].x /= b_div; rb[i].y /= b_div; rb[i].z /= b_div; rb[i].w /= b_div; }
  }
  slab_store<AL == A_MK, WB>(As[0], ra);
  slab_store<BL == B_NK, WB>(Bs[0], rb);
  __syncthreads();

  for (int s = 0; s < slabs; ++s) {
    const int cur = s & 1;
    const bool more = (s + 1 < slabs);
    if (more) {
      slab_load<AL == A_MK, EDGE, WB>(A, lda, m0, M, (s + 1) * BK, K, avec, ra);
      slab_load<BL == B_NK, EDGE, WB>(B, ldb, n0, N, (s + 1) * BK, K, bvec, rb);
    }
    const float* as = As[cur] + wm * 32 * WB + l32;
    const float* bs = Bs[cur] + wn * 32 * WB + l32;
    if (!idle_quadrant)
#pragma unroll
    for (int ks = 0; ks < BK / 2; ++ks) {
      const int krow = (ks * 2 + h) * LDS_STRIDE;
      float a[WB], b[WB];
#pragma unroll
      for (int i = 0; i < WB; ++i) a[i] = as[krow + 32 * i];
#pragma unroll
      for (int i = 0; i < WB; ++i) b[i] = bs[krow + 32 * i];
#pragma unroll
      for (int i = 0; i < WB; ++i)
#pragma unroll
        for (int j = 0; j < WB; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (more) {
      if (a_div != 1.0f) {
#pragma unroll
        for (int i = 0; i < WB; ++i) { ra[i].x /= a_div; ra[i].y /= a_div; ra[i].z /= a_div; ra[i].w /= a_div; }
      }
      if (b_div != 1.0f) {
#pragma unroll
        for (int i = 0; i < WB; ++i) { rb[i].x /= b_div; rb[i].y /= b_div; rb[i].z /= b_div; rb[i].w /= b_div; }
      }
      slab_store<AL == A_MK, WB>(As[cur ^ 1], ra);
      slab_store<BL == B_NK, WB>(Bs[cur ^ 1], rb);
    }
    __syncthreads();
  }
  }

  // ---- epilogue -------------------------------------------------------------------
  // accumulator element e of tile (i,j): row = 32*i + 8*(e/4) + 4*h + e%4, col = 32*j + l32
  float local = 0.f;      // sum of squares or running max
  bool local_nan = false;
  float* __restrict__ C = P.C;
  const long long ldc = P.ldc;
  // Symmetric products over whole tiles write their epilogue like the main loop, with the addresses on the scalar side:
  // every vector-ALU instruction here is taken from the matrix pipe of the other workgroups on the SIMD, and the general
  // epilogue below spends 750 (store) to 1900 (Newton M) of them per wavefront on 64-bit addresses and per-element
  // predicates.  A block of 32 x 32 above the diagonal is stored as computed and, turned in LDS, as its mirror image; a
  // block ON the diagonal (four per diagonal tile) keeps what lies on or above the diagonal and mirrors what lies strictly
  // above it, the other elements' stores pointed past the buffer resource; blocks below the diagonal are dropped.
  constexpr bool FAST_SYM = TRI && !EDGE && WB == 2 && (EPI == EPI_STORE || EPI == EPI_NEWTON_M);
  bool stored = false;
  if constexpr (FAST_SYM) {
    stored = true;
    const bool diag_tile = tm == tn;
    if (!diag_tile || wm <= wn) {
      const int ld = (int)ldc;
      const int tile_bytes = ((BM - 1) * ld + BN) * 4;
      constexpr int NOWHERE = 0x7ffffff0;  // a byte offset past every resource: the store is dropped
      const __amdgpu_buffer_rsrc_t cd = __builtin_amdgcn_make_buffer_rsrc(C + (long long)m0 * ldc + n0, 0, tile_bytes, 0x00020000);
      float* const C2 = P.C2;
      const __amdgpu_buffer_rsrc_t c2d = __builtin_amdgcn_make_buffer_rsrc(C2 + (long long)m0 * ldc + n0, 0, tile_bytes, 0x00020000);
      const float mp_scale = sc.mp_scale, mp_diag = sc.mp_diag;
      const int order = P.d;
      // as computed: element e of block (i, j) is row 32 i + 8 (e / 4) + 4 h + e % 4, column 32 j + l32 of the wavefront's quadrant
      const int vdir = ((wm * 64 + 4 * h) * ld + wn * 64 + l32) * 4;
      unsigned worst = 0;  // largest |M - I| as a bit pattern: NaN above infinity above every finite value
#pragma unroll
      for (int i = 0; i < WB; ++i)
#pragma unroll
        for (int j = 0; j < WB; ++j) {
          const bool on_diagonal = diag_tile && wm == wn && i == j;
          if (diag_tile && wm == wn && i > j) continue;
          if (!on_diagonal) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
              const int soff = ((i * 32 + 8 * (e >> 2) + (e & 3)) * ld + j * 32) * 4;
              const float v = acc[i][j][e];
              __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), cd, vdir, soff, 0);
              if (EPI == EPI_NEWTON_M) {
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(__fmul_rn(v, mp_scale)), c2d, vdir, soff, 0);
                worst = max(worst, __float_as_uint(v) & 0x7fffffffu);
              }
            }
          } else {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
              const int soff = ((i * 32 + 8 * (e >> 2) + (e & 3)) * ld + j * 32) * 4;
              const int rb = 8 * (e >> 2) + (e & 3) + 4 * h;  // row inside the block; l32 is the column
              const bool keep = rb <= l32, unit = rb == l32 && m0 + wm * 64 + i * 32 + rb < order;
              const int voff = keep ? vdir : NOWHERE;
              const float v = acc[i][j][e];
              __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), cd, voff, soff, 0);
              if (EPI == EPI_NEWTON_M) {
                float mp = __fmul_rn(v, mp_scale);
                if (unit) mp = __fadd_rn(mp, mp_diag);
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(mp), c2d, voff, soff, 0);
                // the diagonal beyond the order is padding (zero, and not part of the error)
                const float dv = unit ? v - 1.0f : ((rb == l32) ? 0.0f : v);
                if (keep) worst = max(worst, __float_as_uint(dv) & 0x7fffffffu);
              }
            }
          }
        }
      // mirrored: each 32 x 32 block is turned in LDS (a private region per wavefront) and leaves as 16-byte stores
      constexpr int TS = 36;
      float* stage = (wave < 2) ? &As[wave & 1][0] : &Bs[wave & 1][0];
      const int vmir = ((wn * 64 + (lane >> 3)) * ld + wm * 64 + (lane & 7) * 4) * 4;
      float* const put = stage + l32 * TS + 4 * h;
      const float* const get = stage + (lane >> 3) * TS + (lane & 7) * 4;
#pragma unroll
      for (int i = 0; i < WB; ++i)
#pragma unroll
        for (int j = 0; j < WB; ++j) {
          const bool on_diagonal = diag_tile && wm == wn && i == j;
          if (diag_tile && wm == wn && i > j) continue;
#pragma unroll
          for (int q = 0; q < 4; ++q)
            *reinterpret_cast<float4*>(put + 8 * q) = make_float4(acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
          __builtin_amdgcn_wave_barrier();
          asm volatile("" ::: "memory");
#pragma unroll
          for (int it = 0; it < 4; ++it) {
            const float4 v = *reinterpret_cast<const float4*>(get + 8 * it * TS);
            // The position of the four rows goes into the resource's base, not into the store's scalar offset: a
            // 16-byte buffer store WITH a scalar offset register, followed at once by a vector-ALU instruction that
            // writes its data registers, stored that instruction's result as the first of its four values now and then
            // (the compiler pads this hazard only for stores without a scalar offset register, as here).
            const long long at = (long long)((j * 32 + 8 * it) * ld + i * 32);
            const __amdgpu_buffer_rsrc_t to = __builtin_amdgcn_make_buffer_rsrc(C + (long long)n0 * ldc + m0 + at, 0, tile_bytes, 0x00020000);
            const __amdgpu_buffer_rsrc_t to2 = __builtin_amdgcn_make_buffer_rsrc(C2 + (long long)n0 * ldc + m0 + at, 0, tile_bytes, 0x00020000);
            if (!on_diagonal) {
              const vuint4 raw = {__float_as_uint(v.x), __float_as_uint(v.y), __float_as_uint(v.z), __float_as_uint(v.w)};
              __builtin_amdgcn_raw_buffer_store_b128(raw, to, vmir, 0, 0);
              if (EPI == EPI_NEWTON_M) {
                const vuint4 mp = {__float_as_uint(__fmul_rn(v.x, mp_scale)), __float_as_uint(__fmul_rn(v.y, mp_scale)),
                                   __float_as_uint(__fmul_rn(v.z, mp_scale)), __float_as_uint(__fmul_rn(v.w, mp_scale))};
                __builtin_amdgcn_raw_buffer_store_b128(mp, to2, vmir, 0, 0);
              }
            } else {
              // this lane holds row c = lane / 8 + 8 it of the mirror image, columns r4 .. r4 + 3: those left of c are kept
              const int c = (lane >> 3) + 8 * it, r4 = (lane & 7) * 4;
              const float vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
              for (int k = 0; k < 4; ++k) {
                const int voff = (c > r4 + k) ? vmir + 4 * k : NOWHERE;
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(vv[k]), to, voff, 0, 0);
                if (EPI == EPI_NEWTON_M) __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(__fmul_rn(vv[k], mp_scale)), to2, voff, 0, 0);
              }
            }
          }
          __builtin_amdgcn_wave_barrier();
          asm volatile("" ::: "memory");
        }
      if (EPI == EPI_NEWTON_M) local = __uint_as_float(worst);
    }
  }
  // the same for plain products over whole tiles (the preconditioning pair, the rotations of the eigenvalue-corrected step)
  constexpr bool FAST_PLAIN = !TRI && !LOWER && !EDGE && WB == 2 && (EPI == EPI_STORE || EPI == EPI_STORE_SQNORM);
  if constexpr (FAST_PLAIN) {
    stored = true;
    const int ld = (int)ldc;
    const __amdgpu_buffer_rsrc_t cd =
        __builtin_amdgcn_make_buffer_rsrc(C + (long long)m0 * ldc + n0, 0, ((BM - 1) * ld + BN) * 4, 0x00020000);
    const int vdir = ((wm * 64 + 4 * h) * ld + wn * 64 + l32) * 4;
#pragma unroll
    for (int i = 0; i < WB; ++i)
#pragma unroll
      for (int j = 0; j < WB; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const float v = acc[i][j][e];
          __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), cd, vdir, ((i * 32 + 8 * (e >> 2) + (e & 3)) * ld + j * 32) * 4, 0);
          if (EPI == EPI_STORE_SQNORM) local += v * v;
        }
  }
  // C -= product over whole tiles (the block-reflector updates of the QR refresh): k is 32 to 128 there, so the tile is
  // mostly epilogue; a block's sixteen old values are all requested before the first difference is stored
  constexpr bool FAST_SUB = EPI == EPI_SUB && !TRI && !EDGE;
  if constexpr (FAST_SUB) {
    stored = true;
    const int ld = (int)ldc;
    const __amdgpu_buffer_rsrc_t cd =
        __builtin_amdgcn_make_buffer_rsrc(C + (long long)m0 * ldc + n0, 0, ((BM - 1) * ld + BN) * 4, 0x00020000);
    const int vdir = ((wm * 32 * WB + 4 * h) * ld + wn * 32 * WB + l32) * 4;
#pragma unroll
    for (int i = 0; i < WB; ++i)
#pragma unroll
      for (int j = 0; j < WB; ++j) {
        float old[16];
#pragma unroll
        for (int e = 0; e < 16; ++e)
          old[e] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(cd, vdir, ((i * 32 + 8 * (e >> 2) + (e & 3)) * ld + j * 32) * 4, 0));
#pragma unroll
        for (int e = 0; e < 16; ++e)
          __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(old[e] - acc[i][j][e]), cd, vdir, ((i * 32 + 8 * (e >> 2) + (e & 3)) * ld + j * 32) * 4, 0);
      }
  }
  // The fused eigenvalue-correction epilogue over whole tiles: two state arrays are read and three written per element,
  // with two IEEE divisions and a square root in between.  The general epilogue below handles one element at a time
  // behind 64-bit addresses (a round trip to memory per element, each waiting for the stores of the one before it);
  // here eight elements' old values are requested together, through buffer resources with scalar row offsets.
  constexpr bool FAST_EC = EPI == EPI_EC_FUSED && !TRI && !LOWER && !EDGE && WB == 2;
  if constexpr (FAST_EC) {
    stored = true;
    const int ld = (int)ldc;
    const int tile_bytes = ((BM - 1) * ld + BN) * 4;
    const long long at = (long long)m0 * ldc + n0;
    const bool has_m = P.C2 != nullptr;
    const __amdgpu_buffer_rsrc_t cd = __builtin_amdgcn_make_buffer_rsrc(C + at, 0, tile_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t c2d = __builtin_amdgcn_make_buffer_rsrc(has_m ? P.C2 + at : C + at, 0, has_m ? tile_bytes : 0, 0x00020000);
    const __amdgpu_buffer_rsrc_t c3d = __builtin_amdgcn_make_buffer_rsrc(P.C3 + at, 0, tile_bytes, 0x00020000);
    const int vdir = ((wm * 64 + 4 * h) * ld + wn * 64 + l32) * 4;
    const float alpha = sc.alpha, beta = sc.beta, mom_w = sc.mom_w, mom_div = sc.mom_div, div = sc.div, pow_exp = sc.pow_exp, eps = sc.eps;
#pragma unroll
    for (int i = 0; i < WB; ++i)
#pragma unroll
      for (int j = 0; j < WB; ++j)
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          float sq_old[8], m_old[8];
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            const int e = 8 * half + q;
            const int soff = ((i * 32 + 8 * (e >> 2) + (e & 3)) * ld + j * 32) * 4;
            sq_old[q] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(cd, vdir, soff, 0));
            m_old[q] = has_m ? __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(c2d, vdir, soff, 0)) : 0.f;
          }
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            const int e = 8 * half + q;
            const int soff = ((i * 32 + 8 * (e >> 2) + (e & 3)) * ld + j * 32) * 4;
            const float v = acc[i][j][e];
            const float sq = __fadd_rn(__fmul_rn(sq_old[q], beta), __fmul_rn(__fmul_rn(alpha, v), v));
            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(sq), cd, vdir, soff, 0);
            float num = v;
            if (has_m) {
              // torch.lerp(m, g, w): m + w (g - m) for w < 0.5, g - (g - m)(1 - w) otherwise
              const float m_0 = m_old[q];
              const float m_1 = mom_w < 0.5f ? m_0 + mom_w * (v - m_0) : v - (v - m_0) * (1.0f - mom_w);
              __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(m_1), c2d, vdir, soff, 0);
              num = m_1 / mom_div;
            }
            const float x = sq / div;
            const float r = (pow_exp == 0.5f) ? sqrtf(x) : powf(x, pow_exp);
            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(num / (r + eps)), c3d, vdir, soff, 0);
          }
        }
  }
  // The factor update over whole tiles: a read-modify-write of the packed upper triangle.  The general epilogue below
  // handles one element at a time (its load, a wait for it and for the store before it, the store: 64 round trips to
  // memory per wavefront, as long as the main loop of a 1024-deep product); here the sixteen old values of a block are
  // requested together.  Element (r, c), c >= r, of the packed matrix of order n lives at r n - r (r + 1) / 2 + c; for
  // row r0 + k that is k (n - r0) - k (k + 1) / 2 past row r0's, so an element's offset is one multiply-add.  The
  // elements below the diagonal (blocks on the diagonal of a diagonal tile) are pointed past the resource.
  constexpr bool FAST_SYRK = EPI == EPI_SYRK_EMA && TRI && !EDGE && WB == 2;
  if constexpr (FAST_SYRK) {
    if (N <= 16384) {  // byte offsets and the resource's extent stay below 2^31
      stored = true;
      const bool diag_tile = tm == tn;
      if (!diag_tile || wm <= wn) {
        constexpr int NOWHERE = 0x7ffffff0;
        const int n = N;
        const __amdgpu_buffer_rsrc_t cd = __builtin_amdgcn_make_buffer_rsrc(C, 0, n * (n + 1) / 2 * 4, 0x00020000);
        const float alpha = sc.alpha, beta = sc.beta;
#pragma unroll
        for (int i = 0; i < WB; ++i)
#pragma unroll
          for (int j = 0; j < WB; ++j) {
            const bool on_diagonal = diag_tile && wm == wn && i == j;
            if (diag_tile && wm == wn && i > j) continue;
            const int r0 = m0 + wm * 64 + i * 32 + 4 * h, c = n0 + wn * 64 + j * 32 + l32;
            const int first = (r0 * n - r0 * (r0 + 1) / 2 + c) * 4, pitch = (n - r0) * 4;
            int voff[16];
            float old[16];
#pragma unroll
            for (int e = 0; e < 16; ++e) {
              const int k = 8 * (e >> 2) + (e & 3);
              voff[e] = first + k * pitch - 2 * k * (k + 1);
              if (on_diagonal && k + 4 * h > l32) voff[e] = NOWHERE;
              old[e] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(cd, voff[e], 0, 0));
            }
#pragma unroll
            for (int e = 0; e < 16; ++e)
              __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(__builtin_fmaf(acc[i][j][e], alpha, old[e] * beta)), cd, voff[e], 0, 0);
          }
      }
    }
  }
  if (!stored) {
#pragma unroll
  for (int i = 0; i < WB; ++i) {
#pragma unroll
    for (int j = 0; j < WB; ++j) {
      const int col = n0 + wn * 32 * WB + j * 32 + l32;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = m0 + wm * 32 * WB + i * 32 + 8 * (e >> 2) + 4 * h + (e & 3);
        const float v = acc[i][j][e];
        // A diagonal tile of a symmetric product recomputes its lower half; that half is dropped and replaced by the
        // mirror image of the upper one, so that every symmetric product leaves an exactly mirrored matrix.
        const bool lower = TRI && (EPI == EPI_STORE || EPI == EPI_NEWTON_M) && tm == tn && row > col;
        if (EPI == EPI_STORE) {
          if (!lower && (!EDGE || (row < M && col < N))) C[(long long)row * ldc + col] = v;
          if (TRI && EDGE && (tm != tn || row < col) && row < M && col < N) C[(long long)col * ldc + row] = v;
        } else if (EPI == EPI_STORE_SQNORM) {
          if (!EDGE || (row < M && col < N)) {
            C[(long long)row * ldc + col] = v;
            local += v * v;
          }
        } else if (EPI == EPI_SYRK_EMA) {
          // packed row-major upper triangle of an N x N matrix: (r,c), c >= r, lives at
          // r*N - r*(r-1)/2 + (c - r)
          if (row < M && col < N && col >= row) {
            const long long off = (long long)row * N - ((long long)row * (row - 1)) / 2 + (col - row);
            // factor.mul_(beta2).add_(gram, alpha=w): the product with beta2 is rounded, the addition fuses alpha * gram
            // (ATen's add with alpha is one fmadd per element)
            const float old = C[off];
            C[off] = __builtin_fmaf(v, sc.alpha, old * sc.beta);
          }
        } else if (EPI == EPI_SYRK_EMA64) {
          // the factor matrix is kept in fp64: the fp32 Gram matrix entry is widened, then averaged in double
          if (row < M && col < N && col >= row) {
            const long long off = (long long)row * N - ((long long)row * (row - 1)) / 2 + (col - row);
            double* C64 = reinterpret_cast<double*>(C);
            C64[off] = __builtin_fma((double)v, sc.alpha64, C64[off] * sc.beta64);
          }
        } else if (EPI == EPI_SQ_EMA) {
          if (!EDGE || (row < M && col < N)) {
            const long long o = (long long)row * ldc + col;
            C[o] = __fadd_rn(__fmul_rn(C[o], sc.beta), __fmul_rn(__fmul_rn(sc.alpha, v), v));
          }
        } else if (EPI == EPI_DIVPOW) {
          if (!EDGE || (row < M && col < N)) {
            const long long o = (long long)row * ldc + col;
            const float x = P.C2[o] / sc.div;
            const float r = (sc.pow_exp == 0.5f) ? sqrtf(x) : powf(x, sc.pow_exp);
            C[o] = v / (r + sc.eps);
            if (P.C3) P.C3[o] = v * sc.mom_div;
          }
        } else if (EPI == EPI_EC_FUSED) {
          if (!EDGE || (row < M && col < N)) {
            const long long o = (long long)row * ldc + col;
            const float sq = __fadd_rn(__fmul_rn(C[o], sc.beta), __fmul_rn(__fmul_rn(sc.alpha, v), v));
            C[o] = sq;
            float num = v;
            if (P.C2) {
              // torch.lerp(m, g, w): m + w (g - m) for w < 0.5, g - (g - m)(1 - w) otherwise
              const float m0 = P.C2[o];
              const float m1 = sc.mom_w < 0.5f ? m0 + sc.mom_w * (v - m0) : v - (v - m0) * (1.0f - sc.mom_w);
              P.C2[o] = m1;
              num = m1 / sc.mom_div;
            }
            const float x = sq / sc.div;
            const float r = (sc.pow_exp == 0.5f) ? sqrtf(x) : powf(x, sc.pow_exp);
            P.C3[o] = num / (r + sc.eps);
          }
        } else if (EPI == EPI_SUB) {
          if (!EDGE || (row < M && col < N)) {
            const long long o = (long long)row * ldc + col;
            C[o] = C[o] - v;
          }
        } else if (EPI == EPI_HORNER) {
          // operands are zero padded to the tile grid, so every (row, col) is in bounds and the padding stays zero
          const long long o = (long long)row * ldc + col;
          float r = __fmul_rn(v, sc.alpha);
          if (sc.beta != 0.0f) r = __fadd_rn(r, __fmul_rn(P.C2[o], sc.beta));
          if (row == col && row < P.d) r = __fadd_rn(r, sc.mp_diag);
          C[o] = r;
        } else if (EPI == EPI_NEWTON_M) {
          // operands are zero padded to the tile grid, so every (row, col) is in bounds
          if (!lower) {
            C[(long long)row * ldc + col] = v;
            float mp = __fmul_rn(v, sc.mp_scale);
            if (row == col && row < P.d) mp = __fadd_rn(mp, sc.mp_diag);
            P.C2[(long long)row * ldc + col] = mp;
            if (TRI && EDGE && (tm != tn || row < col)) {
              C[(long long)col * ldc + row] = v;
              P.C2[(long long)col * ldc + row] = mp;
            }
            if (row < P.d && col < P.d) {
              const float dv = fabsf(v - (row == col ? 1.0f : 0.0f));
              if (dv != dv) local_nan = true;
              local = fmaxf(local, dv);
            }
          }
        }
      }
    }
  }
  if (TRI && !EDGE && (EPI == EPI_STORE || EPI == EPI_NEWTON_M)) {
    // Mirror image of everything above the diagonal: each 32 x 32 accumulator block is transposed through the (now
    // idle) operand buffers, one private region per wavefront, and leaves as 16-byte stores along the rows of C.
    // In a diagonal tile the blocks below the diagonal are skipped (their computed values are dropped) and the
    // blocks on it mirror only their strictly upper part, element by element.
    const bool diag = (tm == tn);
    if (!diag || wm <= wn) {
      constexpr int TS = 36;  // 32 + 4: keeps float4 alignment
      float* stage = (wave < 2) ? &As[wave & 1][0] : &Bs[wave & 1][0];
#pragma unroll
      for (int i = 0; i < WB; ++i) {
#pragma unroll
        for (int j = 0; j < WB; ++j) {
          const int br = wm * WB + i, bc = wn * WB + j;  // position of the block inside the tile, in blocks of 32
          if (diag && br > bc) continue;
          const bool on_diagonal = diag && br == bc;
#pragma unroll
          for (int q = 0; q < 4; ++q)  // stage[col][row]: the four accumulator values of a group are four consecutive rows
            *reinterpret_cast<float4*>(stage + l32 * TS + 8 * q + 4 * h) =
                make_float4(acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
          __builtin_amdgcn_wave_barrier();
          asm volatile("" ::: "memory");
#pragma unroll
          for (int it = 0; it < 4; ++it) {
            const int c = (lane >> 3) + 8 * it, r4 = (lane & 7) * 4;
            const float4 v = *reinterpret_cast<const float4*>(stage + c * TS + r4);
            const long long o = (long long)(n0 + wn * 32 * WB + j * 32 + c) * ldc + (m0 + wm * 32 * WB + i * 32 + r4);
            if (!on_diagonal) {
              *reinterpret_cast<float4*>(C + o) = v;
              if (EPI == EPI_NEWTON_M)  // strictly below the diagonal: M_p has no diagonal term here
                *reinterpret_cast<float4*>(P.C2 + o) = make_float4(__fmul_rn(v.x, sc.mp_scale), __fmul_rn(v.y, sc.mp_scale),
                                                                   __fmul_rn(v.z, sc.mp_scale), __fmul_rn(v.w, sc.mp_scale));
            } else {
              const float vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
              for (int k = 0; k < 4; ++k)
                if (c > r4 + k) {  // target (row c, column r4 + k) of the block lies strictly below the diagonal
                  C[o + k] = vv[k];
                  if (EPI == EPI_NEWTON_M) P.C2[o + k] = __fmul_rn(vv[k], sc.mp_scale);
                }
            }
          }
          __builtin_amdgcn_wave_barrier();
          asm volatile("" ::: "memory");
        }
      }
    }
  }
  }  // !stored
  if (EPI == EPI_STORE_SQNORM) {
    local = wave_sum(local);
    if (lane == 0) red[wave] = local;
    __syncthreads();
    if (threadIdx.x == 0) P.C2[tm * P.tiles_n + tn] = (red[0] + red[1]) + (red[2] + red[3]);
  } else if (EPI == EPI_NEWTON_M) {
    if (local_nan) local = __builtin_nanf("");
    local = wave_max_nan(local);
    if (lane == 0) {
      // non-negative floats order like their bit patterns; a NaN pattern (0x7fc00000) is above +inf
      atomicMax(P.err_bits, __float_as_uint(local != local ? __builtin_nanf("") : local));
    }
  }
}

}  // namespace sa
