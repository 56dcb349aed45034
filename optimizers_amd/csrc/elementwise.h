// HBM-bound kernels of the Shampoo step: grafting second moment + filtered gradient,
// norm reductions, the final parameter update, and the symmetric pack / unpack / Newton
// initialisation passes over factor matrices.
//
// Elementwise work is cut into chunks of 4096 consecutive block elements (256 threads x
// 4 x float4); a chunk table maps a workgroup to (block, first element), so one launch
// covers every ragged block of a parameter group and fills all 256 CUs.  Reductions are
// wavefront shuffles -> one LDS slot per wavefront -> one partial per chunk, summed in a
// fixed order by a second tiny kernel, so results do not depend on scheduling.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/shampoo_amd.h"
#include "gemm.h"

namespace sa {

constexpr int EW_THREADS = 256;
constexpr int EW_CHUNK = 4096;

struct BlockDev {
  float* param;
  float* grad;
  float* filtered_grad;
  float* adagrad;
  float* momentum;
  float* ghat_tmp;        // lerp(m, g, 1-beta3) when beta3 != beta1, else nullptr
  const float* ghat_src;  // where the (undivided) filtered gradient is read from after the prologue
  const float* p_src;     // direction the update kernel consumes
  long long ld;           // row stride of param / grad
  long long ghat_ld;
  long long p_ld;
  int rows, cols;
  int chunk_begin, chunk_end;  // range in the per-chunk partial arrays
  int ptile_begin, ptile_end;  // range in the per-tile partial array (preconditioned blocks)
  int vec;                // every pointer of this block is 16-byte aligned and rows hold multiples of 4
  int p_vec;              // same for p_src
  int p_is_ghat;          // block has no preconditioned dim: direction = filtered gradient
  int mid;                // order-3 block d0 x d1 x d2 flattened to rows = d0 * d1: d1, else 0
  long long ld_outer;     // stride of dim 0 of an order-3 block
  int contig;             // param / grad view is contiguous in the block's own element order
  int p_like_grad;        // p_src is the gradient view itself (strided like param / grad)
  float* g3_dense;        // order 3: dense d0 x d1 x d2 copy of the gradient for the factor updates, or nullptr
  float* g3_perm;         // order 3: the same permuted to d1 x d0 x d2, or nullptr
  float* g3_ghat;         // order 3, beta1 == 0: dense copy of the gradient for the mode products, or nullptr
  float* g3_stat;         // order 3, eigenvalue-corrected: dense copy of the gradient for the rotated second moment
  float* weight_buffer;    // z sequence of primal averaging, or null
};

// offset of element e (block's own row-major order) inside the strided param / grad view
__device__ __forceinline__ long long view_offset(const BlockDev& B, int e) {
  if (B.contig) return e;
  const int r = e / B.cols, c = e - r * B.cols;
  if (B.mid > 0) {
    const int o = r / B.mid;
    return (long long)o * B.ld_outer + (long long)(r - o * B.mid) * B.ld + c;
  }
  return (long long)r * B.ld + c;
}
__device__ __forceinline__ long long direction_offset(const BlockDev& B, int e) {
  if (B.p_like_grad) return view_offset(B, e);
  return (B.p_ld == B.cols) ? (long long)e : (long long)(e / B.cols) * B.p_ld + (e % B.cols);
}

struct ChunkRef { int block; int start; };

// 16-byte streaming (non-temporal) accesses: data touched once per step should not evict reusable lines
typedef float vfloat4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 nt_load4(const float* p) {
  const vfloat4 v = __builtin_nontemporal_load(reinterpret_cast<const vfloat4*>(p));
  return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void nt_store4(const float4& x, float* p) {
  vfloat4 v = {x.x, x.y, x.z, x.w};
  __builtin_nontemporal_store(v, reinterpret_cast<vfloat4*>(p));
}

__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) red[wave] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

__device__ __forceinline__ float lerp_like_torch(float a, float b, float w) {
  // ATen lerp: a + w*(b-a) for w < 0.5, else b - (b-a)*(1-w)
  const float diff = b - a;
  return (w < 0.5f) ? a + w * diff : b - diff * (1.0f - w);
}

struct PreOut { float graft; float ghat; };

// One element of: v <- b2 v + w g^2 ; m <- lerp(m, g, 1-b1) ; ghat = m / bc1 ;
// graft = ghat / (sqrt(v / bc2) + eps)
__device__ __forceinline__ PreOut pre_element(float g, float& m, float& v, float& gh_tmp,
                                              const sa_step_scalars& s, bool has_m, bool has_v,
                                              bool beta3_differs) {
  PreOut o;
  if (has_v) {
    float vv = v;
    if (s.graft_beta2 != 1.0f) vv = vv * s.graft_beta2;
    vv = vv + (s.graft_weight * g) * g;
    v = vv;
  }
  float num;
  if (has_m) {
    float mm = m;
    if (beta3_differs) {
      gh_tmp = lerp_like_torch(mm, g, s.lerp_weight3);
      num = gh_tmp;
    }
    mm = lerp_like_torch(mm, g, s.lerp_weight1);
    m = mm;
    if (!beta3_differs) num = mm;
  } else {
    num = g;
  }
  o.ghat = num / s.bias_correction1;
  if (s.graft_type == SA_GRAFT_ADAGRAD) {
    const float den = sqrtf(v / s.graft_bias_correction2) + s.graft_epsilon;
    o.graft = o.ghat / den;
  } else {
    o.graft = o.ghat;
  }
  return o;
}

__device__ __forceinline__ float apply_element(float p, float& w, float& mom, const sa_step_scalars& s,
                                               float scale, bool has_mom, float& z, bool has_avg) {
  p = p * scale;
  if (s.weight_decay_alpha != 0.0f) {
    // with primal averaging the decay shrinks the z sequence instead of entering the direction, which the averaging
    // reuses (distributed_shampoo.py:1202-1254)
    if (has_avg) z = z * (1.0f - s.lr * s.weight_decay_alpha);
    else p = p + s.weight_decay_alpha * w;
  }
  if (has_mom) {
    float mb = mom * s.momentum;
    mb = mb + (1.0f - s.dampening) * p;
    mom = mb;
    p = s.use_nesterov ? (p * (1.0f - s.dampening)) + s.momentum * mb : mb;
  }
  p = p * (-s.lr);
  if (has_avg) {
    const float t = z - w;
    z = z + p;
    p = p * s.averaging_direction_coeff;
    p = p + s.averaging_buffer_coeff * t;
  }
  w = w + p;
  return p;
}

// MODE 0: prologue of a preconditioned step (updates v, m; partial norms).
// MODE 1: whole grafting-only step (also applies the update to W).
template <int MODE>
__global__ __launch_bounds__(EW_THREADS) void grafting_kernel(const BlockDev* __restrict__ blocks,
                                                             const ChunkRef* __restrict__ chunks,
                                                             sa_step_scalars s,
                                                             float* __restrict__ graft_partial,
                                                             float* __restrict__ ghat_partial) {
  __shared__ float red[4];
  const ChunkRef cr = chunks[blockIdx.x];
  const BlockDev& B = blocks[cr.block];
  const int n_el = B.rows * B.cols;
  const bool has_m = B.filtered_grad != nullptr, has_v = B.adagrad != nullptr;
  const bool has_mom = B.momentum != nullptr && s.momentum != 0.0f;
  // classic momentum and primal averaging exclude each other: one auxiliary state buffer per block
  const bool has_avg = B.weight_buffer != nullptr && s.use_primal_averaging != 0;
  const bool has_aux = has_mom || has_avg;
  float* __restrict__ aux = has_avg ? B.weight_buffer : B.momentum;
  const bool b3 = B.ghat_tmp != nullptr;
  float gsum = 0.f, hsum = 0.f;
  constexpr int NIT = EW_CHUNK / (EW_THREADS * 4);
  // Whole, vectorisable chunk (the common case): every load is issued before the first use, so each
  // thread keeps up to 16 x 16 bytes in flight; streamed data bypasses the caches it would only pollute.
  const bool whole = (cr.start + EW_CHUNK <= n_el) && (B.vec != 0);
  if (whole) {
    long long gi[NIT];
    float4 g[NIT], m[NIT], v[NIT], w[NIT], mo[NIT];
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int e = cr.start + (it * EW_THREADS + threadIdx.x) * 4;
      gi[it] = view_offset(B, e);
      g[it] = nt_load4(B.grad + gi[it]);
    }
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int e = cr.start + (it * EW_THREADS + threadIdx.x) * 4;
      m[it] = has_m ? nt_load4(B.filtered_grad + e) : make_float4(0, 0, 0, 0);
      v[it] = has_v ? nt_load4(B.adagrad + e) : make_float4(0, 0, 0, 0);
      if (MODE == 1) {
        w[it] = nt_load4(B.param + gi[it]);
        mo[it] = has_aux ? nt_load4(aux + e) : make_float4(0, 0, 0, 0);
      }
    }
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int e = cr.start + (it * EW_THREADS + threadIdx.x) * 4;
      float4 t = make_float4(0, 0, 0, 0);
      PreOut o0 = pre_element(g[it].x, m[it].x, v[it].x, t.x, s, has_m, has_v, b3);
      PreOut o1 = pre_element(g[it].y, m[it].y, v[it].y, t.y, s, has_m, has_v, b3);
      PreOut o2 = pre_element(g[it].z, m[it].z, v[it].z, t.z, s, has_m, has_v, b3);
      PreOut o3 = pre_element(g[it].w, m[it].w, v[it].w, t.w, s, has_m, has_v, b3);
      if (has_m) nt_store4(m[it], B.filtered_grad + e);
      if (has_v) nt_store4(v[it], B.adagrad + e);
      if (b3) *reinterpret_cast<float4*>(B.ghat_tmp + e) = t;
      if (MODE == 0) {
        gsum += (o0.graft * o0.graft + o1.graft * o1.graft) + (o2.graft * o2.graft + o3.graft * o3.graft);
        hsum += (o0.ghat * o0.ghat + o1.ghat * o1.ghat) + (o2.ghat * o2.ghat + o3.ghat * o3.ghat);
      } else {
        apply_element(o0.graft, w[it].x, mo[it].x, s, 1.0f, has_mom, mo[it].x, has_avg);
        apply_element(o1.graft, w[it].y, mo[it].y, s, 1.0f, has_mom, mo[it].y, has_avg);
        apply_element(o2.graft, w[it].z, mo[it].z, s, 1.0f, has_mom, mo[it].z, has_avg);
        apply_element(o3.graft, w[it].w, mo[it].w, s, 1.0f, has_mom, mo[it].w, has_avg);
        *reinterpret_cast<float4*>(B.param + gi[it]) = w[it];
        if (has_aux) nt_store4(mo[it], aux + e);
      }
    }
  } else
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int e = cr.start + (it * EW_THREADS + threadIdx.x) * 4;
    if (e >= n_el) continue;
    const long long gi = view_offset(B, e);
    const bool vec = (e + 3 < n_el) && (B.vec != 0);
    if (vec) {
      float4 g = *reinterpret_cast<const float4*>(B.grad + gi);
      float4 m = has_m ? *reinterpret_cast<const float4*>(B.filtered_grad + e) : make_float4(0, 0, 0, 0);
      float4 v = has_v ? *reinterpret_cast<const float4*>(B.adagrad + e) : make_float4(0, 0, 0, 0);
      float4 t = make_float4(0, 0, 0, 0);
      PreOut o0 = pre_element(g.x, m.x, v.x, t.x, s, has_m, has_v, b3);
      PreOut o1 = pre_element(g.y, m.y, v.y, t.y, s, has_m, has_v, b3);
      PreOut o2 = pre_element(g.z, m.z, v.z, t.z, s, has_m, has_v, b3);
      PreOut o3 = pre_element(g.w, m.w, v.w, t.w, s, has_m, has_v, b3);
      if (has_m) *reinterpret_cast<float4*>(B.filtered_grad + e) = m;
      if (has_v) *reinterpret_cast<float4*>(B.adagrad + e) = v;
      if (b3) *reinterpret_cast<float4*>(B.ghat_tmp + e) = t;
      if (MODE == 0) {
        gsum += (o0.graft * o0.graft + o1.graft * o1.graft) + (o2.graft * o2.graft + o3.graft * o3.graft);
        hsum += (o0.ghat * o0.ghat + o1.ghat * o1.ghat) + (o2.ghat * o2.ghat + o3.ghat * o3.ghat);
      } else {
        float4 w = *reinterpret_cast<const float4*>(B.param + gi);
        float4 mo = has_aux ? *reinterpret_cast<const float4*>(aux + e) : make_float4(0, 0, 0, 0);
        apply_element(o0.graft, w.x, mo.x, s, 1.0f, has_mom, mo.x, has_avg);
        apply_element(o1.graft, w.y, mo.y, s, 1.0f, has_mom, mo.y, has_avg);
        apply_element(o2.graft, w.z, mo.z, s, 1.0f, has_mom, mo.z, has_avg);
        apply_element(o3.graft, w.w, mo.w, s, 1.0f, has_mom, mo.w, has_avg);
        *reinterpret_cast<float4*>(B.param + gi) = w;
        if (has_aux) *reinterpret_cast<float4*>(aux + e) = mo;
      }
    } else {
      for (int k = 0; k < 4 && e + k < n_el; ++k) {
        const int ee = e + k;
        const long long gk = view_offset(B, ee);
        float g = B.grad[gk];
        float m = has_m ? B.filtered_grad[ee] : 0.f;
        float v = has_v ? B.adagrad[ee] : 0.f;
        float t = 0.f;
        PreOut o = pre_element(g, m, v, t, s, has_m, has_v, b3);
        if (has_m) B.filtered_grad[ee] = m;
        if (has_v) B.adagrad[ee] = v;
        if (b3) B.ghat_tmp[ee] = t;
        if (MODE == 0) {
          gsum += o.graft * o.graft;
          hsum += o.ghat * o.ghat;
        } else {
          float w = B.param[gk];
          float mo = has_aux ? aux[ee] : 0.f;
          apply_element(o.graft, w, mo, s, 1.0f, has_mom, mo, has_avg);
          B.param[gk] = w;
          if (has_aux) aux[ee] = mo;
        }
      }
    }
  }
  if (MODE == 0) {
    const float gs = block_sum(gsum, red);
    __syncthreads();
    const float hs = block_sum(hsum, red);
    if (threadIdx.x == 0) {
      graft_partial[blockIdx.x] = gs;
      ghat_partial[blockIdx.x] = hs;
    }
  }
}

// norms[b] = sum of graft partials, norms[n + b] = sum of the direction's partials; one workgroup per block.
__global__ __launch_bounds__(EW_THREADS) void reduce_norms_kernel(const BlockDev* __restrict__ blocks,
                                                                 const int* __restrict__ active_blocks,
                                                                 int n_blocks,
                                                                 const float* __restrict__ graft_partial,
                                                                 const float* __restrict__ ghat_partial,
                                                                 const float* __restrict__ ptile_partial,
                                                                 float* __restrict__ norms) {
  __shared__ float red[4];
  const int b = active_blocks[blockIdx.x];
  const BlockDev& B = blocks[b];
  float a = 0.f;
  for (int i = B.chunk_begin + threadIdx.x; i < B.chunk_end; i += EW_THREADS) a += graft_partial[i];
  const float g = block_sum(a, red);
  __syncthreads();
  float c = 0.f;
  if (B.p_is_ghat) {
    for (int i = B.chunk_begin + threadIdx.x; i < B.chunk_end; i += EW_THREADS) c += ghat_partial[i];
  } else {
    for (int i = B.ptile_begin + threadIdx.x; i < B.ptile_end; i += EW_THREADS) c += ptile_partial[i];
  }
  const float p = block_sum(c, red);
  if (threadIdx.x == 0) {
    norms[b] = g;
    norms[n_blocks + b] = p;
  }
}

// W <- W - lr * (momentum(P * ||graft|| / (||P|| + 1e-16) + alpha W))
__global__ __launch_bounds__(EW_THREADS) void apply_kernel(const BlockDev* __restrict__ blocks,
                                                          const ChunkRef* __restrict__ chunks,
                                                          sa_step_scalars s, int n_blocks,
                                                          const float* __restrict__ norms) {
  const ChunkRef cr = chunks[blockIdx.x];
  const BlockDev& B = blocks[cr.block];
  const int n_el = B.rows * B.cols;
  const bool has_mom = B.momentum != nullptr && s.momentum != 0.0f;
  // classic momentum and primal averaging exclude each other: one auxiliary state buffer per block
  const bool has_avg = B.weight_buffer != nullptr && s.use_primal_averaging != 0;
  const bool has_aux = has_mom || has_avg;
  float* __restrict__ aux = has_avg ? B.weight_buffer : B.momentum;
  const float p_div = B.p_is_ghat ? s.bias_correction1 : 1.0f;
  float scale = 1.0f;
  if (s.graft_type != SA_GRAFT_NONE) {
    const float gn = sqrtf(norms[cr.block]);
    const float pn = sqrtf(norms[n_blocks + cr.block]) + 1e-16f;
    scale = gn / pn;
  }
  constexpr int NIT = EW_CHUNK / (EW_THREADS * 4);
  const bool whole = (cr.start + EW_CHUNK <= n_el) && (B.vec != 0) && (B.p_vec != 0);
  if (whole) {
    long long wi[NIT];
    float4 p[NIT], w[NIT], mo[NIT];
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int e = cr.start + (it * EW_THREADS + threadIdx.x) * 4;
      wi[it] = view_offset(B, e);
      const long long pi = direction_offset(B, e);
      p[it] = nt_load4(B.p_src + pi);
      w[it] = nt_load4(B.param + wi[it]);
      mo[it] = has_aux ? nt_load4(aux + e) : make_float4(0, 0, 0, 0);
    }
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int e = cr.start + (it * EW_THREADS + threadIdx.x) * 4;
      apply_element(p[it].x / p_div, w[it].x, mo[it].x, s, scale, has_mom, mo[it].x, has_avg);
      apply_element(p[it].y / p_div, w[it].y, mo[it].y, s, scale, has_mom, mo[it].y, has_avg);
      apply_element(p[it].z / p_div, w[it].z, mo[it].z, s, scale, has_mom, mo[it].z, has_avg);
      apply_element(p[it].w / p_div, w[it].w, mo[it].w, s, scale, has_mom, mo[it].w, has_avg);
      *reinterpret_cast<float4*>(B.param + wi[it]) = w[it];
      if (has_aux) nt_store4(mo[it], aux + e);
    }
  } else
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int e = cr.start + (it * EW_THREADS + threadIdx.x) * 4;
    if (e >= n_el) continue;
    const long long wi = view_offset(B, e);
    const long long pi = direction_offset(B, e);
    const bool vec = (e + 3 < n_el) && (B.vec != 0) && (B.p_vec != 0);
    if (vec) {
      float4 p = *reinterpret_cast<const float4*>(B.p_src + pi);
      float4 w = *reinterpret_cast<const float4*>(B.param + wi);
      float4 mo = has_aux ? *reinterpret_cast<const float4*>(aux + e) : make_float4(0, 0, 0, 0);
      apply_element(p.x / p_div, w.x, mo.x, s, scale, has_mom, mo.x, has_avg);
      apply_element(p.y / p_div, w.y, mo.y, s, scale, has_mom, mo.y, has_avg);
      apply_element(p.z / p_div, w.z, mo.z, s, scale, has_mom, mo.z, has_avg);
      apply_element(p.w / p_div, w.w, mo.w, s, scale, has_mom, mo.w, has_avg);
      *reinterpret_cast<float4*>(B.param + wi) = w;
      if (has_aux) *reinterpret_cast<float4*>(aux + e) = mo;
    } else {
      for (int k = 0; k < 4 && e + k < n_el; ++k) {
        const int ee = e + k;
        const long long wk = view_offset(B, ee);
        const long long pk = direction_offset(B, ee);
        float w = B.param[wk];
        float mo = has_aux ? aux[ee] : 0.f;
        apply_element(B.p_src[pk] / p_div, w, mo, s, scale, has_mom, mo, has_avg);
        B.param[wk] = w;
        if (has_aux) aux[ee] = mo;
      }
    }
  }
}

// W += coeff * (Z - W) over the chunks of every block with a weight buffer (train / eval switch of primal averaging).
__global__ __launch_bounds__(EW_THREADS) void move_params_kernel(const BlockDev* __restrict__ blocks,
                                                                const ChunkRef* __restrict__ chunks, float coeff) {
  const ChunkRef cr = chunks[blockIdx.x];
  const BlockDev& B = blocks[cr.block];
  if (B.weight_buffer == nullptr) return;
  const int n_el = B.rows * B.cols;
  constexpr int NIT = EW_CHUNK / (EW_THREADS * 4);
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int e0 = cr.start + (it * EW_THREADS + threadIdx.x) * 4;
    for (int k = 0; k < 4 && e0 + k < n_el; ++k) {
      const long long wi = view_offset(B, e0 + k);
      const float w = B.param[wi];
      const float t = B.weight_buffer[e0 + k] - w;
      B.param[wi] = w + t * coeff;
    }
  }
}

// Dense (and dim-1-first) copies of the gradient of every order-3 block.  which = 0: for the factor updates
// (g3_dense, g3_perm); which = 1: for the mode products of a step without filtered gradient (g3_ghat);
// which = 2: for the rotated second moment of eigenvalue-corrected blocks (g3_stat).
__global__ __launch_bounds__(EW_THREADS) void gather3_kernel(const BlockDev* __restrict__ blocks,
                                                            const ChunkRef* __restrict__ chunks, int which) {
  const ChunkRef cr = chunks[blockIdx.x];
  const BlockDev& B = blocks[cr.block];
  if (B.mid <= 0) return;
  float* dense = which == 0 ? B.g3_dense : (which == 1 ? B.g3_ghat : B.g3_stat);
  float* perm = which == 0 ? B.g3_perm : nullptr;
  if (dense == nullptr && perm == nullptr) return;
  const int n_el = B.rows * B.cols, d0 = B.rows / B.mid;
  for (int it = 0; it < EW_CHUNK / EW_THREADS; ++it) {
    const int e = cr.start + it * EW_THREADS + threadIdx.x;
    if (e >= n_el) break;
    const float v = B.grad[view_offset(B, e)];
    if (dense) dense[e] = v;
    if (perm) {
      const int r = e / B.cols, c = e - r * B.cols, i0 = r / B.mid, i1 = r - i0 * B.mid;
      perm[((long long)i1 * d0 + i0) * B.cols + c] = v;
    }
  }
}

// G += wd * W in place on the gradient.
__global__ __launch_bounds__(EW_THREADS) void l2_kernel(const BlockDev* __restrict__ blocks,
                                                       const ChunkRef* __restrict__ chunks, float wd) {
  const ChunkRef cr = chunks[blockIdx.x];
  const BlockDev& B = blocks[cr.block];
  const int n_el = B.rows * B.cols;
  for (int it = 0; it < EW_CHUNK / EW_THREADS; ++it) {
    const int e = cr.start + it * EW_THREADS + threadIdx.x;
    if (e >= n_el) break;
    const long long gi = view_offset(B, e);
    B.grad[gi] = B.grad[gi] + wd * B.param[gi];
  }
}

// ---------------------------------------------------------------------------------------
// Symmetric factor passes.  A factor of dimension d is stored packed (row-major upper
// triangle, (r,c), c >= r at r*d - r*(r-1)/2 + c - r) in optimizer state and dense, mirrored
// and zero padded to dpad x dpad (dpad a multiple of 128) in the workspace.  All three
// passes walk pairs of 64x64 tiles (bi <= bj): the upper tile is read coalesced and its
// transpose is produced through LDS.
// ---------------------------------------------------------------------------------------

constexpr int ST = 64;  // symmetric pass tile

struct SymFactor {
  const float* packed_in;  // packed source (factor for Newton init, inverse for unpack)
  float* packed_out;       // packed destination (commit)
  const float* dense_in;   // dense source (commit)
  const float* dense_in_alt;  // commit: read instead of dense_in when *select != 0
  const int* select;       // optional
  const int* gate;         // optional (commit): the factor is skipped unless gate_index < *gate
  int gate_index;
  float* dense_out[4];     // dense destinations (Newton init: M, M_p, X, and optionally X M_p)
  unsigned int* err_bits;
  const float* norm_partial;  // Newton init: per-chunk partial sums of squares
  const float* scale;      // Newton init: optional per-factor multiplier applied after the division by bc2
  int n_norm_partial;
  int d, dpad;
  int tile_begin;          // first tile-pair id
  int tiles;               // dpad / ST
  int root;
  int enabled;
};

__device__ __forceinline__ long long packed_off(int r, int c, int d) {
  return (long long)r * d - ((long long)r * (r - 1)) / 2 + (c - r);
}

__device__ __forceinline__ void sym_locate(const SymFactor* __restrict__ f, int n, int id, int& fi, int& bi, int& bj) {
  int lo = 0, hi = n - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (f[mid].tile_begin <= id) lo = mid; else hi = mid - 1;
  }
  fi = lo;
  int t = id - f[lo].tile_begin;
  bi = 0;
  int rowlen = f[lo].tiles;
  while (t >= rowlen) { t -= rowlen; ++bi; --rowlen; }
  bj = bi + t;
}

enum SymMode { SYM_UNPACK = 0, SYM_NEWTON_INIT = 1, SYM_COMMIT = 2 };

// SYM_UNPACK:      dense_out[0] = mirror(packed_in)
// SYM_NEWTON_INIT: a = packed_in / bc2 (+ eps on the diagonal); z = (root+1)/(2 ||A||_F);
//                  dense_out[0] = M = z a, dense_out[1] = M_p = M*mp_scale + mp_diag I,
//                  dense_out[2] = X = z^(1/root) I, dense_out[3] = X M_p = z^(1/root) M_p (optional), err = max |M - I|
// SYM_COMMIT:      packed_out = upper(dense_in) (if packed_out), dense_out[0] = mirror(upper(dense_in))
template <int MODE>
__global__ __launch_bounds__(256) void sym_pass_kernel(const SymFactor* __restrict__ factors, int n_factors,
                                                      float bc2, float eps, float mp_scale, float mp_diag) {
  __shared__ float tile[ST][ST + 1];
  __shared__ float zsh;
  int fi, bi, bj;
  sym_locate(factors, n_factors, blockIdx.x, fi, bi, bj);
  const SymFactor& F = factors[fi];
  if (!F.enabled) return;
  if (MODE == SYM_COMMIT && F.gate != nullptr && F.gate_index >= *F.gate) return;
  const float* __restrict__ dense_in = F.dense_in;
  if (MODE == SYM_COMMIT && F.select != nullptr && *F.select != 0) dense_in = F.dense_in_alt;
  const int d = F.d, dpad = F.dpad;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;        // loads: 64 columns x 4 rows
  const int qx = (threadIdx.x & 15) * 4, qy = threadIdx.x >> 4;  // stores: 16 groups of four columns x 16 rows

  float z = 1.0f, x0 = 0.f;
  if (MODE == SYM_NEWTON_INIT) {
    // ||A||_F^2 from the per-chunk partial sums, added in their order by one thread; the workgroup fetches them together
    // (a thread that loads and adds them one after the other holds its workgroup for the latency of every load)
    __shared__ float part[256];
    float ssum = 0.f;
    for (int base = 0; base < F.n_norm_partial; base += 256) {
      const int i = base + (int)threadIdx.x;
      part[threadIdx.x] = i < F.n_norm_partial ? F.norm_partial[i] : 0.f;
      __syncthreads();
      if (threadIdx.x == 0) {
        const int m = min(256, F.n_norm_partial - base);
        for (int k = 0; k < m; ++k) ssum += part[k];
      }
      __syncthreads();
    }
    if (threadIdx.x == 0) zsh = (float)(F.root + 1) / (2.0f * sqrtf(ssum));
    __syncthreads();
    z = zsh;
    x0 = powf(z, 1.0f / (float)F.root);
  }

  // load the upper tile (rows of block bi, cols of block bj); symmetric value for the diagonal tile
  for (int rr = ty; rr < ST; rr += 4) {
    const int r = bi * ST + rr, c = bj * ST + tx;
    float v = 0.f;
    if (r < d && c < d) {
      if (MODE == SYM_COMMIT) {
        const int rs = min(r, c), cs = max(r, c);
        v = dense_in[(long long)rs * dpad + cs];
      } else {
        const int rs = min(r, c), cs = max(r, c);
        v = F.packed_in[packed_off(rs, cs, d)];
        if (MODE == SYM_NEWTON_INIT) {
          v = v / bc2;
          if (F.scale != nullptr) v = v * F.scale[0];
          if (r == c && eps != 0.0f) v = v + eps;
        }
      }
    }
    tile[rr][tx] = v;
  }
  __syncthreads();

  float errmax = 0.f;
  bool errnan = false;
  // upper placement (bi, bj) and, for off-diagonal tiles, the mirrored placement (bj, bi); four columns per thread,
  // 16-byte stores (rows of the dense matrices start on 256-byte boundaries: dpad is a multiple of the tile)
  for (int pass = 0; pass < ((bi == bj) ? 1 : 2); ++pass) {
#pragma unroll
    for (int rr = qy; rr < ST; rr += 16) {
      const int r = (pass == 0 ? bi : bj) * ST + rr;
      const int c = (pass == 0 ? bj : bi) * ST + qx;
      float v[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] = (pass == 0) ? tile[rr][qx + k] : tile[qx + k][rr];
      const long long o = (long long)r * dpad + c;
      if (MODE == SYM_UNPACK) {
        *reinterpret_cast<float4*>(F.dense_out[0] + o) = make_float4(v[0], v[1], v[2], v[3]);
      } else if (MODE == SYM_COMMIT) {
        *reinterpret_cast<float4*>(F.dense_out[0] + o) = make_float4(v[0], v[1], v[2], v[3]);
        if (pass == 0 && F.packed_out != nullptr && r < d) {
#pragma unroll
          for (int k = 0; k < 4; ++k)
            if (c + k < d && c + k >= r) F.packed_out[packed_off(r, c + k, d)] = v[k];
        }
      } else {
        float m[4], mp[4], xd[4], x1[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          m[k] = z * v[k];
          mp[k] = __fmul_rn(m[k], mp_scale);
          const bool diag = (r == c + k && r < d);
          if (diag) mp[k] = __fadd_rn(mp[k], mp_diag);
          xd[k] = diag ? x0 : 0.f;
          // X is a multiple of the identity, so the first X M_p is x0 * M_p entry by entry: exactly what the product
          // would give (every other term of the dot product is an exact zero)
          x1[k] = __fmul_rn(x0, mp[k]);
          if (r < d && c + k < d) {
            const float dv = fabsf(m[k] - (r == c + k ? 1.0f : 0.0f));
            if (dv != dv) errnan = true;
            errmax = fmaxf(errmax, dv);
          }
        }
        *reinterpret_cast<float4*>(F.dense_out[0] + o) = make_float4(m[0], m[1], m[2], m[3]);
        *reinterpret_cast<float4*>(F.dense_out[1] + o) = make_float4(mp[0], mp[1], mp[2], mp[3]);
        *reinterpret_cast<float4*>(F.dense_out[2] + o) = make_float4(xd[0], xd[1], xd[2], xd[3]);
        if (F.dense_out[3] != nullptr)
          *reinterpret_cast<float4*>(F.dense_out[3] + o) = make_float4(x1[0], x1[1], x1[2], x1[3]);
      }
    }
  }
  if (MODE == SYM_NEWTON_INIT) {
    if (errnan) errmax = __builtin_nanf("");
    errmax = wave_max_nan(errmax);
    if ((threadIdx.x & 63) == 0) atomicMax(F.err_bits, __float_as_uint(errmax));
  }
}

// State tensors without symmetric packing: dense d x d matrices (row stride d, both triangles) on the caller's side,
// packed upper triangles on the library's.  One workgroup per pair of 64 x 64 tiles (bi <= bj), as in sym_pass_kernel.
//   TO_DENSE: dense = mirror(packed)        otherwise: packed = upper(dense)
struct DenseStateJob {
  void* packed;
  void* dense;
  int d;
  int tiles;       // ceil(d / ST)
  int tile_begin;  // first tile-pair id
};

template <typename T, bool TO_DENSE>
__global__ __launch_bounds__(256) void sym_state_kernel(const DenseStateJob* __restrict__ jobs, int n_jobs) {
  __shared__ T tile[ST][ST + 1];
  int lo = 0, hi = n_jobs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (jobs[mid].tile_begin <= (int)blockIdx.x) lo = mid; else hi = mid - 1;
  }
  const DenseStateJob& J = jobs[lo];
  int t = blockIdx.x - J.tile_begin, bi = 0, rowlen = J.tiles;
  while (t >= rowlen) { t -= rowlen; ++bi; --rowlen; }
  const int bj = bi + t;
  const int d = J.d;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  T* __restrict__ packed = static_cast<T*>(J.packed);
  T* __restrict__ dense = static_cast<T*>(J.dense);
  if (!TO_DENSE) {
    for (int rr = ty; rr < ST; rr += 4) {
      const int r = bi * ST + rr, c = bj * ST + tx;
      if (r < d && c < d && c >= r) packed[packed_off(r, c, d)] = dense[(long long)r * d + c];
    }
    return;
  }
  for (int rr = ty; rr < ST; rr += 4) {
    const int r = bi * ST + rr, c = bj * ST + tx;
    T v = 0;
    if (r < d && c < d) v = packed[packed_off(min(r, c), max(r, c), d)];
    tile[rr][tx] = v;
  }
  __syncthreads();
  for (int pass = 0; pass < ((bi == bj) ? 1 : 2); ++pass)
    for (int rr = ty; rr < ST; rr += 4) {
      const int r = (pass == 0 ? bi : bj) * ST + rr;
      const int c = (pass == 0 ? bj : bi) * ST + tx;
      if (r < d && c < d) dense[(long long)r * d + c] = (pass == 0) ? tile[rr][tx] : tile[tx][rr];
    }
}

// Per-factor, per-chunk sums of squares of the bias-corrected, ridged matrix (off-diagonal
// entries of the packed triangle count twice) and a non-finite flag.
struct NormJob {
  const float* src;     // packed factor, or dense matrix when dense != 0
  const float* src_alt; // dense only: read instead of src when *select != 0 (which of two ping-pong buffers holds the result)
  const int* select;    // optional
  float* partial;       // n_chunks partial sums
  float* scale;         // optional per-factor multiplier applied after the division by bc2 (trace scaling)
  int* nonfinite;       // set to 1 when a non-finite value is seen
  int d, dpad, dense;
  int chunk_begin;      // first workgroup id of this job
  int n_chunks;
  int enabled;
};

constexpr int NORM_CHUNK = 16384;

template <bool CHECK_ONLY>
__global__ __launch_bounds__(256) void factor_norm_kernel(const NormJob* __restrict__ jobs, int n_jobs,
                                                         float bc2, float eps) {
  __shared__ float red[4];
  int lo = 0, hi = n_jobs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (jobs[mid].chunk_begin <= (int)blockIdx.x) lo = mid; else hi = mid - 1;
  }
  const NormJob& J = jobs[lo];
  if (!J.enabled) return;
  const int chunk = blockIdx.x - J.chunk_begin;
  const int d = J.d;
  float acc = 0.f;
  bool bad = false;
  if (J.dense) {
    // dense d x d inside a dpad-strided buffer; chunked by rows
    const float* __restrict__ src = (J.select != nullptr && *J.select != 0) ? J.src_alt : J.src;
    const long long total = (long long)d * d;
    const long long e0 = (long long)chunk * NORM_CHUNK;
    const long long e1 = min(e0 + NORM_CHUNK, total);
    long long e = e0 + threadIdx.x;
    int r = (int)(e / d), c = (int)(e % d);  // once; then the column advances by 256 per element
    for (; e < e1; e += 256) {
      const float v = src[(long long)r * J.dpad + c];
      if (!(fabsf(v) <= 3.4028234663852886e38f)) bad = true;
      c += 256;
      while (c >= d) { c -= d; ++r; }
    }
  } else {
    const long long total = (long long)d * (d + 1) / 2;
    const long long e0 = (long long)chunk * NORM_CHUNK;
    const long long e1 = min(e0 + NORM_CHUNK, total);
    // The row of a thread's first element is found once (closed-form guess + a short search); from there the position
    // inside the row advances by 256 per element, rows getting one entry shorter each.
    long long e = e0 + threadIdx.x;
    if (e < e1) {
      const double dd = (double)d + 0.5;
      int r = (int)(dd - sqrt(dd * dd - 2.0 * (double)e));
      if (r < 0) r = 0;
      if (r > d - 1) r = d - 1;
      while (r > 0 && packed_off(r, r, d) > e) --r;
      while (r + 1 < d && packed_off(r + 1, r + 1, d) <= e) ++r;
      int idx = (int)(e - packed_off(r, r, d));  // 0 = the diagonal entry of row r
      int len = d - r;
      for (; e < e1; e += 256) {
        const bool diag = (idx == 0);
        float v = J.src[e] / bc2;
        if (J.scale != nullptr) v = v * J.scale[0];
        if (!(fabsf(v) <= 3.4028234663852886e38f)) bad = true;
        if (diag && eps != 0.0f) v = v + eps;
        acc += diag ? v * v : 2.0f * (v * v);
        idx += 256;
        while (len > 0 && idx >= len) { idx -= len; --len; }
      }
    }
  }
  if (bad) *J.nonfinite = 1;
  if (!CHECK_ONLY) {
    const float s = block_sum(acc, red);
    if (threadIdx.x == 0) J.partial[chunk] = s;
  }
}

// Trace scaling: scale = max(trace(factor / bc2), floor) ^ (-exponent), one workgroup per job
// (reference: shampoo_preconditioner_list.py:366-371).
__global__ __launch_bounds__(256) void trace_scale_kernel(const NormJob* __restrict__ jobs, float bc2, float floor,
                                                         float exponent) {
  __shared__ float red[4];
  const NormJob& J = jobs[blockIdx.x];
  if (!J.enabled || J.scale == nullptr) return;
  const int d = J.d;
  float acc = 0.f;
  for (int i = threadIdx.x; i < d; i += 256) acc += J.src[packed_off(i, i, d)] / bc2;
  const float trace = block_sum(acc, red);
  // a NaN trace stays NaN (like torch.clamp), so the finiteness check that follows sees it
  if (threadIdx.x == 0) J.scale[0] = powf(trace != trace ? trace : fmaxf(trace, floor), -exponent);
}

// ---- start of the coupled higher-order iteration (reference: matrix_functions.py:528-572) ---------------
// The bias-corrected factor sits dense (dpad-strided, zero padded) in A.
struct HoJob {
  float* A;         // dense factor; becomes M = z (A + eps I)
  float* Mp;        // M_p of the first (plain Newton) step: M * s + (1 - s) I
  float* X;         // z^(1/root) I
  float* rowsum;    // d absolute row sums
  float* params;    // [0] z = 1 / trace(A + eps I), [1] eps = max(rel * |A|_inf, abs), [2] |A|_inf
  int d, dpad;
};

// grid (ceil(max d / 4), jobs): one wavefront per row
__global__ __launch_bounds__(256) void ho_rowsum_kernel(const HoJob* __restrict__ jobs) {
  const HoJob& J = jobs[blockIdx.y];
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= J.d) return;
  const float* __restrict__ a = J.A + (long long)row * J.dpad;
  float acc = 0.f;
  for (int c = lane; c < J.d; c += 64) acc += fabsf(a[c]);
  acc = wave_sum(acc);
  if (lane == 0) J.rowsum[row] = acc;
}

// one workgroup per job
__global__ __launch_bounds__(256) void ho_setup_kernel(const HoJob* __restrict__ jobs, float rel_eps, float abs_eps) {
  __shared__ float red[4];
  __shared__ float eps_sh;
  const HoJob& J = jobs[blockIdx.x];
  float mx = 0.f;
  bool nan = false;
  for (int i = threadIdx.x; i < J.d; i += 256) {
    const float v = J.rowsum[i];
    if (v != v) nan = true;
    mx = fmaxf(mx, v);
  }
  if (nan) mx = __builtin_nanf("");
  mx = wave_max_nan(mx);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  if (threadIdx.x == 0) {
    float m = red[0];
    for (int w = 1; w < 4; ++w) m = (m != m || red[w] != red[w]) ? __builtin_nanf("") : fmaxf(m, red[w]);
    const float scaled = m * rel_eps;
    eps_sh = scaled != scaled ? scaled : fmaxf(scaled, abs_eps);  // torch.clamp(min=...) keeps a NaN
    J.params[1] = eps_sh;
    J.params[2] = m;
  }
  __syncthreads();
  const float eps = eps_sh;
  float acc = 0.f;
  for (int i = threadIdx.x; i < J.d; i += 256) acc += J.A[(long long)i * J.dpad + i] + eps;
  const float trace = block_sum(acc, red);
  if (threadIdx.x == 0) J.params[0] = 1.0f / trace;
}

// grid (ceil(max dpad^2 / 1024), jobs); ridge_only: A <- A + eps I and nothing else
__global__ __launch_bounds__(256) void ho_start_kernel(const HoJob* __restrict__ jobs, int root, int ridge_only) {
  const HoJob& J = jobs[blockIdx.y];
  const long long total = (long long)J.dpad * J.dpad;
  const long long e0 = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;
  if (e0 >= total) return;
  const float z = ridge_only ? 1.0f : J.params[0], eps = J.params[1];
  const float s = -1.0f / (float)root, one_minus_s = 1.0f - (-1.0f / (float)root);
  const float x0 = ridge_only ? 0.f : powf(z, 1.0f / (float)root);
  const int r = (int)(e0 / J.dpad), c0 = (int)(e0 % J.dpad);  // dpad is a multiple of 4: one row per thread
  float4 a = *reinterpret_cast<const float4*>(J.A + e0);
  float av[4] = {a.x, a.y, a.z, a.w}, mv[4], pv[4], xv[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const bool diag = (c0 + k == r) && r < J.d;
    float v = av[k];
    if (diag) v = v + eps;
    const float m = ridge_only ? v : z * v;
    mv[k] = m;
    float mp = __fmul_rn(m, s);
    if (diag) mp = __fadd_rn(mp, one_minus_s);
    pv[k] = mp;
    xv[k] = diag ? x0 : 0.f;
  }
  *reinterpret_cast<float4*>(J.A + e0) = make_float4(mv[0], mv[1], mv[2], mv[3]);
  if (!ridge_only) {
    *reinterpret_cast<float4*>(J.Mp + e0) = make_float4(pv[0], pv[1], pv[2], pv[3]);
    *reinterpret_cast<float4*>(J.X + e0) = make_float4(xv[0], xv[1], xv[2], xv[3]);
  }
}

// Loop control of the higher-order iteration (matrix_functions.py:574-619), one thread per factor.  `call` counts
// the evaluations: 0 follows the start (the first step always runs), 1 follows that step (its error becomes the
// reference error), later calls compare the new error with the kept one: more than 1.2 x, or equal below 1e-3,
// ends the loop with the last update in place.  flag: 0 converged, 1 iteration limit, 2 early stop.
struct HigherOrderCtl {
  unsigned int* err_bits;
  int* active;
  int* iterations;
  int* final_parity;
  float* final_err;
  float* kept_err;
  int* flag;
};

__global__ void higher_order_control_kernel(HigherOrderCtl c, const int* __restrict__ ids, int n, float tol, int max_iter,
                                            int call, int cur_parity) {
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int f = ids[i];
    if (!c.active[f]) continue;
    const float fresh = __uint_as_float(c.err_bits[f]);
    c.err_bits[f] = 0u;
    bool go;
    int flag = 0;
    if (call == 0) {
      go = true;
    } else {
      float err = c.kept_err[f];
      bool early = false;
      if (call == 1) err = fresh;
      else if (fresh > err * 1.2f || (fresh == err && err < 1e-3f)) early = true;
      else err = fresh;
      c.kept_err[f] = err;
      go = !early && (err > tol) && (c.iterations[f] < max_iter);
      flag = early ? 2 : ((err > tol) ? 1 : 0);
    }
    if (go) {
      c.iterations[f] += 1;
    } else {
      c.active[f] = 0;
      c.final_parity[f] = cur_parity;
      c.final_err[f] = c.kept_err[f];
      c.flag[f] = flag;
    }
  }
}

// Convergence bookkeeping of the batched Newton loop: one thread per factor.
struct NewtonCtl {
  unsigned int* err_bits;
  int* active;
  int* iterations;
  int* final_parity;
  float* final_err;
};

// `mailbox` (optional) is host memory the device can write: after the pass it holds (seq << 32) | number of factors
// still active, so that the host can follow the loop without synchronising the stream.
__global__ void newton_control_kernel(NewtonCtl c, const int* __restrict__ ids, int n, float tol, int max_iter,
                                      int cur_parity, int* __restrict__ n_active,
                                      unsigned long long* __restrict__ mailbox = nullptr, unsigned int seq = 0) {
  __shared__ int cnt;
  if (threadIdx.x == 0) cnt = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int f = ids[i];
    if (!c.active[f]) continue;
    const float err = __uint_as_float(c.err_bits[f]);
    // same test as `while error > tolerance and iteration < max_iterations`: NaN ends the loop
    const bool go = (err > tol) && (c.iterations[f] < max_iter);
    if (go) {
      c.iterations[f] += 1;
      atomicAdd(&cnt, 1);
    } else {
      c.active[f] = 0;
      c.final_parity[f] = cur_parity;
      c.final_err[f] = err;
    }
    c.err_bits[f] = 0u;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    *n_active = cnt;
    if (mailbox != nullptr) {
      __threadfence_system();
      __hip_atomic_store(mailbox, ((unsigned long long)seq << 32) | (unsigned int)cnt, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
}

// Start of a batch of coupled iterations: the listed factors become active with cleared error, iteration count and
// parity; every other factor's entries stay as they are.
__global__ void newton_activate_kernel(NewtonCtl c, const int* __restrict__ ids, int n) {
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
    const int f = ids[i];
    c.active[f] = 1;
    c.err_bits[f] = 0u;
    c.iterations[f] = 0;
    c.final_parity[f] = 0;
    c.final_err[f] = 0.f;
  }
}

// *first_bad = position (in the order of ids) of the first factor whose input or result holds nan / inf, n if none:
// the reference works through the factors one by one and raises at that one, so only the results before it are stored.
__global__ void first_bad_kernel(const int* __restrict__ ids, int n, const int* __restrict__ bad_input,
                                 const int* __restrict__ bad_result, int* __restrict__ first_bad) {
  __shared__ int best;
  if (threadIdx.x == 0) best = n;
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x)
    if (bad_input[ids[i]] != 0 || bad_result[ids[i]] != 0) atomicMin(&best, i);
  __syncthreads();
  if (threadIdx.x == 0) *first_bad = best;
}

// Plain float4 copy of n4 vectors: the known-traffic kernel HBM counters are scaled against.
__global__ __launch_bounds__(256) void copy_kernel(const float4* __restrict__ src, float4* __restrict__ dst, long long n4) {
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (long long)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

__global__ void copy_strided_kernel(const float* __restrict__ src, long long lds_, float* __restrict__ dst,
                                    int rows, int cols) {
  const long long n = (long long)rows * cols;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (long long)gridDim.x * blockDim.x)
    dst[e] = src[(e / cols) * lds_ + (e % cols)];
}

// dst += src over up to VIEW_ADD_BATCH pairs of strided views of at most three dims (the parameter update of the
// default distributor: every block of a parameter is a view into it, the directions are usually dense).  The jobs
// travel as a kernel argument, so a call needs no device table.  Work is cut into runs of 4 elements of the
// innermost dim: blockIdx.y is the job, the x grid strides over its runs.
constexpr int VIEW_ADD_BATCH = 24;
struct ViewAddJob {
  float* dst;
  const float* src;
  unsigned int n0, n1, n2;      // sizes, outermost first (unused leading dims are 1)
  unsigned int vec;             // both innermost strides are 1 and every run start is 16-byte aligned
  long long d0, d1, d2;         // element strides of dst
  long long s0, s1, s2;         // element strides of src
};
struct ViewAddBatch {
  ViewAddJob job[VIEW_ADD_BATCH];
};

__global__ __launch_bounds__(256) void view_add_kernel(ViewAddBatch batch) {
  const ViewAddJob& J = batch.job[blockIdx.y];
  const unsigned int runs_per_row = (J.n2 + 3u) >> 2;
  const unsigned long long rows = (unsigned long long)J.n0 * J.n1;
  const unsigned long long runs = rows * runs_per_row;
  for (unsigned long long r = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; r < runs;
       r += (unsigned long long)gridDim.x * blockDim.x) {
    const unsigned long long row = r / runs_per_row;
    const unsigned int c = (unsigned int)(r - row * runs_per_row) << 2;
    const unsigned int i0 = (unsigned int)(row / J.n1), i1 = (unsigned int)(row - (unsigned long long)i0 * J.n1);
    float* d = J.dst + i0 * J.d0 + i1 * J.d1 + c * J.d2;
    const float* s = J.src + i0 * J.s0 + i1 * J.s1 + c * J.s2;
    if (J.vec) {
      float4 a = *reinterpret_cast<float4*>(d);
      const float4 b = *reinterpret_cast<const float4*>(s);
      a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
      *reinterpret_cast<float4*>(d) = a;
    } else {
      const unsigned int m = min(4u, J.n2 - c);
      for (unsigned int k = 0; k < m; ++k) d[k * J.d2] += s[k * J.s2];
    }
  }
}

}  // namespace sa
