// libshampoo_amd.so: C ABI (include/shampoo_amd.h) over the gfx950 kernels in gemm.h and
// elementwise.h.  Host side of the library: the ragged batched descriptor tables of a
// parameter group ("plan"), the batched coupled-Newton driver, and per-phase HIP-event timing.

#include <hip/hip_runtime.h>
#include <dlfcn.h>

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/shampoo_amd.h"
#include "eigh.h"
#include "eigh64.h"
#include "elementwise.h"
#include "gemm.h"
#include "gemm64.h"
#include "qr.h"
#include "tridiag.h"

using namespace sa;

namespace {

thread_local std::string g_err;

int fail(int code, const std::string& msg) {
  g_err = msg;
  return code;
}

#define HIPCHECK(expr)                                                                     \
  do {                                                                                     \
    hipError_t e__ = (expr);                                                               \
    if (e__ != hipSuccess)                                                                 \
      return fail(SA_ERR_HIP, std::string(#expr) + " failed: " + hipGetErrorString(e__)); \
  } while (0)

#define SACHECK(expr)             \
  do {                            \
    int r__ = (expr);             \
    if (r__ != SA_OK) return r__; \
  } while (0)

inline long long round_up(long long x, long long a) { return (x + a - 1) / a * a; }

// A host-built table mirrored on the device.  The host copy is pinned so the upload is a
// true asynchronous copy; an event guards the pinned copy against being rewritten while a
// previous upload may still be reading it.
template <class T>
struct Table {
  T* host = nullptr;
  T* dev = nullptr;
  size_t cap = 0;
  size_t n = 0;
  hipEvent_t ev = nullptr;
  bool pending = false;
  // what the device copy holds and the stream that put it there: a rewrite that produces the same bytes for the same
  // stream (the usual case from the second step on: the tables depend on addresses and shapes only) uploads nothing
  std::vector<unsigned char> shadow;
  hipStream_t shadow_stream = nullptr;
  bool shadow_valid = false;

  int reserve(size_t m) {
    if (m <= cap) return SA_OK;
    SACHECK(wait());
    shadow_valid = false;
    size_t ncap = std::max<size_t>(m, cap * 2 + 16);
    T* nh = nullptr;
    T* nd = nullptr;
    HIPCHECK(hipHostMalloc(reinterpret_cast<void**>(&nh), ncap * sizeof(T), hipHostMallocDefault));
    HIPCHECK(hipMalloc(reinterpret_cast<void**>(&nd), ncap * sizeof(T)));
    if (host) {
      std::memcpy(nh, host, n * sizeof(T));
      HIPCHECK(hipHostFree(host));
    }
    if (dev) HIPCHECK(hipFree(dev));
    host = nh;
    dev = nd;
    cap = ncap;
    return SA_OK;
  }
  int wait() {
    if (pending) {
      HIPCHECK(hipEventSynchronize(ev));
      pending = false;
    }
    return SA_OK;
  }
  // start a rewrite of `m` entries
  int begin(size_t m) {
    SACHECK(wait());
    SACHECK(reserve(m));
    n = m;
    return SA_OK;
  }
  int upload(hipStream_t s) {
    if (n == 0) return SA_OK;
    const size_t bytes = n * sizeof(T);
    if (shadow_valid && shadow_stream == s && shadow.size() == bytes && std::memcmp(shadow.data(), host, bytes) == 0) return SA_OK;
    shadow.assign(reinterpret_cast<const unsigned char*>(host), reinterpret_cast<const unsigned char*>(host) + bytes);
    shadow_stream = s;
    shadow_valid = true;
    if (!ev) HIPCHECK(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
    HIPCHECK(hipMemcpyAsync(dev, host, n * sizeof(T), hipMemcpyHostToDevice, s));
    HIPCHECK(hipEventRecord(ev, s));
    pending = true;
    return SA_OK;
  }
  void destroy() {
    if (pending) (void)hipEventSynchronize(ev);
    if (host) (void)hipHostFree(host);
    if (dev) (void)hipFree(dev);
    if (ev) (void)hipEventDestroy(ev);
    host = nullptr; dev = nullptr; ev = nullptr; cap = n = 0; pending = false; shadow_valid = false;
  }
};

inline long long operand_bytes(long long rows, long long cols, long long ld) { return ((rows - 1) * ld + cols) * (long long)sizeof(float); }

// May the unguarded main loop of grouped_gemm_kernel run this problem?  Whole 128 x 128 tiles, K in pairs of slabs,
// 16-byte loads, and operands that a buffer resource can span (its extent is a 32-bit byte count).
inline bool unguarded_ok(const GemmProblem& p) {
  if (p.M % BM || p.N % BN || p.K % (2 * BK) || !p.a_vec || !p.b_vec) return false;
  const long long lim = 0x7fffffffLL;
  // either layout: the larger of the two possible extents bounds the operand
  const long long a = std::max(operand_bytes(p.M, p.K, p.lda), operand_bytes(p.K, p.M, p.lda));
  const long long b = std::max(operand_bytes(p.N, p.K, p.ldb), operand_bytes(p.K, p.N, p.ldb));
  return a < lim && b < lim;
}

struct GemmTable {
  Table<GemmProblem> t;
  int total_tiles = 0;
  int total_tiles_s = 0;  // the same launch cut into 64 x 64 tiles
  bool aligned = true;  // every problem may use the unguarded loader
  std::vector<GemmProblem> build;
  int* live = nullptr;  // device: n + 1 tile offsets over the active problems (launch_gemm_live)
  size_t live_cap = 0;

  void clear() { build.clear(); total_tiles = 0; total_tiles_s = 0; aligned = true; }
  void add(GemmProblem p, bool triangular) {
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    p.tile_begin = total_tiles;
    total_tiles += triangular ? p.tiles_n * (p.tiles_n + 1) / 2 : p.tiles_m * p.tiles_n;
    p.tiles_m_s = (p.M + 63) / 64;
    p.tiles_n_s = (p.N + 63) / 64;
    p.tile_begin_s = total_tiles_s;
    total_tiles_s += triangular ? p.tiles_n_s * (p.tiles_n_s + 1) / 2 : p.tiles_m_s * p.tiles_n_s;
    if (!unguarded_ok(p)) aligned = false;
    build.push_back(p);
  }
  int commit(hipStream_t s) {
    SACHECK(t.begin(build.size()));
    if (!build.empty()) std::memcpy(t.host, build.data(), build.size() * sizeof(GemmProblem));
    return t.upload(s);
  }
  int need_live() {
    if (live_cap >= t.n + 1) return SA_OK;
    if (live) HIPCHECK(hipFree(live));
    live = nullptr; live_cap = 0;
    HIPCHECK(hipMalloc(&live, live_ints((int)t.n) * sizeof(int)));
    live_cap = t.n + 1;
    return SA_OK;
  }
  void destroy() {
    t.destroy();
    if (live) (void)hipFree(live);
    live = nullptr; live_cap = 0;
  }
};

inline int vec_ok(const void* p, long long ld) { return ((reinterpret_cast<uintptr_t>(p) & 15) == 0 && (ld % 4) == 0) ? 1 : 0; }

template <int AL, int BL, int EPI, bool EDGE, bool TRI = (EPI == EPI_SYRK_EMA || EPI == EPI_SYRK_EMA64)>
int launch_gemm(const GemmTable& g, GemmScalars sc, hipStream_t s) {
  if (g.total_tiles == 0) return SA_OK;
  const int per = (g.total_tiles + NUM_XCD - 1) / NUM_XCD;
  hipLaunchKernelGGL((grouped_gemm_kernel<AL, BL, EPI, EDGE, TRI>), dim3(per * NUM_XCD), dim3(GEMM_THREADS), 0, s,
                     g.t.dev, (int)g.t.n, g.total_tiles, sc, (const int*)nullptr);
  HIPCHECK(hipGetLastError());
  return SA_OK;
}
int SMALL_LAUNCH_TILES = 256;  // launches below this many 128 x 128 tiles run as 64 x 64 tiles (coupled Newton loop)

// launch_gemm over the problems whose `active` flag is set when the launch runs: a one-workgroup pass lays the live
// tiles out first, so the skipped problems leave no holes in the walk (and no idle XCDs).
// few_live: the caller expects so few of the problems to be active that their large tiles would not fill the chip; the
// live tiles are then laid out and walked as 64 x 64 tiles (same bits; a wrong guess only costs the small tiles' lower rate)
template <int AL, int BL, int EPI, bool EDGE, bool TRI>
int launch_gemm_live(GemmTable& g, GemmScalars sc, hipStream_t s, bool few_live = false) {
  if (g.total_tiles == 0) return SA_OK;
  if (few_live && g.total_tiles >= SMALL_LAUNCH_TILES && g.total_tiles_s > 0) {
    SACHECK(g.need_live());
    const int per = (g.total_tiles_s + NUM_XCD - 1) / NUM_XCD, cap = per + per / 4 + 1;
    hipLaunchKernelGGL(gemm_live_tiles_kernel, dim3(1), dim3(256), 0, s, g.t.dev, (int)g.t.n, TRI ? 1 : 0, g.live, cap, 1);
    hipLaunchKernelGGL((grouped_gemm_kernel<AL, BL, EPI, EDGE, TRI, false, 1>), dim3(cap * NUM_XCD), dim3(GEMM_THREADS), 0, s,
                       g.t.dev, (int)g.t.n, g.total_tiles_s, sc, (const int*)g.live);
    HIPCHECK(hipGetLastError());
    return SA_OK;
  }
  // a launch that fits the chip twice over at most is latency bound: the extra pass would cost more than idle XCDs
  if (g.total_tiles < SMALL_LAUNCH_TILES) {
    // too few large tiles to fill the chip: the same problems as 64 x 64 tiles (four times the workgroups)
    const int per = (g.total_tiles_s + NUM_XCD - 1) / NUM_XCD;
    hipLaunchKernelGGL((grouped_gemm_kernel<AL, BL, EPI, EDGE, TRI, false, 1>), dim3(per * NUM_XCD), dim3(GEMM_THREADS), 0, s,
                       g.t.dev, (int)g.t.n, g.total_tiles_s, sc, (const int*)nullptr);
    HIPCHECK(hipGetLastError());
    return SA_OK;
  }
  if (g.total_tiles < 2048) return launch_gemm<AL, BL, EPI, EDGE, TRI>(g, sc, s);
  SACHECK(g.need_live());
  // runs of equal work may differ in their numbers of tiles: a quarter more workgroups per XCD than an even split needs
  const int per = (g.total_tiles + NUM_XCD - 1) / NUM_XCD, cap = per + per / 4 + 1;
  hipLaunchKernelGGL(gemm_live_tiles_kernel, dim3(1), dim3(256), 0, s, g.t.dev, (int)g.t.n, TRI ? 1 : 0, g.live, cap, 0);
  hipLaunchKernelGGL((grouped_gemm_kernel<AL, BL, EPI, EDGE, TRI>), dim3(cap * NUM_XCD), dim3(GEMM_THREADS), 0, s,
                     g.t.dev, (int)g.t.n, g.total_tiles, sc, (const int*)g.live);
  HIPCHECK(hipGetLastError());
  return SA_OK;
}
// WB = 1: 64 x 64 tiles (the problems' tiles_m_s / tiles_n_s / tile_begin_s describe the walk)
template <int AL, int BL, int EPI, bool EDGE, bool LOWER = false, int WB = 2>
int launch_gemm_raw(const GemmProblem* dev, int n, int total_tiles, GemmScalars sc, hipStream_t s) {
  if (total_tiles == 0) return SA_OK;
  const int per = (total_tiles + NUM_XCD - 1) / NUM_XCD;
  hipLaunchKernelGGL((grouped_gemm_kernel<AL, BL, EPI, EDGE, false, LOWER, WB>), dim3(per * NUM_XCD), dim3(GEMM_THREADS), 0, s, dev, n,
                     total_tiles, sc, (const int*)nullptr);
  HIPCHECK(hipGetLastError());
  return SA_OK;
}

template <int AL, int BL, int EPI>
int launch_gemm_auto(const GemmTable& g, GemmScalars sc, hipStream_t s) {
  return g.aligned ? launch_gemm<AL, BL, EPI, false>(g, sc, s) : launch_gemm<AL, BL, EPI, true>(g, sc, s);
}

// launch_gemm_auto in 64 x 64 tiles whatever the size of the launch: for products whose tiles hold little arithmetic
// (K of 32 or 128, or outputs of 32 to 96 rows or columns), where four times the workgroups hide more latency and a
// ragged edge wastes a smaller tile
template <int AL, int BL, int EPI>
int launch_gemm_small_tiles(const GemmTable& g, GemmScalars sc, hipStream_t s) {
  if (g.total_tiles_s == 0) return SA_OK;
  const int per = (g.total_tiles_s + NUM_XCD - 1) / NUM_XCD;
  if (g.aligned)
    hipLaunchKernelGGL((grouped_gemm_kernel<AL, BL, EPI, false, false, false, 1>), dim3(per * NUM_XCD), dim3(GEMM_THREADS), 0, s,
                       g.t.dev, (int)g.t.n, g.total_tiles_s, sc, (const int*)nullptr);
  else
    hipLaunchKernelGGL((grouped_gemm_kernel<AL, BL, EPI, true, false, false, 1>), dim3(per * NUM_XCD), dim3(GEMM_THREADS), 0, s,
                       g.t.dev, (int)g.t.n, g.total_tiles_s, sc, (const int*)nullptr);
  HIPCHECK(hipGetLastError());
  return SA_OK;
}

// launch_gemm_auto, with 64 x 64 tiles when the launch is small and every problem is whole tiles
template <int AL, int BL, int EPI>
int launch_gemm_auto_small(const GemmTable& g, GemmScalars sc, hipStream_t s) {
  if (!g.aligned || g.total_tiles == 0 || g.total_tiles >= SMALL_LAUNCH_TILES) return launch_gemm_auto<AL, BL, EPI>(g, sc, s);
  constexpr bool TRI = (EPI == EPI_SYRK_EMA || EPI == EPI_SYRK_EMA64);
  const int per = (g.total_tiles_s + NUM_XCD - 1) / NUM_XCD;
  hipLaunchKernelGGL((grouped_gemm_kernel<AL, BL, EPI, false, TRI, false, 1>), dim3(per * NUM_XCD), dim3(GEMM_THREADS), 0, s,
                     g.t.dev, (int)g.t.n, g.total_tiles_s, sc, (const int*)nullptr);
  HIPCHECK(hipGetLastError());
  return SA_OK;
}

GemmScalars unit_scalars() { return GemmScalars{1.0f, 1.0f, 1.0f, 0.0f, 0.0f, 0.0f, 1.0f, 1.0f, 0.0f, 0.0f, 1.0f, 1.0, 0.0}; }

// ---- phase timing -------------------------------------------------------------------------
struct Phase {
  std::vector<std::pair<hipEvent_t, hipEvent_t>> spans;
  size_t used = 0;
  double work = 0.0;      // algorithmic flops or bytes
  double executed = 0.0;  // flops actually issued (differs when symmetric products are halved)
  int launches = 0;
};
bool g_profiling = false;
// Symmetric-product policy of the Newton GEMMs: 0 = always full products (the reference's arithmetic),
// 1 = always upper-triangle tiles mirrored, 2 = per factor, symmetric only when the factor's previous solve
// converged within SYM_MAX_PREVIOUS_ITERATIONS (condition number <~ 1e4, where the two variants agree to
// < 1e-4; measured deviation grows like 3e-9 x condition number for both).
int g_symmetric_newton = 2;
// eigh solver: 0 = by order (block Jacobi below TRD_MIN_DIM), 1 = always block Jacobi, 2 = tridiagonalisation wherever it fits
int g_eigh_solver = 0;
constexpr int SYM_MAX_PREVIOUS_ITERATIONS = 14;
constexpr int SYM_REDO_ITERATIONS = 17;  // a symmetric solve that needed more is repeated with full products
std::map<std::string, Phase> g_phases;

// Named ranges for a tracer (rocprofv3 --marker-trace): with SHAMPOO_AMD_ROCTX=1 in the environment every phase of a call
// is bracketed on the host by roctxRangePush / roctxRangePop, the counterpart of the record_function ranges of the
// reference (preconditioner/preconditioner_list.py:23-46).  The marker library is looked up when the first phase starts,
// so nothing links against it and a process that does not ask for ranges never loads it.
struct Roctx {
  int (*push)(const char*) = nullptr;
  int (*pop)() = nullptr;
  Roctx() {
    const char* want = std::getenv("SHAMPOO_AMD_ROCTX");
    if (!want || want[0] == '\0' || want[0] == '0') return;
    for (const char* lib : {"librocprofiler-sdk-roctx.so", "libroctx64.so"}) {
      void* h = dlopen(lib, RTLD_NOW | RTLD_GLOBAL);
      if (!h) continue;
      push = reinterpret_cast<int (*)(const char*)>(dlsym(h, "roctxRangePushA"));
      pop = reinterpret_cast<int (*)()>(dlsym(h, "roctxRangePop"));
      if (push && pop) return;
      push = nullptr; pop = nullptr;
    }
  }
};
const Roctx& roctx() { static const Roctx r; return r; }

struct Span {
  Phase* ph = nullptr;
  hipStream_t s = nullptr;
  hipEvent_t stop = nullptr;
  bool range = false;
  Span(const char* name, hipStream_t st, double work, int launches, bool reset) {
    if (roctx().push) { (void)roctx().push(name); range = true; }
    if (!g_profiling) return;
    ph = &g_phases[name];
    if (reset) { ph->used = 0; ph->work = 0.0; ph->executed = 0.0; ph->launches = 0; }
    if (ph->used == ph->spans.size()) {
      hipEvent_t a, b;
      if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) { ph = nullptr; return; }
      ph->spans.emplace_back(a, b);
    }
    s = st;
    (void)hipEventRecord(ph->spans[ph->used].first, s);
    stop = ph->spans[ph->used].second;
    ph->used++;
    ph->work += work;
    ph->launches += launches;
  }
  ~Span() {
    if (ph) (void)hipEventRecord(stop, s);
    if (range) (void)roctx().pop();
  }
};

struct Factor {
  int block, side, d, dpad, root;
  float* factor;
  float* inv;
  float* eigvec;
  long long dense_off;   // offset (floats) of this factor inside the dense inverse cache
  long long norm_off;    // offset into the norm-partial array
  int norm_chunks;
  int wave;              // the amortized computations work through the factors in waves that share one scratch region
  long long wave_off;    // offset (floats) of this factor inside every dense scratch array of its wave
  long long eig_off;     // offset (floats) into the kept eigenvalue estimates (plans with eigenvector state)
};

}  // namespace

struct sa_plan {
  int n_blocks = 0;
  int symmetric_newton = 2;  // product policy of the coupled Newton iteration (sa_plan_set_symmetric_newton)
  int eigh_solver = 0;       // solver behind the eigendecompositions (sa_plan_set_eigh_solver)
  std::vector<sa_block_desc> blocks;
  std::vector<float*> grads;
  bool grads_bound = false;
  bool tables_valid = false;
  int table_mode = -1;  // 0: ghat from grad, 1: from filtered_grad, 2: from the beta3 temporary
  std::vector<Factor> factors;
  std::vector<int> block_factor[SA_MAX_ORDER];
  std::vector<long long> elem_off;
  std::vector<int> chunk_begin_all, ptile_begin_all;  // per block, over ALL blocks (fixed layout)
  long long total_elems = 0, dense_total = 0, norm_partials_total = 0;
  int total_chunks_all = 0, total_ptiles_all = 0;

  // Waves: consecutive factors whose dense scratch arrays (8 per factor, 16 with fp64 factors) fit the scratch budget
  // together.  An amortized computation handles one wave after the other in the same scratch region, so the workspace
  // grows with the budget instead of with the number of factors.  One wave (no budget) is the layout of a plan whose
  // factors are all solved at once.
  long long scratch_budget_bytes = 0;      // 0 = no limit
  std::vector<long long> wave_dense;       // per wave: floats of one dense scratch array
  int cur_wave = -1;                       // the wave an amortized computation is working on, -1 = every factor
  long long off_eigvals = 0, eig_total = 0;

  // workspace carve-up
  char* ws = nullptr;
  long long ws_bytes = 0, ws_needed = 0;
  long long off_inv_dense = 0, off_norms = 0, off_graft_partial = 0, off_ghat_partial = 0, off_ptile_partial = 0,
            off_norm_partial = 0, off_scratch = 0, scratch_floats = 0;
  bool inv_cache_valid = false;

  // device tables
  Table<BlockDev> t_blocks;
  Table<ChunkRef> t_chunks;
  Table<int> t_active_blocks;
  GemmTable syrk0, syrk1, g1_store, g1_norm, g2_norm, g2g_norm;
  GemmTable syrk0e, syrk1e;  // Gram problems that need the guarded loader (vectors: k = 1; ragged blocks), launched apart so that
                             // they do not force it on the rest
  // factor matrices kept in fp64 (factor_matrix_dtype = float64): fp64 averages in the SYRK epilogue, fp64 coupled
  // Newton root inverse on a scratch region twice the size; the inverse roots stay fp32
  bool factor_f64 = false;
  Table<Factor64> t_f64;
  Table<Eig64Job> t_eig64;
  Table<CastJob> t_cast;
  Table<Transpose64> t_tr64;
  double* d_norm64 = nullptr;  // one squared norm per factor
  struct GemmTable64 {
    Table<GemmProblem64> t;
    int total_tiles = 0;
    std::vector<GemmProblem64> build;
    void clear() { build.clear(); total_tiles = 0; }
    void add(GemmProblem64 q) {
      q.tiles = q.n / BM64;
      q.tile_begin = total_tiles;
      total_tiles += q.tiles * q.tiles;
      build.push_back(q);
    }
  };
  GemmTable64 n64_a[2], n64_pow[8], n64_m[2], n64_a0;
  Table<ChunkRef> t_all_chunks;  // chunks of every block, masked or not (train / eval switch of primal averaging)
  // KL-Shampoo: the Gram matrices of a two-sided block are taken of the gradient preconditioned along the other dim
  bool kl = false;
  GemmTable kl_right, kl_left;  // G X_R -> T buffer, X_L G -> P buffer
  // Newton, [0] full products / [1] symmetric products: X*M_p with M_p^2 per parity, power chain, M update per parity
  GemmTable nt_a[2][2], nt_pow[2][8], nt_m[2][2];
  GemmTable nt_a0[2];  // first iteration: launch A without X M_p (the init kernel wrote it)
  // Second lane of the coupled Newton iteration: a batch whose launches are too short to keep the chip busy between one
  // dependent stage and the next is cut into two halves that iterate side by side on two streams, each with its own
  // tables, control pass and mailbox.
  struct NewtonLane2 {
    GemmTable a[2][2], pow[2][8], m[2][2], a0[2];
    Table<int> ids;
    Table<SymFactor> sym;
  } nlane2;
  hipStream_t newton_stream = nullptr;
  hipEvent_t newton_ev[2] = {nullptr, nullptr};
  unsigned int ctl_seq2 = 0;
  int newton_split_tiles = 0;  // batches of fewer tiles per stage iterate as two halves (0 = never, the default)
  GemmTable nt_h[8];      // Horner products of the higher-order iteration
  // mode products of order-3 blocks: [mode 1 | mode 0 | mode 2][first stage (divides by bias_correction1)][last stage (norm)]
  GemmTable g3[3][2][2];
  // eigenvalue-corrected order-3 blocks: [statistic | rotate | rotate back][mode 1 | mode 0 | mode 2][first][last]
  GemmTable e3[3][3][2][2];
  bool has_order3 = false;
  Table<HoJob> t_ho;
  std::vector<int> newton_history;  // per factor: iterations of its last converged solve, 0 = none
  Table<SymFactor> t_sym;
  Table<NormJob> t_normjobs;
  Table<int> t_ids;
  // the same kinds of tables for the result pass of the coupled Newton call: a table per role keeps its content from
  // step to step, so nothing is uploaded again
  Table<int> t_ids_out;
  Table<NormJob> t_normjobs_out;
  Table<SymFactor> t_sym_out;
  Table<JacobiFactor> t_jacobi;
  Table<int2> t_sched;
  Table<EigInit> t_eiginit;
  Table<EigFinal> t_eigfinal;
  GemmTable eig_gemm;
  GemmTable ec_stat1, ec_stat2, ec_stat_l, ec_stat_r;          // corrected-eigenvalue update
  GemmTable ec_p1, ec_p1d, ec_p2, ec_p2d, ec_p3, ec_p3n, ec_p4, ec_p4n;  // eigenvalue-corrected preconditioning
  struct QrInner { Table<QrPanel> panel; GemmTable upd[3], merge[3]; };
  // Tables of the QR refresh.  Panels factored in registers (orders up to 1024) keep a set per panel and per outer block:
  // a refresh rewrites every set with the bytes it already holds and uploads nothing (an upload is a copy command of its
  // own on the stream, seven per panel).  Taller factors have narrow panels, hundreds of them: they share rings of four
  // and two sets, so that the host can fill the tables of the next panels while the GPU works.
  struct QrOuter { GemmTable g[6]; };
  std::vector<std::unique_ptr<QrInner>> qr_in;
  std::vector<std::unique_ptr<QrOuter>> qr_outer;
  GemmTable qr_aq, qr_b;
  Table<TrdJob> t_trd, t_trd_ql;  // every factor of the batch; those that take the QL iteration
  Table<TransposeJob> t_transpose;
  hipStream_t trd_stream = nullptr;  // second lane of the tridiagonalisation; applies QL rotations concurrently with the next chase
  int trd_lanes = 3;                 // the tridiagonalisation reduces a batch in this many parts side by side, one stream each
  hipStream_t trd_lane_stream[2] = {nullptr, nullptr};
  hipEvent_t trd_lane_ev[3] = {nullptr, nullptr, nullptr};
  hipEvent_t trd_ev[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
  Table<GemmProblem> t_trd_gemm;
  Table<RowScale> t_rowscale;
  Table<RankJob> t_rank;
  Table<RowsToCols> t_rows2cols;
  GemmTable eig_gemm_t;
  Table<Copy2D> t_copy;
  Table<DenseStateJob> t_dense_state[2];
  Table<NormPair> t_normpair;
  Table<SortJob> t_sort;
  bool eigenvalue_corrected = false;  // blocks carry a second moment in the eigenbasis (corrected_eigenvalues)
  bool has_eigvec = false;            // some factor stores its eigenvectors (eigenvalue-corrected or eigendecomposed Shampoo)
  // Eigenvalue-corrected blocks of order 2 with both eigenbases keep Q_L^T m Q_R, the filtered gradient in the eigenbasis,
  // next to m itself.  While the bases stand still it follows m by the same moving average (the rotation is linear), which
  // saves rotating m on every step.  It belongs to the filtered gradient after `rotm_version` prologues; -1 = not valid.
  long long off_rotm = 0;
  long long m_version = 0, rotm_version = -1;
  long long shared_rotation_steps = 0;  // steps that took the shared-rotation path
  std::vector<char> rotm_active;        // which blocks were active when the copy was last known to be consistent
  int n_active_blocks = 0;

  // Newton control state (device) and pinned readback
  unsigned int* d_err = nullptr;
  int* d_active = nullptr;
  int* d_report = nullptr;  // one allocation: d_iters, d_final_err, d_flags_in, d_flags, d_first_bad in this order
  int* d_iters = nullptr;
  int* d_final_parity = nullptr;
  float* d_final_err = nullptr;
  int* d_flags = nullptr;
  int* d_nactive = nullptr;
  int* h_pinned = nullptr;  // 6 * F + 16 ints
  int* d_flags_in = nullptr;   // per factor: the bias-corrected factor holds nan / inf (Newton path; d_flags then holds the results' flags)
  int* d_first_bad = nullptr;  // position in the batch of the first factor with a non-finite input or result
  // The coupled iterations are enqueued ahead of the device: every control pass reports (sequence number << 32 | factors
  // still active) into this word of pinned host memory, which the host polls instead of synchronising the stream.
  unsigned long long* h_mailbox = nullptr;
  unsigned long long* d_mailbox = nullptr;  // the same word as the device addresses it
  unsigned int ctl_seq = 0;

  // where the eigenvalue estimates of the last eigenbasis refresh sit in the workspace (valid until the next call)
  struct EigSource { const float* base = nullptr; long long stride = 0; const int* order = nullptr; };
  std::vector<EigSource> eig_source;

  // higher-order iteration: per factor {z, eps, |A|_inf, -}, the kept error and the termination flag
  float* d_ho = nullptr;
  float* d_kept_err = nullptr;
  int* d_hoflag = nullptr;

  // trace scaling of the bias-corrected factor before any root inverse / eigenbasis computation
  float* d_scale = nullptr;  // one multiplier per factor
  bool trace_scaling = false;
  float trace_exponent = 0.5f, trace_floor = 0.0f;
  const float* scale_of(int factor) const { return trace_scaling ? d_scale + factor : nullptr; }

  float* f(long long off) const { return reinterpret_cast<float*>(ws) + off; }
};

namespace {

void compute_layout(sa_plan* p) {
  long long o = 0;
  auto take = [&](long long n) { long long r = o; o += round_up(std::max<long long>(n, 1), 64); return r; };
  p->off_inv_dense = take(p->dense_total);
  p->off_norms = take(2LL * p->n_blocks);
  p->off_graft_partial = take(p->total_chunks_all);
  p->off_ghat_partial = take(p->total_chunks_all);
  p->off_ptile_partial = take(p->total_ptiles_all);
  p->off_norm_partial = take(p->norm_partials_total);
  // waves of consecutive factors under the scratch budget (at least one factor per wave)
  const long long mult = p->factor_f64 ? 16LL : 8LL;
  const long long budget = p->scratch_budget_bytes > 0 ? p->scratch_budget_bytes / (long long)sizeof(float) : -1;
  p->wave_dense.clear();
  long long cur = 0, widest = 0;
  for (Factor& f : p->factors) {
    const long long sz = (long long)f.dpad * f.dpad;
    if (p->wave_dense.empty() || (budget >= 0 && cur > 0 && mult * (cur + sz) > budget)) {
      p->wave_dense.push_back(0);
      cur = 0;
    }
    f.wave = (int)p->wave_dense.size() - 1;
    f.wave_off = cur;
    cur += sz;
    p->wave_dense.back() = cur;
    widest = std::max(widest, cur);
  }
  p->scratch_floats = std::max(mult * widest, 4LL * round_up(p->total_elems, 64) + 256);
  p->off_scratch = take(p->scratch_floats);
  p->off_eigvals = take(p->has_eigvec ? p->eig_total : 0);
  p->off_rotm = take(p->eigenvalue_corrected ? p->total_elems : 0);
  p->ws_needed = o * (long long)sizeof(float);
}

// dense array k (0..7) of the Newton scratch: X0 X1 M0 M1 Mp0 Mp1 S1 S2
inline float* newton_buf(const sa_plan* p, int k, const Factor& F) {
  return p->f(p->off_scratch + (long long)k * p->wave_dense[F.wave] + F.wave_off);
}
inline bool in_wave(const sa_plan* p, int factor) { return p->cur_wave < 0 || p->factors[factor].wave == p->cur_wave; }
enum { NB_X0 = 0, NB_X1 = 1, NB_M0 = 2, NB_M1 = 3, NB_MP0 = 4, NB_MP1 = 5, NB_S1 = 6, NB_S2 = 7 };

inline float* tbuf(const sa_plan* p) { return p->f(p->off_scratch); }
inline float* pbuf(const sa_plan* p) { return p->f(p->off_scratch + round_up(p->total_elems, 64) + 64); }
inline float* ghbuf(const sa_plan* p) { return p->f(p->off_scratch + 2 * (round_up(p->total_elems, 64) + 64)); }
inline float* t2buf(const sa_plan* p) { return p->f(p->off_scratch + 3 * (round_up(p->total_elems, 64) + 64)); }

// Packed fp32 factor the fp32 solvers read: the state itself, or (plans with float64 factors) its rounded copy in the
// ninth scratch array, which stage_fp32_factors refreshes.
inline const float* packed32(const sa_plan* p, const Factor& f) {
  return p->factor_f64 ? newton_buf(p, 8, f) : f.factor;
}

int stage_fp32_factors(sa_plan* p, const std::vector<int>& ids, hipStream_t s) {
  if (!p->factor_f64 || ids.empty()) return SA_OK;
  SACHECK(p->t_cast.begin(ids.size()));
  long long most = 0;
  for (size_t i = 0; i < ids.size(); ++i) {
    const Factor& f = p->factors[ids[i]];
    const long long n = (long long)f.d * (f.d + 1) / 2;
    p->t_cast.host[i] = CastJob{reinterpret_cast<const double*>(f.factor), newton_buf(p, 8, f), n};
    most = std::max(most, n);
  }
  SACHECK(p->t_cast.upload(s));
  hipLaunchKernelGGL(f64_cast_kernel, dim3((unsigned)std::min<long long>((most + 255) / 256, 1024), (unsigned)ids.size()), dim3(256), 0, s,
                     p->t_cast.dev);
  HIPCHECK(hipGetLastError());
  return SA_OK;
}

int need_ws(const sa_plan* p) {
  if (!p->ws) return fail(SA_ERR_WORKSPACE, "no workspace bound (sa_plan_bind_workspace)");
  return SA_OK;
}

bool block_active(const sa_plan* p, int b) { return p->grads[b] != nullptr; }

// Rebuild every table that depends on the bound gradients / mask / filtered-gradient mode.
int rebuild_tables(sa_plan* p, int mode, hipStream_t s) {
  SACHECK(need_ws(p));
  const int nb = p->n_blocks;
  // blocks
  SACHECK(p->t_blocks.begin(nb));
  std::vector<int> active;
  std::vector<ChunkRef> chunks;
  for (int b = 0; b < nb; ++b) {
    const sa_block_desc& d = p->blocks[b];
    BlockDev& B = p->t_blocks.host[b];
    std::memset(&B, 0, sizeof(B));
    B.param = d.param;
    B.grad = p->grads[b];
    B.filtered_grad = d.filtered_grad;
    B.adagrad = d.adagrad;
    B.momentum = d.momentum_buffer;
    B.weight_buffer = d.weight_buffer;
    B.ld = d.ld;
    B.rows = d.rows;
    B.cols = d.cols;
    B.mid = d.mid;
    B.ld_outer = d.ld_outer;
    const long long eo = p->elem_off[b];
    // a block is preconditioned if a side has a Kronecker factor or, for eigenvalue-corrected Shampoo, a fixed basis
    const bool precond = p->block_factor[0][b] >= 0 || p->block_factor[1][b] >= 0 || p->block_factor[2][b] >= 0 ||
                         (d.corrected_eigenvalues && (d.eigenvectors[0] || d.eigenvectors[1] || d.eigenvectors[2]));
    B.ghat_tmp = (mode == 2) ? ghbuf(p) + eo : nullptr;
    if (mode == 0) {
      if (d.mid > 0 && precond) {
        // the mode products of an order-3 block read a dense copy of the gradient (gathered before they run)
        B.ghat_src = ghbuf(p) + eo; B.ghat_ld = d.cols;
        B.g3_ghat = ghbuf(p) + eo;
      } else {
        B.ghat_src = B.grad; B.ghat_ld = d.ld;
      }
    }
    else if (mode == 1) { B.ghat_src = d.filtered_grad; B.ghat_ld = d.cols; }
    else { B.ghat_src = ghbuf(p) + eo; B.ghat_ld = d.cols; }
    B.p_is_ghat = precond ? 0 : 1;
    if (precond) { B.p_src = pbuf(p) + eo; B.p_ld = d.cols; }
    else { B.p_src = B.ghat_src; B.p_ld = B.ghat_ld; B.p_like_grad = (B.ghat_src == B.grad) ? 1 : 0; }
    if (d.mid > 0 && block_active(p, b)) {
      // dense copies for the factor updates: d0 x (d1 d2) in the T buffer, d1 x (d0 d2) in the P buffer
      if (d.factor[0] || d.factor[2]) B.g3_dense = tbuf(p) + eo;
      if (d.factor[1]) B.g3_perm = pbuf(p) + eo;
      // the rotated second moment is updated from a dense copy of the raw gradient
      if (d.corrected_eigenvalues && precond) B.g3_stat = ghbuf(p) + eo;
    }
    const bool contig = (d.ld == d.cols) && (d.mid == 0 || d.ld_outer == (long long)d.mid * d.ld);
    B.contig = contig ? 1 : 0;
    auto al = [](const void* q) { return q == nullptr || (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    const bool shape_ok = contig || (d.cols % 4 == 0 && d.ld % 4 == 0 && (d.mid == 0 || d.ld_outer % 4 == 0));
    B.vec = (shape_ok && al(B.param) && al(B.grad) && al(B.filtered_grad) && al(B.adagrad) && al(B.momentum) && al(B.weight_buffer) &&
             al(B.ghat_tmp)) ? 1 : 0;
    const bool p_contig = (B.p_ld == d.cols);
    B.p_vec = ((p_contig || (d.cols % 4 == 0 && B.p_ld % 4 == 0)) && al(B.p_src)) ? 1 : 0;
    B.chunk_begin = B.chunk_end = 0;
    B.ptile_begin = p->ptile_begin_all[b];
    B.ptile_end = p->ptile_begin_all[b + 1];
    if (block_active(p, b)) {
      active.push_back(b);
      B.chunk_begin = (int)chunks.size();
      const long long n_el = (long long)d.rows * d.cols;
      for (long long e = 0; e < n_el; e += EW_CHUNK) chunks.push_back(ChunkRef{b, (int)e});
      B.chunk_end = (int)chunks.size();
    }
  }
  SACHECK(p->t_blocks.upload(s));
  SACHECK(p->t_chunks.begin(chunks.size()));
  if (!chunks.empty()) std::memcpy(p->t_chunks.host, chunks.data(), chunks.size() * sizeof(ChunkRef));
  SACHECK(p->t_chunks.upload(s));
  SACHECK(p->t_active_blocks.begin(active.size()));
  if (!active.empty()) std::memcpy(p->t_active_blocks.host, active.data(), active.size() * sizeof(int));
  SACHECK(p->t_active_blocks.upload(s));
  p->n_active_blocks = (int)active.size();

  // factor-update tables
  p->syrk0.clear();
  p->syrk1.clear();
  p->syrk0e.clear();
  p->syrk1e.clear();
  auto add_syrk = [&](int which, const GemmProblem& q) {
    const bool al = q.M % BM == 0 && q.N % BN == 0 && q.K % BK == 0 && q.a_vec && q.b_vec;
    (which == 0 ? (al ? p->syrk0 : p->syrk0e) : (al ? p->syrk1 : p->syrk1e)).add(q, true);
  };
  p->kl_right.clear();
  p->kl_left.clear();
  for (int b : active) {
    const sa_block_desc& d = p->blocks[b];
    const float* G = p->grads[b];
    if (p->kl && d.mid == 0 && d.factor[0] && d.factor[1]) {
      // KL-Shampoo (shampoo_preconditioner_list.py:1945-1987): L from G X_R, R from X_L G, X the stored inverse roots
      const Factor& fl = p->factors[p->block_factor[0][b]];
      const Factor& fr = p->factors[p->block_factor[1][b]];
      const float* XL = p->f(p->off_inv_dense) + fl.dense_off;
      const float* XR = p->f(p->off_inv_dense) + fr.dense_off;
      const long long eo = p->elem_off[b];
      float* TR = tbuf(p) + eo;
      float* TL = pbuf(p) + eo;
      GemmProblem r{};
      r.A = G; r.lda = d.ld; r.a_vec = vec_ok(G, d.ld);
      r.B = XR; r.ldb = fr.dpad; r.b_vec = vec_ok(XR, fr.dpad);
      r.C = TR; r.ldc = d.cols; r.M = d.rows; r.N = d.cols; r.K = d.cols;
      p->kl_right.add(r, false);
      GemmProblem l{};
      l.A = XL; l.lda = fl.dpad; l.a_vec = vec_ok(XL, fl.dpad);
      l.B = G; l.ldb = d.ld; l.b_vec = vec_ok(G, d.ld);
      l.C = TL; l.ldc = d.cols; l.M = d.rows; l.N = d.cols; l.K = d.rows;
      p->kl_left.add(l, false);
      GemmProblem q{};
      q.A = TR; q.B = TR; q.C = d.factor[0];
      q.lda = d.cols; q.ldb = d.cols; q.ldc = 0;
      q.M = d.rows; q.N = d.rows; q.K = d.cols;
      q.a_vec = q.b_vec = vec_ok(TR, d.cols);
      add_syrk(0, q);
      GemmProblem w{};
      w.A = TL; w.B = TL; w.C = d.factor[1];
      w.lda = d.cols; w.ldb = d.cols; w.ldc = 0;
      w.M = d.cols; w.N = d.cols; w.K = d.rows;
      w.a_vec = w.b_vec = vec_ok(TL, d.cols);
      add_syrk(1, w);
      continue;
    }
    if (d.mid > 0) {
      // order 3, from the dense copies: factor k = unfolding_k unfolding_k^T
      const BlockDev& B = p->t_blocks.host[b];
      const int d0 = d.rows / d.mid, d1 = d.mid, d2 = d.cols;
      auto gram = [&](const float* T, long long ld, int dim, int K, float* C, bool k_major) {
        GemmProblem q{};
        q.A = T; q.B = T; q.C = C;
        q.lda = ld; q.ldb = ld; q.ldc = 0;
        q.M = dim; q.N = dim; q.K = K;
        q.a_vec = q.b_vec = vec_ok(T, ld);
        add_syrk(k_major ? 1 : 0, q);
      };
      if (d.factor[0]) gram(B.g3_dense, (long long)d1 * d2, d0, d1 * d2, d.factor[0], false);
      if (d.factor[1]) gram(B.g3_perm, (long long)d0 * d2, d1, d0 * d2, d.factor[1], false);
      if (d.factor[2]) gram(B.g3_dense, d2, d2, d0 * d1, d.factor[2], true);
      continue;
    }
    if (d.factor[0]) {  // L = G G^T  (rows x rows, K = cols)
      GemmProblem q{};
      q.A = G; q.B = G; q.C = d.factor[0];
      q.lda = d.ld; q.ldb = d.ld; q.ldc = 0;
      q.M = d.rows; q.N = d.rows; q.K = d.cols;
      q.a_vec = q.b_vec = vec_ok(G, d.ld);
      add_syrk(0, q);
    }
    if (d.factor[1]) {  // R = G^T G  (cols x cols, K = rows)
      GemmProblem q{};
      q.A = G; q.B = G; q.C = d.factor[1];
      q.lda = d.ld; q.ldb = d.ld; q.ldc = 0;
      q.M = d.cols; q.N = d.cols; q.K = d.rows;
      q.a_vec = q.b_vec = vec_ok(G, d.ld);
      add_syrk(1, q);
    }
  }
  SACHECK(p->syrk0.commit(s));
  SACHECK(p->syrk1.commit(s));
  SACHECK(p->syrk0e.commit(s));
  SACHECK(p->syrk1e.commit(s));
  SACHECK(p->kl_right.commit(s));
  SACHECK(p->kl_left.commit(s));

  // eigenvalue-corrected tables
  for (GemmTable* g : {&p->ec_stat1, &p->ec_stat2, &p->ec_stat_l, &p->ec_stat_r, &p->ec_p1, &p->ec_p1d, &p->ec_p2, &p->ec_p2d,
                       &p->ec_p3, &p->ec_p3n, &p->ec_p4, &p->ec_p4n})
    g->clear();
  for (auto& a : p->e3) for (auto& b2 : a) for (auto& c2 : b2) for (auto& g : c2) g.clear();
  if (p->eigenvalue_corrected) {
    for (int b : active) {
      const sa_block_desc& d = p->blocks[b];
      BlockDev& B = p->t_blocks.host[b];
      if (d.mid > 0) {
        // order 3: three chains of mode products with the eigenbases (stage order mode 1, mode 0, mode 2):
        // statistic (raw gradient, squared EMA at the end), rotation of the filtered gradient (division at the end),
        // rotation back (norm at the end)
        const float* Q[3] = {d.eigenvectors[1], d.eigenvectors[0], d.eigenvectors[2]};
        const int d0 = d.rows / d.mid, d1 = d.mid, d2 = d.cols;
        const int qd[3] = {d1, d0, d2};
        int n_stages = 0;
        for (const float* q : Q) n_stages += q ? 1 : 0;
        if (!d.corrected_eigenvalues || n_stages == 0) continue;
        const long long eo3 = p->elem_off[b];
        float* part3 = p->f(p->off_ptile_partial) + p->ptile_begin_all[b];
        auto tile_count = [](long long m, long long n) { return (int)(((m + BM - 1) / BM) * ((n + BN - 1) / BN)); };
        float* pong[2] = {tbuf(p) + eo3, t2buf(p) + eo3};
        int flip = 0;
        const float* rotated = nullptr;  // result of the rotation chain
        for (int chain = 0; chain < 3; ++chain) {
          const float* src = chain == 0 ? B.g3_stat : (chain == 1 ? B.ghat_src : rotated);
          int done = 0;
          for (int kind = 0; kind < 3; ++kind) {
            if (!Q[kind]) continue;
            const bool first = done == 0, last = done == n_stages - 1;
            float* out;
            if (last && chain == 0) out = d.corrected_eigenvalues;
            else if (last && chain == 2) out = pbuf(p) + eo3;
            else { out = pong[flip]; flip ^= 1; }
            float* c2 = nullptr;
            if (last && chain == 1) c2 = d.corrected_eigenvalues;
            if (last && chain == 2) c2 = part3;
            GemmTable& tab = p->e3[chain][kind][first ? 1 : 0][last ? 1 : 0];
            const float* Qk = Q[kind];
            const int dk = qd[kind];
            if (kind == 0) {
              const int per = tile_count(d1, d2);
              for (int i0 = 0; i0 < d0; ++i0) {
                GemmProblem q{};
                q.A = Qk; q.lda = dk; q.a_vec = vec_ok(Qk, dk);
                q.B = src + (long long)i0 * d1 * d2; q.ldb = d2; q.b_vec = vec_ok(q.B, q.ldb);
                q.C = out + (long long)i0 * d1 * d2; q.ldc = d2;
                q.M = d1; q.N = d2; q.K = d1;
                if (c2) q.C2 = (chain == 2) ? c2 + (long long)i0 * per : c2 + (long long)i0 * d1 * d2;
                tab.add(q, false);
              }
              if (last && chain == 2) B.ptile_end = B.ptile_begin + d0 * per;
            } else if (kind == 1) {
              GemmProblem q{};
              q.A = Qk; q.lda = dk; q.a_vec = vec_ok(Qk, dk);
              q.B = src; q.ldb = (long long)d1 * d2; q.b_vec = vec_ok(q.B, q.ldb);
              q.C = out; q.ldc = (long long)d1 * d2;
              q.M = d0; q.N = d1 * d2; q.K = d0;
              q.C2 = c2;
              if (last && chain == 2) B.ptile_end = B.ptile_begin + tile_count(d0, (long long)d1 * d2);
              tab.add(q, false);
            } else {
              GemmProblem q{};
              q.A = src; q.lda = d2; q.a_vec = vec_ok(q.A, q.lda);
              q.B = Qk; q.ldb = dk; q.b_vec = vec_ok(Qk, dk);
              q.C = out; q.ldc = d2;
              q.M = d0 * d1; q.N = d2; q.K = d2;
              q.C2 = c2;
              if (last && chain == 2) B.ptile_end = B.ptile_begin + tile_count((long long)d0 * d1, d2);
              tab.add(q, false);
            }
            src = out;
            ++done;
          }
          if (chain == 1) rotated = src;
        }
        continue;
      }
      // eigenvectors[side] without factor[side] is a fixed basis: it rotates, but has no statistics and is never
      // refreshed (an ignored basis change, shampoo_preconditioner_list.py:1843-1865, passes the identity)
      const float* QL = d.eigenvectors[0];
      const float* QR = d.eigenvectors[1];
      const int f0 = QL ? 0 : -1, f1 = QR ? 0 : -1;
      if (!d.corrected_eigenvalues || (f0 < 0 && f1 < 0)) continue;
      const long long eo = p->elem_off[b];
      float* part = p->f(p->off_ptile_partial) + p->ptile_begin_all[b];
      const float* G = p->grads[b];
      auto mk = [&](const float* A, long long lda, const float* Bm, long long ldb, float* C, float* C2, int K) {
        GemmProblem q{};
        q.A = A; q.lda = lda; q.a_vec = vec_ok(A, lda);
        q.B = Bm; q.ldb = ldb; q.b_vec = vec_ok(Bm, ldb);
        q.C = C; q.C2 = C2; q.ldc = d.cols;
        q.M = d.rows; q.N = d.cols; q.K = K;
        return q;
      };
      float* T = tbuf(p) + eo;
      float* T2 = t2buf(p) + eo;
      float* Pb = pbuf(p) + eo;
      if (f0 >= 0 && f1 >= 0) {
        p->ec_stat1.add(mk(QL, d.rows, G, d.ld, T, nullptr, d.rows), false);                       // T = QL^T G   (A_KM)
        // corr <- EMA (T QR)^2; the fused form of the step also advances the rotated filtered gradient and writes T2
        GemmProblem st2 = mk(T, d.cols, QR, d.cols, d.corrected_eigenvalues, mode == 1 ? p->f(p->off_rotm) + eo : nullptr, d.cols);
        st2.C3 = T2;
        p->ec_stat2.add(st2, false);
        p->ec_p1.add(mk(QL, d.rows, B.ghat_src, B.ghat_ld, T, nullptr, d.rows), false);             // T = QL^T Ghat (b_div)
        GemmProblem p2 = mk(T, d.cols, QR, d.cols, T2, d.corrected_eigenvalues, d.cols);             // T2 = (T QR)/den
        if (mode == 1) p2.C3 = p->f(p->off_rotm) + eo;  // and Q_L^T m Q_R itself
        p->ec_p2.add(p2, false);
        p->ec_p3.add(mk(QL, d.rows, T2, d.cols, T, nullptr, d.rows), false);                         // T = QL T2
        p->ec_p4.add(mk(T, d.cols, QR, d.cols, Pb, part, d.cols), false);                            // P = T QR^T (B_NK)
      } else if (f0 >= 0) {
        p->ec_stat_l.add(mk(QL, d.rows, G, d.ld, d.corrected_eigenvalues, nullptr, d.rows), false);
        p->ec_p1d.add(mk(QL, d.rows, B.ghat_src, B.ghat_ld, T2, d.corrected_eigenvalues, d.rows), false);
        p->ec_p3n.add(mk(QL, d.rows, T2, d.cols, Pb, part, d.rows), false);
      } else {
        p->ec_stat_r.add(mk(G, d.ld, QR, d.cols, d.corrected_eigenvalues, nullptr, d.cols), false);
        p->ec_p2d.add(mk(B.ghat_src, B.ghat_ld, QR, d.cols, T2, d.corrected_eigenvalues, d.cols), false);
        p->ec_p4n.add(mk(T2, d.cols, QR, d.cols, Pb, part, d.cols), false);
      }
    }
  }
  for (GemmTable* g : {&p->ec_stat1, &p->ec_stat2, &p->ec_stat_l, &p->ec_stat_r, &p->ec_p1, &p->ec_p1d, &p->ec_p2, &p->ec_p2d,
                       &p->ec_p3, &p->ec_p3n, &p->ec_p4, &p->ec_p4n})
    SACHECK(g->commit(s));
  for (auto& a : p->e3) for (auto& b2 : a) for (auto& c2 : b2) for (auto& g : c2) SACHECK(g.commit(s));

  // preconditioning tables (root-inverse Shampoo)
  p->g1_store.clear(); p->g1_norm.clear(); p->g2_norm.clear(); p->g2g_norm.clear();
  for (auto& a : p->g3) for (auto& b2 : a) for (auto& g : b2) g.clear();
  for (int b : active) {
    if (p->eigenvalue_corrected) break;
    const sa_block_desc& d = p->blocks[b];
    BlockDev& B = p->t_blocks.host[b];
    const int f0 = p->block_factor[0][b], f1 = p->block_factor[1][b];
    const long long eo = p->elem_off[b];
    float* part = p->f(p->off_ptile_partial) + p->ptile_begin_all[b];
    if (d.mid > 0) {
      // P = Ghat x_1 X1 x_0 X0 x_2 X2 on dense buffers (mode products commute; each dim keeps its place)
      const int f2 = p->block_factor[2][b];
      const int d0 = d.rows / d.mid, d1 = d.mid, d2 = d.cols;
      const int kinds[3] = {f1, f0, f2};  // stage order: mode 1, mode 0, mode 2
      int n_stages = 0;
      for (int k : kinds) n_stages += k >= 0 ? 1 : 0;
      const float* src = B.ghat_src;  // dense d0 x d1 x d2
      float* pong[2] = {tbuf(p) + eo, t2buf(p) + eo};
      int done = 0;
      for (int kind = 0; kind < 3; ++kind) {
        if (kinds[kind] < 0) continue;
        const Factor& F = p->factors[kinds[kind]];
        const float* X = p->f(p->off_inv_dense) + F.dense_off;
        const bool first = done == 0, last = done == n_stages - 1;
        float* out = last ? pbuf(p) + eo : pong[done & 1];
        GemmTable& tab = p->g3[kind][first ? 1 : 0][last ? 1 : 0];
        auto tile_count = [](long long m, long long n) { return (int)(((m + BM - 1) / BM) * ((n + BN - 1) / BN)); };
        if (kind == 0) {  // every slice i0: X1 (d1 x d1) . src[i0] (d1 x d2)
          const int per = tile_count(d1, d2);
          for (int i0 = 0; i0 < d0; ++i0) {
            GemmProblem q{};
            q.A = X; q.lda = F.dpad; q.a_vec = 1;
            q.B = src + (long long)i0 * d1 * d2; q.ldb = d2; q.b_vec = vec_ok(q.B, q.ldb);
            q.C = out + (long long)i0 * d1 * d2; q.ldc = d2;
            q.M = d1; q.N = d2; q.K = d1;
            if (last) q.C2 = part + (long long)i0 * per;
            tab.add(q, false);
          }
          if (last) B.ptile_end = B.ptile_begin + d0 * per;
        } else if (kind == 1) {  // X0 (d0 x d0) . src as d0 x (d1 d2)
          GemmProblem q{};
          q.A = X; q.lda = F.dpad; q.a_vec = 1;
          q.B = src; q.ldb = (long long)d1 * d2; q.b_vec = vec_ok(q.B, q.ldb);
          q.C = out; q.ldc = (long long)d1 * d2;
          q.M = d0; q.N = d1 * d2; q.K = d0;
          if (last) { q.C2 = part; B.ptile_end = B.ptile_begin + tile_count(d0, (long long)d1 * d2); }
          tab.add(q, false);
        } else {  // src as (d0 d1) x d2 . X2 (d2 x d2)
          GemmProblem q{};
          q.A = src; q.lda = d2; q.a_vec = vec_ok(q.A, q.lda);
          q.B = X; q.ldb = F.dpad; q.b_vec = 1;
          q.C = out; q.ldc = d2;
          q.M = d0 * d1; q.N = d2; q.K = d2;
          if (last) { q.C2 = part; B.ptile_end = B.ptile_begin + tile_count((long long)d0 * d1, d2); }
          tab.add(q, false);
        }
        src = out;
        ++done;
      }
      continue;
    }
    if (f0 >= 0) {
      const Factor& F = p->factors[f0];
      GemmProblem q{};
      q.A = p->f(p->off_inv_dense) + F.dense_off; q.lda = F.dpad; q.a_vec = 1;
      q.B = B.ghat_src; q.ldb = B.ghat_ld; q.b_vec = vec_ok(B.ghat_src, B.ghat_ld);
      q.M = d.rows; q.N = d.cols; q.K = d.rows;
      q.ldc = d.cols;
      if (f1 >= 0) { q.C = tbuf(p) + eo; p->g1_store.add(q, false); }
      else { q.C = pbuf(p) + eo; q.C2 = part; p->g1_norm.add(q, false); }
    }
    if (f1 >= 0) {
      const Factor& F = p->factors[f1];
      GemmProblem q{};
      q.B = p->f(p->off_inv_dense) + F.dense_off; q.ldb = F.dpad; q.b_vec = 1;
      q.M = d.rows; q.N = d.cols; q.K = d.cols;
      q.C = pbuf(p) + eo; q.ldc = d.cols; q.C2 = part;
      if (f0 >= 0) {
        q.A = tbuf(p) + eo; q.lda = d.cols; q.a_vec = vec_ok(q.A, q.lda);
        p->g2_norm.add(q, false);
      } else {
        q.A = B.ghat_src; q.lda = B.ghat_ld; q.a_vec = vec_ok(q.A, q.lda);
        p->g2g_norm.add(q, false);
      }
    }
  }
  SACHECK(p->g1_store.commit(s));
  SACHECK(p->g1_norm.commit(s));
  SACHECK(p->g2_norm.commit(s));
  SACHECK(p->g2g_norm.commit(s));
  for (auto& a : p->g3) for (auto& b2 : a) for (auto& g : b2) SACHECK(g.commit(s));
  if (p->has_order3) SACHECK(p->t_blocks.upload(s));  // ptile ranges of order-3 blocks were set above
  p->tables_valid = true;
  // new gradient pointers alone leave the rotated filtered gradient valid; a block that joins or leaves does not (its
  // filtered gradient stood still while the version counter ran on), and neither does another source of Ghat
  std::vector<char> now(nb, 0);
  for (int b : active) now[b] = 1;
  if (now != p->rotm_active || mode != p->table_mode) p->rotm_version = -1;
  p->rotm_active.swap(now);
  p->table_mode = mode;
  return SA_OK;
}

int mode_of(const sa_step_scalars* s) { return s->filtered_grad_mode; }

int ensure_tables(sa_plan* p, const sa_step_scalars* s, hipStream_t st) {
  if (!p->grads_bound) return fail(SA_ERR_STATE, "gradients not bound (sa_plan_bind_gradients)");
  const int mode = s ? mode_of(s) : (p->table_mode < 0 ? 1 : p->table_mode);
  if (!p->tables_valid || p->table_mode != mode) return rebuild_tables(p, mode, st);
  return SA_OK;
}

int validate_scalars(const sa_plan* p, const sa_step_scalars* s) {
  if (!s) return fail(SA_ERR_INVALID, "step scalars are NULL");
  for (int b = 0; b < p->n_blocks; ++b) {
    const sa_block_desc& d = p->blocks[b];
    if (s->beta1 != 0.0f && !d.filtered_grad) return fail(SA_ERR_INVALID, "beta1 != 0 needs filtered_grad state in every block");
    if (s->graft_type == SA_GRAFT_ADAGRAD && !d.adagrad) return fail(SA_ERR_INVALID, "adagrad-family grafting needs adagrad state in every block");
    if (s->momentum != 0.0f && !d.momentum_buffer) return fail(SA_ERR_INVALID, "momentum != 0 needs momentum_buffer state in every block");
    if (s->use_primal_averaging && !d.weight_buffer) return fail(SA_ERR_INVALID, "primal averaging needs weight_buffer state in every block");
    if (s->use_primal_averaging && s->momentum != 0.0f) return fail(SA_ERR_INVALID, "classic momentum and primal averaging exclude each other");
  }
  if (!(s->bias_correction1 != 0.0f) || !(s->graft_bias_correction2 != 0.0f)) return fail(SA_ERR_INVALID, "bias corrections must be non-zero divisors");
  if (s->filtered_grad_mode < 0 || s->filtered_grad_mode > 2 || (s->filtered_grad_mode == 0) != (s->beta1 == 0.0f))
    return fail(SA_ERR_INVALID, "filtered_grad_mode must be 0 exactly when beta1 == 0, else 1 (beta3 == beta1) or 2");
  return SA_OK;
}

// packed -> dense mirrored cache of every inverse root
int refresh_inverse_cache(sa_plan* p, hipStream_t s) {
  if (p->inv_cache_valid || p->factors.empty() || p->eigenvalue_corrected) { p->inv_cache_valid = true; return SA_OK; }
  const int F = (int)p->factors.size();
  SACHECK(p->t_sym.begin(F));
  int tiles = 0;
  for (int i = 0; i < F; ++i) {
    const Factor& f = p->factors[i];
    SymFactor& S = p->t_sym.host[i];
    std::memset(&S, 0, sizeof(S));
    S.packed_in = f.inv;
    S.dense_out[0] = p->f(p->off_inv_dense) + f.dense_off;
    S.d = f.d; S.dpad = f.dpad; S.tiles = f.dpad / ST; S.root = f.root; S.enabled = 1;
    S.tile_begin = tiles;
    tiles += S.tiles * (S.tiles + 1) / 2;
  }
  SACHECK(p->t_sym.upload(s));
  hipLaunchKernelGGL((sym_pass_kernel<SYM_UNPACK>), dim3(tiles), dim3(256), 0, s, p->t_sym.dev, F, 1.0f, 0.0f, 0.0f, 0.0f);
  HIPCHECK(hipGetLastError());
  p->inv_cache_valid = true;
  return SA_OK;
}

}  // namespace

// ============================================================================================
// C ABI
// ============================================================================================

// Launches one chain of the order-3 eigenvalue-corrected tables.  chain 0 / 1 multiply by the transposed bases
// (into the eigenbasis), chain 2 by the bases (back); `mid` are the scalars of the stages that are not last,
// `fin` those of the last stage (first[] variants add the division of the source operand).
template <int EPI_LAST>
static int launch_e3_chain(sa_plan* p, int chain, const GemmScalars& mid, const GemmScalars& fin, float src_div, hipStream_t s) {
  for (int kind = 0; kind < 3; ++kind)
    for (int first = 0; first < 2; ++first) {
      GemmScalars a = mid, b = fin;
      if (first && src_div != 1.0f) {
        (kind == 2 ? a.a_div : a.b_div) = src_div;
        (kind == 2 ? b.a_div : b.b_div) = src_div;
      }
      GemmTable& t0 = p->e3[chain][kind][first][0];
      GemmTable& t1 = p->e3[chain][kind][first][1];
      if (chain < 2) {
        if (kind < 2) {
          SACHECK((launch_gemm_auto<A_KM, B_KN, EPI_STORE>(t0, a, s)));
          SACHECK((launch_gemm_auto<A_KM, B_KN, EPI_LAST>(t1, b, s)));
        } else {
          SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_STORE>(t0, a, s)));
          SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_LAST>(t1, b, s)));
        }
      } else {
        if (kind < 2) {
          SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_STORE>(t0, a, s)));
          SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_LAST>(t1, b, s)));
        } else {
          SACHECK((launch_gemm_auto<A_MK, B_NK, EPI_STORE>(t0, a, s)));
          SACHECK((launch_gemm_auto<A_MK, B_NK, EPI_LAST>(t1, b, s)));
        }
      }
    }
  return SA_OK;
}

template <int EPI>
static int launch_gemm64(sa_plan::GemmTable64& g, double mp_scale, double mp_diag, hipStream_t s) {
  if (g.total_tiles == 0) return SA_OK;
  const int per = (g.total_tiles + NUM_XCD - 1) / NUM_XCD;
  hipLaunchKernelGGL((grouped_gemm64_kernel<EPI>), dim3(per * NUM_XCD), dim3(GEMM_THREADS), 0, s, g.t.dev, (int)g.t.n,
                     g.total_tiles, mp_scale, mp_diag);
  HIPCHECK(hipGetLastError());
  return SA_OK;
}

// Runs an amortized computation wave by wave.  `run(iterations, status)` is the computation itself: it handles the
// factors of p->cur_wave (all of them for -1), writes every entry of its two output arrays (skipped factors included)
// and may leave eigenvalue sources that point into the scratch region.  The reference works through the factors in
// order and raises at the first non-finite one, so a wave that reports such a factor ends the call: later waves stay
// untouched and skipped.
template <class Run>
static int for_each_wave(sa_plan* p, int32_t* iterations_out, int32_t* status_out, hipStream_t s, Run&& run) {
  const int F = (int)p->factors.size();
  const int n_waves = (int)p->wave_dense.size();
  if (n_waves <= 1 || F == 0) {
    p->cur_wave = -1;
    return run(iterations_out, status_out);
  }
  for (int i = 0; i < F; ++i) {
    if (iterations_out) iterations_out[i] = 0;
    status_out[i] = SA_FACTOR_SKIPPED;
  }
  std::vector<int32_t> it(F, 0), st(F, SA_FACTOR_SKIPPED);
  std::vector<sa_plan::EigSource> kept(F);
  bool any_source = false;
  int rc = SA_OK;
  for (int w = 0; w < n_waves && rc == SA_OK; ++w) {
    bool any = false;
    for (int i = 0; i < F && !any; ++i) any = p->factors[i].wave == w && block_active(p, p->factors[i].block);
    if (!any) continue;
    p->cur_wave = w;
    rc = run(it.data(), st.data());
    p->cur_wave = -1;
    if (rc != SA_OK) break;
    bool stop = false;
    for (int i = 0; i < F; ++i) {
      if (p->factors[i].wave != w) continue;
      if (iterations_out) iterations_out[i] = it[i];
      status_out[i] = st[i];
      stop = stop || st[i] == SA_FACTOR_INPUT_NONFINITE || st[i] == SA_FACTOR_RESULT_NONFINITE;
      // eigenvalue estimates left in the scratch region move to their kept place before the next wave overwrites them
      if ((int)p->eig_source.size() == F && p->eig_source[i].base != nullptr) {
        const sa_plan::EigSource& e = p->eig_source[i];
        float* dst = p->f(p->off_eigvals) + p->factors[i].eig_off;
        const int d = p->factors[i].d;
        hipLaunchKernelGGL(gather_strided_kernel, dim3((d + 255) / 256), dim3(256), 0, s, e.base, e.stride, e.order, dst, d);
        if (hipGetLastError() != hipSuccess) { rc = fail(SA_ERR_HIP, "gather of eigenvalue estimates failed"); break; }
        kept[i] = sa_plan::EigSource{dst, 1, nullptr};
        any_source = true;
      }
    }
    if (stop) break;
  }
  p->cur_wave = -1;
  if (any_source) p->eig_source = kept;
  return rc;
}

extern "C" {

const char* sa_last_error(void) { return g_err.c_str(); }
int32_t sa_abi_version(void) { return 4; }
static_assert(sizeof(sa_block_desc) == 168, "sa_block_desc layout changed: bump sa_abi_version and the ctypes mirror");
static_assert(sizeof(sa_step_scalars) == 76, "sa_step_scalars layout changed: bump sa_abi_version and the ctypes mirror");

int32_t sa_set_profiling(int32_t enabled) {
  // switching the timers on forgets what earlier runs recorded: a phase that the coming calls never enter reads -1
  if (enabled != 0 && !g_profiling)
    for (auto& kv : g_phases) { kv.second.used = 0; kv.second.work = 0.0; kv.second.executed = 0.0; kv.second.launches = 0; }
  g_profiling = enabled != 0;
  return SA_OK;
}

double sa_phase_ms(const char* phase) {
  auto it = g_phases.find(phase ? phase : "");
  if (it == g_phases.end() || it->second.used == 0) return -1.0;
  double total = 0.0;
  for (size_t i = 0; i < it->second.used; ++i) {
    float ms = 0.f;
    if (hipEventSynchronize(it->second.spans[i].second) != hipSuccess) return -1.0;
    if (hipEventElapsedTime(&ms, it->second.spans[i].first, it->second.spans[i].second) != hipSuccess) return -1.0;
    total += ms;
  }
  return total;
}
double sa_phase_flops(const char* phase) {
  auto it = g_phases.find(phase ? phase : "");
  return it == g_phases.end() ? -1.0 : it->second.work;
}
double sa_phase_executed_flops(const char* phase) {
  auto it = g_phases.find(phase ? phase : "");
  return it == g_phases.end() ? -1.0 : it->second.executed;
}
int32_t sa_plan_set_kl_shampoo(sa_plan* p, int32_t enabled) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  if (enabled) {
    if (p->eigenvalue_corrected) return fail(SA_ERR_STATE, "KL-Shampoo needs inverse roots: not an eigenvalue-corrected plan");
    for (int b = 0; b < p->n_blocks; ++b) {
      const sa_block_desc& d = p->blocks[b];
      if (d.mid > 0 && (d.factor[0] != nullptr) + (d.factor[1] != nullptr) + (d.factor[2] != nullptr) > 1)
        return fail(SA_ERR_UNSUPPORTED, "KL-Shampoo is built for blocks of order 1 and 2");
    }
  }
  p->kl = enabled != 0;
  p->tables_valid = false;
  return SA_OK;
}

int32_t sa_plan_set_trace_scaling(sa_plan* p, int32_t enabled, float exponent, float floor) {
  if (!p) return fail(SA_ERR_INVALID, "sa_plan_set_trace_scaling: null plan");
  if (enabled && !(exponent > 0.0f && exponent <= 1.0f))
    return fail(SA_ERR_INVALID, "sa_plan_set_trace_scaling: exponent must be in (0, 1]");
  p->trace_scaling = enabled != 0;
  p->trace_exponent = exponent;
  p->trace_floor = floor;
  return SA_OK;
}

int32_t sa_set_eigh_solver(int32_t solver) {
  g_eigh_solver = solver < 0 ? 0 : (solver > 3 ? 3 : solver);
  return SA_OK;
}

int32_t sa_set_small_launch_tiles(int32_t tiles) {
  if (tiles < 0) return fail(SA_ERR_INVALID, "sa_set_small_launch_tiles: negative");
  SMALL_LAUNCH_TILES = tiles;
  return SA_OK;
}

int32_t sa_plan_set_symmetric_newton(sa_plan* p, int32_t policy) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  p->symmetric_newton = policy < 0 ? 0 : (policy > 2 ? 2 : policy);
  return SA_OK;
}

int32_t sa_plan_set_eigh_solver(sa_plan* p, int32_t solver) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  p->eigh_solver = solver < 0 ? 0 : (solver > 3 ? 3 : solver);
  return SA_OK;
}

int32_t sa_plan_rebind_params(sa_plan* p, float* const* params) {
  if (!p || !params) return fail(SA_ERR_INVALID, "sa_plan_rebind_params: NULL argument");
  for (int b = 0; b < p->n_blocks; ++b)
    if (!params[b]) return fail(SA_ERR_INVALID, "sa_plan_rebind_params: block " + std::to_string(b) + " has a NULL parameter");
  for (int b = 0; b < p->n_blocks; ++b) p->blocks[b].param = params[b];
  p->tables_valid = false;
  return SA_OK;
}

int32_t sa_set_symmetric_newton(int32_t enabled) {
  g_symmetric_newton = enabled < 0 ? 0 : (enabled > 2 ? 2 : enabled);
  return SA_OK;
}
int32_t sa_phase_launches(const char* phase) {
  auto it = g_phases.find(phase ? phase : "");
  return it == g_phases.end() ? -1 : it->second.launches;
}

int32_t sa_plan_create(const sa_block_desc* blocks, int32_t n_blocks, sa_plan** plan_out) {
  if (!blocks || n_blocks <= 0 || !plan_out) return fail(SA_ERR_INVALID, "sa_plan_create: bad arguments");
  sa_plan* p = new sa_plan();
  p->n_blocks = n_blocks;
  p->symmetric_newton = g_symmetric_newton;
  p->eigh_solver = g_eigh_solver;
  p->blocks.assign(blocks, blocks + n_blocks);
  p->grads.assign(n_blocks, nullptr);
  for (auto& bf : p->block_factor) bf.assign(n_blocks, -1);
  p->elem_off.resize(n_blocks);
  p->chunk_begin_all.resize(n_blocks + 1);
  p->ptile_begin_all.resize(n_blocks + 1);
  long long eo = 0, dense = 0, normp = 0;
  int chunks = 0, ptiles = 0;
  for (int b = 0; b < n_blocks; ++b) {
    const sa_block_desc& d = blocks[b];
    if (d.rows <= 0 || d.cols <= 0 || !d.param || d.ld < d.cols) {
      delete p;
      return fail(SA_ERR_INVALID, "sa_plan_create: block " + std::to_string(b) + " has a bad shape, stride or NULL param");
    }
    if ((long long)d.rows * d.cols >= (1LL << 31)) {
      delete p;
      return fail(SA_ERR_UNSUPPORTED, "sa_plan_create: block with 2^31 or more elements");
    }
    if (d.mid < 0 || (d.mid > 0 && (d.rows % d.mid != 0 || d.ld_outer < (long long)d.mid * d.ld))) {
      delete p;
      return fail(SA_ERR_INVALID, "sa_plan_create: block " + std::to_string(b) + " has a bad order-3 shape (mid, ld_outer)");
    }
    if (d.mid == 0 && (d.factor[2] || d.eigenvectors[2])) {
      delete p;
      return fail(SA_ERR_INVALID, "sa_plan_create: a third factor needs an order-3 block (mid > 0)");
    }
    if (d.mid > 0) p->has_order3 = true;
    p->elem_off[b] = eo;
    eo += round_up((long long)d.rows * d.cols, 64);
    p->chunk_begin_all[b] = chunks;
    chunks += (int)(((long long)d.rows * d.cols + EW_CHUNK - 1) / EW_CHUNK);
    p->ptile_begin_all[b] = ptiles;
    {
      auto tiles = [](long long m, long long n) { return (int)(((m + BM - 1) / BM) * ((n + BN - 1) / BN)); };
      int need = tiles(d.rows, d.cols);
      if (d.mid > 0) {  // the last mode product of an order-3 block may be any of the three
        const int d0 = d.rows / d.mid;
        need = std::max(need, std::max(d0 * tiles(d.mid, d.cols), tiles(d0, (long long)d.mid * d.cols)));
      }
      ptiles += need;
    }
    for (int side = 0; side < SA_MAX_ORDER; ++side) {
      if (!d.factor[side]) {
        if (d.eigenvectors[side] && d.corrected_eigenvalues) { p->eigenvalue_corrected = true; p->has_eigvec = true; }  // fixed basis
        continue;
      }
      if ((!d.inv_factor[side] && !d.eigenvectors[side]) || (d.inv_factor[side] && d.root[side] < 1)) {
        delete p;
        return fail(SA_ERR_INVALID, "sa_plan_create: factor without inverse / eigenvector storage or with root < 1");
      }
      if (d.eigenvectors[side] && !d.corrected_eigenvalues && !d.inv_factor[side]) {
        delete p;
        return fail(SA_ERR_INVALID, "sa_plan_create: eigenvectors need corrected_eigenvalues (eigenvalue-corrected Shampoo) or "
                                    "an inverse root (eigendecomposed Shampoo)");
      }
      if (d.eigenvectors[side] && d.corrected_eigenvalues && d.inv_factor[side]) {
        delete p;
        return fail(SA_ERR_INVALID, "sa_plan_create: a factor has either corrected_eigenvalues or an inverse root, not both");
      }
      Factor f{};
      f.block = b; f.side = side;
      if (d.mid > 0) f.d = side == 0 ? d.rows / d.mid : (side == 1 ? d.mid : d.cols);
      else f.d = side == 0 ? d.rows : d.cols;
      f.dpad = (int)round_up(f.d, BM);
      f.root = d.root[side];
      f.factor = d.factor[side];
      f.inv = d.inv_factor[side];
      f.eigvec = d.eigenvectors[side];
      f.dense_off = dense;
      dense += (long long)f.dpad * f.dpad;
      f.eig_off = p->eig_total;
      p->eig_total += f.dpad;
      f.norm_off = normp;
      f.norm_chunks = (int)(((long long)f.d * (f.d + 1) / 2 + NORM_CHUNK - 1) / NORM_CHUNK);
      normp += f.norm_chunks;
      if (f.eigvec) p->has_eigvec = true;
      if (f.eigvec && d.corrected_eigenvalues) p->eigenvalue_corrected = true;
      p->block_factor[side][b] = (int)p->factors.size();
      p->factors.push_back(f);
    }
  }
  p->chunk_begin_all[n_blocks] = chunks;
  p->ptile_begin_all[n_blocks] = ptiles;
  p->total_elems = eo;
  p->dense_total = dense;
  p->norm_partials_total = normp;
  p->total_chunks_all = chunks;
  p->total_ptiles_all = ptiles;
  compute_layout(p);
  const size_t F = std::max<size_t>(p->factors.size(), 1);
  auto dm = [&](void** q, size_t bytes) { return hipMalloc(q, bytes); };
  // what a root-inverse call reports lies in one allocation, in the order the host reads it, so that one copy brings it
  // back: iteration counts, final errors, non-finite flags of the inputs and of the results, position of the first bad factor
  if (dm((void**)&p->d_err, F * 4) != hipSuccess || dm((void**)&p->d_active, F * 4) != hipSuccess ||
      dm((void**)&p->d_report, (4 * F + 16) * 4) != hipSuccess || dm((void**)&p->d_final_parity, F * 4) != hipSuccess ||
      dm((void**)&p->d_nactive, 64) != hipSuccess || dm((void**)&p->d_scale, F * 4) != hipSuccess ||
      dm((void**)&p->d_ho, F * 16) != hipSuccess || dm((void**)&p->d_kept_err, F * 4) != hipSuccess ||
      dm((void**)&p->d_hoflag, F * 4) != hipSuccess ||
      hipHostMalloc((void**)&p->h_pinned, (6 * F + 16) * sizeof(int), hipHostMallocDefault) != hipSuccess ||
      hipHostMalloc((void**)&p->h_mailbox, 64, hipHostMallocMapped) != hipSuccess ||
      hipHostGetDevicePointer((void**)&p->d_mailbox, p->h_mailbox, 0) != hipSuccess) {
    sa_plan_destroy(p);
    return fail(SA_ERR_HIP, "sa_plan_create: device allocation of control arrays failed");
  }
  p->d_iters = p->d_report;
  p->d_final_err = reinterpret_cast<float*>(p->d_report + F);
  p->d_flags_in = p->d_report + 2 * F;
  p->d_flags = p->d_report + 3 * F;
  p->d_first_bad = p->d_report + 4 * F;
  std::memset(p->h_mailbox, 0, 64);
  *plan_out = p;
  return SA_OK;
}

void sa_plan_destroy(sa_plan* p) {
  if (!p) return;
  p->t_blocks.destroy(); p->t_chunks.destroy(); p->t_active_blocks.destroy();
  for (GemmTable* g : {&p->kl_right, &p->kl_left}) g->t.destroy();
  for (GemmTable* g : {&p->syrk0, &p->syrk1, &p->syrk0e, &p->syrk1e, &p->g1_store, &p->g1_norm, &p->g2_norm, &p->g2g_norm, &p->nt_a[0][0], &p->nt_a0[0], &p->nt_a0[1],
                       &p->nt_a[0][1], &p->nt_m[0][0], &p->nt_m[0][1], &p->nt_a[1][0], &p->nt_a[1][1], &p->nt_m[1][0],
                       &p->nt_m[1][1]})
    g->destroy();
  for (auto& row : p->nt_pow) for (auto& g : row) g.destroy();
  for (auto& row : p->nlane2.a) for (auto& g : row) g.destroy();
  for (auto& row : p->nlane2.pow) for (auto& g : row) g.destroy();
  for (auto& row : p->nlane2.m) for (auto& g : row) g.destroy();
  for (auto& g : p->nlane2.a0) g.destroy();
  p->nlane2.ids.destroy(); p->nlane2.sym.destroy();
  if (p->newton_stream) (void)hipStreamDestroy(p->newton_stream);
  for (hipEvent_t e : p->newton_ev) if (e) (void)hipEventDestroy(e);
  for (auto& g : p->nt_h) g.t.destroy();
  for (auto& a : p->g3) for (auto& b2 : a) for (auto& g : b2) g.t.destroy();
  for (auto& a : p->e3) for (auto& b2 : a) for (auto& c2 : b2) for (auto& g : c2) g.t.destroy();
  p->t_all_chunks.destroy();
  p->t_f64.destroy(); p->t_eig64.destroy(); p->t_tr64.destroy(); p->t_cast.destroy();
  for (auto* g : {&p->n64_a[0], &p->n64_a[1], &p->n64_m[0], &p->n64_m[1], &p->n64_a0}) g->t.destroy();
  for (auto& g : p->n64_pow) g.t.destroy();
  if (p->d_norm64) (void)hipFree(p->d_norm64);
  p->t_ho.destroy();
  p->t_sym.destroy(); p->t_normjobs.destroy(); p->t_ids.destroy();
  p->t_jacobi.destroy(); p->t_sched.destroy(); p->t_eiginit.destroy(); p->t_eigfinal.destroy(); p->eig_gemm.t.destroy();
  if (p->trd_stream) { (void)hipStreamSynchronize(p->trd_stream); (void)hipStreamDestroy(p->trd_stream); }
  for (hipStream_t q : p->trd_lane_stream) if (q) { (void)hipStreamSynchronize(q); (void)hipStreamDestroy(q); }
  for (hipEvent_t e : p->trd_lane_ev) if (e) (void)hipEventDestroy(e);
  for (hipEvent_t e : p->trd_ev) if (e) (void)hipEventDestroy(e);
  p->t_dense_state[0].destroy(); p->t_dense_state[1].destroy();
  p->t_ids_out.destroy(); p->t_normjobs_out.destroy(); p->t_sym_out.destroy();
  p->t_trd.destroy(); p->t_trd_ql.destroy(); p->t_transpose.destroy(); p->t_trd_gemm.destroy(); p->t_rowscale.destroy(); p->eig_gemm_t.t.destroy(); p->t_rank.destroy(); p->t_rows2cols.destroy();
  for (GemmTable* g : {&p->ec_stat1, &p->ec_stat2, &p->ec_stat_l, &p->ec_stat_r, &p->ec_p1, &p->ec_p1d, &p->ec_p2, &p->ec_p2d,
                       &p->ec_p3, &p->ec_p3n, &p->ec_p4, &p->ec_p4n, &p->qr_aq, &p->qr_b})
    g->t.destroy();
  for (auto& r : p->qr_in) { r->panel.destroy(); for (auto& g : r->upd) g.t.destroy(); for (auto& g : r->merge) g.t.destroy(); }
  for (auto& a : p->qr_outer) for (auto& g : a->g) g.t.destroy();
  p->t_copy.destroy(); p->t_normpair.destroy(); p->t_sort.destroy();
  for (void* q : {(void*)p->d_err, (void*)p->d_active, (void*)p->d_report, (void*)p->d_final_parity, (void*)p->d_nactive,
                  (void*)p->d_scale, (void*)p->d_ho, (void*)p->d_kept_err, (void*)p->d_hoflag})
    if (q) (void)hipFree(q);
  if (p->h_pinned) (void)hipHostFree(p->h_pinned);
  if (p->h_mailbox) (void)hipHostFree(p->h_mailbox);
  delete p;
}

int64_t sa_plan_workspace_bytes(const sa_plan* p) { return p ? p->ws_needed : 0; }

int32_t sa_plan_bind_workspace(sa_plan* p, void* workspace, int64_t bytes) {
  if (!p || !workspace) return fail(SA_ERR_INVALID, "sa_plan_bind_workspace: NULL argument");
  if (bytes < p->ws_needed) return fail(SA_ERR_WORKSPACE, "workspace too small: need " + std::to_string(p->ws_needed) + " bytes");
  if (reinterpret_cast<uintptr_t>(workspace) & 255) return fail(SA_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  p->ws = static_cast<char*>(workspace);
  p->ws_bytes = bytes;
  p->inv_cache_valid = false;
  p->tables_valid = false;
  p->rotm_version = -1;
  return SA_OK;
}

int32_t sa_plan_num_factors(const sa_plan* p) { return p ? (int32_t)p->factors.size() : 0; }

int64_t sa_plan_shared_rotation_steps(const sa_plan* p) { return p ? p->shared_rotation_steps : 0; }

int32_t sa_plan_set_tridiagonal_lanes(sa_plan* p, int32_t lanes) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  if (lanes < 1 || lanes > 4) return fail(SA_ERR_INVALID, "sa_plan_set_tridiagonal_lanes: 1 to 4 lanes");
  p->trd_lanes = lanes;
  return SA_OK;
}

int32_t sa_plan_set_newton_split_tiles(sa_plan* p, int32_t tiles) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  if (tiles < 0) return fail(SA_ERR_INVALID, "sa_plan_set_newton_split_tiles: the tile count must not be negative");
  p->newton_split_tiles = tiles;
  return SA_OK;
}

int32_t sa_plan_invalidate_inverse_cache(sa_plan* p) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  p->inv_cache_valid = false;
  p->rotm_version = -1;
  return SA_OK;
}

int32_t sa_plan_bind_gradients(sa_plan* p, float* const* grads, void* stream) {
  if (!p || !grads) return fail(SA_ERR_INVALID, "sa_plan_bind_gradients: NULL argument");
  (void)stream;
  bool changed = !p->grads_bound;
  for (int b = 0; b < p->n_blocks; ++b) {
    if (p->grads[b] != grads[b]) { p->grads[b] = grads[b]; changed = true; }
  }
  p->grads_bound = true;
  if (changed) p->tables_valid = false;
  return SA_OK;
}

int32_t sa_add_l2_regularization(sa_plan* p, float weight_decay, void* stream) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, nullptr, s));
  if (p->t_chunks.n == 0) return SA_OK;
  hipLaunchKernelGGL(l2_kernel, dim3((unsigned)p->t_chunks.n), dim3(EW_THREADS), 0, s, p->t_blocks.dev, p->t_chunks.dev, weight_decay);
  HIPCHECK(hipGetLastError());
  return SA_OK;
}

static int update_factor_matrices(sa_plan* p, double beta2, double weighting_factor, hipStream_t s);

int32_t sa_update_factor_matrices(sa_plan* p, float beta2, float weighting_factor, void* stream) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  if (p->factor_f64) return fail(SA_ERR_STATE, "the factor matrices of this plan are fp64: use sa_update_factor_matrices_f64");
  return update_factor_matrices(p, beta2, weighting_factor, static_cast<hipStream_t>(stream));
}

int32_t sa_update_factor_matrices_f64(sa_plan* p, double beta2, double weighting_factor, void* stream) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  if (!p->factor_f64) return fail(SA_ERR_STATE, "the factor matrices of this plan are fp32: use sa_update_factor_matrices");
  return update_factor_matrices(p, beta2, weighting_factor, static_cast<hipStream_t>(stream));
}

static int update_factor_matrices(sa_plan* p, double beta2, double weighting_factor, hipStream_t s) {
  SACHECK(ensure_tables(p, nullptr, s));
  GemmScalars sc = unit_scalars();
  sc.alpha = (float)weighting_factor;
  sc.beta = (float)beta2;
  sc.alpha64 = weighting_factor;
  sc.beta64 = beta2;
  double flops = 0.0;
  for (const GemmTable* g : {&p->syrk0, &p->syrk1, &p->syrk0e, &p->syrk1e})
    for (const GemmProblem& q : g->build) flops += (double)q.N * q.N * q.K;  // symmetric half: d^2 k
  int launches = (p->syrk0.total_tiles ? 1 : 0) + (p->syrk1.total_tiles ? 1 : 0) + (p->syrk0e.total_tiles ? 1 : 0) + (p->syrk1e.total_tiles ? 1 : 0);
  if (p->has_order3 && p->t_chunks.n) {
    hipLaunchKernelGGL(gather3_kernel, dim3((unsigned)p->t_chunks.n), dim3(EW_THREADS), 0, s, p->t_blocks.dev, p->t_chunks.dev, 0);
    HIPCHECK(hipGetLastError());
  }
  if (p->kl && (p->kl_right.total_tiles || p->kl_left.total_tiles)) {
    SACHECK(refresh_inverse_cache(p, s));
    SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_STORE>(p->kl_right, unit_scalars(), s)));
    SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_STORE>(p->kl_left, unit_scalars(), s)));
  }
  Span span("syrk", s, flops, launches, true);
  if (p->factor_f64) {
    SACHECK((launch_gemm_auto<A_MK, B_NK, EPI_SYRK_EMA64>(p->syrk0, sc, s)));
    SACHECK((launch_gemm_auto<A_KM, B_KN, EPI_SYRK_EMA64>(p->syrk1, sc, s)));
    SACHECK((launch_gemm_auto<A_MK, B_NK, EPI_SYRK_EMA64>(p->syrk0e, sc, s)));
    SACHECK((launch_gemm_auto<A_KM, B_KN, EPI_SYRK_EMA64>(p->syrk1e, sc, s)));
  } else {
    SACHECK((launch_gemm_auto_small<A_MK, B_NK, EPI_SYRK_EMA>(p->syrk0, sc, s)));
    SACHECK((launch_gemm_auto_small<A_KM, B_KN, EPI_SYRK_EMA>(p->syrk1, sc, s)));
    SACHECK((launch_gemm_auto<A_MK, B_NK, EPI_SYRK_EMA>(p->syrk0e, sc, s)));
    SACHECK((launch_gemm_auto<A_KM, B_KN, EPI_SYRK_EMA>(p->syrk1e, sc, s)));
  }
  return SA_OK;
}

int32_t sa_update_grafting_and_filtered_grad(sa_plan* p, const sa_step_scalars* sc, void* stream) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  SACHECK(validate_scalars(p, sc));
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, sc, s));
  if (p->t_chunks.n == 0) return SA_OK;
  double bytes = 0.0;
  for (int b = 0; b < p->n_blocks; ++b)
    if (block_active(p, b)) {
      const sa_block_desc& d = p->blocks[b];
      const double n = (double)d.rows * d.cols;
      bytes += 4.0 * n * (1 + (d.filtered_grad && sc->beta1 != 0.0f ? 2 : 0) + (d.adagrad && sc->graft_type == SA_GRAFT_ADAGRAD ? 2 : 0));
    }
  Span span("grafting", s, bytes, 1, true);
  hipLaunchKernelGGL((grafting_kernel<0>), dim3((unsigned)p->t_chunks.n), dim3(EW_THREADS), 0, s, p->t_blocks.dev,
                     p->t_chunks.dev, *sc, p->f(p->off_graft_partial), p->f(p->off_ghat_partial));
  HIPCHECK(hipGetLastError());
  ++p->m_version;
  return SA_OK;
}

int32_t sa_grafting_only_step(sa_plan* p, const sa_step_scalars* sc, void* stream) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  SACHECK(validate_scalars(p, sc));
  if (sc->graft_type == SA_GRAFT_NONE) return fail(SA_ERR_INVALID, "sa_grafting_only_step needs a grafting method");
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, sc, s));
  if (p->t_chunks.n == 0) return SA_OK;
  hipLaunchKernelGGL((grafting_kernel<1>), dim3((unsigned)p->t_chunks.n), dim3(EW_THREADS), 0, s, p->t_blocks.dev,
                     p->t_chunks.dev, *sc, p->f(p->off_graft_partial), p->f(p->off_ghat_partial));
  HIPCHECK(hipGetLastError());
  ++p->m_version;
  return SA_OK;
}

int32_t sa_precondition(sa_plan* p, const sa_step_scalars* sc, void* stream) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  SACHECK(validate_scalars(p, sc));
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, sc, s));
  SACHECK(refresh_inverse_cache(p, s));
  double flops = 0.0;
  int launches = 0;
  for (const GemmTable* g : {&p->g1_store, &p->g1_norm, &p->g2_norm, &p->g2g_norm}) {
    for (const GemmProblem& q : g->build) flops += 2.0 * q.M * q.N * q.K;
    launches += g->total_tiles ? 1 : 0;
  }
  for (auto& a : p->g3) for (auto& b2 : a) for (auto& g : b2) {
    for (const GemmProblem& q : g.build) flops += 2.0 * q.M * q.N * q.K;
    launches += g.total_tiles ? 1 : 0;
  }
  if (p->has_order3 && p->table_mode == 0 && p->t_chunks.n) {
    hipLaunchKernelGGL(gather3_kernel, dim3((unsigned)p->t_chunks.n), dim3(EW_THREADS), 0, s, p->t_blocks.dev, p->t_chunks.dev, 1);
    HIPCHECK(hipGetLastError());
  }
  {
    Span span("precondition_gemm", s, flops, launches, true);
    GemmScalars a = unit_scalars();
    a.b_div = sc->bias_correction1;
    // the left factor is the mirrored inverse root: exactly symmetric, so it is read through its transpose, whose
    // slabs load and store as 16-byte rows (same values, same results)
    SACHECK((launch_gemm_auto_small<A_KM, B_KN, EPI_STORE>(p->g1_store, a, s)));
    SACHECK((launch_gemm_auto<A_KM, B_KN, EPI_STORE_SQNORM>(p->g1_norm, a, s)));
    SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_STORE_SQNORM>(p->g2_norm, unit_scalars(), s)));
    GemmScalars c = unit_scalars();
    c.a_div = sc->bias_correction1;
    SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_STORE_SQNORM>(p->g2g_norm, c, s)));
    // order-3 blocks: mode 1, mode 0, mode 2; the stage that reads the filtered gradient divides it
    for (int kind = 0; kind < 3; ++kind)
      for (int first = 0; first < 2; ++first) {
        GemmScalars g = unit_scalars();
        if (first) (kind == 2 ? g.a_div : g.b_div) = sc->bias_correction1;
        SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_STORE>(p->g3[kind][first][0], g, s)));
        SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_STORE_SQNORM>(p->g3[kind][first][1], g, s)));
      }
  }
  if (p->n_active_blocks) {
    hipLaunchKernelGGL(reduce_norms_kernel, dim3(p->n_active_blocks), dim3(EW_THREADS), 0, s, p->t_blocks.dev,
                       p->t_active_blocks.dev, p->n_blocks, p->f(p->off_graft_partial), p->f(p->off_ghat_partial),
                       p->f(p->off_ptile_partial), p->f(p->off_norms));
    HIPCHECK(hipGetLastError());
  }
  return SA_OK;
}

int32_t sa_apply_update(sa_plan* p, const sa_step_scalars* sc, void* stream) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  SACHECK(validate_scalars(p, sc));
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, sc, s));
  if (p->t_chunks.n == 0) return SA_OK;
  double bytes = 0.0;
  for (int b = 0; b < p->n_blocks; ++b)
    if (block_active(p, b)) {
      const sa_block_desc& d = p->blocks[b];
      bytes += 4.0 * (double)d.rows * d.cols *
               (3 + ((d.momentum_buffer && sc->momentum != 0.0f) || (d.weight_buffer && sc->use_primal_averaging) ? 2 : 0));
    }
  Span span("apply", s, bytes, 1, true);
  hipLaunchKernelGGL(apply_kernel, dim3((unsigned)p->t_chunks.n), dim3(EW_THREADS), 0, s, p->t_blocks.dev,
                     p->t_chunks.dev, *sc, p->n_blocks, p->f(p->off_norms));
  HIPCHECK(hipGetLastError());
  return SA_OK;
}

int32_t sa_move_params_towards_weight_buffer(sa_plan* p, float coeff, void* stream) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // the block table must exist; gradients need not be bound for this call
  if (!p->tables_valid) {
    if (!p->grads_bound) { p->grads.assign(p->n_blocks, nullptr); }
    SACHECK(rebuild_tables(p, p->table_mode < 0 ? 0 : p->table_mode, s));
    p->tables_valid = p->grads_bound;
  }
  std::vector<ChunkRef> chunks;
  for (int b = 0; b < p->n_blocks; ++b) {
    const sa_block_desc& d = p->blocks[b];
    if (!d.weight_buffer) continue;
    const long long n_el = (long long)d.rows * d.cols;
    for (long long e = 0; e < n_el; e += EW_CHUNK) chunks.push_back(ChunkRef{b, (int)e});
  }
  if (chunks.empty()) return SA_OK;
  SACHECK(p->t_all_chunks.begin(chunks.size()));
  std::memcpy(p->t_all_chunks.host, chunks.data(), chunks.size() * sizeof(ChunkRef));
  SACHECK(p->t_all_chunks.upload(s));
  hipLaunchKernelGGL(move_params_kernel, dim3((unsigned)chunks.size()), dim3(EW_THREADS), 0, s, p->t_blocks.dev, p->t_all_chunks.dev, coeff);
  HIPCHECK(hipGetLastError());
  return SA_OK;
}

int32_t sa_plan_read_eigenvalues(sa_plan* p, int32_t factor, float* out, void* stream) {
  if (!p || !out) return fail(SA_ERR_INVALID, "sa_plan_read_eigenvalues: NULL argument");
  if (factor < 0 || factor >= (int)p->factors.size()) return fail(SA_ERR_INVALID, "sa_plan_read_eigenvalues: factor out of range");
  if ((int)p->eig_source.size() != (int)p->factors.size() || !p->eig_source[factor].base)
    return fail(SA_ERR_STATE, "sa_plan_read_eigenvalues: the last call on this plan did not refresh this factor's eigenbasis");
  const sa_plan::EigSource& e = p->eig_source[factor];
  const int d = p->factors[factor].d;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(gather_strided_kernel, dim3((d + 255) / 256), dim3(256), 0, s, e.base, e.stride, e.order, out, d);
  HIPCHECK(hipGetLastError());
  return SA_OK;
}

int32_t sa_plan_read_norms(sa_plan* p, float* graft_sq, float* precond_sq, void* stream) {
  if (!p || !graft_sq || !precond_sq) return fail(SA_ERR_INVALID, "NULL argument");
  SACHECK(need_ws(p));
  hipStream_t s = static_cast<hipStream_t>(stream);
  std::vector<float> tmp(2 * p->n_blocks);
  HIPCHECK(hipMemcpyAsync(tmp.data(), p->f(p->off_norms), tmp.size() * sizeof(float), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipStreamSynchronize(s));
  std::memcpy(graft_sq, tmp.data(), p->n_blocks * sizeof(float));
  std::memcpy(precond_sq, tmp.data() + p->n_blocks, p->n_blocks * sizeof(float));
  return SA_OK;
}

int32_t sa_plan_read_preconditioned(sa_plan* p, int32_t block, float* out, void* stream) {
  if (!p || !out || block < 0 || block >= p->n_blocks) return fail(SA_ERR_INVALID, "bad argument");
  SACHECK(need_ws(p));
  if (!p->tables_valid) return fail(SA_ERR_STATE, "no step has run");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const BlockDev& B = p->t_blocks.host[block];
  hipLaunchKernelGGL(copy_strided_kernel, dim3(256), dim3(256), 0, s, B.p_src, B.p_ld, out, B.rows, B.cols);
  HIPCHECK(hipGetLastError());
  return SA_OK;
}

// --------------------------------------------------------------------------------------------
// Batched coupled inverse Newton
// --------------------------------------------------------------------------------------------

// Products that raise a matrix to the power `root` by left-to-right binary exponentiation: after the leading bit,
// every lower bit is a squaring ('S'), followed by a product with the base ('M') when the bit is set.
// The first squaring shares a launch with X M_p; at most four further products fit the per-iteration tables.
static int power_ops(int root, std::vector<char>* ops) {
  ops->clear();
  if (root < 1) return fail(SA_ERR_INVALID, "root must be positive");
  int top = 0;
  while ((root >> (top + 1)) != 0) ++top;
  for (int bit = top - 1; bit >= 0; --bit) {
    ops->push_back('S');
    if ((root >> bit) & 1) ops->push_back('M');
  }
  if (ops->size() > 5) return fail(SA_ERR_UNSUPPORTED, "root " + std::to_string(root) + " needs too many products for the power chain");
  return SA_OK;
}

// Waits, without synchronising the stream, until the control pass with sequence number `seq` (or a later one) has
// reported into the plan's mailbox; *n_active = the count it reported.  The stream is queried now and then so that a
// failed launch or a lost report ends the wait with an error instead of a hang.
static int wait_for_control(sa_plan* p, unsigned int seq, hipStream_t s, int* n_active, int lane = 0) {
  volatile unsigned long long* box = p->h_mailbox + 4 * lane;
  const auto t0 = std::chrono::steady_clock::now();
  for (unsigned long long spin = 0;; ++spin) {
    const unsigned long long v = *box;
    if ((unsigned int)(v >> 32) >= seq) { *n_active = (int)(unsigned int)(v & 0xffffffffull); return SA_OK; }
    if ((spin & 0x3fff) == 0x3fff) {
      const hipError_t q = hipStreamQuery(s);
      if (q == hipSuccess) {
        const unsigned long long w = *box;
        if ((unsigned int)(w >> 32) >= seq) { *n_active = (int)(unsigned int)(w & 0xffffffffull); return SA_OK; }
        return fail(SA_ERR_HIP, "coupled iteration: the stream is idle but the control pass did not report");
      }
      if (q != hipErrorNotReady) return fail(SA_ERR_HIP, std::string("coupled iteration: ") + hipGetErrorString(q));
      if (std::chrono::steady_clock::now() - t0 > std::chrono::seconds(120))
        return fail(SA_ERR_HIP, "coupled iteration: no report from the control pass within 120 s");
    }
  }
}

// One batch of coupled Newton iterations (all factors of one root, or one half of them) as a resumable run:
// start() enqueues the start matrices and uploads the tables, every step() enqueues one iteration.  `symmetric[i]`
// selects the product variant of ids[i].  The loop is enqueued ahead of the device: the control pass after every
// iteration decides on the device which factors go on (the products skip the others), and the host only follows its
// reports, `lag` iterations behind, to stop enqueueing once no factor is active.  Nothing is read back here; iteration
// counts, final errors and parities stay in the plan's device arrays.  Lane 0 uses the plan's own tables, mailbox word
// and the caller's stream; lane 1 the second set, for a half that iterates beside lane 0 on the plan's second stream.
struct NewtonRun {
  sa_plan* p = nullptr;
  std::vector<int> ids;
  std::vector<char> symmetric;
  int root = 0, max_iter = 0, lane = 0;
  float eps = 0.f, bc2 = 1.f, tol = 0.f;
  hipStream_t s = nullptr;
  // state
  int n = 0, parity = 0, lag = 1, expected = 0, it = 0;
  unsigned int seq0 = 0;
  bool done = false;
  bool spans = true;  // record one timing span per iteration (off when two lanes overlap: their spans would add up twice)
  float alpha = 0.f, one_minus_alpha = 0.f;
  std::vector<char> ops;
  // per product variant: (iterations of the factor's previous solve, its large tiles per product), and the tiles' sum
  std::vector<std::pair<int, long long>> previous[2];
  long long previous_tiles[2] = {0, 0};

  GemmTable (&nt_a())[2][2] { return lane ? p->nlane2.a : p->nt_a; }
  GemmTable (&nt_pow())[2][8] { return lane ? p->nlane2.pow : p->nt_pow; }
  GemmTable (&nt_m())[2][2] { return lane ? p->nlane2.m : p->nt_m; }
  GemmTable (&nt_a0())[2] { return lane ? p->nlane2.a0 : p->nt_a0; }
  Table<int>& t_ids() { return lane ? p->nlane2.ids : p->t_ids; }
  Table<SymFactor>& t_sym() { return lane ? p->nlane2.sym : p->t_sym; }
  unsigned int& seq() { return lane ? p->ctl_seq2 : p->ctl_seq; }
  int* d_nactive() { return p->d_nactive + 8 * lane; }
  unsigned long long* d_mailbox() { return p->d_mailbox + 4 * lane; }
  NewtonCtl ctl() { return NewtonCtl{p->d_err, p->d_active, p->d_iters, p->d_final_parity, p->d_final_err}; }

  int start() {
    n = (int)ids.size();
    if (n == 0) { done = true; return SA_OK; }
    // torch.linalg.matrix_power(M_p, root) as a chain of products
    SACHECK(power_ops(root, &ops));
    alpha = (float)(-1.0 / root);                   // M.mul(alpha)
    one_minus_alpha = (float)(1.0 - (-1.0 / root));  // .add_(I, alpha = 1 - alpha)

    // ---- init: M0, Mp0, X0, err --------------------------------------------------------------
    SACHECK(t_ids().begin(n));
    std::memcpy(t_ids().host, ids.data(), n * sizeof(int));
    SACHECK(t_ids().upload(s));
    // the batch starts active with cleared counters; every other factor keeps its state
    hipLaunchKernelGGL(newton_activate_kernel, dim3(1), dim3(256), 0, s, ctl(), t_ids().dev, n);
    HIPCHECK(hipGetLastError());
    SACHECK(t_sym().begin(n));
    int sym_tiles = 0;
    for (int i = 0; i < n; ++i) {
      const Factor& f = p->factors[ids[i]];
      SymFactor& S = t_sym().host[i];
      std::memset(&S, 0, sizeof(S));
      S.packed_in = f.factor;
      S.scale = p->scale_of(ids[i]);
      S.dense_out[0] = newton_buf(p, NB_M0, f);
      S.dense_out[1] = newton_buf(p, NB_MP0, f);
      S.dense_out[2] = newton_buf(p, NB_X0, f);
      S.dense_out[3] = newton_buf(p, NB_X1, f);
      S.err_bits = p->d_err + ids[i];
      S.norm_partial = p->f(p->off_norm_partial) + f.norm_off;
      S.n_norm_partial = f.norm_chunks;
      S.d = f.d; S.dpad = f.dpad; S.tiles = f.dpad / ST; S.root = root; S.enabled = 1;
      S.tile_begin = sym_tiles;
      sym_tiles += S.tiles * (S.tiles + 1) / 2;
    }
    SACHECK(t_sym().upload(s));
    hipLaunchKernelGGL((sym_pass_kernel<SYM_NEWTON_INIT>), dim3(sym_tiles), dim3(256), 0, s, t_sym().dev, n, bc2, eps,
                       alpha, one_minus_alpha);
    HIPCHECK(hipGetLastError());

    // ---- GEMM tables -------------------------------------------------------------------------
    for (int v = 0; v < 2; ++v) {
      for (int par = 0; par < 2; ++par) { nt_a()[v][par].clear(); nt_m()[v][par].clear(); }
      nt_a0()[v].clear();
      for (int k = 0; k < 8; ++k) nt_pow()[v][k].clear();
    }
    auto prob = [&](const Factor& f, const float* A, const float* B, float* C) {
      GemmProblem q{};
      q.A = A; q.B = B; q.C = C;
      q.lda = q.ldb = q.ldc = f.dpad;
      q.M = q.N = q.K = f.dpad;
      q.d = f.d;
      q.a_vec = q.b_vec = 1;
      q.active = p->d_active + (&f - p->factors.data());
      return q;
    };
    for (int v = 0; v < 2; ++v) { previous[v].clear(); previous_tiles[v] = 0; }
    const bool have_history = (int)p->newton_history.size() == (int)p->factors.size();
    for (int i = 0; i < n; ++i) {
      const Factor& f = p->factors[ids[i]];
      const bool sym = symmetric[i] != 0;
      const int v = sym ? 1 : 0;
      {
        const long long t = f.dpad / BM, tiles = sym ? t * (t + 1) / 2 : t * t;
        previous[v].push_back({have_history ? p->newton_history[ids[i]] : 0, tiles});
        previous_tiles[v] += tiles;
      }
      // buffer that finally holds M_p^root (depends only on the chain length)
      const float* power = nullptr;
      for (int par = 0; par < 2; ++par) {
        const float* X = newton_buf(p, par ? NB_X1 : NB_X0, f);
        float* Xn = newton_buf(p, par ? NB_X0 : NB_X1, f);
        const float* Mp = newton_buf(p, par ? NB_MP1 : NB_MP0, f);
        float* Mpn = newton_buf(p, par ? NB_MP0 : NB_MP1, f);
        const float* M = newton_buf(p, par ? NB_M1 : NB_M0, f);
        float* Mn = newton_buf(p, par ? NB_M0 : NB_M1, f);
        float* S1 = newton_buf(p, NB_S1, f);
        float* S2 = newton_buf(p, NB_S2, f);
        // launch A: X <- X M_p, and the first squaring if the root needs one
        nt_a()[v][par].add(prob(f, X, Mp, Xn), sym);
        if (!ops.empty()) nt_a()[v][par].add(prob(f, Mp, Mp, S1), sym);
        if (!ops.empty() && par == 0) nt_a0()[v].add(prob(f, Mp, Mp, S1), sym);
        // the remaining chain reads only S1 / S2 / M_p of this parity
        const float* cur = ops.empty() ? Mp : S1;
        int slot = par * 4;  // nt_pow[0..3] parity 0, [4..7] parity 1
        float* pong[2] = {S2, S1};
        int which = 0;
        for (size_t q = 1; q < ops.size(); ++q) {
          nt_pow()[v][slot++].add(prob(f, cur, ops[q] == 'S' ? cur : Mp, pong[which]), sym);
          cur = pong[which];
          which ^= 1;
        }
        power = cur;
        GemmProblem m = prob(f, power, M, Mn);
        m.C2 = Mpn;
        m.err_bits = p->d_err + ids[i];
        nt_m()[v][par].add(m, sym);
      }
    }
    for (int v = 0; v < 2; ++v) {
      for (int par = 0; par < 2; ++par) { SACHECK(nt_a()[v][par].commit(s)); SACHECK(nt_m()[v][par].commit(s)); }
      SACHECK(nt_a0()[v].commit(s));
      for (int k = 0; k < 8; ++k) SACHECK(nt_pow()[v][k].commit(s));
    }

    parity = 0;
    seq0 = seq();
    hipLaunchKernelGGL(newton_control_kernel, dim3(1), dim3(256), 0, s, ctl(), t_ids().dev, n, tol, max_iter, parity, d_nactive(),
                       d_mailbox(), ++seq());
    HIPCHECK(hipGetLastError());
    // small batches finish an iteration faster than the host enqueues the next one: stay further ahead there (an
    // iteration enqueued after the last factor stopped costs a few launches of workgroups that exit at once)
    long long tiles_per_stage = 0;
    for (int v = 0; v < 2; ++v) tiles_per_stage += nt_m()[v][0].total_tiles;
    lag = tiles_per_stage >= 2048 ? 1 : 3;
    // Factors drift slowly between two amortized computations, so the batch most likely needs as many iterations as its
    // slowest factor took last time.  Up to that count the host runs ahead as above; from there on it waits for the
    // control pass that decides the very iteration it is about to enqueue, so that a correct guess enqueues no iteration
    // that finds nothing to do (and a short guess costs one host round trip per extra iteration).
    expected = 0;
    if ((int)p->newton_history.size() == (int)p->factors.size()) {
      for (int i : ids) {
        if (p->newton_history[i] <= 0) { expected = 0; break; }
        expected = std::max(expected, p->newton_history[i]);
      }
    }
    it = 0;
    done = false;
    return SA_OK;
  }

  // Enqueues one more iteration, or finds that the batch has finished.
  int step(int* launches_acc) {
    if (done) return SA_OK;
    if (it >= max_iter) { done = true; return SA_OK; }
    // control pass k (k = 0 is the one of start()) decides iteration k; before iteration `it` is enqueued, pass it - lag
    // must have reported, and any newer report that shows no active factor ends the loop
    int n_active = 1;
    if (expected > 0 && it >= expected) {
      SACHECK(wait_for_control(p, seq0 + 1 + (unsigned int)it, s, &n_active, lane));
    } else if (it >= lag) {
      SACHECK(wait_for_control(p, seq0 + 1 + (unsigned int)(it - lag), s, &n_active, lane));
    } else {
      const unsigned long long v = *(volatile unsigned long long*)(p->h_mailbox + 4 * lane);
      if ((unsigned int)(v >> 32) > seq0) n_active = (int)(unsigned int)(v & 0xffffffffull);
    }
    if (n_active == 0) { done = true; return SA_OK; }
    GemmScalars unit = unit_scalars();
    GemmScalars msc = unit_scalars();
    msc.mp_scale = alpha;
    msc.mp_diag = one_minus_alpha;
    {
      int nl = 0;
      for (int v = 0; v < 2; ++v) {
        nl += ((it == 0 ? nt_a0()[v] : nt_a()[v][parity]).total_tiles ? 1 : 0) + (nt_m()[v][parity].total_tiles ? 1 : 0);
        for (int k = 0; k < 4; ++k) nl += nt_pow()[v][parity * 4 + k].total_tiles ? 1 : 0;
      }
      std::unique_ptr<Span> span;
      if (spans) span.reset(new Span("newton_gemm", s, 0.0, nl, false));
      else if (g_profiling) g_phases["newton_gemm"].launches += nl;
      // Towards the end only a few factors still iterate, and their large tiles no longer reach every CU.  Which factors
      // those are is known on the device only; the host goes by the iterations every factor took in its previous solve
      // (factors drift slowly), or, once the batch has outlived that guess, by the count of the last control pass.
      bool few[2];
      for (int v = 0; v < 2; ++v) {
        long long live = 0, largest = 0;
        for (const auto& e : previous[v]) {
          if (e.first <= 0 || e.first > it) live += e.second;
          largest = std::max(largest, e.second);
        }
        if (expected > 0 && it >= expected) live = std::max(live, (long long)n_active * largest);
        // judged by the tiles of one product per factor, so the choice is the same for every stage of the iteration; the
        // bound is a little above one large tile per CU (measured: with 400 to 800 live tiles of order 2048 the small
        // tiles are the slower choice, below 320 they gain 1 % of the step on the GPT-2 parameter set)
        few[v] = previous_tiles[v] > 0 && live > 0 && live < SMALL_LAUNCH_TILES + SMALL_LAUNCH_TILES / 4;
      }
      // the two variants touch disjoint factors, so their launches of one stage are independent
      // symmetric variant: every operand is an exactly mirrored matrix, so A is read through its transpose (slabs
      // load and store as 16-byte rows instead of four scalar LDS stores per thread; same values, same results)
      SACHECK((launch_gemm_live<A_KM, B_KN, EPI_STORE, false, true>(it == 0 ? nt_a0()[1] : nt_a()[1][parity], unit, s, few[1])));
      SACHECK((launch_gemm_live<A_MK, B_KN, EPI_STORE, false, false>(it == 0 ? nt_a0()[0] : nt_a()[0][parity], unit, s, few[0])));
      for (int k = 0; k < 4; ++k) {
        SACHECK((launch_gemm_live<A_KM, B_KN, EPI_STORE, false, true>(nt_pow()[1][parity * 4 + k], unit, s, few[1])));
        SACHECK((launch_gemm_live<A_MK, B_KN, EPI_STORE, false, false>(nt_pow()[0][parity * 4 + k], unit, s, few[0])));
      }
      SACHECK((launch_gemm_live<A_KM, B_KN, EPI_NEWTON_M, false, true>(nt_m()[1][parity], msc, s, few[1])));
      SACHECK((launch_gemm_live<A_MK, B_KN, EPI_NEWTON_M, false, false>(nt_m()[0][parity], msc, s, few[0])));
      *launches_acc += nl;
    }
    parity ^= 1;
    hipLaunchKernelGGL(newton_control_kernel, dim3(1), dim3(256), 0, s, ctl(), t_ids().dev, n, tol, max_iter, parity, d_nactive(),
                       d_mailbox(), ++seq());
    HIPCHECK(hipGetLastError());
    ++it;
    return SA_OK;
  }
};

// The coupled Newton iterations of `ids` (one root).  Optionally (sa_plan_set_newton_split_tiles, off by default) a
// batch whose stages are short launches is cut into two halves that iterate side by side, the second on the plan's own
// stream: every stage of an iteration depends on the stage before it, so one half alone leaves the chip idle while a
// launch ramps up and while its last workgroups finish, and the other half's launch can fill that.  The factors are
// independent of each other, so the halves give the bits the whole batch gives.  Measured on the GPT-2 parameter set
// the halves are slower (73.8 against 69.6 ms per step: two control passes, two tile-layout passes per stage and launches
// of half the size cost more than the overlap returns), hence the default.
static int newton_batch(sa_plan* p, const std::vector<int>& ids, const std::vector<char>& symmetric, int root, float eps,
                        float bc2, int max_iter, float tol, hipStream_t s, int* launches_acc) {
  if (ids.empty()) return SA_OK;
  long long tiles = 0;
  for (size_t i = 0; i < ids.size(); ++i) {
    const long long t = p->factors[ids[i]].dpad / BM;
    tiles += symmetric[i] ? t * (t + 1) / 2 : t * t;
  }
  const bool split = p->newton_split_tiles > 0 && tiles < p->newton_split_tiles && tiles >= 512 && ids.size() >= 8;
  NewtonRun run[2];
  for (int h = 0; h < 2; ++h) {
    run[h].p = p; run[h].root = root; run[h].max_iter = max_iter; run[h].lane = h;
    run[h].eps = eps; run[h].bc2 = bc2; run[h].tol = tol; run[h].s = s; run[h].spans = !split;
  }
  if (!split) {
    run[0].ids = ids; run[0].symmetric = symmetric;
    SACHECK(run[0].start());
    while (!run[0].done) SACHECK(run[0].step(launches_acc));
    return SA_OK;
  }
  // halves of equal work: the factors in descending order of their tile count, dealt out in turn
  std::vector<int> order(ids.size());
  for (size_t i = 0; i < order.size(); ++i) order[i] = (int)i;
  std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return p->factors[ids[x]].dpad > p->factors[ids[y]].dpad; });
  for (size_t k = 0; k < order.size(); ++k) {
    run[k & 1].ids.push_back(ids[order[k]]);
    run[k & 1].symmetric.push_back(symmetric[order[k]]);
  }
  if (!p->newton_stream) HIPCHECK(hipStreamCreateWithFlags(&p->newton_stream, hipStreamNonBlocking));
  for (hipEvent_t& e : p->newton_ev)
    if (!e) HIPCHECK(hipEventCreateWithFlags(&e, hipEventDisableTiming));
  run[1].s = p->newton_stream;
  // the second stream starts behind everything the caller's stream holds so far, and the caller's stream goes on
  // behind the second stream's last iteration
  HIPCHECK(hipEventRecord(p->newton_ev[0], s));
  HIPCHECK(hipStreamWaitEvent(p->newton_stream, p->newton_ev[0], 0));
  {
    Span span("newton_gemm", s, 0.0, 0, false);  // one span over both lanes: from here to the join on the caller's stream
    SACHECK(run[0].start());
    SACHECK(run[1].start());
    while (!run[0].done || !run[1].done) {
      SACHECK(run[0].step(launches_acc));
      SACHECK(run[1].step(launches_acc));
    }
    HIPCHECK(hipEventRecord(p->newton_ev[1], p->newton_stream));
    HIPCHECK(hipStreamWaitEvent(s, p->newton_ev[1], 0));
  }
  return SA_OK;
}

// Shared front end of the root-inverse paths: which factors are to be recomputed, Frobenius norm
// partials of the ridged, bias-corrected factor, and the finiteness check of the input.  On return `todo`
// holds the factors that precede the first non-finite one (the reference raises there).
static int root_inverse_prologue(sa_plan* p, float bias_correction2, float norm_eps, int32_t* iterations_out,
                                 int32_t* status_out, hipStream_t s, std::vector<int>* todo) {
  const int F = (int)p->factors.size();
  todo->clear();
  for (int i = 0; i < F; ++i) {
    iterations_out[i] = 0;
    status_out[i] = SA_FACTOR_SKIPPED;
    if (block_active(p, p->factors[i].block) && in_wave(p, i)) todo->push_back(i);
  }
  if (todo->empty()) return SA_OK;
  // factors that are not recomputed below must keep a valid dense copy of their stored inverse
  SACHECK(refresh_inverse_cache(p, s));
  SACHECK(stage_fp32_factors(p, *todo, s));  // float64 factors: the fp32 solvers below work on the rounded copy
  HIPCHECK(hipMemsetAsync(p->d_flags, 0, F * sizeof(int), s));
  HIPCHECK(hipMemsetAsync(p->d_err, 0, F * sizeof(int), s));
  HIPCHECK(hipMemsetAsync(p->d_iters, 0, F * sizeof(int), s));
  HIPCHECK(hipMemsetAsync(p->d_active, 0, F * sizeof(int), s));
  HIPCHECK(hipMemsetAsync(p->d_final_parity, 0, F * sizeof(int), s));
  SACHECK(p->t_normjobs.begin(todo->size()));
  int chunks = 0;
  for (size_t i = 0; i < todo->size(); ++i) {
    const Factor& f = p->factors[(*todo)[i]];
    NormJob& J = p->t_normjobs.host[i];
    std::memset(&J, 0, sizeof(J));
    J.src = packed32(p, f);
    J.partial = p->f(p->off_norm_partial) + f.norm_off;
    J.scale = const_cast<float*>(p->scale_of((*todo)[i]));
    J.nonfinite = p->d_flags + (*todo)[i];
    J.d = f.d; J.dpad = f.dpad; J.dense = 0;
    J.chunk_begin = chunks;
    J.n_chunks = f.norm_chunks;
    J.enabled = 1;
    chunks += f.norm_chunks;
  }
  SACHECK(p->t_normjobs.upload(s));
  if (p->trace_scaling)
    hipLaunchKernelGGL(trace_scale_kernel, dim3((unsigned)todo->size()), dim3(256), 0, s, p->t_normjobs.dev, bias_correction2,
                       p->trace_floor, p->trace_exponent);
  hipLaunchKernelGGL((factor_norm_kernel<false>), dim3(chunks), dim3(256), 0, s, p->t_normjobs.dev, (int)todo->size(),
                     bias_correction2, norm_eps);
  HIPCHECK(hipGetLastError());
  int* h_flags = p->h_pinned + F;
  HIPCHECK(hipMemcpyAsync(h_flags, p->d_flags, F * sizeof(int), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipStreamSynchronize(s));
  size_t limit = todo->size();
  for (size_t i = 0; i < todo->size(); ++i)
    if (h_flags[(*todo)[i]]) { status_out[(*todo)[i]] = SA_FACTOR_INPUT_NONFINITE; limit = i; break; }
  todo->resize(limit);
  return SA_OK;
}

// Shared back end: finiteness of every result X (dense, dpad-strided), then pack + mirror the results that
// precede the first non-finite one into inv_factor and the dense inverse cache.
// With `failures_are_local` a non-finite result only marks its own factor SA_FACTOR_SOLVER_FAILED (the solver
// raised; the previous inverse stays) and every other result is committed; n_ok then counts nothing useful.
static int root_inverse_epilogue(sa_plan* p, const std::vector<int>& todo, const std::vector<const float*>& X,
                                 int32_t* status_out, hipStream_t s, size_t* n_ok, bool failures_are_local = false) {
  const int F = (int)p->factors.size();
  int* h_bad = p->h_pinned + 3 * F;
  HIPCHECK(hipMemsetAsync(p->d_flags, 0, F * sizeof(int), s));
  SACHECK(p->t_normjobs.begin(todo.size()));
  int chunks = 0;
  for (size_t i = 0; i < todo.size(); ++i) {
    const Factor& f = p->factors[todo[i]];
    NormJob& J = p->t_normjobs.host[i];
    std::memset(&J, 0, sizeof(J));
    J.src = X[i];
    J.partial = nullptr;
    J.nonfinite = p->d_flags + todo[i];
    J.d = f.d; J.dpad = f.dpad; J.dense = 1;
    J.chunk_begin = chunks;
    J.n_chunks = (int)(((long long)f.d * f.d + NORM_CHUNK - 1) / NORM_CHUNK);
    J.enabled = 1;
    chunks += J.n_chunks;
  }
  SACHECK(p->t_normjobs.upload(s));
  hipLaunchKernelGGL((factor_norm_kernel<true>), dim3(chunks), dim3(256), 0, s, p->t_normjobs.dev, (int)todo.size(), 1.0f, 0.0f);
  HIPCHECK(hipGetLastError());
  HIPCHECK(hipMemcpyAsync(h_bad, p->d_flags, F * sizeof(int), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipStreamSynchronize(s));
  size_t ok = todo.size();
  std::vector<size_t> keep;
  for (size_t i = 0; i < todo.size(); ++i) {
    if (h_bad[todo[i]]) {
      if (failures_are_local) { status_out[todo[i]] = SA_FACTOR_SOLVER_FAILED; continue; }
      status_out[todo[i]] = SA_FACTOR_RESULT_NONFINITE; ok = i; break;
    }
    keep.push_back(i);
  }
  *n_ok = ok;
  ok = keep.size();
  if (ok > 0) {
    SACHECK(p->t_sym.begin(ok));
    int tiles = 0;
    for (size_t k = 0; k < ok; ++k) {
      const size_t i = keep[k];
      const Factor& f = p->factors[todo[i]];
      SymFactor& S = p->t_sym.host[k];
      std::memset(&S, 0, sizeof(S));
      S.dense_in = X[i];
      S.packed_out = f.inv;
      S.dense_out[0] = p->f(p->off_inv_dense) + f.dense_off;
      S.d = f.d; S.dpad = f.dpad; S.tiles = f.dpad / ST; S.root = f.root; S.enabled = 1;
      S.tile_begin = tiles;
      tiles += S.tiles * (S.tiles + 1) / 2;
    }
    SACHECK(p->t_sym.upload(s));
    hipLaunchKernelGGL((sym_pass_kernel<SYM_COMMIT>), dim3(tiles), dim3(256), 0, s, p->t_sym.dev, (int)ok, 1.0f, 0.0f, 0.0f, 0.0f);
    HIPCHECK(hipGetLastError());
    HIPCHECK(hipStreamSynchronize(s));
  }
  return SA_OK;
}

static int sa_compute_root_inverses_newton_wave(sa_plan* p, float bias_correction2, float epsilon, int32_t max_iterations,
                                        float tolerance, int32_t* iterations_out, int32_t* status_out, void* stream) {
  if (!p || !iterations_out || !status_out) return fail(SA_ERR_INVALID, "sa_compute_root_inverses_newton: NULL argument");
  if (p->factor_f64) return fail(SA_ERR_STATE, "the factor matrices of this plan are fp64: use sa_compute_root_inverses_newton_f64");
  if (!(bias_correction2 != 0.0f) || max_iterations < 0) return fail(SA_ERR_INVALID, "bad bias correction or max_iterations");
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, nullptr, s));
  const int F = (int)p->factors.size();
  if (F == 0) return SA_OK;
  if (g_profiling) { Phase& ph = g_phases["newton_gemm"]; ph.used = 0; ph.work = 0.0; ph.executed = 0.0; ph.launches = 0; }
  std::vector<int> todo;
  for (int i = 0; i < F; ++i) {
    iterations_out[i] = 0;
    status_out[i] = SA_FACTOR_SKIPPED;
    if (block_active(p, p->factors[i].block) && in_wave(p, i)) todo.push_back(i);
  }
  if (todo.empty()) return SA_OK;
  const int n = (int)todo.size();

  // The whole call is enqueued without waiting for the device: finiteness of the inputs, the iterations, finiteness of
  // the results and the commit of every result that precedes the first non-finite factor (decided on the device, the
  // reference raises there) -- then ONE readback tells the host what happened.
  // ---- inputs: Frobenius norm partials of the ridged, bias-corrected factors and their non-finite flags ----
  SACHECK(refresh_inverse_cache(p, s));  // factors that are not recomputed must keep a valid dense copy of their stored inverse
  HIPCHECK(hipMemsetAsync(p->d_flags_in, 0, 2 * F * sizeof(int), s));  // and d_flags, which follows it
  bool result_flags_clear = true;
  SACHECK(p->t_normjobs.begin(n));
  {
    int chunks = 0;
    for (int k = 0; k < n; ++k) {
      const Factor& f = p->factors[todo[k]];
      NormJob& J = p->t_normjobs.host[k];
      std::memset(&J, 0, sizeof(J));
      J.src = f.factor;
      J.partial = p->f(p->off_norm_partial) + f.norm_off;
      J.scale = const_cast<float*>(p->scale_of(todo[k]));
      J.nonfinite = p->d_flags_in + todo[k];
      J.d = f.d; J.dpad = f.dpad; J.dense = 0;
      J.chunk_begin = chunks;
      J.n_chunks = f.norm_chunks;
      J.enabled = 1;
      chunks += f.norm_chunks;
    }
    SACHECK(p->t_normjobs.upload(s));
    if (p->trace_scaling)
      hipLaunchKernelGGL(trace_scale_kernel, dim3((unsigned)n), dim3(256), 0, s, p->t_normjobs.dev, bias_correction2,
                         p->trace_floor, p->trace_exponent);
    hipLaunchKernelGGL((factor_norm_kernel<false>), dim3(chunks), dim3(256), 0, s, p->t_normjobs.dev, n, bias_correction2, epsilon);
    HIPCHECK(hipGetLastError());
  }

  // iterate, one batch per distinct root; product variant per factor from the policy and the factor's history
  if ((int)p->newton_history.size() != F) p->newton_history.assign(F, 0);
  std::vector<char> sym(F, 0);
  for (int i : todo) {
    const int h = p->newton_history[i];
    sym[i] = p->symmetric_newton == 1 || (p->symmetric_newton == 2 && h > 0 && h <= SYM_MAX_PREVIOUS_ITERATIONS);
  }
  int launches = 0;
  auto solve = [&](const std::vector<int>& subset) -> int {
    // the subset starts active with cleared counters; every other factor is inactive and keeps its counters
    HIPCHECK(hipMemsetAsync(p->d_active, 0, F * sizeof(int), s));
    std::map<int, std::vector<int>> by_root;
    for (int i : subset) by_root[p->factors[i].root].push_back(i);
    for (auto& kv : by_root) {
      std::vector<char> variant(kv.second.size());
      for (size_t k = 0; k < kv.second.size(); ++k) variant[k] = sym[kv.second[k]];
      SACHECK(newton_batch(p, kv.second, variant, kv.first, epsilon, bias_correction2, max_iterations, tolerance, s, &launches));
    }
    return SA_OK;
  };
  // ---- results: non-finite flags of X (the buffer the factor's final parity names), the first bad factor, and the
  // commit (pack + mirror into inv_factor and the dense inverse cache) of everything in front of it ----
  auto finish = [&]() -> int {
    if (!result_flags_clear) HIPCHECK(hipMemsetAsync(p->d_flags, 0, F * sizeof(int), s));
    result_flags_clear = false;
    SACHECK(p->t_normjobs_out.begin(n));
    int chunks = 0;
    for (int k = 0; k < n; ++k) {
      const Factor& f = p->factors[todo[k]];
      NormJob& J = p->t_normjobs_out.host[k];
      std::memset(&J, 0, sizeof(J));
      J.src = newton_buf(p, NB_X0, f);
      J.src_alt = newton_buf(p, NB_X1, f);
      J.select = p->d_final_parity + todo[k];
      J.nonfinite = p->d_flags + todo[k];
      J.d = f.d; J.dpad = f.dpad; J.dense = 1;
      J.chunk_begin = chunks;
      J.n_chunks = (int)(((long long)f.d * f.d + NORM_CHUNK - 1) / NORM_CHUNK);
      J.enabled = 1;
      chunks += J.n_chunks;
    }
    SACHECK(p->t_normjobs_out.upload(s));
    hipLaunchKernelGGL((factor_norm_kernel<true>), dim3(chunks), dim3(256), 0, s, p->t_normjobs_out.dev, n, 1.0f, 0.0f);
    HIPCHECK(hipGetLastError());
    SACHECK(p->t_ids_out.begin(n));
    std::memcpy(p->t_ids_out.host, todo.data(), n * sizeof(int));
    SACHECK(p->t_ids_out.upload(s));
    hipLaunchKernelGGL(first_bad_kernel, dim3(1), dim3(256), 0, s, p->t_ids_out.dev, n, p->d_flags_in, p->d_flags, p->d_first_bad);
    HIPCHECK(hipGetLastError());
    SACHECK(p->t_sym_out.begin(n));
    int tiles = 0;
    for (int k = 0; k < n; ++k) {
      const Factor& f = p->factors[todo[k]];
      SymFactor& S = p->t_sym_out.host[k];
      std::memset(&S, 0, sizeof(S));
      S.dense_in = newton_buf(p, NB_X0, f);
      S.dense_in_alt = newton_buf(p, NB_X1, f);
      S.select = p->d_final_parity + todo[k];
      S.gate = p->d_first_bad;
      S.gate_index = k;
      S.packed_out = f.inv;
      S.dense_out[0] = p->f(p->off_inv_dense) + f.dense_off;
      S.d = f.d; S.dpad = f.dpad; S.tiles = f.dpad / ST; S.root = f.root; S.enabled = 1;
      S.tile_begin = tiles;
      tiles += S.tiles * (S.tiles + 1) / 2;
    }
    SACHECK(p->t_sym_out.upload(s));
    hipLaunchKernelGGL((sym_pass_kernel<SYM_COMMIT>), dim3(tiles), dim3(256), 0, s, p->t_sym_out.dev, n, 1.0f, 0.0f, 0.0f, 0.0f);
    HIPCHECK(hipGetLastError());
    // the one readback of the call
    int* h = p->h_pinned;
    HIPCHECK(hipMemcpyAsync(h, p->d_report, (4 * F + 1) * sizeof(int), hipMemcpyDeviceToHost, s));
    HIPCHECK(hipStreamSynchronize(s));
    return SA_OK;
  };
  std::vector<int> iters(F, 0);
  std::vector<float> errs(F, 0.0f);
  double flops = 0.0, executed = 0.0;
  auto account = [&](const std::vector<int>& subset) {
    // iteration counts and final errors of the subset just solved; algorithmic and executed flops of its products
    std::vector<char> ops;
    for (int i : subset) {
      iters[i] = p->h_pinned[i];
      std::memcpy(&errs[i], p->h_pinned + F + i, sizeof(float));
      if (iters[i] <= 0) continue;
      const Factor& f = p->factors[i];
      (void)power_ops(f.root, &ops);
      const double products = (double)iters[i] * (2.0 + (double)ops.size()) - 1.0;  // the first X M_p is not a product
      const double d = f.d, t = f.dpad / BM;
      flops += (sym[i] ? d * d * (d + 1.0) : 2.0 * d * d * d) * products;
      executed += 2.0 * BM * BN * (double)f.dpad * (sym[i] ? t * (t + 1) / 2 : t * t) * products;
    }
  };
  SACHECK(solve(todo));
  SACHECK(finish());
  account(todo);
  int first_bad = p->h_pinned[4 * F];
  if (p->symmetric_newton == 2) {
    // a factor whose conditioning worsened since its last solve gets the reference's full products after all
    std::vector<int> redo;
    for (int k = 0; k < n && k < first_bad; ++k) {
      const int i = todo[k];
      if (sym[i] && (iters[i] > SYM_REDO_ITERATIONS || !(errs[i] <= tolerance))) { redo.push_back(i); sym[i] = 0; }
    }
    if (!redo.empty()) {
      SACHECK(solve(redo));
      SACHECK(finish());
      account(redo);
      first_bad = p->h_pinned[4 * F];
    }
  }
  if (g_profiling) {
    Phase& ph = g_phases["newton_gemm"];
    ph.work += flops;
    ph.executed += executed;
  }
  const int* h_in = p->h_pinned + 2 * F;
  for (int k = 0; k < n; ++k) {
    const int i = todo[k];
    if (k < first_bad) {
      p->newton_history[i] = (errs[i] <= tolerance) ? iters[i] : 0;
      iterations_out[i] = iters[i];
      status_out[i] = (errs[i] <= tolerance) ? SA_FACTOR_OK : SA_FACTOR_NOT_CONVERGED;
    } else if (k == first_bad) {
      p->newton_history[i] = 0;
      if (h_in[i]) status_out[i] = SA_FACTOR_INPUT_NONFINITE;
      else { iterations_out[i] = iters[i]; status_out[i] = SA_FACTOR_RESULT_NONFINITE; }
    } else {
      p->newton_history[i] = 0;  // not stored: the next solve of this factor starts with full products
    }
  }
  (void)launches;
  return SA_OK;
}

int32_t sa_compute_root_inverses_newton(sa_plan* p, float bias_correction2, float epsilon, int32_t max_iterations, float tolerance, int32_t* iterations_out, int32_t* status_out, void* stream) {
  if (!p || !status_out) return fail(SA_ERR_INVALID, "sa_compute_root_inverses_newton: NULL argument");
  return for_each_wave(p, iterations_out, status_out, static_cast<hipStream_t>(stream), [&](int32_t* it__, int32_t* st__) {
    return sa_compute_root_inverses_newton_wave(p, bias_correction2, epsilon, max_iterations, tolerance, it__, st__, stream);
  });
}

// --------------------------------------------------------------------------------------------
// Factor matrices in fp64: coupled Newton in double precision (reference: the same matrix_inverse_root_newton,
// matrix_functions.py:368-437, on a torch.float64 factor; the result is cast to the fp32 inverse-root state,
// shampoo_preconditioner_list.py:672-678)
// --------------------------------------------------------------------------------------------

int32_t sa_plan_set_factor_dtype(sa_plan* p, int32_t bits) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  if (bits != 32 && bits != 64) return fail(SA_ERR_INVALID, "factor dtype must be 32 or 64 bits");
  if (p->ws) return fail(SA_ERR_STATE, "sa_plan_set_factor_dtype must be called before the workspace is bound");
  if (bits == 64) {
    if (p->kl) return fail(SA_ERR_UNSUPPORTED, "fp64 factor matrices are not built for KL-Shampoo");
    for (const Factor& f : p->factors)
      if (!f.inv && !f.eigvec) return fail(SA_ERR_STATE, "fp64 factor matrices need inverse-root or eigenvector storage");
    if (!p->d_norm64 && !p->factors.empty())
      HIPCHECK(hipMalloc(reinterpret_cast<void**>(&p->d_norm64), p->factors.size() * sizeof(double)));
  }
  p->factor_f64 = bits == 64;
  compute_layout(p);
  return SA_OK;
}

int32_t sa_plan_set_scratch_budget(sa_plan* p, int64_t bytes) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  if (bytes < 0) return fail(SA_ERR_INVALID, "sa_plan_set_scratch_budget: negative budget");
  if (p->ws) return fail(SA_ERR_STATE, "sa_plan_set_scratch_budget must be called before the workspace is bound");
  p->scratch_budget_bytes = bytes;
  compute_layout(p);
  return SA_OK;
}

int32_t sa_plan_num_waves(const sa_plan* p) { return p ? (int32_t)p->wave_dense.size() : 0; }

static inline double* newton_buf64(const sa_plan* p, int k, const Factor& F) {
  return reinterpret_cast<double*>(p->f(p->off_scratch)) + (long long)k * p->wave_dense[F.wave] + F.wave_off;
}

static int commit64(sa_plan::GemmTable64& g, hipStream_t s) {
  SACHECK(g.t.begin(g.build.size()));
  if (!g.build.empty()) std::memcpy(g.t.host, g.build.data(), g.build.size() * sizeof(GemmProblem64));
  return g.t.upload(s);
}

static int newton_batch64(sa_plan* p, const std::vector<int>& ids, int root, const std::vector<double>& ridge, double bc2,
                          int max_iter, float tol, hipStream_t s) {
  const int n = (int)ids.size();
  if (n == 0) return SA_OK;
  std::vector<char> ops;
  SACHECK(power_ops(root, &ops));
  const double alpha = -1.0 / root, one_minus_alpha = 1.0 - alpha;
  SACHECK(p->t_ids.begin(n));
  std::memcpy(p->t_ids.host, ids.data(), n * sizeof(int));
  SACHECK(p->t_ids.upload(s));
  SACHECK(p->t_f64.begin(n));
  int nmax = 0;
  for (int i = 0; i < n; ++i) {
    const Factor& f = p->factors[ids[i]];
    Factor64& J = p->t_f64.host[i];
    std::memset(&J, 0, sizeof(J));
    J.packed = reinterpret_cast<const double*>(f.factor);
    J.M = newton_buf64(p, NB_M0, f); J.Mp = newton_buf64(p, NB_MP0, f); J.X = newton_buf64(p, NB_X0, f);
    J.X1 = newton_buf64(p, NB_X1, f);
    J.norm_sq = p->d_norm64 + ids[i];
    J.nonfinite = p->d_flags + ids[i];
    J.ridge = ridge[ids[i]];
    J.d = f.d; J.n = f.dpad;
    nmax = std::max(nmax, f.dpad);
  }
  SACHECK(p->t_f64.upload(s));
  const unsigned gx = (unsigned)std::min<long long>(((long long)nmax * nmax + 255) / 256, 2048);
  hipLaunchKernelGGL(f64_newton_start_kernel, dim3(gx, n), dim3(256), 0, s, p->t_f64.dev, bc2, root, alpha, one_minus_alpha);
  HIPCHECK(hipGetLastError());

  for (int par = 0; par < 2; ++par) { p->n64_a[par].clear(); p->n64_m[par].clear(); }
  p->n64_a0.clear();
  for (auto& g : p->n64_pow) g.clear();
  auto prob = [&](const Factor& f, const double* A, const double* B, double* C) {
    GemmProblem64 q{};
    q.A = A; q.B = B; q.C = C;
    q.n = f.dpad; q.d = f.d;
    q.active = p->d_active + (&f - p->factors.data());
    return q;
  };
  for (int i = 0; i < n; ++i) {
    const Factor& f = p->factors[ids[i]];
    for (int par = 0; par < 2; ++par) {
      const double* X = newton_buf64(p, par ? NB_X1 : NB_X0, f);
      double* Xn = newton_buf64(p, par ? NB_X0 : NB_X1, f);
      const double* Mp = newton_buf64(p, par ? NB_MP1 : NB_MP0, f);
      double* Mpn = newton_buf64(p, par ? NB_MP0 : NB_MP1, f);
      const double* M = newton_buf64(p, par ? NB_M1 : NB_M0, f);
      double* Mn = newton_buf64(p, par ? NB_M0 : NB_M1, f);
      double* S1 = newton_buf64(p, NB_S1, f);
      double* S2 = newton_buf64(p, NB_S2, f);
      p->n64_a[par].add(prob(f, X, Mp, Xn));
      if (!ops.empty()) p->n64_a[par].add(prob(f, Mp, Mp, S1));
      if (!ops.empty() && par == 0) p->n64_a0.add(prob(f, Mp, Mp, S1));  // first iteration: X M_p came from the start kernel
      const double* cur = ops.empty() ? Mp : S1;
      int slot = par * 4;
      double* pong[2] = {S2, S1};
      int which = 0;
      for (size_t q = 1; q < ops.size(); ++q) {
        p->n64_pow[slot++].add(prob(f, cur, ops[q] == 'S' ? cur : Mp, pong[which]));
        cur = pong[which];
        which ^= 1;
      }
      GemmProblem64 m = prob(f, cur, M, Mn);
      m.C2 = Mpn;
      m.err_bits = p->d_err + ids[i];
      p->n64_m[par].add(m);
    }
  }
  for (int par = 0; par < 2; ++par) { SACHECK(commit64(p->n64_a[par], s)); SACHECK(commit64(p->n64_m[par], s)); }
  SACHECK(commit64(p->n64_a0, s));
  for (auto& g : p->n64_pow) SACHECK(commit64(g, s));

  // the start error is 1 (M = z A is far from I): one control pass with err = +inf activates every factor
  NewtonCtl ctl{p->d_err, p->d_active, p->d_iters, p->d_final_parity, p->d_final_err};
  int parity = 0;
  const int Fall = (int)p->factors.size();
  {
    std::vector<unsigned int> inf_bits(Fall, 0x7f800000u);
    HIPCHECK(hipMemcpyAsync(p->d_err, inf_bits.data(), Fall * sizeof(unsigned int), hipMemcpyHostToDevice, s));
    HIPCHECK(hipStreamSynchronize(s));
  }
  hipLaunchKernelGGL(newton_control_kernel, dim3(1), dim3(256), 0, s, ctl, p->t_ids.dev, n, tol, max_iter, parity, p->d_nactive);
  HIPCHECK(hipGetLastError());
  int* h_active = p->h_pinned;
  HIPCHECK(hipMemcpyAsync(h_active, p->d_active, Fall * sizeof(int), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipStreamSynchronize(s));
  for (int it = 0; it < max_iter; ++it) {
    int live = 0;
    double flops = 0.0;
    for (int i = 0; i < n; ++i)
      if (h_active[ids[i]]) { ++live; const double d = p->factors[ids[i]].d; flops += 2.0 * d * d * d * (2.0 + ops.size() - (it == 0 ? 1.0 : 0.0)); }
    if (!live) break;
    {
      Span span("newton_gemm_f64", s, flops, 2 + (int)ops.size() - 1, it == 0);
      SACHECK(launch_gemm64<EPI64_STORE>(it == 0 ? p->n64_a0 : p->n64_a[parity], 0.0, 0.0, s));
      for (int k = 0; k < 4; ++k) SACHECK(launch_gemm64<EPI64_STORE>(p->n64_pow[parity * 4 + k], 0.0, 0.0, s));
      SACHECK(launch_gemm64<EPI64_NEWTON_M>(p->n64_m[parity], alpha, one_minus_alpha, s));
    }
    parity ^= 1;
    hipLaunchKernelGGL(newton_control_kernel, dim3(1), dim3(256), 0, s, ctl, p->t_ids.dev, n, tol, max_iter, parity, p->d_nactive);
    HIPCHECK(hipGetLastError());
    HIPCHECK(hipMemcpyAsync(h_active, p->d_active, Fall * sizeof(int), hipMemcpyDeviceToHost, s));
    HIPCHECK(hipStreamSynchronize(s));
  }
  return SA_OK;
}

static int sa_compute_root_inverses_newton_f64_wave(sa_plan* p, float bias_correction2, double epsilon, int32_t max_iterations,
                                            double tolerance, int32_t widen_ridge_on_failure, int32_t* iterations_out,
                                            int32_t* status_out, void* stream) {
  if (!p || !iterations_out || !status_out) return fail(SA_ERR_INVALID, "sa_compute_root_inverses_newton_f64: NULL argument");
  if (!p->factor_f64) return fail(SA_ERR_STATE, "the factor matrices of this plan are fp32");
  if (!(bias_correction2 != 0.0f) || max_iterations < 0) return fail(SA_ERR_INVALID, "bad bias correction or max_iterations");
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, nullptr, s));
  const int F = (int)p->factors.size();
  if (F == 0) return SA_OK;
  std::vector<int> todo;
  for (int i = 0; i < F; ++i) {
    iterations_out[i] = 0;
    status_out[i] = SA_FACTOR_SKIPPED;
    if (block_active(p, p->factors[i].block) && in_wave(p, i)) todo.push_back(i);
  }
  if (todo.empty()) return SA_OK;
  SACHECK(refresh_inverse_cache(p, s));  // factors that are not recomputed keep a valid dense copy
  const double bc2 = (double)bias_correction2;
  int* h_bad = p->h_pinned + 3 * F;
  std::vector<double> ridge(F, epsilon);

  auto jobs = [&](const std::vector<int>& ids) -> int {
    SACHECK(p->t_f64.begin(ids.size()));
    for (size_t i = 0; i < ids.size(); ++i) {
      const Factor& f = p->factors[ids[i]];
      Factor64& J = p->t_f64.host[i];
      std::memset(&J, 0, sizeof(J));
      J.packed = reinterpret_cast<const double*>(f.factor);
      J.norm_sq = p->d_norm64 + ids[i];
      J.nonfinite = p->d_flags + ids[i];
      J.inv_packed = f.inv;
      J.inv_dense = p->f(p->off_inv_dense) + f.dense_off;
      J.ridge = ridge[ids[i]];
      J.d = f.d; J.n = f.dpad;
    }
    return p->t_f64.upload(s);
  };
  // norm and finiteness of the bias-corrected factors; the reference raises at the first non-finite one
  auto norms = [&](const std::vector<int>& ids) -> int {
    SACHECK(jobs(ids));
    hipLaunchKernelGGL(f64_norm_kernel, dim3((unsigned)ids.size()), dim3(256), 0, s, p->t_f64.dev, bc2);
    HIPCHECK(hipGetLastError());
    return SA_OK;
  };
  HIPCHECK(hipMemsetAsync(p->d_flags, 0, F * sizeof(int), s));
  SACHECK(norms(todo));
  HIPCHECK(hipMemcpyAsync(h_bad, p->d_flags, F * sizeof(int), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipStreamSynchronize(s));
  for (size_t i = 0; i < todo.size(); ++i)
    if (h_bad[todo[i]]) { status_out[todo[i]] = SA_FACTOR_INPUT_NONFINITE; todo.resize(i); break; }
  if (todo.empty()) return SA_OK;

  std::vector<int> par(F, 0);
  std::vector<float> errs(F, 0.0f);
  if (g_profiling) { Phase& ph = g_phases["newton_gemm_f64"]; ph.used = 0; ph.work = 0.0; ph.executed = 0.0; ph.launches = 0; }
  auto solve = [&](const std::vector<int>& subset) -> int {
    std::vector<int> ones(F, 0);
    for (int i : subset) ones[i] = 1;
    HIPCHECK(hipMemsetAsync(p->d_iters, 0, F * sizeof(int), s));
    HIPCHECK(hipMemsetAsync(p->d_final_parity, 0, F * sizeof(int), s));
    HIPCHECK(hipMemcpyAsync(p->d_active, ones.data(), F * sizeof(int), hipMemcpyHostToDevice, s));
    HIPCHECK(hipStreamSynchronize(s));
    std::map<int, std::vector<int>> by_root;
    for (int i : subset) by_root[p->factors[i].root].push_back(i);
    for (auto& kv : by_root)
      SACHECK(newton_batch64(p, kv.second, kv.first, ridge, bc2, max_iterations, (float)tolerance, s));
    HIPCHECK(hipMemcpyAsync(p->h_pinned, p->d_iters, F * sizeof(int), hipMemcpyDeviceToHost, s));
    HIPCHECK(hipMemcpyAsync(p->h_pinned + F, p->d_final_parity, F * sizeof(int), hipMemcpyDeviceToHost, s));
    HIPCHECK(hipMemcpyAsync(p->h_pinned + 2 * F, p->d_final_err, F * sizeof(float), hipMemcpyDeviceToHost, s));
    HIPCHECK(hipStreamSynchronize(s));
    for (int i : subset) {
      iterations_out[i] = p->h_pinned[i];
      par[i] = p->h_pinned[F + i];
      std::memcpy(&errs[i], p->h_pinned + 2 * F + i, sizeof(float));
    }
    return SA_OK;
  };
  SACHECK(solve(todo));
  if (widen_ridge_on_failure) {
    // A factor that is not positive definite above epsilon (Gram matrices are fp32 products: a rank-deficient factor has
    // eigenvalues of either sign of the order 1e-7 ||A||) makes the iteration diverge.  The eigendecomposition the
    // caller stands in for shifts such a spectrum by its smallest eigenvalue; here the ridge grows to 2^-21 ||A||_F.
    std::vector<int> redo;
    for (int i : todo)
      if (!(errs[i] <= (float)tolerance)) redo.push_back(i);
    if (!redo.empty()) {
      std::vector<double> norm_sq(F, 0.0);
      HIPCHECK(hipMemcpy(norm_sq.data(), p->d_norm64, F * sizeof(double), hipMemcpyDeviceToHost));
      for (int i : redo) ridge[i] = epsilon + std::ldexp(std::sqrt(norm_sq[i]), -21);
      HIPCHECK(hipMemsetAsync(p->d_flags, 0, F * sizeof(int), s));
      SACHECK(norms(redo));
      SACHECK(solve(redo));
    }
  }

  // finiteness of the fp32 results first; the factors that precede the first bad one are stored
  auto run_commit = [&](const std::vector<int>& ids, int check_only) -> int {
    SACHECK(jobs(ids));
    int nmax = 0;
    for (size_t i = 0; i < ids.size(); ++i) {
      const Factor& f = p->factors[ids[i]];
      p->t_f64.host[i].result = newton_buf64(p, par[ids[i]] ? NB_X1 : NB_X0, f);
      nmax = std::max(nmax, f.dpad);
    }
    SACHECK(p->t_f64.upload(s));
    const unsigned gx = (unsigned)std::min<long long>(((long long)nmax * nmax + 255) / 256, 2048);
    hipLaunchKernelGGL(f64_commit_kernel, dim3(gx, (unsigned)ids.size()), dim3(256), 0, s, p->t_f64.dev, check_only);
    HIPCHECK(hipGetLastError());
    return SA_OK;
  };
  HIPCHECK(hipMemsetAsync(p->d_flags, 0, F * sizeof(int), s));
  SACHECK(run_commit(todo, 1));
  HIPCHECK(hipMemcpyAsync(h_bad, p->d_flags, F * sizeof(int), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipStreamSynchronize(s));
  std::vector<int> good;
  for (int i : todo) {
    if (h_bad[i]) { status_out[i] = SA_FACTOR_RESULT_NONFINITE; break; }
    good.push_back(i);
    status_out[i] = (errs[i] <= (float)tolerance) ? SA_FACTOR_OK : SA_FACTOR_NOT_CONVERGED;
  }
  if (!good.empty()) {
    SACHECK(run_commit(good, 0));
    HIPCHECK(hipStreamSynchronize(s));
  }
  return SA_OK;
}

int32_t sa_compute_root_inverses_newton_f64(sa_plan* p, float bias_correction2, double epsilon, int32_t max_iterations, double tolerance, int32_t widen_ridge_on_failure, int32_t* iterations_out, int32_t* status_out, void* stream) {
  if (!p || !status_out) return fail(SA_ERR_INVALID, "sa_compute_root_inverses_newton_f64: NULL argument");
  return for_each_wave(p, iterations_out, status_out, static_cast<hipStream_t>(stream), [&](int32_t* it__, int32_t* st__) {
    return sa_compute_root_inverses_newton_f64_wave(p, bias_correction2, epsilon, max_iterations, tolerance, widen_ridge_on_failure, it__, st__, stream);
  });
}

// --------------------------------------------------------------------------------------------
// Batched coupled higher-order iteration (reference: matrix_functions.py:439-661)
// --------------------------------------------------------------------------------------------

constexpr int HO_MAX_ORDER = 8;

static int higher_order_batch(sa_plan* p, const std::vector<int>& ids, int root, int order, float rel_eps, float abs_eps,
                              float bc2, int max_iter, float tol, hipStream_t s, double* flops_acc, int* launches_acc) {
  const int n = (int)ids.size();
  if (n == 0) return SA_OK;
  std::vector<char> ops;
  SACHECK(power_ops(root, &ops));
  const int horner = order - 2;  // products that build M_p from I - M
  // b_0 = 1, b_i = b_{i-1} (1 + (i - 1) p) / (i p): exact integer products, one division per entry
  std::vector<double> b(order, 1.0);
  {
    double num = 1.0, den = 1.0;
    for (int i = 1; i < order; ++i) { num *= 1.0 + (i - 1.0) * root; den *= (double)i * root; b[i] = num / den; }
  }

  // ---- start: A dense, |A|_inf, eps, z, then M, M_p of the plain Newton step, X -------------------------
  SACHECK(p->t_ids.begin(n));
  std::memcpy(p->t_ids.host, ids.data(), n * sizeof(int));
  SACHECK(p->t_ids.upload(s));
  SACHECK(p->t_eiginit.begin(n));
  SACHECK(p->t_ho.begin(n));
  int tiles = 0, dmax = 0, dpadmax = 0;
  for (int i = 0; i < n; ++i) {
    const Factor& f = p->factors[ids[i]];
    EigInit& J = p->t_eiginit.host[i];
    std::memset(&J, 0, sizeof(J));
    J.packed = packed32(p, f); J.scale = p->scale_of(ids[i]); J.A = newton_buf(p, NB_M0, f); J.V = newton_buf(p, NB_X0, f);
    J.d = f.d; J.dpad = f.dpad; J.tiles = f.dpad / 64; J.enabled = 1; J.tile_begin = tiles;
    tiles += J.tiles * J.tiles;
    HoJob& H = p->t_ho.host[i];
    std::memset(&H, 0, sizeof(H));
    H.A = newton_buf(p, NB_M0, f); H.Mp = newton_buf(p, NB_MP1, f); H.X = newton_buf(p, NB_X0, f);
    H.rowsum = newton_buf(p, NB_S1, f); H.params = p->d_ho + 4 * ids[i];
    H.d = f.d; H.dpad = f.dpad;
    dmax = std::max(dmax, f.d); dpadmax = std::max(dpadmax, f.dpad);
  }
  SACHECK(p->t_eiginit.upload(s));
  SACHECK(p->t_ho.upload(s));
  const unsigned start_blocks = (unsigned)(((long long)dpadmax * dpadmax + 1023) / 1024);
  hipLaunchKernelGGL(eig_init_kernel, dim3(tiles), dim3(256), 0, s, p->t_eiginit.dev, n, bc2, 0.0f);
  hipLaunchKernelGGL(ho_rowsum_kernel, dim3((dmax + 3) / 4, n), dim3(256), 0, s, p->t_ho.dev);
  hipLaunchKernelGGL(ho_setup_kernel, dim3(n), dim3(256), 0, s, p->t_ho.dev, rel_eps, abs_eps);
  hipLaunchKernelGGL(ho_start_kernel, dim3(start_blocks, n), dim3(256), 0, s, p->t_ho.dev, root, 0);
  HIPCHECK(hipGetLastError());

  // ---- GEMM tables (full products) -----------------------------------------------------------------------
  for (int par = 0; par < 2; ++par) { p->nt_a[0][par].clear(); p->nt_m[0][par].clear(); }
  for (int k = 0; k < 8; ++k) { p->nt_pow[0][k].clear(); p->nt_h[k].clear(); }
  auto prob = [&](const Factor& f, const float* A, const float* B, float* C) {
    GemmProblem q{};
    q.A = A; q.B = B; q.C = C;
    q.lda = q.ldb = q.ldc = f.dpad;
    q.M = q.N = q.K = f.dpad;
    q.d = f.d;
    q.a_vec = q.b_vec = 1;
    q.active = p->d_active + (&f - p->factors.data());
    return q;
  };
  for (int i = 0; i < n; ++i) {
    const Factor& f = p->factors[ids[i]];
    float* Mp0 = newton_buf(p, NB_MP0, f);
    float* Mp1 = newton_buf(p, NB_MP1, f);
    float* S1 = newton_buf(p, NB_S1, f);
    float* S2 = newton_buf(p, NB_S2, f);
    for (int par = 0; par < 2; ++par) {
      const float* X = newton_buf(p, par ? NB_X1 : NB_X0, f);
      float* Xn = newton_buf(p, par ? NB_X0 : NB_X1, f);
      const float* M = newton_buf(p, par ? NB_M1 : NB_M0, f);
      float* Mn = newton_buf(p, par ? NB_M0 : NB_M1, f);
      // order 2: the epilogue of the last product writes the next M_p itself, alternating between the two M_p
      // arrays; order >= 3: it writes I - M to Mp0 and the Horner products leave M_p in Mp1
      const float* Mp = (order == 2 && par == 1) ? Mp0 : Mp1;
      float* seed = (order == 2 && par == 1) ? Mp1 : Mp0;
      p->nt_a[0][par].add(prob(f, X, Mp, Xn), false);
      if (!ops.empty()) p->nt_a[0][par].add(prob(f, Mp, Mp, S1), false);
      const float* cur = ops.empty() ? Mp : S1;
      int slot = par * 4;
      float* pong[2] = {S2, S1};
      int which = 0;
      for (size_t q = 1; q < ops.size(); ++q) {
        p->nt_pow[0][slot++].add(prob(f, cur, ops[q] == 'S' ? cur : Mp, pong[which]), false);
        cur = pong[which];
        which ^= 1;
      }
      GemmProblem m = prob(f, cur, M, Mn);
      m.C2 = seed;
      m.err_bits = p->d_err + ids[i];
      p->nt_m[0][par].add(m, false);
    }
    const float* prev = Mp0;
    for (int k = 0; k < horner; ++k) {
      float* out = (k == horner - 1) ? Mp1 : ((k & 1) ? S2 : S1);
      GemmProblem h = prob(f, prev, Mp0, out);
      h.C2 = Mp0;  // read only
      p->nt_h[k].add(h, false);
      prev = out;
    }
  }
  for (int par = 0; par < 2; ++par) { SACHECK(p->nt_a[0][par].commit(s)); SACHECK(p->nt_m[0][par].commit(s)); }
  for (int k = 0; k < 8; ++k) { SACHECK(p->nt_pow[0][k].commit(s)); SACHECK(p->nt_h[k].commit(s)); }

  HigherOrderCtl ctl{p->d_err, p->d_active, p->d_iters, p->d_final_parity, p->d_final_err, p->d_kept_err, p->d_hoflag};
  int parity = 0;
  hipLaunchKernelGGL(higher_order_control_kernel, dim3(1), dim3(256), 0, s, ctl, p->t_ids.dev, n, tol, max_iter, 0, parity);
  HIPCHECK(hipGetLastError());
  int* h_active = p->h_pinned;
  const int Fall = (int)p->factors.size();
  HIPCHECK(hipMemcpyAsync(h_active, p->d_active, Fall * sizeof(int), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipStreamSynchronize(s));
  GemmScalars unit = unit_scalars();
  GemmScalars msc = unit_scalars();
  if (order == 2) { msc.mp_scale = (float)(-b[1]); msc.mp_diag = (float)(b[1] + b[0]); }
  else { msc.mp_scale = -1.0f; msc.mp_diag = 1.0f; }
  for (int it = 0; it <= max_iter; ++it) {
    const int gemms = 1 + (int)ops.size() + 1 + (it >= 1 ? horner : 0);
    double flops = 0.0;
    int live = 0;
    for (int i = 0; i < n; ++i)
      if (h_active[ids[i]]) {
        const double d = p->factors[ids[i]].d;
        flops += 2.0 * d * d * d * gemms;
        ++live;
      }
    if (!live) break;
    {
      int nl = (p->nt_a[0][parity].total_tiles ? 1 : 0) + (p->nt_m[0][parity].total_tiles ? 1 : 0) + (it >= 1 ? horner : 0);
      for (int k = 0; k < 4; ++k) nl += p->nt_pow[0][parity * 4 + k].total_tiles ? 1 : 0;
      Span span("newton_gemm", s, flops, nl, false);
      if (g_profiling) g_phases["newton_gemm"].executed += flops;
      if (it >= 1) {
        for (int k = 0; k < horner; ++k) {
          GemmScalars hs = unit_scalars();
          // first product: b_{o-1} (I-M)^2 + b_{o-2} (I-M) + b_{o-3} I; later ones: M_p (I-M) + b_i I
          hs.alpha = (k == 0) ? (float)b[order - 1] : 1.0f;
          hs.beta = (k == 0) ? (float)b[order - 2] : 0.0f;
          hs.mp_diag = (float)b[order - 3 - k];
          SACHECK((launch_gemm<A_MK, B_KN, EPI_HORNER, false, false>(p->nt_h[k], hs, s)));
        }
      }
      SACHECK((launch_gemm<A_MK, B_KN, EPI_STORE, false, false>(p->nt_a[0][parity], unit, s)));
      for (int k = 0; k < 4; ++k)
        SACHECK((launch_gemm<A_MK, B_KN, EPI_STORE, false, false>(p->nt_pow[0][parity * 4 + k], unit, s)));
      SACHECK((launch_gemm<A_MK, B_KN, EPI_NEWTON_M, false, false>(p->nt_m[0][parity], msc, s)));
      *flops_acc += flops;
      *launches_acc += nl;
    }
    parity ^= 1;
    hipLaunchKernelGGL(higher_order_control_kernel, dim3(1), dim3(256), 0, s, ctl, p->t_ids.dev, n, tol, max_iter, it + 1, parity);
    HIPCHECK(hipGetLastError());
    HIPCHECK(hipMemcpyAsync(h_active, p->d_active, Fall * sizeof(int), hipMemcpyDeviceToHost, s));
    HIPCHECK(hipStreamSynchronize(s));
  }
  return SA_OK;
}

// |A_r X^p - I|_max of the finished factors of one root (matrix_functions.py:622-626): A_r is rebuilt in Mp0,
// X^p goes through S1 / S2, the product lands in the M array that does not hold the final M.
static int higher_order_residuals(sa_plan* p, const std::vector<int>& ids, const std::vector<int>& par, int root, float bc2,
                                  hipStream_t s) {
  const int n = (int)ids.size();
  if (n == 0) return SA_OK;
  std::vector<char> ops;
  SACHECK(power_ops(root, &ops));
  SACHECK(p->t_eiginit.begin(n));
  SACHECK(p->t_ho.begin(n));
  int tiles = 0, dpadmax = 0;
  for (int i = 0; i < n; ++i) {
    const Factor& f = p->factors[ids[i]];
    EigInit& J = p->t_eiginit.host[i];
    std::memset(&J, 0, sizeof(J));
    J.packed = packed32(p, f); J.scale = p->scale_of(ids[i]); J.A = newton_buf(p, NB_MP0, f); J.V = newton_buf(p, NB_MP1, f);
    J.d = f.d; J.dpad = f.dpad; J.tiles = f.dpad / 64; J.enabled = 1; J.tile_begin = tiles;
    tiles += J.tiles * J.tiles;
    HoJob& H = p->t_ho.host[i];
    std::memset(&H, 0, sizeof(H));
    H.A = newton_buf(p, NB_MP0, f); H.params = p->d_ho + 4 * ids[i]; H.d = f.d; H.dpad = f.dpad;
    dpadmax = std::max(dpadmax, f.dpad);
  }
  SACHECK(p->t_eiginit.upload(s));
  SACHECK(p->t_ho.upload(s));
  hipLaunchKernelGGL(eig_init_kernel, dim3(tiles), dim3(256), 0, s, p->t_eiginit.dev, n, bc2, 0.0f);
  hipLaunchKernelGGL(ho_start_kernel, dim3((unsigned)(((long long)dpadmax * dpadmax + 1023) / 1024), n), dim3(256), 0, s,
                     p->t_ho.dev, root, 1);
  HIPCHECK(hipGetLastError());
  for (int k = 0; k < 8; ++k) p->nt_pow[0][k].clear();
  p->nt_m[0][0].clear();
  for (int i = 0; i < n; ++i) {
    const Factor& f = p->factors[ids[i]];
    auto prob = [&](const float* A, const float* B, float* C) {
      GemmProblem q{};
      q.A = A; q.B = B; q.C = C;
      q.lda = q.ldb = q.ldc = f.dpad;
      q.M = q.N = q.K = f.dpad;
      q.d = f.d;
      q.a_vec = q.b_vec = 1;
      return q;
    };
    const float* X = newton_buf(p, par[ids[i]] ? NB_X1 : NB_X0, f);
    float* S1 = newton_buf(p, NB_S1, f);
    float* S2 = newton_buf(p, NB_S2, f);
    const float* cur = X;
    int slot = 0;
    float* pong[2] = {S1, S2};
    int which = 0;
    for (char op : ops) {
      p->nt_pow[0][slot++].add(prob(cur, op == 'S' ? cur : X, pong[which]), false);
      cur = pong[which];
      which ^= 1;
    }
    GemmProblem m = prob(newton_buf(p, NB_MP0, f), cur, newton_buf(p, par[ids[i]] ? NB_M0 : NB_M1, f));
    m.C2 = newton_buf(p, NB_MP1, f);
    m.err_bits = p->d_err + ids[i];
    p->nt_m[0][0].add(m, false);
  }
  for (int k = 0; k < 8; ++k) SACHECK(p->nt_pow[0][k].commit(s));
  SACHECK(p->nt_m[0][0].commit(s));
  GemmScalars unit = unit_scalars();
  for (int k = 0; k < 8; ++k) SACHECK((launch_gemm<A_MK, B_KN, EPI_STORE, false, false>(p->nt_pow[0][k], unit, s)));
  SACHECK((launch_gemm<A_MK, B_KN, EPI_NEWTON_M, false, false>(p->nt_m[0][0], unit, s)));
  return SA_OK;
}

static int sa_compute_root_inverses_higher_order_wave(sa_plan* p, float bias_correction2, float rel_epsilon, float abs_epsilon,
                                              int32_t max_iterations, float tolerance, int32_t order,
                                              int32_t* iterations_out, int32_t* status_out, void* stream) {
  if (!p || !iterations_out || !status_out) return fail(SA_ERR_INVALID, "sa_compute_root_inverses_higher_order: NULL argument");
  if (!(bias_correction2 != 0.0f) || max_iterations < 0) return fail(SA_ERR_INVALID, "bad bias correction or max_iterations");
  if (order < 2 || order > HO_MAX_ORDER)
    return fail(SA_ERR_UNSUPPORTED, "the higher-order iteration is built for orders 2.." + std::to_string(HO_MAX_ORDER));
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, nullptr, s));
  const int F = (int)p->factors.size();
  if (F == 0) return SA_OK;
  if (g_profiling) { Phase& ph = g_phases["newton_gemm"]; ph.used = 0; ph.work = 0.0; ph.executed = 0.0; ph.launches = 0; }
  std::vector<int> todo;
  SACHECK(root_inverse_prologue(p, bias_correction2, 0.0f, iterations_out, status_out, s, &todo));
  if (todo.empty()) return SA_OK;

  std::vector<int> ones(F, 0);
  for (int i : todo) ones[i] = 1;
  HIPCHECK(hipMemsetAsync(p->d_err, 0, F * sizeof(int), s));
  HIPCHECK(hipMemsetAsync(p->d_iters, 0, F * sizeof(int), s));
  HIPCHECK(hipMemsetAsync(p->d_final_parity, 0, F * sizeof(int), s));
  HIPCHECK(hipMemsetAsync(p->d_hoflag, 0, F * sizeof(int), s));
  HIPCHECK(hipMemsetAsync(p->d_kept_err, 0, F * sizeof(float), s));
  HIPCHECK(hipMemcpyAsync(p->d_active, ones.data(), F * sizeof(int), hipMemcpyHostToDevice, s));
  HIPCHECK(hipStreamSynchronize(s));
  std::map<int, std::vector<int>> by_root;
  for (int i : todo) by_root[p->factors[i].root].push_back(i);
  double flops = 0.0;
  int launches = 0;
  for (auto& kv : by_root)
    SACHECK(higher_order_batch(p, kv.second, kv.first, order, rel_epsilon, abs_epsilon, bias_correction2, max_iterations,
                               tolerance, s, &flops, &launches));
  std::vector<int> iters(F, 0), par(F, 0), flag(F, 0);
  HIPCHECK(hipMemcpyAsync(p->h_pinned, p->d_iters, F * sizeof(int), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipMemcpyAsync(p->h_pinned + F, p->d_final_parity, F * sizeof(int), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipMemcpyAsync(p->h_pinned + 2 * F, p->d_hoflag, F * sizeof(int), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipMemsetAsync(p->d_err, 0, F * sizeof(int), s));
  HIPCHECK(hipStreamSynchronize(s));
  for (int i : todo) { iters[i] = p->h_pinned[i]; par[i] = p->h_pinned[F + i]; flag[i] = p->h_pinned[2 * F + i]; }

  // the reference's accuracy gate: |A_r X^p - I|_max above 0.1 is a solver failure
  for (auto& kv : by_root) SACHECK(higher_order_residuals(p, kv.second, par, kv.first, bias_correction2, s));
  HIPCHECK(hipMemcpyAsync(p->h_pinned + 3 * F, p->d_err, F * sizeof(int), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipStreamSynchronize(s));
  std::vector<int> pass;
  std::vector<const float*> X;
  for (int i : todo) {
    float residual;
    std::memcpy(&residual, p->h_pinned + 3 * F + i, sizeof(float));
    iterations_out[i] = iters[i];
    if (residual > 0.1f) { status_out[i] = SA_FACTOR_SOLVER_FAILED; continue; }
    status_out[i] = flag[i] == 1 ? SA_FACTOR_NOT_CONVERGED : SA_FACTOR_OK;
    pass.push_back(i);
    X.push_back(newton_buf(p, par[i] ? NB_X1 : NB_X0, p->factors[i]));
  }
  size_t ok = 0;
  if (!pass.empty()) SACHECK(root_inverse_epilogue(p, pass, X, status_out, s, &ok, true));
  return SA_OK;
}

int32_t sa_compute_root_inverses_higher_order(sa_plan* p, float bias_correction2, float rel_epsilon, float abs_epsilon, int32_t max_iterations, float tolerance, int32_t order, int32_t* iterations_out, int32_t* status_out, void* stream) {
  if (!p || !status_out) return fail(SA_ERR_INVALID, "sa_compute_root_inverses_higher_order: NULL argument");
  return for_each_wave(p, iterations_out, status_out, static_cast<hipStream_t>(stream), [&](int32_t* it__, int32_t* st__) {
    return sa_compute_root_inverses_higher_order_wave(p, bias_correction2, rel_epsilon, abs_epsilon, max_iterations, tolerance, order, it__, st__, stream);
  });
}

// --------------------------------------------------------------------------------------------
// Batched eigendecomposition through tridiagonalisation (orders >= TRD_MIN_DIM)
// --------------------------------------------------------------------------------------------

constexpr int TRD_MIN_DIM = 512;
constexpr int TQL_MAX_ITER = 30;  // QL sweeps allowed per factor: TQL_MAX_ITER x order, as in LAPACK's steqr

// layout of the small arrays inside a factor's M1 array (floats)
inline long long trd_p_offset(const Factor&) { return 0; }                                   // panel buffer: 96 x dpad of the 128 x dpad reserved
inline long long trd_vec_offset(const Factor& f, int k) { return 2LL * f.dpad * TRD_PW + (long long)k * f.dpad; }
inline long long trd_diag_offset(const Factor& f) { return trd_vec_offset(f, 2); }           // vbuf, ybuf, diag, off, tau
inline long long trd_tmat_offset(const Factor& f) { return trd_vec_offset(f, 9); }           // dpad x 32 (after two fp64 vectors)
inline long long trd_int_offset(const Factor& f) { return trd_tmat_offset(f) + (long long)f.dpad * TRD_NB; }

static int trd_side_stream(sa_plan* p) {
  if (p->trd_stream) return SA_OK;
  HIPCHECK(hipStreamCreateWithFlags(&p->trd_stream, hipStreamNonBlocking));  // default priority
  for (hipStream_t& q : p->trd_lane_stream) HIPCHECK(hipStreamCreateWithFlags(&q, hipStreamNonBlocking));
  for (hipEvent_t& e : p->trd_ev) HIPCHECK(hipEventCreateWithFlags(&e, hipEventDisableTiming));
  for (hipEvent_t& e : p->trd_lane_ev) HIPCHECK(hipEventCreateWithFlags(&e, hipEventDisableTiming));
  return SA_OK;
}

// Eigendecomposition of the dense matrices in the M0 arrays of `ids` (all of one order).  On return the rows of
// the X0 array are the eigenvectors and trd_diag_offset() of the M1 array holds the eigenvalues.  X0 must hold
// the identity on entry.  Uses X1 (Householder vectors), Mp1 (V T), S1, M1 and Mp0 as scratch.
static int eigh_tridiagonal(sa_plan* p, const std::vector<int>& ids, hipStream_t s, int32_t* sweeps_out, int* not_converged) {
  const int n = (int)ids.size();
  if (n == 0) return SA_OK;
  const int d = p->factors[ids[0]].d, dpad = p->factors[ids[0]].dpad;
  const long long ld = dpad;
  const int panels = (d - 1 + TRD_NB - 1) / TRD_NB;

  SACHECK(p->t_trd.begin(n));
  for (int k = 0; k < n; ++k) {
    const Factor& f = p->factors[ids[k]];
    TrdJob& J = p->t_trd.host[k];
    std::memset(&J, 0, sizeof(J));
    float* m1 = newton_buf(p, NB_M1, f);
    J.A = newton_buf(p, NB_M0, f);
    J.Y = newton_buf(p, NB_X0, f);
    J.Vall = newton_buf(p, NB_X1, f);
    J.P1 = m1 + trd_p_offset(f);
    J.P2 = J.P1 + (long long)dpad * TRD_NB;
    J.vbuf = m1 + trd_vec_offset(f, 0);
    J.ybuf = m1 + trd_vec_offset(f, 1);
    J.part = newton_buf(p, NB_S2, f);
    J.diag = m1 + trd_vec_offset(f, 2);
    J.off = m1 + trd_vec_offset(f, 3);
    J.tau = m1 + trd_vec_offset(f, 4);
    J.qd = reinterpret_cast<double*>(m1 + trd_vec_offset(f, 5));
    J.qe = reinterpret_cast<double*>(m1 + trd_vec_offset(f, 7));
    J.d1buf = m1 + trd_tmat_offset(f);
    J.apre = J.d1buf + ld;
    J.t12 = J.apre + ld;
    J.hdr = reinterpret_cast<int*>(m1 + trd_int_offset(f));
    J.state = J.hdr + 2 * TQL_HDR;
    J.rot = reinterpret_cast<float2*>(newton_buf(p, NB_MP0, f));
    // bisection + inverse iteration, after the reduction and the formation of Q1^T: Z takes the place of A, the
    // small tables that of the panel buffers, the E-wide tables those of the buffers of the two finished phases
    J.S128 = J.part;  // the symmetric products are done when Q1 is accumulated
    J.T128 = J.P1;    // so are the panels (dpad x 128 floats)
    J.Z = J.A;
    J.lam = reinterpret_cast<double*>(J.P1);
    J.blk_s = reinterpret_cast<int*>(J.P1 + 2 * ld);
    J.blk_e = J.blk_s + ld;
    J.fail = J.blk_e + ld;
    J.chunk = dpad / 4;
    const long long tab = ld * J.chunk;  // doubles per table: half a dense array
    J.lu_a = reinterpret_cast<double*>(newton_buf(p, NB_S2, f));
    J.lu_b = J.lu_a + tab;
    J.lu_d = reinterpret_cast<double*>(newton_buf(p, NB_MP0, f));
    J.lu_c = J.lu_d + tab;
    J.lu_x = reinterpret_cast<double*>(newton_buf(p, NB_MP1, f));
    J.lu_f = reinterpret_cast<unsigned char*>(J.lu_x + tab);
    J.d = d; J.dpad = dpad;
    HIPCHECK(hipMemsetAsync(J.Vall, 0, sizeof(float) * ld * ld, s));
    HIPCHECK(hipMemsetAsync(J.vbuf, 0, sizeof(float) * 5 * ld, s));
  }
  SACHECK(p->t_trd.upload(s));
  const TrdJob* jobs = p->t_trd.dev;

  // GEMM problem tables: [trailing update per panel | V T for every panel | G = (V T)^T Y per panel | Y -= V G per panel]
  std::vector<GemmProblem> probs;
  // The reduction runs the factors as one or two lanes (halves of the batch on two streams, see step 1): the trailing
  // update has one table per panel and lane.
  constexpr int ML = 4;  // most lanes
  const int lanes = std::max(1, std::min({p->trd_lanes, ML, n / 2}));
  int lane_n[ML] = {0, 0, 0, 0}, lane_first[ML] = {0, 0, 0, 0};
  for (int h = 0; h < lanes; ++h) {
    lane_n[h] = n / lanes + (h < n % lanes ? 1 : 0);
    lane_first[h] = h == 0 ? 0 : lane_first[h - 1] + lane_n[h - 1];
  }
  std::vector<int> trail_off(ML * panels, 0), trail_tiles(ML * panels, 0);
  // small: walked in 64 x 64 tiles.  The rank-64 / rank-128 updates of a large matrix are a read-modify-write of that
  // matrix with a short product in between: small tiles put four times as many independent chains of loads on a CU
  // (rank-64 update of 32 triangles of order 4096: 0.62 ms against 0.83 ms with 128 x 128 tiles).
  auto push = [&](const float* A, long long lda, const float* B, long long ldb, float* C, long long ldc, int M, int N, int K,
                  int* tiles, bool lower = false, bool small = false) {
    GemmProblem q{};
    q.A = A; q.lda = lda; q.a_vec = vec_ok(A, lda);
    q.B = B; q.ldb = ldb; q.b_vec = vec_ok(B, ldb);
    q.C = C; q.ldc = ldc; q.M = M; q.N = N; q.K = K;
    if (small) {
      q.tiles_m_s = (M + 63) / 64;
      q.tiles_n_s = (N + 63) / 64;
      q.tile_begin_s = *tiles;
      *tiles += lower ? q.tiles_n_s * (q.tiles_n_s + 1) / 2 : q.tiles_m_s * q.tiles_n_s;
    } else {
      q.tiles_m = (M + BM - 1) / BM;
      q.tiles_n = (N + BN - 1) / BN;
      q.tile_begin = *tiles;
      *tiles += lower ? q.tiles_n * (q.tiles_n + 1) / 2 : q.tiles_m * q.tiles_n;
    }
    probs.push_back(q);
  };
  for (int b = 0; b < panels; ++b) {
    const int q0 = std::min(b * TRD_NB + TRD_NB, d - 1);  // first row / column after the panel
    for (int h = 0; h < lanes; ++h) {
      trail_off[ML * b + h] = (int)probs.size();
      if (d - q0 > 0)
        for (int k = lane_first[h]; k < lane_first[h] + lane_n[h]; ++k) {
          const TrdJob& J = p->t_trd.host[k];
          // every reader of the trailing matrix uses its lower triangle only: so does the update
          // (the panels are stored by columns: both operands are read as K x M / K x N with unit stride along the rows).
          // The updated region starts at the tile boundary at or in front of q0 and runs to the padded order, so that
          // every tile is whole and aligned and the unguarded loader and epilogue serve: the rows and columns in front of
          // q0 belong to the reduced part, which nothing reads again (the products multiply them by the zeros in front
          // of the Householder vector), and the panel is zero beyond the order.
          const int q0a = q0 & ~(BM - 1);
          push(J.P1 + q0a, ld, J.P2 + q0a, ld, J.A + q0a * ld + q0a, ld, dpad - q0a, dpad - q0a, TRD_PW, &trail_tiles[ML * b + h], true, true);
        }
    }
  }
  // accumulation of Q1 = H_0 H_1 ... with block reflectors of 128 vectors, last block first (only the trailing corner
  // of Q differs from the identity then): [S = V^T V for every block | V T for every block | G = V^T Q per block |
  // Q -= (V T) G per block]
  const int qblocks = (d - 1 + TRD_QB - 1) / TRD_QB;
  const int s_off = (int)probs.size();
  int s_tiles = 0;
  for (int b = 0; b < qblocks; ++b)
    for (int k = 0; k < n; ++k) {
      const TrdJob& J = p->t_trd.host[k];
      const int p0 = b * TRD_QB;
      const float* V = J.Vall + p0 * ld + p0;
      // (all of these run to the padded order: the Householder vectors are zero there, and whole tiles need no guards)
      push(V, ld, V, ld, J.S128 + (long long)b * TRD_QB * TRD_QB, TRD_QB, TRD_QB, TRD_QB, dpad - p0, &s_tiles);
    }
  const int s_count = (int)probs.size() - s_off;
  const int vt_off = (int)probs.size();
  int vt_tiles = 0;
  for (int b = 0; b < qblocks; ++b)
    for (int k = 0; k < n; ++k) {
      const Factor& f = p->factors[ids[k]];
      const TrdJob& J = p->t_trd.host[k];
      const int p0 = b * TRD_QB;
      float* VT = newton_buf(p, NB_MP1, f);
      push(J.Vall + p0 * ld + p0, ld, J.T128 + (long long)b * TRD_QB * TRD_QB, TRD_QB, VT + p0 * ld + p0, ld, dpad - p0, TRD_QB, TRD_QB,
           &vt_tiles);
    }
  const int vt_count = (int)probs.size() - vt_off;
  std::vector<int> g1_off(qblocks), g1_tiles(qblocks, 0), g2_off(qblocks), g2_tiles(qblocks, 0);
  for (int b = 0; b < qblocks; ++b) {
    const int p0 = b * TRD_QB;
    g1_off[b] = (int)probs.size();
    for (int k = 0; k < n; ++k) {
      const Factor& f = p->factors[ids[k]];
      const TrdJob& J = p->t_trd.host[k];
      push(J.Vall + p0 * ld + p0, ld, J.Y + p0 * ld + p0, ld, newton_buf(p, NB_S1, f), ld, TRD_QB, dpad - p0, dpad - p0, &g1_tiles[b]);
    }
    g2_off[b] = (int)probs.size();
    for (int k = 0; k < n; ++k) {
      const Factor& f = p->factors[ids[k]];
      const TrdJob& J = p->t_trd.host[k];
      push(newton_buf(p, NB_MP1, f) + p0 * ld + p0, ld, newton_buf(p, NB_S1, f), ld, J.Y + p0 * ld + p0, ld, dpad - p0, dpad - p0, TRD_QB,
           &g2_tiles[b], false, true);
    }
  }
  SACHECK(p->t_trd_gemm.begin(probs.size()));
  std::memcpy(p->t_trd_gemm.host, probs.data(), probs.size() * sizeof(GemmProblem));
  SACHECK(p->t_trd_gemm.upload(s));
  const GemmProblem* gp = p->t_trd_gemm.dev;
  const GemmScalars unit = unit_scalars();

  // ---- 1. tridiagonalise
  {
    Span span("tridiagonalize", s, 2.0 / 3.0 * (double)d * d * d * n, 3 * d, true);  // bytes of the matrix-vector products (one triangle)
    static bool symv_attr = false;
    if (!symv_attr) {
      HIPCHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(trd_symv_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   2 * TRD_MAX_DIM * (int)sizeof(float)));
      symv_attr = true;
    }
    // Per column two launches on one stream: the column step, then the product of that column together with the
    // row terms of the next column step (extra workgroups of the same launch).  The column step is one workgroup per
    // factor and all latency, and every launch waits for the one before it, so a batch on one stream leaves most of the
    // chip idle for a quarter of the time: the batch is reduced in `lanes` parts on as many streams (streams the plan
    // owns take the parts after the first), whose column steps and launch gaps fall into each other's products: 32
    // factors of order 4096 take 415 / 376 / 361 / 527 ms with 1 / 2 / 3 / 4 lanes (four streams are as many as the
    // process has hardware queues).  The factors are independent of each other: the bits are those of one lane.
    hipStream_t sl[ML] = {s, s, s, s};
    if (lanes >= 2) {
      SACHECK(trd_side_stream(p));
      HIPCHECK(hipEventRecord(p->trd_ev[4], s));
      for (int h = 1; h < lanes; ++h) {
        sl[h] = h == 1 ? p->trd_stream : p->trd_lane_stream[h - 2];
        HIPCHECK(hipStreamWaitEvent(sl[h], p->trd_ev[4], 0));
      }
    }
    auto launch_col = [&](int h, int j, int p0, int flags) {
      const TrdJob* jl = jobs + lane_first[h];
      const dim3 g(lane_n[h]);
      if (d <= TRD_COL_THREADS) hipLaunchKernelGGL(trd_col_kernel<1>, g, dim3(TRD_COL_THREADS), 0, sl[h], jl, j, p0, flags);
      else if (d <= 2 * TRD_COL_THREADS) hipLaunchKernelGGL(trd_col_kernel<2>, g, dim3(TRD_COL_THREADS), 0, sl[h], jl, j, p0, flags);
      else if (d <= 4 * TRD_COL_THREADS) hipLaunchKernelGGL(trd_col_kernel<4>, g, dim3(TRD_COL_THREADS), 0, sl[h], jl, j, p0, flags);
      else hipLaunchKernelGGL(trd_col_kernel<TRD_ROWS_PER_THREAD>, g, dim3(TRD_COL_THREADS), 0, sl[h], jl, j, p0, flags);
    };
    // product of column j (j < 0: none) and the row terms of column step (aj, p0, flags)
    auto launch_product = [&](int h, int j, int aj, int p0, int flags) {
      int nbk = 0;
      if (j >= 0) {
        const int sbase = (j + 1) & ~(TRD_SB - 1);
        nbk = (d - sbase + TRD_SB - 1) / TRD_SB;
      }
      const size_t lds = std::max<size_t>(2 * (size_t)nbk * TRD_SB, 4 * TRD_NB) * sizeof(float);
      hipLaunchKernelGGL(trd_symv_kernel, dim3(TRD_AUX_WGS + (nbk + 1) / 2, lane_n[h]), dim3(256), lds, sl[h], jobs + lane_first[h], j,
                         TRD_AUX_WGS, aj, p0, flags);
    };
    for (int b = 0; b < panels; ++b) {
      const int p0 = b * TRD_NB, kcols = std::min(TRD_NB, d - 1 - p0);
      for (int h = 0; h < lanes; ++h) {
        hipLaunchKernelGGL(trd_clear_panel_kernel, dim3(std::max(1, dpad / 32), lane_n[h]), dim3(256), 0, sl[h], jobs + lane_first[h]);
        launch_product(h, -1, p0, p0, 2);  // first column of the panel: after the clear and the trailing update
      }
      for (int i = 0; i < kcols; ++i) {
        const int j = p0 + i;
        for (int h = 0; h < lanes; ++h) {
          launch_col(h, j, p0, (i > 0 ? 1 : 0) | 2);
          launch_product(h, j, j + 1, p0, i + 1 < kcols ? 3 : 1);
        }
      }
      for (int h = 0; h < lanes; ++h) {
        launch_col(h, p0 + kcols, p0, 1);
        HIPCHECK(hipGetLastError());
        SACHECK((launch_gemm_raw<A_KM, B_KN, EPI_SUB, false, true, 1>(gp + trail_off[ML * b + h], lane_n[h], trail_tiles[ML * b + h], unit, sl[h])));
      }
    }
    // last diagonal entry (a fresh, empty panel: no pending corrections)
    for (int h = 0; h < lanes; ++h) {
      launch_product(h, -1, d - 1, d - 1, 2);
      launch_col(h, d - 1, d - 1, 2);
    }
    HIPCHECK(hipGetLastError());
    for (int h = 1; h < lanes; ++h) {
      HIPCHECK(hipEventRecord(p->trd_lane_ev[h - 1], sl[h]));
      HIPCHECK(hipStreamWaitEvent(s, p->trd_lane_ev[h - 1], 0));
    }
  }

  // ---- 2. Q1 = H_0 H_1 ... in the Y array (identity on entry): Q <- (I - V_b T_b V_b^T) Q for b = last .. 0, which
  // touches only Q[p0:, p0:] (the rest of those rows and columns is still the identity's)
  {
    double flops = 0.0;
    for (int b = 0; b < qblocks; ++b) { const double m = d - b * TRD_QB; flops += (4.0 * m * m + 4.0 * m * TRD_QB) * TRD_QB * n; }
    Span span("form_q", s, flops, 2 * qblocks + 3, true);
    static bool t128_attr = false;
    if (!t128_attr) {
      HIPCHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(trd_tfactor128_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   2 * TRD_QB * TRD_QB * (int)sizeof(float)));
      t128_attr = true;
    }
    // row j of Vall is the Householder vector of column j: V^T is the array as it stands
    SACHECK((launch_gemm_raw<A_MK, B_NK, EPI_STORE, false>(gp + s_off, s_count, s_tiles, unit, s)));
    hipLaunchKernelGGL(trd_tfactor128_kernel, dim3(qblocks, n), dim3(256), 2 * TRD_QB * TRD_QB * sizeof(float), s, jobs);
    HIPCHECK(hipGetLastError());
    SACHECK((launch_gemm_raw<A_KM, B_KN, EPI_STORE, false>(gp + vt_off, vt_count, vt_tiles, unit, s)));
    for (int b = qblocks - 1; b >= 0; --b) {
      SACHECK((launch_gemm_raw<A_MK, B_KN, EPI_STORE, false>(gp + g1_off[b], n, g1_tiles[b], unit, s)));
      SACHECK((launch_gemm_raw<A_MK, B_KN, EPI_SUB, false, false, 1>(gp + g2_off[b], n, g2_tiles[b], unit, s)));
    }
  }

  // ---- 3. eigendecomposition of T
  static bool attr_set = false;
  if (!attr_set) {
    HIPCHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(tql_sweeps_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                 2 * TRD_MAX_DIM * (int)sizeof(double)));
    HIPCHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(tdc_bisect_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                 2 * TRD_MAX_DIM * (int)sizeof(double)));
    attr_set = true;
  }
  std::vector<int> ql;  // positions in the job table of the factors that take the QL iteration
  if (p->eigh_solver == 3) {
    for (int k = 0; k < n; ++k) ql.push_back(k);
  } else {
    // bisection + inverse iteration, one thread per eigenpair; then rows of X0 <- Z^T Q1^T
    Span span("tridiagonal_eig", s, 0.0, 0, true);
    hipLaunchKernelGGL(tdc_setup_kernel, dim3(n), dim3(256), 0, s, jobs);
    hipLaunchKernelGGL(tdc_bisect_kernel, dim3((d + 255) / 256, n), dim3(256), 2 * (size_t)dpad * sizeof(double), s, jobs);
    const int E = dpad / 4;
    for (int first = 0; first < d; first += E)
      hipLaunchKernelGGL(tdc_invit_kernel, dim3((E + 127) / 128, n), dim3(128), 0, s, jobs, first);
    hipLaunchKernelGGL(tdc_cluster_kernel, dim3(d, n), dim3(64), 0, s, jobs);
    hipLaunchKernelGGL(tdc_verify_kernel, dim3((d + 255) / 256, n), dim3(256), 0, s, jobs);
    HIPCHECK(hipGetLastError());
    int* h_fail = p->h_pinned;
    for (int k = 0; k < n; ++k)
      HIPCHECK(hipMemcpyAsync(h_fail + k, p->t_trd.host[k].fail, sizeof(int), hipMemcpyDeviceToHost, s));
    HIPCHECK(hipStreamSynchronize(s));
    std::vector<int> good;
    for (int k = 0; k < n; ++k) (h_fail[k] ? ql : good).push_back(k);
    if (!good.empty()) {
      const int ng = (int)good.size();
      SACHECK(p->t_trd_gemm.begin(ng));
      SACHECK(p->t_copy.begin(ng));
      int tiles = 0;
      for (int g = 0; g < ng; ++g) {
        const int k = good[g];
        const Factor& f = p->factors[ids[k]];
        const TrdJob& J = p->t_trd.host[k];
        float* out = newton_buf(p, NB_S1, f);
        GemmProblem q{};
        q.A = J.Z; q.lda = ld; q.a_vec = vec_ok(J.Z, ld);
        q.B = J.Y; q.ldb = ld; q.b_vec = vec_ok(J.Y, ld);  // Q1, read as Q1^T
        // to the padded order (Z is zero there and Q1 the identity, so the padding of `out` comes out zero): whole tiles, no guards
        q.C = out; q.ldc = ld; q.M = dpad; q.N = dpad; q.K = dpad;
        q.tiles_m = dpad / BM;
        q.tiles_n = dpad / BN;
        q.tile_begin = tiles;
        tiles += q.tiles_m * q.tiles_n;
        p->t_trd_gemm.host[g] = q;
        Copy2D& C = p->t_copy.host[g];
        std::memset(&C, 0, sizeof(C));
        C.src = out; C.lds_ = ld; C.dst = J.Y; C.ldd = ld; C.rows = d; C.cols = d;
        sweeps_out[ids[k]] = 1;
        not_converged[ids[k]] = 0;
      }
      SACHECK(p->t_trd_gemm.upload(s));
      SACHECK(p->t_copy.upload(s));
      SACHECK((launch_gemm_raw<A_KM, B_NK, EPI_STORE, false>(p->t_trd_gemm.dev, ng, tiles, unit, s)));
      hipLaunchKernelGGL(copy2d_kernel, dim3(64, ng), dim3(256), 0, s, p->t_copy.dev);
      HIPCHECK(hipGetLastError());
    }
  }
  if (!ql.empty()) {
    // implicit QL on T, rotations applied to the rows of Y chunk by chunk
    const int n = (int)ql.size();
    SACHECK(p->t_trd_ql.begin(n));
    for (int k = 0; k < n; ++k) p->t_trd_ql.host[k] = p->t_trd.host[ql[k]];
    SACHECK(p->t_trd_ql.upload(s));
    const TrdJob* jobs = p->t_trd_ql.dev;
    {
      // the QL iteration rotates the rows of Y = Q1^T: transpose Q1 through the (free) G buffer
      SACHECK(p->t_transpose.begin(n));
      SACHECK(p->t_copy.begin(n));
      for (int k = 0; k < n; ++k) {
        const Factor& f = p->factors[ids[ql[k]]];
        const TrdJob& J = p->t_trd_ql.host[k];
        p->t_transpose.host[k] = TransposeJob{J.Y, newton_buf(p, NB_S1, f), d, dpad};
        Copy2D& C = p->t_copy.host[k];
        std::memset(&C, 0, sizeof(C));
        C.src = newton_buf(p, NB_S1, f); C.lds_ = ld; C.dst = J.Y; C.ldd = ld; C.rows = d; C.cols = d;
      }
      SACHECK(p->t_transpose.upload(s));
      SACHECK(p->t_copy.upload(s));
      hipLaunchKernelGGL(trd_transpose_kernel, dim3((d + 31) / 32, (d + 31) / 32, n), dim3(256), 0, s, p->t_transpose.dev);
      hipLaunchKernelGGL(copy2d_kernel, dim3(64, n), dim3(256), 0, s, p->t_copy.dev);
      HIPCHECK(hipGetLastError());
    }
    Span span("tridiagonal_ql", s, 0.0, 0, true);
    hipLaunchKernelGGL(tql_init_kernel, dim3(n), dim3(256), 0, s, jobs);
    HIPCHECK(hipGetLastError());
    const size_t ql_lds = 2 * (size_t)dpad * sizeof(double);
    const long long max_chunks = ((long long)TQL_MAX_ITER * d + TQL_K - 1) / TQL_K + 1;
    std::vector<int> state_host(8 * n);
    bool all_done = false;
    // The rotations of chunk c are applied on a second stream while lane 0 of every factor already chases
    // chunk c + 1; the two log buffers alternate, guarded by events in both directions.
    SACHECK(trd_side_stream(p));
    hipStream_t s2 = p->trd_stream;
    HIPCHECK(hipEventRecord(p->trd_ev[4], s));
    HIPCHECK(hipStreamWaitEvent(s2, p->trd_ev[4], 0));
    long long launched = 0;
    for (long long c = 0; c < max_chunks && !all_done; ++c) {
      const int buf = (int)(c & 1);
      if (c >= 2) HIPCHECK(hipStreamWaitEvent(s, p->trd_ev[2 + buf], 0));  // apply(c - 2) has released this buffer
      hipLaunchKernelGGL(tql_sweeps_kernel, dim3(n), dim3(64), ql_lds, s, jobs, buf, TQL_MAX_ITER * d);
      HIPCHECK(hipEventRecord(p->trd_ev[buf], s));
      HIPCHECK(hipStreamWaitEvent(s2, p->trd_ev[buf], 0));
      hipLaunchKernelGGL(tql_apply_kernel, dim3((d + 255) / 256, n), dim3(256), 0, s2, jobs, buf);
      HIPCHECK(hipEventRecord(p->trd_ev[2 + buf], s2));
      HIPCHECK(hipGetLastError());
      ++launched;
      if ((c & 7) == 7) {
        for (int k = 0; k < n; ++k)
          HIPCHECK(hipMemcpyAsync(state_host.data() + 8 * k, p->t_trd_ql.host[k].state, 6 * sizeof(int), hipMemcpyDeviceToHost, s));
        HIPCHECK(hipStreamSynchronize(s));
        all_done = true;
        for (int k = 0; k < n; ++k)
          if (!state_host[8 * k + 2] && !state_host[8 * k + 3]) all_done = false;
      }
    }
    // join: everything later on s sees the finished Y
    if (launched >= 1) HIPCHECK(hipStreamWaitEvent(s, p->trd_ev[2 + (int)((launched - 1) & 1)], 0));
    if (launched >= 2) HIPCHECK(hipStreamWaitEvent(s, p->trd_ev[2 + (int)((launched - 2) & 1)], 0));
    for (int k = 0; k < n; ++k)
      HIPCHECK(hipMemcpyAsync(state_host.data() + 8 * k, p->t_trd_ql.host[k].state, 6 * sizeof(int), hipMemcpyDeviceToHost, s));
    HIPCHECK(hipStreamSynchronize(s));
    for (int k = 0; k < n; ++k) {
      sweeps_out[ids[ql[k]]] = state_host[8 * k + 4];
      not_converged[ids[ql[k]]] = (state_host[8 * k + 2] && !state_host[8 * k + 3]) ? 0 : 1;
    }
    hipLaunchKernelGGL(tql_finish_kernel, dim3(n), dim3(256), 0, s, jobs);
    HIPCHECK(hipGetLastError());
  }
  return SA_OK;
}

// --------------------------------------------------------------------------------------------
// Batched eigendecomposition root inverse (block Jacobi)
// --------------------------------------------------------------------------------------------

// Frobenius norms of the ridged, bias-corrected factors from the partial sums root_inverse_prologue left
// (the absolute rotation threshold of the Jacobi solver).
static int factor_frobenius_norms(sa_plan* p, const std::vector<int>& todo, hipStream_t s, std::vector<float>* fro) {
  fro->resize(todo.size());
  std::vector<float> partials(p->norm_partials_total);
  HIPCHECK(hipMemcpyAsync(partials.data(), p->f(p->off_norm_partial), partials.size() * sizeof(float), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipStreamSynchronize(s));
  for (size_t i = 0; i < todo.size(); ++i) {
    const Factor& f = p->factors[todo[i]];
    double acc = 0.0;
    for (int c = 0; c < f.norm_chunks; ++c) acc += partials[f.norm_off + c];
    (*fro)[i] = (float)std::sqrt(acc);
  }
  return SA_OK;
}

// Eigendecomposition of the dense matrices in the M0 arrays of the factors `todo` (X0 must hold the identity).
// Block Jacobi for small orders: eigenvalues end up on the diagonal of M0 and eigenvectors in the columns of X0.
// Tridiagonalisation + QL otherwise (via_trd[i] = 1): eigenvalues in a vector, eigenvectors in the rows of X0.
// `fro[k]` is the Frobenius norm of the matrix of todo[k]; active[i] != 0 on return marks a factor that did not converge.
static int eigh_solve(sa_plan* p, const std::vector<int>& todo, const std::vector<float>& fro, int max_sweeps, int32_t* sweeps_out,
                      std::vector<int>& active, std::vector<char>& via_trd, hipStream_t s) {
  const int F = (int)p->factors.size();
  const int n = (int)todo.size();
  // solver per factor: block Jacobi for small orders, tridiagonalisation + QL for the rest
  std::vector<int> jac, jac_pos;            // factor ids / positions in todo
  std::map<int, std::vector<int>> trd_by_d; // order -> factor ids
  for (int k = 0; k < n; ++k) {
    const Factor& f = p->factors[todo[k]];
    if (p->eigh_solver != 1 && (p->eigh_solver >= 2 || f.d >= TRD_MIN_DIM) && f.dpad >= 256 && f.d <= TRD_MAX_DIM)
      trd_by_d[f.d].push_back(todo[k]);
    else { jac.push_back(todo[k]); jac_pos.push_back(k); }
  }
  active.assign(F, 0);
  via_trd.assign(F, 0);

  if (!jac.empty()) {
    const int nj = (int)jac.size();
    // tournament schedules, one per distinct block count
    std::map<int, size_t> sched_off;
    std::vector<int2> sched;
    int max_nb = 0, max_dpad = 0;
    for (int i = 0; i < nj; ++i) {
      const int nb = p->factors[jac[i]].dpad / JB;
      max_nb = std::max(max_nb, nb);
      max_dpad = std::max(max_dpad, p->factors[jac[i]].dpad);
      if (sched_off.count(nb)) continue;
      sched_off[nb] = sched.size();
      const int m = nb - 1;
      for (int r = 0; r < nb - 1; ++r)
        for (int k = 0; k < nb / 2; ++k) {
          int a, b;
          if (k == 0) { a = 0; b = (r % m) + 1; }
          else { a = ((r + k) % m) + 1; b = ((r - k + m) % m) + 1; }
          sched.push_back(make_int2(std::min(a, b), std::max(a, b)));
        }
    }
    SACHECK(p->t_sched.begin(sched.size()));
    std::memcpy(p->t_sched.host, sched.data(), sched.size() * sizeof(int2));
    SACHECK(p->t_sched.upload(s));
    SACHECK(p->t_jacobi.begin(nj));
    int pairs = 0;
    for (int i = 0; i < nj; ++i) {
      const Factor& f = p->factors[jac[i]];
      JacobiFactor& J = p->t_jacobi.host[i];
      std::memset(&J, 0, sizeof(J));
      J.A = newton_buf(p, NB_M0, f);
      J.V = newton_buf(p, NB_X0, f);
      J.U = newton_buf(p, NB_S2, f);
      J.nb = f.dpad / JB;
      J.sched = p->t_sched.dev + sched_off[J.nb];
      J.rotations = p->d_iters + jac[i];
      J.rot_mass = p->d_final_err + jac[i];
      J.active = p->d_active + jac[i];
      J.thr_abs = 1e-9f * fro[jac_pos[i]];
      J.thr_diag = 2.4e-7f * fro[jac_pos[i]];  // 2^-22 ||A||_F: below the eigenvalue resolution of an fp32 matrix
      J.d = f.d; J.dpad = f.dpad;
      J.pair_begin = pairs;
      pairs += J.nb / 2;
    }
    SACHECK(p->t_jacobi.upload(s));
    for (int i : jac) active[i] = 1;
    HIPCHECK(hipMemcpyAsync(p->d_active, active.data(), F * sizeof(int), hipMemcpyHostToDevice, s));
    HIPCHECK(hipStreamSynchronize(s));

    int live = nj;
    for (int sweep = 0; sweep < max_sweeps && live > 0; ++sweep) {
      HIPCHECK(hipMemsetAsync(p->d_iters, 0, F * sizeof(int), s));
      HIPCHECK(hipMemsetAsync(p->d_final_err, 0, F * sizeof(float), s));
      double work = 0.0;
      for (int i = 0; i < nj; ++i)
        if (active[jac[i]]) { const double d = p->factors[jac[i]].dpad; work += 3.0 * 2.0 * d * d * JP * (d / JB - 1); }
      {
        Span span("jacobi", s, work, 3 * (max_nb - 1), sweep == 0);
        for (int r = 0; r < max_nb - 1; ++r) {
          hipLaunchKernelGGL(jacobi_pivot_kernel, dim3(pairs), dim3(256), 0, s, p->t_jacobi.dev, nj, r);
          hipLaunchKernelGGL(jacobi_cols_kernel, dim3(pairs, max_dpad / 128, 2), dim3(256), 0, s, p->t_jacobi.dev, nj, r);
          hipLaunchKernelGGL(jacobi_rows_kernel, dim3(pairs, max_dpad / 128, 1), dim3(256), 0, s, p->t_jacobi.dev, nj, r);
        }
        HIPCHECK(hipGetLastError());
      }
      HIPCHECK(hipMemcpyAsync(p->h_pinned, p->d_iters, F * sizeof(int), hipMemcpyDeviceToHost, s));
      HIPCHECK(hipMemcpyAsync(p->h_pinned + F, p->d_final_err, F * sizeof(float), hipMemcpyDeviceToHost, s));
      HIPCHECK(hipStreamSynchronize(s));
      live = 0;
      const float* mass = reinterpret_cast<const float*>(p->h_pinned + F);
      for (int k = 0; k < nj; ++k) {
        const int i = jac[k];
        if (!active[i]) continue;
        sweeps_out[i] = sweep + 1;
        // converged when the sweep removed less than (5e-7 ||A||_F)^2 of off-diagonal mass
        const double tol = 5e-7 * (double)fro[jac_pos[k]];
        if (p->h_pinned[i] == 0 || (double)mass[i] < tol * tol) active[i] = 0; else ++live;
      }
      HIPCHECK(hipMemcpyAsync(p->d_active, active.data(), F * sizeof(int), hipMemcpyHostToDevice, s));
      HIPCHECK(hipStreamSynchronize(s));
    }
  }
  for (auto& kv : trd_by_d) {
    SACHECK(eigh_tridiagonal(p, kv.second, s, sweeps_out, active.data()));
    for (int i : kv.second) via_trd[i] = 1;
  }

  return SA_OK;
}

static int sa_compute_root_inverses_eigh_wave(sa_plan* p, float bias_correction2, float epsilon, const float* roots,
                                      int32_t stability, float rank_rtol, float rank_atol, int32_t max_sweeps, int32_t* sweeps_out,
                                      int32_t* status_out, void* stream) {
  if (!p || !roots || !sweeps_out || !status_out) return fail(SA_ERR_INVALID, "sa_compute_root_inverses_eigh: NULL argument");
  if (!(bias_correction2 != 0.0f) || max_sweeps < 1) return fail(SA_ERR_INVALID, "bad bias correction or max_sweeps");
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, nullptr, s));
  const int F = (int)p->factors.size();
  if (F == 0) return SA_OK;
  for (int i = 0; i < F; ++i)
    if (!(roots[i] > 0.0f)) return fail(SA_ERR_INVALID, "Root " + std::to_string(roots[i]) + " should be positive!");
  if (stability < 0 || stability > 2) return fail(SA_ERR_INVALID, "stability must be 0, 1 or 2");
  if (stability == 2 && epsilon != 0.0f)
    return fail(SA_ERR_INVALID, "epsilon=" + std::to_string(epsilon) + " should be 0.0 when using pseudo-inverse!");
  const float ridge = (stability == 1) ? epsilon : 0.0f;
  std::vector<int> todo;
  SACHECK(root_inverse_prologue(p, bias_correction2, ridge, sweeps_out, status_out, s, &todo));
  if (todo.empty()) return SA_OK;
  const int n = (int)todo.size();

  std::vector<float> fro;
  SACHECK(factor_frobenius_norms(p, todo, s, &fro));

  // A <- unpack(factor / bc2) + ridge I, V <- I
  SACHECK(p->t_eiginit.begin(n));
  int tiles = 0;
  for (int i = 0; i < n; ++i) {
    const Factor& f = p->factors[todo[i]];
    EigInit& J = p->t_eiginit.host[i];
    std::memset(&J, 0, sizeof(J));
    J.packed = packed32(p, f);
    J.scale = p->scale_of(todo[i]);
    J.A = newton_buf(p, NB_M0, f);
    J.V = newton_buf(p, NB_X0, f);
    J.d = f.d; J.dpad = f.dpad; J.tiles = f.dpad / 64; J.enabled = 1;
    J.tile_begin = tiles;
    tiles += J.tiles * J.tiles;
  }
  SACHECK(p->t_eiginit.upload(s));
  hipLaunchKernelGGL(eig_init_kernel, dim3(tiles), dim3(256), 0, s, p->t_eiginit.dev, n, bias_correction2, ridge);
  HIPCHECK(hipGetLastError());

  std::vector<int> active;
  std::vector<char> via_trd;
  SACHECK(eigh_solve(p, todo, fro, max_sweeps, sweeps_out, active, via_trd, s));

  // X = V diag(f(lambda)) V^T
  SACHECK(p->t_eigfinal.begin(n));
  SACHECK(p->t_rowscale.begin(n));
  p->eig_gemm.clear();
  p->eig_gemm_t.clear();
  int slabs = 0, slabs_t = 0, n_t = 0;
  for (int i = 0; i < n; ++i) {
    const Factor& f = p->factors[todo[i]];
    EigFinal& J = p->t_eigfinal.host[i];
    std::memset(&J, 0, sizeof(J));
    const bool t = via_trd[todo[i]] != 0;
    // Jacobi leaves the eigenvalues on the diagonal of A and the eigenvectors in the columns of V;
    // the tridiagonal path leaves them in a vector (start of the Mp1 array) and in the rows of V
    J.lambda_in = t ? newton_buf(p, NB_M1, f) + trd_diag_offset(f) : newton_buf(p, NB_M0, f);
    J.lambda_stride = t ? 1 : (long long)f.dpad + 1;
    J.V = newton_buf(p, NB_X0, f);
    J.Vs = newton_buf(p, NB_S1, f);
    J.lambda_out = newton_buf(p, NB_MP0, f);
    J.weight_out = newton_buf(p, NB_MP0, f) + f.dpad;
    J.d = f.d; J.dpad = f.dpad;
    J.exponent = -1.0f / roots[todo[i]];
    J.row_begin = slabs;
    J.enabled = 1;
    J.scale_cols = t ? 0 : 1;
    GemmProblem q{};
    q.A = t ? J.V : J.Vs; q.B = t ? J.Vs : J.V; q.C = newton_buf(p, NB_X1, f);
    q.lda = q.ldb = q.ldc = f.dpad;
    q.M = q.N = q.K = f.dpad;
    q.a_vec = q.b_vec = 1;
    if (t) {
      RowScale& R = p->t_rowscale.host[n_t++];
      R.Y = J.V; R.Ys = J.Vs; R.w = J.weight_out; R.dpad = f.dpad; R.row_begin = slabs_t;
      slabs_t += f.dpad / 8;
      p->eig_gemm_t.add(q, false);
    } else {
      p->eig_gemm.add(q, false);
    }
    slabs += f.dpad / 8;
  }
  p->t_rowscale.n = n_t;
  SACHECK(p->t_eigfinal.upload(s));
  SACHECK(p->t_rowscale.upload(s));
  SACHECK(p->eig_gemm.commit(s));
  SACHECK(p->eig_gemm_t.commit(s));
  hipLaunchKernelGGL(eig_weights_kernel, dim3(n), dim3(256), 0, s, p->t_eigfinal.dev, epsilon, stability, rank_rtol, rank_atol);
  hipLaunchKernelGGL(eig_scale_cols_kernel, dim3(slabs), dim3(256), 0, s, p->t_eigfinal.dev, n);
  if (n_t) hipLaunchKernelGGL(eig_scale_rows_kernel, dim3(slabs_t), dim3(256), 0, s, p->t_rowscale.dev, n_t);
  HIPCHECK(hipGetLastError());
  SACHECK((launch_gemm<A_MK, B_NK, EPI_STORE, false, false>(p->eig_gemm, unit_scalars(), s)));    // (V w) V^T
  SACHECK((launch_gemm<A_KM, B_KN, EPI_STORE, false, false>(p->eig_gemm_t, unit_scalars(), s)));  // Y^T (w Y)

  std::vector<const float*> X(n);
  for (int i = 0; i < n; ++i) X[i] = newton_buf(p, NB_X1, p->factors[todo[i]]);
  size_t ok = 0;
  SACHECK(root_inverse_epilogue(p, todo, X, status_out, s, &ok));
  for (size_t i = 0; i < ok; ++i) status_out[todo[i]] = active[todo[i]] ? SA_FACTOR_NOT_CONVERGED : SA_FACTOR_OK;
  return SA_OK;
}

int32_t sa_compute_root_inverses_eigh(sa_plan* p, float bias_correction2, float epsilon, const float* roots, int32_t stability, float rank_rtol, float rank_atol, int32_t max_sweeps, int32_t* sweeps_out, int32_t* status_out, void* stream) {
  if (!p || !status_out) return fail(SA_ERR_INVALID, "sa_compute_root_inverses_eigh: NULL argument");
  return for_each_wave(p, sweeps_out, status_out, static_cast<hipStream_t>(stream), [&](int32_t* it__, int32_t* st__) {
    return sa_compute_root_inverses_eigh_wave(p, bias_correction2, epsilon, roots, stability, rank_rtol, rank_atol, max_sweeps, it__, st__, stream);
  });
}

// --------------------------------------------------------------------------------------------
// Factor matrices in fp64 with an eigendecomposition root inverse: A = factor / bc2 (+ epsilon I) in double,
// (lambda, Q) = eigh(A) to double precision (fp32 solver, then Newton-Schulz and Jacobi in fp64: eigh64.h), the weights of
// matrix_inverse_root_from_eigendecomposition and X = Q diag(w) Q^T in double, cast to the fp32 inverse-root state
// (matrix_functions.py:179-279, 306-366, 725-770; shampoo_preconditioner_list.py:672-678)
// --------------------------------------------------------------------------------------------
static int sa_compute_root_inverses_eigh_f64_wave(sa_plan* p, float bias_correction2, double epsilon, const float* roots,
                                                  int32_t stability, double rank_rtol, double rank_atol, int32_t max_sweeps,
                                                  int32_t* sweeps_out, int32_t* status_out, void* stream) {
  if (!p || !roots || !sweeps_out || !status_out) return fail(SA_ERR_INVALID, "sa_compute_root_inverses_eigh_f64: NULL argument");
  if (!p->factor_f64) return fail(SA_ERR_STATE, "the factor matrices of this plan are fp32");
  if (!(bias_correction2 != 0.0f) || max_sweeps < 1) return fail(SA_ERR_INVALID, "bad bias correction or max_sweeps");
  if (stability < 0 || stability > 2) return fail(SA_ERR_INVALID, "stability must be 0, 1 or 2");
  if (stability == 2 && epsilon != 0.0)
    return fail(SA_ERR_INVALID, "epsilon=" + std::to_string(epsilon) + " should be 0.0 when using pseudo-inverse!");
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, nullptr, s));
  const int F = (int)p->factors.size();
  if (F == 0) return SA_OK;
  std::vector<int> todo;
  for (int i = 0; i < F; ++i) {
    sweeps_out[i] = 0;
    status_out[i] = SA_FACTOR_SKIPPED;
    if (!(roots[i] > 0.0f)) return fail(SA_ERR_INVALID, "Root " + std::to_string(roots[i]) + " should be positive!");
    if (block_active(p, p->factors[i].block) && in_wave(p, i)) todo.push_back(i);
  }
  if (todo.empty()) return SA_OK;
  SACHECK(refresh_inverse_cache(p, s));
  const double bc2 = (double)bias_correction2;
  const double ridge = (stability == 1) ? epsilon : 0.0;
  int* h_bad = p->h_pinned + 3 * F;

  // ---- finiteness and Frobenius norm of the bias-corrected factors (the reference raises at the first bad one)
  {
    SACHECK(p->t_f64.begin(todo.size()));
    for (size_t i = 0; i < todo.size(); ++i) {
      const Factor& f = p->factors[todo[i]];
      Factor64& J = p->t_f64.host[i];
      std::memset(&J, 0, sizeof(J));
      J.packed = reinterpret_cast<const double*>(f.factor);
      J.norm_sq = p->d_norm64 + todo[i];
      J.nonfinite = p->d_flags + todo[i];
      J.ridge = ridge;
      J.d = f.d; J.n = f.dpad;
    }
    SACHECK(p->t_f64.upload(s));
    HIPCHECK(hipMemsetAsync(p->d_flags, 0, F * sizeof(int), s));
    hipLaunchKernelGGL(f64_norm_kernel, dim3((unsigned)todo.size()), dim3(256), 0, s, p->t_f64.dev, bc2);
    HIPCHECK(hipGetLastError());
  }
  std::vector<double> norm_sq(F, 0.0);
  HIPCHECK(hipMemcpyAsync(h_bad, p->d_flags, F * sizeof(int), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipStreamSynchronize(s));
  HIPCHECK(hipMemcpy(norm_sq.data(), p->d_norm64, F * sizeof(double), hipMemcpyDeviceToHost));
  for (size_t i = 0; i < todo.size(); ++i)
    if (h_bad[todo[i]]) { status_out[todo[i]] = SA_FACTOR_INPUT_NONFINITE; todo.resize(i); break; }
  if (todo.empty()) return SA_OK;

  // ---- jobs, ordered by padded order so that the Jacobi launches (whose step count is the order) take contiguous
  // runs of the table.  fp64 arrays 4..7 of the scratch region lie behind everything the fp32 solvers use (fp32 arrays
  // 0..7 = fp64 arrays 0..3); arrays 0..3 serve as fp64 scratch once the fp32 eigenvectors have been taken over.
  const int n = (int)todo.size();
  std::vector<int> ids(todo);
  std::stable_sort(ids.begin(), ids.end(), [&](int a, int b) { return p->factors[a].dpad < p->factors[b].dpad; });
  SACHECK(p->t_eig64.begin(n));
  int nmax = 0;
  for (int k = 0; k < n; ++k) {
    const Factor& f = p->factors[ids[k]];
    Eig64Job& J = p->t_eig64.host[k];
    std::memset(&J, 0, sizeof(J));
    J.packed = reinterpret_cast<const double*>(f.factor);
    J.A = newton_buf64(p, 4, f);
    J.X = newton_buf64(p, 5, f);
    J.T = newton_buf64(p, 6, f);
    J.B = newton_buf64(p, 7, f);
    J.P = newton_buf64(p, 2, f);
    J.cs = newton_buf64(p, 1, f);
    J.lambda = J.cs + f.dpad;
    J.A32 = newton_buf(p, NB_M0, f);
    J.V32 = newton_buf(p, NB_X0, f);
    J.rotations = p->d_iters + ids[k];
    J.nonfinite = p->d_flags + ids[k];
    J.ridge = ridge;
    J.exponent = -1.0 / (double)roots[ids[k]];
    J.d = f.d; J.n = f.dpad;
    nmax = std::max(nmax, f.dpad);
  }
  SACHECK(p->t_eig64.upload(s));
  const unsigned gx = (unsigned)std::min<long long>(((long long)nmax * nmax + 255) / 256, 2048);
  hipLaunchKernelGGL(eig64_init_kernel, dim3(gx, n), dim3(256), 0, s, p->t_eig64.dev, bc2);
  HIPCHECK(hipGetLastError());

  // ---- fp32 eigenvectors of the rounded matrices
  std::vector<float> fro(n);
  for (int k = 0; k < n; ++k) fro[k] = (float)std::sqrt(norm_sq[ids[k]]);
  std::vector<int> active;
  std::vector<char> via_trd;
  std::vector<int32_t> sweeps32(F, 0);
  SACHECK(eigh_solve(p, ids, fro, max_sweeps, sweeps32.data(), active, via_trd, s));
  for (int k = 0; k < n; ++k) p->t_eig64.host[k].rows_are_vectors = via_trd[ids[k]] ? 1 : 0;
  SACHECK(p->t_eig64.wait());
  SACHECK(p->t_eig64.upload(s));
  hipLaunchKernelGGL(eig64_take_vectors_kernel, dim3(gx, n), dim3(256), 0, s, p->t_eig64.dev);
  HIPCHECK(hipGetLastError());

  // ---- fp64 products: tables [G = T X | P = X G | P = A X | B = T P | A = B T]
  sa_plan::GemmTable64* tab = p->n64_pow;
  for (int t = 0; t < 5; ++t) tab[t].clear();
  for (int k = 0; k < n; ++k) {
    const Factor& f = p->factors[ids[k]];
    const Eig64Job& J = p->t_eig64.host[k];
    double* G = newton_buf64(p, 3, f);
    auto prob = [&](const double* A, const double* B, double* C) {
      GemmProblem64 q{};
      q.A = A; q.B = B; q.C = C; q.n = f.dpad; q.d = f.d;
      return q;
    };
    tab[0].add(prob(J.T, J.X, G));
    tab[1].add(prob(J.X, G, J.P));
    tab[2].add(prob(J.A, J.X, J.P));
    tab[3].add(prob(J.T, J.P, J.B));
    tab[4].add(prob(J.B, J.T, J.A));
  }
  for (int t = 0; t < 5; ++t) SACHECK(commit64(tab[t], s));
  SACHECK(p->t_tr64.begin(n));
  for (int k = 0; k < n; ++k) p->t_tr64.host[k] = Transpose64{p->t_eig64.host[k].X, p->t_eig64.host[k].T, p->factors[ids[k]].dpad};
  SACHECK(p->t_tr64.upload(s));
  auto transpose_x = [&]() -> int {
    hipLaunchKernelGGL(transpose64_kernel, dim3(nmax / 32, nmax / 32, n), dim3(256), 0, s, p->t_tr64.dev);
    HIPCHECK(hipGetLastError());
    return SA_OK;
  };
  // two Newton-Schulz steps make X orthogonal to rounding
  for (int it = 0; it < 2; ++it) {
    SACHECK(transpose_x());
    SACHECK(launch_gemm64<EPI64_STORE>(tab[0], 0.0, 0.0, s));
    SACHECK(launch_gemm64<EPI64_STORE>(tab[1], 0.0, 0.0, s));
    hipLaunchKernelGGL(eig64_polar_step_kernel, dim3(gx, n), dim3(256), 0, s, p->t_eig64.dev);
    HIPCHECK(hipGetLastError());
  }
  // B = X^T A X
  SACHECK(transpose_x());
  SACHECK(launch_gemm64<EPI64_STORE>(tab[2], 0.0, 0.0, s));
  SACHECK(launch_gemm64<EPI64_STORE>(tab[3], 0.0, 0.0, s));

  // ---- Jacobi sweeps in fp64, the factors of one padded order together
  std::vector<char> not_converged(F, 0);
  for (int k0 = 0; k0 < n;) {
    const int nn = p->factors[ids[k0]].dpad;
    int k1 = k0;
    while (k1 < n && p->factors[ids[k1]].dpad == nn) ++k1;
    const int m = k1 - k0;
    const Eig64Job* sub = p->t_eig64.dev + k0;
    bool done = false;
    int sweep = 0;
    for (; sweep < max_sweeps && !done; ++sweep) {
      HIPCHECK(hipMemsetAsync(p->d_iters, 0, F * sizeof(int), s));
      for (int r = 0; r < nn - 1; ++r) {
        hipLaunchKernelGGL(eig64_rotations_kernel, dim3((nn / 2 + 255) / 256, m), dim3(256), 0, s, sub, r);
        hipLaunchKernelGGL(eig64_apply_kernel, dim3((nn / 2 + 255) / 256, nn / 2 + nn, m), dim3(256), 0, s, sub, r);
      }
      HIPCHECK(hipGetLastError());
      HIPCHECK(hipMemcpyAsync(p->h_pinned, p->d_iters, F * sizeof(int), hipMemcpyDeviceToHost, s));
      HIPCHECK(hipStreamSynchronize(s));
      done = true;
      for (int k = k0; k < k1; ++k)
        if (p->h_pinned[ids[k]] != 0) done = false;
    }
    for (int k = k0; k < k1; ++k) {
      sweeps_out[ids[k]] = sweep;
      not_converged[ids[k]] = done ? 0 : 1;
    }
    k0 = k1;
  }

  // ---- weights, X diag(w) X^T, cast and commit
  HIPCHECK(hipMemsetAsync(p->d_flags, 0, F * sizeof(int), s));
  hipLaunchKernelGGL(eig64_weights_kernel, dim3(n), dim3(256), 0, s, p->t_eig64.dev, epsilon, stability, rank_rtol, rank_atol);
  hipLaunchKernelGGL(eig64_scale_columns_kernel, dim3(gx, n), dim3(256), 0, s, p->t_eig64.dev);
  HIPCHECK(hipGetLastError());
  SACHECK(transpose_x());
  SACHECK(launch_gemm64<EPI64_STORE>(tab[4], 0.0, 0.0, s));
  auto run_commit = [&](const std::vector<int>& which, int check_only) -> int {
    SACHECK(p->t_f64.begin(which.size()));
    int nm = 0;
    for (size_t i = 0; i < which.size(); ++i) {
      const Factor& f = p->factors[which[i]];
      Factor64& J = p->t_f64.host[i];
      std::memset(&J, 0, sizeof(J));
      J.result = newton_buf64(p, 4, f);
      J.inv_packed = f.inv;
      J.inv_dense = p->f(p->off_inv_dense) + f.dense_off;
      J.nonfinite = p->d_flags + which[i];
      J.d = f.d; J.n = f.dpad;
      nm = std::max(nm, f.dpad);
    }
    SACHECK(p->t_f64.upload(s));
    const unsigned g2 = (unsigned)std::min<long long>(((long long)nm * nm + 255) / 256, 2048);
    hipLaunchKernelGGL(f64_commit_kernel, dim3(g2, (unsigned)which.size()), dim3(256), 0, s, p->t_f64.dev, check_only);
    HIPCHECK(hipGetLastError());
    return SA_OK;
  };
  SACHECK(run_commit(todo, 1));
  HIPCHECK(hipMemcpyAsync(h_bad, p->d_flags, F * sizeof(int), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipStreamSynchronize(s));
  std::vector<int> good;
  for (int i : todo) {
    if (h_bad[i]) { status_out[i] = SA_FACTOR_RESULT_NONFINITE; break; }
    good.push_back(i);
    status_out[i] = (not_converged[i] || active[i]) ? SA_FACTOR_NOT_CONVERGED : SA_FACTOR_OK;
  }
  if (!good.empty()) {
    SACHECK(run_commit(good, 0));
    HIPCHECK(hipStreamSynchronize(s));
  }
  return SA_OK;
}

int32_t sa_compute_root_inverses_eigh_f64(sa_plan* p, float bias_correction2, double epsilon, const float* roots, int32_t stability,
                                          double rank_rtol, double rank_atol, int32_t max_sweeps, int32_t* sweeps_out,
                                          int32_t* status_out, void* stream) {
  if (!p || !status_out) return fail(SA_ERR_INVALID, "sa_compute_root_inverses_eigh_f64: NULL argument");
  return for_each_wave(p, sweeps_out, status_out, static_cast<hipStream_t>(stream), [&](int32_t* it__, int32_t* st__) {
    return sa_compute_root_inverses_eigh_f64_wave(p, bias_correction2, epsilon, roots, stability, rank_rtol, rank_atol, max_sweeps,
                                                  it__, st__, stream);
  });
}

// --------------------------------------------------------------------------------------------
// Eigenvalue-corrected Shampoo (SOAP)
// --------------------------------------------------------------------------------------------

// Eigenbasis refresh of eigenvalue-corrected Shampoo through a full eigendecomposition
// (EighEigendecompositionConfig, matrix_functions.py:725-770 and :885-900): eigenvectors in ascending order of
// their eigenvalues replace the stored basis.  With tolerance != 0 a factor whose current basis already satisfies
// ||B - diag B||_F <= tolerance ||B||_F, B = Q^T A Q, keeps it.
static int sa_refresh_eigenbases_eigh_wave(sa_plan* p, float bias_correction2, float epsilon, float tolerance, int32_t max_sweeps,
                                   int32_t* sweeps_out, int32_t* status_out, void* stream) {
  if (!p || !sweeps_out || !status_out) return fail(SA_ERR_INVALID, "sa_refresh_eigenbases_eigh: NULL argument");
  if (p->factors.empty()) return SA_OK;  // nothing is preconditioned
  if (!p->has_eigvec) return fail(SA_ERR_STATE, "plan has no eigenvector state");
  if (!(bias_correction2 != 0.0f) || max_sweeps < 1) return fail(SA_ERR_INVALID, "bad bias correction or max_sweeps");
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, nullptr, s));
  const int F = (int)p->factors.size();
  if (F == 0) return SA_OK;
  p->eig_source.assign(F, sa_plan::EigSource{});
  p->rotm_version = -1;  // the eigenbases change
  std::vector<int> todo;
  SACHECK(root_inverse_prologue(p, bias_correction2, epsilon, sweeps_out, status_out, s, &todo));
  if (todo.empty()) return SA_OK;

  auto init_dense = [&](const std::vector<int>& ids) -> int {  // M0 <- unpack(factor / bc2) + eps I, X0 <- I
    SACHECK(p->t_eiginit.begin(ids.size()));
    int tiles = 0;
    for (size_t i = 0; i < ids.size(); ++i) {
      const Factor& f = p->factors[ids[i]];
      EigInit& J = p->t_eiginit.host[i];
      std::memset(&J, 0, sizeof(J));
      J.packed = packed32(p, f); J.scale = p->scale_of(ids[i]); J.A = newton_buf(p, NB_M0, f); J.V = newton_buf(p, NB_X0, f);
      J.d = f.d; J.dpad = f.dpad; J.tiles = f.dpad / 64; J.enabled = 1; J.tile_begin = tiles;
      tiles += J.tiles * J.tiles;
    }
    SACHECK(p->t_eiginit.upload(s));
    hipLaunchKernelGGL(eig_init_kernel, dim3(tiles), dim3(256), 0, s, p->t_eiginit.dev, (int)ids.size(), bias_correction2, epsilon);
    HIPCHECK(hipGetLastError());
    return SA_OK;
  };
  SACHECK(init_dense(todo));

  std::vector<int> solve = todo;
  if (tolerance != 0.0f) {
    // B = Q^T (A Q) with the stored basis: X1 <- Q (padded), M1 <- A Q, S1 <- Q^T M1
    const int n = (int)todo.size();
    SACHECK(p->t_copy.begin(n));
    SACHECK(p->t_normpair.begin(n));
    p->qr_aq.clear();
    p->qr_b.clear();
    for (int k = 0; k < n; ++k) {
      const Factor& f = p->factors[todo[k]];
      Copy2D& C = p->t_copy.host[k];
      std::memset(&C, 0, sizeof(C));
      C.src = f.eigvec; C.lds_ = f.d; C.dst = newton_buf(p, NB_X1, f); C.ldd = f.dpad; C.rows = f.d; C.cols = f.d;
      GemmProblem q{};
      q.A = newton_buf(p, NB_M0, f); q.lda = f.dpad; q.a_vec = 1;
      q.B = newton_buf(p, NB_X1, f); q.ldb = f.dpad; q.b_vec = 1;
      q.C = newton_buf(p, NB_M1, f); q.ldc = f.dpad; q.M = q.N = q.K = f.d;
      p->qr_aq.add(q, false);
      GemmProblem b{};
      b.A = newton_buf(p, NB_X1, f); b.lda = f.dpad; b.a_vec = 1;
      b.B = newton_buf(p, NB_M1, f); b.ldb = f.dpad; b.b_vec = 1;
      b.C = newton_buf(p, NB_S1, f); b.ldc = f.dpad; b.M = b.N = b.K = f.d;
      p->qr_b.add(b, false);
      NormPair& J = p->t_normpair.host[k];
      J.B = newton_buf(p, NB_S1, f); J.ldb = f.dpad; J.d = f.d;
      J.out_all = p->d_final_err + todo[k];
      J.out_diag = reinterpret_cast<float*>(p->d_err) + todo[k];
    }
    SACHECK(p->t_copy.upload(s));
    SACHECK(p->t_normpair.upload(s));
    SACHECK(p->qr_aq.commit(s));
    SACHECK(p->qr_b.commit(s));
    hipLaunchKernelGGL(copy2d_kernel, dim3(64, n), dim3(256), 0, s, p->t_copy.dev);
    HIPCHECK(hipGetLastError());
    SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_STORE>(p->qr_aq, unit_scalars(), s)));
    SACHECK((launch_gemm_auto<A_KM, B_KN, EPI_STORE>(p->qr_b, unit_scalars(), s)));
    hipLaunchKernelGGL(diag_off_norm_kernel, dim3(n), dim3(FACTOR_PASS_THREADS), 0, s, p->t_normpair.dev);
    HIPCHECK(hipGetLastError());
    HIPCHECK(hipMemcpyAsync(p->h_pinned, p->d_final_err, F * sizeof(float), hipMemcpyDeviceToHost, s));
    HIPCHECK(hipMemcpyAsync(p->h_pinned + F, p->d_err, F * sizeof(float), hipMemcpyDeviceToHost, s));
    HIPCHECK(hipStreamSynchronize(s));
    const float* h_all = reinterpret_cast<const float*>(p->h_pinned);
    const float* h_diag = reinterpret_cast<const float*>(p->h_pinned + F);
    solve.clear();
    for (int i : todo) {
      const float norm = std::sqrt(h_all[i]), dnorm = std::sqrt(h_diag[i]);
      const float off = std::sqrt(norm * norm - dnorm * dnorm);
      if (off <= tolerance * norm) {
        status_out[i] = SA_FACTOR_OK;  // the stored basis stays; its eigenvalue estimates are diag(Q^T A Q)
        const Factor& f = p->factors[i];
        p->eig_source[i] = sa_plan::EigSource{newton_buf(p, NB_S1, f), (long long)f.dpad + 1, nullptr};
      } else {
        solve.push_back(i);
      }
    }
    HIPCHECK(hipMemsetAsync(p->d_err, 0, F * sizeof(int), s));
    if (solve.empty()) return SA_OK;
  }

  const int n = (int)solve.size();
  std::vector<float> fro_all, fro(n);
  SACHECK(factor_frobenius_norms(p, todo, s, &fro_all));
  for (int k = 0; k < n; ++k)
    fro[k] = fro_all[std::find(todo.begin(), todo.end(), solve[k]) - todo.begin()];
  std::vector<int> active;
  std::vector<char> via_trd;
  SACHECK(eigh_solve(p, solve, fro, max_sweeps, sweeps_out, active, via_trd, s));

  // ascending order, sorted eigenvectors (columns) -> S1, finiteness, then into the state
  SACHECK(p->t_rank.begin(n));
  SACHECK(p->t_copy.begin(n));
  SACHECK(p->t_rows2cols.begin(n));
  SACHECK(p->t_normjobs.begin(n));
  int n_cols = 0, n_rows = 0, chunks = 0, dmax = 0;
  for (int k = 0; k < n; ++k) {
    const Factor& f = p->factors[solve[k]];
    const bool t = via_trd[solve[k]] != 0;
    dmax = std::max(dmax, f.d);
    RankJob& R = p->t_rank.host[k];
    R.lambda_in = t ? newton_buf(p, NB_M1, f) + trd_diag_offset(f) : newton_buf(p, NB_M0, f);
    R.lambda_stride = t ? 1 : (long long)f.dpad + 1;
    R.order = reinterpret_cast<int*>(newton_buf(p, NB_MP0, f));
    R.d = f.d;
    p->eig_source[solve[k]] = sa_plan::EigSource{R.lambda_in, R.lambda_stride, R.order};
    if (t) {
      RowsToCols& C = p->t_rows2cols.host[n_rows++];
      C.src = newton_buf(p, NB_X0, f); C.lds_ = f.dpad; C.dst = newton_buf(p, NB_S1, f); C.ldd = f.dpad; C.order = R.order; C.d = f.d;
    } else {
      Copy2D& C = p->t_copy.host[n_cols++];
      std::memset(&C, 0, sizeof(C));
      C.src = newton_buf(p, NB_X0, f); C.lds_ = f.dpad; C.dst = newton_buf(p, NB_S1, f); C.ldd = f.dpad;
      C.rows = f.d; C.cols = f.d; C.perm = R.order;
    }
    NormJob& J = p->t_normjobs.host[k];
    std::memset(&J, 0, sizeof(J));
    J.src = newton_buf(p, NB_S1, f); J.nonfinite = p->d_flags + solve[k];
    J.d = f.d; J.dpad = f.dpad; J.dense = 1; J.chunk_begin = chunks;
    J.n_chunks = (int)(((long long)f.d * f.d + NORM_CHUNK - 1) / NORM_CHUNK); J.enabled = 1;
    chunks += J.n_chunks;
  }
  p->t_copy.n = n_cols;
  p->t_rows2cols.n = n_rows;
  SACHECK(p->t_rank.upload(s));
  SACHECK(p->t_copy.upload(s));
  SACHECK(p->t_rows2cols.upload(s));
  SACHECK(p->t_normjobs.upload(s));
  HIPCHECK(hipMemsetAsync(p->d_flags, 0, F * sizeof(int), s));
  hipLaunchKernelGGL(eig_rank_kernel, dim3(n), dim3(256), 0, s, p->t_rank.dev);
  if (n_cols) hipLaunchKernelGGL(copy2d_kernel, dim3(64, n_cols), dim3(256), 0, s, p->t_copy.dev);
  if (n_rows) hipLaunchKernelGGL(rows_to_sorted_cols_kernel, dim3((dmax + 31) / 32, (dmax + 31) / 32, n_rows), dim3(256), 0, s, p->t_rows2cols.dev);
  hipLaunchKernelGGL((factor_norm_kernel<true>), dim3(chunks), dim3(256), 0, s, p->t_normjobs.dev, n, 1.0f, 0.0f);
  HIPCHECK(hipGetLastError());
  int* h_bad = p->h_pinned + 3 * F;
  HIPCHECK(hipMemcpyAsync(h_bad, p->d_flags, F * sizeof(int), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipStreamSynchronize(s));
  int ok = n;
  for (int k = 0; k < n; ++k)
    if (k < ok && h_bad[solve[k]]) { status_out[solve[k]] = SA_FACTOR_RESULT_NONFINITE; ok = k; }
  if (ok > 0) {
    SACHECK(p->t_copy.begin(ok));
    for (int k = 0; k < ok; ++k) {
      const Factor& f = p->factors[solve[k]];
      Copy2D& C = p->t_copy.host[k];
      std::memset(&C, 0, sizeof(C));
      C.src = newton_buf(p, NB_S1, f); C.lds_ = f.dpad; C.dst = f.eigvec; C.ldd = f.d; C.rows = f.d; C.cols = f.d;
      status_out[solve[k]] = active[solve[k]] ? SA_FACTOR_NOT_CONVERGED : SA_FACTOR_OK;
    }
    SACHECK(p->t_copy.upload(s));
    hipLaunchKernelGGL(copy2d_kernel, dim3(64, ok), dim3(256), 0, s, p->t_copy.dev);
    HIPCHECK(hipGetLastError());
    HIPCHECK(hipStreamSynchronize(s));
  }
  return SA_OK;
}

int32_t sa_refresh_eigenbases_eigh(sa_plan* p, float bias_correction2, float epsilon, float tolerance, int32_t max_sweeps, int32_t* sweeps_out, int32_t* status_out, void* stream) {
  if (!p || !status_out) return fail(SA_ERR_INVALID, "sa_refresh_eigenbases_eigh: NULL argument");
  return for_each_wave(p, sweeps_out, status_out, static_cast<hipStream_t>(stream), [&](int32_t* it__, int32_t* st__) {
    return sa_refresh_eigenbases_eigh_wave(p, bias_correction2, epsilon, tolerance, max_sweeps, it__, st__, stream);
  });
}

// Inverse roots of eigendecomposed Shampoo from the stored eigendecompositions: X = Q diag(w) Q^T with the weights
// of matrix_inverse_root_from_eigendecomposition (matrix_functions.py:179-279), the same post-processing as the eigh
// root inverse.  The reference forms these products in every step (shampoo_preconditioner_list.py:1793-1832); they
// change only when (Q, lambda) change, so they are formed once per amortized computation (and after a checkpoint
// load) and kept like the inverse roots of root-inverse Shampoo.
static int sa_compute_root_inverses_from_eigendecomposition_wave(sa_plan* p, const float* const* eigenvalues, float epsilon,
                                                         const float* roots, int32_t stability, float rank_rtol, float rank_atol,
                                                         int32_t* status_out, void* stream) {
  if (!p || !eigenvalues || !roots || !status_out)
    return fail(SA_ERR_INVALID, "sa_compute_root_inverses_from_eigendecomposition: NULL argument");
  if (p->factors.empty()) return SA_OK;  // nothing is preconditioned
  if (!p->has_eigvec || p->eigenvalue_corrected) return fail(SA_ERR_STATE, "plan is not an eigendecomposed-Shampoo plan");
  if (stability < 0 || stability > 2) return fail(SA_ERR_INVALID, "stability must be 0, 1 or 2");
  if (stability == 2 && epsilon != 0.0f)
    return fail(SA_ERR_INVALID, "epsilon=" + std::to_string(epsilon) + " should be 0.0 when using pseudo-inverse!");
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, nullptr, s));
  const int F = (int)p->factors.size();
  std::vector<int> todo;
  for (int i = 0; i < F; ++i) {
    status_out[i] = SA_FACTOR_SKIPPED;
    const Factor& f = p->factors[i];
    if (!block_active(p, f.block) || !in_wave(p, i)) continue;
    if (!f.eigvec || !f.inv) return fail(SA_ERR_STATE, "factor " + std::to_string(i) + " has no eigenvector or inverse-root storage");
    if (!eigenvalues[i]) return fail(SA_ERR_INVALID, "eigenvalues[" + std::to_string(i) + "] is NULL");
    if (!(roots[i] > 0.0f)) return fail(SA_ERR_INVALID, "Root " + std::to_string(roots[i]) + " should be positive!");
    todo.push_back(i);
  }
  if (todo.empty()) return SA_OK;
  // factors that are not recomputed below must keep a valid dense copy of their stored inverse
  SACHECK(refresh_inverse_cache(p, s));
  const int n = (int)todo.size();
  SACHECK(p->t_copy.begin(n));
  SACHECK(p->t_eigfinal.begin(n));
  p->eig_gemm.clear();
  int slabs = 0;
  for (int k = 0; k < n; ++k) {
    const Factor& f = p->factors[todo[k]];
    float* V = newton_buf(p, NB_X0, f);
    // zero padded copy of Q (the state keeps it d x d)
    HIPCHECK(hipMemsetAsync(V, 0, sizeof(float) * (size_t)f.dpad * f.dpad, s));
    Copy2D& C = p->t_copy.host[k];
    std::memset(&C, 0, sizeof(C));
    C.src = f.eigvec; C.lds_ = f.d; C.dst = V; C.ldd = f.dpad; C.rows = f.d; C.cols = f.d;
    EigFinal& J = p->t_eigfinal.host[k];
    std::memset(&J, 0, sizeof(J));
    J.lambda_in = eigenvalues[todo[k]];
    J.lambda_stride = 1;
    J.V = V;
    J.Vs = newton_buf(p, NB_S1, f);
    J.lambda_out = newton_buf(p, NB_MP0, f);
    J.weight_out = newton_buf(p, NB_MP0, f) + f.dpad;
    J.d = f.d; J.dpad = f.dpad;
    J.exponent = -1.0f / roots[todo[k]];
    J.row_begin = slabs;
    J.enabled = 1;
    J.scale_cols = 1;
    slabs += f.dpad / 8;
    GemmProblem q{};
    q.A = J.Vs; q.B = J.V; q.C = newton_buf(p, NB_X1, f);
    q.lda = q.ldb = q.ldc = f.dpad;
    q.M = q.N = q.K = f.dpad;
    q.a_vec = q.b_vec = 1;
    p->eig_gemm.add(q, false);
  }
  SACHECK(p->t_copy.upload(s));
  SACHECK(p->t_eigfinal.upload(s));
  SACHECK(p->eig_gemm.commit(s));
  hipLaunchKernelGGL(copy2d_kernel, dim3(64, n), dim3(256), 0, s, p->t_copy.dev);
  hipLaunchKernelGGL(eig_weights_kernel, dim3(n), dim3(256), 0, s, p->t_eigfinal.dev, epsilon, stability, rank_rtol, rank_atol);
  hipLaunchKernelGGL(eig_scale_cols_kernel, dim3(slabs), dim3(256), 0, s, p->t_eigfinal.dev, n);
  HIPCHECK(hipGetLastError());
  SACHECK((launch_gemm<A_MK, B_NK, EPI_STORE, false, false>(p->eig_gemm, unit_scalars(), s)));  // (Q w) Q^T
  std::vector<const float*> X(n);
  for (int k = 0; k < n; ++k) X[k] = newton_buf(p, NB_X1, p->factors[todo[k]]);
  size_t ok = 0;
  SACHECK(root_inverse_epilogue(p, todo, X, status_out, s, &ok));
  for (size_t i = 0; i < ok; ++i) status_out[todo[i]] = SA_FACTOR_OK;
  return SA_OK;
}

int32_t sa_compute_root_inverses_from_eigendecomposition(sa_plan* p, const float* const* eigenvalues, float epsilon, const float* roots, int32_t stability,
                                                         float rank_rtol, float rank_atol, int32_t* status_out, void* stream) {
  if (!p || !status_out) return fail(SA_ERR_INVALID, "sa_compute_root_inverses_from_eigendecomposition: NULL argument");
  return for_each_wave(p, nullptr, status_out, static_cast<hipStream_t>(stream), [&](int32_t*, int32_t* st__) {
    return sa_compute_root_inverses_from_eigendecomposition_wave(p, eigenvalues, epsilon, roots, stability, rank_rtol, rank_atol, st__, stream);
  });
}

int32_t sa_update_corrected_eigenvalues(sa_plan* p, float beta2, float weighting_factor, void* stream) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  if (!p->eigenvalue_corrected) return fail(SA_ERR_STATE, "plan has no eigenvector state");
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, nullptr, s));
  GemmScalars sc = unit_scalars();
  sc.alpha = weighting_factor;
  sc.beta = beta2;
  double flops = 0.0;
  for (const GemmTable* g : {&p->ec_stat1, &p->ec_stat2, &p->ec_stat_l, &p->ec_stat_r})
    for (const GemmProblem& q : g->build) flops += 2.0 * q.M * q.N * q.K;
  Span span("eigenbasis_rotation", s, flops, 4, true);
  SACHECK((launch_gemm_auto<A_KM, B_KN, EPI_STORE>(p->ec_stat1, unit_scalars(), s)));
  SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_SQ_EMA>(p->ec_stat2, sc, s)));
  SACHECK((launch_gemm_auto<A_KM, B_KN, EPI_SQ_EMA>(p->ec_stat_l, sc, s)));
  SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_SQ_EMA>(p->ec_stat_r, sc, s)));
  if (p->has_order3 && p->t_chunks.n) {
    hipLaunchKernelGGL(gather3_kernel, dim3((unsigned)p->t_chunks.n), dim3(EW_THREADS), 0, s, p->t_blocks.dev, p->t_chunks.dev, 2);
    HIPCHECK(hipGetLastError());
    SACHECK(launch_e3_chain<EPI_SQ_EMA>(p, 0, unit_scalars(), sc, 1.0f, s));
  }
  return SA_OK;
}

// Preconditioning of eigenvalue-corrected blocks.  rotated_ready: the blocks with both eigenbases already hold their
// divided, rotated filtered gradient (the fused statistic launch wrote it), so only the rotation back is left for them.
static int precondition_eigenvalue_corrected(sa_plan* p, const sa_step_scalars* sc, float bias_correction2, float epsilon,
                                             float root, bool rotated_ready, hipStream_t s) {
  double flops = 0.0;
  for (const GemmTable* g : {&p->ec_p1, &p->ec_p1d, &p->ec_p2, &p->ec_p2d, &p->ec_p3, &p->ec_p3n, &p->ec_p4, &p->ec_p4n}) {
    if (rotated_ready && (g == &p->ec_p1 || g == &p->ec_p2)) continue;
    for (const GemmProblem& q : g->build) flops += 2.0 * q.M * q.N * q.K;
  }
  {
    Span span("precondition_gemm", s, flops, rotated_ready ? 6 : 8, true);
    GemmScalars u = unit_scalars();
    GemmScalars bdiv = u; bdiv.b_div = sc->bias_correction1;
    GemmScalars den = u; den.div = bias_correction2; den.pow_exp = 1.0f / root; den.eps = epsilon;
    GemmScalars den_b = den; den_b.b_div = sc->bias_correction1;
    GemmScalars den_a = den; den_a.a_div = sc->bias_correction1;
    GemmScalars den_seed = den; den_seed.mom_div = sc->bias_correction1;  // the product is Q_L^T (m / bc1) Q_R
    if (!rotated_ready) {
      SACHECK((launch_gemm_auto<A_KM, B_KN, EPI_STORE>(p->ec_p1, bdiv, s)));
      SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_DIVPOW>(p->ec_p2, den_seed, s)));
      if (p->table_mode == 1) p->rotm_version = p->m_version;
    }
    SACHECK((launch_gemm_auto<A_KM, B_KN, EPI_DIVPOW>(p->ec_p1d, den_b, s)));
    SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_DIVPOW>(p->ec_p2d, den_a, s)));
    SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_STORE>(p->ec_p3, u, s)));
    SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_STORE_SQNORM>(p->ec_p3n, u, s)));
    SACHECK((launch_gemm_auto<A_MK, B_NK, EPI_STORE_SQNORM>(p->ec_p4, u, s)));
    SACHECK((launch_gemm_auto<A_MK, B_NK, EPI_STORE_SQNORM>(p->ec_p4n, u, s)));
    if (p->has_order3 && p->t_chunks.n) {
      if (p->table_mode == 0) {
        hipLaunchKernelGGL(gather3_kernel, dim3((unsigned)p->t_chunks.n), dim3(EW_THREADS), 0, s, p->t_blocks.dev, p->t_chunks.dev, 1);
        HIPCHECK(hipGetLastError());
      }
      SACHECK(launch_e3_chain<EPI_DIVPOW>(p, 1, u, den, sc->bias_correction1, s));
      SACHECK(launch_e3_chain<EPI_STORE_SQNORM>(p, 2, u, u, 1.0f, s));
    }
  }
  if (p->n_active_blocks) {
    hipLaunchKernelGGL(reduce_norms_kernel, dim3(p->n_active_blocks), dim3(EW_THREADS), 0, s, p->t_blocks.dev,
                       p->t_active_blocks.dev, p->n_blocks, p->f(p->off_graft_partial), p->f(p->off_ghat_partial),
                       p->f(p->off_ptile_partial), p->f(p->off_norms));
    HIPCHECK(hipGetLastError());
  }
  return SA_OK;
}

int32_t sa_precondition_eigenvalue_corrected(sa_plan* p, const sa_step_scalars* sc, float bias_correction2, float epsilon,
                                             float root, void* stream) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  if (!p->eigenvalue_corrected) return fail(SA_ERR_STATE, "plan has no eigenvector state");
  if (!(root > 0.0f) || !(bias_correction2 != 0.0f)) return fail(SA_ERR_INVALID, "bad root or bias correction");
  SACHECK(validate_scalars(p, sc));
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, sc, s));
  return precondition_eigenvalue_corrected(p, sc, bias_correction2, epsilon, root, false, s);
}

int32_t sa_update_and_precondition_eigenvalue_corrected(sa_plan* p, const sa_step_scalars* sc, float beta2, float weighting_factor,
                                                        float bias_correction2, float epsilon, float root, void* stream) {
  if (!p) return fail(SA_ERR_INVALID, "NULL plan");
  if (!p->eigenvalue_corrected) return fail(SA_ERR_STATE, "plan has no eigenvector state");
  if (!(root > 0.0f) || !(bias_correction2 != 0.0f)) return fail(SA_ERR_INVALID, "bad root or bias correction");
  SACHECK(validate_scalars(p, sc));
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, sc, s));
  if (p->table_mode == 2)
    return fail(SA_ERR_UNSUPPORTED, "beta3 != beta1: call sa_update_corrected_eigenvalues before the prologue and "
                                    "sa_precondition_eigenvalue_corrected after it");
  // The rotated gradient of the statistic is also what the filtered gradient needs: with beta1 = 0 it is the
  // numerator itself, otherwise Q_L^T m Q_R follows it by m's own moving average as long as the stored copy belongs to
  // the filtered gradient of the previous step in these bases.
  const bool fused = p->table_mode == 0 || (p->table_mode == 1 && p->rotm_version >= 0 && p->rotm_version == p->m_version - 1);
  if (!fused) {
    SACHECK(sa_update_corrected_eigenvalues(p, beta2, weighting_factor, stream));
    return precondition_eigenvalue_corrected(p, sc, bias_correction2, epsilon, root, false, s);
  }
  GemmScalars st = unit_scalars();
  st.alpha = weighting_factor;
  st.beta = beta2;
  GemmScalars fu = st;
  fu.div = bias_correction2; fu.pow_exp = 1.0f / root; fu.eps = epsilon;
  fu.mom_w = sc->lerp_weight1; fu.mom_div = sc->bias_correction1;
  double flops = 0.0;
  for (const GemmTable* g : {&p->ec_stat1, &p->ec_stat2, &p->ec_stat_l, &p->ec_stat_r})
    for (const GemmProblem& q : g->build) flops += 2.0 * q.M * q.N * q.K;
  {
    Span span("eigenbasis_rotation", s, flops, 4, true);
    SACHECK((launch_gemm_auto<A_KM, B_KN, EPI_STORE>(p->ec_stat1, unit_scalars(), s)));
    SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_EC_FUSED>(p->ec_stat2, fu, s)));
    SACHECK((launch_gemm_auto<A_KM, B_KN, EPI_SQ_EMA>(p->ec_stat_l, st, s)));
    SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_SQ_EMA>(p->ec_stat_r, st, s)));
    if (p->has_order3 && p->t_chunks.n) {
      hipLaunchKernelGGL(gather3_kernel, dim3((unsigned)p->t_chunks.n), dim3(EW_THREADS), 0, s, p->t_blocks.dev, p->t_chunks.dev, 2);
      HIPCHECK(hipGetLastError());
      SACHECK(launch_e3_chain<EPI_SQ_EMA>(p, 0, unit_scalars(), st, 1.0f, s));
    }
  }
  if (p->table_mode == 1) p->rotm_version = p->m_version;
  ++p->shared_rotation_steps;
  return precondition_eigenvalue_corrected(p, sc, bias_correction2, epsilon, root, true, s);
}

// Blocked Householder QR of B (NB_X0) for the active factors; the reflectors are applied from the right to
// Qacc (NB_X1):  Qacc <- Qacc H_1 H_2 ... H_d.  Two levels of blocking: LDS-resident panels inside outer blocks.
static int qr_accumulate(sa_plan* p, const std::vector<int>& ids, hipStream_t s) {
  const int n = (int)ids.size();
  int dmax = 0, dpad_min = 1 << 30;
  for (int i : ids) {
    dmax = std::max(dmax, p->factors[i].d);
    dpad_min = std::min(dpad_min, p->factors[i].dpad);
  }
  // panels of up to 1024 rows are factored in registers (32 columns wide), taller ones in LDS (narrower)
  const bool in_registers = dmax <= QR_THREADS;
  const int lds_floats = 34816;  // 136 KB for the panel, the rest of the 160 KB holds the small arrays
  const int ip = in_registers ? QR_MAX_PANEL : std::min(QR_MAX_PANEL, lds_floats / dmax - 1);  // panel width
  if (ip < 1) return fail(SA_ERR_UNSUPPORTED, "QR refresh: factor dimension too large for an LDS resident panel");
  static bool attr_set = false;
  if (!attr_set) {
    HIPCHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(qr_panel_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                 lds_floats * (int)sizeof(float)));
    attr_set = true;
  }
  // Outer blocks pay off where the trailing matrix is large; their scratch (below) needs dpad >= 512.
  const int OB = dpad_min >= 512 ? QR_OUTER : ip;
  // scratch of a factor.  NB_S1: V (dpad x OB) | T (OB x OB) | S (OB x 32) | X (OB x 32).
  //                       NB_S2: W (OB x dpad) | W2 (OB x dpad), later Z (d x OB) | Z2 (d x OB) in the same place.
  auto mk = [&](int i, const float* A, long long lda, const float* Bm, long long ldb, float* C, long long ldc, int M, int N, int K) {
    GemmProblem q{};
    q.A = A; q.lda = lda; q.a_vec = vec_ok(A, lda);
    q.B = Bm; q.ldb = ldb; q.b_vec = vec_ok(Bm, ldb);
    q.C = C; q.ldc = ldc; q.M = M; q.N = N; q.K = K;
    q.active = p->d_active + i;
    return q;
  };
  const GemmScalars u = unit_scalars();
  GemmScalars neg = u;
  neg.a_div = -1.0f;
  int inner_no = 0, outer_no = 0;
  for (int J0 = 0; J0 < dmax; J0 += OB, ++outer_no) {
    for (int off = 0; off < OB && J0 + off < dmax; off += ip, ++inner_no) {
      const size_t in_slot = in_registers ? (size_t)inner_no : (size_t)(inner_no % 4);
      while (p->qr_in.size() <= in_slot) p->qr_in.emplace_back(new sa_plan::QrInner());
      sa_plan::QrInner& R = *p->qr_in[in_slot];
      const int j0 = J0 + off;
      SACHECK(R.panel.begin(n));
      for (int k = 0; k < 3; ++k) { R.upd[k].clear(); R.merge[k].clear(); }
      int jobs = 0, max_rows = 0;
      for (int i : ids) {
        const Factor& f = p->factors[i];
        if (j0 >= f.d) continue;
        const int ob = std::min(OB, f.d - J0);  // width of this factor's outer block
        const int pc = std::min(ip, ob - off), rows = f.d - j0;
        const int n_in = ob - off - pc;         // columns of the outer block after this panel
        float* B = newton_buf(p, NB_X0, f);
        float* V = newton_buf(p, NB_S1, f);
        float* T = V + (long long)f.dpad * OB;
        float* S = T + OB * OB;
        float* X = S + OB * QR_MAX_PANEL;
        float* W = newton_buf(p, NB_S2, f);
        float* W2 = W + (long long)OB * f.dpad;
        float* Vi = V + (long long)off * OB + off;  // this panel's vectors inside V (whose rows start at J0)
        float* Ti = T + (long long)off * OB + off;
        QrPanel& J = R.panel.host[jobs++];
        std::memset(&J, 0, sizeof(J));
        J.B = B; J.ldb = f.dpad; J.d = f.d; J.j0 = j0; J.pcols = pc; J.active = p->d_active + i;
        J.V = V + off; J.ldv = OB; J.top = off;
        J.T = T + off; J.ldt = OB; J.t_rows = ob;
        max_rows = std::max(max_rows, rows);
        if (n_in > 0) {
          float* Bt = B + (long long)j0 * f.dpad + j0 + pc;  // rest of the outer block, B[j0:, j0+pc : J0+ob]
          R.upd[0].add(mk(i, Vi, OB, Bt, f.dpad, W, f.dpad, pc, n_in, rows), false);   // W = V_i^T Bt    (A_KM)
          R.upd[1].add(mk(i, Ti, OB, W, f.dpad, W2, f.dpad, pc, n_in, pc), false);     // W2 = T_i^T W    (A_KM)
          R.upd[2].add(mk(i, Vi, OB, W2, f.dpad, Bt, f.dpad, rows, n_in, pc), false);  // Bt -= V_i W2    (A_MK, SUB)
        }
        if (off > 0) {
          // T[0:off, off:off+pc] = -T[0:off, 0:off] (V[:, 0:off]^T V_i) T_i; V_i is zero above row off
          R.merge[0].add(mk(i, V + (long long)off * OB, OB, Vi, OB, S, QR_MAX_PANEL, off, pc, rows), false);  // S = V_prev^T V_i (A_KM)
          R.merge[1].add(mk(i, T, OB, S, QR_MAX_PANEL, X, QR_MAX_PANEL, off, pc, off), false);               // X = T_prev S     (A_MK)
          R.merge[2].add(mk(i, X, QR_MAX_PANEL, Ti, OB, T + off, OB, off, pc, pc), false);                   // T12 = (-X) T_i   (A_MK)
        }
      }
      if (!jobs) break;
      R.panel.n = jobs;
      SACHECK(R.panel.upload(s));
      for (int k = 0; k < 3; ++k) { SACHECK(R.upd[k].commit(s)); SACHECK(R.merge[k].commit(s)); }
      const size_t lds_bytes = (size_t)max_rows * (ip + 1) * sizeof(float);
      if (in_registers) hipLaunchKernelGGL(qr_panel_rows_kernel, dim3(jobs), dim3(QR_THREADS), 0, s, R.panel.dev);
      else hipLaunchKernelGGL(qr_panel_kernel, dim3(jobs), dim3(QR_THREADS), lds_bytes, s, R.panel.dev);
      HIPCHECK(hipGetLastError());
      // the products over the panel's rows have 32 rows or columns of output: in 64 x 64 tiles they waste a quarter of the
      // matrix instructions that 128 x 128 tiles spend on rows and columns nobody keeps
      SACHECK((launch_gemm_small_tiles<A_KM, B_KN, EPI_STORE>(R.upd[0], u, s)));
      SACHECK((launch_gemm<A_KM, B_KN, EPI_STORE, true>(R.upd[1], u, s)));
      SACHECK((launch_gemm_small_tiles<A_MK, B_KN, EPI_SUB>(R.upd[2], u, s)));
      SACHECK((launch_gemm_small_tiles<A_KM, B_KN, EPI_STORE>(R.merge[0], u, s)));
      SACHECK((launch_gemm<A_MK, B_KN, EPI_STORE, true>(R.merge[1], u, s)));
      SACHECK((launch_gemm<A_MK, B_KN, EPI_STORE, true>(R.merge[2], neg, s)));
    }
    // the outer block's reflectors I - V T V^T on the trailing matrix (from the left, transposed) and on Qacc (from the right)
    const size_t out_slot = in_registers ? (size_t)outer_no : (size_t)(outer_no % 2);
    while (p->qr_outer.size() <= out_slot) p->qr_outer.emplace_back(new sa_plan::QrOuter());
    GemmTable* G = p->qr_outer[out_slot]->g;
    for (int k = 0; k < 6; ++k) G[k].clear();
    bool any = false;
    for (int i : ids) {
      const Factor& f = p->factors[i];
      if (J0 >= f.d) continue;
      any = true;
      const int ob = std::min(OB, f.d - J0), rows0 = f.d - J0, ntrail = f.d - J0 - ob;
      float* B = newton_buf(p, NB_X0, f);
      float* Qacc = newton_buf(p, NB_X1, f);
      float* V = newton_buf(p, NB_S1, f);
      float* T = V + (long long)f.dpad * OB;
      float* W = newton_buf(p, NB_S2, f);
      float* W2 = W + (long long)OB * f.dpad;
      float* Z = W;
      float* Z2 = W2;
      if (ntrail > 0) {
        float* Bt = B + (long long)J0 * f.dpad + J0 + ob;  // trailing matrix B[J0:, J0+ob:]
        G[0].add(mk(i, V, OB, Bt, f.dpad, W, f.dpad, ob, ntrail, rows0), false);   // W = V^T Bt      (A_KM)
        G[1].add(mk(i, T, OB, W, f.dpad, W2, f.dpad, ob, ntrail, ob), false);      // W2 = T^T W      (A_KM)
        G[2].add(mk(i, V, OB, W2, f.dpad, Bt, f.dpad, rows0, ntrail, ob), false);  // Bt -= V W2      (A_MK, SUB)
      }
      float* Qt = Qacc + J0;  // Qacc[:, J0:]
      G[3].add(mk(i, Qt, f.dpad, V, OB, Z, OB, f.d, ob, rows0), false);   // Z = Qt V       (NN)
      G[4].add(mk(i, Z, OB, T, OB, Z2, OB, f.d, ob, ob), false);          // Z2 = Z T       (NN)
      G[5].add(mk(i, Z2, OB, V, OB, Qt, f.dpad, f.d, rows0, ob), false);  // Qt -= Z2 V^T   (B_NK, SUB)
    }
    if (!any) break;
    for (int k = 0; k < 6; ++k) SACHECK(G[k].commit(s));
    // full outer blocks of aligned factors take the unguarded loader
    SACHECK((launch_gemm_auto<A_KM, B_KN, EPI_STORE>(G[0], u, s)));
    SACHECK((launch_gemm_small_tiles<A_KM, B_KN, EPI_STORE>(G[1], u, s)));
    SACHECK((launch_gemm_small_tiles<A_MK, B_KN, EPI_SUB>(G[2], u, s)));
    SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_STORE>(G[3], u, s)));
    SACHECK((launch_gemm_small_tiles<A_MK, B_KN, EPI_STORE>(G[4], u, s)));
    SACHECK((launch_gemm_small_tiles<A_MK, B_NK, EPI_SUB>(G[5], u, s)));
  }
  return SA_OK;
}

static int sa_refresh_eigenbases_qr_wave(sa_plan* p, float bias_correction2, float epsilon, int32_t max_iterations, float tolerance,
                                 int32_t* iterations_out, int32_t* status_out, void* stream) {
  if (!p || !iterations_out || !status_out) return fail(SA_ERR_INVALID, "sa_refresh_eigenbases_qr: NULL argument");
  if (p->factors.empty()) return SA_OK;  // nothing is preconditioned
  if (!p->has_eigvec) return fail(SA_ERR_STATE, "plan has no eigenvector state");
  if (!(bias_correction2 != 0.0f) || max_iterations < 0) return fail(SA_ERR_INVALID, "bad bias correction or max_iterations");
  hipStream_t s = static_cast<hipStream_t>(stream);
  SACHECK(ensure_tables(p, nullptr, s));
  const int F = (int)p->factors.size();
  if (F == 0) return SA_OK;
  p->eig_source.assign(F, sa_plan::EigSource{});
  p->rotm_version = -1;  // the eigenbases change
  std::vector<int> todo;
  SACHECK(root_inverse_prologue(p, bias_correction2, epsilon, iterations_out, status_out, s, &todo));
  if (todo.empty()) return SA_OK;
  const int n = (int)todo.size();

  // A = unpack(factor / bc2) + eps I (NB_M0); Qacc = current eigenbasis (NB_X1)
  SACHECK(p->t_eiginit.begin(n));
  SACHECK(p->t_copy.begin(n));
  int tiles = 0;
  for (int i = 0; i < n; ++i) {
    const Factor& f = p->factors[todo[i]];
    EigInit& J = p->t_eiginit.host[i];
    std::memset(&J, 0, sizeof(J));
    J.packed = packed32(p, f); J.scale = p->scale_of(todo[i]); J.A = newton_buf(p, NB_M0, f); J.V = nullptr;  // the basis comes from the state
    J.d = f.d; J.dpad = f.dpad; J.tiles = f.dpad / 64; J.enabled = 1; J.tile_begin = tiles;
    tiles += J.tiles * J.tiles;
    Copy2D& C = p->t_copy.host[i];
    std::memset(&C, 0, sizeof(C));
    C.src = f.eigvec; C.lds_ = f.d; C.dst = newton_buf(p, NB_X1, f); C.ldd = f.dpad; C.rows = f.d; C.cols = f.d;
  }
  SACHECK(p->t_eiginit.upload(s));
  SACHECK(p->t_copy.upload(s));
  hipLaunchKernelGGL(eig_init_kernel, dim3(tiles), dim3(256), 0, s, p->t_eiginit.dev, n, bias_correction2, epsilon);
  hipLaunchKernelGGL(copy2d_kernel, dim3(64, n), dim3(256), 0, s, p->t_copy.dev);
  HIPCHECK(hipGetLastError());

  std::vector<int> active(F, 0), iters(F, 0);
  for (int i : todo) active[i] = 1;
  auto build_AQ = [&](bool also_B) -> int {
    p->qr_aq.clear();
    p->qr_b.clear();
    for (int i : todo) {
      const Factor& f = p->factors[i];
      GemmProblem q{};
      q.A = newton_buf(p, NB_M0, f); q.lda = f.dpad; q.a_vec = 1;
      q.B = newton_buf(p, NB_X1, f); q.ldb = f.dpad; q.b_vec = 1;
      q.C = newton_buf(p, NB_M1, f); q.ldc = f.dpad; q.M = q.N = q.K = f.d;
      p->qr_aq.add(q, false);  // Y = A Qacc
      if (also_B) {
        GemmProblem b{};
        b.A = newton_buf(p, NB_X1, f); b.lda = f.dpad; b.a_vec = 1;   // Qacc^T (A_KM)
        b.B = newton_buf(p, NB_M1, f); b.ldb = f.dpad; b.b_vec = 1;
        b.C = newton_buf(p, NB_X0, f); b.ldc = f.dpad; b.M = b.N = b.K = f.d;
        p->qr_b.add(b, true);   // B = Qacc^T Y = Qacc^T A Qacc is symmetric: upper-triangle tiles, mirrored
      }
    }
    SACHECK(p->qr_aq.commit(s));
    SACHECK(p->qr_b.commit(s));
    SACHECK((launch_gemm_auto<A_MK, B_KN, EPI_STORE>(p->qr_aq, unit_scalars(), s)));
    if (also_B) {
      if (p->qr_b.aligned) SACHECK((launch_gemm<A_KM, B_KN, EPI_STORE, false, true>(p->qr_b, unit_scalars(), s)));
      else SACHECK((launch_gemm<A_KM, B_KN, EPI_STORE, true, true>(p->qr_b, unit_scalars(), s)));
    }
    return SA_OK;
  };

  for (int it = 0; it < max_iterations; ++it) {
    SACHECK(build_AQ(true));
    // criterion ||B - diag B||_F <= tol ||B||_F, evaluated like the reference (fp32, sqrt of a difference)
    SACHECK(p->t_normpair.begin(n));
    for (int k = 0; k < n; ++k) {
      const Factor& f = p->factors[todo[k]];
      NormPair& J = p->t_normpair.host[k];
      J.B = newton_buf(p, NB_X0, f); J.ldb = f.dpad; J.d = f.d;
      J.out_all = p->d_final_err + todo[k];
      J.out_diag = reinterpret_cast<float*>(p->d_err) + todo[k];
    }
    SACHECK(p->t_normpair.upload(s));
    hipLaunchKernelGGL(diag_off_norm_kernel, dim3(n), dim3(FACTOR_PASS_THREADS), 0, s, p->t_normpair.dev);
    HIPCHECK(hipGetLastError());
    HIPCHECK(hipMemcpyAsync(p->h_pinned, p->d_final_err, F * sizeof(float), hipMemcpyDeviceToHost, s));
    HIPCHECK(hipMemcpyAsync(p->h_pinned + F, p->d_err, F * sizeof(float), hipMemcpyDeviceToHost, s));
    HIPCHECK(hipStreamSynchronize(s));
    const float* h_all = reinterpret_cast<const float*>(p->h_pinned);
    const float* h_diag = reinterpret_cast<const float*>(p->h_pinned + F);
    std::vector<int> go;
    for (int k = 0; k < n; ++k) {
      const int i = todo[k];
      if (!active[i]) continue;
      const float norm = std::sqrt(h_all[i]), dnorm = std::sqrt(h_diag[i]);
      const float off = std::sqrt(norm * norm - dnorm * dnorm);  // NaN when rounding makes it negative: iterate
      const bool below = off <= tolerance * norm;
      if (below) active[i] = 0; else go.push_back(i);
    }
    if (go.empty()) break;
    HIPCHECK(hipMemcpyAsync(p->d_active, active.data(), F * sizeof(int), hipMemcpyHostToDevice, s));
    HIPCHECK(hipStreamSynchronize(s));
    double flops = 0.0;
    for (int i : go) { const double d = p->factors[i].d; flops += (4.0 / 3.0 + 2.0) * d * d * d; }
    {
      Span span("qr_refresh", s, flops, 7 * ((p->factors[go[0]].d + 31) / 32), it == 0);
      SACHECK(qr_accumulate(p, go, s));
    }
    for (int i : go) iters[i] += 1;
  }
  // eigenvalue estimates = Rayleigh quotients of the final basis, stable ascending order, permuted columns
  SACHECK(build_AQ(false));
  SACHECK(p->t_sort.begin(n));
  SACHECK(p->t_copy.begin(n));
  for (int k = 0; k < n; ++k) {
    const Factor& f = p->factors[todo[k]];
    SortJob& J = p->t_sort.host[k];
    J.Q = newton_buf(p, NB_X1, f); J.ldq = f.dpad;
    J.Y = newton_buf(p, NB_M1, f); J.ldy = f.dpad;
    J.ev = newton_buf(p, NB_S2, f) + 2LL * f.dpad * QR_MAX_PANEL;
    J.order = reinterpret_cast<int*>(J.ev + f.dpad);
    J.d = f.d;
    p->eig_source[todo[k]] = sa_plan::EigSource{J.ev, 1, J.order};
    Copy2D& C = p->t_copy.host[k];
    std::memset(&C, 0, sizeof(C));
    C.src = newton_buf(p, NB_X1, f); C.lds_ = f.dpad; C.dst = newton_buf(p, NB_X0, f); C.ldd = f.dpad;
    C.rows = f.d; C.cols = f.d; C.perm = J.order;
  }
  SACHECK(p->t_sort.upload(s));
  SACHECK(p->t_copy.upload(s));
  hipLaunchKernelGGL(rayleigh_sort_kernel, dim3(n), dim3(FACTOR_PASS_THREADS), 0, s, p->t_sort.dev);
  hipLaunchKernelGGL(copy2d_kernel, dim3(64, n), dim3(256), 0, s, p->t_copy.dev);  // sorted basis -> NB_X0
  HIPCHECK(hipGetLastError());

  // finiteness of the new bases, then copy those that precede the first bad one into the state
  const int Fall = F;
  int* h_bad = p->h_pinned + 3 * Fall;
  HIPCHECK(hipMemsetAsync(p->d_flags, 0, Fall * sizeof(int), s));
  SACHECK(p->t_normjobs.begin(n));
  int chunks = 0;
  for (int k = 0; k < n; ++k) {
    const Factor& f = p->factors[todo[k]];
    NormJob& J = p->t_normjobs.host[k];
    std::memset(&J, 0, sizeof(J));
    J.src = newton_buf(p, NB_X0, f); J.nonfinite = p->d_flags + todo[k];
    J.d = f.d; J.dpad = f.dpad; J.dense = 1; J.chunk_begin = chunks;
    J.n_chunks = (int)(((long long)f.d * f.d + NORM_CHUNK - 1) / NORM_CHUNK); J.enabled = 1;
    chunks += J.n_chunks;
  }
  SACHECK(p->t_normjobs.upload(s));
  hipLaunchKernelGGL((factor_norm_kernel<true>), dim3(chunks), dim3(256), 0, s, p->t_normjobs.dev, n, 1.0f, 0.0f);
  HIPCHECK(hipGetLastError());
  HIPCHECK(hipMemcpyAsync(h_bad, p->d_flags, Fall * sizeof(int), hipMemcpyDeviceToHost, s));
  HIPCHECK(hipStreamSynchronize(s));
  int ok = n;
  for (int k = 0; k < n; ++k) {
    iterations_out[todo[k]] = iters[todo[k]];
    if (k < ok && h_bad[todo[k]]) { status_out[todo[k]] = SA_FACTOR_RESULT_NONFINITE; ok = k; }
  }
  if (ok > 0) {
    SACHECK(p->t_copy.begin(ok));
    for (int k = 0; k < ok; ++k) {
      const Factor& f = p->factors[todo[k]];
      Copy2D& C = p->t_copy.host[k];
      std::memset(&C, 0, sizeof(C));
      C.src = newton_buf(p, NB_X0, f); C.lds_ = f.dpad; C.dst = f.eigvec; C.ldd = f.d; C.rows = f.d; C.cols = f.d;
      status_out[todo[k]] = SA_FACTOR_OK;
    }
    SACHECK(p->t_copy.upload(s));
    hipLaunchKernelGGL(copy2d_kernel, dim3(64, ok), dim3(256), 0, s, p->t_copy.dev);
    HIPCHECK(hipGetLastError());
    HIPCHECK(hipStreamSynchronize(s));
  }
  return SA_OK;
}

int32_t sa_refresh_eigenbases_qr(sa_plan* p, float bias_correction2, float epsilon, int32_t max_iterations, float tolerance, int32_t* iterations_out, int32_t* status_out, void* stream) {
  if (!p || !status_out) return fail(SA_ERR_INVALID, "sa_refresh_eigenbases_qr: NULL argument");
  return for_each_wave(p, iterations_out, status_out, static_cast<hipStream_t>(stream), [&](int32_t* it__, int32_t* st__) {
    return sa_refresh_eigenbases_qr_wave(p, bias_correction2, epsilon, max_iterations, tolerance, it__, st__, stream);
  });
}

// --------------------------------------------------------------------------------------------
// Dense state tensors (state layout without symmetric packing)
// --------------------------------------------------------------------------------------------

static int dense_state_pass(sa_plan* p, void* const* dense_factor, void* const* dense_inv, bool to_dense, hipStream_t s) {
  const int F = (int)p->factors.size();
  for (int which = 0; which < 2; ++which) {
    void* const* dense = which == 0 ? dense_factor : dense_inv;
    if (!dense) continue;
    Table<DenseStateJob>& T = p->t_dense_state[which];
    SACHECK(T.begin(F));
    int n = 0, tiles = 0;
    for (int i = 0; i < F; ++i) {
      const Factor& f = p->factors[i];
      void* packed = which == 0 ? static_cast<void*>(f.factor) : static_cast<void*>(f.inv);
      if (!dense[i] || !packed) continue;
      DenseStateJob& J = T.host[n++];
      J.packed = packed;
      J.dense = dense[i];
      J.d = f.d;
      J.tiles = (f.d + ST - 1) / ST;
      J.tile_begin = tiles;
      tiles += J.tiles * (J.tiles + 1) / 2;
    }
    if (n == 0) continue;
    T.n = n;
    SACHECK(T.upload(s));
    const bool f64 = which == 0 && p->factor_f64;
    if (f64 && to_dense) hipLaunchKernelGGL((sym_state_kernel<double, true>), dim3(tiles), dim3(256), 0, s, T.dev, n);
    else if (f64) hipLaunchKernelGGL((sym_state_kernel<double, false>), dim3(tiles), dim3(256), 0, s, T.dev, n);
    else if (to_dense) hipLaunchKernelGGL((sym_state_kernel<float, true>), dim3(tiles), dim3(256), 0, s, T.dev, n);
    else hipLaunchKernelGGL((sym_state_kernel<float, false>), dim3(tiles), dim3(256), 0, s, T.dev, n);
    HIPCHECK(hipGetLastError());
  }
  return SA_OK;
}

int32_t sa_plan_export_dense_state(sa_plan* p, void* const* dense_factor, void* const* dense_inv, void* stream) {
  if (!p) return fail(SA_ERR_INVALID, "sa_plan_export_dense_state: NULL plan");
  return dense_state_pass(p, dense_factor, dense_inv, true, static_cast<hipStream_t>(stream));
}

int32_t sa_plan_import_dense_state(sa_plan* p, void* const* dense_factor, void* const* dense_inv, void* stream) {
  if (!p) return fail(SA_ERR_INVALID, "sa_plan_import_dense_state: NULL plan");
  return dense_state_pass(p, dense_factor, dense_inv, false, static_cast<hipStream_t>(stream));
}

// --------------------------------------------------------------------------------------------
// Single GEMM (tests, microbenchmarks)
// --------------------------------------------------------------------------------------------

// One problem table per stream (work on one stream is ordered, so a table is never rewritten under a launch that still
// reads it), guarded by a mutex: the call may be made from several threads.
static std::mutex g_test_mutex;
static std::map<hipStream_t, GemmTable> g_test_tables;

int32_t sa_gemm_f32(const float* A, const float* B, float* C, int32_t M, int32_t N, int32_t K, int64_t lda, int64_t ldb,
                    int64_t ldc, int32_t a_layout, int32_t b_layout, int32_t batch, int64_t stride_a, int64_t stride_b,
                    int64_t stride_c, void* stream) {
  if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0 || batch <= 0) return fail(SA_ERR_INVALID, "sa_gemm_f32: bad arguments");
  hipStream_t s = static_cast<hipStream_t>(stream);
  std::lock_guard<std::mutex> lock(g_test_mutex);
  GemmTable& g_test_table = g_test_tables[s];
  g_test_table.clear();
  for (int i = 0; i < batch; ++i) {
    GemmProblem q{};
    q.A = A + i * stride_a; q.B = B + i * stride_b; q.C = C + i * stride_c;
    q.lda = lda; q.ldb = ldb; q.ldc = ldc;
    q.M = M; q.N = N; q.K = K;
    q.a_vec = vec_ok(q.A, lda);
    q.b_vec = vec_ok(q.B, ldb);
    g_test_table.add(q, false);
  }
  SACHECK(g_test_table.commit(s));
  Span span("gemm", s, 2.0 * M * N * K * batch, 1, true);
  GemmScalars u = unit_scalars();
  if (a_layout == 0 && b_layout == 0) return launch_gemm_auto<A_MK, B_KN, EPI_STORE>(g_test_table, u, s);
  if (a_layout == 0 && b_layout == 1) return launch_gemm_auto<A_MK, B_NK, EPI_STORE>(g_test_table, u, s);
  if (a_layout == 1 && b_layout == 0) return launch_gemm_auto<A_KM, B_KN, EPI_STORE>(g_test_table, u, s);
  if (a_layout == 1 && b_layout == 1) return launch_gemm_auto<A_KM, B_NK, EPI_STORE>(g_test_table, u, s);
  return fail(SA_ERR_INVALID, "sa_gemm_f32: layouts must be 0 or 1");
}

// --------------------------------------------------------------------------------------------
// sa_gemm_f32 for callers that cannot allocate (HIP graph capture, serving loops): the problem table, which
// sa_gemm_f32 keeps in a device buffer the library allocates and uploads, lives in a file-scope device array and is
// written by a small kernel from the call's own arguments.  No hipMalloc / hipFree / copy is issued.
// --------------------------------------------------------------------------------------------

constexpr int STATIC_GEMM_MAX_BATCH = SA_GEMM_STATIC_MAX_BATCH;
constexpr int STATIC_GEMM_MAX_DEVICES = 64;
static_assert(sizeof(GemmProblem) == 128, "the documented size of the static table (128 KB) assumes 128-byte problems");
static __device__ __align__(256) unsigned char scratch[STATIC_GEMM_MAX_BATCH * sizeof(GemmProblem)];
// device address of `scratch` on every GPU this process has used it on (each GPU holds its own copy of the array)
static GemmProblem* g_scratch_ptr[STATIC_GEMM_MAX_DEVICES] = {nullptr};

__global__ void static_gemm_fill_kernel(GemmProblem* __restrict__ table, const float* A, const float* B, float* C, int M, int N,
                                        int K, long long lda, long long ldb, long long ldc, int batch, long long stride_a,
                                        long long stride_b, long long stride_c, int a_vec, int b_vec) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= batch) return;
  GemmProblem q;
  q.A = A + i * stride_a;
  q.B = B + i * stride_b;
  q.C = C + i * stride_c;
  q.C2 = nullptr; q.C3 = nullptr; q.err_bits = nullptr; q.active = nullptr;
  q.lda = lda; q.ldb = ldb; q.ldc = ldc;
  q.M = M; q.N = N; q.K = K;
  q.tiles_m = (M + BM - 1) / BM;
  q.tiles_n = (N + BN - 1) / BN;
  q.tile_begin = i * q.tiles_m * q.tiles_n;
  q.tiles_m_s = (M + 63) / 64;
  q.tiles_n_s = (N + 63) / 64;
  q.tile_begin_s = i * q.tiles_m_s * q.tiles_n_s;
  q.d = 0;
  q.a_vec = a_vec; q.b_vec = b_vec;
  table[i] = q;
}

int32_t sa_gemm_f32_static(const float* A, const float* B, float* C, int32_t M, int32_t N, int32_t K, int64_t lda, int64_t ldb,
                           int64_t ldc, int32_t a_layout, int32_t b_layout, int32_t batch, int64_t stride_a, int64_t stride_b,
                           int64_t stride_c, void* stream) {
  if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0 || batch <= 0) return fail(SA_ERR_INVALID, "sa_gemm_f32_static: bad arguments");
  if (a_layout < 0 || a_layout > 1 || b_layout < 0 || b_layout > 1) return fail(SA_ERR_INVALID, "sa_gemm_f32_static: layouts must be 0 or 1");
  if (batch > STATIC_GEMM_MAX_BATCH)
    return fail(SA_ERR_INVALID, "sa_gemm_f32_static: batch " + std::to_string(batch) + " exceeds the static problem table (" +
                                    std::to_string(STATIC_GEMM_MAX_BATCH) + " problems); use sa_gemm_f32");
  const long long tiles_each = (long long)((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  if (tiles_each * batch > 0x7fffffffLL / 2) return fail(SA_ERR_INVALID, "sa_gemm_f32_static: too many tiles for one launch");
  int dev = -1;
  HIPCHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= STATIC_GEMM_MAX_DEVICES) return fail(SA_ERR_UNSUPPORTED, "sa_gemm_f32_static: device index out of range");
  if (stream) {  // the table is the current device's copy of the array: the stream must belong to that device
    int stream_dev = -1;
    HIPCHECK(hipStreamGetDevice(static_cast<hipStream_t>(stream), &stream_dev));
    if (stream_dev != dev)
      return fail(SA_ERR_INVALID, "sa_gemm_f32_static: the stream belongs to device " + std::to_string(stream_dev) +
                                      " but device " + std::to_string(dev) + " is current");
  }
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    HIPCHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return fail(SA_ERR_HIP, "sa_gemm_f32_static: the static problem table has no device address");
    g_scratch_ptr[dev] = static_cast<GemmProblem*>(ptr);
  }
  GemmProblem* table = g_scratch_ptr[dev];
  hipStream_t s = static_cast<hipStream_t>(stream);
  // every problem of the batch may use 16-byte loads only if the first one may and the batch stride keeps the alignment
  const int a_vec = (vec_ok(A, lda) && (batch == 1 || stride_a % 4 == 0)) ? 1 : 0;
  const int b_vec = (vec_ok(B, ldb) && (batch == 1 || stride_b % 4 == 0)) ? 1 : 0;
  GemmProblem shape{};
  shape.M = M; shape.N = N; shape.K = K; shape.lda = lda; shape.ldb = ldb; shape.a_vec = a_vec; shape.b_vec = b_vec;
  const bool aligned = unguarded_ok(shape);
  hipLaunchKernelGGL(static_gemm_fill_kernel, dim3((batch + 255) / 256), dim3(256), 0, s, table, A, B, C, M, N, K, (long long)lda,
                     (long long)ldb, (long long)ldc, batch, (long long)stride_a, (long long)stride_b, (long long)stride_c, a_vec,
                     b_vec);
  HIPCHECK(hipGetLastError());
  const int total_tiles = (int)(tiles_each * batch);
  GemmScalars u = unit_scalars();
#define SA_STATIC_GEMM(AL, BL)                                                                         \
  return aligned ? launch_gemm_raw<AL, BL, EPI_STORE, false>(table, batch, total_tiles, u, s)          \
                 : launch_gemm_raw<AL, BL, EPI_STORE, true>(table, batch, total_tiles, u, s)
  if (a_layout == 0 && b_layout == 0) { SA_STATIC_GEMM(A_MK, B_KN); }
  if (a_layout == 0 && b_layout == 1) { SA_STATIC_GEMM(A_MK, B_NK); }
  if (a_layout == 1 && b_layout == 0) { SA_STATIC_GEMM(A_KM, B_KN); }
  SA_STATIC_GEMM(A_KM, B_NK);
#undef SA_STATIC_GEMM
}

int32_t sa_copy_f32(const float* src, float* dst, int64_t n, void* stream) {
  if (!src || !dst || n <= 0 || (n & 3) || ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15))
    return fail(SA_ERR_INVALID, "sa_copy_f32: need 16-byte aligned pointers and n a multiple of 4");
  hipStream_t s = static_cast<hipStream_t>(stream);
  Span span("copy", s, 8.0 * (double)n, 1, true);
  hipLaunchKernelGGL(copy_kernel, dim3(256 * 16), dim3(256), 0, s, reinterpret_cast<const float4*>(src),
                     reinterpret_cast<float4*>(dst), (long long)(n / 4));
  HIPCHECK(hipGetLastError());
  return SA_OK;
}

int32_t sa_add_to_views(const sa_view* dst, const sa_view* src, int32_t n, void* stream) {
  if (n < 0 || (n > 0 && (!dst || !src))) return fail(SA_ERR_INVALID, "sa_add_to_views: null view table");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // validate everything before the first launch: a bad pair must leave every destination untouched
  for (int i = 0; i < n; ++i) {
    const sa_view &D = dst[i], &S = src[i];
    if (D.order < 0 || D.order > SA_MAX_ORDER || S.order != D.order)
      return fail(SA_ERR_INVALID, "sa_add_to_views: pair " + std::to_string(i) + ": orders must agree and be at most " +
                                      std::to_string(SA_MAX_ORDER));
    for (int k = 0; k < D.order; ++k) {
      if (D.size[k] != S.size[k] || D.size[k] < 0 || D.size[k] > 0x7fffffffLL)
        return fail(SA_ERR_INVALID, "sa_add_to_views: pair " + std::to_string(i) + ": sizes differ in dim " + std::to_string(k));
      if (D.size[k] > 1 && D.stride[k] <= 0)
        return fail(SA_ERR_INVALID, "sa_add_to_views: pair " + std::to_string(i) + ": destination views must not overlap themselves");
    }
    long long numel = 1;
    for (int k = 0; k < D.order; ++k) numel *= D.size[k];
    if (numel > 0 && (!D.data || !S.data)) return fail(SA_ERR_INVALID, "sa_add_to_views: pair " + std::to_string(i) + ": null data pointer");
  }
  ViewAddBatch batch;
  int filled = 0;
  unsigned long long most_runs = 0;
  double bytes = 0.0;
  bool first_launch = true;
  auto flush = [&]() -> int32_t {
    if (filled == 0) return SA_OK;
    const unsigned int gx = (unsigned int)std::min<unsigned long long>((most_runs + 255) / 256, 1024);
    Span span("view_add", s, bytes, 1, first_launch);
    first_launch = false;
    hipLaunchKernelGGL(view_add_kernel, dim3(gx, filled), dim3(256), 0, s, batch);
    HIPCHECK(hipGetLastError());
    filled = 0;
    most_runs = 0;
    bytes = 0.0;
    return SA_OK;
  };
  for (int i = 0; i < n; ++i) {
    const sa_view &D = dst[i], &S = src[i];
    ViewAddJob J{};
    unsigned int sz[3] = {1, 1, 1};
    long long ds[3] = {0, 0, 0}, ss[3] = {0, 0, 0};
    for (int k = 0; k < D.order; ++k) {  // right-align: a 2-D view is (1, rows, cols)
      sz[3 - D.order + k] = (unsigned int)D.size[k];
      ds[3 - D.order + k] = D.stride[k];
      ss[3 - D.order + k] = S.stride[k];
    }
    const unsigned long long numel = (unsigned long long)sz[0] * sz[1] * sz[2];
    if (numel == 0) continue;
    if (sz[2] == 1) { ds[2] = 1; ss[2] = 1; }  // strides of extent-1 dims are arbitrary
    J.dst = static_cast<float*>(D.data);
    J.src = static_cast<const float*>(S.data);
    J.n0 = sz[0]; J.n1 = sz[1]; J.n2 = sz[2];
    J.d0 = ds[0]; J.d1 = ds[1]; J.d2 = ds[2];
    J.s0 = ss[0]; J.s1 = ss[1]; J.s2 = ss[2];
    auto rows_aligned = [&](const void* p, const long long* st) {
      return (reinterpret_cast<uintptr_t>(p) & 15) == 0 && (sz[0] == 1 || (st[0] & 3) == 0) && (sz[1] == 1 || (st[1] & 3) == 0);
    };
    J.vec = (ds[2] == 1 && ss[2] == 1 && (sz[2] & 3) == 0 && rows_aligned(D.data, ds) && rows_aligned(S.data, ss)) ? 1u : 0u;
    batch.job[filled++] = J;
    most_runs = std::max<unsigned long long>(most_runs, (unsigned long long)sz[0] * sz[1] * ((sz[2] + 3) / 4));
    bytes += 12.0 * (double)numel;
    if (filled == VIEW_ADD_BATCH) {
      const int32_t st = flush();
      if (st != SA_OK) return st;
    }
  }
  return flush();
}

}  // extern "C"
