// C ABI of the gfx950 int8 affine backend: argument checks, kernel selection, launches.
// Declarations and the reference call sites each entry point replaces: include/marian_hip_int8.h
#include "../../include/marian_hip_int8.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <random>

#include "abi_common.h"
#include "gemm_mfma32_kernel.h"
#include "gemm_pair_kernel.h"
#include "gemm_stream32_kernel.h"
#include "gemm_stream_kernel.h"
#include "quantize_kernels.h"
#ifdef MARIAN_HIP_TUNING
// kernel families that only measurements select, and the switches that select them
#include "../../include/marian_hip_int8_tuning.h"
#include "probe_kernels.h"
#endif

using namespace marian_hip;

namespace {
thread_local int g_last_hip_error = 0;
// set by the launcher whose kernel fills GemmArgs::absmax_out itself
thread_local bool t_absmax_written = false;
}

int marian_hip::record_hip_error(int e) {
  g_last_hip_error = e;
  return MARIAN_HIP_ERR_HIP;
}

int marian_hip::launch_absmax_partials(const float* A, unsigned long n, float* partials, int* n_partials, void* stream) {
  const size_t n4 = (size_t)n / 4, per_block = (size_t)kQuantThreads * 8;   // eight 16-byte loads per thread
  size_t g = (n4 + per_block - 1) / per_block;
  if(g < 1) g = 1;
  if(g > (size_t)kMaxPartials) g = kMaxPartials;
  hipLaunchKernelGGL(absmax_partial_kernel, dim3((unsigned)g), dim3(kQuantThreads), 0, reinterpret_cast<hipStream_t>(stream),
                     A, n4, partials);
  const hipError_t e = hipGetLastError();
  if(e != hipSuccess) return marian_hip::record_hip_error((int)e);
  *n_partials = (int)g;
  return MARIAN_HIP_OK;
}

namespace {

// The shipped library has no switches: kernel_override() is the constant 0 there and the
// measurement ids named in the comments below exist in the tuning build only.
#ifdef MARIAN_HIP_TUNING
std::atomic<int> g_kernel_override{0};
std::atomic<long long*> g_prof{nullptr};
inline int kernel_override() { return g_kernel_override.load(std::memory_order_relaxed); }
#else
constexpr int kernel_override() { return 0; }
#endif

int hip_fail(hipError_t e) { return marian_hip::record_hip_error((int)e); }

#define MH_HIP(expr)                            \
  do {                                          \
    hipError_t e_ = (expr);                     \
    if(e_ != hipSuccess) return hip_fail(e_);   \
  } while(0)

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

constexpr int64_t kMaxElems = 2147483647LL;

constexpr int kMaxDevices = 64;

// The current device, as an index into the per-device caches below.
inline int current_device(int* dev) {
  MH_HIP(hipGetDevice(dev));
  if(*dev < 0 || *dev >= kMaxDevices) return MARIAN_HIP_ERR_RANGE;
  return MARIAN_HIP_OK;
}

// Raises a kernel's dynamic LDS limit, once per kernel and device (`done`: one bit per device).
template <typename KernelT>
int allow_lds(KernelT kernel, int bytes, std::atomic<uint64_t>& done) {
  if(bytes <= 48 * 1024) return MARIAN_HIP_OK;
  int dev = 0;
  int st = current_device(&dev);
  if(st != MARIAN_HIP_OK) return st;
  const uint64_t bit = 1ull << dev;
  if(done.load(std::memory_order_acquire) & bit) return MARIAN_HIP_OK;
  MH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                             hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
  done.fetch_or(bit, std::memory_order_release);
  return MARIAN_HIP_OK;
}

template <int MT, int NT, int WN, int KW, int PF>
int launch_stream(const GemmArgs& a, hipStream_t st) {
  using Cfg = StreamCfg<MT, NT, WN, KW, PF>;
  auto kernel = gemm_stream_kernel<MT, NT, WN, KW, PF>;
  static std::atomic<uint64_t> lds_done{0};
  const int lds_status = allow_lds(kernel, Cfg::kLdsBytes, lds_done);
  if(lds_status != MARIAN_HIP_OK) return lds_status;
  int blocks = (a.n_out + Cfg::kColsPerBlock - 1) / Cfg::kColsPerBlock;
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(Cfg::kThreads), Cfg::kLdsBytes, st, a);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

// Compute units of the current device (looked up once per device; 256 if the query fails).
int compute_units() {
  static std::atomic<int> cus[kMaxDevices];
  int dev = 0;
  if(hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  int n = cus[dev].load(std::memory_order_relaxed);
  if(n > 0) return n;
  if(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
    n = 256;
  cus[dev].store(n, std::memory_order_relaxed);
  return n;
}

// Whether a large-M launch of `workgroups` workgroups leaves the abs-max of its output itself: one
// slot per workgroup (not for accumulator dumps).
inline bool big_leaves_absmax(const GemmArgs& a, long long workgroups) {
  return a.absmax_out && !a.dump && workgroups <= kAbsmaxSlots;
}

// The split form (loading waves beside the multiplying ones): whole K blocks only; any M and N.
template <int BM, int BN, int WM, int WN, int NSTAGE, bool NT>
int launch_big_split(const GemmArgs& a, hipStream_t st) {
  using Cfg = BigCfg<BM, BN, WM, WN, NSTAGE>;
  if(a.K % Cfg::BK != 0) return MARIAN_HIP_ERR_SHAPE;
  const int tiles_n = (a.n_out + BN - 1) / BN;
  const int tiles_m = (a.M + BM - 1) / BM;
  static std::atomic<uint64_t> lds_done[2];
  GemmArgs a2 = a;
  if(big_leaves_absmax(a, (long long)tiles_n * tiles_m)) {
    auto kernel = gemm_mfma32_split_kernel<BM, BN, WM, WN, NSTAGE, NT, true>;
    const int lds_status = allow_lds(kernel, Cfg::kLdsBytes, lds_done[1]);
    if(lds_status != MARIAN_HIP_OK) return lds_status;
    a2.absmax_used = tiles_n * tiles_m;
    hipLaunchKernelGGL(kernel, dim3(tiles_n * tiles_m), dim3(2 * Cfg::kThreads), Cfg::kLdsBytes, st, a2, tiles_n, tiles_m);
    MH_HIP(hipGetLastError());
    t_absmax_written = true;
    return MARIAN_HIP_OK;
  }
  auto kernel = gemm_mfma32_split_kernel<BM, BN, WM, WN, NSTAGE, NT, false>;
  const int lds_status = allow_lds(kernel, Cfg::kLdsBytes, lds_done[0]);
  if(lds_status != MARIAN_HIP_OK) return lds_status;
  hipLaunchKernelGGL(kernel, dim3(tiles_n * tiles_m), dim3(2 * Cfg::kThreads), Cfg::kLdsBytes, st, a2, tiles_n, tiles_m);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

template <int BM, int BN, int WM, int WN, int NSTAGE, bool PAIRED = true, bool NT = false>
int launch_big(const GemmArgs& a, hipStream_t st) {
  using Cfg = BigCfg<BM, BN, WM, WN, NSTAGE>;
  // whole 128-column K blocks, or (paired-fragment form) a last block of 64 columns
  const int tiles_n = (a.n_out + BN - 1) / BN;
  const int tiles_m = (a.M + BM - 1) / BM;
  if(a.K % Cfg::BK != 0) {
    if(a.K % 64 != 0) return MARIAN_HIP_ERR_SHAPE;   // (refused by the argument checks already)
    // (the plain-fragment forms, which only measurements select, have no half block)
    if constexpr(!Cfg::kHalfTailOk || !PAIRED) {
      return launch_big<128, 128, 2, 4, 2, true, NT>(a, st);
    } else {
      auto half = gemm_mfma32_kernel<BM, BN, WM, WN, NSTAGE, true, NT, true>;
      static std::atomic<uint64_t> half_lds_done{0};
      const int half_lds_status = allow_lds(half, Cfg::kLdsBytes, half_lds_done);
      if(half_lds_status != MARIAN_HIP_OK) return half_lds_status;
      hipLaunchKernelGGL(half, dim3(tiles_n * tiles_m), dim3(Cfg::kThreads), Cfg::kLdsBytes, st, a,
                         tiles_n, tiles_m);
      MH_HIP(hipGetLastError());
      return MARIAN_HIP_OK;
    }
  }
  if constexpr(PAIRED) {
    if(big_leaves_absmax(a, (long long)tiles_n * tiles_m)) {
      auto kernel = gemm_mfma32_kernel<BM, BN, WM, WN, NSTAGE, true, NT, false, true>;
      static std::atomic<uint64_t> amax_lds_done{0};
      const int lds_status = allow_lds(kernel, Cfg::kLdsBytes, amax_lds_done);
      if(lds_status != MARIAN_HIP_OK) return lds_status;
      GemmArgs a2 = a;
      a2.absmax_used = tiles_n * tiles_m;
      hipLaunchKernelGGL(kernel, dim3(tiles_n * tiles_m), dim3(Cfg::kThreads), Cfg::kLdsBytes, st, a2, tiles_n, tiles_m);
      MH_HIP(hipGetLastError());
      t_absmax_written = true;
      return MARIAN_HIP_OK;
    }
  }
  auto kernel = gemm_mfma32_kernel<BM, BN, WM, WN, NSTAGE, PAIRED, NT>;
  static std::atomic<uint64_t> lds_done{0};
  const int lds_status = allow_lds(kernel, Cfg::kLdsBytes, lds_done);
  if(lds_status != MARIAN_HIP_OK) return lds_status;
  hipLaunchKernelGGL(kernel, dim3(tiles_n * tiles_m), dim3(Cfg::kThreads), Cfg::kLdsBytes, st, a,
                     tiles_n, tiles_m);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

// ---- outputs that are not a whole number of main tiles ----
// With whole and partial tiles alike (the launchers above) a few rows or columns past a whole number
// of tiles add a row or column of full-price tiles, and where the whole tiles just fill the chip
// that is a second round of workgroups: 4100 instead of 4096 rows cost +55 %.  The ragged launch
// gives the whole main tiles to the first workgroups and covers the rest with small tiles, which
// run in the slots the main tiles leave or as a short tail.  It is taken when it saves a round.
struct Ragged {
  bool use = false;
  RaggedPlan plan;
  int workgroups = 0;
};
// BM x BN: main tile; EBM x EBN: tiles of the strip below; RBM x RBN: tiles of the strip to the right;
// per_cu: main workgroups that share a CU; plain_cost: what a tile of the launch that would run
// otherwise costs relative to a main tile of this one.
// The choice compares rounds of workgroups: the plain launch needs ceil(all tiles / slots) rounds of
// main-tile time; the ragged one ceil(whole tiles / slots), its small tiles (a fifth of a main
// tile's time, measured at K = 1024) running in the slots the whole tiles leave idle and, what
// does not fit there, as a tail.
inline Ragged plan_ragged(const GemmArgs& a, int BM, int BN, int EBM, int EBN, int RBM, int RBN, int per_cu,
                          double plain_cost = 1.0) {
  Ragged r;
  const int ov = kernel_override() % 1000;
  if(a.K % 128 != 0 || ov == 350) return r;   // (measurement id 350: never)
  const long long cm = (a.M + BM - 1) / BM, cn = (a.n_out + BN - 1) / BN;
  const long long fm = a.M / BM, fn = a.n_out / BN;
  const long long slots = (long long)compute_units() * per_cu;
  if(fm * fn == 0 || fm * fn == cm * cn) return r;
  const int rows_left = a.M - (int)fm * BM, cols_left = a.n_out - (int)fn * BN;
  r.plan.main_tiles_n = (int)fn;
  r.plan.main_tiles_m = (int)fm;
  r.plan.bottom_tiles_m = (rows_left + EBM - 1) / EBM;
  r.plan.bottom_tiles_n = rows_left ? (a.n_out + EBN - 1) / EBN : 0;
  r.plan.right_tiles_n = (cols_left + RBN - 1) / RBN;
  r.plan.right_tiles_m = cols_left ? ((int)fm * BM + RBM - 1) / RBM : 0;
  const long long edge = (long long)r.plan.bottom_tiles_m * r.plan.bottom_tiles_n + (long long)r.plan.right_tiles_m * r.plan.right_tiles_n;
  r.workgroups = (int)(fm * fn + edge);
  constexpr double kEdgeCost = 0.2;
  const long long rounds_f = (fm * fn + slots - 1) / slots, rounds_c = (cm * cn + slots - 1) / slots;
  const long long idle = rounds_f * slots - fm * fn;           // slots the whole tiles leave, a main tile's time each
  const long long tail = edge - idle * (long long)(1.0 / kEdgeCost);
  const double ragged_time = (double)rounds_f + (tail > 0 ? (double)((tail + slots - 1) / slots) * kEdgeCost : 0.0);
  const double plain_time = (double)rounds_c * plain_cost;
  // (measurement ids 351 and 361 .. 368: whenever there is a whole main tile)
  r.use = ragged_time + 0.02 < plain_time || ov == 351 || (ov >= 361 && ov <= 368);
  return r;
}

// Main tile BM x BN with WM x WN waves; the edge tiles are 64 x 128 below and 128 x 64 to the right,
// with the same number of waves.
template <int BM, int BN, int WM, int WN, int NSTAGE, bool NT, bool AMAX>
int launch_big_ragged_as(const GemmArgs& a, const Ragged& r, hipStream_t st) {
  constexpr bool eight = WM * WN == 8;
  constexpr int EWM = 2, EWN = eight ? 4 : 2, ES = 3;              // 64 x 128 (three stages: a small tile's K loop waits for its loads, not for its products)
  constexpr int RWM = eight ? 4 : 2, RWN = 2, RS = 3;              // 128 x 64
  using Cfg = BigCfg<BM, BN, WM, WN, NSTAGE>;
  using ECfg = BigCfg<64, 128, EWM, EWN, ES>;
  using RCfg = BigCfg<128, 64, RWM, RWN, RS>;
  constexpr int lds = Cfg::kLdsBytes > ECfg::kLdsBytes ? (Cfg::kLdsBytes > RCfg::kLdsBytes ? Cfg::kLdsBytes : RCfg::kLdsBytes)
                                                       : (ECfg::kLdsBytes > RCfg::kLdsBytes ? ECfg::kLdsBytes : RCfg::kLdsBytes);
  auto kernel = gemm_mfma32_ragged_kernel<BM, BN, WM, WN, NSTAGE, 64, 128, EWM, EWN, ES, 128, 64, RWM, RWN, RS, NT, AMAX>;
  static std::atomic<uint64_t> lds_done{0};
  const int lds_status = allow_lds(kernel, lds, lds_done);
  if(lds_status != MARIAN_HIP_OK) return lds_status;
  GemmArgs a2 = a;
  a2.absmax_used = r.workgroups;
  hipLaunchKernelGGL(kernel, dim3(r.workgroups), dim3(Cfg::kThreads), lds, st, a2, r.plan);
  MH_HIP(hipGetLastError());
  if(AMAX) t_absmax_written = true;
  return MARIAN_HIP_OK;
}

// The launch for a main tile shape: ragged where that saves a round, else whole and partial tiles alike.
template <int BM, int BN, int WM, int WN, int NSTAGE, bool NT>
int launch_big_auto(const GemmArgs& a, hipStream_t st, int per_cu) {
  const Ragged r = plan_ragged(a, BM, BN, 64, 128, 128, 64, per_cu);
  if(!r.use) return launch_big<BM, BN, WM, WN, NSTAGE, true, NT>(a, st);
  if(big_leaves_absmax(a, r.workgroups)) return launch_big_ragged_as<BM, BN, WM, WN, NSTAGE, NT, true>(a, r, st);
  return launch_big_ragged_as<BM, BN, WM, WN, NSTAGE, NT, false>(a, r, st);
}

// Two side-by-side 256x128 tiles per workgroup, the first written out while the second is multiplied.
inline bool pair_kernel_ok(const GemmArgs& a) {   // everything but the shape
  return !a.dump && !a.idx && a.K % PairCfg::BK == 0 && a.K / PairCfg::BK >= PairCfg::kSideBlocks &&
         (!a.bias || aligned(a.bias, 16));
}
inline bool pair_kernel_fits(const GemmArgs& a) {
  return pair_kernel_ok(a) && a.M % PairCfg::BM == 0 && a.n_out % (2 * PairCfg::BN) == 0;
}

template <bool NT, bool AMAX>
int launch_pair_as(const GemmArgs& a, hipStream_t st) {
  auto kernel = gemm_pair_kernel<NT, AMAX>;
  static std::atomic<uint64_t> lds_done{0};
  const int lds_status = allow_lds(kernel, PairCfg::kLdsBytes, lds_done);
  if(lds_status != MARIAN_HIP_OK) return lds_status;
  int pairs_n = a.n_out / (2 * PairCfg::BN);
  int tiles_m = a.M / PairCfg::BM;
  GemmArgs a2 = a;
  a2.absmax_used = pairs_n * tiles_m;
  hipLaunchKernelGGL(kernel, dim3(pairs_n * tiles_m), dim3(PairCfg::kThreads), PairCfg::kLdsBytes, st, a2,
                     pairs_n, tiles_m);
  MH_HIP(hipGetLastError());
  if(AMAX) t_absmax_written = true;
  return MARIAN_HIP_OK;
}

template <bool NT>
int launch_pair(const GemmArgs& a, hipStream_t st) {
  if(!pair_kernel_fits(a)) return launch_big<256, 256, 2, 4, 2>(a, st);
  if(big_leaves_absmax(a, (long long)(a.n_out / (2 * PairCfg::BN)) * (a.M / PairCfg::BM))) return launch_pair_as<NT, true>(a, st);
  return launch_pair_as<NT, false>(a, st);
}

template <bool NT, bool AMAX>
int launch_pair_ragged_as(const GemmArgs& a, const Ragged& r, hipStream_t st) {
  using ECfg = BigCfg<64, 128, 2, 2, 3>;
  using RCfg = BigCfg<128, 64, 2, 2, 3>;
  constexpr int lds = PairCfg::kLdsBytes > ECfg::kLdsBytes ? (PairCfg::kLdsBytes > RCfg::kLdsBytes ? PairCfg::kLdsBytes : RCfg::kLdsBytes)
                                                           : (ECfg::kLdsBytes > RCfg::kLdsBytes ? ECfg::kLdsBytes : RCfg::kLdsBytes);
  auto kernel = gemm_pair_ragged_kernel<NT, AMAX>;
  static std::atomic<uint64_t> lds_done{0};
  const int lds_status = allow_lds(kernel, lds, lds_done);
  if(lds_status != MARIAN_HIP_OK) return lds_status;
  // A tile pair fills the LDS of its CU, so small tiles behind the pairs would wait for pairs to
  // end; ahead of them they delay a few pairs by their own, short time (measurement id 352 keeps them
  // behind)
  RaggedPlan plan = r.plan;
  int workgroups = r.workgroups;
  const int n_small = r.workgroups - plan.main_tiles_n * plan.main_tiles_m;
  if(kernel_override() % 1000 != 352) {
    plan.lead = (n_small + 7) / 8 * 8;
    workgroups = plan.lead + plan.main_tiles_n * plan.main_tiles_m;
  }
  if(AMAX && workgroups > kAbsmaxSlots) return launch_pair_ragged_as<NT, false>(a, r, st);   // (one slot per workgroup)
  GemmArgs a2 = a;
  a2.absmax_used = workgroups;
  hipLaunchKernelGGL(kernel, dim3(workgroups), dim3(PairCfg::kThreads), lds, st, a2, plan);
  MH_HIP(hipGetLastError());
  if(AMAX) t_absmax_written = true;
  return MARIAN_HIP_OK;
}

// ---- small-M weight-streaming kernels on the 32x32x32 MFMA ----
inline int stream32_fused_lds_bytes(int mt32, int K) { return mt32 * 32 * K; }

// The fused form keeps the fp32 activations of the whole call in registers and their int8 form
// for all of K in LDS.
inline bool stream32_can_fuse(int64_t M, int64_t K) {
  const int mt32 = M <= 32 ? 1 : (M <= 64 ? 2 : 4);
  return M <= 128 && M * K <= kFusedMaxElems && stream32_fused_lds_bytes(mt32, (int)K) <= 64 * 1024;
}

struct FusedSrc {   // what the fused modes read and write besides GemmArgs
  const float* A = nullptr;
  int8_t* aq_out = nullptr;
  const float* partials = nullptr;
  int n_partials = 0;
};

// Several weight matrices behind one activation tensor: the table the kernel reads, built for
// `cols` output columns per workgroup.
struct GroupLaunch {
  GroupTable table;
  int cols;
};

template <int MT32, int WN, int KW, int PW, int MODE, int ROWS = 32 * MT32, int NG = 4>
int launch_stream32(const GemmArgs& a, const FusedSrc& f, hipStream_t st, const GroupLaunch* groups = nullptr) {
  if constexpr(MODE == kFusedAll && NG == 4) {   // at most two groups of 16 values per thread
    if((long long)a.M * a.K <= kFusedMaxElems / 2)
      return launch_stream32<MT32, WN, KW, PW, MODE, ROWS, 2>(a, f, st);
  }
  using Cfg = Stream32Cfg<MT32, WN, KW, PW>;
  auto kernel = gemm_stream32_kernel<MT32, WN, KW, PW, MODE, NG, ROWS>;
  constexpr int kMaxLds = 64 * 1024 > Cfg::kLdsBytes ? 64 * 1024 : Cfg::kLdsBytes;
  static std::atomic<uint64_t> lds_done{0};
  const int lds_status = allow_lds(kernel, kMaxLds, lds_done);
  if(lds_status != MARIAN_HIP_OK) return lds_status;
  // (kFusedAll: all of K, and at least one whole chunk so that the first chunk needs no bounds)
  int lds = Cfg::kStageBytes;
  if(MODE == kFusedAll && lds < stream32_fused_lds_bytes(MT32, a.K)) lds = stream32_fused_lds_bytes(MT32, a.K);
  if(lds < Cfg::kReduceBytes) lds = Cfg::kReduceBytes;
  int blocks = (a.n_out + Cfg::kColsPerBlock - 1) / Cfg::kColsPerBlock;
  int m_tiles = (a.M + ROWS - 1) / ROWS;   // (kFusedAll with full-height tiles: M <= ROWS)
  GemmArgs a2 = a;
  if constexpr(MODE == kFusedTiled) {
    if(groups) {
      if(groups->cols != Cfg::kColsPerBlock) return MARIAN_HIP_ERR_SHAPE;   // (table built for another kernel)
      auto gkernel = gemm_stream32_kernel<MT32, WN, KW, PW, MODE, NG, ROWS, GroupTable>;
      static std::atomic<uint64_t> glds_done{0};
      const int glds_status = allow_lds(gkernel, kMaxLds, glds_done);
      if(glds_status != MARIAN_HIP_OK) return glds_status;
      a2.stream_out = 0;
      a2.absmax_out = nullptr;
      hipLaunchKernelGGL(gkernel, dim3(groups->table.block0[groups->table.n], m_tiles), dim3(Cfg::kThreads), lds, st,
                         a2, f.A, f.aq_out, f.partials, f.n_partials, groups->table);
      MH_HIP(hipGetLastError());
      return MARIAN_HIP_OK;
    }
  }
  // (measured: 10.0 instead of 11.1 us for the 8 MB output of the 64 x 32000 call; outputs of
  // less than a MB are up to 0.5 us slower with them.  The next kernel then finds the output in
  // HBM rather than in the memory-side cache: a log-softmax over 16 MB of logits takes 14.1
  // instead of 12.0 us, which is why the limit sits above the layer outputs of a decoder.)
  a2.stream_out = (long long)a.M * a.n_out * 4 >= (4ll << 20) ? 1 : 0;
  if(a.absmax_out) {   // one slot per wave
    if((long long)blocks * m_tiles * Cfg::kWaves <= kAbsmaxSlots) t_absmax_written = true;
    else a2.absmax_out = nullptr;
  }
  hipLaunchKernelGGL(kernel, dim3(blocks, m_tiles), dim3(Cfg::kThreads), lds, st, a2, f.A,
                     f.aq_out, f.partials, f.n_partials, NoGroups());
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

// Picks the number of K sub-steps a wave holds per chunk: the smallest instantiated value that
// covers K in one chunk, else the largest whose activations fit the 64 KB LDS stage
// (MT32 * KW * PW <= 64).  kFusedTiled stages fp32 values in registers: at most 4 per wave (8 when K is not split).
template <int MT32, int MODE>
int launch_stream32_kw(const GemmArgs& a, const FusedSrc& f, hipStream_t st, int kw, bool half_rows = false,
                       const GroupLaunch* g = nullptr) {
  const int need = (a.K / 32 + kw - 1) / kw;   // sub-steps per wave if K is one chunk
  if constexpr(MODE == kFusedTiled) {
    static_assert(MT32 == 1, "tiled fused form: 32 (or 16) rows per workgroup");
    switch(kw) {
      case 1: return launch_stream32<1, 8, 1, 8, MODE>(a, f, st, g);
      case 2: return launch_stream32<1, 4, 2, 4, MODE>(a, f, st, g);
      case 4:
        if(half_rows) return launch_stream32<1, 2, 4, 4, MODE, 16>(a, f, st, g);
        if(need > 4 && kernel_override() % 1000 != 690)
          return launch_stream32<1, 2, 4, 8, MODE>(a, f, st, g);   // long rows: half as many chunks (measurement id 690 keeps the shorter ones)
        return launch_stream32<1, 2, 4, 4, MODE>(a, f, st, g);
      default:
        if(need > 4 && half_rows && kernel_override() % 1000 != 670)
          return launch_stream32<1, 1, 8, 8, MODE, 16>(a, f, st, g);   // long rows: half as many chunks (measurement id 670 keeps the shorter ones)
        if(need > 2) {
          if(half_rows) return launch_stream32<1, 1, 8, 4, MODE, 16>(a, f, st, g);
          return launch_stream32<1, 1, 8, 4, MODE>(a, f, st, g);
        }
        if(half_rows) return launch_stream32<1, 1, 8, 2, MODE, 16>(a, f, st, g);
        return launch_stream32<1, 1, 8, 2, MODE>(a, f, st, g);
    }
  } else {
    switch(kw) {
      case 1: return launch_stream32<MT32, 8, 1, 8, MODE>(a, f, st);
      case 2: return launch_stream32<MT32, 4, 2, 8, MODE>(a, f, st);
      case 4:
        if constexpr(MT32 <= 2) {
          if(need > 4) return launch_stream32<MT32, 2, 4, 8, MODE>(a, f, st);
        }
        return launch_stream32<MT32, 2, 4, 4, MODE>(a, f, st);
      default:
        if constexpr(MT32 == 1 && MODE == kFusedAll) {
          if(half_rows) {
            if(need > 4) return launch_stream32<1, 1, 8, 8, MODE, 16>(a, f, st);
            if(need > 2) return launch_stream32<1, 1, 8, 4, MODE, 16>(a, f, st);
            return launch_stream32<1, 1, 8, 2, MODE, 16>(a, f, st);
          }
        }
        if constexpr(MT32 == 1) {
          if(need > 4) return launch_stream32<MT32, 1, 8, 8, MODE>(a, f, st);
        }
        if constexpr(MT32 <= 2) {
          if(need > 2) return launch_stream32<MT32, 1, 8, 4, MODE>(a, f, st);
        }
        return launch_stream32<MT32, 1, 8, 2, MODE>(a, f, st);
    }
  }
}

// The K split and the tile height of the tiled fused form for a call.  K split: the widest (most
// loads in flight per weight row) that stays within one workgroup per CU, the narrowest if none
// does.  Every workgroup quantizes the activation rows it multiplies; with 16 rows instead of 32
// that work halves and the workgroups double - taken when they still fit one per CU.
struct TiledPlan {
  int kw;
  bool half_rows;
};
TiledPlan plan_tiled(int M, int K, int n_out, int kw_override) {
  const int tiles = (n_out + 31) / 32, m_tiles = (M + 31) / 32;
  int kw = 8;
  while(kw > 1 && (long long)((tiles * kw + 7) / 8) * m_tiles > compute_units()) kw >>= 1;
  if(kw_override) kw = kw_override;
  while(kw > 1 && K / 32 < kw) kw >>= 1;
  const int ov = kernel_override() % 1000;   // 640 / 641: force 32 / 16 rows
  const long long blocks32 = (long long)((tiles * kw + 7) / 8) * m_tiles;
  const bool half_rows = kw >= 4 && ov != 640 && (ov == 641 || (M > 16 && 2 * blocks32 <= compute_units()));
  return TiledPlan{kw, half_rows};
}

// kw_override: 0 = pick the K split from the number of workgroups it gives.
// mt_override: 0 = activation rows per workgroup chosen here (kFusedAll takes all of M,
// kFusedTiled 32).
template <int MODE>
int launch_stream32_auto(const GemmArgs& a, const FusedSrc& f, hipStream_t st, int kw_override,
                         int mt_override = 0) {
  const int tiles = (a.n_out + 31) / 32;
  int mt = a.M <= 32 ? 1 : (a.M <= 64 ? 2 : 4);
  if(MODE == kPrequant) {
    // few weight tiles: split M over workgroups as well, so that more CUs pull on the operands
    // and each workgroup stages fewer activation rows
    if(tiles < 256 && mt > 1) mt = 1;
    if(mt_override) mt = mt_override;
  }
  if(MODE == kFusedTiled) mt = 1;
  const int m_tiles = MODE == kFusedAll ? 1 : (a.M + mt * 32 - 1) / (mt * 32);
  // the widest K split (most loads in flight per weight row) that stays within one workgroup
  // per CU; the narrowest if none does
  int kw = 8;
  while(kw > 1 && (long long)((tiles * kw + 7) / 8) * m_tiles > compute_units()) kw >>= 1;
  if(kw_override) kw = kw_override;
  while(kw > 1 && a.K / 32 < kw) kw >>= 1;
  if constexpr(MODE == kFusedTiled) {
    const TiledPlan plan = plan_tiled(a.M, a.K, a.n_out, kw_override);
    return launch_stream32_kw<1, MODE>(a, f, st, plan.kw, plan.half_rows);
  } else {
    if constexpr(MODE == kFusedAll) {
      // The smallest inputs (at most two 16-value groups per thread of four waves): one wave per
      // SIMD.  The kernel is a chain of short dependent phases there, bound by instruction issue,
      // and a wave that has its SIMD to itself issues twice as fast.  (K up to 1024: one chunk.)
      // (measurement ids 660 / 661 force eight / four waves)
      {
        const int ov = kernel_override() % 1000;
        const int S = a.K / 32;
        const bool four = !kw_override && ov != 660 && ov != 650 && ov != 651 && S >= 8 && S <= 32 &&
                          (long long)a.M * a.K <= 2 * 16 * 256 && a.M <= 32 &&
                          (ov == 661 || tiles <= compute_units());
        if(four) {
          const int need = (S + 3) / 4;
          if(need > 4) return launch_stream32<1, 1, 4, 8, MODE, 32, 2>(a, f, st);
          if(need > 2) return launch_stream32<1, 1, 4, 4, MODE, 32, 2>(a, f, st);
          return launch_stream32<1, 1, 4, 2, MODE, 32, 2>(a, f, st);
        }
      }
      // Few weight tiles: 16-row workgroups (all of them take the abs-max over the whole input,
      // each quantizes and multiplies its own rows), if they fit one per CU with the widest K
      // split.  (measurement ids 650 / 651 force full-height / 16-row workgroups)
      const int ov = kernel_override() % 1000;
      const bool rows16 = a.K / 32 >= 8 && !kw_override && ov != 650 &&
                          (ov == 651 || (a.M > 16 && (long long)tiles * ((a.M + 15) / 16) <= compute_units()));
      if(rows16) return launch_stream32_kw<1, MODE>(a, f, st, 8, true);
    }
    if(mt == 1) return launch_stream32_kw<1, MODE>(a, f, st, kw);
    if(mt == 2) return launch_stream32_kw<2, MODE>(a, f, st, kw);
    return launch_stream32_kw<4, MODE>(a, f, st, kw);
  }
}

// wide: many weight rows, every wave streams its own rows over the whole K
// narrow: few weight rows, the four waves split K and reduce
template <int MT>
int launch_stream_mt(const GemmArgs& a, hipStream_t st, bool wide) {
  if(wide) return launch_stream<MT, 2, 4, 1, 4>(a, st);
  return launch_stream<MT, 1, 1, 4, (MT >= 8 ? 1 : 2)>(a, st);
}

int launch_stream_auto(const GemmArgs& a, hipStream_t st, int force_wide) {
  const int n_tiles = (a.n_out + 15) / 16;
  bool wide = n_tiles >= 1024;
  if(force_wide == 1) wide = true;
  if(force_wide == 2) wide = false;
  if(a.M <= 16) return launch_stream_mt<1>(a, st, wide);
  if(a.M <= 32) return launch_stream_mt<2>(a, st, wide);
  if(a.M <= 64) return launch_stream_mt<4>(a, st, wide);
  return launch_stream_mt<8>(a, st, wide);
}

int launch_gemm(const GemmArgs& a, hipStream_t st) {
#ifdef MARIAN_HIP_TUNING
  const int which = kernel_override() % 1000;
  switch(which) {
    case 101: if(a.M <= 128) return launch_stream_auto(a, st, 1); break;
    case 102: if(a.M <= 128) return launch_stream_auto(a, st, 2); break;
    case 301: return launch_big<256, 256, 2, 4, 2>(a, st);
    case 302: return launch_big<128, 128, 2, 2, 2>(a, st);
    case 303: return launch_big<256, 128, 2, 2, 2>(a, st);
    case 304: return launch_big<256, 128, 4, 2, 2>(a, st);
    case 305: return launch_big<128, 256, 2, 2, 2>(a, st);
    case 306: return launch_big<256, 256, 2, 2, 2, false>(a, st);
    case 315: return launch_big<256, 256, 2, 4, 2, false>(a, st);
    case 316: return launch_big<256, 128, 2, 2, 2, false>(a, st);
    case 317: return launch_big<128, 256, 2, 2, 2, false>(a, st);
    case 330: return launch_pair<false>(a, st);
    case 331: return launch_pair<true>(a, st);
    case 307: return launch_big<128, 128, 2, 2, 3>(a, st);
    case 308: return launch_big<256, 128, 2, 2, 3>(a, st);
    case 309: return launch_big<128, 64, 2, 2, 2>(a, st);
    case 310: return launch_big<64, 128, 2, 2, 2>(a, st);
    case 311: return launch_big<128, 128, 4, 2, 2>(a, st);
    case 312: return launch_big<128, 128, 2, 4, 2>(a, st);
    case 313: return launch_big<128, 64, 2, 2, 3>(a, st);
    case 314: return launch_big<128, 64, 4, 2, 2>(a, st);
    // 361 .. 368: a main tile shape with small tiles for the rest wherever a whole main tile exists
    // (plain and non-temporal stores); shapes or calls the form does not take fall through
    case 361: case 365:
      if(pair_kernel_ok(a)) {
        const Ragged r = plan_ragged(a, PairCfg::BM, 2 * PairCfg::BN, 64, 128, 128, 64, 1);
        if(r.use) {
          if(big_leaves_absmax(a, r.workgroups)) return launch_pair_ragged_as<true, true>(a, r, st);
          return launch_pair_ragged_as<true, false>(a, r, st);
        }
      }
      break;
    case 362: return launch_big_auto<256, 256, 2, 4, 2, false>(a, st, 1);
    case 366: return launch_big_auto<256, 256, 2, 4, 2, true>(a, st, 1);
    case 363: return launch_big_auto<128, 128, 2, 4, 2, false>(a, st, 2);
    case 367: return launch_big_auto<128, 128, 2, 4, 2, true>(a, st, 2);
    // 371 .. 377: the split form (whole K blocks; other calls fall through)
    case 371: if(a.K % 128 == 0) return launch_big_split<128, 128, 2, 2, 3, false>(a, st); break;
    case 372: if(a.K % 128 == 0) return launch_big_split<128, 128, 2, 2, 3, true>(a, st); break;
    case 373: if(a.K % 128 == 0) return launch_big_split<128, 128, 2, 2, 4, true>(a, st); break;
    case 375: if(a.K % 128 == 0) return launch_big_split<128, 64, 2, 2, 3, true>(a, st); break;
    case 376: if(a.K % 128 == 0) return launch_big_split<128, 64, 2, 2, 4, true>(a, st); break;
    case 377: if(a.K % 128 == 0) return launch_big_split<128, 64, 2, 2, 4, false>(a, st); break;
    case 374: if(a.K % 128 == 0) return launch_big_split<128, 128, 2, 2, 4, false>(a, st); break;
    case 364: return launch_big_auto<128, 128, 2, 2, 3, false>(a, st, 1);
    case 368: return launch_big_auto<128, 128, 2, 2, 3, true>(a, st, 1);
    case 501: return launch_stream32_auto<kPrequant>(a, FusedSrc(), st, 0);
    case 521: return launch_stream32_auto<kPrequant>(a, FusedSrc(), st, 0, 1);
    case 522: return launch_stream32_auto<kPrequant>(a, FusedSrc(), st, 0, 2);
    case 524: return launch_stream32_auto<kPrequant>(a, FusedSrc(), st, 0, 4);
    case 511: return launch_stream32_auto<kPrequant>(a, FusedSrc(), st, 1);
    case 512: return launch_stream32_auto<kPrequant>(a, FusedSrc(), st, 2);
    case 514: return launch_stream32_auto<kPrequant>(a, FusedSrc(), st, 4);
    case 518: return launch_stream32_auto<kPrequant>(a, FusedSrc(), st, 8);
    default: break;
  }
#endif
  // Small M (decode): the weights are streamed once, the activations sit in LDS.
  //  - up to 8 rows (16 for narrow outputs): the 16x16x64 MFMA kernel, one 16-row tile
  //  - otherwise the 32x32x32 MFMA kernel, which also tiles M (shortlisted output layer, M = 256)
  const int tiles32 = (a.n_out + 31) / 32;
  if(a.M <= 8 || (a.M <= 16 && tiles32 < 512)) return launch_stream_auto(a, st, 2);
  //    (few columns, M up to 512; beyond 256 rows with K >= 2048 and 1024 or more columns the
  //    128x64-tile kernel below is 20 % faster)
  if(a.M <= 128 || (a.M <= 512 && tiles32 < 128 &&
                    (a.M <= 256 || a.K < 2048 || tiles32 < 32)))
    return launch_stream32_auto<kPrequant>(a, FusedSrc(), st, 0);
  // large outputs: 256x256 tiles (one per CU keeps operand traffic lowest); otherwise 128x128
  // tiles with a three-deep LDS ring so that enough loads are in flight per CU
  const long long tiles256 = ((a.M + 255) / 256) * (long long)((a.n_out + 255) / 256);
  // an output that would fit the L2 caches (8 x 4 MB) is streamed out with non-temporal stores
  const bool stream_out = (long long)a.M * a.n_out * 4 <= (32ll << 20) && !a.dump;
  if(tiles256 >= 192) {
    // short K: the fp32 output is most of the bytes; write one tile out while the next is multiplied
    if(a.K <= 1536 && kernel_override() % 1000 != 332) {
      if(pair_kernel_fits(a)) return launch_pair<true>(a, st);
      if(pair_kernel_ok(a)) {   // whole tile pairs + small tiles for the rest (the 256x256-tile kernel,
                                // which would take the output otherwise, is about a tenth slower per tile)
        const Ragged r = plan_ragged(a, PairCfg::BM, 2 * PairCfg::BN, 64, 128, 128, 64, 1, 1.1);
        if(r.use) {
          if(big_leaves_absmax(a, r.workgroups)) return launch_pair_ragged_as<true, true>(a, r, st);
          return launch_pair_ragged_as<true, false>(a, r, st);
        }
      }
    }
    if(stream_out) return launch_big_auto<256, 256, 2, 4, 2, true>(a, st, 1);
    return launch_big_auto<256, 256, 2, 4, 2, false>(a, st, 1);
  }
  // two or more 128x128 tiles per CU: eight waves and two LDS stages, so that two workgroups share
  // a CU and one multiplies while the other writes its tile out; otherwise four waves, three stages
  const long long tiles128 = ((a.M + 127) / 128) * (long long)((a.n_out + 127) / 128);
  if(tiles128 >= 2 * compute_units()) {
    if(stream_out) return launch_big_auto<128, 128, 2, 4, 2, true>(a, st, 2);
    return launch_big_auto<128, 128, 2, 4, 2, false>(a, st, 2);
  }
  // so few 128x128 tiles that half the CUs would idle: 128x64 tiles (measured -20 % to -25 % for
  // M = 512 .. 1024, K = 4096, N = 1024; measurement id 340 keeps the square tiles)
  // Tiles of which a CU gets one: whole K blocks go to the split form - four more waves per workgroup
  // issue the loads, the multiplying waves spend no issue slots on them (measured -6 % to -10 %;
  // measurement id 369 keeps the four-wave form, 378 takes the split form wherever K allows).  Only
  // where CUs stay idle: a chip full of eight-wave workgroups is ahead by 2 - 8 % on a machine that
  // has been idle (4096 x 4096 x 1024 19.9 against 21.1 us) and far behind on one that has not -
  // after a minute of other launches 25 - 29 against 23 - 25 us, 4096 x 2048 x 1024 19 - 23 against
  // 14 us, 4096 x 6144 x 1024 31 - 32 against 29.5 us - while launches of fewer tiles than CUs keep
  // their gain in both states.
  const int ov_split = kernel_override() % 1000;
  const bool split = a.K % 128 == 0 && ov_split != 369 && (ov_split == 378 || tiles128 < compute_units());
  if(2 * tiles128 <= compute_units() && kernel_override() % 1000 != 340) {
    if(split) return stream_out ? launch_big_split<128, 64, 2, 2, 4, true>(a, st) : launch_big_split<128, 64, 2, 2, 4, false>(a, st);
    if(stream_out) return launch_big<128, 64, 2, 2, 3, true, true>(a, st);
    return launch_big<128, 64, 2, 2, 3>(a, st);
  }
  // A few rows or columns more than one 128x128 tile per CU: whole tiles plus small ones, by the
  // eight-wave form, two of whose workgroups share a CU - the small tiles then run beside the whole
  // ones from the start (measured: 2050 x 1024 x 2056 11.7 instead of 15.4 us with the four-wave form,
  // whose 96 KB of LDS leave no room for a second workgroup, and 17.3 us with 289 tiles alike).
  {
    const Ragged r = plan_ragged(a, 128, 128, 64, 128, 128, 64, 1);
    if(r.use) {
      const bool amax = big_leaves_absmax(a, r.workgroups);
      if(stream_out) return amax ? launch_big_ragged_as<128, 128, 2, 4, 2, true, true>(a, r, st)
                                 : launch_big_ragged_as<128, 128, 2, 4, 2, true, false>(a, r, st);
      return amax ? launch_big_ragged_as<128, 128, 2, 4, 2, false, true>(a, r, st)
                  : launch_big_ragged_as<128, 128, 2, 4, 2, false, false>(a, r, st);
    }
  }
  if(split) return stream_out ? launch_big_split<128, 128, 2, 2, 3, true>(a, st) : launch_big_split<128, 128, 2, 2, 3, false>(a, st);
  if(stream_out) return launch_big<128, 128, 2, 2, 3, true, true>(a, st);
  return launch_big<128, 128, 2, 2, 3>(a, st);
}

int check_gemm(const int8_t* Aq, const int8_t* Bq, const void* out, const float* bias,
               const uint32_t* idx, int64_t n_idx, int64_t M, int64_t K, int64_t N) {
  if(M < 0 || K <= 0 || N < 0 || (K % 64) != 0 || (N % 8) != 0) return MARIAN_HIP_ERR_SHAPE;
  if(idx && (n_idx < 0 || (n_idx % 8) != 0)) return MARIAN_HIP_ERR_SHAPE;
  const int64_t n_out = idx ? n_idx : N;
  if(M == 0 || n_out == 0) return MARIAN_HIP_OK;  // empty batch: nothing is dereferenced
  if(!Aq || !Bq || !out) return MARIAN_HIP_ERR_NULL;
  if(M * K > kMaxElems || K * N > kMaxElems || M * n_out > kMaxElems) return MARIAN_HIP_ERR_RANGE;
  if(!aligned(Aq, 16) || !aligned(Bq, 16) || !aligned(out, 16)) return MARIAN_HIP_ERR_ALIGN;
  if((bias && !aligned(bias, 4)) || (idx && !aligned(idx, 4))) return MARIAN_HIP_ERR_ALIGN;
  return MARIAN_HIP_OK;
}

int run_gemm(const int8_t* Aq, const int8_t* Bq, const float* bias, const uint32_t* idx,
             int64_t n_idx, void* out, int64_t M, int64_t K, int64_t N, float scale, int relu,
             int dump, void* stream, float* absmax_out = nullptr) {
  int st = check_gemm(Aq, Bq, out, bias, idx, n_idx, M, K, N);
  if(st != MARIAN_HIP_OK) return st;
  const int64_t n_out = idx ? n_idx : N;
  if(M == 0 || n_out == 0) return MARIAN_HIP_OK;
  GemmArgs a;
  a.Aq = Aq; a.Bq = Bq; a.bias = bias; a.idx = idx; a.out = out;
  a.M = (int)M; a.K = (int)K; a.N = (int)N; a.n_out = (int)n_out;
  a.scale = scale; a.relu = relu ? 1 : 0; a.dump = dump;
#ifdef MARIAN_HIP_TUNING
  a.dbg = kernel_override() / 1000;
  a.prof = g_prof.load(std::memory_order_relaxed);
#endif
  a.absmax_out = absmax_out;
  return launch_gemm(a, reinterpret_cast<hipStream_t>(stream));
}

// One-pass prepareA: from this many values on (below, two launches are as fast or faster), how long a
// workgroup polls before it helps itself (each poll is a memory round trip of about a microsecond),
// and the nonce that starts its tags (random per process, so that words left in recycled device
// memory by another process do not match).
constexpr size_t kOnePassMinElems = 4u << 20;   // (measured: 8 MB of input - no gain; 16.8 MB: 10.3 -> 9.4 us; 67 MB: 30.4 -> 21.1 us)
constexpr int kOnePassSpinLimit = 20000;
unsigned next_nonce() {
  static std::atomic<unsigned> nonce{(unsigned)std::random_device{}() | 1u};
  return nonce.fetch_add(0x9E3779B1u, std::memory_order_relaxed);
}

int absmax_blocks(size_t n4) {
  size_t per_block = (size_t)kQuantThreads * 8;  // eight 16-byte loads per thread
  size_t g = (n4 + per_block - 1) / per_block;
  if(g < 1) g = 1;
  if(g > (size_t)kMaxPartials) g = kMaxPartials;
  return (int)g;
}

// Quantization of n values whose abs-max the producer left in kAbsmaxSlots slots (measurement id
// 710 keeps the narrow kernel for large inputs).
int quantize_with_known_absmax(const float* A, size_t n, const float* absmax_in, int8_t* Aq, hipStream_t st) {
  if(n >= (1u << 20) && n / 16 <= 0xFFFFFFFFull && kernel_override() % 1000 != 710) {
    // a 64 KB set per workgroup and step; up to four workgroups' worth of sets per CU at a time
    const size_t sets = (n / 64 + 255) / 256;
    size_t blocks = sets;
    if(blocks > 4 * (size_t)compute_units()) blocks = 4 * (size_t)compute_units();
    hipLaunchKernelGGL(quantize_a_wide_kernel, dim3((int)blocks), dim3(1024), 0, st, A, (unsigned)(n / 16), absmax_in,
                       (int)kAbsmaxSlots, Aq);
    MH_HIP(hipGetLastError());
    return MARIAN_HIP_OK;
  }
  size_t qblocks = (n / 16 + kQuantThreads - 1) / kQuantThreads;
  if(qblocks > 4096) qblocks = 4096;
  hipLaunchKernelGGL(quantize_a_kernel, dim3((int)qblocks), dim3(kQuantThreads), 0, st, A, n / 16, absmax_in,
                     (int)kAbsmaxSlots, Aq);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

}  // namespace

extern "C" {

const char* marian_hip_status_string(int status) {
  switch(status) {
    case MARIAN_HIP_OK: return "ok";
    case MARIAN_HIP_ERR_NULL: return "required pointer is null";
    case MARIAN_HIP_ERR_SHAPE: return "bad shape (need K % 64 == 0, N % 8 == 0, n_idx % 8 == 0, sizes >= 0)";
    case MARIAN_HIP_ERR_ALIGN: return "pointer alignment (16 bytes for matrices, 4 for bias/idx)";
    case MARIAN_HIP_ERR_WORKSPACE: return "workspace too small";
    case MARIAN_HIP_ERR_HIP: return "HIP runtime error";
    case MARIAN_HIP_ERR_RANGE: return "tensor too large for 32-bit element indices";
    case MARIAN_HIP_ERR_STATIC_LIMIT:
      return "activations exceed MARIAN_HIP_STATIC_MAX_ELEMS, the capacity of the library's static scratch";
    case MARIAN_HIP_ERR_ALIAS: return "input and output overlap";
    default: return "unknown status";
  }
}

int marian_hip_last_hip_error(void) { return g_last_hip_error; }

int marian_hip_int8_abi_version(void) { return 3; }

size_t marian_hip_int8_workspace_bytes(void) { return kWorkspaceBytes; }

#ifdef MARIAN_HIP_TUNING
int marian_hip_int8_set_kernel(int which) { return g_kernel_override.exchange(which); }

void marian_hip_int8_debug_profile(long long* p) { g_prof.store(p); }

int marian_hip_probe_stream(const void* src, size_t read_bytes, void* dst, size_t write_bytes, int workgroups,
                            int threads, int loads_in_flight, int nontemporal, void* stream) {
  if(!src || !dst) return MARIAN_HIP_ERR_NULL;
  if(workgroups <= 0 || threads <= 0 || threads > 1024 || threads % 64 != 0) return MARIAN_HIP_ERR_SHAPE;
  if(!aligned(src, 16) || !aligned(dst, 16)) return MARIAN_HIP_ERR_ALIGN;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const v4i* s = reinterpret_cast<const v4i*>(src);
  v4i* d = reinterpret_cast<v4i*>(dst);
  const size_t rv = read_bytes / 16, wv = write_bytes / 16;
#define MH_PROBE(U, NT) hipLaunchKernelGGL((probe_stream_kernel<U, NT>), dim3(workgroups), dim3(threads), 0, st, s, rv, d, wv)
  if(loads_in_flight >= 8) { if(nontemporal) MH_PROBE(8, true); else MH_PROBE(8, false); }
  else if(loads_in_flight >= 4) { if(nontemporal) MH_PROBE(4, true); else MH_PROBE(4, false); }
  else { if(nontemporal) MH_PROBE(1, true); else MH_PROBE(1, false); }
#undef MH_PROBE
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_probe_mfma(const void* data, int iters, int workgroups, long long* clocks, int* sink, void* stream) {
  if(!data || !clocks || !sink) return MARIAN_HIP_ERR_NULL;
  if(iters <= 0 || workgroups <= 0) return MARIAN_HIP_ERR_SHAPE;
  hipLaunchKernelGGL(probe_mfma_kernel, dim3(workgroups), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                     reinterpret_cast<const v4i*>(data), iters, clocks, sink);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_probe_mix(const void* src, size_t span_bytes, size_t stagger_bytes, int waves, int reads, int mfmas, int dmas, int gloads,
                         int split, int iters, int workgroups, long long* clocks, int* sink, void* stream) {
  if(!src || !clocks || !sink) return MARIAN_HIP_ERR_NULL;
  if(iters <= 0 || workgroups <= 0 || (waves != 4 && waves != 8 && waves != 16)) return MARIAN_HIP_ERR_SHAPE;
  if((mfmas > 0 && waves > 8) || (split && waves != 8)) return MARIAN_HIP_ERR_SHAPE;
  if(span_bytes < 65536 || (span_bytes & (span_bytes - 1)) != 0 || span_bytes > (1ull << 31)) return MARIAN_HIP_ERR_SHAPE;
  if(stagger_bytes % 1024 != 0 || stagger_bytes > span_bytes) return MARIAN_HIP_ERR_SHAPE;
  if(!aligned(src, 16)) return MARIAN_HIP_ERR_ALIGN;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  constexpr int kLds = 128 * 1024;
#define MH_MIX(R, M, D, G) MH_MIX2(R, M, D, G, false)
#define MH_MIX2(R, M, D, G, S)                                                                                  \
  if(reads == R && mfmas == M && dmas == D && gloads == G && (split != 0) == S) {                              \
    auto kernel = probe_mix_kernel<R, M, D, G, S>;                                                             \
    static std::atomic<uint64_t> lds_done{0};                                                                  \
    const int lds_status = allow_lds(kernel, kLds, lds_done);                                                  \
    if(lds_status != MARIAN_HIP_OK) return lds_status;                                                         \
    hipLaunchKernelGGL(kernel, dim3(workgroups), dim3(waves * 64), kLds, st, reinterpret_cast<const int8_t*>(src), \
                       (unsigned)span_bytes, (unsigned)stagger_bytes, iters, clocks, sink);                                             \
    MH_HIP(hipGetLastError());                                                                                 \
    return MARIAN_HIP_OK;                                                                                      \
  }
  MH_MIX(16, 0, 0, 0) MH_MIX(16, 0, 8, 0) MH_MIX(16, 0, 4, 0)
  MH_MIX(0, 0, 16, 0) MH_MIX(0, 0, 0, 16) MH_MIX(0, 0, 8, 8)
  MH_MIX(0, 8, 0, 0) MH_MIX(4, 8, 0, 0) MH_MIX(6, 8, 0, 0) MH_MIX(8, 8, 0, 0) MH_MIX(12, 8, 0, 0) MH_MIX(16, 8, 0, 0)
  MH_MIX(0, 8, 4, 0) MH_MIX(0, 8, 8, 0) MH_MIX(0, 8, 0, 4) MH_MIX(0, 8, 0, 8)
  MH_MIX(8, 8, 4, 0) MH_MIX(6, 8, 3, 0) MH_MIX(6, 8, 2, 0) MH_MIX(4, 8, 1, 2) MH_MIX(4, 8, 2, 2) MH_MIX(4, 8, 2, 4)
  MH_MIX2(8, 8, 4, 0, true) MH_MIX2(6, 8, 3, 0, true) MH_MIX2(0, 8, 4, 0, true) MH_MIX2(8, 8, 3, 0, true)
  MH_MIX(8, 8, 3, 0) MH_MIX(8, 8, 2, 0) MH_MIX2(8, 8, 2, 0, true) MH_MIX(12, 8, 4, 0)
#undef MH_MIX
#undef MH_MIX2
  return MARIAN_HIP_ERR_SHAPE;   // (a mix that is not instantiated)
}
#endif

int marian_hip_int8_prepare_a(const float* A, int8_t* Aq, int64_t M, int64_t K, void* workspace,
                              size_t workspace_bytes, void* stream) {
  if(M < 0 || K <= 0 || (K % 64) != 0) return MARIAN_HIP_ERR_SHAPE;
  if(M == 0) return MARIAN_HIP_OK;  // empty batch: nothing is dereferenced
  if(!A || !Aq) return MARIAN_HIP_ERR_NULL;
  if(M * K > kMaxElems) return MARIAN_HIP_ERR_RANGE;
  if(!aligned(A, 16) || !aligned(Aq, 16)) return MARIAN_HIP_ERR_ALIGN;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const size_t n = (size_t)M * (size_t)K;
  if(n <= (size_t)kSingleBlockMaxElems) {
    hipLaunchKernelGGL(prepare_a_single_block_kernel, dim3(1), dim3(kSingleBlockThreads), 0, st,
                       A, (int)(n / 16), Aq);
    MH_HIP(hipGetLastError());
    return MARIAN_HIP_OK;
  }
  if(!workspace) return MARIAN_HIP_ERR_NULL;
  if(workspace_bytes < kWorkspaceBytes) return MARIAN_HIP_ERR_WORKSPACE;
  if(!aligned(workspace, 8)) return MARIAN_HIP_ERR_ALIGN;
  // One pass over the input where it fits the register files of the chip's CUs (one workgroup per
  // CU: 16.7 M values on 256 CUs) and is large enough for the second read to cost more than the
  // exchange of the abs-max between the workgroups (measurement ids 700 / 701 force two passes /
  // one pass; 702: one pass with no patience, every workgroup scans the whole input itself).
  {
    const int ov = kernel_override() % 1000;
    const int cus = compute_units() < kOnePassMaxGroups ? compute_units() : kOnePassMaxGroups;
    const size_t n16 = n / 16;
    int sets = 1;
    while(sets < 4 && (n16 + 1024 * (size_t)sets - 1) / (1024 * (size_t)sets) > (size_t)cus) sets *= 2;
    const size_t groups = (n16 + 1024 * (size_t)sets - 1) / (1024 * (size_t)sets);
    const bool fits = groups <= (size_t)cus;
    if(fits && ov != 700 && (n >= kOnePassMinElems || ov == 701 || ov == 702)) {
      unsigned char* ws = reinterpret_cast<unsigned char*>(workspace);
      unsigned long long* slots = reinterpret_cast<unsigned long long*>(ws + kOnePassSlotsOffset);
      unsigned long long* gen = reinterpret_cast<unsigned long long*>(ws + kOnePassGenOffset);
      unsigned long long* mail = reinterpret_cast<unsigned long long*>(ws + kOnePassMailOffset);
      const unsigned nonce = next_nonce();
      const int spins = ov == 702 ? 0 : kOnePassSpinLimit;
      if(sets == 1)
        hipLaunchKernelGGL(prepare_a_onepass_kernel<1>, dim3((int)groups), dim3(1024), 0, st, A, (unsigned)n16, Aq, slots, gen, mail, nonce, spins);
      else if(sets == 2)
        hipLaunchKernelGGL(prepare_a_onepass_kernel<2>, dim3((int)groups), dim3(1024), 0, st, A, (unsigned)n16, Aq, slots, gen, mail, nonce, spins);
      else
        hipLaunchKernelGGL(prepare_a_onepass_kernel<4>, dim3((int)groups), dim3(1024), 0, st, A, (unsigned)n16, Aq, slots, gen, mail, nonce, spins);
      MH_HIP(hipGetLastError());
      return MARIAN_HIP_OK;
    }
  }
  float* partials = reinterpret_cast<float*>(workspace);
  const int g = absmax_blocks(n / 4);
  hipLaunchKernelGGL(absmax_partial_kernel, dim3(g), dim3(kQuantThreads), 0, st, A, n / 4,
                     partials);
  MH_HIP(hipGetLastError());
  size_t qblocks = (n / 16 + kQuantThreads - 1) / kQuantThreads;
  if(qblocks > 4096) qblocks = 4096;
  hipLaunchKernelGGL(quantize_a_kernel, dim3((int)qblocks), dim3(kQuantThreads), 0, st, A, n / 16,
                     (const float*)partials, g, Aq);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_int8_prepare_b(const float* W, int8_t* Bq, int64_t K, int64_t N, void* workspace,
                              size_t workspace_bytes, void* stream) {
  if(K <= 0 || N <= 0 || (K % 64) != 0 || (N % 8) != 0) return MARIAN_HIP_ERR_SHAPE;
  if(!W || !Bq || !workspace) return MARIAN_HIP_ERR_NULL;
  if(K * N > kMaxElems) return MARIAN_HIP_ERR_RANGE;
  if(!aligned(W, 16) || !aligned(Bq, 16) || !aligned(workspace, 4)) return MARIAN_HIP_ERR_ALIGN;
  if(workspace_bytes < kWorkspaceBytes) return MARIAN_HIP_ERR_WORKSPACE;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const size_t n = (size_t)K * (size_t)N;
  float* partials = reinterpret_cast<float*>(workspace);
  const int g = absmax_blocks(n / 4);
  hipLaunchKernelGGL(absmax_partial_kernel, dim3(g), dim3(kQuantThreads), 0, st, W, n / 4,
                     partials);
  MH_HIP(hipGetLastError());
  dim3 grid((unsigned)((N + 63) / 64), (unsigned)(K / 64));
  hipLaunchKernelGGL(quantize_b_transpose_kernel, grid, dim3(256), 0, st, W, (int)K, (int)N,
                     (const float*)partials, g, Bq);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_int8_prepare_b_quantized_transposed(const int8_t* in, int8_t* out, int64_t K,
                                                   int64_t N, void* stream) {
  if(!in || !out) return MARIAN_HIP_ERR_NULL;
  if(K <= 0 || N <= 0) return MARIAN_HIP_ERR_SHAPE;
  if((K % 64) != 0 || (N % 8) != 0) return MARIAN_HIP_ERR_SHAPE;
  if(K * N > kMaxElems) return MARIAN_HIP_ERR_RANGE;
  if(!aligned(in, 16) || !aligned(out, 16)) return MARIAN_HIP_ERR_ALIGN;
  // the two layouts are permutations of each other: not in place
  const uintptr_t a0 = reinterpret_cast<uintptr_t>(in), b0 = reinterpret_cast<uintptr_t>(out);
  const uintptr_t bytes = (uintptr_t)K * (uintptr_t)N + sizeof(float);
  if(a0 < b0 + bytes && b0 < a0 + bytes) return MARIAN_HIP_ERR_ALIAS;
  const size_t chunks = (size_t)K * (size_t)N / 16;
  hipLaunchKernelGGL(retile_b_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), in, (int)K, (int)N, out);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_int8_affine(const int8_t* Aq, const int8_t* Bq, const float* bias, float* out,
                           int64_t M, int64_t K, int64_t N, float scale, int relu, void* stream) {
  return run_gemm(Aq, Bq, bias, nullptr, 0, out, M, K, N, scale, relu, 0, stream);
}

static int affine_f32_impl(const float* A, int8_t* Aq, const int8_t* Bq, const float* bias,
                           const uint32_t* idx, int64_t n_idx, float* out, int64_t M, int64_t K,
                           int64_t N, float scale, int relu, const float* absmax_in,
                           float* absmax_out, void* workspace, size_t workspace_bytes,
                           void* stream) {
  int st = check_gemm(Aq, Bq, out, bias, idx, n_idx, M, K, N);
  if(st != MARIAN_HIP_OK) return st;
  const int64_t n_out = idx ? n_idx : N;
  if(M == 0) return MARIAN_HIP_OK;
  if(!A) return MARIAN_HIP_ERR_NULL;
  if(!aligned(A, 16)) return MARIAN_HIP_ERR_ALIGN;
  // Measurement ids: 600 = separate prepareA and GEMM launches; 611/612/614/618 = one fused
  // kernel with that K split; 620 = abs-max launch + tiled fused kernel, 621/622/624/628 with
  // that K split.
  const int which = kernel_override() % 1000;
  hipStream_t hst = reinterpret_cast<hipStream_t>(stream);
  GemmArgs a;
  a.Aq = Aq; a.Bq = Bq; a.bias = bias; a.idx = idx; a.out = out;
  a.M = (int)M; a.K = (int)K; a.N = (int)N; a.n_out = (int)n_out;
  a.scale = scale; a.relu = relu ? 1 : 0; a.dump = 0;
#ifdef MARIAN_HIP_TUNING
  a.prof = g_prof.load(std::memory_order_relaxed);
#endif
  a.absmax_out = absmax_out;
  FusedSrc f;
  f.A = A; f.aq_out = Aq;
  const bool want_tiled = which >= 620 && which <= 628;
  if(n_out > 0 && stream32_can_fuse(M, K) && which != 600 && !want_tiled) {
    int kw = 0;
    if(which >= 611 && which <= 618) kw = which - 610;
    return launch_stream32_auto<kFusedAll>(a, f, hst, kw);
  }
  // Mid-size activations: every workgroup quantizes its own 16 or 32 rows, so the work is
  // repeated once per 32..256 output columns; measured to pay (one launch fewer) for short rows
  // and moderate output widths, and for longer rows when few columns leave room for 16-row
  // workgroups with an eight-way K split (at most 64 K values per workgroup).
  const bool tiled_ok = n_out > 0 && workspace && workspace_bytes >= kWorkspaceBytes &&
                        aligned(workspace, 4);
  bool tiled = want_tiled;
  if(tiled_ok && !tiled && M <= 256 && n_out <= 8192) {
    const TiledPlan plan = plan_tiled((int)M, (int)K, (int)n_out, 0);
    tiled = K <= 1024 ||
            (K <= 4096 && plan.kw == 8 && (long long)(plan.half_rows ? 16 : 32) * K <= 65536);
  }
  if(tiled_ok && which != 600 && tiled) {
    if(absmax_in) {   // the producer of A left its abs-max: no launch for it
      f.partials = absmax_in;
      f.n_partials = kAbsmaxSlots;
    } else {
      const size_t n = (size_t)M * (size_t)K;
      float* partials = reinterpret_cast<float*>(workspace);
      const int g = absmax_blocks(n / 4);
      hipLaunchKernelGGL(absmax_partial_kernel, dim3(g), dim3(kQuantThreads), 0, hst, A, n / 4,
                         partials);
      MH_HIP(hipGetLastError());
      f.partials = partials;
      f.n_partials = g;
    }
    return launch_stream32_auto<kFusedTiled>(a, f, hst, want_tiled ? which - 620 : 0);
  }
  if(absmax_in) {   // quantize with the abs-max the producer left, then the GEMM
    st = quantize_with_known_absmax(A, (size_t)M * (size_t)K, absmax_in, Aq, hst);
    if(st != MARIAN_HIP_OK) return st;
  } else {
    st = marian_hip_int8_prepare_a(A, Aq, M, K, workspace, workspace_bytes, stream);
    if(st != MARIAN_HIP_OK) return st;
  }
  return run_gemm(Aq, Bq, bias, idx, n_idx, out, M, K, N, scale, relu, 0, stream, absmax_out);
}

// abs-max of a finished output for the next call, when the kernel that wrote it did not leave it
static int absmax_after(const float* out, int64_t M, int64_t n_out, float* absmax_out, hipStream_t st) {
  const size_t n = (size_t)M * (size_t)n_out;
  const int g = absmax_blocks(n / 4);   // n_out % 8 == 0; g <= 1024 partials
  hipLaunchKernelGGL(zero_floats_kernel, dim3(2), dim3(kQuantThreads), 0, st, absmax_out + g, kAbsmaxSlots - g);
  hipLaunchKernelGGL(absmax_partial_kernel, dim3(g), dim3(kQuantThreads), 0, st, out, n / 4, absmax_out);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_int8_affine_f32(const float* A, int8_t* Aq, const int8_t* Bq, const float* bias,
                               const uint32_t* idx, int64_t n_idx, float* out, int64_t M,
                               int64_t K, int64_t N, float scale, int relu, void* workspace,
                               size_t workspace_bytes, void* stream) {
  return affine_f32_impl(A, Aq, Bq, bias, idx, n_idx, out, M, K, N, scale, relu, nullptr, nullptr,
                         workspace, workspace_bytes, stream);
}

int marian_hip_int8_affine_f32_chained(const float* A, int8_t* Aq, const int8_t* Bq,
                                       const float* bias, const uint32_t* idx, int64_t n_idx,
                                       float* out, int64_t M, int64_t K, int64_t N, float scale,
                                       int relu, const float* absmax_in, float* absmax_out,
                                       void* workspace, size_t workspace_bytes, void* stream) {
  if((absmax_in && !aligned(absmax_in, 4)) || (absmax_out && !aligned(absmax_out, 4)))
    return MARIAN_HIP_ERR_ALIGN;
  t_absmax_written = false;
  int st = affine_f32_impl(A, Aq, Bq, bias, idx, n_idx, out, M, K, N, scale, relu, absmax_in,
                           absmax_out, workspace, workspace_bytes, stream);
  if(st != MARIAN_HIP_OK || !absmax_out || t_absmax_written) return st;
  const int64_t n_out = idx ? n_idx : N;
  if(M == 0 || n_out == 0) return MARIAN_HIP_OK;
  return absmax_after(out, M, n_out, absmax_out, reinterpret_cast<hipStream_t>(stream));
}


int marian_hip_int8_affine_f32_grouped(const float* A, int8_t* Aq, int64_t n_groups,
                                       const int8_t* const* Bq, const float* const* bias,
                                       float* const* out, const int64_t* N, int64_t M, int64_t K,
                                       float scale, int relu, const float* absmax_in, void* workspace,
                                       size_t workspace_bytes, void* stream) {
  if(n_groups < 1 || n_groups > kMaxGroups) return MARIAN_HIP_ERR_SHAPE;
  if(!Bq || !out || !N) return MARIAN_HIP_ERR_NULL;
  int64_t total_blocks32 = 0;
  for(int64_t g = 0; g < n_groups; ++g) {
    int st = check_gemm(Aq, Bq[g], out[g], bias ? bias[g] : nullptr, nullptr, 0, M, K, N[g]);
    if(st != MARIAN_HIP_OK) return st;
    total_blocks32 += (N[g] + 31) / 32;
  }
  if(absmax_in && !aligned(absmax_in, 4)) return MARIAN_HIP_ERR_ALIGN;
  if(M == 0) return MARIAN_HIP_OK;
  if(!A || !Aq) return MARIAN_HIP_ERR_NULL;
  if(!aligned(A, 16)) return MARIAN_HIP_ERR_ALIGN;
  hipStream_t hst = reinterpret_cast<hipStream_t>(stream);
  const bool have_ws = workspace && workspace_bytes >= kWorkspaceBytes && aligned(workspace, 4);
  // One launch for all matrices where the quantize-on-stage kernel takes the call (the same limits
  // as for a single matrix of the summed width).
  bool one_launch = false;
  TiledPlan plan{1, false};
  if(total_blocks32 > 0 && (absmax_in || have_ws) && M <= 256 && total_blocks32 * 32 <= 8192) {
    plan = plan_tiled((int)M, (int)K, (int)(total_blocks32 * 32), 0);
    one_launch = K <= 1024 || (K <= 4096 && plan.kw == 8 && (long long)(plan.half_rows ? 16 : 32) * K <= 65536);
  }
  if(one_launch) {
    GroupLaunch gl;
    gl.cols = 32 * (8 / plan.kw);
    gl.table.n = 0;
    gl.table.block0[0] = 0;
    for(int64_t g = 0; g < n_groups; ++g) {
      if(N[g] == 0) continue;
      const int i = gl.table.n++;
      gl.table.Bq[i] = Bq[g];
      gl.table.bias[i] = bias ? bias[g] : nullptr;
      gl.table.out[i] = out[g];
      gl.table.N[i] = (int)N[g];
      gl.table.block0[i + 1] = gl.table.block0[i] + (int)((N[g] + gl.cols - 1) / gl.cols);
    }
    for(int i = gl.table.n; i < kMaxGroups; ++i) {   // unused entries: never selected
      gl.table.Bq[i] = nullptr; gl.table.bias[i] = nullptr; gl.table.out[i] = nullptr; gl.table.N[i] = 0;
      gl.table.block0[i + 1] = gl.table.block0[gl.table.n];
    }
    GemmArgs a;
    a.Aq = Aq; a.Bq = gl.table.Bq[0]; a.bias = gl.table.bias[0]; a.idx = nullptr; a.out = gl.table.out[0];
    a.M = (int)M; a.K = (int)K; a.N = gl.table.N[0]; a.n_out = gl.table.N[0];
    a.scale = scale; a.relu = relu ? 1 : 0; a.dump = 0;
#ifdef MARIAN_HIP_TUNING
    a.prof = g_prof.load(std::memory_order_relaxed);
#endif
    FusedSrc f;
    f.A = A; f.aq_out = Aq;
    if(absmax_in) {
      f.partials = absmax_in;
      f.n_partials = kAbsmaxSlots;
    } else {
      const size_t n = (size_t)M * (size_t)K;
      float* partials = reinterpret_cast<float*>(workspace);
      const int g = absmax_blocks(n / 4);
      hipLaunchKernelGGL(absmax_partial_kernel, dim3(g), dim3(kQuantThreads), 0, hst, A, n / 4, partials);
      MH_HIP(hipGetLastError());
      f.partials = partials;
      f.n_partials = g;
    }
    return launch_stream32_kw<1, kFusedTiled>(a, f, hst, plan.kw, plan.half_rows, &gl);
  }
  // Otherwise the activations are quantized once and every matrix gets its own multiplication.
  if(absmax_in) {
    int st = quantize_with_known_absmax(A, (size_t)M * (size_t)K, absmax_in, Aq, hst);
    if(st != MARIAN_HIP_OK) return st;
  } else {
    int st = marian_hip_int8_prepare_a(A, Aq, M, K, workspace, workspace_bytes, stream);
    if(st != MARIAN_HIP_OK) return st;
  }
  for(int64_t g = 0; g < n_groups; ++g) {
    int st = run_gemm(Aq, Bq[g], bias ? bias[g] : nullptr, nullptr, 0, out[g], M, K, N[g], scale, relu, 0, stream);
    if(st != MARIAN_HIP_OK) return st;
  }
  return MARIAN_HIP_OK;
}

// ---- the entry point that allocates nothing -------------------------------------------------
// Device memory the call needs besides its inputs and outputs - the quantized activations with
// their quantMult tail, and the abs-max partials - lives in one file-scope array per GPU.  In host
// code the array's name is only a handle: its device address comes from hipGetSymbolAddress, once
// per device, and only that address is handed to kernels.
namespace {
constexpr size_t kStaticMaxElems = MARIAN_HIP_STATIC_MAX_ELEMS;
constexpr size_t kStaticAqBytes = kStaticMaxElems + 256;   // payload, tail, padding to 256
constexpr size_t kStaticBytes = kStaticAqBytes + kWorkspaceBytes;
}  // namespace
static __device__ __align__(256) unsigned char scratch[kStaticBytes];
namespace {
std::atomic<unsigned char*> g_scratch_ptr[kMaxDevices];

// Address of the current device's copy of `scratch` (looked up on the first call per device).
static int static_scratch(unsigned char** out) {
  int dev = 0;
  const int dst = current_device(&dev);
  if(dst != MARIAN_HIP_OK) return dst;
  unsigned char* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if(!p) {
    void* sym = nullptr;
    MH_HIP(hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)));
    if(!sym) return MARIAN_HIP_ERR_NULL;
    p = static_cast<unsigned char*>(sym);
    g_scratch_ptr[dev].store(p, std::memory_order_release);   // (every thread finds the same address)
  }
  *out = p;
  return MARIAN_HIP_OK;
}
}  // namespace

int marian_hip_int8_affine_f32_static(const float* A, const int8_t* Bq, const float* bias,
                                      const uint32_t* idx, int64_t n_idx, float* out, int64_t M,
                                      int64_t K, int64_t N, float scale, int relu, void* stream) {
  // sizes first, so that an oversized call is refused before anything touches the device
  if(M < 0 || K <= 0 || N < 0 || (K % 64) != 0 || (N % 8) != 0) return MARIAN_HIP_ERR_SHAPE;
  if(M > 0 && (uint64_t)M * (uint64_t)K > (uint64_t)kStaticMaxElems) return MARIAN_HIP_ERR_STATIC_LIMIT;
  if(M == 0) return MARIAN_HIP_OK;
  unsigned char* base = nullptr;
  int st = static_scratch(&base);
  if(st != MARIAN_HIP_OK) return st;
  int8_t* Aq = reinterpret_cast<int8_t*>(base);
  void* workspace = base + kStaticAqBytes;
  // The quantized activations and the abs-max partials are written earlier in the same call than
  // they are read.  The hand-over area of the one-pass prepareA (M * K >= 4 Mi: arrival slots,
  // generation word, mailboxes) is different: its words persist from call to call and are matched
  // by tag (a per-process nonce plus the generation word, top bit always set), so a word left by
  // an earlier call - or the zeros the array starts with - never passes for a fresh one.  Nothing
  // has to be cleared between calls.
  return affine_f32_impl(A, Aq, Bq, bias, idx, n_idx, out, M, K, N, scale, relu, nullptr, nullptr,
                         workspace, kWorkspaceBytes, stream);
}

int marian_hip_int8_affine_shortlist(const int8_t* Aq, const int8_t* Bq, const float* bias,
                                     const uint32_t* idx, int64_t n_idx, float* out, int64_t M,
                                     int64_t K, int64_t N, float scale, int relu, void* stream) {
  if(!idx) return MARIAN_HIP_ERR_NULL;
  return run_gemm(Aq, Bq, bias, idx, n_idx, out, M, K, N, scale, relu, 0, stream);
}

int marian_hip_int8_multiply_i32(const int8_t* Aq, const int8_t* Bq, const uint32_t* idx,
                                 int64_t n_idx, int32_t* acc, int64_t M, int64_t K, int64_t N,
                                 void* stream) {
  return run_gemm(Aq, Bq, nullptr, idx, idx ? n_idx : 0, acc, M, K, N, 1.0f, 0, 1, stream);
}

}  // extern "C"
