// extern "C" entry points of libgmlp.so (declared in include/gmlp.h): argument validation,
// tile-class selection and kernel launches.  All validation happens before the first HIP call,
// so the error paths can be exercised on a machine without a GPU.
#include "gmlp.h"

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <mutex>
#include <vector>

#include "launch.hpp"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

#define GMLP_REQUIRE_PTR(p)                                                         \
  if ((p) == nullptr) return fail(GMLP_EINVAL, "%s: argument '%s' is NULL", __func__, #p)
#define GMLP_REQUIRE_ALIGNED(p)                                                     \
  if ((p) != nullptr && !aligned16(p))                                              \
  return fail(GMLP_EALIGN, "%s: argument '%s' is not 16-byte aligned", __func__, #p)
#define GMLP_REQUIRE_DTYPE(d)                                                       \
  if ((d) != GMLP_F16 && (d) != GMLP_BF16 && (d) != GMLP_F32)                       \
  return fail(GMLP_EINVAL, "%s: dtype %d is not GMLP_F16/GMLP_BF16/GMLP_F32", __func__, (int)(d))

#define GMLP_REQUIRE_ACT(a)                                                         \
  if ((a) < 0 || (a) >= gmlp::ACT_COUNT)                                            \
  return fail(GMLP_EINVAL, "%s: act %d is not one of the GMLP_ACT_* codes", __func__, (int)(a))

static_assert(GMLP_COLSUM_STATIC_MAX_C == gmlp::COLSUM_STATIC_MAX_C, "public limit of gmlp_colsum_static");
static_assert((int)GMLP_ACT_SILU == (int)gmlp::ACT_SILU && (int)GMLP_ACT_GELU == (int)gmlp::ACT_GELU &&
                  (int)GMLP_ACT_RELU == (int)gmlp::ACT_RELU && (int)GMLP_ACT_LEAKY_RELU == (int)gmlp::ACT_LEAKY_RELU &&
                  (int)GMLP_ACT_SIGMOID == (int)gmlp::ACT_SIGMOID && (int)GMLP_ACT_TANH == (int)gmlp::ACT_TANH &&
                  (int)GMLP_ACT_IDENTITY == (int)gmlp::ACT_IDENTITY && gmlp::ACT_COUNT == 7,
              "device activation codes are the public ones");

const int64_t kMaxDim = (int64_t)1 << 30;

int check_dims(const char* fn, int64_t M, int64_t K, int64_t N) {
  if (M < 1 || K < 1 || N < 1) return fail(GMLP_ESHAPE, "%s: M, K, N must be >= 1 (got %lld, %lld, %lld)", fn,
                                           (long long)M, (long long)K, (long long)N);
  if (M > kMaxDim || K > kMaxDim || N > kMaxDim || M * N >= ((int64_t)1 << 40) ||
      M * K >= ((int64_t)1 << 40))
    return fail(GMLP_ESHAPE, "%s: dimension too large", fn);
  return 0;
}

int check_mult8(const char* fn, const char* name, int64_t v) {
  if (v % 8 != 0)
    return fail(GMLP_ESHAPE, "%s: %s = %lld must be a multiple of 8 (16-byte rows)", fn, name, (long long)v);
  return 0;
}

int make_dropout(const char* fn, float p, uint64_t seed, uint64_t offset, gmlp::DropoutParams* d) {
  if (!(p >= 0.0f) || !(p < 1.0f))
    return fail(GMLP_EINVAL, "%s: dropout_p = %g must satisfy 0 <= p < 1", fn, (double)p);
  d->enabled = p > 0.0f ? 1 : 0;
  double t = std::floor((double)p * 4294967296.0);
  d->threshold = t >= 4294967295.0 ? 4294967295u : (uint32_t)t;
  d->scale = 1.0f / (1.0f - p);
  d->seed_lo = (uint32_t)seed;
  d->seed_hi = (uint32_t)(seed >> 32);
  d->off_lo = (uint32_t)offset;
  d->off_hi = (uint32_t)(offset >> 32);
  return 0;
}

// Calls f(T{}) with T = the storage type named by `dtype` (already validated).
template <typename F>
hipError_t by_dtype(int dtype, F&& f) {
  if (dtype == GMLP_F16) return f(gmlp::f16{});
  if (dtype == GMLP_BF16) return f(gmlp::bf16{});
  return f(float{});
}

int hip_result(const char* fn, hipError_t e) {
  if (e == hipSuccess) return GMLP_OK;
  return fail(GMLP_EHIP, "%s: HIP error %d (%s)", fn, (int)e, hipGetErrorString(e));
}

// Scheduling groups of 8 tile-rows when the A operand (rows x red) is the smaller one, of 8
// tile-columns (negative) when B (cols x red, `sets` of them) is: see tile_of_grouped.
int pick_group(int64_t rows, int64_t cols, int sets = 1) { return sets * cols < rows ? -8 : 8; }

// Compute units of the current device.
int num_cu() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Accelerator dies (XCDs, each with an L2 of its own) behind the current device: the hardware
// deals consecutive workgroup ids round-robin to them.  A gfx950 XCD has 32 active compute units,
// so a whole MI355X shows 8 and a partition of it 4, 2 or 1.
int num_xcd() {
  int n = num_cu() / 32;
  return n < 1 ? 1 : n > 8 ? 8 : n;
}

// LARGE or MEDIUM_FULL for a grid of `large_tiles` large or `medium_tiles` small tiles, by
// estimated time in rounds of workgroups (see pick_tile).
int group_tile_class(int64_t large_tiles, int64_t medium_tiles) {
  auto rounds = [](int64_t tiles, int64_t slots) {
    double part = (double)(tiles % slots) / (double)slots;
    return (double)(tiles / slots) + (part > 0.0 ? 0.6 + 0.4 * part : 0.0);
  };
  const int64_t cus = num_cu();
  const double large_time = rounds(large_tiles, cus);
  const double medium_time = rounds(medium_tiles, 2 * cus) * (2.0 / 3.0);
  return large_time <= medium_time ? gmlp::TILE_LARGE : gmlp::TILE_MEDIUM_FULL;
}

// Tile class for an output of rows x cols with reduction length red (all in elements).
// The pipelined kernels (LARGE: 256 x bn_large tiles, one workgroup per CU; MEDIUM_FULL: tiles of
// half that in each direction, two per CU) take any rows and cols; they need 32-bit byte offsets
// into the operands, padded to whole tiles, and a reduction that is a multiple of 64 unless both
// operands are reduction-strided (`both_ks`).  Everything else runs on the predicated MEDIUM class.
// Between the two pipelined classes the choice is estimated time in rounds of workgroups: a round
// of small tiles (two per CU) takes 2/3 of a round of large ones (a quarter of the work at 75 % of
// the throughput, two at a time), and a last round filled to the fraction f costs 0.6 + 0.4 f of
// a full one (the busy CUs clock higher, but not in proportion; fitted to measurements).
int pick_tile(int dtype, int64_t rows, int64_t cols, int64_t red, int bn_large, bool both_ks = false) {
  if (dtype == GMLP_F32) return gmlp::TILE_MEDIUM;  // the float32 kernel has one tile shape
  auto up = [](int64_t v, int64_t q) { return (v + q - 1) / q * q; };
  // the buffer base sits up to 4 KB below the operand (shared-M0 loads)
  const int64_t limit = ((int64_t)1 << 31) - 4096;
  bool offsets_fit = up(rows, 256) * up(red, 64) * 2 < limit && up(cols, 256) * up(red, 64) * 2 < limit;
  if (!offsets_fit || (red % 64 != 0 && !both_ks)) return gmlp::TILE_MEDIUM;
  const int64_t large_tiles = (up(rows, 256) / 256) * (up(cols, bn_large) / bn_large);
  const int64_t medium_tiles = (up(rows, 128) / 128) * (up(cols, bn_large / 2) / (bn_large / 2));
  return group_tile_class(large_tiles, medium_tiles);
}

// Number of workgroups that should share one output tile of a rows x cols GEMM with `red_tiles`
// 64-wide reduction tiles, or 1.  A GEMM with a few output tiles and a long reduction (down
// projection and input gradient of a short batch) leaves most of the chip idle and is bound by
// streaming the weights; splitting the reduction fills two 128-tile workgroups per CU.  Each split
// keeps at least 8 reduction tiles.
int pick_splits(int dtype, int64_t rows, int64_t cols, int64_t red, int64_t red_tiles, int bn_large = 256) {
  if (pick_tile(dtype, rows, cols, red, bn_large) != gmlp::TILE_MEDIUM_FULL) return 1;
  const int64_t bn = bn_large / 2;
  const int64_t tiles = ((rows + 127) / 128) * ((cols + bn - 1) / bn);
  int64_t s = 2 * num_cu() / tiles;
  if (s > red_tiles / 8) s = red_tiles / 8;
  if (s > 16) s = 16;
  if (s < 2) return 1;
  // the kernel gives every split ceil(red_tiles / s) reduction tiles: drop the splits that this
  // leaves empty
  const int64_t per = (red_tiles + s - 1) / s;
  return (int)((red_tiles + per - 1) / per);
}

// For a rows x cols output on 256 x 256 tiles whose grid ends in a thinly filled round of
// workgroups (at most half full): the number of tile ROWS that make whole rounds, or 0.  The
// backward GEMMs read their weight operand reduction-strided, so they are cut along the rows of
// the output (token rows: every other operand is row-major in them) where the forward GEMMs are cut
// along the columns.
int64_t whole_round_tile_rows(int dtype, int64_t rows, int64_t cols, int64_t red) {
  if (dtype == GMLP_F32 || pick_tile(dtype, rows, cols, red, 256) != gmlp::TILE_LARGE) return 0;
  const int64_t tiles_m = (rows + 255) / 256, tiles_n = (cols + 255) / 256, cus = num_cu();
  const int64_t rounds = tiles_m * tiles_n / cus, tail = tiles_m * tiles_n % cus;
  const int64_t whole = rounds * cus / tiles_n;
  return rounds >= 1 && tail > 0 && 2 * tail <= cus && whole >= 1 && whole < tiles_m ? whole : 0;
}

// Stream-K plan for a grid of `tiles` large output tiles with `kt` 64-wide reduction tiles each
// (tiles of all problems of a grouped launch together).  The tiles beyond the last whole round of
// workgroups (one per compute unit) are shared out by reduction range when that beats running them
// as a thinly filled round: a round filled to the fraction f costs about 0.6 + 0.4 f of a full one
// (see pick_tile) against f with stream-K, plus the partial sums' round trip through memory and the
// second launch (about 45 us, i.e. 30 reduction tiles' time): worth it when (1 - f) * kt > 50.
// Every stream-K workgroup gets at least 8 reduction tiles.
struct StreamK {
  int tiles = 0, wgs = 0, chunks = 0;
  size_t ws_bytes = 0;
};
StreamK plan_streamk(int dtype, int64_t tiles, int64_t kt) {
  StreamK p;
  const int64_t cus = num_cu(), tail = tiles % cus;
  if (dtype == GMLP_F32 || tail == 0 || kt < 8) return p;
  if ((double)(cus - tail) / (double)cus * (double)kt <= 50.0) return p;
  int64_t wgs = tail * kt / 8;
  if (wgs > cus) wgs = cus;
  if (wgs < 1 || tail * kt >= ((int64_t)1 << 30)) return p;
  p.tiles = (int)tail;
  p.wgs = (int)wgs;
  // A whole number of pieces per tile when that still fills (nearly) all compute units: the
  // workgroups of an XCD then walk neighbouring tiles over the same reduction range and share
  // operand panels in L2 (measured on 128 tiles in halves: the pieces' launch 123 -> 116 us).
  const int64_t per_tile = wgs / tail;
  if (per_tile >= 2 && per_tile * tail * 10 >= wgs * 9 && kt / per_tile >= 8) {
    p.chunks = (int)per_tile;
    p.wgs = (int)(per_tile * tail);
  }
  p.ws_bytes = (size_t)(p.tiles + p.wgs) * 65536 * sizeof(float);  // 256 x 256 accumulators per slot
  return p;
}
// Applies the plan to a launch's arguments when the caller's workspace can hold it.
bool use_streamk(const StreamK& p, gmlp::GemmArgs& ga, void* workspace, size_t workspace_bytes) {
  if (p.tiles == 0 || workspace == nullptr || workspace_bytes < p.ws_bytes) return false;
  ga.sk_tiles = p.tiles;
  ga.sk_wgs = p.wgs;
  ga.sk_chunks = p.chunks;
  ga.sk_ws = (float*)workspace;
  return true;
}
int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

size_t split_workspace_bytes(int splits, int64_t rows, int64_t cols, int accumulator_sets = 1) {
  return splits > 1 ? (size_t)splits * accumulator_sets * rows * cols * sizeof(float) : 0;
}

std::mutex& lds_registry_mutex() {
  static std::mutex m;
  return m;
}
std::vector<gmlp::LdsKernel*>& lds_registry() {
  static std::vector<gmlp::LdsKernel*> v;
  return v;
}

}  // namespace

namespace gmlp {

LdsKernel::LdsKernel(const void* k, int b) : kernel(k), bytes(b), done{} {
  std::lock_guard<std::mutex> lock(lds_registry_mutex());
  lds_registry().push_back(this);
}

hipError_t prepare_lds_kernels() {
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev)) return e;
  std::lock_guard<std::mutex> lock(lds_registry_mutex());
  for (LdsKernel* k : lds_registry()) {
    if (hipError_t e = hipFuncSetAttribute(k->kernel, hipFuncAttributeMaxDynamicSharedMemorySize, k->bytes)) return e;
    if (dev >= 0 && dev < 64) k->done[dev].store(1, std::memory_order_release);
  }
  return hipSuccess;
}

}  // namespace gmlp

extern "C" {

int gmlp_abi_version(void) { return GMLP_ABI_VERSION; }
const char* gmlp_last_error(void) { return g_err; }

int gmlp_init(void) {
  (void)num_cu();
  if (hipError_t e = gmlp::prepare_lds_kernels()) return hip_result(__func__, e);
  float* scratch = nullptr;
  return hip_result(__func__, gmlp::colsum_static_scratch(&scratch, nullptr));
}

size_t gmlp_workspace_bytes(int op, int64_t M, int64_t K, int64_t N, int dtype) {
  // gmlp_dw_bwd_grouped: any set of problems (the plan depends on all of them together): the most
  // a plan can take, a slot per compute unit for the shared-out tiles and for the workgroups
  if (op == GMLP_OP_DW_BWD_GROUPED) return dtype == GMLP_F32 ? 0 : (size_t)2 * num_cu() * 65536 * sizeof(float);
  if (M < 1 || N < 1) return 0;
  if (op == GMLP_OP_COLSUM) return gmlp::colsum_workspace_bytes(M, N);
  if (K < 1) return 0;
  // Each operation asks for the larger of what its split-reduction form (short batches) and its
  // stream-K form (large tiles whose grid ends in a thinly filled round) would use.
  auto larger = [](size_t a, size_t b) { return a > b ? a : b; };
  auto sk = [&](int64_t rows, int64_t cols, int64_t red_tiles, int bn, bool both_ks = false) -> size_t {
    if (pick_tile(dtype, rows, cols, red_tiles * 64, bn, both_ks) != gmlp::TILE_LARGE) return 0;
    return plan_streamk(dtype, cdiv(rows, 256) * cdiv(cols, bn), red_tiles).ws_bytes;
  };
  // gmlp_gateup_fwd(M, K, N): two accumulator sets [M,N], reduction K
  if (op == GMLP_OP_GATEUP_FWD)
    return larger(split_workspace_bytes(pick_splits(dtype, M, N, K, (K + 63) / 64, 128), M, N, 2),
                  K % 64 == 0 ? sk(M, N, K / 64, 128) : 0);
  // gmlp_linear_fwd(M, R = K, C = N): out [M,N], reduction K
  if (op == GMLP_OP_LINEAR_FWD)
    return larger(split_workspace_bytes(pick_splits(dtype, M, N, K, (K + 63) / 64), M, N),
                  K % 64 == 0 ? sk(M, N, K / 64, 256) : 0);
  // gmlp_dx_bwd(M, K, N): out [M,K], reduction over two segments of N
  if (op == GMLP_OP_DX_BWD)
    return larger(split_workspace_bytes(pick_splits(dtype, M, K, N, 2 * ((N + 63) / 64)), M, K),
                  N % 64 == 0 ? sk(M, K, 2 * (N / 64), 256) : 0);
  // gmlp_dh_bwd(M, K, N): out [M,N], reduction K
  if (op == GMLP_OP_DH_BWD) return K % 64 == 0 ? sk(M, N, K / 64, 256) : 0;
  // gmlp_dw_bwd(Mred = M, R = K, C = N): out [K,N], reduction over the M token rows
  if (op == GMLP_OP_DW_BWD) return sk(K, N, (M + 63) / 64, 256, true);
  return 0;
}

int gmlp_gateup_fwd(const void* x, const void* w_gate, const void* w_up, const void* b_gate,
                    const void* b_up, void* h, void* g_save, void* u_save, uint8_t* mask_out,
                    int64_t M, int64_t K, int64_t N, int dtype, int act, float dropout_p,
                    uint64_t seed, uint64_t offset, void* workspace, size_t workspace_bytes,
                    void* stream) {
  using namespace gmlp;
  GMLP_REQUIRE_PTR(x); GMLP_REQUIRE_PTR(w_gate); GMLP_REQUIRE_PTR(w_up); GMLP_REQUIRE_PTR(h);
  GMLP_REQUIRE_DTYPE(dtype);
  GMLP_REQUIRE_ACT(act);
  DropoutParams d;
  if (int rc = make_dropout(__func__, dropout_p, seed, offset, &d)) return rc;
  if (int rc = check_dims(__func__, M, K, N)) return rc;
  if (int rc = check_mult8(__func__, "K", K)) return rc;
  if (int rc = check_mult8(__func__, "N", N)) return rc;
  GMLP_REQUIRE_ALIGNED(x); GMLP_REQUIRE_ALIGNED(w_gate); GMLP_REQUIRE_ALIGNED(w_up);
  GMLP_REQUIRE_ALIGNED(b_gate); GMLP_REQUIRE_ALIGNED(b_up); GMLP_REQUIRE_ALIGNED(h);
  GMLP_REQUIRE_ALIGNED(g_save); GMLP_REQUIRE_ALIGNED(u_save); GMLP_REQUIRE_ALIGNED(mask_out);
  GMLP_REQUIRE_ALIGNED(workspace);

  hipStream_t s = (hipStream_t)stream;
  hipError_t e = by_dtype(dtype, [&](auto tag) -> hipError_t {
    typedef decltype(tag) T;
    // The GEMM over output columns [col0, col0 + cols): every per-column pointer moves along, the
    // row pitch of the outputs stays N.
    auto run = [&](int64_t col0, int64_t cols, bool may_split, int force_class, const StreamK* sk = nullptr) -> hipError_t {
      GemmArgs ga = {};
      ga.nxcd = num_xcd();
      if (sk) use_streamk(*sk, ga, workspace, workspace_bytes);
      ga.A[0] = x; ga.A[1] = x;
      ga.B[0] = (const T*)w_gate + col0 * K; ga.B[1] = (const T*)w_up + col0 * K;
      ga.M = (int)M; ga.N = (int)cols; ga.K = (int)K; ga.lda = (int)K; ga.ldb = (int)K;
      ga.nseg = 1; ga.group_m = pick_group(M, cols, 2); ga.rotate = M <= 512;
      auto at = [&](const void* p) { return p ? (const T*)p + col0 : nullptr; };
      typename EpiGateUp<T>::Args ea = {(T*)at(h), (T*)at(g_save), (T*)at(u_save), mask_out ? mask_out + col0 : nullptr,
                                        at(b_gate), at(b_up), (int)N, act, d, (size_t)col0};
      if constexpr (!std::is_same<T, float>::value) {
        const int splits = may_split ? pick_splits(dtype, M, cols, K, (K + 63) / 64, 128) : 1;
        if (splits > 1 && workspace != nullptr && workspace_bytes >= split_workspace_bytes(splits, M, cols, 2)) {
          // per split: the gate partial sums [M,cols], then the up partial sums [M,cols]
          ga.splits = splits;
          typename EpiPartial<T>::Args pa = {(float*)workspace, (size_t)2 * M * cols, (size_t)M * cols, (int)cols};
          if (hipError_t err = launch_gateup_split<T>(ga, pa, s)) return err;
          return launch_splitk_reduce<T, EpiGateUp<T>>((const float*)workspace, splits, (size_t)2 * M * cols,
                                                       (size_t)M * cols, ea, M, cols, s);
        }
      }
      return launch_gateup<T>(force_class >= 0 ? force_class : pick_tile(dtype, M, cols, K, 128), ga, ea, s);
    };
    // A grid of large tiles that ends in a thinly filled round of workgroups runs as two launches:
    // the tile columns that make whole rounds, and the remaining columns as a problem of their own,
    // for which pick_tile usually chooses the small tiles (measured on the gate/up GEMM: 1.375
    // rounds 114 -> 95 us, 5.375 rounds 627 -> 611 us, 3.5 rounds 416 -> 407 us).
    if (dtype != GMLP_F32 && pick_tile(dtype, M, N, K, 128) == TILE_LARGE) {
      const int64_t tiles_m = (M + 255) / 256, tiles_n = (N + 127) / 128, cus = num_cu();
      // a long reduction: the tiles of the last round are shared out by reduction range instead
      const StreamK sk = plan_streamk(dtype, tiles_m * tiles_n, K / 64);
      if (sk.tiles > 0 && workspace != nullptr && workspace_bytes >= sk.ws_bytes) return run(0, N, false, TILE_LARGE, &sk);
      const int64_t rounds = tiles_m * tiles_n / cus, tail = tiles_m * tiles_n % cus;
      const int64_t whole_cols = rounds * cus / tiles_m;  // tile columns of the whole rounds
      if (rounds >= 1 && tail > 0 && 2 * tail <= cus && whole_cols >= 1 && whole_cols < tiles_n) {
        if (hipError_t err = run(0, whole_cols * 128, false, TILE_LARGE)) return err;
        return run(whole_cols * 128, N - whole_cols * 128, false, -1);
      }
    }
    return run(0, N, true, -1);
  });
  return hip_result(__func__, e);
}

int gmlp_linear_fwd(const void* a, const void* w, const void* bias, void* out, int64_t M, int64_t R,
                    int64_t C, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  using namespace gmlp;
  GMLP_REQUIRE_PTR(a); GMLP_REQUIRE_PTR(w); GMLP_REQUIRE_PTR(out);
  GMLP_REQUIRE_DTYPE(dtype);
  if (int rc = check_dims(__func__, M, R, C)) return rc;
  if (int rc = check_mult8(__func__, "R", R)) return rc;
  if (int rc = check_mult8(__func__, "C", C)) return rc;
  GMLP_REQUIRE_ALIGNED(a); GMLP_REQUIRE_ALIGNED(w); GMLP_REQUIRE_ALIGNED(bias);
  GMLP_REQUIRE_ALIGNED(out); GMLP_REQUIRE_ALIGNED(workspace);

  hipStream_t s = (hipStream_t)stream;
  hipError_t e = by_dtype(dtype, [&](auto tag) -> hipError_t {
    typedef decltype(tag) T;
    // The GEMM over output columns [col0, col0 + cols); the row pitch of `out` stays C.
    auto run = [&](int64_t col0, int64_t cols, bool may_split, int force_class, const StreamK* sk = nullptr) -> hipError_t {
      GemmArgs ga = {};
      ga.nxcd = num_xcd();
      if (sk) use_streamk(*sk, ga, workspace, workspace_bytes);
      ga.A[0] = a; ga.A[1] = a;
      ga.B[0] = (const T*)w + col0 * R; ga.B[1] = ga.B[0];
      ga.M = (int)M; ga.N = (int)cols; ga.K = (int)R; ga.lda = (int)R; ga.ldb = (int)R;
      ga.nseg = 1; ga.group_m = pick_group(M, cols); ga.rotate = M <= 512;
      typename EpiStore<T>::Args ea = {(T*)out + col0, bias ? (const T*)bias + col0 : nullptr, (int)C};
      if constexpr (!std::is_same<T, float>::value) {
        const int splits = may_split ? pick_splits(dtype, M, cols, R, (R + 63) / 64) : 1;
        if (splits > 1 && workspace != nullptr && workspace_bytes >= split_workspace_bytes(splits, M, cols)) {
          ga.splits = splits;
          typename EpiPartial<T>::Args pa = {(float*)workspace, (size_t)M * cols, 0, (int)cols};
          if (hipError_t err = launch_linear_split<T>(ga, pa, s)) return err;
          return launch_splitk_reduce<T, EpiStore<T>>((const float*)workspace, splits, (size_t)M * cols, 0, ea, M, cols, s);
        }
      }
      return launch_linear<T>(force_class >= 0 ? force_class : pick_tile(dtype, M, cols, R, 256), ga, ea, s);
    };
    // whole rounds of large tiles, then the remaining tile columns as a problem of their own (see
    // gmlp_gateup_fwd)
    if (dtype != GMLP_F32 && pick_tile(dtype, M, C, R, 256) == TILE_LARGE) {
      const int64_t tiles_m = (M + 255) / 256, tiles_n = (C + 255) / 256, cus = num_cu();
      const StreamK sk = plan_streamk(dtype, tiles_m * tiles_n, R / 64);
      if (sk.tiles > 0 && workspace != nullptr && workspace_bytes >= sk.ws_bytes) return run(0, C, false, TILE_LARGE, &sk);
      const int64_t rounds = tiles_m * tiles_n / cus, tail = tiles_m * tiles_n % cus;
      const int64_t whole_cols = rounds * cus / tiles_m;
      if (rounds >= 1 && tail > 0 && 2 * tail <= cus && whole_cols >= 1 && whole_cols < tiles_n) {
        if (hipError_t err = run(0, whole_cols * 256, false, TILE_LARGE)) return err;
        return run(whole_cols * 256, C - whole_cols * 256, false, -1);
      }
    }
    return run(0, C, true, -1);
  });
  return hip_result(__func__, e);
}

int gmlp_dh_bwd(const void* dy, const void* w_down, const void* g, const void* u, void* dg, void* du,
                int64_t M, int64_t K, int64_t N, int dtype, int act, float dropout_p, uint64_t seed,
                uint64_t offset, void* workspace, size_t workspace_bytes, void* stream) {
  using namespace gmlp;
  GMLP_REQUIRE_PTR(dy); GMLP_REQUIRE_PTR(w_down); GMLP_REQUIRE_PTR(g); GMLP_REQUIRE_PTR(u);
  GMLP_REQUIRE_PTR(dg); GMLP_REQUIRE_PTR(du);
  GMLP_REQUIRE_DTYPE(dtype);
  GMLP_REQUIRE_ACT(act);
  DropoutParams d;
  if (int rc = make_dropout(__func__, dropout_p, seed, offset, &d)) return rc;
  if (int rc = check_dims(__func__, M, K, N)) return rc;
  if (int rc = check_mult8(__func__, "K", K)) return rc;
  if (int rc = check_mult8(__func__, "N", N)) return rc;
  GMLP_REQUIRE_ALIGNED(dy); GMLP_REQUIRE_ALIGNED(w_down); GMLP_REQUIRE_ALIGNED(g);
  GMLP_REQUIRE_ALIGNED(u); GMLP_REQUIRE_ALIGNED(dg); GMLP_REQUIRE_ALIGNED(du);
  GMLP_REQUIRE_ALIGNED(workspace);

  // dH[M,N] = dY[M,K] · W_down[K,N]: reduction over K; B is reduction-strided ([K,N] row-major).
  hipStream_t s = (hipStream_t)stream;
  hipError_t e = by_dtype(dtype, [&](auto tag) -> hipError_t {
    typedef decltype(tag) T;
    // The GEMM over output rows [row0, row0 + rows): every per-row pointer moves along.
    auto run = [&](int64_t row0, int64_t rows, int force_class, const StreamK* sk = nullptr) -> hipError_t {
      GemmArgs ga = {};
      ga.nxcd = num_xcd();
      if (sk) use_streamk(*sk, ga, workspace, workspace_bytes);
      ga.A[0] = (const T*)dy + row0 * K; ga.A[1] = ga.A[0]; ga.B[0] = w_down; ga.B[1] = w_down;
      ga.M = (int)rows; ga.N = (int)N; ga.K = (int)K; ga.lda = (int)K; ga.ldb = (int)N;
      ga.nseg = 1; ga.group_m = pick_group(rows, N);
      const size_t e0 = (size_t)row0 * N;
      typename EpiDh<T>::Args ea = {(const T*)g + e0, (const T*)u + e0, (T*)dg + e0, (T*)du + e0, (int)N, act, d, e0};
      return launch_dh<T>(force_class >= 0 ? force_class : pick_tile(dtype, rows, N, K, 256), ga, ea, s);
    };
    if (dtype != GMLP_F32 && pick_tile(dtype, M, N, K, 256) == TILE_LARGE) {
      const StreamK sk = plan_streamk(dtype, cdiv(M, 256) * cdiv(N, 256), K / 64);
      if (sk.tiles > 0 && workspace != nullptr && workspace_bytes >= sk.ws_bytes) return run(0, M, TILE_LARGE, &sk);
    }
    int64_t whole = whole_round_tile_rows(dtype, M, N, K);
    if (whole > 0) {
      if (hipError_t err = run(0, whole * 256, TILE_LARGE)) return err;
      return run(whole * 256, M - whole * 256, -1);
    }
    return run(0, M, -1);
  });
  return hip_result(__func__, e);
}

int gmlp_gating_bwd(const void* dh, const void* g, const void* u, void* dg, void* du, int64_t M,
                    int64_t N, int dtype, int act, float dropout_p, uint64_t seed, uint64_t offset,
                    void* stream) {
  using namespace gmlp;
  GMLP_REQUIRE_PTR(dh); GMLP_REQUIRE_PTR(g); GMLP_REQUIRE_PTR(u); GMLP_REQUIRE_PTR(dg);
  GMLP_REQUIRE_PTR(du);
  GMLP_REQUIRE_DTYPE(dtype);
  GMLP_REQUIRE_ACT(act);
  DropoutParams d;
  if (int rc = make_dropout(__func__, dropout_p, seed, offset, &d)) return rc;
  if (int rc = check_dims(__func__, M, 8, N)) return rc;
  if (int rc = check_mult8(__func__, "N", N)) return rc;
  GMLP_REQUIRE_ALIGNED(dh); GMLP_REQUIRE_ALIGNED(g); GMLP_REQUIRE_ALIGNED(u);
  GMLP_REQUIRE_ALIGNED(dg); GMLP_REQUIRE_ALIGNED(du);
  hipStream_t s = (hipStream_t)stream;
  hipError_t e = by_dtype(dtype, [&](auto tag) {
    typedef decltype(tag) T;
    return launch_gating_bwd<T>((const T*)dh, (const T*)g, (const T*)u, (T*)dg, (T*)du, M, N, act, d, s);
  });
  return hip_result(__func__, e);
}

int gmlp_dx_bwd(const void* dg, const void* du, const void* w_gate, const void* w_up, void* dx,
                int64_t M, int64_t K, int64_t N, int dtype, void* workspace, size_t workspace_bytes,
                void* stream) {
  using namespace gmlp;
  GMLP_REQUIRE_PTR(dg); GMLP_REQUIRE_PTR(du); GMLP_REQUIRE_PTR(w_gate); GMLP_REQUIRE_PTR(w_up);
  GMLP_REQUIRE_PTR(dx);
  GMLP_REQUIRE_DTYPE(dtype);
  if (int rc = check_dims(__func__, M, K, N)) return rc;
  if (int rc = check_mult8(__func__, "K", K)) return rc;
  if (int rc = check_mult8(__func__, "N", N)) return rc;
  GMLP_REQUIRE_ALIGNED(dg); GMLP_REQUIRE_ALIGNED(du); GMLP_REQUIRE_ALIGNED(w_gate);
  GMLP_REQUIRE_ALIGNED(w_up); GMLP_REQUIRE_ALIGNED(dx); GMLP_REQUIRE_ALIGNED(workspace);

  // dX[M,K] = dG[M,N]·W_gate[N,K] + dU[M,N]·W_up[N,K]: two reduction segments of length N.
  hipStream_t s = (hipStream_t)stream;
  hipError_t e = by_dtype(dtype, [&](auto tag) -> hipError_t {
    typedef decltype(tag) T;
    // The GEMM over output rows [row0, row0 + rows).
    auto run = [&](int64_t row0, int64_t rows, bool may_split, int force_class, const StreamK* sk = nullptr) -> hipError_t {
      GemmArgs ga = {};
      ga.nxcd = num_xcd();
      if (sk) use_streamk(*sk, ga, workspace, workspace_bytes);
      ga.A[0] = (const T*)dg + row0 * N; ga.A[1] = (const T*)du + row0 * N; ga.B[0] = w_gate; ga.B[1] = w_up;
      ga.M = (int)rows; ga.N = (int)K; ga.K = (int)N; ga.lda = (int)N; ga.ldb = (int)K;
      ga.nseg = 2; ga.group_m = pick_group(rows, K);
      // (no rotated reduction order here: a piece has room for one change of direction, and with
      // two reduction segments that is the step from dG·W_gate to dU·W_up)
      typename EpiStore<T>::Args ea = {(T*)dx + row0 * K, nullptr, (int)K};
      if constexpr (!std::is_same<T, float>::value) {
        const int splits = may_split ? pick_splits(dtype, rows, K, N, 2 * ((N + 63) / 64)) : 1;
        if (splits > 1 && workspace != nullptr && workspace_bytes >= split_workspace_bytes(splits, rows, K)) {
          ga.splits = splits;
          typename EpiPartial<T>::Args pa = {(float*)workspace, (size_t)rows * K, 0, (int)K};
          if (hipError_t err = launch_dx_split<T>(ga, pa, s)) return err;
          return launch_splitk_reduce<T, EpiStore<T>>((const float*)workspace, splits, (size_t)rows * K, 0, ea, rows, K, s);
        }
      }
      return launch_dx<T>(force_class >= 0 ? force_class : pick_tile(dtype, rows, K, N, 256), ga, ea, s);
    };
    if (dtype != GMLP_F32 && pick_tile(dtype, M, K, N, 256) == TILE_LARGE) {
      const StreamK sk = plan_streamk(dtype, cdiv(M, 256) * cdiv(K, 256), 2 * (N / 64));
      if (sk.tiles > 0 && workspace != nullptr && workspace_bytes >= sk.ws_bytes) return run(0, M, false, TILE_LARGE, &sk);
    }
    int64_t whole = whole_round_tile_rows(dtype, M, K, N);
    if (whole > 0) {
      if (hipError_t err = run(0, whole * 256, false, TILE_LARGE)) return err;
      return run(whole * 256, M - whole * 256, false, -1);
    }
    return run(0, M, true, -1);
  });
  return hip_result(__func__, e);
}

int gmlp_dw_bwd(const void* lhs, const void* rhs, void* dw, int64_t Mred, int64_t R, int64_t C,
                int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  using namespace gmlp;
  GMLP_REQUIRE_PTR(lhs); GMLP_REQUIRE_PTR(rhs); GMLP_REQUIRE_PTR(dw);
  GMLP_REQUIRE_DTYPE(dtype);
  if (int rc = check_dims(__func__, Mred, R, C)) return rc;
  if (int rc = check_mult8(__func__, "R", R)) return rc;
  if (int rc = check_mult8(__func__, "C", C)) return rc;
  GMLP_REQUIRE_ALIGNED(lhs); GMLP_REQUIRE_ALIGNED(rhs); GMLP_REQUIRE_ALIGNED(dw);
  GMLP_REQUIRE_ALIGNED(workspace);

  // dW[R,C] = lhs[Mred,R]ᵀ · rhs[Mred,C]: both operands reduction-strided.
  GemmArgs ga = {};
      ga.nxcd = num_xcd();
  ga.A[0] = lhs; ga.A[1] = lhs; ga.B[0] = rhs; ga.B[1] = rhs;
  ga.M = (int)R; ga.N = (int)C; ga.K = (int)Mred; ga.lda = (int)R; ga.ldb = (int)C;
  ga.nseg = 1; ga.group_m = pick_group(R, C);
  int tc = pick_tile(dtype, R, C, Mred, 256, true);
  if (tc == TILE_LARGE) use_streamk(plan_streamk(dtype, cdiv(R, 256) * cdiv(C, 256), cdiv(Mred, 64)), ga, workspace, workspace_bytes);
  hipStream_t s = (hipStream_t)stream;
  hipError_t e = by_dtype(dtype, [&](auto tag) {
    typedef decltype(tag) T;
    typename EpiStore<T>::Args ea = {(T*)dw, nullptr, (int)C};
    return launch_dw<T>(tc, ga, ea, s);
  });
  return hip_result(__func__, e);
}

size_t gmlp_dw_bwd_grouped_workspace_bytes(int count, int64_t Mred, const int64_t* R, const int64_t* C, int dtype) {
  using namespace gmlp;
  if (count < 1 || count > GEMM_GROUP_MAX || R == nullptr || C == nullptr || Mred < 1 || dtype == GMLP_F32) return 0;
  int64_t tiles256 = 0, tiles128 = 0;
  for (int i = 0; i < count; ++i) {
    if (R[i] < 1 || C[i] < 1 || pick_tile(dtype, R[i], C[i], Mred, 256, true) == TILE_MEDIUM) return 0;
    tiles256 += cdiv(R[i], 256) * cdiv(C[i], 256);
    tiles128 += cdiv(R[i], 128) * cdiv(C[i], 128);
  }
  if (group_tile_class(tiles256, tiles128) != TILE_LARGE) return 0;
  const StreamK sk = plan_streamk(dtype, tiles256, cdiv(Mred, 64));
  return sk.tiles > cdiv(R[count - 1], 256) * cdiv(C[count - 1], 256) ? 0 : sk.ws_bytes;
}

int gmlp_dw_bwd_grouped(int count, const void* const* lhs, const void* const* rhs, void* const* dw,
                        int64_t Mred, const int64_t* R, const int64_t* C, int dtype, void* workspace,
                        size_t workspace_bytes, void* stream) {
  using namespace gmlp;
  if (count < 1 || count > GEMM_GROUP_MAX)
    return fail(GMLP_EINVAL, "%s: count = %d must be in 1..%d", __func__, count, GEMM_GROUP_MAX);
  GMLP_REQUIRE_PTR(lhs); GMLP_REQUIRE_PTR(rhs); GMLP_REQUIRE_PTR(dw); GMLP_REQUIRE_PTR(R);
  GMLP_REQUIRE_PTR(C);
  GMLP_REQUIRE_DTYPE(dtype);
  // One grid when every problem runs on a pipelined tile class; the class is chosen for the
  // problems together (their tiles share the rounds of workgroups).
  bool pipelined = true;
  for (int i = 0; i < count; ++i) {
    GMLP_REQUIRE_PTR(lhs[i]); GMLP_REQUIRE_PTR(rhs[i]); GMLP_REQUIRE_PTR(dw[i]);
    if (int rc = check_dims(__func__, Mred, R[i], C[i])) return rc;
    if (int rc = check_mult8(__func__, "R", R[i])) return rc;
    if (int rc = check_mult8(__func__, "C", C[i])) return rc;
    GMLP_REQUIRE_ALIGNED(lhs[i]); GMLP_REQUIRE_ALIGNED(rhs[i]); GMLP_REQUIRE_ALIGNED(dw[i]);
    pipelined = pipelined && pick_tile(dtype, R[i], C[i], Mred, 256, true) != TILE_MEDIUM;
  }
  if (!pipelined) {
    for (int i = 0; i < count; ++i)
      if (int rc = gmlp_dw_bwd(lhs[i], rhs[i], dw[i], Mred, R[i], C[i], dtype, workspace, workspace_bytes, stream)) return rc;
    return GMLP_OK;
  }
  int64_t tiles256 = 0, tiles128 = 0;
  for (int i = 0; i < count; ++i) {
    tiles256 += ((R[i] + 255) / 256) * ((C[i] + 255) / 256);
    tiles128 += ((R[i] + 127) / 128) * ((C[i] + 127) / 128);
  }
  const int group_class = group_tile_class(tiles256, tiles128);
  hipStream_t s = (hipStream_t)stream;
  auto fill = [&](GemmArgs& ga, int i) {
    ga = GemmArgs{};
    ga.nxcd = num_xcd();
    ga.A[0] = lhs[i]; ga.A[1] = lhs[i]; ga.B[0] = rhs[i]; ga.B[1] = rhs[i];
    ga.M = (int)R[i]; ga.N = (int)C[i]; ga.K = (int)Mred; ga.lda = (int)R[i]; ga.ldb = (int)C[i];
    ga.nseg = 1; ga.group_m = pick_group(R[i], C[i]);
  };
  // A grid of large tiles that ends in a thinly filled round: the last problem gives up a band of
  // its output (whole tile rows or tile columns, whichever comes closer to the tiles of that last
  // round), which runs as a launch of its own on the tile class that suits it; the rest then makes
  // whole rounds.  Both operands are reduction-strided, so the band is a range of columns of one
  // of them: the pointer moves along the rows and the buffer size is trimmed to match.
  int64_t band_rows = 0, band_cols = 0;  // size of the band, in output rows or columns (one is 0)
  const int last = count - 1;
  // With a long reduction the last round's tiles (the last ones of the last problem) are shared out
  // by reduction range instead (stream-K), if the last problem has that many tiles.
  StreamK sk;
  if (group_class == TILE_LARGE) {
    sk = plan_streamk(dtype, tiles256, cdiv(Mred, 64));
    if (sk.tiles > cdiv(R[last], 256) * cdiv(C[last], 256) || workspace == nullptr || workspace_bytes < sk.ws_bytes) sk = StreamK{};
  }
  if (group_class == TILE_LARGE && sk.tiles == 0) {
    const int64_t cus = num_cu(), rounds = tiles256 / cus, tail = tiles256 % cus;
    const int64_t tr = (R[last] + 255) / 256, tc = (C[last] + 255) / 256;
    // (worth it for a few rounds only: measured -7 % at 2 rounds, -1 % and less from 8 rounds on)
    if (rounds >= 1 && rounds <= 4 && tail > 0 && 2 * tail <= cus) {
      const int64_t by_rows = (tail + tc - 1) / tc, by_cols = (tail + tr - 1) / tr;  // tile rows / columns
      const bool rows_fit = by_rows < tr, cols_fit = by_cols < tc;
      if (cols_fit && (!rows_fit || by_cols * tr <= by_rows * tc)) band_cols = C[last] - (tc - by_cols) * 256;
      else if (rows_fit) band_rows = R[last] - (tr - by_rows) * 256;
      const int64_t br = band_rows ? band_rows : R[last], bc = band_cols ? band_cols : C[last];
      if ((band_rows || band_cols) && pick_tile(dtype, br, bc, Mred, 256, true) == TILE_MEDIUM) band_rows = band_cols = 0;
    }
  }
  hipError_t e = by_dtype(dtype, [&](auto tag) -> hipError_t {
    typedef decltype(tag) T;
    if constexpr (std::is_same<T, float>::value) {
      return hipErrorInvalidValue;  // not reached: float32 problems take the separate launches above
    } else {
      GemmGroup<typename EpiStore<T>::Args> grp = {};
      grp.count = count;
      for (int i = 0; i < count; ++i) {
        fill(grp.ga[i], i);
        grp.ea[i] = typename EpiStore<T>::Args{(T*)dw[i], nullptr, (int)C[i]};
      }
      grp.ga[last].M -= (int)band_rows;
      grp.ga[last].N -= (int)band_cols;
      use_streamk(sk, grp.ga[last], workspace, workspace_bytes);
      if (hipError_t err = launch_dw_group<T>(group_class, grp, s)) return err;
      if (band_rows == 0 && band_cols == 0) return hipSuccess;
      GemmArgs ga;
      fill(ga, last);
      const int64_t r0 = band_rows ? R[last] - band_rows : 0, c0 = band_cols ? C[last] - band_cols : 0;
      ga.A[0] = ga.A[1] = (const T*)lhs[last] + r0;
      ga.B[0] = ga.B[1] = (const T*)rhs[last] + c0;
      ga.a_trim = (int)(r0 * sizeof(T));
      ga.b_trim = (int)(c0 * sizeof(T));
      ga.M = (int)(R[last] - r0);
      ga.N = (int)(C[last] - c0);
      ga.group_m = pick_group(ga.M, ga.N);
      typename EpiStore<T>::Args ea = {(T*)dw[last] + r0 * C[last] + c0, nullptr, (int)C[last]};
      return launch_dw<T>(pick_tile(dtype, ga.M, ga.N, Mred, 256, true), ga, ea, s);
    }
  });
  return hip_result(__func__, e);
}

int gmlp_colsum(const void* a, void* out, void* workspace, int64_t M, int64_t C, int dtype,
                void* stream) {
  const void* as[1] = {a};
  void* outs[1] = {out};
  return gmlp_colsum_grouped(1, as, outs, workspace, M, &C, dtype, stream);
}

int gmlp_colsum_static(const void* a, void* out, int64_t M, int64_t C, int dtype, void* stream) {
  using namespace gmlp;
  GMLP_REQUIRE_PTR(a); GMLP_REQUIRE_PTR(out);
  GMLP_REQUIRE_DTYPE(dtype);
  if (int rc = check_dims(__func__, M, 8, C)) return rc;
  if (int rc = check_mult8(__func__, "C", C)) return rc;
  if (C > COLSUM_STATIC_MAX_C)
    return fail(GMLP_ESHAPE, "%s: C = %lld exceeds the %lld columns the library's static scratch array holds "
                "(use gmlp_colsum with a workspace)", __func__, (long long)C, (long long)COLSUM_STATIC_MAX_C);
  GMLP_REQUIRE_ALIGNED(a); GMLP_REQUIRE_ALIGNED(out);
  hipStream_t s = (hipStream_t)stream;
  hipError_t e = by_dtype(dtype, [&](auto tag) {
    typedef decltype(tag) T;
    return launch_colsum_static<T>((const T*)a, (T*)out, M, C, s);
  });
  return hip_result(__func__, e);
}

int gmlp_colsum_grouped(int count, const void* const* a, void* const* out, void* workspace, int64_t M,
                        const int64_t* C, int dtype, void* stream) {
  using namespace gmlp;
  if (count < 1 || count > COLSUM_GROUP_MAX)
    return fail(GMLP_EINVAL, "%s: count = %d must be in 1..%d", __func__, count, COLSUM_GROUP_MAX);
  GMLP_REQUIRE_PTR(a); GMLP_REQUIRE_PTR(out); GMLP_REQUIRE_PTR(C); GMLP_REQUIRE_PTR(workspace);
  GMLP_REQUIRE_DTYPE(dtype);
  GMLP_REQUIRE_ALIGNED(workspace);
  for (int i = 0; i < count; ++i) {
    GMLP_REQUIRE_PTR(a[i]); GMLP_REQUIRE_PTR(out[i]);
    if (int rc = check_dims(__func__, M, 8, C[i])) return rc;
    if (int rc = check_mult8(__func__, "C", C[i])) return rc;
    GMLP_REQUIRE_ALIGNED(a[i]); GMLP_REQUIRE_ALIGNED(out[i]);
  }
  hipStream_t s = (hipStream_t)stream;
  hipError_t e = by_dtype(dtype, [&](auto tag) {
    typedef decltype(tag) T;
    ColsumGroup<T> g = {};
    char* ws = (char*)workspace;
    for (int i = 0; i < count; ++i) {
      g.a[i] = (const T*)a[i];
      g.out[i] = (T*)out[i];
      g.ws[i] = (float*)ws;
      g.C[i] = C[i];
      ws += colsum_workspace_bytes(M, C[i]);
    }
    return launch_colsum_group<T>(g, count, M, s);
  });
  return hip_result(__func__, e);
}

int gmlp_decode_fwd(const void* x, const void* w_gate, const void* w_up, const void* w_down,
                    const void* b_gate, const void* b_up, const void* b_down, void* h_scratch,
                    void* y, void* workspace, int64_t M, int64_t K, int64_t N, int dtype, int act,
                    void* stream) {
  using namespace gmlp;
  (void)workspace;
  GMLP_REQUIRE_PTR(x); GMLP_REQUIRE_PTR(w_gate); GMLP_REQUIRE_PTR(w_up); GMLP_REQUIRE_PTR(w_down);
  GMLP_REQUIRE_PTR(h_scratch); GMLP_REQUIRE_PTR(y);
  GMLP_REQUIRE_DTYPE(dtype);
  GMLP_REQUIRE_ACT(act);
  if (int rc = check_dims(__func__, M, K, N)) return rc;
  if (dtype == GMLP_F32) return fail(GMLP_ESHAPE, "%s: float32 is not supported by the skinny-M kernels", __func__);
  if (M > 32 || (M > 16 && !decode_stream_supported((int)M, (int)K, (int)N)))
    return fail(GMLP_ESHAPE,
                "%s: M = %lld exceeds the skinny-M limit (32 when K and N are multiples of 256, at least 768, "
                "and K*N < 2^30; 16 otherwise)",
                __func__, (long long)M);
  if (K % 32 != 0) return fail(GMLP_ESHAPE, "%s: K = %lld must be a multiple of 32", __func__, (long long)K);
  if (N % 256 != 0) return fail(GMLP_ESHAPE, "%s: N = %lld must be a multiple of 256", __func__, (long long)N);
  GMLP_REQUIRE_ALIGNED(x); GMLP_REQUIRE_ALIGNED(w_gate); GMLP_REQUIRE_ALIGNED(w_up);
  GMLP_REQUIRE_ALIGNED(w_down); GMLP_REQUIRE_ALIGNED(b_gate); GMLP_REQUIRE_ALIGNED(b_up);
  GMLP_REQUIRE_ALIGNED(b_down); GMLP_REQUIRE_ALIGNED(h_scratch); GMLP_REQUIRE_ALIGNED(y);
  hipStream_t s = (hipStream_t)stream;
  hipError_t e =
      dtype == GMLP_F16
          ? launch_decode<f16>((const f16*)x, (const f16*)w_gate, (const f16*)w_up, (const f16*)w_down,
                               (const f16*)b_gate, (const f16*)b_up, (const f16*)b_down,
                               (f16*)h_scratch, (f16*)y, (int)M, (int)K, (int)N, act, s)
          : launch_decode<bf16>((const bf16*)x, (const bf16*)w_gate, (const bf16*)w_up,
                                (const bf16*)w_down, (const bf16*)b_gate, (const bf16*)b_up,
                                (const bf16*)b_down, (bf16*)h_scratch, (bf16*)y, (int)M, (int)K,
                                (int)N, act, s);
  return hip_result(__func__, e);
}

int gmlp_dropout_mask(uint8_t* mask, int64_t M, int64_t N, float dropout_p, uint64_t seed,
                      uint64_t offset, void* stream) {
  using namespace gmlp;
  GMLP_REQUIRE_PTR(mask);
  DropoutParams d;
  if (int rc = make_dropout(__func__, dropout_p, seed, offset, &d)) return rc;
  if (int rc = check_dims(__func__, M, 8, N)) return rc;
  if (int rc = check_mult8(__func__, "N", N)) return rc;
  GMLP_REQUIRE_ALIGNED(mask);
  return hip_result(__func__, launch_dropout_mask(mask, M, N, d, (hipStream_t)stream));
}


}  // extern "C"

// ---------------------------------------------------------------- whole passes in one call
namespace {

// Workspace of a backward pass: what its launches ask for, one after the other on one stream, so
// one buffer of the largest request serves them all.
struct BwdWorkspace {
  size_t act = 0;     // gmlp_dh_bwd, then gmlp_dx_bwd
  size_t dw = 0;      // gmlp_dw_bwd_grouped
  size_t colsum = 0;  // gmlp_colsum_grouped
  size_t total() const { return std::max(act, std::max(dw, colsum)); }
};
BwdWorkspace plan_bwd_workspace(int64_t M, int64_t K, int64_t N, int dtype, bool gate, bool up, bool down,
                                bool bias_gate, bool bias_up, bool bias_down) {
  BwdWorkspace w;
  const size_t dh = gmlp_workspace_bytes(GMLP_OP_DH_BWD, M, K, N, dtype);
  const size_t dx = gmlp_workspace_bytes(GMLP_OP_DX_BWD, M, K, N, dtype);
  w.act = dh > dx ? dh : dx;
  int64_t R[3], C[3];
  int n = 0;
  if (gate) { R[n] = N; C[n] = K; ++n; }
  if (up) { R[n] = N; C[n] = K; ++n; }
  if (down) { R[n] = K; C[n] = N; ++n; }
  if (n > 0) w.dw = gmlp_dw_bwd_grouped_workspace_bytes(n, M, R, C, dtype);
  // without stream-K a problem that takes the single-launch path may still ask for its own
  if (n > 0 && w.dw == 0) {
    for (int i = 0; i < n; ++i) {
      const size_t one = gmlp_workspace_bytes(GMLP_OP_DW_BWD, M, R[i], C[i], dtype);
      if (one > w.dw) w.dw = one;
    }
  }
  if (bias_gate) w.colsum += gmlp::colsum_workspace_bytes(M, N);
  if (bias_up) w.colsum += gmlp::colsum_workspace_bytes(M, N);
  if (bias_down) w.colsum += gmlp::colsum_workspace_bytes(M, K);
  return w;
}

}  // namespace

extern "C" {

size_t gmlp_mlp_workspace_bytes(int pass, int64_t M, int64_t K, int64_t N, int dtype) {
  if (M < 1 || K < 1 || N < 1) return 0;
  if (pass == GMLP_PASS_FWD) {
    const size_t a = gmlp_workspace_bytes(GMLP_OP_GATEUP_FWD, M, K, N, dtype);
    const size_t b = gmlp_workspace_bytes(GMLP_OP_LINEAR_FWD, M, N, K, dtype);
    return a > b ? a : b;
  }
  if (pass == GMLP_PASS_BWD) return plan_bwd_workspace(M, K, N, dtype, true, true, true, true, true, true).total();
  return 0;
}

int gmlp_mlp_fwd(const void* x, const void* w_gate, const void* w_up, const void* w_down, const void* b_gate,
                 const void* b_up, const void* b_down, void* y, void* h, void* g_save, void* u_save, int64_t M,
                 int64_t K, int64_t N, int dtype, int act, float dropout_p, uint64_t seed, uint64_t offset,
                 void* workspace, size_t workspace_bytes, void* stream) {
  GMLP_REQUIRE_PTR(x); GMLP_REQUIRE_PTR(w_gate); GMLP_REQUIRE_PTR(w_up); GMLP_REQUIRE_PTR(w_down);
  GMLP_REQUIRE_PTR(y); GMLP_REQUIRE_PTR(h);
  GMLP_REQUIRE_DTYPE(dtype);
  GMLP_REQUIRE_ACT(act);
  gmlp::DropoutParams d;
  if (int rc = make_dropout(__func__, dropout_p, seed, offset, &d)) return rc;
  if (int rc = check_dims(__func__, M, K, N)) return rc;
  if (int rc = check_mult8(__func__, "K", K)) return rc;
  if (int rc = check_mult8(__func__, "N", N)) return rc;
  GMLP_REQUIRE_ALIGNED(x); GMLP_REQUIRE_ALIGNED(w_gate); GMLP_REQUIRE_ALIGNED(w_up); GMLP_REQUIRE_ALIGNED(w_down);
  GMLP_REQUIRE_ALIGNED(b_gate); GMLP_REQUIRE_ALIGNED(b_up); GMLP_REQUIRE_ALIGNED(b_down); GMLP_REQUIRE_ALIGNED(y);
  GMLP_REQUIRE_ALIGNED(h); GMLP_REQUIRE_ALIGNED(g_save); GMLP_REQUIRE_ALIGNED(u_save); GMLP_REQUIRE_ALIGNED(workspace);
  // both launches are on `stream`, one after the other: they share the workspace
  if (int rc = gmlp_gateup_fwd(x, w_gate, w_up, b_gate, b_up, h, g_save, u_save, nullptr, M, K, N, dtype, act, dropout_p,
                               seed, offset, workspace, workspace_bytes, stream))
    return rc;
  return gmlp_linear_fwd(h, w_down, b_down, y, M, N, K, dtype, workspace, workspace_bytes, stream);
}

int gmlp_mlp_bwd(const void* dy, const void* x, const void* w_gate, const void* w_up, const void* w_down,
                 const void* g, const void* u, const void* h, void* dg, void* du, void* dx, void* dw_gate,
                 void* dw_up, void* dw_down, void* db_gate, void* db_up, void* db_down, int64_t M, int64_t K,
                 int64_t N, int dtype, int act, float dropout_p, uint64_t seed, uint64_t offset, void* workspace,
                 size_t workspace_bytes, void* stream) {
  GMLP_REQUIRE_PTR(dy);
  GMLP_REQUIRE_DTYPE(dtype);
  GMLP_REQUIRE_ACT(act);
  gmlp::DropoutParams d;
  if (int rc = make_dropout(__func__, dropout_p, seed, offset, &d)) return rc;
  if (int rc = check_dims(__func__, M, K, N)) return rc;
  if (int rc = check_mult8(__func__, "K", K)) return rc;
  if (int rc = check_mult8(__func__, "N", N)) return rc;
  // what each requested output needs
  const bool hidden = dx || dw_gate || dw_up || db_gate || db_up;  // anything behind dG, dU
  if (hidden) {
    GMLP_REQUIRE_PTR(w_down); GMLP_REQUIRE_PTR(g); GMLP_REQUIRE_PTR(u); GMLP_REQUIRE_PTR(dg); GMLP_REQUIRE_PTR(du);
  }
  if (dx) { GMLP_REQUIRE_PTR(w_gate); GMLP_REQUIRE_PTR(w_up); }
  if (dw_gate || dw_up) GMLP_REQUIRE_PTR(x);
  if (dw_down) GMLP_REQUIRE_PTR(h);
  GMLP_REQUIRE_ALIGNED(dy); GMLP_REQUIRE_ALIGNED(x); GMLP_REQUIRE_ALIGNED(w_gate); GMLP_REQUIRE_ALIGNED(w_up);
  GMLP_REQUIRE_ALIGNED(w_down); GMLP_REQUIRE_ALIGNED(g); GMLP_REQUIRE_ALIGNED(u); GMLP_REQUIRE_ALIGNED(h);
  GMLP_REQUIRE_ALIGNED(dg); GMLP_REQUIRE_ALIGNED(du); GMLP_REQUIRE_ALIGNED(dx); GMLP_REQUIRE_ALIGNED(dw_gate);
  GMLP_REQUIRE_ALIGNED(dw_up); GMLP_REQUIRE_ALIGNED(dw_down); GMLP_REQUIRE_ALIGNED(db_gate); GMLP_REQUIRE_ALIGNED(db_up);
  GMLP_REQUIRE_ALIGNED(db_down); GMLP_REQUIRE_ALIGNED(workspace);

  const BwdWorkspace need = plan_bwd_workspace(M, K, N, dtype, dw_gate, dw_up, dw_down, db_gate, db_up, db_down);
  // Every launch gets the caller's buffer when it is large enough for that launch, and none
  // otherwise (same results from the plain form of the launch).  Bias gradients cannot do without.
  auto fits = [&](size_t bytes) { return workspace != nullptr && bytes > 0 && bytes <= workspace_bytes; };
  void* const ws_cs = fits(need.colsum) ? workspace : nullptr;
  void* const ws_dw = fits(need.dw) ? workspace : nullptr;
  void* const ws_act = fits(need.act) ? workspace : nullptr;
  const size_t n_dw = ws_dw ? workspace_bytes : 0, n_act = ws_act ? workspace_bytes : 0;
  if (need.colsum > 0 && ws_cs == nullptr)
    return fail(GMLP_EINVAL, "%s: bias gradients need a workspace of at least %zu bytes (gmlp_mlp_workspace_bytes)",
                __func__, need.colsum);

  const void* lhs[3]; const void* rhs[3]; void* dws[3]; int64_t R[3], C[3];
  int n = 0;
  if (dw_gate) { lhs[n] = dg; rhs[n] = x; dws[n] = dw_gate; R[n] = N; C[n] = K; ++n; }
  if (dw_up) { lhs[n] = du; rhs[n] = x; dws[n] = dw_up; R[n] = N; C[n] = K; ++n; }
  if (dw_down) { lhs[n] = dy; rhs[n] = h; dws[n] = dw_down; R[n] = K; C[n] = N; ++n; }
  const void* cs_in[3]; void* cs_out[3]; int64_t cs_c[3];
  int nb = 0;
  if (db_gate) { cs_in[nb] = dg; cs_out[nb] = db_gate; cs_c[nb] = N; ++nb; }
  if (db_up) { cs_in[nb] = du; cs_out[nb] = db_up; cs_c[nb] = N; ++nb; }
  if (db_down) { cs_in[nb] = dy; cs_out[nb] = db_down; cs_c[nb] = K; ++nb; }

  if (hidden)
    if (int rc = gmlp_dh_bwd(dy, w_down, g, u, dg, du, M, K, N, dtype, act, dropout_p, seed, offset, ws_act, n_act, stream))
      return rc;
  // Everything on the caller's stream, one launch after the other.  Running the weight gradients
  // on a second stream next to dX was measured and is not done: two grids that each fill the chip
  // run 2.5 to 4 % slower side by side than one after the other (M=8192, K=4096, N=14336), and where
  // grids under-fill the chip (M=2048, K=2048, N=5632) the two event waits that fork and join the
  // streams cost what the overlap gains.
  int rc = GMLP_OK;
  if (dx) rc = gmlp_dx_bwd(dg, du, w_gate, w_up, dx, M, K, N, dtype, ws_act, n_act, stream);
  if (rc == GMLP_OK && n > 0) rc = gmlp_dw_bwd_grouped(n, lhs, rhs, dws, M, R, C, dtype, ws_dw, n_dw, stream);
  if (rc == GMLP_OK && nb > 0) rc = gmlp_colsum_grouped(nb, cs_in, cs_out, ws_cs, M, cs_c, dtype, stream);
  return rc;
}

}  // extern "C"
