// LDS-tiled MFMA GEMM for gfx950 with pluggable operand orientation and fused epilogues.
//
//   C[M,N] (+)= sum over segments s, reduction k of  A_s[m,k] * B_s[n,k]
//
// Each operand is either reduction-contiguous ("KC": memory is [rows, K], K fastest) or
// reduction-strided ("KS": memory is [K, rows], rows fastest).  The six GEMMs of the gated MLP
// (gate/up, down, dH, dX, dW_gate/up, dW_down) are the combinations (KC,KC), (KC,KS), (KS,KS).
// NB = 2 keeps two B operands and two accumulator sets per output element (gate and up share the
// x tile), so the SiLU-gating epilogue sees both values in the same lane.
//
// Work decomposition: one workgroup (WGM x WGN wavefronts of 64 lanes) per BM x BN output tile,
// each wavefront owning a (BM/WGM) x (BN/WGN) sub-tile as a grid of 32x32 MFMA accumulators.
// Global memory -> registers -> LDS with two LDS stages; LDS rows of KC tiles are XOR-swizzled in
// 16-byte chunks so that both the 16-byte stores and the ds_read_b128 fragment loads are free of
// bank conflicts.  The MFMA is issued with operands swapped (B fragment as the instruction's A
// operand), so a lane ends up with 4 consecutive output columns of one row: 8-byte stores.
#pragma once
#include "common.hpp"

namespace gmlp {

struct GemmArgs {
  const void* A[2];  // per reduction segment
  const void* B[2];  // per reduction segment (NB == 1) or per accumulator set (NB == 2)
  int M, N, K;       // output rows, output cols, reduction length of one segment
  int lda, ldb;      // leading dimensions (elements)
  int nseg;          // number of reduction segments (1 or 2)
  int group_m;       // tile-rows per scheduling group; negative: -group_m tile-COLUMNS per group
  int splits;        // pipelined kernel with a split-reduction epilogue only: number of workgroups
                     // that share one output tile, each reducing a contiguous range of 64-wide
                     // reduction tiles into a partial result of its own (0 or 1: no split)
  int a_trim, b_trim;  // pipelined kernel: bytes to take off the size of a reduction-strided operand
                     // whose pointer has been moved along its rows to address a range of output
                     // rows / columns (the operand then ends that many bytes earlier than its row
                     // count times its pitch says)
  int rotate;        // pipelined kernel: the workgroups of tile column c start their reduction
                     // range at tile c mod length and wrap around.  For short batches, which are
                     // bound by streaming the B operand (the weights): the workgroups would
                     // otherwise all read the same offset along their rows at the same time, which
                     // for the usual power-of-two row pitches crowds onto a few memory channels.
                     // Workgroups that share B rows keep the same order, so they still share them
                     // in L2.
  // Stream-K (pipelined kernel, non-split epilogues): the last sk_tiles output tiles (in workgroup
  // order) are not computed one per workgroup; their reduction tiles are shared out evenly over
  // sk_wgs extra workgroups at the end of the grid, which leave partial sums in sk_ws
  // ((sk_wgs + sk_tiles) slots of one output tile's accumulators, fp32), added up in a fixed order
  // by a second launch.  sk_tiles == 0: every tile has a workgroup of its own.
  int sk_tiles, sk_wgs;
  int sk_chunks;     // > 0: sk_wgs == sk_chunks * sk_tiles and every tile is cut into sk_chunks equal
                     // reduction ranges, one workgroup each (slot = workgroup); 0: even ranges over the
                     // (tile, reduction tile) sequence, which may straddle tiles
  float* sk_ws;
  int nxcd;          // accelerator dies of the device (each with its own L2) the hardware deals
                     // workgroup ids to, round-robin (0 is read as 1: no remapping)
};

// Workgroup id -> output tile.  The hardware deals consecutive workgroup ids round-robin to the
// device's XCDs (each with its own L2; 8 on a whole MI355X); xcd_contiguous undoes that so each XCD
// walks a contiguous run of indices, and tile_of walks tiles in groups of `group_m` tile-rows
// (column-major inside a group) for operand reuse in L2.
__device__ __forceinline__ int xcd_contiguous(int pid, int nwg, int nxcd) {
  if (nxcd <= 1) return pid;
  int xcd = pid % nxcd, loc = pid / nxcd;
  int per = nwg / nxcd, rem = nwg % nxcd;
  return xcd * per + (xcd < rem ? xcd : rem) + loc;
}
__device__ __forceinline__ void tile_of(int t, int tiles_m, int tiles_n, int group_m, int& tm, int& tn) {
  int in_group = group_m * tiles_n;
  int gid = t / in_group;
  int first_m = gid * group_m;
  int gsz = tiles_m - first_m < group_m ? tiles_m - first_m : group_m;
  int r = t - gid * in_group;
  tm = first_m + r % gsz;
  tn = r / gsz;
}
// group > 0: groups of `group` tile-rows, walked column by column: an XCD's successive rounds of
// workgroups keep their A panels and move on to new B panels.  group < 0: the same with rows and
// columns exchanged (B panels kept).  The kept operand should be the smaller one: it is the one
// the memory-side cache can still hold when the next round asks for it again.
__device__ __forceinline__ void tile_of_grouped(int t, int tiles_m, int tiles_n, int group, int& tm, int& tn) {
  const bool by_columns = group < 0;
  int major, minor;
  tile_of(t, by_columns ? tiles_n : tiles_m, by_columns ? tiles_m : tiles_n, by_columns ? -group : group,
          major, minor);
  tm = by_columns ? minor : major;
  tn = by_columns ? major : minor;
}
__device__ __forceinline__ void map_tile(int pid, int nwg, int nxcd, int tiles_m, int tiles_n, int group_m,
                                         int& tm, int& tn) {
  tile_of_grouped(xcd_contiguous(pid, nwg, nxcd), tiles_m, tiles_n, group_m, tm, tn);
}

template <int BK>
__device__ __forceinline__ int swizzle_chunk(int row, int c) {
  // 16 consecutive rows x one 16-byte chunk must hit 64 distinct banks.
  if (BK == 64) return c ^ ((row >> 1) & 7);
  return c ^ ((row >> 2) & 3);
}

// One operand tile: ROWS output-dimension rows by BK reduction elements.
template <typename T, int ROWS, int BK, bool KS, int NT, bool EDGE>
struct OperandTile {
  typedef typename Traits<T>::vec8 vec8;
  static constexpr int CHUNKS = ROWS * BK / 8;
  static constexpr int PER_THREAD = CHUNKS / NT;
  static_assert(CHUNKS % NT == 0, "tile chunks must divide evenly over the workgroup");
  static constexpr int KS_LD = ROWS + 8;  // padded row length of a KS tile in LDS (elements)
  static constexpr int LDS_ELEMS = KS ? BK * KS_LD : ROWS * BK;

  uint4 regs[PER_THREAD];

  // global -> registers.  r0: first output-dim row of the tile, k0: first reduction index.
  __device__ __forceinline__ void gload(const T* __restrict__ p, int ld, int r0, int k0, int rtot,
                                        int ktot, int tid) {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      int q = tid + i * NT;
      if (!KS) {
        int row = q / (BK / 8), c = q % (BK / 8);
        int gr = r0 + row, gk = k0 + c * 8;
        bool ok = !EDGE || (gr < rtot && gk < ktot);
        regs[i] = ok ? *(const uint4*)(p + (size_t)gr * ld + gk) : make_uint4(0, 0, 0, 0);
      } else {
        int krow = q / (ROWS / 8), c = q % (ROWS / 8);
        int gk = k0 + krow, gr = r0 + c * 8;
        bool ok = !EDGE || (gk < ktot && gr < rtot);
        regs[i] = ok ? *(const uint4*)(p + (size_t)gk * ld + gr) : make_uint4(0, 0, 0, 0);
      }
    }
  }

  // registers -> LDS
  __device__ __forceinline__ void sstore(T* lds, int tid) const {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      int q = tid + i * NT;
      if (!KS) {
        int row = q / (BK / 8), c = q % (BK / 8);
        *(uint4*)(lds + row * BK + swizzle_chunk<BK>(row, c) * 8) = regs[i];
      } else {
        int krow = q / (ROWS / 8), c = q % (ROWS / 8);
        *(uint4*)(lds + krow * KS_LD + c * 8) = regs[i];
      }
    }
  }

  // LDS -> MFMA fragment for the 32 rows starting at `row0`, reduction step `ks` (16 elements).
  static __device__ __forceinline__ vec8 frag(const T* lds, int row0, int ks, int lane) {
    int row = row0 + (lane & 31);
    if (!KS) {
      int c = ks * 2 + (lane >> 5);
      return *(const vec8*)(lds + row * BK + swizzle_chunk<BK>(row, c) * 8);
    } else {
      vec8 f;
      int kb = ks * 16 + 8 * (lane >> 5);
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = lds[(kb + j) * KS_LD + row];
      return f;
    }
  }
};

template <typename T, int BM, int BN, int BK, int WGM, int WGN, bool A_KS, bool B_KS, int NB,
          bool EDGE>
struct GemmConfig {
  static constexpr int NT = WGM * WGN * 64;
  static constexpr int WTM = BM / WGM, WTN = BN / WGN;
  static constexpr int TM = WTM / 32, TN = WTN / 32;
  typedef OperandTile<T, BM, BK, A_KS, NT, EDGE> ATile;
  typedef OperandTile<T, BN, BK, B_KS, NT, EDGE> BTile;
  static constexpr int STAGE_ELEMS = ATile::LDS_ELEMS + NB * BTile::LDS_ELEMS;
  static constexpr int LDS_BYTES = 2 * STAGE_ELEMS * (int)sizeof(T);
};

template <typename T, int BM, int BN, int BK, int WGM, int WGN, bool A_KS, bool B_KS, int NB,
          bool EDGE, typename Epi>
__global__ void __launch_bounds__(WGM* WGN * 64)
    gemm_kernel(GemmArgs ga, typename Epi::Args ea) {
  typedef GemmConfig<T, BM, BN, BK, WGM, WGN, A_KS, B_KS, NB, EDGE> Cfg;
  typedef typename Cfg::ATile ATile;
  typedef typename Cfg::BTile BTile;
  typedef typename Traits<T>::vec8 vec8;
  constexpr int TM = Cfg::TM, TN = Cfg::TN;

  extern __shared__ __align__(16) char smem_raw[];
  T* smem = (T*)smem_raw;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN;

  const int tiles_m = (ga.M + BM - 1) / BM, tiles_n = (ga.N + BN - 1) / BN;
  int tm_i, tn_i;
  map_tile(blockIdx.x, gridDim.x, ga.nxcd, tiles_m, tiles_n, ga.group_m, tm_i, tn_i);
  const int m0 = tm_i * BM, n0 = tn_i * BN;

  f32x16 acc[NB][TM][TN];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[b][i][j][r] = 0.f;

  ATile at;
  BTile bt[NB];

  const int kt_seg = (ga.K + BK - 1) / BK;
  const int kt_total = kt_seg * ga.nseg;

  auto issue_loads = [&](int kt) {
    int seg = kt / kt_seg;
    int k0 = (kt - seg * kt_seg) * BK;
    at.gload((const T*)ga.A[seg], ga.lda, m0, k0, ga.M, ga.K, tid);
#pragma unroll
    for (int b = 0; b < NB; ++b)
      bt[b].gload((const T*)ga.B[NB == 2 ? b : seg], ga.ldb, n0, k0, ga.N, ga.K, tid);
  };
  auto commit = [&](int stage) {
    T* s = smem + stage * Cfg::STAGE_ELEMS;
    at.sstore(s, tid);
#pragma unroll
    for (int b = 0; b < NB; ++b) bt[b].sstore(s + ATile::LDS_ELEMS + b * BTile::LDS_ELEMS, tid);
  };

  issue_loads(0);
  commit(0);
  __syncthreads();

  for (int kt = 0; kt < kt_total; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < kt_total) issue_loads(kt + 1);

    const T* sa = smem + cur * Cfg::STAGE_ELEMS;
    const T* sb = sa + ATile::LDS_ELEMS;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      vec8 af[TM];
#pragma unroll
      for (int i = 0; i < TM; ++i) af[i] = ATile::frag(sa, wm * Cfg::WTM + i * 32, ks, lane);
#pragma unroll
      for (int b = 0; b < NB; ++b) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          vec8 bf = BTile::frag(sb + b * BTile::LDS_ELEMS, wn * Cfg::WTN + j * 32, ks, lane);
#pragma unroll
          for (int i = 0; i < TM; ++i) acc[b][i][j] = Traits<T>::mfma(bf, af[i], acc[b][i][j]);
        }
      }
    }

    if (kt + 1 < kt_total) commit(cur ^ 1);
    __syncthreads();
  }

  // Epilogue: lane holds, for row m, 4 consecutive columns per group g.
  const int mrow = lane & 31, nsub = 4 * (lane >> 5);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    int m = m0 + wm * Cfg::WTM + i * 32 + mrow;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        int n = n0 + wn * Cfg::WTN + j * 32 + 8 * g + nsub;
        if (EDGE && (m >= ga.M || n >= ga.N)) continue;
        float v0[4], v1[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          v0[r] = acc[0][i][j][4 * g + r];
          v1[r] = acc[NB - 1][i][j][4 * g + r];
        }
        Epi::template apply<4>(ea, m, n, v0, v1);
      }
    }
  }
}

// ----------------------------------------------------------------------------- epilogues
// Every epilogue handles W (4 or 8) consecutive columns n..n+W-1 of one output row m; v0/v1 are
// the fp32 accumulators of the first/second accumulator set.

template <typename T, int W>
struct PackW;
template <typename T>
struct PackW<T, 4> { typedef typename Traits<T>::vec4 type; };
template <typename T>
struct PackW<T, 8> { typedef typename Traits<T>::vec8 type; };

// STREAM: non-temporal store, for results nobody reads soon (layer outputs, gradients handed to
// other layers or to the optimizer): they then do not push operand panels out of the caches.
template <typename T, int W, bool STREAM = false>
__device__ __forceinline__ void store_w(T* p, const float* v) {
  typename PackW<T, W>::type o;
#pragma unroll
  for (int r = 0; r < W; ++r) o[r] = Traits<T>::from_f32(v[r]);
  if (STREAM) __builtin_nontemporal_store(o, (typename PackW<T, W>::type*)p);
  else *(typename PackW<T, W>::type*)p = o;
}
template <typename T, int W>
__device__ __forceinline__ void load_w(const T* p, float* v) {
  typename PackW<T, W>::type o = *(const typename PackW<T, W>::type*)p;
#pragma unroll
  for (int r = 0; r < W; ++r) v[r] = Traits<T>::to_f32(o[r]);
}
template <typename T, int W>
__device__ __forceinline__ void add_w(const T* p, float* v) {
  float t[W];
  load_w<T, W>(p, t);
#pragma unroll
  for (int r = 0; r < W; ++r) v[r] += t[r];
}
template <int W>
__device__ __forceinline__ void keep_w(const DropoutParams& d, size_t e, bool* keep) {
#pragma unroll
  for (int q = 0; q < W / 4; ++q) dropout_keep4(d, (e >> 2) + q, keep + 4 * q);
}

// out = acc (+ bias[n])
template <typename T>
struct EpiStore {
  struct Args {
    T* out;
    const T* bias;  // nullable
    int ldc;
  };
  template <int W>
  static __device__ __forceinline__ void apply(const Args& a, int m, int n, float* v, float*) {
    if (a.bias) add_w<T, W>(a.bias + n, v);
    store_w<T, W, true>(a.out + (size_t)m * a.ldc + n, v);
  }
  // Nothing worth fetching ahead of time (see EpiDh), no activation to specialise on.
  static constexpr int PREFETCH_DEPTH = 0;
  static constexpr bool HAS_ACT = false;
  static constexpr bool SPLIT = false;
  template <int W>
  struct Prefetch {};
  template <int W>
  static __device__ __forceinline__ void prefetch(const Args&, int, int, Prefetch<W>&) {}
  template <int W, int ACT>
  static __device__ __forceinline__ void apply(const Args& a, int m, int n, float* v, float* w,
                                               const Prefetch<W>&) {
    apply<W>(a, m, n, v, w);
  }
  // Accumulator-layout interface: the arithmetic runs on 4 consecutive columns of one row, as an
  // MFMA leaves them in a lane, and yields the output planes already rounded to T; the kernel then
  // transposes 2-byte elements through LDS instead of 4-byte ones.  Same operations per element
  // as apply(), so the results are bit-identical.  Everything that would branch (optional biases,
  // optional outputs) stays out of the way of the accumulators: biases arrive as values (zeros
  // when absent), optional outputs are whole planes that a uniform branch skips.
  static constexpr bool PACKED = true;
  static constexpr int PLANES = 1;
  static constexpr int NBIAS = 1;
  static constexpr bool STREAM_OUT = true;
  static __device__ __forceinline__ int planes_on(const Args&) { return 1; }
  static __device__ __forceinline__ T* plane(const Args& a, int) { return a.out; }
  static __device__ __forceinline__ void bias4(const Args& a, int n, float (&b)[NBIAS][4]) {
#pragma unroll
    for (int r = 0; r < 4; ++r) b[0][r] = 0.f;
    if (a.bias) load_w<T, 4>(a.bias + n, b[0]);
  }
  static __device__ __forceinline__ void pack4(const Args&, int, int, const float (&b)[NBIAS][4],
                                               const float* v, const float*,
                                               typename PackW<T, 4>::type (&o)[PLANES]) {
#pragma unroll
    for (int r = 0; r < 4; ++r) o[0][r] = Traits<T>::from_f32(v[r] + b[0][r]);
  }
};

// Split reduction: workgroup `split` of an output tile stores its fp32 partial sums to
// ws[split][acc][m][n] (acc: accumulator set, for NB == 2); splitk_reduce (aux.hip) adds the
// partials up and applies the real epilogue.
template <typename T>
struct EpiPartial {
  struct Args {
    float* ws;
    size_t split_stride;  // elements between the partial results of consecutive splits
    size_t acc_stride;    // elements between the two accumulator sets of one split (0: one set)
    int ldc;
  };
  static constexpr int PREFETCH_DEPTH = 0;
  static constexpr bool HAS_ACT = false;
  static constexpr bool SPLIT = true;
  static constexpr bool PACKED = false;
  template <int W>
  struct Prefetch {};
  template <int W>
  static __device__ __forceinline__ void prefetch(const Args&, int, int, Prefetch<W>&) {}
  template <int W, int ACT>
  static __device__ __forceinline__ void apply(const Args& a, int m, int n, float* v0, float* v1,
                                               const Prefetch<W>&) {
    float* p = a.ws + (size_t)m * a.ldc + n;
#pragma unroll
    for (int q = 0; q < W / 4; ++q) *(f32x4*)(p + 4 * q) = *(const f32x4*)(v0 + 4 * q);
    if (a.acc_stride) {
#pragma unroll
      for (int q = 0; q < W / 4; ++q) *(f32x4*)(p + a.acc_stride + 4 * q) = *(const f32x4*)(v1 + 4 * q);
    }
  }
};

// G = acc0 + b_gate, U = acc1 + b_up, H = dropout(act(G) * U)
template <typename T>
struct EpiGateUp {
  struct Args {
    T* h;
    T* g_save;          // nullable
    T* u_save;          // nullable
    uint8_t* mask_out;  // nullable
    const T* b_gate;    // nullable
    const T* b_up;      // nullable
    int ldc;
    int act;            // Act code
    DropoutParams drop;
    size_t drop_e0;     // element index, in the whole [M, ldc] tensor, of what h points at: the
                        // dropout counter of an element is its index in the whole tensor, also
                        // when a launch covers a range of columns only
  };
  // ACT: activation fixed at compile time, or ACT_RUNTIME to read a.act.  A kernel whose epilogue
  // is unrolled many times instantiates both and branches once, so that the usual SiLU path stays
  // as compact as if it were the only one (HAS_ACT tells it that the choice exists).
  static constexpr bool HAS_ACT = true;
  static constexpr bool SPLIT = false;
  template <int W, int ACT = ACT_RUNTIME>
  static __device__ __forceinline__ void apply(const Args& a, int m, int n, float* g, float* u) {
    if (a.b_gate) add_w<T, W>(a.b_gate + n, g);
    if (a.b_up) add_w<T, W>(a.b_up + n, u);
    size_t e = (size_t)m * a.ldc + n;
    float h[W];
    act_fwd_w<W, ACT>(a.act, g, h);
#pragma unroll
    for (int r = 0; r < W; ++r) h[r] *= u[r];
    if (a.drop.enabled) {
      bool keep[W];
      keep_w<W>(a.drop, e + a.drop_e0, keep);
#pragma unroll
      for (int r = 0; r < W; ++r) h[r] = keep[r] ? h[r] * a.drop.scale : 0.f;
      if (a.mask_out) {
#pragma unroll
        for (int q = 0; q < W / 4; ++q) {
          uint32_t packed = 0;
#pragma unroll
          for (int r = 0; r < 4; ++r) packed |= (keep[4 * q + r] ? 1u : 0u) << (8 * r);
          *(uint32_t*)(a.mask_out + e + 4 * q) = packed;
        }
      }
    } else if (a.mask_out) {
#pragma unroll
      for (int q = 0; q < W / 4; ++q) *(uint32_t*)(a.mask_out + e + 4 * q) = 0x01010101u;
    }
    store_w<T, W>(a.h + e, h);
    if (a.g_save) store_w<T, W>(a.g_save + e, g);
    if (a.u_save) store_w<T, W>(a.u_save + e, u);
  }
  static constexpr int PREFETCH_DEPTH = 0;
  template <int W>
  struct Prefetch {};
  template <int W>
  static __device__ __forceinline__ void prefetch(const Args&, int, int, Prefetch<W>&) {}
  template <int W, int ACT>
  static __device__ __forceinline__ void apply(const Args& a, int m, int n, float* g, float* u,
                                               const Prefetch<W>&) {
    apply<W, ACT>(a, m, n, g, u);
  }
  static constexpr bool PACKED = false;  // see EpiGateUpPacked
};

// The same epilogue for kernels that run it in the accumulator layout (see EpiStore): SiLU, no
// keep-mask output, G and U kept both or not at all (packed_eligible; the launcher picks the
// kernel).  Planes H, G, U; the optional parts are uniform branches around small pieces of
// straight-line code.
template <typename T>
struct EpiGateUpPacked : EpiGateUp<T> {
  typedef typename EpiGateUp<T>::Args Args;
  static constexpr bool PACKED = true;
  static constexpr int PLANES = 3;
  static constexpr int NBIAS = 2;
  static constexpr bool STREAM_OUT = false;
  static bool packed_eligible(const Args& a) {
    return a.mask_out == nullptr && a.act == ACT_SILU && (a.g_save == nullptr) == (a.u_save == nullptr);
  }
  static __device__ __forceinline__ int planes_on(const Args& a) { return a.g_save != nullptr ? 3 : 1; }
  static __device__ __forceinline__ T* plane(const Args& a, int p) {
    return p == 0 ? a.h : p == 1 ? a.g_save : a.u_save;
  }
  static __device__ __forceinline__ void bias4(const Args& a, int n, float (&b)[NBIAS][4]) {
#pragma unroll
    for (int r = 0; r < 4; ++r) b[0][r] = b[1][r] = 0.f;
    if (a.b_gate) load_w<T, 4>(a.b_gate + n, b[0]);
    if (a.b_up) load_w<T, 4>(a.b_up + n, b[1]);
  }
  static __device__ __forceinline__ void pack4(const Args& a, int m, int n, const float (&b)[NBIAS][4],
                                               const float* gacc, const float* uacc,
                                               typename PackW<T, 4>::type (&o)[PLANES]) {
    float g[4], u[4], h[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      g[r] = gacc[r] + b[0][r];
      u[r] = uacc[r] + b[1][r];
    }
    act_fwd_w<4, ACT_SILU>(ACT_SILU, g, h);
#pragma unroll
    for (int r = 0; r < 4; ++r) h[r] *= u[r];
    if (a.drop.enabled) {
      bool keep[4];
      keep_w<4>(a.drop, (size_t)m * a.ldc + n + a.drop_e0, keep);
#pragma unroll
      for (int r = 0; r < 4; ++r) h[r] = keep[r] ? h[r] * a.drop.scale : 0.f;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      o[0][r] = Traits<T>::from_f32(h[r]);
      o[1][r] = Traits<T>::from_f32(g[r]);
      o[2][r] = Traits<T>::from_f32(u[r]);
    }
  }
};

// Gating backward on W consecutive elements: dA = dH*keep/(1-p); dU = dA*act(G); dG = dA*U*act'(G)
template <typename T, int W, int ACT = ACT_RUNTIME>
__device__ __forceinline__ void gating_bwd_core(int act, const DropoutParams& drop, size_t e, float* dh,
                                                typename PackW<T, W>::type gp,
                                                typename PackW<T, W>::type up, T* dg, T* du,
                                                size_t drop_e0 = 0) {
  float dgv[W], duv[W];
  if (drop.enabled) {
    bool keep[W];
    keep_w<W>(drop, e + drop_e0, keep);  // drop_e0: see EpiGateUp::Args
#pragma unroll
    for (int r = 0; r < W; ++r) dh[r] = keep[r] ? dh[r] * drop.scale : 0.f;
  }
  float gv[W], av[W], dv[W];
#pragma unroll
  for (int r = 0; r < W; ++r) gv[r] = Traits<T>::to_f32(gp[r]);
  act_fwd_grad_w<W, ACT>(act, gv, av, dv);
#pragma unroll
  for (int r = 0; r < W; ++r) {
    duv[r] = dh[r] * av[r];
    dgv[r] = dh[r] * Traits<T>::to_f32(up[r]) * dv[r];
  }
  store_w<T, W, true>(dg + e, dgv);  // 2*M*N elements: more than the caches keep for the next kernels
  store_w<T, W, true>(du + e, duv);
}
template <typename T, int W>
__device__ __forceinline__ void gating_bwd_w(int act, const DropoutParams& drop, size_t e,
                                             float* dh, const T* g, const T* u, T* dg, T* du,
                                             size_t drop_e0 = 0) {
  typedef typename PackW<T, W>::type pack;
  gating_bwd_core<T, W>(act, drop, e, dh, *(const pack*)(g + e), *(const pack*)(u + e), dg, du, drop_e0);
}

template <typename T>
struct EpiDh {
  struct Args {
    const T* g;
    const T* u;
    T* dg;
    T* du;
    int ldc;
    int act;  // Act code
    DropoutParams drop;
    size_t drop_e0;  // see EpiGateUp::Args
  };
  template <int W>
  static __device__ __forceinline__ void apply(const Args& a, int m, int n, float* dh, float*) {
    gating_bwd_w<T, W>(a.act, a.drop, (size_t)m * a.ldc + n, dh, a.g, a.u, a.dg, a.du, a.drop_e0);
  }
  // G and U come from HBM and every workgroup of a round reaches its epilogue at about the same
  // time; a kernel that can, fetches them this many W-wide items ahead of their use.
  // (8 W-wide items; 12 and 16 measured the same)
  static constexpr int PREFETCH_DEPTH = 8;
  template <int W>
  struct Prefetch {
    typename PackW<T, W>::type g, u;
  };
  template <int W>
  static __device__ __forceinline__ void prefetch(const Args& a, int m, int n, Prefetch<W>& p) {
    typedef typename PackW<T, W>::type pack;
    size_t e = (size_t)m * a.ldc + n;
    p.g = __builtin_nontemporal_load((const pack*)(a.g + e));  // read once
    p.u = __builtin_nontemporal_load((const pack*)(a.u + e));
  }
  static constexpr bool HAS_ACT = true;
  static constexpr bool SPLIT = false;
  static constexpr bool PACKED = false;  // G and U arrive row-wise: the arithmetic stays behind the transpose
  template <int W, int ACT>
  static __device__ __forceinline__ void apply(const Args& a, int m, int n, float* dh, float*,
                                               const Prefetch<W>& p) {
    gating_bwd_core<T, W, ACT>(a.act, a.drop, (size_t)m * a.ldc + n, dh, p.g, p.u, a.dg, a.du, a.drop_e0);
  }
};

}  // namespace gmlp
