// Pipelined full-tile MFMA GEMM for gfx950.
//
// Same contract as gemm_kernel (gemm.hpp): C[M,N] = sum_s sum_k A_s[m,k] * B_s[n,k], operands
// reduction-contiguous (KC) or reduction-strided (KS), NB accumulator sets, fused epilogue.
// Reduction tiles of 64 elements travel global -> LDS without passing through registers
// (gemm_tiles.hpp) into a two-slot ring (three slots for the A operand of the plain-store GEMMs with a
// long reduction, see PipeConfig::A3); the epilogue transposes accumulators (or finished
// results) through LDS so that every global access is a 16-byte, row-contiguous one.
//
// Ragged edges cost nothing in the main loop: operands are read through buffer descriptors of
// their exact size, so whatever a tile addresses beyond the END of an operand reads as zero.
//   * M and N need not be multiples of the tile: rows of a KC operand beyond the last one lie
//     beyond its end; columns of a KS operand beyond the last one alias the next reduction row,
//     which only feeds output rows/columns that the epilogue does not store.
//   * K need not be a multiple of 64 when BOTH operands are KS (reduction rows beyond K lie beyond
//     the end: the weight gradients, whose reduction runs over the tokens).  With a KC operand K
//     must be a multiple of 64 (its tail would alias the next row); the host checks.
//
// Per 512/MI-wide reduction step a wavefront issues G groups of TM MFMAs: group g multiplies one
// B fragment (accumulator set b, column block j; G = NB * TN) with the step's TM A fragments.
// Operands roll through registers instead of being double-buffered a whole step at a time:
//   * A fragments: two banks of TM; during step s, group g fetches A fragment g of step s+1;
//   * B fragments: a ring of 4; group g fetches the B fragment of group g+LA (LA = 3 by default).
// That is 2*TM + 4 fragments in flight (72 VGPRs for the 16x16x32 shape instead of 128), which is
// what lets v_mfma_f32_16x16x32 be used with a 128x128 register tile: it moves a fifth fewer
// register bytes per FLOP than 32x32x16 (4 accumulator floats per lane and instruction instead of
// 16), and on MI355X, where these kernels run power-limited, that shows up as clock.
//
// A reduction tile's ring slot is retired at ONE barrier, placed in the tile's last step where the
// rolling fetches stop addressing the tile: before group G-LA.  After it, the last LA groups fetch
// the next tile's first B fragments and all of its first A fragments, and the global->LDS refill of
// the freed slot starts, paced over the following MFMA slots.
//
// With a split-reduction epilogue (Epi::SPLIT) several workgroups share an output tile, each
// reducing its own range of reduction tiles into a partial result.
#pragma once
#include "gemm_tiles.hpp"

namespace gmlp {

// Two-entry ring: one global->LDS load per this many MFMA cycles (32, 96 and 128 measured slower).
constexpr int LOAD_CYCLES = 64;
// MFMA groups between the fetch of a B fragment and its use (2 measured 0.3 % slower).
constexpr int B_LOOKAHEAD = 3;

// Kernels that get the three-entry A ring (see PipeConfig::A3): those with a reduction-contiguous A
// operand other than dH, i.e. gate/up, the down projection and the input gradient.  The long
// reductions over the intermediate size gain most (they stall on a full vector-memory queue
// otherwise), gate/up gains from a cold start only.  dH's epilogue prefetch and the weight
// gradients' two transposed operands leave no registers for it (spills when tried).
template <typename T, typename Epi>
constexpr bool wants_ring_a3() {
  return !std::is_same<Epi, EpiDh<T>>::value;
}

template <typename T, int BM, int BN, int MI, int WGM, int WGN, bool A_KS, bool B_KS, int NB, bool RING_A3 = false>
struct PipeConfig {
  static_assert(MI == 16, "the loop is written for v_mfma_f32_16x16x32 (4 accumulator floats per lane)");
  static constexpr int BK = 64, NS = 2;
  static constexpr int NW = WGM * WGN;
  static constexpr int WTM = BM / WGM, WTN = BN / WGN;
  static constexpr int TM = WTM / MI, TN = WTN / MI, G = NB * TN;
  static constexpr int KF = 512 / MI;            // reduction elements per MFMA
  static constexpr int KSTEPS = BK / KF;
  static constexpr int MFMA_CYCLES = 16;
  typedef LdsTile<T, BM, BK, A_KS, NW> ATile;
  typedef LdsTile<T, BN, BK, B_KS, NW> BTile;
  static constexpr int STAGE = ATile::BYTES + NB * BTile::BYTES;
  static constexpr int LOADS = ATile::PER_WAVE + NB * BTile::PER_WAVE;  // per wave per tile
  static constexpr int EPI_LD = WTN + 4;                                // fp32 staging row
  static constexpr int EPI_WAVE_BYTES = NB * MI * EPI_LD * 4;
  // A3: THREE ring entries of the A operand and two of the B operand(s), all of a workgroup's
  // 160 KiB (80 KiB for the 128-row tiles: two workgroups per CU as before).  The A loads of a tile then have two tiles' time to land, so a tile's loads can be
  // spread evenly over the tile (B in its first half, A in its second) instead of going out back
  // to back at the rate the texture addresser can take at best, which is where a load that misses
  // L2 backs the queue up into the issuing wavefronts (down projection: queue-full stalls 166 -> 10
  // clocks per tile, 2664 -> 2451 clocks per tile, -4 % run time; input gradient -2 %).
  static constexpr bool A3 = RING_A3 && (BM == 256 || BM == 128) && !A_KS;
  static constexpr int MAIN_BYTES = A3 ? 3 * ATile::BYTES + NS * NB * BTile::BYTES : NS * STAGE;
  static_assert(MAIN_BYTES <= 160 * 1024, "a workgroup has 160 KiB of LDS");
  static constexpr int LDS_BYTES = MAIN_BYTES > NW * EPI_WAVE_BYTES ? MAIN_BYTES : NW * EPI_WAVE_BYTES;
  static_assert(G >= 2 && TM >= 2 && TM % 2 == 0, "rolling scheme needs >= 2 groups and an even TM");
  static_assert((KSTEPS * G) % 4 == 0, "B ring index must be static");
  static_assert(TM <= G, "one A fetch per group must cover the next step");
  static_assert(KSTEPS % 2 == 0, "A banks alternate by step and every tile starts on bank 0");
  static_assert(NS == 2, "the retiring barrier waits for everything in flight");
};

template <typename T, int BM, int BN, int MI, int WGM, int WGN, bool A_KS, bool B_KS, int NB,
          typename Epi, bool SK = false>
__device__ __forceinline__ void gemm_pipelined_body(const GemmArgs& ga, const typename Epi::Args& ea_in,
                                                    int pid, int nwg) {
  typedef PipeConfig<T, BM, BN, MI, WGM, WGN, A_KS, B_KS, NB, wants_ring_a3<T, Epi>()> Cfg;
  typedef typename Cfg::ATile ATile;
  typedef typename Cfg::BTile BTile;
  typedef typename Traits<T>::vec8 vec8;
  typedef f32x4 acc_t;
  constexpr int BK = Cfg::BK, NS = Cfg::NS;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, G = Cfg::G, WTM = Cfg::WTM, WTN = Cfg::WTN;
  constexpr int KSTEPS = Cfg::KSTEPS, STAGE = Cfg::STAGE, L = Cfg::LOADS;
  constexpr int LOAD_SLOTS = LOAD_CYCLES / Cfg::MFMA_CYCLES;  // MFMA slots per load
  constexpr int TILE_SLOTS = KSTEPS * G * TM;                         // MFMA slots per tile
  constexpr bool A3 = Cfg::A3;
  constexpr int LA = B_LOOKAHEAD;
  static_assert(LA >= 2 && LA <= 3 && LA <= G, "B ring has 4 entries");
  constexpr int HEAD_SLOTS = LA * TM;  // slots between the retiring barrier and the tile's end
  // Fragment fetches sit in slots 0 and 1 of a group; with four or more slots per load the loads
  // keep away from them.
  constexpr int LOAD_PHASE = LOAD_SLOTS >= 4 ? 2 : 0;
  static_assert(LOAD_SLOTS >= 1 && L * LOAD_SLOTS <= TILE_SLOTS, "a tile's loads must fit a tile");
  static_assert((L - 1) * LOAD_SLOTS + LOAD_PHASE < HEAD_SLOTS + (KSTEPS - 1) * G * TM + TM - 1,
                "a tile's last load goes out before the load state moves on (first group of the last step)");

  extern __shared__ __align__(1024) char smem_raw[];
  char* smem = smem_raw;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;

  const int tiles_m = (ga.M + BM - 1) / BM, tiles_n = (ga.N + BN - 1) / BN;
  const int ntiles = tiles_m * tiles_n;
  const int kt_seg = (ga.K + BK - 1) / BK;
  const int kt_all = kt_seg * ga.nseg;  // 64-wide reduction tiles of one output tile
  typename Epi::Args ea = ea_in;

  // What this workgroup computes, as a sequence of pieces (output tile, range of reduction tiles):
  //   * one whole tile (the usual case; workgroup -> tile in XCD-contiguous, grouped order);
  //   * with a split-reduction epilogue, one tile's share `split` of the reduction: all tiles of
  //     split 0, then all tiles of split 1, ...;
  //   * stream-K (SK, a kernel instance and a launch of its own behind the launch that covers the
  //     other tiles): ga.sk_wgs workgroups share out the reduction tiles of the problem's last
  //     ga.sk_tiles output tiles evenly, as one range of (tile, reduction tile) pairs each; a range
  //     covers the end of one tile and the start of the next (or more), and every piece leaves
  //     its partial sums in accumulator layout in slot (workgroup + tile) of ga.sk_ws, from where
  //     streamk_fixup_kernel adds a tile's pieces up in reduction order and runs the epilogue.
  //     (One kernel with a run-time choice between the epilogue and the partial store was measured
  //     1.5 to 2 % slower on every launch: the branches sit inside the unrolled epilogue loops, since
  //     a second loop over the accumulators makes the compiler copy all of them to VGPRs first.)
  static_assert(!(SK && Epi::SPLIT), "stream-K pieces replace the epilogue");
  const int dp_tiles = ntiles - (Epi::SPLIT ? 0 : ga.sk_tiles);
  constexpr bool streamk = SK;
  int sk_wg = 0;
  long long sk_cursor = 0, sk_end = 0;  // position in the stream-K iteration space: tile * kt_all + reduction tile
  if (streamk) {
    sk_wg = xcd_contiguous(pid, ga.sk_wgs, ga.nxcd);
    const long long iters = (long long)ga.sk_tiles * kt_all;
    sk_cursor = iters * sk_wg / ga.sk_wgs;
    sk_end = iters * (sk_wg + 1) / ga.sk_wgs;
  }
  const int u_dp = streamk ? 0 : xcd_contiguous(pid, Epi::SPLIT ? nwg : dp_tiles, ga.nxcd);
  const int split = Epi::SPLIT ? u_dp / ntiles : 0;
  if constexpr (Epi::SPLIT) ea.ws += (size_t)split * ea.split_stride;

  // Per piece (set at the top of the piece loop further down): tile origin, reduction range, the
  // order in which the range is read from memory (the sum does not mind: see GemmArgs::rotate).
  int m0 = 0, n0 = 0, kt_first = 0, kt_total = 0, kt_len = 0, rot = 0;
  uint32_t a_org = 0, b_org = 0;
  float* partial_slot = nullptr;  // stream-K piece: where its partial sums go

  acc_t acc[G][TM];

  // Per-lane load offsets (constant), per-operand tile origins and per-tile strides (uniform).
  // Buffer addressing uses 32-bit byte offsets from each operand's base; the host checks sizes.
  // Up to four consecutive loads of an operand share one LDS base in M0 and differ by the
  // instruction's immediate offset q*1024; the immediate also moves the global address, so lane
  // offsets carry DMA_BIAS - q*1024 and the buffer descriptors start DMA_BIAS below the operand.
  constexpr int DMA_BIAS = 3072;
  uint32_t aoff[ATile::PER_WAVE], boff[BTile::PER_WAVE];
#pragma unroll
  for (int i = 0; i < ATile::PER_WAVE; ++i)
    aoff[i] = ATile::lane_offset(i, ga.lda, wave, lane) + DMA_BIAS - (i & 3) * 1024;
#pragma unroll
  for (int i = 0; i < BTile::PER_WAVE; ++i)
    boff[i] = BTile::lane_offset(i, ga.ldb, wave, lane) + DMA_BIAS - (i & 3) * 1024;
  const uint32_t a_step = A_KS ? (uint32_t)BK * ga.lda * 2 : (uint32_t)BK * 2;
  const uint32_t b_step = B_KS ? (uint32_t)BK * ga.ldb * 2 : (uint32_t)BK * 2;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void*)smem;
  const uint32_t a_bytes = (uint32_t)(A_KS ? ga.K : ga.M) * ga.lda * 2 + DMA_BIAS - (uint32_t)ga.a_trim;
  const uint32_t b_bytes = (uint32_t)(B_KS ? ga.K : ga.N) * ga.ldb * 2 + DMA_BIAS - (uint32_t)ga.b_trim;
  const buffer_rsrc ra[2] = {make_rsrc((const char*)ga.A[0] - DMA_BIAS, a_bytes),
                             make_rsrc((const char*)ga.A[1] - DMA_BIAS, a_bytes)};
  const buffer_rsrc rb[2] = {make_rsrc((const char*)ga.B[0] - DMA_BIAS, b_bytes),
                             make_rsrc((const char*)ga.B[1] - DMA_BIAS, b_bytes)};

  // Global->LDS load number x (0 .. L-1) of this wavefront for reduction tile kt_req: operand and
  // index within the operand's loads.
  auto load_index = [](int x) __attribute__((always_inline)) {
    return x < ATile::PER_WAVE ? x : (x - ATile::PER_WAVE) % BTile::PER_WAVE;
  };
  // Load x is the first of its M0 group.
  auto starts_group = [&](int x) __attribute__((always_inline)) { return (load_index(x) & 3) == 0; };
  // M0 for the group that load x starts.
  auto dma_base = [&](int kt_req, int x) __attribute__((always_inline)) {
    uint32_t s = lds_base + (kt_req & (NS - 1)) * STAGE;
    if (x < ATile::PER_WAVE) {
      set_lds_dma_base(s + (wave * ATile::PER_WAVE + x) * 1024);
    } else {
      int y = x - ATile::PER_WAVE, bsel = y / BTile::PER_WAVE, i = y % BTile::PER_WAVE;
      set_lds_dma_base(s + ATile::BYTES + bsel * BTile::BYTES + (wave * BTile::PER_WAVE + i) * 1024);
    }
  };
  // Where the loads of ONE reduction tile read from, as scalar state that moves on tile by tile
  // through the piece's tiles in the order they are read.  Moving on is two scalar additions, and
  // at most once per piece something else: the step into the second reduction segment (other
  // operands: dX only) or the wrap-around of a rotated range (see rot; the host never asks for
  // both).  That event is prepared when the piece starts and applied without a branch: a branch
  // inside the unrolled tile body makes the register allocator shuffle accumulators, and
  // recomputing the addresses per load, as the kernel first did, cost some 35 scalar instructions
  // per tile in two clumps, each of which held up the MFMA issue for a dozen slots.  Beyond the
  // piece's last tile the state simply keeps stepping: only the few loads that the last but one
  // tile issues ahead read there, into a ring slot nobody reads again, and whatever lies beyond
  // the end of an operand reads as zeros.
  uint32_t ld_soff_a = 0, ld_soff_b = 0, ld_event_a = 0, ld_event_b = 0;
  // (the two segments' descriptors differ in their first two words only, the base address: the
  // state keeps those as one 64-bit scalar per operand, so that switching is one select each)
  auto rsrc_head = [](const buffer_rsrc& r) __attribute__((always_inline)) {
    return (uint64_t)(uint32_t)r[0] | ((uint64_t)(uint32_t)r[1] << 32);
  };
  uint64_t ld_head_a = rsrc_head(ra[0]), ld_head_b = rsrc_head(rb[0]);
  int ld_countdown = -1;  // advances left before the event; negative: none to come
  bool ld_event_seg = false;
  auto load_state_start = [&]() __attribute__((always_inline)) {
    int kt = kt_first + rot;
    const int seg = kt >= kt_seg ? 1 : 0;
    const int kk = kt - seg * kt_seg;
    ld_soff_a = a_org + kk * a_step;
    ld_soff_b = b_org + kk * b_step;
    ld_head_a = rsrc_head(seg ? ra[1] : ra[0]);
    ld_head_b = rsrc_head(seg ? rb[1] : rb[0]);
    ld_countdown = -1;
    ld_event_seg = false;
    if (rot > 0) {  // wrap around from the range's last tile to its first
      const int seg0 = kt_first >= kt_seg ? 1 : 0, kk0 = kt_first - seg0 * kt_seg;
      ld_countdown = kt_total - 1 - kt;
      ld_event_a = a_org + kk0 * a_step;
      ld_event_b = b_org + kk0 * b_step;
    } else if (seg == 0 && kt_total > kt_seg) {  // on into the second segment
      ld_countdown = kt_seg - 1 - kk;
      ld_event_a = a_org;
      ld_event_b = b_org;
      ld_event_seg = true;
    }
  };
  auto load_state_advance = [&]() __attribute__((always_inline)) {
    const bool fire = ld_countdown == 0;
    const uint32_t na = ld_soff_a + a_step, nb = ld_soff_b + b_step;
    ld_soff_a = fire ? ld_event_a : na;
    ld_soff_b = fire ? ld_event_b : nb;
    ld_countdown -= 1;
    if constexpr (NB == 1) {  // (two accumulator sets: one reduction segment by construction)
      const bool sw = fire && ld_event_seg;
      ld_head_a = sw ? rsrc_head(ra[1]) : ld_head_a;
      ld_head_b = sw ? rsrc_head(rb[1]) : ld_head_b;
    }
  };
  // Load x of the tile the state stands at (M0 must hold its group's base).
  auto issue_one = [&](int x) __attribute__((always_inline)) {
    buffer_rsrc r;
    uint32_t voff, soff;
    if (x < ATile::PER_WAVE) {
      r = buffer_rsrc{(int)(uint32_t)ld_head_a, (int)(uint32_t)(ld_head_a >> 32), ra[0][2], ra[0][3]};
      voff = aoff[x];
      soff = ld_soff_a;
    } else {
      int y = x - ATile::PER_WAVE, bsel = y / BTile::PER_WAVE, i = y % BTile::PER_WAVE;
      r = NB == 2 ? rb[bsel] : buffer_rsrc{(int)(uint32_t)ld_head_b, (int)(uint32_t)(ld_head_b >> 32), rb[0][2], rb[0][3]};
      voff = boff[i];
      soff = ld_soff_b;
    }
    switch (load_index(x) & 3) {
      case 0: load16_to_lds_at<0>(r, voff, soff); break;
      case 1: load16_to_lds_at<1024>(r, voff, soff); break;
      case 2: load16_to_lds_at<2048>(r, voff, soff); break;
      default: load16_to_lds_at<3072>(r, voff, soff); break;
    }
  };

  // ---- A3: separate load states for the two operands (the A loads run one tile ahead of the B
  // loads), and the A ring's entries as byte offsets that rotate tile by tile.
  constexpr int A_ENTRY = ATile::BYTES, A_RING = 3 * ATile::BYTES, B_ENTRY = NB * BTile::BYTES;
  constexpr int LDA = ATile::PER_WAVE, LDB = NB * BTile::PER_WAVE;  // loads per wave and tile
  uint32_t l3_soff[2] = {0, 0}, l3_event[2] = {0, 0};
  uint64_t l3_head[2] = {0, 0};
  int l3_cd[2] = {-1, -1};
  bool l3_seg = false;
  auto l3_start = [&]() __attribute__((always_inline)) {
    load_state_start();
    l3_soff[0] = ld_soff_a; l3_soff[1] = ld_soff_b;
    l3_event[0] = ld_event_a; l3_event[1] = ld_event_b;
    l3_head[0] = ld_head_a; l3_head[1] = ld_head_b;
    l3_cd[0] = l3_cd[1] = ld_countdown;
    l3_seg = ld_event_seg;
  };
  auto l3_advance = [&](int op) __attribute__((always_inline)) {
    const bool fire = l3_cd[op] == 0;
    const uint32_t nx = l3_soff[op] + (op == 0 ? a_step : b_step);
    l3_soff[op] = fire ? l3_event[op] : nx;
    l3_cd[op] -= 1;
    if constexpr (NB == 1) {
      const bool sw = fire && l3_seg;
      l3_head[op] = sw ? rsrc_head(op == 0 ? ra[1] : rb[1]) : l3_head[op];
    }
  };
  // Load z of a tile in issue order: the B loads first (z < LDB), then the A loads.
  auto l3_is_b = [](int z) __attribute__((always_inline)) { return z < LDB; };
  auto l3_index = [](int z) __attribute__((always_inline)) { return z < LDB ? z % BTile::PER_WAVE : z - LDB; };
  auto l3_starts_group = [&](int z) __attribute__((always_inline)) { return (l3_index(z) & 3) == 0; };
  // M0 for the group that load z starts; b_parity: ring entry of the B tile being filled,
  // a_off: ring offset of the A tile being filled.
  auto l3_base = [&](int z, int b_parity, uint32_t a_off) __attribute__((always_inline)) {
    if (l3_is_b(z)) {
      const int bsel = z / BTile::PER_WAVE, i = z % BTile::PER_WAVE;
      set_lds_dma_base(lds_base + A_RING + b_parity * B_ENTRY + bsel * BTile::BYTES +
                       (wave * BTile::PER_WAVE + i) * 1024);
    } else {
      set_lds_dma_base(lds_base + a_off + (wave * ATile::PER_WAVE + (z - LDB)) * 1024);
    }
  };
  auto l3_issue = [&](int z) __attribute__((always_inline)) {
    buffer_rsrc r;
    uint32_t voff, soff;
    if (l3_is_b(z)) {
      const int bsel = z / BTile::PER_WAVE, i = z % BTile::PER_WAVE;
      r = NB == 2 ? rb[bsel] : buffer_rsrc{(int)(uint32_t)l3_head[1], (int)(uint32_t)(l3_head[1] >> 32), rb[0][2], rb[0][3]};
      voff = boff[i];
      soff = l3_soff[1];
    } else {
      r = buffer_rsrc{(int)(uint32_t)l3_head[0], (int)(uint32_t)(l3_head[0] >> 32), ra[0][2], ra[0][3]};
      voff = aoff[z - LDB];
      soff = l3_soff[0];
    }
    switch (l3_index(z) & 3) {
      case 0: load16_to_lds_at<0>(r, voff, soff); break;
      case 1: load16_to_lds_at<1024>(r, voff, soff); break;
      case 2: load16_to_lds_at<2048>(r, voff, soff); break;
      default: load16_to_lds_at<3072>(r, voff, soff); break;
    }
  };
  auto a3_next = [](uint32_t off) __attribute__((always_inline)) {
    const uint32_t n = off + A_ENTRY;
    return n == (uint32_t)A_RING ? 0u : n;
  };
  auto a3_prev = [](uint32_t off) __attribute__((always_inline)) {
    return off == 0u ? (uint32_t)(A_RING - A_ENTRY) : off - A_ENTRY;
  };

  vec8 af[2][TM];  // A fragments: bank = step parity
  vec8 bq[4];      // B fragment ring: entry = (step * G + group) % 4
  auto fetch_a = [&](int bank, int i, int kt, int ks) __attribute__((always_inline)) {
    const char* s = smem + (kt & (NS - 1)) * STAGE;
    af[bank][i] = ATile::template frag_mi<MI>(s, wm * WTM + i * MI, ks, lane);
  };
  auto fetch_b = [&](int entry, int g, int kt, int ks) __attribute__((always_inline)) {
    const char* s = smem + (kt & (NS - 1)) * STAGE;
    const int bsel = g / TN, j = g % TN;
    bq[entry] = BTile::template frag_mi<MI>(s + ATile::BYTES + bsel * BTile::BYTES,
                                            wn * WTN + j * MI, ks, lane);
  };

  auto fetch_a3 = [&](int bank, int i, uint32_t a_off, int ks) __attribute__((always_inline)) {
    af[bank][i] = ATile::template frag_mi<MI>(smem + a_off, wm * WTM + i * MI, ks, lane);
  };
  auto fetch_b3 = [&](int entry, int g, int kt, int ks) __attribute__((always_inline)) {
    const char* s = smem + A_RING + (kt & 1) * B_ENTRY;
    const int bsel = g / TN, j = g % TN;
    bq[entry] = BTile::template frag_mi<MI>(s + bsel * BTile::BYTES, wn * WTN + j * MI, ks, lane);
  };

  // One reduction tile.  NEXT: tile kt+1 exists.  The wavefront is alone on its SIMD: whatever
  // issues between two MFMAs is hidden behind the matrix pipe, so every group is laid out as TM
  // slots of {one MFMA; at most a couple of LDS fetches or one global->LDS load} and the
  // scheduler is told to keep the slots.
  auto tile_body = [&](int kt, auto next_c) __attribute__((always_inline)) {
    constexpr bool NEXT = decltype(next_c)::value;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const bool last = ks == KSTEPS - 1;
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const bool handover = last && g >= G - LA;  // groups that already work for tile kt+1
        if (NEXT && last && g == G - LA) {
          // No fetch addresses this tile's slot any more: wait until tile kt+1 has landed,
          // barrier, then the slot can be refilled.
          wait_vmem<0>();
          __syncthreads();
          if (LOAD_PHASE == 0) dma_base(kt + NS, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          acc[g][i] = Traits<T>::mfma16(bq[(ks * G + g) % 4], af[ks & 1][i], acc[g][i]);
          // --- B fragment of the group LA ahead
          if (i == 0) {
            const int g2 = g + LA;
            if (g2 < G) fetch_b((ks * G + g2) % 4, g2, kt, ks);
            else if (!last) fetch_b(((ks + 1) * G + g2 - G) % 4, g2 - G, kt, ks + 1);
            else if (NEXT) fetch_b((g2 - G) % 4, g2 - G, kt + 1, 0);
          }
          // --- A fragments of the next step: one per group, or all of them after the handover
          if (!last) {
            if (i == 1 && g < TM) fetch_a((ks + 1) & 1, g, kt, ks + 1);
          } else if (NEXT && handover) {
            constexpr int AH = (TM + LA - 1) / LA;  // A fragments per handover group
            const int h = (g - (G - LA)) * AH + (i - 1);
            if (i >= 1 && i <= AH && h < TM) fetch_a(0, h, kt + 1, 0);
          }
          // --- paced refill of the ring slot retired at the last barrier; slots are counted from
          // that barrier, so a tile's loads start in the previous tile's handover groups.  Load x
          // goes to slot x*LOAD_SLOTS + LOAD_PHASE, a new M0 one slot earlier.
          // --- the load state moves on from tile kt+1, whose last load went out during the first
          // step, to tile kt+2: in a slot of the last step that has nothing else to issue
          if (NEXT && last && g == 0 && i == TM - 1) load_state_advance();
          if (NEXT) {
            const int slot = handover ? (g - (G - LA)) * TM + i : HEAD_SLOTS + (ks * G + g) * TM + i;
            const int lkt = handover ? kt + NS : kt + NS - 1;
            if (slot % LOAD_SLOTS == LOAD_PHASE && slot / LOAD_SLOTS < L) issue_one(slot / LOAD_SLOTS);
            const int nx = (slot + 1) / LOAD_SLOTS;
            if ((slot + 1) % LOAD_SLOTS == LOAD_PHASE && nx < L && starts_group(nx)) dma_base(lkt, nx);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };

  // The same for the A3 ring.  Slots are counted from the last barrier (the one in tile kt-1): it
  // frees the B entry of tile kt-1, which takes tile kt+1, and the A entry of tile kt-1, which
  // takes tile kt+2.  The LDA + LDB loads go out one per LSL slots, the B loads first (they must
  // land by the barrier in tile kt), then the A loads (which have until the barrier in tile kt+1):
  // the barrier in tile kt waits for everything but those LDA youngest loads.
  auto tile_body3 = [&](int kt, auto next_c) __attribute__((always_inline)) {
    constexpr bool NEXT = decltype(next_c)::value;
    constexpr int L3 = LDA + LDB;
    constexpr int LSL = TILE_SLOTS / L3, PH = LSL >= 4 ? 2 : 0;
    static_assert(L3 * LSL <= TILE_SLOTS && LSL >= 1, "a tile's loads must fit a tile");
    static_assert((LDB - 1) * LSL + PH < HEAD_SLOTS + (KSTEPS - 1) * G * TM + TM - 1, "last B load before the B state moves on");
    static_assert(LDB * LSL >= HEAD_SLOTS, "A loads go out in the tile proper");
    static_assert((L3 - 1) * LSL + PH < HEAD_SLOTS + (KSTEPS - 1) * G * TM + (G - LA - 1) * TM + TM - 1, "last A load before the A state moves on");
    // (derived from the tile counter: a ring position carried from tile to tile as a variable of
    // its own made the register allocator move accumulators around inside the loop)
    const uint32_t a_rd = ((uint32_t)(kt - kt_first) % 3u) * (uint32_t)A_ENTRY;
    const uint32_t a_nxt = a3_next(a_rd), a_fill = a3_prev(a_rd);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const bool last = ks == KSTEPS - 1;
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const bool handover = last && g >= G - LA;
        if (NEXT && last && g == G - LA) {
          wait_vmem<LDA>();  // all but the A loads of the tile after next
          __syncthreads();
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          acc[g][i] = Traits<T>::mfma16(bq[(ks * G + g) % 4], af[ks & 1][i], acc[g][i]);
          if (i == 0) {
            const int g2 = g + LA;
            if (g2 < G) fetch_b3((ks * G + g2) % 4, g2, kt, ks);
            else if (!last) fetch_b3(((ks + 1) * G + g2 - G) % 4, g2 - G, kt, ks + 1);
            else if (NEXT) fetch_b3((g2 - G) % 4, g2 - G, kt + 1, 0);
          }
          if (!last) {
            if (i == 1 && g < TM) fetch_a3((ks + 1) & 1, g, a_rd, ks + 1);
          } else if (NEXT && handover) {
            constexpr int AH = (TM + LA - 1) / LA;
            const int h = (g - (G - LA)) * AH + (i - 1);
            if (i >= 1 && i <= AH && h < TM) fetch_a3(0, h, a_nxt, 0);
          }
          if (NEXT) {
            const int slot = handover ? (g - (G - LA)) * TM + i : HEAD_SLOTS + (ks * G + g) * TM + i;
            // B entry being filled: behind this tile's barrier that of tile kt (with tile kt+2),
            // before it that of tile kt-1 (with tile kt+1); A entry: a_fill, tile kt+2, always
            // before the barrier.
            const int b_parity = handover ? (kt & 1) : ((kt + 1) & 1);
            if (slot % LSL == PH && slot / LSL < L3) l3_issue(slot / LSL);
            const int nz = (slot + 1) / LSL;
            if ((slot + 1) % LSL == PH && nz < L3 && l3_starts_group(nz)) l3_base(nz, b_parity, a_fill);
            if (last && g == 0 && i == TM - 1) l3_advance(1);
            if (last && g == G - LA - 1 && i == TM - 1) l3_advance(0);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };

  for (;;) {  // pieces of this workgroup (one, unless stream-K)
  int u_tile;
  if (streamk && ga.sk_chunks > 0) {
    // Whole-number pieces per tile: workgroup w takes reduction chunk w / sk_tiles of tile
    // w % sk_tiles, so that the workgroups of an XCD (consecutive w) walk neighbouring tiles over the
    // same reduction range and share operand panels in L2 as the one-tile-per-workgroup grid does.
    const int s_tile = sk_wg % ga.sk_tiles, chunk = sk_wg / ga.sk_tiles;
    kt_first = chunk * kt_all / ga.sk_chunks;
    kt_total = (chunk + 1) * kt_all / ga.sk_chunks;
    sk_cursor = sk_end = 0;
    u_tile = dp_tiles + s_tile;
    partial_slot = ga.sk_ws + (size_t)sk_wg * (size_t)(BM * BN * NB);
  } else if (streamk) {
    const unsigned s_tile = (unsigned)sk_cursor / (unsigned)kt_all;
    const unsigned tile_begin = s_tile * (unsigned)kt_all, tile_end = tile_begin + (unsigned)kt_all;
    kt_first = (int)((unsigned)sk_cursor - tile_begin);
    kt_total = (int)(((unsigned)sk_end < tile_end ? (unsigned)sk_end : tile_end) - tile_begin);
    sk_cursor = tile_begin + (unsigned)kt_total;
    u_tile = dp_tiles + (int)s_tile;
    partial_slot = ga.sk_ws + (size_t)(sk_wg + (int)s_tile) * (size_t)(BM * BN * NB);
  } else {
    u_tile = u_dp - split * ntiles;
    kt_first = 0;
    kt_total = kt_all;
    if constexpr (Epi::SPLIT) {
      const int per = (kt_all + ga.splits - 1) / ga.splits;
      kt_first = split * per;
      kt_total = kt_first + per < kt_all ? kt_first + per : kt_all;
    }
  }
  {
    int tm_i, tn_i;
    tile_of_grouped(u_tile, tiles_m, tiles_n, ga.group_m, tm_i, tn_i);
    // workgroup-uniform by construction; say so, the tile origins feed scalar operands
    m0 = __builtin_amdgcn_readfirstlane(tm_i) * BM;
    n0 = __builtin_amdgcn_readfirstlane(tn_i) * BN;
    kt_first = __builtin_amdgcn_readfirstlane(kt_first);
    kt_total = __builtin_amdgcn_readfirstlane(kt_total);
    kt_len = kt_total - kt_first;
    rot = ga.rotate && kt_len > 0 ? tn_i % kt_len : 0;
    a_org = A_KS ? (uint32_t)m0 * 2 : (uint32_t)m0 * ga.lda * 2;
    b_org = B_KS ? (uint32_t)n0 * 2 : (uint32_t)n0 * ga.ldb * 2;
  }
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int r = 0; r < (int)(sizeof(acc_t) / 4); ++r) acc[g][i][r] = 0.f;

  // Prologue: tile 0 .. NS-2 entirely, and of tile NS-1 the loads the handover groups would have
  // issued (tile 0's own slots issue the rest); wait for tile 0.
  constexpr int HEAD_LOADS = (HEAD_SLOTS - LOAD_PHASE + LOAD_SLOTS - 1) / LOAD_SLOTS;
  constexpr int L_HEAD = HEAD_LOADS < L ? HEAD_LOADS : L;
  if constexpr (A3) {
    constexpr int L3 = LDA + LDB, LSL3 = TILE_SLOTS / L3, PH3 = LSL3 >= 4 ? 2 : 0;
    constexpr int HEAD_B = (HEAD_SLOTS - PH3 + LSL3 - 1) / LSL3 < LDB ? (HEAD_SLOTS - PH3 + LSL3 - 1) / LSL3 : LDB;
    l3_start();
    // tile 0 (A entry 0, B entry kt_first & 1), tile 1's A (entry 1) and the B loads of tile 1 that
    // the handover slots of a tile before would have issued
#pragma unroll
    for (int z = LDB; z < L3; ++z) {
      if (l3_starts_group(z)) l3_base(z, 0, 0u);
      l3_issue(z);
    }
#pragma unroll
    for (int z = 0; z < LDB; ++z) {
      if (l3_starts_group(z)) l3_base(z, kt_first & 1, 0u);
      l3_issue(z);
    }
    l3_advance(0);
    l3_advance(1);
#pragma unroll
    for (int z = LDB; z < L3; ++z) {
      if (l3_starts_group(z)) l3_base(z, 0, (uint32_t)A_ENTRY);
      l3_issue(z);
    }
#pragma unroll
    for (int z = 0; z < HEAD_B; ++z) {
      if (l3_starts_group(z)) l3_base(z, (kt_first + 1) & 1, 0u);
      l3_issue(z);
    }
    l3_advance(0);
    wait_vmem<LDA + HEAD_B>();
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TM; ++i) fetch_a3(0, i, 0u, 0);
#pragma unroll
    for (int g = 0; g < LA; ++g) fetch_b3(g, g, kt_first, 0);
  } else {
    load_state_start();
#pragma unroll
    for (int x = 0; x < L; ++x) {
      if (starts_group(x)) dma_base(kt_first, x);
      issue_one(x);
    }
    load_state_advance();
#pragma unroll
    for (int x = 0; x < L_HEAD; ++x) {
      if (starts_group(x)) dma_base(kt_first + 1, x);
      issue_one(x);
    }
    wait_vmem<L_HEAD>();
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TM; ++i) fetch_a(0, i, kt_first, 0);
#pragma unroll
    for (int g = 0; g < LA; ++g) fetch_b(g, g, kt_first, 0);
  }
  __builtin_amdgcn_sched_barrier(0);

  // Epilogue work items of a wavefront: MI-row slab i of its tile, then (row, 8-column group)
  // items spread over the lanes.  What an epilogue reads from global memory is fetched
  // PREFETCH_DEPTH items ahead, starting before the last reduction tile; items beyond the edge of
  // the output fetch the last valid row / column group instead (no branch around the loads) and
  // are dropped when it comes to storing.
  constexpr int ITEMS = MI * WTN / 8 / 64;  // items per lane and slab
  constexpr int NITEMS = TM * ITEMS;
  constexpr int PD = Epi::PREFETCH_DEPTH < NITEMS ? Epi::PREFETCH_DEPTH : NITEMS;
  static_assert(MI * WTN / 8 % 64 == 0, "slab items must divide over the lanes");
  auto item_pos = [&](int q, int& row, int& m, int& n, int& cg) __attribute__((always_inline)) {
    int i = q / ITEMS, item = (q % ITEMS) * 64 + lane;
    row = item / (WTN / 8);
    cg = item % (WTN / 8);
    m = m0 + wm * WTM + i * MI + row;
    n = n0 + wn * WTN + cg * 8;
  };
  typename Epi::template Prefetch<8> pf[PD > 0 ? PD : 1];

  int kt = kt_first;
  for (; kt + 1 < kt_total; ++kt) {
    if constexpr (A3) tile_body3(kt, std::true_type{});
    else tile_body(kt, std::true_type{});
  }
  // (the operand fragments are still live during the last reduction tile: the first PD_EARLY
  // items are fetched before it, the rest of the PD behind it)
  constexpr int PD_EARLY = PD < 8 ? PD : 8;
  if (PD > 0 && !streamk) {
#pragma unroll
    for (int q = 0; q < PD_EARLY; ++q) {
      int row, m, n, cg;
      item_pos(q, row, m, n, cg);
      Epi::template prefetch<8>(ea, min(m, ga.M - 1), min(n, ga.N - 8), pf[q]);
    }
  }
  if constexpr (A3) tile_body3(kt, std::false_type{});
  else tile_body(kt, std::false_type{});
  if (PD > PD_EARLY && !streamk) {
#pragma unroll
    for (int q = PD_EARLY; q < PD; ++q) {
      int row, m, n, cg;
      item_pos(q, row, m, n, cg);
      Epi::template prefetch<8>(ea, min(m, ga.M - 1), min(n, ga.N - 8), pf[q]);
    }
    wait_vmem<2 * (PD - PD_EARLY)>();
  } else {
    wait_vmem<0>();  // redundant tail loads must not land in the epilogue's staging area
  }

  // ---- epilogue: transpose MI-row slabs through LDS, after which each lane owns 8 consecutive
  // columns of one row: the fp32 accumulators themselves, with the arithmetic behind the transpose
  // (slabs), or, where the epilogue offers it, the finished 16-bit results (further down).
  __syncthreads();  // all wavefronts are done reading operand tiles
  // A stream-K piece stores its accumulators as they are instead (16 bytes per lane and
  // accumulator, contiguous over the wavefront; streamk_fixup_kernel knows the layout).  That
  // store sits inside the loops below, next to the staging store it replaces: a second loop over
  // the accumulators in a branch of its own makes the compiler copy all of them to VGPRs first.
  constexpr int AV = (int)(sizeof(acc_t) / 4);
  float* const sk_slot = partial_slot + ((size_t)wave * (G * TM) * 64 + lane) * AV;
  constexpr int ELD = Cfg::EPI_LD;
  float* stg = (float*)(smem + wave * Cfg::EPI_WAVE_BYTES);
  const int mrow = lane & (MI - 1), nsub = 4 * (lane / MI);
  // The slab loop exists once per activation the epilogue offers, each with the activation fixed
  // at compile time: a run-time switch inside the loop would leave every path threading its way
  // through several times its own code (measured: +7 % for relu to +30 % for gelu on the kernel).
  auto slabs = [&](auto act_c) __attribute__((always_inline)) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const int b = g / TN, j = g % TN;
        const f32x4 o = acc[g][i];
        if (streamk) *(f32x4*)(sk_slot + (size_t)(g * TM + i) * 64 * AV) = o;
        else *(f32x4*)(stg + (b * MI + mrow) * ELD + j * MI + nsub) = o;
      }
      if (streamk) continue;
      // Same-wavefront LDS writes and reads are ordered; no barrier needed for a private slab.
#pragma unroll
      for (int it = 0; it < ITEMS; ++it) {
        const int q = i * ITEMS + it;
        int row, m, n, cg;
        item_pos(q, row, m, n, cg);
        alignas(16) float v0[8], v1[8];
        const float* p0 = stg + row * ELD + cg * 8;
        *(f32x4*)v0 = *(const f32x4*)p0;
        *(f32x4*)(v0 + 4) = *(const f32x4*)(p0 + 4);
        if (NB == 2) {
          const float* p1 = p0 + MI * ELD;
          *(f32x4*)v1 = *(const f32x4*)p1;
          *(f32x4*)(v1 + 4) = *(const f32x4*)(p1 + 4);
        }
        if (m < ga.M && n < ga.N) Epi::template apply<8, ACT>(ea, m, n, v0, v1, pf[q % (PD > 0 ? PD : 1)]);
        if (q + PD < NITEMS) {
          int row2, m2, n2, cg2;
          item_pos(q + PD, row2, m2, n2, cg2);
          Epi::template prefetch<8>(ea, min(m2, ga.M - 1), min(n2, ga.N - 8), pf[q % (PD > 0 ? PD : 1)]);
        }
      }
    }
  };
  // Epilogues that offer it run their arithmetic in the accumulator layout (a lane holds 4
  // consecutive columns of one row per 16x16 block) and hand over results already rounded to T:
  // the transpose through LDS then moves 2-byte elements, one plane per output tensor.  The loop
  // over the accumulators is one piece of straight-line code (alternatives that read the
  // accumulators in several branches made the compiler copy all of them to VGPRs first).
  // Staging of a wavefront: planes x [16 rows][WTN elements], row r's 8-byte unit u stored at
  // u ^ 2 (r >> SH): the 32 lanes of a half-wave write (16 rows x 2 units) hit 64 distinct banks,
  // and a 16-byte read of chunk c of row r finds it at c ^ (r >> SH), 16 lanes covering all banks.
  if constexpr (Epi::PACKED) {
    typedef typename PackW<T, 4>::type vec4;
    constexpr int P = Epi::PLANES;
    constexpr int UPR = WTN / 4;                       // 8-byte units per staging row
    constexpr int SH = UPR >= 32 ? 0 : (UPR == 16 ? 1 : 2);
    static_assert(UPR == 32 || UPR == 16 || UPR == 8, "wavefront tiles are 32 to 128 columns wide");
    static_assert(P * MI * WTN * 2 <= Cfg::EPI_WAVE_BYTES, "staging planes must fit the wavefront's share");
    char* stp = smem + wave * Cfg::EPI_WAVE_BYTES;
    const int cq = lane / MI;                          // which 4 columns of a 16-column block
    const int planes_on = Epi::planes_on(ea);          // uniform
    // biases of this lane's columns (zeros when there is none); columns past the edge read the
    // last valid group instead and are dropped when it comes to storing
    float bias[TN][Epi::NBIAS][4];
#pragma unroll
    for (int j = 0; j < TN; ++j) Epi::bias4(ea, min(n0 + wn * WTN + j * MI + 4 * cq, ga.N - 4), bias[j]);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int m = m0 + wm * WTM + i * MI + mrow;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int n = n0 + wn * WTN + j * MI + 4 * cq;
        float v0[4], v1[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          v0[r] = acc[j][i][r];
          if constexpr (NB == 2) v1[r] = acc[TN + j][i][r];
          else v1[r] = 0.f;
        }
        if (streamk) {
          *(f32x4*)(sk_slot + (size_t)(j * TM + i) * 64 * AV) = f32x4{v0[0], v0[1], v0[2], v0[3]};
          if constexpr (NB == 2) *(f32x4*)(sk_slot + (size_t)((TN + j) * TM + i) * 64 * AV) = f32x4{v1[0], v1[1], v1[2], v1[3]};
          continue;
        }
        vec4 o[P];
        Epi::pack4(ea, m, n, bias[j], v0, v1, o);
        const int unit = (4 * j + cq) ^ (2 * (mrow >> SH));
        *(vec4*)(stp + mrow * (WTN * 2) + unit * 8) = o[0];
        if (P > 1 && planes_on > 1) {
#pragma unroll
          for (int pl = 1; pl < P; ++pl)
            *(vec4*)(stp + pl * (MI * WTN * 2) + mrow * (WTN * 2) + unit * 8) = o[pl];
        }
      }
      if (streamk) continue;
#pragma unroll
      for (int it = 0; it < ITEMS; ++it) {
        int row, m2, n2, cg;
        item_pos(i * ITEMS + it, row, m2, n2, cg);
        const int chunk = cg ^ (row >> SH);
        const bool inside = m2 < ga.M && n2 < ga.N;
#pragma unroll
        for (int pl = 0; pl < P; ++pl) {
          if (pl > 0 && planes_on <= 1) break;
          vec8 val = *(const vec8*)(stp + pl * (MI * WTN * 2) + row * (WTN * 2) + chunk * 16);
          if (inside) {
            vec8* q = (vec8*)(Epi::plane(ea, pl) + (size_t)m2 * ea.ldc + n2);
            if (Epi::STREAM_OUT) __builtin_nontemporal_store(val, q);
            else *q = val;
          }
        }
      }
    }
  } else if constexpr (Epi::HAS_ACT) {
    switch (ea.act) {
      case ACT_SILU: slabs(std::integral_constant<int, ACT_SILU>{}); break;
      case ACT_GELU: slabs(std::integral_constant<int, ACT_GELU>{}); break;
      case ACT_RELU: slabs(std::integral_constant<int, ACT_RELU>{}); break;
      case ACT_LEAKY_RELU: slabs(std::integral_constant<int, ACT_LEAKY_RELU>{}); break;
      case ACT_SIGMOID: slabs(std::integral_constant<int, ACT_SIGMOID>{}); break;
      case ACT_TANH: slabs(std::integral_constant<int, ACT_TANH>{}); break;
      default: slabs(std::integral_constant<int, ACT_IDENTITY>{}); break;
    }
  } else {
    slabs(std::integral_constant<int, ACT_RUNTIME>{});
  }
  if (!streamk || (unsigned)sk_cursor >= (unsigned)sk_end) break;
  __syncthreads();  // the next piece's loads overwrite what this piece's wavefronts were reading
  }  // pieces
}

// Second stage of stream-K: adds up the pieces of each stream-K tile in reduction order (fixed, so
// the result does not depend on timing) and runs the GEMM's epilogue on the sums, four consecutive
// columns of one row per lane as the accumulators hold them.  Same thread -> element map as
// gemm_pipelined_body; workgroup (tile, i) handles the MI-row slab i of every wavefront's part of
// the tile, all its column blocks in flight at once (the kernel is bound by load latency).
template <typename T, int BM, int BN, int MI, int WGM, int WGN, int NB, typename Epi>
__global__ void __launch_bounds__(WGM* WGN * 64) streamk_fixup_kernel(GemmArgs ga, typename Epi::Args ea) {
  typedef PipeConfig<T, BM, BN, MI, WGM, WGN, false, false, NB> Cfg;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, G = Cfg::G, WTM = Cfg::WTM, WTN = Cfg::WTN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / WGN, wn = wave % WGN;
  const int tiles_m = (ga.M + BM - 1) / BM, tiles_n = (ga.N + BN - 1) / BN;
  const int dp_tiles = tiles_m * tiles_n - ga.sk_tiles;
  const int s_tile = blockIdx.x / TM, i = blockIdx.x % TM;
  int tm_i, tn_i;
  tile_of_grouped(dp_tiles + s_tile, tiles_m, tiles_n, ga.group_m, tm_i, tn_i);
  const int m0 = tm_i * BM, n0 = tn_i * BN;
  const unsigned kt_all = (unsigned)(((ga.K + 63) / 64) * ga.nseg);
  const unsigned iters = (unsigned)ga.sk_tiles * kt_all, wgs = (unsigned)ga.sk_wgs;
  const unsigned lo = (unsigned)s_tile * kt_all, hi = lo + kt_all;
  // first workgroup whose range [iters*w/wgs, iters*(w+1)/wgs) reaches into this tile
  unsigned w_first = (unsigned)((unsigned long long)lo * wgs / iters);
  while (w_first > 0 && (unsigned)((unsigned long long)iters * w_first / wgs) > lo) --w_first;
  while ((unsigned)((unsigned long long)iters * (w_first + 1) / wgs) <= lo) ++w_first;
  const size_t slot_floats = (size_t)BM * BN * NB;
  const int mrow = lane & 15, cq = lane >> 4;
  f32x4 v[NB][TN];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int j = 0; j < TN; ++j) v[b][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  // the tile's pieces in reduction order: chunk c in slot c * sk_tiles + tile, or the workgroups
  // whose ranges reach into the tile, workgroup w's piece in slot w + tile
  const bool chunked = ga.sk_chunks > 0;
  const unsigned w_begin = chunked ? 0u : w_first;
  for (unsigned w = w_begin; chunked ? w < (unsigned)ga.sk_chunks
                                     : (w < wgs && (unsigned)((unsigned long long)iters * w / wgs) < hi); ++w) {
    const size_t slot_index = chunked ? (size_t)w * ga.sk_tiles + s_tile : (size_t)w + s_tile;
    const float* slot = ga.sk_ws + slot_index * slot_floats + ((size_t)wave * (G * TM) * 64 + lane) * 4;
    f32x4 t[NB][TN];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int j = 0; j < TN; ++j) t[b][j] = *(const f32x4*)(slot + (size_t)((b * TN + j) * TM + i) * 256);
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int j = 0; j < TN; ++j) v[b][j] += t[b][j];
  }
  const int m = m0 + wm * WTM + i * MI + mrow;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int n = n0 + wn * WTN + j * MI + 4 * cq;
    if (m < ga.M && n < ga.N) {
      float a0[4] = {v[0][j][0], v[0][j][1], v[0][j][2], v[0][j][3]};
      float a1[4] = {v[NB - 1][j][0], v[NB - 1][j][1], v[NB - 1][j][2], v[NB - 1][j][3]};
      Epi::template apply<4>(ea, m, n, a0, a1);
    }
  }
}

template <typename T, int BM, int BN, int MI, int WGM, int WGN, bool A_KS, bool B_KS, int NB,
          typename Epi, bool SK = false>
__global__ void __launch_bounds__(WGM* WGN * 64)
    gemm_kernel_pipelined(GemmArgs ga, typename Epi::Args ea) {
  gemm_pipelined_body<T, BM, BN, MI, WGM, WGN, A_KS, B_KS, NB, Epi, SK>(ga, ea, blockIdx.x, gridDim.x);
}

// The stream-K launches behind a launch that left ga.sk_tiles tiles out: the pieces, then the sums.
template <typename T, int BM, int BN, int MI, int WGM, int WGN, bool A_KS, bool B_KS, int NB,
          typename Epi>
hipError_t launch_streamk_tail(const GemmArgs& ga, const typename Epi::Args& ea, hipStream_t s) {
  if constexpr (!Epi::SPLIT && BM == 256) {
    typedef PipeConfig<T, BM, BN, MI, WGM, WGN, A_KS, B_KS, NB, wants_ring_a3<T, Epi>()> Cfg;
    constexpr auto kern = gemm_kernel_pipelined<T, BM, BN, MI, WGM, WGN, A_KS, B_KS, NB, Epi, true>;
    if (hipError_t e = allow_dynamic_lds(lds_kernel_of<kern, Cfg::LDS_BYTES>, s)) return e;
    hipLaunchKernelGGL(kern, dim3(ga.sk_wgs), dim3(Cfg::NW * 64), Cfg::LDS_BYTES, s, ga, ea);
    if (hipError_t e = hipGetLastError()) return e;
    hipLaunchKernelGGL((streamk_fixup_kernel<T, BM, BN, MI, WGM, WGN, NB, Epi>), dim3(ga.sk_tiles * Cfg::TM),
                       dim3(Cfg::NW * 64), 0, s, ga, ea);
    return hipGetLastError();
  } else {
    return hipErrorInvalidValue;  // the host plans stream-K for the large tiles only
  }
}

template <typename T, int BM, int BN, int MI, int WGM, int WGN, bool A_KS, bool B_KS, int NB,
          typename Epi>
__global__ void __launch_bounds__(WGM* WGN * 64)
    gemm_group_kernel_pipelined(GemmGroup<typename Epi::Args> grp) {
  int g = 0;
#pragma unroll
  for (int i = 1; i < GEMM_GROUP_MAX; ++i)
    if (i < grp.count && (int)blockIdx.x >= grp.first[i]) g = i;
  GemmArgs ga = grp.ga[0];
  typename Epi::Args ea = grp.ea[0];
#pragma unroll
  for (int i = 1; i < GEMM_GROUP_MAX; ++i)
    if (g == i) { ga = grp.ga[i]; ea = grp.ea[i]; }
  gemm_pipelined_body<T, BM, BN, MI, WGM, WGN, A_KS, B_KS, NB, Epi>(
      ga, ea, (int)blockIdx.x - grp.first[g], grp.first[g + 1] - grp.first[g]);
}

template <typename T, int BM, int BN, int MI, int WGM, int WGN, bool A_KS, bool B_KS, int NB,
          typename Epi>
hipError_t launch_gemm_pipelined(const GemmArgs& ga, const typename Epi::Args& ea, hipStream_t s) {
  typedef PipeConfig<T, BM, BN, MI, WGM, WGN, A_KS, B_KS, NB, wants_ring_a3<T, Epi>()> Cfg;
  constexpr auto kern = gemm_kernel_pipelined<T, BM, BN, MI, WGM, WGN, A_KS, B_KS, NB, Epi>;
  if (hipError_t e = allow_dynamic_lds(lds_kernel_of<kern, Cfg::LDS_BYTES>, s)) return e;
  const int splits = Epi::SPLIT ? ga.splits : 1;
  const int tiles = ((ga.M + BM - 1) / BM) * ((ga.N + BN - 1) / BN);
  const bool sk = !Epi::SPLIT && ga.sk_tiles > 0;
  dim3 grid(sk ? tiles - ga.sk_tiles : tiles * splits), block(Cfg::NW * 64);
  if (grid.x > 0) {
    hipLaunchKernelGGL(kern, grid, block, Cfg::LDS_BYTES, s, ga, ea);
    if (hipError_t e = hipGetLastError()) return e;
  }
  return sk ? launch_streamk_tail<T, BM, BN, MI, WGM, WGN, A_KS, B_KS, NB, Epi>(ga, ea, s) : hipSuccess;
}

template <typename T, int BM, int BN, int MI, int WGM, int WGN, bool A_KS, bool B_KS, int NB,
          typename Epi>
hipError_t launch_gemm_group_pipelined(GemmGroup<typename Epi::Args>& grp, hipStream_t s) {
  typedef PipeConfig<T, BM, BN, MI, WGM, WGN, A_KS, B_KS, NB, wants_ring_a3<T, Epi>()> Cfg;
  constexpr auto kern = gemm_group_kernel_pipelined<T, BM, BN, MI, WGM, WGN, A_KS, B_KS, NB, Epi>;
  if (hipError_t e = allow_dynamic_lds(lds_kernel_of<kern, Cfg::LDS_BYTES>, s)) return e;
  int total = 0;
  for (int g = 0; g < grp.count; ++g) {
    grp.first[g] = total;
    const int tiles = ((grp.ga[g].M + BM - 1) / BM) * ((grp.ga[g].N + BN - 1) / BN);
    total += tiles - grp.ga[g].sk_tiles;
  }
  for (int g = grp.count; g <= GEMM_GROUP_MAX; ++g) grp.first[g] = total;
  if (total > 0) {  // (stream-K may have taken every tile of a single problem)
    hipLaunchKernelGGL(kern, dim3(total), dim3(Cfg::NW * 64), Cfg::LDS_BYTES, s, grp);
    if (hipError_t e = hipGetLastError()) return e;
  }
  for (int g = 0; g < grp.count; ++g) {
    if (grp.ga[g].sk_tiles <= 0) continue;
    if (hipError_t e = launch_streamk_tail<T, BM, BN, MI, WGM, WGN, A_KS, B_KS, NB, Epi>(grp.ga[g], grp.ea[g], s)) return e;
  }
  return hipSuccess;
}

}  // namespace gmlp
