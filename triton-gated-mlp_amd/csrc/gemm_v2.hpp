// Full-tile MFMA GEMM for gfx950 with direct global->LDS loads and a register-pipelined main loop.
//
// Same contract as gemm_kernel (gemm.hpp): C[M,N] = sum_s sum_k A_s[m,k] * B_s[n,k], operands
// reduction-contiguous (KC) or reduction-strided (KS), NB accumulator sets, fused epilogue; but
// restricted to whole BM x BN tiles and K % BK == 0, which lets it
//   * move tiles with buffer_load_dwordx4 ... lds: each lane's 16 bytes land in LDS at
//     (wave base + 16*lane) without passing through VGPRs; bank-conflict-free layouts are obtained
//     by permuting WHICH 16-byte chunk of a row each lane fetches (XOR swizzle on the global side).
//     Addresses are (buffer base) + (wave-uniform SGPR tile offset) + (constant per-lane VGPR
//     offset), so stepping to the next reduction tile costs scalar adds only;
//   * read reduction-strided operands with ds_read_b64_tr_b16, which hands each lane 4 consecutive
//     reduction elements of one output row out of a [k][row] tile;
//   * keep NS-1 reduction tiles in flight in an NS-deep LDS ring, and the MFMA operands of the
//     next 16-wide reduction step in registers while the current step's MFMAs issue, including
//     across the workgroup barrier that retires a ring slot;
//   * run the epilogue on 8 consecutive columns per lane: accumulators are transposed through LDS
//     so that every global access of the epilogue is a 16-byte, row-contiguous one.
#pragma once
#include <type_traits>

#include "gemm.hpp"
#include "lds_dma.hpp"

namespace gmlp {

// One operand tile of ROWS output-dimension rows by BK reduction elements.
//   KC layout: row r at byte r*BK*2; 16-byte chunk c at position c ^ swz(r), swz chosen so that 16
//              consecutive rows x one chunk cover all 64 LDS banks (ds_read_b128 conflict-free).
//   KS layout: reduction row k at byte k*ROWS*2; 16-byte chunk c at position c ^ (4*(k&3)), so
//              the 4 reduction rows x 32 bytes one transpose read gathers sit in distinct banks.
template <typename T, int ROWS, int BK, bool KS, int NWAVES>
struct TileV2 {
  typedef typename Traits<T>::vec8 vec8;
  static_assert(BK == 32 || BK == 64, "BK is 32 or 64");
  static constexpr int BYTES = ROWS * BK * 2;
  static constexpr int INSTR = BYTES / 1024;  // wave-wide 1 KiB load instructions per tile
  static constexpr int PER_WAVE = INSTR / NWAVES;
  static_assert(INSTR % NWAVES == 0 && PER_WAVE >= 1, "tile must split evenly over the wavefronts");
  static constexpr int CPR_KC = BK / 8;        // chunks per row, KC
  static constexpr int RPI_KC = 64 / CPR_KC;   // rows per load instruction, KC

  static __device__ __forceinline__ int swz_kc(int row) {
    return BK == 64 ? ((row >> 1) & 7) : ((row >> 2) & 3);
  }

  // Byte offset, relative to the tile origin (row r0, reduction index k0), of the 16 bytes this
  // lane fetches with the wavefront's i-th load instruction.  Constant for the whole kernel.
  static __device__ __forceinline__ uint32_t lane_offset(int i, int ld, int wave, int lane) {
    int I = wave * PER_WAVE + i;
    if constexpr (!KS) {
      int row = I * RPI_KC + lane / CPR_KC, pos = lane % CPR_KC;
      int c = pos ^ swz_kc(row);
      return (uint32_t)(row * ld + c * 8) * 2u;
    } else {
      constexpr int CPR = ROWS / 8;  // chunks per reduction row
      constexpr int RPI = 64 / CPR;  // reduction rows per instruction
      static_assert(CPR <= 64 && CPR >= 16, "KS tiles have 128..512 rows");
      int krow = I * RPI + lane / CPR, pos = lane % CPR;
      int c = pos ^ (4 * (krow & 3));
      return (uint32_t)(krow * ld + c * 8) * 2u;
    }
  }

  // MFMA fragment (8 reduction elements per lane) for rows row0..row0+31, reduction step ks.
  static __device__ __forceinline__ vec8 frag(const char* lds_tile, int row0, int ks, int lane) {
    if constexpr (!KS) {
      int row = row0 + (lane & 31);
      int c = ks * 2 + (lane >> 5);
      return *(const vec8*)(lds_tile + row * (BK * 2) + ((c ^ swz_kc(row)) << 4));
    } else {
      // 16-lane group g: rows row0 + 16*(g&1) .. +15, reduction kb .. kb+3 (two reads: +0, +4).
      // Lane r of the group addresses reduction row kb + r/4, rows nb + 4*(r%4) .. +3; the
      // transpose read returns to lane i the 4 reduction elements of row nb + i.
      int g = lane >> 4, r = lane & 15;
      int n = row0 + 16 * (g & 1) + 4 * (r & 3);
      int kq = r >> 2;  // == reduction row & 3
      int kb = ks * 16 + 8 * (g >> 1);
      int c = (n >> 3) ^ (4 * kq);
      const char* a0 = lds_tile + (kb + kq) * (ROWS * 2) + (c << 4) + ((n & 7) << 1);
      i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4*)a0);
      i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) i16x4*)(a0 + 4 * (ROWS * 2)));
      i16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(vec8, both);
    }
  }
};

// Raises the dynamic-LDS limit of `kernel` on the current device (needed above 64 KiB).  Called on
// every launch: the attribute is per device, and the call only touches host-side state.
inline hipError_t allow_dynamic_lds(const void* kernel, int bytes) {
  return hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

template <typename T, int BM, int BN, int BK, int NS, int WGM, int WGN, bool A_KS, bool B_KS,
          int NB>
struct ConfigV2 {
  static constexpr int NW = WGM * WGN;
  static constexpr int WTM = BM / WGM, WTN = BN / WGN, TM = WTM / 32, TN = WTN / 32;
  static constexpr int KSTEPS = BK / 16;
  typedef TileV2<T, BM, BK, A_KS, NW> ATile;
  typedef TileV2<T, BN, BK, B_KS, NW> BTile;
  static constexpr int STAGE = ATile::BYTES + NB * BTile::BYTES;
  static constexpr int LOADS = ATile::PER_WAVE + NB * BTile::PER_WAVE;  // per wave per tile
  // epilogue staging: per wavefront NB x 32 rows x (WTN + 4) fp32
  static constexpr int EPI_LD = WTN + 4;
  static constexpr int EPI_WAVE_BYTES = NB * 32 * EPI_LD * 4;
  static constexpr int MAIN_BYTES = NS * STAGE;
  static constexpr int LDS_BYTES = MAIN_BYTES > NW * EPI_WAVE_BYTES ? MAIN_BYTES : NW * EPI_WAVE_BYTES;
  static_assert((NS & (NS - 1)) == 0 && NS >= 2, "ring depth is a power of two");
  static_assert((NS - 1) * LOADS < 64, "vmcnt is a 6-bit counter");
};

#ifndef GMLP_V2_LOAD_STRIDE
#define GMLP_V2_LOAD_STRIDE 2
#endif

// Body of the kernel: workgroup `pid` of the `nwg` that cover one GEMM.
template <typename T, int BM, int BN, int BK, int NS, int WGM, int WGN, bool A_KS, bool B_KS,
          int NB, typename Epi>
__device__ __forceinline__ void gemm_v2_body(const GemmArgs& ga, const typename Epi::Args& ea,
                                             int pid, int nwg) {
  constexpr int LOAD_STRIDE = GMLP_V2_LOAD_STRIDE;
  typedef ConfigV2<T, BM, BN, BK, NS, WGM, WGN, A_KS, B_KS, NB> Cfg;
  typedef typename Cfg::ATile ATile;
  typedef typename Cfg::BTile BTile;
  typedef typename Traits<T>::vec8 vec8;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, WTM = Cfg::WTM, WTN = Cfg::WTN;
  constexpr int KSTEPS = Cfg::KSTEPS, STAGE = Cfg::STAGE, L = Cfg::LOADS;

  extern __shared__ __align__(1024) char smem_raw[];
  char* smem = smem_raw;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;

  const int tiles_m = ga.M / BM, tiles_n = ga.N / BN;
  int tm_i, tn_i;
  map_tile(pid, nwg, tiles_m, tiles_n, ga.group_m, tm_i, tn_i);
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

  const int kt_seg = ga.K / BK;
  const int kt_total = kt_seg * ga.nseg;

  // Per-lane load offsets (constant), per-operand tile origins and per-tile strides (uniform).
  // Buffer addressing uses 32-bit byte offsets from each operand's base; the host checks sizes.
  uint32_t aoff[ATile::PER_WAVE], boff[BTile::PER_WAVE];
#pragma unroll
  for (int i = 0; i < ATile::PER_WAVE; ++i) aoff[i] = ATile::lane_offset(i, ga.lda, wave, lane);
#pragma unroll
  for (int i = 0; i < BTile::PER_WAVE; ++i) boff[i] = BTile::lane_offset(i, ga.ldb, wave, lane);
  const uint32_t a_step = A_KS ? (uint32_t)BK * ga.lda * 2 : (uint32_t)BK * 2;
  const uint32_t b_step = B_KS ? (uint32_t)BK * ga.ldb * 2 : (uint32_t)BK * 2;
  const uint32_t a_org = A_KS ? (uint32_t)m0 * 2 : (uint32_t)m0 * ga.lda * 2;
  const uint32_t b_org = B_KS ? (uint32_t)n0 * 2 : (uint32_t)n0 * ga.ldb * 2;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void*)smem;
  const buffer_rsrc ra[2] = {make_rsrc(ga.A[0]), make_rsrc(ga.A[1])};
  const buffer_rsrc rb[2] = {make_rsrc(ga.B[0]), make_rsrc(ga.B[1])};

  // Global->LDS load number x (0 .. L-1) of this wavefront for reduction tile kt.
  // Tiles past the end are replaced by the last tile: the ring then always holds NS-1 tiles in
  // flight, the redundant copies land in slots nobody reads again.
  auto issue_one = [&](int kt_req, int x) __attribute__((always_inline)) {
    int kt = kt_req < kt_total ? kt_req : kt_total - 1;
    int seg = kt >= kt_seg ? 1 : 0;
    int kk = kt - seg * kt_seg;
    uint32_t s = lds_base + (kt_req & (NS - 1)) * STAGE;
    if (x < ATile::PER_WAVE) {
      load16_to_lds(seg ? ra[1] : ra[0], aoff[x], a_org + kk * a_step,
                    s + (wave * ATile::PER_WAVE + x) * 1024);
    } else {
      int y = x - ATile::PER_WAVE, bsel = y / BTile::PER_WAVE, i = y % BTile::PER_WAVE;
      load16_to_lds(NB == 2 ? rb[bsel] : (seg ? rb[1] : rb[0]), boff[i], b_org + kk * b_step,
                    s + ATile::BYTES + bsel * BTile::BYTES + (wave * BTile::PER_WAVE + i) * 1024);
    }
  };
  auto issue_tile = [&](int kt) __attribute__((always_inline)) {
#pragma unroll
    for (int x = 0; x < L; ++x) issue_one(kt, x);
  };

  vec8 af[2][TM], bf[2][NB][TN];
  // Fragment number f (0 .. NFRAG-1) of reduction step ks of tile kt into register buffer `buf`.
  constexpr int NFRAG = TM + NB * TN;
  auto load_frag = [&](int buf, int kt, int ks, int f) __attribute__((always_inline)) {
    const char* s = smem + (kt & (NS - 1)) * STAGE;
    if (f < TM) {
      af[buf][f] = ATile::frag(s, wm * WTM + f * 32, ks, lane);
    } else {
      int bsel = (f - TM) / TN, j = (f - TM) % TN;
      bf[buf][bsel][j] = BTile::frag(s + ATile::BYTES + bsel * BTile::BYTES, wn * WTN + j * 32, ks, lane);
    }
  };

  // One 16-wide reduction step.  The wavefront is alone on its SIMD: whatever issues between two
  // MFMAs is hidden behind the matrix pipe, whatever issues in a block ahead of them drains it.
  // So the step is laid out as NMFMA slots of {one MFMA; one operand read for the next step, or a
  // share of the global->LDS loads of a tile}, and the scheduler is told to keep the slots.
  constexpr int NMFMA = NB * TM * TN;
  static_assert(NFRAG <= NMFMA, "operand reads must fit in the MFMA slots");
  // The refill of a ring slot starts in the step that retires it and is paced at one load per
  // LOAD_STRIDE slots (the vector-memory front end takes a 1 KiB wavefront load every ~16 cycles
  // for the whole CU; issuing faster blocks the wavefront, and the MFMAs queued behind it).
  // g0 = slot number of this step's first MFMA, counted from the retiring step's first slot.
  static_assert(L * LOAD_STRIDE <= KSTEPS * NMFMA, "a tile's loads must fit in one tile of slots");
  auto step = [&](int buf, auto frags_c, int fkt, int fks, auto loads_c, int g0, int lkt) __attribute__((always_inline)) {
    constexpr bool FRAGS = decltype(frags_c)::value, LOADS = decltype(loads_c)::value;
#pragma unroll
    for (int q = 0; q < NMFMA; ++q) {
      const int b = q / (TN * TM), j = (q / TM) % TN, i = q % TM;
      acc[b][i][j] = Traits<T>::mfma(bf[buf][b][j], af[buf][i], acc[b][i][j]);
      if (FRAGS && q < NFRAG) load_frag(buf ^ 1, fkt, fks, q);
      const int g = g0 + q;
      if (LOADS && g % LOAD_STRIDE == 0 && g / LOAD_STRIDE < L) issue_one(lkt, g / LOAD_STRIDE);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // One reduction tile kt (ring slot kt % NS).  NEXT: tile kt+1 exists; then this tile's last step
  // retires the slot: wait until tile kt+1 has landed (the NS-2 younger tiles stay in flight),
  // barrier, start refilling the slot with tile kt+NS and read tile kt+1's first operands.  The
  // earlier steps carry the rest of the refill that tile kt-1's retirement started.
  auto tile_body = [&](int kt, auto next_c) __attribute__((always_inline)) {
    constexpr bool NEXT = decltype(next_c)::value;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const int buf = (KSTEPS & 1) ? ((kt + ks) & 1) : (ks & 1);
      if (ks < KSTEPS - 1) {
        step(buf, std::true_type{}, kt, ks + 1, std::integral_constant<bool, NEXT>{}, (ks + 1) * NMFMA,
             kt - 1 + NS);
      } else if (NEXT) {
        wait_vmem<(NS - 2) * L>();
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        step(buf, std::true_type{}, kt + 1, 0, std::true_type{}, 0, kt + NS);
      } else {
        step(buf, std::false_type{}, 0, 0, std::false_type{}, 0, 0);
      }
    }
  };

  // Prologue: tiles 0 .. NS-2 entirely, and of tile NS-1 the loads a retiring step would issue
  // (tile 0's first steps issue the rest); wait for tile 0.
  constexpr int L_HEAD = (NMFMA + LOAD_STRIDE - 1) / LOAD_STRIDE < L ? (NMFMA + LOAD_STRIDE - 1) / LOAD_STRIDE : L;
#pragma unroll
  for (int p = 0; p < NS - 1; ++p) issue_tile(p);
#pragma unroll
  for (int x = 0; x < L_HEAD; ++x) issue_one(NS - 1, x);
  wait_vmem<(NS - 2) * L + L_HEAD>();
  __syncthreads();
#pragma unroll
  for (int f = 0; f < NFRAG; ++f) load_frag(0, 0, 0, f);
  __builtin_amdgcn_sched_barrier(0);

  int kt = 0;
  for (; kt + 1 < kt_total; ++kt) tile_body(kt, std::true_type{});
  tile_body(kt, std::false_type{});
  wait_vmem<0>();  // redundant tail loads must not land in the epilogue's staging area

  // ---- epilogue: transpose 32-row slabs of the accumulators through LDS (fp32), then each lane
  // owns 8 consecutive columns of one row.
  __syncthreads();  // all wavefronts are done reading operand tiles
  constexpr int ELD = Cfg::EPI_LD;
  float* stg = (float*)(smem + wave * Cfg::EPI_WAVE_BYTES);
  const int mrow = lane & 31, nsub = 4 * (lane >> 5);
  constexpr int ITEMS = 32 * WTN / 8;  // (row, 8-column group) items per slab
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          f32x4 v;
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] = acc[b][i][j][4 * g + r];
          *(f32x4*)(stg + (b * 32 + mrow) * ELD + j * 32 + 8 * g + nsub) = v;
        }
    // Same-wavefront LDS writes and reads are ordered; no barrier needed for a private slab.
#pragma unroll
    for (int it = 0; it < ITEMS / 64; ++it) {
      int item = it * 64 + lane;
      int row = item / (WTN / 8), cg = item % (WTN / 8);
      alignas(16) float v0[8], v1[8];
      const float* p0 = stg + row * ELD + cg * 8;
      *(f32x4*)v0 = *(const f32x4*)p0;
      *(f32x4*)(v0 + 4) = *(const f32x4*)(p0 + 4);
      if (NB == 2) {
        const float* p1 = p0 + 32 * ELD;
        *(f32x4*)v1 = *(const f32x4*)p1;
        *(f32x4*)(v1 + 4) = *(const f32x4*)(p1 + 4);
      }
      int m = m0 + wm * WTM + i * 32 + row;
      int n = n0 + wn * WTN + cg * 8;
      Epi::template apply<8>(ea, m, n, v0, v1);
    }
  }
}

template <typename T, int BM, int BN, int BK, int NS, int WGM, int WGN, bool A_KS, bool B_KS,
          int NB, typename Epi>
__global__ void __launch_bounds__(WGM* WGN * 64)
    gemm_kernel_v2(GemmArgs ga, typename Epi::Args ea) {
  gemm_v2_body<T, BM, BN, BK, NS, WGM, WGN, A_KS, B_KS, NB, Epi>(ga, ea, blockIdx.x, gridDim.x);
}

// Up to GEMM_GROUP_MAX independent GEMMs of one kind in a single launch: workgroups
// [first[g], first[g+1]) belong to problem g.  One launch instead of several removes the partially
// filled last round of workgroups of each problem.
constexpr int GEMM_GROUP_MAX = 3;
template <typename EpiArgs>
struct GemmGroup {
  GemmArgs ga[GEMM_GROUP_MAX];
  EpiArgs ea[GEMM_GROUP_MAX];
  int first[GEMM_GROUP_MAX + 1];
  int count;
};

template <typename T, int BM, int BN, int BK, int NS, int WGM, int WGN, bool A_KS, bool B_KS,
          int NB, typename Epi>
__global__ void __launch_bounds__(WGM* WGN * 64)
    gemm_group_kernel_v2(GemmGroup<typename Epi::Args> grp) {
  int g = 0;
#pragma unroll
  for (int i = 1; i < GEMM_GROUP_MAX; ++i)
    if (i < grp.count && (int)blockIdx.x >= grp.first[i]) g = i;
  // copy the selected problem to registers with uniform (scalar) selects
  GemmArgs ga = grp.ga[0];
  typename Epi::Args ea = grp.ea[0];
#pragma unroll
  for (int i = 1; i < GEMM_GROUP_MAX; ++i)
    if (g == i) { ga = grp.ga[i]; ea = grp.ea[i]; }
  gemm_v2_body<T, BM, BN, BK, NS, WGM, WGN, A_KS, B_KS, NB, Epi>(
      ga, ea, (int)blockIdx.x - grp.first[g], grp.first[g + 1] - grp.first[g]);
}

template <typename T, int BM, int BN, int BK, int NS, int WGM, int WGN, bool A_KS, bool B_KS,
          int NB, typename Epi>
hipError_t launch_gemm_group_v2(GemmGroup<typename Epi::Args>& grp, hipStream_t s) {
  typedef ConfigV2<T, BM, BN, BK, NS, WGM, WGN, A_KS, B_KS, NB> Cfg;
  auto kern = gemm_group_kernel_v2<T, BM, BN, BK, NS, WGM, WGN, A_KS, B_KS, NB, Epi>;
  if (hipError_t e = allow_dynamic_lds((const void*)kern, Cfg::LDS_BYTES)) return e;
  int total = 0;
  for (int g = 0; g < grp.count; ++g) {
    grp.first[g] = total;
    total += (grp.ga[g].M / BM) * (grp.ga[g].N / BN);
  }
  for (int g = grp.count; g <= GEMM_GROUP_MAX; ++g) grp.first[g] = total;
  hipLaunchKernelGGL(kern, dim3(total), dim3(Cfg::NW * 64), Cfg::LDS_BYTES, s, grp);
  return hipGetLastError();
}

template <typename T, int BM, int BN, int BK, int NS, int WGM, int WGN, bool A_KS, bool B_KS,
          int NB, typename Epi>
hipError_t launch_gemm_v2(const GemmArgs& ga, const typename Epi::Args& ea, hipStream_t s) {
  typedef ConfigV2<T, BM, BN, BK, NS, WGM, WGN, A_KS, B_KS, NB> Cfg;
  auto kern = gemm_kernel_v2<T, BM, BN, BK, NS, WGM, WGN, A_KS, B_KS, NB, Epi>;
  if (hipError_t e = allow_dynamic_lds((const void*)kern, Cfg::LDS_BYTES)) return e;
  dim3 grid((ga.M / BM) * (ga.N / BN)), block(Cfg::NW * 64);
  hipLaunchKernelGGL(kern, grid, block, Cfg::LDS_BYTES, s, ga, ea);
  return hipGetLastError();
}

}  // namespace gmlp
