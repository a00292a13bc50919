// fp32 compatibility path: the same six GEMMs and fused epilogues on v_mfma_f32_32x32x2_f32, for
// callers that keep the module in float32 (as the reference's own tests do).
//
// 128 x (NB * BN) x 32 tiles per workgroup of 4 wavefronts (2 x 2), each wavefront 64 rows x BN/2
// columns per accumulator set (64 accumulator registers either way: BN = 128 for one set, 64 for
// two).  Predicated loads (any M, N, K % 4 == 0), staged through registers: the next reduction
// tile is fetched from global memory while the MFMAs of the current one run, then written to the
// single LDS buffer between two barriers.
#include "launch.hpp"

namespace gmlp {

constexpr int F32_BM = 128, F32_BK = 32;
constexpr int F32_KC_LD = F32_BK + 1;  // [rows][k] tile, odd stride: conflict-free column reads

template <int ROWS>
struct F32Tile {
  static constexpr int KS_LD = ROWS + 4;                 // [k][rows] tile
  static constexpr int VEC = ROWS * F32_BK / 4 / 256;    // float4 loads per thread and tile
  static constexpr int ELEMS_KC = ROWS * F32_KC_LD, ELEMS_KS = F32_BK * KS_LD;

  // Global -> registers, zero outside the matrix.  KC: memory [rows, K]; KS: memory [K, rows].
  template <bool KS>
  static __device__ __forceinline__ void gload(const float* __restrict__ p, int ld, int r0, int k0,
                                               int rtot, int ktot, int tid, f32x4* v) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      int q = tid + i * 256;
      v[i] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (!KS) {
        int row = q / (F32_BK / 4), c = q % (F32_BK / 4);
        int gr = r0 + row, gk = k0 + c * 4;
        if (gr < rtot && gk < ktot) v[i] = *(const f32x4*)(p + (size_t)gr * ld + gk);
      } else {
        int krow = q / (ROWS / 4), c = q % (ROWS / 4);
        int gk = k0 + krow, gr = r0 + c * 4;
        if (gk < ktot && gr < rtot) v[i] = *(const f32x4*)(p + (size_t)gk * ld + gr);
      }
    }
  }
  template <bool KS>
  static __device__ __forceinline__ void commit(float* lds, int tid, const f32x4* v) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      int q = tid + i * 256;
      if (!KS) {
        int row = q / (F32_BK / 4), c = q % (F32_BK / 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) lds[row * F32_KC_LD + c * 4 + e] = v[i][e];
      } else {
        int krow = q / (ROWS / 4), c = q % (ROWS / 4);
        *(f32x4*)(lds + krow * KS_LD + c * 4) = v[i];
      }
    }
  }
  template <bool KS>
  static __device__ __forceinline__ float frag(const float* lds, int row, int k) {
    return KS ? lds[k * KS_LD + row] : lds[row * F32_KC_LD + k];
  }
};

template <bool A_KS, bool B_KS, int NB, typename Epi>
__global__ void __launch_bounds__(256) gemm_f32_kernel(GemmArgs ga, typename Epi::Args ea) {
  constexpr int BN = NB == 2 ? 64 : 128;  // columns per accumulator set
  constexpr int TM = 2, TN = BN / 64;     // 32x32 MFMA tiles per wavefront: 64 rows x BN/2 columns
  typedef F32Tile<F32_BM> AT;
  typedef F32Tile<BN> BT;
  __shared__ __align__(16) float sa[A_KS ? AT::ELEMS_KS : AT::ELEMS_KC];
  __shared__ __align__(16) float sb[NB][B_KS ? BT::ELEMS_KS : BT::ELEMS_KC];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_n = (ga.N + BN - 1) / BN;
  const int m0 = (blockIdx.x / tiles_n) * F32_BM, n0 = (blockIdx.x % tiles_n) * BN;

  f32x16 acc[NB][TM][TN];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[b][i][j][r] = 0.f;

  const int kt_seg = (ga.K + F32_BK - 1) / F32_BK, kt_total = kt_seg * ga.nseg;
  f32x4 ra[AT::VEC], rb[NB][BT::VEC];
  auto fetch = [&](int kt) __attribute__((always_inline)) {
    int seg = kt / kt_seg, k0 = (kt - seg * kt_seg) * F32_BK;
    AT::template gload<A_KS>((const float*)ga.A[seg], ga.lda, m0, k0, ga.M, ga.K, tid, ra);
#pragma unroll
    for (int b = 0; b < NB; ++b)
      BT::template gload<B_KS>((const float*)ga.B[NB == 2 ? b : seg], ga.ldb, n0, k0, ga.N, ga.K, tid, rb[b]);
  };
  auto commit = [&]() __attribute__((always_inline)) {
    AT::template commit<A_KS>(sa, tid, ra);
#pragma unroll
    for (int b = 0; b < NB; ++b) BT::template commit<B_KS>(sb[b], tid, rb[b]);
  };

  fetch(0);
  commit();
  __syncthreads();
  for (int kt = 0; kt < kt_total; ++kt) {
    if (kt + 1 < kt_total) fetch(kt + 1);  // in flight while the MFMAs below run
#pragma unroll
    for (int ks = 0; ks < F32_BK / 2; ++ks) {
      int k = ks * 2 + (lane >> 5);
      float av[TM], bv[NB][TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) av[i] = AT::template frag<A_KS>(sa, wm * 64 + i * 32 + (lane & 31), k);
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          bv[b][j] = BT::template frag<B_KS>(sb[b], wn * (BN / 2) + j * 32 + (lane & 31), k);
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            // operands swapped: a lane ends up with 4 consecutive output columns of one row
            acc[b][i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[b][j], av[i], acc[b][i][j], 0, 0, 0);
    }
    __syncthreads();  // everyone is done reading this tile
    if (kt + 1 < kt_total) {
      commit();
      __syncthreads();
    }
  }

#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + wm * 64 + i * 32 + (lane & 31);
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        int n = n0 + wn * (BN / 2) + j * 32 + 8 * g + 4 * (lane >> 5);
        if (m >= ga.M || n >= ga.N) continue;
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

template <bool A_KS, bool B_KS, int NB, typename Epi>
static hipError_t launch_f32(const GemmArgs& ga, const typename Epi::Args& ea, hipStream_t s) {
  constexpr int BN = NB == 2 ? 64 : 128;
  int tiles = ((ga.M + F32_BM - 1) / F32_BM) * ((ga.N + BN - 1) / BN);
  hipLaunchKernelGGL((gemm_f32_kernel<A_KS, B_KS, NB, Epi>), dim3(tiles), dim3(256), 0, s, ga, ea);
  return hipGetLastError();
}

template <>
hipError_t launch_gateup<float>(int, const GemmArgs& ga, const EpiGateUp<float>::Args& ea, hipStream_t s) {
  return launch_f32<false, false, 2, EpiGateUp<float>>(ga, ea, s);
}
template <>
hipError_t launch_linear<float>(int, const GemmArgs& ga, const EpiStore<float>::Args& ea, hipStream_t s) {
  return launch_f32<false, false, 1, EpiStore<float>>(ga, ea, s);
}
template <>
hipError_t launch_dh<float>(int, const GemmArgs& ga, const EpiDh<float>::Args& ea, hipStream_t s) {
  return launch_f32<false, true, 1, EpiDh<float>>(ga, ea, s);
}
template <>
hipError_t launch_dx<float>(int, const GemmArgs& ga, const EpiStore<float>::Args& ea, hipStream_t s) {
  return launch_f32<false, true, 1, EpiStore<float>>(ga, ea, s);
}
template <>
hipError_t launch_dw<float>(int, const GemmArgs& ga, const EpiStore<float>::Args& ea, hipStream_t s) {
  return launch_f32<true, true, 1, EpiStore<float>>(ga, ea, s);
}

}  // namespace gmlp
