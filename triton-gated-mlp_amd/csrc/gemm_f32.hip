// fp32 compatibility path: the same six GEMMs and fused epilogues on v_mfma_f32_32x32x2_f32, for
// callers that keep the module in float32 (as the reference's own tests do).  Small predicated
// 64x64x32 tiles, register-staged loads; built for exactness of the interface, not for speed.
#include "launch.hpp"

namespace gmlp {

constexpr int F32_BM = 64, F32_BN = 64, F32_BK = 32;
constexpr int F32_KC_LD = F32_BK + 1;   // [rows][k] tile, odd stride: conflict-free column reads
constexpr int F32_KS_LD = 64 + 32;      // [k][rows] tile

// Loads one operand tile (64 output-dim rows x 32 reduction elements) into LDS, zero-filling
// outside the matrix.  KC: memory [rows, K]; KS: memory [K, rows].  16-byte (4 float) chunks.
template <bool KS>
__device__ __forceinline__ void f32_load_tile(const float* __restrict__ p, int ld, int r0, int k0,
                                              int rtot, int ktot, float* lds, int tid) {
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    int q = tid + i * 256;
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (!KS) {
      int row = q / (F32_BK / 4), c = q % (F32_BK / 4);
      int gr = r0 + row, gk = k0 + c * 4;
      if (gr < rtot && gk < ktot) v = *(const f32x4*)(p + (size_t)gr * ld + gk);
#pragma unroll
      for (int e = 0; e < 4; ++e) lds[row * F32_KC_LD + c * 4 + e] = v[e];
    } else {
      int krow = q / (64 / 4), c = q % (64 / 4);
      int gk = k0 + krow, gr = r0 + c * 4;
      if (gk < ktot && gr < rtot) v = *(const f32x4*)(p + (size_t)gk * ld + gr);
      *(f32x4*)(lds + krow * F32_KS_LD + c * 4) = v;
    }
  }
}

template <bool KS>
__device__ __forceinline__ float f32_frag(const float* lds, int row, int k) {
  return KS ? lds[k * F32_KS_LD + row] : lds[row * F32_KC_LD + k];
}

template <bool A_KS, bool B_KS, int NB, typename Epi>
__global__ void __launch_bounds__(256) gemm_f32_kernel(GemmArgs ga, typename Epi::Args ea) {
  constexpr int A_ELEMS = A_KS ? F32_BK * F32_KS_LD : F32_BM * F32_KC_LD;
  constexpr int B_ELEMS = B_KS ? F32_BK * F32_KS_LD : F32_BN * F32_KC_LD;
  __shared__ __align__(16) float sa[A_ELEMS];
  __shared__ __align__(16) float sb[NB][B_ELEMS];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_n = (ga.N + F32_BN - 1) / F32_BN;
  const int m0 = (blockIdx.x / tiles_n) * F32_BM, n0 = (blockIdx.x % tiles_n) * F32_BN;

  f32x16 acc[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[b][r] = 0.f;

  const int kt_seg = (ga.K + F32_BK - 1) / F32_BK;
  for (int kt = 0; kt < kt_seg * ga.nseg; ++kt) {
    int seg = kt / kt_seg, k0 = (kt - seg * kt_seg) * F32_BK;
    f32_load_tile<A_KS>((const float*)ga.A[seg], ga.lda, m0, k0, ga.M, ga.K, sa, tid);
#pragma unroll
    for (int b = 0; b < NB; ++b)
      f32_load_tile<B_KS>((const float*)ga.B[NB == 2 ? b : seg], ga.ldb, n0, k0, ga.N, ga.K, sb[b], tid);
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < F32_BK / 2; ++ks) {
      int k = ks * 2 + (lane >> 5);
      float av = f32_frag<A_KS>(sa, wm * 32 + (lane & 31), k);
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        float bv = f32_frag<B_KS>(sb[b], wn * 32 + (lane & 31), k);
        // operands swapped: a lane ends up with 4 consecutive output columns of one row
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv, av, acc[b], 0, 0, 0);
      }
    }
    __syncthreads();
  }

  const int m = m0 + wm * 32 + (lane & 31);
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    int n = n0 + wn * 32 + 8 * g + 4 * (lane >> 5);
    if (m >= ga.M || n >= ga.N) continue;
    float v0[4], v1[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      v0[r] = acc[0][4 * g + r];
      v1[r] = acc[NB - 1][4 * g + r];
    }
    Epi::template apply<4>(ea, m, n, v0, v1);
  }
}

template <bool A_KS, bool B_KS, int NB, typename Epi>
static hipError_t launch_f32(const GemmArgs& ga, const typename Epi::Args& ea, hipStream_t s) {
  int tiles = ((ga.M + F32_BM - 1) / F32_BM) * ((ga.N + F32_BN - 1) / F32_BN);
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
