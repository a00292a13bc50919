// Host-side launch interface between the C ABI (api.hip) and the kernel translation units.
#pragma once
#include "gemm.hpp"
#include "gemm_tiles.hpp"

namespace gmlp {

// Tile classes (all four wavefronts per workgroup, 64-wide reduction tiles).
//   LARGE        256x256 output tiles, wavefronts of 128x128, pipelined kernel, whole tiles only
//   MEDIUM_FULL  128x128 output tiles, wavefronts of 64x64, pipelined kernel, whole tiles only;
//                two workgroups per CU, for problems with too few 256x256 tiles to fill the chip
//   MEDIUM       128x128, predicated register-staged kernel: any M, N % 8, K % 8
enum TileClass { TILE_LARGE = 0, TILE_MEDIUM = 1, TILE_MEDIUM_FULL = 2 };

// kinds of GEMM the gated MLP needs; each is instantiated per dtype and tile class.
template <typename T>
hipError_t launch_gateup(int tile_class, const GemmArgs& ga, const typename EpiGateUp<T>::Args& ea,
                         hipStream_t s);  // A KC, B KC, two accumulator sets
template <typename T>
hipError_t launch_linear(int tile_class, const GemmArgs& ga, const typename EpiStore<T>::Args& ea,
                         hipStream_t s);  // A KC, B KC
template <typename T>
hipError_t launch_dh(int tile_class, const GemmArgs& ga, const typename EpiDh<T>::Args& ea,
                     hipStream_t s);  // A KC, B KS
template <typename T>
hipError_t launch_dx(int tile_class, const GemmArgs& ga, const typename EpiStore<T>::Args& ea,
                     hipStream_t s);  // A KC, B KS, two reduction segments
template <typename T>
hipError_t launch_dw(int tile_class, const GemmArgs& ga, const typename EpiStore<T>::Args& ea,
                     hipStream_t s);  // A KS, B KS

// Several weight-gradient GEMMs of one pipelined tile class (LARGE or MEDIUM_FULL) as one grid.
template <typename T>
hipError_t launch_dw_group(int tile_class, GemmGroup<typename EpiStore<T>::Args>& grp, hipStream_t s);

// Generic launcher used by the instantiation units.
template <typename T, int BM, int BN, int BK, int WGM, int WGN, bool A_KS, bool B_KS, int NB,
          bool EDGE, typename Epi>
hipError_t launch_gemm(const GemmArgs& ga, const typename Epi::Args& ea, hipStream_t s) {
  typedef GemmConfig<T, BM, BN, BK, WGM, WGN, A_KS, B_KS, NB, EDGE> Cfg;
  constexpr auto kern = gemm_kernel<T, BM, BN, BK, WGM, WGN, A_KS, B_KS, NB, EDGE, Epi>;
  if (hipError_t e = allow_dynamic_lds(lds_kernel_of<kern, Cfg::LDS_BYTES>, s)) return e;
  int tiles_m = (ga.M + BM - 1) / BM, tiles_n = (ga.N + BN - 1) / BN;
  dim3 grid(tiles_m * tiles_n), block(Cfg::NT);
  hipLaunchKernelGGL(kern, grid, block, Cfg::LDS_BYTES, s, ga, ea);
  return hipGetLastError();
}

// Split-reduction variants (128x128 tiles): partial sums to a fp32 workspace, see splitk_reduce.
template <typename T>
hipError_t launch_linear_split(const GemmArgs& ga, const typename EpiPartial<T>::Args& ea, hipStream_t s);
template <typename T>
hipError_t launch_dx_split(const GemmArgs& ga, const typename EpiPartial<T>::Args& ea, hipStream_t s);
template <typename T>
hipError_t launch_gateup_split(const GemmArgs& ga, const typename EpiPartial<T>::Args& ea, hipStream_t s);

// decode.hip
template <typename T>
hipError_t launch_decode(const T* x, const T* wg, const T* wu, const T* wd, const T* bg,
                         const T* bu, const T* bd, T* h, T* y, int M, int K, int N, int act,
                         hipStream_t s);

// decode_stream.hip: LDS-ring streaming variant for K % 256 == 0 and N % 256 == 0
bool decode_stream_supported(int M, int K, int N);
template <typename T>
hipError_t launch_decode_stream(const T* x, const T* wg, const T* wu, const T* wd, const T* bg,
                                const T* bu, const T* bd, T* h, T* y, int M, int K, int N,
                                int act, hipStream_t s);

// aux.hip
template <typename T>
hipError_t launch_gating_bwd(const T* dh, const T* g, const T* u, T* dg, T* du, int64_t M, int64_t N,
                             int act, const DropoutParams& d, hipStream_t s);
// Second stage of a split reduction: Epi (EpiStore or EpiGateUp) applied to
// sum_s ws[s*split_stride (+ acc_stride) + m*N + n].
template <typename T, typename Epi>
hipError_t launch_splitk_reduce(const float* ws, int splits, size_t split_stride, size_t acc_stride,
                                const typename Epi::Args& ea, int64_t M, int64_t N, hipStream_t s);
constexpr int COLSUM_GROUP_MAX = 3;
template <typename T>
struct ColsumGroup {
  const T* a[COLSUM_GROUP_MAX];   // [M, C[i]]
  T* out[COLSUM_GROUP_MAX];       // [C[i]]
  float* ws[COLSUM_GROUP_MAX];    // colsum_workspace_bytes(M, C[i]) bytes each
  int64_t C[COLSUM_GROUP_MAX];
};
template <typename T>
hipError_t launch_colsum_group(const ColsumGroup<T>& g, int count, int64_t M, hipStream_t s);
size_t colsum_workspace_bytes(int64_t M, int64_t C);
// Column sums of one array with the first stage's partial sums in a static device array of the
// library (no workspace argument, no allocation); C <= COLSUM_STATIC_MAX_C.
constexpr int64_t COLSUM_STATIC_MAX_C = 32768;
// Address of that array on the current device; the first call on a device looks the symbol up
// and refuses to while `s` is capturing.
hipError_t colsum_static_scratch(float** out, hipStream_t s);
template <typename T>
hipError_t launch_colsum_static(const T* a, T* out, int64_t M, int64_t C, hipStream_t s);
hipError_t launch_dropout_mask(uint8_t* mask, int64_t M, int64_t N, const DropoutParams& d,
                               hipStream_t s);

}  // namespace gmlp
