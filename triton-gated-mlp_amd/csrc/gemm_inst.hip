// One translation unit per (dtype, GEMM kind): compiled with -DGMLP_DT=<0|1> -DGMLP_KIND=<0..4>
// so the kernels build in parallel.  Each unit instantiates every tile class.
#include "gemm_pipelined.hpp"
#include "launch.hpp"

namespace gmlp {

#if GMLP_DT == 0
typedef f16 DT;
#else
typedef bf16 DT;
#endif

#define GMLP_LARGE(AKS, BKS, NB, EPI, BN_L) \
  launch_gemm_pipelined<DT, 256, BN_L, 16, 2, 2, AKS, BKS, NB, EPI<DT>>
#define GMLP_MEDIUM(AKS, BKS, NB, EPI, BN_M) \
  launch_gemm_pipelined<DT, 128, BN_M, 16, 2, 2, AKS, BKS, NB, EPI<DT>>
#define GMLP_LARGE_GROUP \
  launch_gemm_group_pipelined<DT, 256, 256, 16, 2, 2, true, true, 1, EpiStore<DT>>
#define GMLP_MEDIUM_GROUP \
  launch_gemm_group_pipelined<DT, 128, 128, 16, 2, 2, true, true, 1, EpiStore<DT>>

#define GMLP_DISPATCH(AKS, BKS, NB, EPI, BN_L, BN_M)                                             \
  if (tile_class == TILE_LARGE) return GMLP_LARGE(AKS, BKS, NB, EPI, BN_L)(ga, ea, s);           \
  if (tile_class == TILE_MEDIUM_FULL) return GMLP_MEDIUM(AKS, BKS, NB, EPI, BN_M)(ga, ea, s);    \
  return launch_gemm<DT, 128, BN_M, 64, 2, 2, AKS, BKS, NB, true, EPI<DT>>(ga, ea, s);

#if GMLP_KIND == 0
template <>
hipError_t launch_gateup<DT>(int tile_class, const GemmArgs& ga, const EpiGateUp<DT>::Args& ea,
                             hipStream_t s) {
  // the usual case (SiLU, no keep-mask output) has kernels of its own, see EpiGateUpPacked
  if (EpiGateUpPacked<DT>::packed_eligible(ea)) {
    if (tile_class == TILE_LARGE) return GMLP_LARGE(false, false, 2, EpiGateUpPacked, 128)(ga, ea, s);
    if (tile_class == TILE_MEDIUM_FULL) return GMLP_MEDIUM(false, false, 2, EpiGateUpPacked, 64)(ga, ea, s);
  }
  GMLP_DISPATCH(false, false, 2, EpiGateUp, 128, 64)
}
template <>
hipError_t launch_gateup_split<DT>(const GemmArgs& ga, const EpiPartial<DT>::Args& ea, hipStream_t s) {
  return launch_gemm_pipelined<DT, 128, 64, 16, 2, 2, false, false, 2, EpiPartial<DT>>(ga, ea, s);
}
#elif GMLP_KIND == 1
template <>
hipError_t launch_linear<DT>(int tile_class, const GemmArgs& ga, const EpiStore<DT>::Args& ea,
                             hipStream_t s) {
  GMLP_DISPATCH(false, false, 1, EpiStore, 256, 128)
}
template <>
hipError_t launch_linear_split<DT>(const GemmArgs& ga, const EpiPartial<DT>::Args& ea, hipStream_t s) {
  return launch_gemm_pipelined<DT, 128, 128, 16, 2, 2, false, false, 1, EpiPartial<DT>>(ga, ea, s);
}
#elif GMLP_KIND == 2
template <>
hipError_t launch_dh<DT>(int tile_class, const GemmArgs& ga, const EpiDh<DT>::Args& ea,
                         hipStream_t s) {
  GMLP_DISPATCH(false, true, 1, EpiDh, 256, 128)
}
#elif GMLP_KIND == 3
template <>
hipError_t launch_dx<DT>(int tile_class, const GemmArgs& ga, const EpiStore<DT>::Args& ea,
                         hipStream_t s) {
  GMLP_DISPATCH(false, true, 1, EpiStore, 256, 128)
}
template <>
hipError_t launch_dx_split<DT>(const GemmArgs& ga, const EpiPartial<DT>::Args& ea, hipStream_t s) {
  return launch_gemm_pipelined<DT, 128, 128, 16, 2, 2, false, true, 1, EpiPartial<DT>>(ga, ea, s);
}
#elif GMLP_KIND == 4
template <>
hipError_t launch_dw<DT>(int tile_class, const GemmArgs& ga, const EpiStore<DT>::Args& ea,
                         hipStream_t s) {
  GMLP_DISPATCH(true, true, 1, EpiStore, 256, 128)
}
template <>
hipError_t launch_dw_group<DT>(int tile_class, GemmGroup<EpiStore<DT>::Args>& grp, hipStream_t s) {
  return tile_class == TILE_LARGE ? GMLP_LARGE_GROUP(grp, s) : GMLP_MEDIUM_GROUP(grp, s);
}
#endif

}  // namespace gmlp
