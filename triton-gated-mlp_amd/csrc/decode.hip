// Skinny-M (M <= 16) forward of the whole gated MLP: the three weight matrices are streamed from
// HBM exactly once; the token block x (and the hidden block H) is small enough to stay in L2.
//
// Phase 1  H[m,n] = act(x·W_gateᵀ + b_g) * (x·W_upᵀ + b_u)
//   one wavefront per block of 16 hidden columns n; v_mfma_f32_16x16x32 with the 16 weight rows as
//   the instruction's A operand and the 16 token rows as its B operand, so a lane accumulates
//   4 consecutive n of one token row.  Each lane loads its weight fragments straight from global
//   memory with 16-byte non-temporal loads (row n = lane%16, reduction chunk = lane/16), kept
//   DEPTH iterations ahead of the MFMAs in registers.
// Phase 2  Y[m,k] = H·W_downᵀ + b_d
//   one workgroup of SPLIT wavefronts per block of 16 output columns; each wavefront reduces a
//   1/SPLIT share of N, partial sums are combined through LDS in a fixed order (deterministic).
#include "launch.hpp"

namespace gmlp {

typedef float f32x4v __attribute__((ext_vector_type(4)));

template <typename T>
struct Mfma16;
template <>
struct Mfma16<f16> {
  static __device__ __forceinline__ f32x4v run(f16x8 a, f16x8 b, f32x4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mfma16<bf16> {
  static __device__ __forceinline__ f32x4v run(bf16x8 a, bf16x8 b, f32x4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};

template <typename V>
__device__ __forceinline__ V stream_load(const void* p) {
  return __builtin_nontemporal_load((const V*)p);
}

constexpr int DEC_UNROLL = 8;  // MFMA steps (32 reduction elements each) per pipeline stage

template <typename T>
__global__ void __launch_bounds__(256)
    decode_gateup_kernel(const T* __restrict__ x, const T* __restrict__ wg,
                         const T* __restrict__ wu, const T* __restrict__ bg,
                         const T* __restrict__ bu, T* __restrict__ h, int M, int K, int N,
                         int act) {
  typedef typename Traits<T>::vec8 vec8;
  constexpr int U = DEC_UNROLL;
  const int lane = threadIdx.x & 63;
  const int nb = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (nb * 16 >= N) return;  // whole wavefront exits together
  const int r16 = lane & 15, kg = lane >> 4;
  const T* pg = wg + (size_t)(nb * 16 + r16) * K + kg * 8;
  const T* pu = wu + (size_t)(nb * 16 + r16) * K + kg * 8;
  const bool mok = r16 < M;
  const T* px = x + (size_t)(mok ? r16 : 0) * K + kg * 8;

  f32x4v accg = {0.f, 0.f, 0.f, 0.f}, accu = {0.f, 0.f, 0.f, 0.f};
  vec8 fg[2][U], fu[2][U], fx[2][U];
  vec8 zero;
#pragma unroll
  for (int j = 0; j < 8; ++j) zero[j] = (T)0.f;

  const int steps = K / (32 * U);
  if (steps > 0) {
#pragma unroll
    for (int j = 0; j < U; ++j) {
      fg[0][j] = stream_load<vec8>(pg + 32 * j);
      fu[0][j] = stream_load<vec8>(pu + 32 * j);
      fx[0][j] = mok ? *(const vec8*)(px + 32 * j) : zero;
    }
  }
  for (int it = 0; it < steps; it += 2) {
    // stage 1 loads (for it+1), compute stage 0; then the reverse.  Two copies keep the
    // register indices static.
    if (it + 1 < steps) {
      int k = (it + 1) * 32 * U;
#pragma unroll
      for (int j = 0; j < U; ++j) {
        fg[1][j] = stream_load<vec8>(pg + k + 32 * j);
        fu[1][j] = stream_load<vec8>(pu + k + 32 * j);
        fx[1][j] = mok ? *(const vec8*)(px + k + 32 * j) : zero;
      }
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
      accg = Mfma16<T>::run(fg[0][j], fx[0][j], accg);
      accu = Mfma16<T>::run(fu[0][j], fx[0][j], accu);
    }
    if (it + 1 >= steps) break;
    if (it + 2 < steps) {
      int k = (it + 2) * 32 * U;
#pragma unroll
      for (int j = 0; j < U; ++j) {
        fg[0][j] = stream_load<vec8>(pg + k + 32 * j);
        fu[0][j] = stream_load<vec8>(pu + k + 32 * j);
        fx[0][j] = mok ? *(const vec8*)(px + k + 32 * j) : zero;
      }
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
      accg = Mfma16<T>::run(fg[1][j], fx[1][j], accg);
      accu = Mfma16<T>::run(fu[1][j], fx[1][j], accu);
    }
  }
  for (int k = steps * 32 * U; k < K; k += 32) {  // remainder when K/32 is not a multiple of U
    vec8 a = stream_load<vec8>(pg + k), b = stream_load<vec8>(pu + k);
    vec8 c = mok ? *(const vec8*)(px + k) : zero;
    accg = Mfma16<T>::run(a, c, accg);
    accu = Mfma16<T>::run(b, c, accu);
  }

  // lane holds token row m = lane%16, hidden columns n = nb*16 + 4*(lane/16) + r
  if (mok) {
    int n = nb * 16 + 4 * kg;
    float g[4], u[4], hv[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) { g[r] = accg[r]; u[r] = accu[r]; }
    if (bg) add_w<T, 4>(bg + n, g);
    if (bu) add_w<T, 4>(bu + n, u);
    act_fwd_w<4>(act, g, hv);
#pragma unroll
    for (int r = 0; r < 4; ++r) hv[r] *= u[r];
    store_w<T, 4>(h + (size_t)r16 * N + n, hv);
  }
}

constexpr int DEC_SPLIT = 8;  // wavefronts per workgroup in phase 2 = reduction splits

template <typename T>
__global__ void __launch_bounds__(DEC_SPLIT * 64)
    decode_down_kernel(const T* __restrict__ hmat, const T* __restrict__ wd,
                       const T* __restrict__ bd, T* __restrict__ y, int M, int K, int N) {
  typedef typename Traits<T>::vec8 vec8;
  constexpr int U = DEC_UNROLL;
  __shared__ float part[DEC_SPLIT][64][4];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int cb = blockIdx.x;  // block of 16 output columns (rows of W_down)
  const int r16 = lane & 15, kg = lane >> 4;
  const int nsplit = N / DEC_SPLIT;
  const T* pw = wd + (size_t)(cb * 16 + r16) * N + (size_t)w * nsplit + kg * 8;
  const bool mok = r16 < M;
  const T* ph = hmat + (size_t)(mok ? r16 : 0) * N + (size_t)w * nsplit + kg * 8;

  f32x4v acc = {0.f, 0.f, 0.f, 0.f};
  vec8 fw[2][U], fh[2][U];
  vec8 zero;
#pragma unroll
  for (int j = 0; j < 8; ++j) zero[j] = (T)0.f;
  const int steps = nsplit / (32 * U);
  if (steps > 0) {
#pragma unroll
    for (int j = 0; j < U; ++j) {
      fw[0][j] = stream_load<vec8>(pw + 32 * j);
      fh[0][j] = mok ? *(const vec8*)(ph + 32 * j) : zero;
    }
  }
  for (int it = 0; it < steps; it += 2) {
    if (it + 1 < steps) {
      int k = (it + 1) * 32 * U;
#pragma unroll
      for (int j = 0; j < U; ++j) {
        fw[1][j] = stream_load<vec8>(pw + k + 32 * j);
        fh[1][j] = mok ? *(const vec8*)(ph + k + 32 * j) : zero;
      }
    }
#pragma unroll
    for (int j = 0; j < U; ++j) acc = Mfma16<T>::run(fw[0][j], fh[0][j], acc);
    if (it + 1 >= steps) break;
    if (it + 2 < steps) {
      int k = (it + 2) * 32 * U;
#pragma unroll
      for (int j = 0; j < U; ++j) {
        fw[0][j] = stream_load<vec8>(pw + k + 32 * j);
        fh[0][j] = mok ? *(const vec8*)(ph + k + 32 * j) : zero;
      }
    }
#pragma unroll
    for (int j = 0; j < U; ++j) acc = Mfma16<T>::run(fw[1][j], fh[1][j], acc);
  }
  for (int k = steps * 32 * U; k < nsplit; k += 32) {
    vec8 a = stream_load<vec8>(pw + k);
    vec8 c = mok ? *(const vec8*)(ph + k) : zero;
    acc = Mfma16<T>::run(a, c, acc);
  }

#pragma unroll
  for (int r = 0; r < 4; ++r) part[w][lane][r] = acc[r];
  __syncthreads();
  if (w == 0 && mok) {
    float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < DEC_SPLIT; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) s[r] += part[i][lane][r];
    int c = cb * 16 + 4 * kg;
    if (bd) add_w<T, 4>(bd + c, s);
    store_w<T, 4>(y + (size_t)r16 * K + c, s);
  }
}

template <typename T>
hipError_t launch_decode(const T* x, const T* wg, const T* wu, const T* wd, const T* bg,
                         const T* bu, const T* bd, T* h, T* y, int M, int K, int N, int act,
                         hipStream_t s) {
  if (decode_stream_supported(M, K, N))
    return launch_decode_stream<T>(x, wg, wu, wd, bg, bu, bd, h, y, M, K, N, act, s);
  int nblocks = N / 16;
  hipLaunchKernelGGL(decode_gateup_kernel<T>, dim3((nblocks + 3) / 4), dim3(256), 0, s, x, wg, wu,
                     bg, bu, h, M, K, N, act);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(decode_down_kernel<T>, dim3(K / 16), dim3(DEC_SPLIT * 64), 0, s, h, wd, bd, y,
                     M, K, N);
  return hipGetLastError();
}

template hipError_t launch_decode<f16>(const f16*, const f16*, const f16*, const f16*, const f16*,
                                       const f16*, const f16*, f16*, f16*, int, int, int, int,
                                       hipStream_t);
template hipError_t launch_decode<bf16>(const bf16*, const bf16*, const bf16*, const bf16*,
                                        const bf16*, const bf16*, const bf16*, bf16*, bf16*, int,
                                        int, int, int, hipStream_t);

}  // namespace gmlp
