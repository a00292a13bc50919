// HBM-bound helper kernels: element-wise gating backward, deterministic column sums (bias
// gradients) and the stand-alone dropout keep-mask generator.
#include "launch.hpp"

namespace gmlp {

template <typename T>
__global__ void __launch_bounds__(256)
    gating_bwd_kernel(const T* __restrict__ dh, const T* __restrict__ g, const T* __restrict__ u,
                      T* __restrict__ dg, T* __restrict__ du, size_t n8, int act,
                      DropoutParams d) {
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += stride) {
    size_t e = i * 8;
    float v[8];
    load_w<T, 8>(dh + e, v);
    gating_bwd_w<T, 8>(act, d, e, v, g, u, dg, du);
  }
}

template <typename T>
hipError_t launch_gating_bwd(const T* dh, const T* g, const T* u, T* dg, T* du, int64_t M, int64_t N,
                             int act, const DropoutParams& d, hipStream_t s) {
  size_t n8 = (size_t)M * N / 8;
  if (n8 == 0) return hipSuccess;
  size_t blocks = (n8 + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  hipLaunchKernelGGL(gating_bwd_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, s, dh, g, u, dg, du,
                     n8, act, d);
  return hipGetLastError();
}
template hipError_t launch_gating_bwd<f16>(const f16*, const f16*, const f16*, f16*, f16*, int64_t,
                                           int64_t, int, const DropoutParams&, hipStream_t);
template hipError_t launch_gating_bwd<bf16>(const bf16*, const bf16*, const bf16*, bf16*, bf16*,
                                            int64_t, int64_t, int, const DropoutParams&,
                                            hipStream_t);
template hipError_t launch_gating_bwd<float>(const float*, const float*, const float*, float*,
                                             float*, int64_t, int64_t, int, const DropoutParams&,
                                             hipStream_t);

// Second stage of a split reduction: adds the partial results up in split order (deterministic)
// and hands 8 consecutive columns of one row to the epilogue the unsplit GEMM would have run.
template <typename T, typename Epi>
__global__ void __launch_bounds__(256)
    splitk_reduce_kernel(const float* __restrict__ ws, int splits, size_t split_stride, size_t acc_stride,
                         typename Epi::Args ea, size_t n8, int N) {
  size_t step = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += step) {
    size_t e = i * 8;
    alignas(16) float v0[8], v1[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) v0[r] = v1[r] = 0.f;
    for (int s = 0; s < splits; ++s) {
      const float* p = ws + (size_t)s * split_stride + e;
      f32x4 a = *(const f32x4*)p, b = *(const f32x4*)(p + 4);
#pragma unroll
      for (int r = 0; r < 4; ++r) { v0[r] += a[r]; v0[4 + r] += b[r]; }
      if (acc_stride) {
        f32x4 c = *(const f32x4*)(p + acc_stride), d = *(const f32x4*)(p + acc_stride + 4);
#pragma unroll
        for (int r = 0; r < 4; ++r) { v1[r] += c[r]; v1[4 + r] += d[r]; }
      }
    }
    Epi::template apply<8>(ea, (int)(e / (size_t)N), (int)(e % (size_t)N), v0, v1);
  }
}

template <typename T, typename Epi>
hipError_t launch_splitk_reduce(const float* ws, int splits, size_t split_stride, size_t acc_stride,
                                const typename Epi::Args& ea, int64_t M, int64_t N, hipStream_t s) {
  size_t n8 = (size_t)M * N / 8;
  if (n8 == 0) return hipSuccess;
  size_t blocks = (n8 + 255) / 256;
  if (blocks > 256 * 8) blocks = 256 * 8;
  hipLaunchKernelGGL((splitk_reduce_kernel<T, Epi>), dim3((unsigned)blocks), dim3(256), 0, s, ws, splits,
                     split_stride, acc_stride, ea, n8, (int)N);
  return hipGetLastError();
}
#define GMLP_REDUCE_INST(T, EPI)                                                                    \
  template hipError_t launch_splitk_reduce<T, EPI<T>>(const float*, int, size_t, size_t,            \
                                                      const EPI<T>::Args&, int64_t, int64_t, hipStream_t);
GMLP_REDUCE_INST(f16, EpiStore)
GMLP_REDUCE_INST(bf16, EpiStore)
GMLP_REDUCE_INST(f16, EpiGateUp)
GMLP_REDUCE_INST(bf16, EpiGateUp)
#undef GMLP_REDUCE_INST

// Column sums in two fixed-order stages: COLSUM_SPLITS row ranges -> fp32 partials -> total.
// Up to COLSUM_GROUP_MAX arrays with the same number of rows share the two launches (the bias
// gradients of one backward pass); blockIdx.z selects the array.
constexpr int COLSUM_SPLITS = 64;

template <typename T>
__global__ void __launch_bounds__(256) colsum_partial_kernel(ColsumGroup<T> g, int64_t M) {
  const T* __restrict__ a = g.a[blockIdx.z];
  float* __restrict__ ws = g.ws[blockIdx.z];
  const int64_t C = g.C[blockIdx.z];
  int64_t c = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (c >= C) return;
  int64_t rows = (M + COLSUM_SPLITS - 1) / COLSUM_SPLITS;
  int64_t r0 = blockIdx.y * rows, r1 = r0 + rows < M ? r0 + rows : M;
  float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  int64_t r = r0;
  for (; r + 4 <= r1; r += 4) {  // four independent 16-byte loads in flight per lane
    float t[4][8];
#pragma unroll
    for (int u = 0; u < 4; ++u) load_w<T, 8>(a + (r + u) * C + c, t[u]);
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int q = 0; q < 8; ++q) s[q] += t[u][q];
  }
  for (; r < r1; ++r) {
    float t[8];
    load_w<T, 8>(a + r * C + c, t);
#pragma unroll
    for (int q = 0; q < 8; ++q) s[q] += t[q];
  }
  float* p = ws + (int64_t)blockIdx.y * C + c;
  *(f32x4*)p = f32x4{s[0], s[1], s[2], s[3]};
  *(f32x4*)(p + 4) = f32x4{s[4], s[5], s[6], s[7]};
}

template <typename T>
__global__ void __launch_bounds__(256) colsum_final_kernel(ColsumGroup<T> g) {
  const float* __restrict__ ws = g.ws[blockIdx.z];
  const int64_t C = g.C[blockIdx.z];
  int64_t c = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (c >= C) return;
  f32x4 s = {0.f, 0.f, 0.f, 0.f};
  for (int i = 0; i < COLSUM_SPLITS; ++i) s += *(const f32x4*)(ws + (int64_t)i * C + c);
  float t[4] = {s[0], s[1], s[2], s[3]};
  store_w<T, 4>(g.out[blockIdx.z] + c, t);
}

size_t colsum_workspace_bytes(int64_t, int64_t C) { return (size_t)COLSUM_SPLITS * C * sizeof(float); }

template <typename T>
hipError_t launch_colsum_group(const ColsumGroup<T>& g, int count, int64_t M, hipStream_t s) {
  int64_t cmax = 0;
  for (int i = 0; i < count; ++i) cmax = g.C[i] > cmax ? g.C[i] : cmax;
  unsigned bx8 = (unsigned)((cmax / 8 + 255) / 256), bx4 = (unsigned)((cmax / 4 + 255) / 256);
  hipLaunchKernelGGL(colsum_partial_kernel<T>, dim3(bx8, COLSUM_SPLITS, count), dim3(256), 0, s, g, M);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(colsum_final_kernel<T>, dim3(bx4, 1, count), dim3(256), 0, s, g);
  return hipGetLastError();
}
template hipError_t launch_colsum_group<f16>(const ColsumGroup<f16>&, int, int64_t, hipStream_t);
template hipError_t launch_colsum_group<bf16>(const ColsumGroup<bf16>&, int, int64_t, hipStream_t);
template hipError_t launch_colsum_group<float>(const ColsumGroup<float>&, int, int64_t, hipStream_t);

// Column sums for callers that cannot allocate: the partial sums of the first stage live in this
// array instead of a caller's workspace.  Every GPU the library runs on holds its own copy, at
// its own address, until the process ends (COLSUM_SPLITS x COLSUM_STATIC_MAX_C floats = 8 MiB).
// The name below is a host-side handle, not a device address: host code only ever uses the
// pointer hipGetSymbolAddress returned for the current device.
static __device__ __align__(256) float scratch[(size_t)COLSUM_SPLITS * COLSUM_STATIC_MAX_C];

hipError_t colsum_static_scratch(float** out, hipStream_t s) {
  static std::atomic<float*> known[64];  // per device
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev)) return e;
  const bool tracked = dev >= 0 && dev < 64;
  float* p = tracked ? known[dev].load(std::memory_order_acquire) : nullptr;
  if (p == nullptr) {
    // first use on this device (gmlp_init makes it ahead of time): a symbol lookup is not
    // something to do while the stream is being captured
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipError_t e = hipStreamIsCapturing(s, &st)) return e;
    if (st != hipStreamCaptureStatusNone) return hipErrorStreamCaptureUnsupported;
    void* q = nullptr;
    if (hipError_t e = hipGetSymbolAddress(&q, HIP_SYMBOL(scratch))) return e;
    if (q == nullptr) return hipErrorInvalidSymbol;
    p = (float*)q;
    if (tracked) known[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return hipSuccess;
}

// The first stage writes every partial sum the second stage reads (all COLSUM_SPLITS row ranges of
// all C columns, zeros for empty ranges), so nothing in the array has to be cleared between calls.
template <typename T>
hipError_t launch_colsum_static(const T* a, T* out, int64_t M, int64_t C, hipStream_t s) {
  float* ws = nullptr;
  if (hipError_t e = colsum_static_scratch(&ws, s)) return e;
  ColsumGroup<T> g = {};
  g.a[0] = a;
  g.out[0] = out;
  g.ws[0] = ws;
  g.C[0] = C;
  return launch_colsum_group<T>(g, 1, M, s);
}
template hipError_t launch_colsum_static<f16>(const f16*, f16*, int64_t, int64_t, hipStream_t);
template hipError_t launch_colsum_static<bf16>(const bf16*, bf16*, int64_t, int64_t, hipStream_t);
template hipError_t launch_colsum_static<float>(const float*, float*, int64_t, int64_t, hipStream_t);

__global__ void __launch_bounds__(256)
    dropout_mask_kernel(uint8_t* __restrict__ mask, size_t n4, DropoutParams d) {
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
    bool keep[4];
    uint32_t packed = 0x01010101u;
    if (d.enabled) {
      dropout_keep4(d, i, keep);
      packed = 0;
#pragma unroll
      for (int r = 0; r < 4; ++r) packed |= (keep[r] ? 1u : 0u) << (8 * r);
    }
    *(uint32_t*)(mask + i * 4) = packed;
  }
}

hipError_t launch_dropout_mask(uint8_t* mask, int64_t M, int64_t N, const DropoutParams& d,
                               hipStream_t s) {
  size_t n4 = (size_t)M * N / 4;
  if (n4 == 0) return hipSuccess;
  size_t blocks = (n4 + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  hipLaunchKernelGGL(dropout_mask_kernel, dim3((unsigned)blocks), dim3(256), 0, s, mask, n4, d);
  return hipGetLastError();
}

}  // namespace gmlp
