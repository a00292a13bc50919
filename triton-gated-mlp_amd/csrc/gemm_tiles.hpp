// LDS operand tiles of the pipelined full-tile GEMM (gemm_pipelined.hpp) and small host helpers.
//
// Tiles move with buffer_load_dwordx4 ... lds: each lane's 16 bytes land in LDS at (wave base +
// 16*lane) without passing through VGPRs; bank-conflict-free layouts are obtained by permuting
// WHICH 16-byte chunk of a row each lane fetches (XOR swizzle on the global side).  Addresses are
// (buffer base) + (wave-uniform SGPR tile offset) + (constant per-lane VGPR offset), so stepping
// to the next reduction tile costs scalar adds only.  Reduction-strided operands are read with
// ds_read_b64_tr_b16, which hands each lane 4 consecutive reduction elements of one output row
// out of a [k][row] tile.
#pragma once
#include <atomic>
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
struct LdsTile {
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

  // MFMA operand fragment (8 reduction elements per lane) for a 16 x 16 x 32 instruction: rows
  // row0 .. row0+15, reduction step ks (32 elements).  Lane l carries row l % 16 and reduction
  // slots 8*(l / 16) .. +7.
  template <int MI>
  static __device__ __forceinline__ vec8 frag_mi(const char* lds_tile, int row0, int ks, int lane) {
    static_assert(MI == 16, "MFMA tile is 16x16x32");
    constexpr int CPS = 64 / MI;  // 16-byte chunks per row per reduction step
    if constexpr (!KS) {
      int row = row0 + (lane & (MI - 1));
      int c = ks * CPS + lane / MI;
      return *(const vec8*)(lds_tile + row * (BK * 2) + ((c ^ swz_kc(row)) << 4));
    } else {
      // 16-lane group g reads rows nb .. nb+15 at reduction kb .. kb+7 with two transpose reads
      // (kb+0..3, kb+4..7): lane r of the group addresses reduction row kb + r/4, rows
      // nb + 4*(r%4) .. +3, and receives the 4 reduction elements of row nb + r.
      int g = lane >> 4, r = lane & 15;
      int nb = row0;
      int kb = ks * 32 + 8 * g;
      int n = nb + 4 * (r & 3);
      int kq = r >> 2;  // == reduction row & 3
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

// Kernels with more than 64 KiB of dynamic LDS need the limit raised per device and per kernel
// (hipFuncSetAttribute), a call that must not be made while a stream is being captured.  Every
// such kernel has one LdsKernel object, registered when the library is loaded: prepare_lds_kernels
// (called by gmlp_init) raises the limit of all of them on the current device up front; a launch
// that still finds its kernel unprepared does it itself unless its stream is capturing, in which
// case it reports hipErrorStreamCaptureUnsupported instead of making the call.
struct LdsKernel {
  const void* kernel;
  int bytes;
  std::atomic<unsigned char> done[64];  // per device
  LdsKernel(const void* k, int b);      // registers itself (api.hip)
};
hipError_t prepare_lds_kernels();  // every registered kernel, on the current device
template <auto KERNEL, int BYTES>
inline LdsKernel lds_kernel_of{(const void*)KERNEL, BYTES};

inline hipError_t allow_dynamic_lds(LdsKernel& k, hipStream_t s) {
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev)) return e;
  const bool tracked = dev >= 0 && dev < 64;
  if (tracked && k.done[dev].load(std::memory_order_acquire)) return hipSuccess;
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipError_t e = hipStreamIsCapturing(s, &st)) return e;
  if (st != hipStreamCaptureStatusNone) return hipErrorStreamCaptureUnsupported;
  if (hipError_t e = hipFuncSetAttribute(k.kernel, hipFuncAttributeMaxDynamicSharedMemorySize, k.bytes)) return e;
  if (tracked) k.done[dev].store(1, std::memory_order_release);
  return hipSuccess;
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

}  // namespace gmlp
