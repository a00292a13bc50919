// Global -> LDS transfers that bypass the vector registers (buffer_load ... lds) and the explicit
// vector-memory waits that order them, shared by the GEMM and the skinny-M streaming kernels.
#pragma once
#include "common.hpp"

namespace gmlp {

typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef short i16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) void lds_void;
typedef int buffer_rsrc __attribute__((ext_vector_type(4)));

// Raw buffer descriptor over `bytes` bytes behind `base` (offsets are 32-bit bytes).  The hardware
// range-checks voffset + soffset + immediate offset against `bytes`, per dword: what lies beyond
// reads as zero, also into LDS, and never faults (checked on gfx950 with a stand-alone probe).
__device__ __forceinline__ buffer_rsrc make_rsrc(const void* base, uint32_t bytes = 0x7FFFFFFFu) {
  uint64_t b = (uint64_t)base;
  buffer_rsrc r = {(int)(uint32_t)b, (int)((b >> 32) & 0xffffu), (int)bytes, 0x00020000};
  return r;
}
// 16 bytes per lane from (rsrc base + soffset + voffset) to LDS byte address (lds_wave_base +
// 16*lane).  Written as assembly on purpose: the compiler's bookkeeping for the LDS-DMA builtins
// makes every later LDS read it cannot disambiguate (the transpose reads) wait for ALL loads in
// flight; here the ordering is explicit instead (wait_vmem + barrier before a slot is read).
// STREAM marks data that is read once (non-temporal: do not keep it in the caches).
template <bool STREAM = false>
__device__ __forceinline__ void load16_to_lds(buffer_rsrc r, uint32_t voffset, uint32_t soffset,
                                              uint32_t lds_wave_base) {
  if (STREAM) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "buffer_load_dwordx4 %1, %2, %3 offen nt lds"
        :
        : "s"(lds_wave_base), "v"(voffset), "s"(r), "s"(soffset)
        : "memory");
  } else {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "buffer_load_dwordx4 %1, %2, %3 offen lds"
        :
        : "s"(lds_wave_base), "v"(voffset), "s"(r), "s"(soffset)
        : "memory");
  }
}

// The same transfer split in two, for loops where instruction issue is tight: M0 (the LDS base) is
// written once for up to four loads, which then differ by the instruction's immediate offset
// (0, 1024, 2048 or 3072).  The immediate is added to the LDS address AND to the global address,
// so the caller passes a voffset that already has it subtracted (see DMA_BIAS in gemm_pipelined.hpp).
// That M0 must stay live until the group's last load cannot be expressed to the compiler (M0 is a
// reserved register: it is not accepted as an operand, and not reliably as a clobber), which has no
// use for M0 of its own in kernels without indirect register
// indexing, message or GWS instructions.  The build does not take that on trust: csrc/check_m0.py
// scans the device assembly of every GEMM unit and fails it if any instruction outside the
// inline-assembly blocks writes or implies M0 in a kernel that contains these loads.
__device__ __forceinline__ void set_lds_dma_base(uint32_t lds_wave_base) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0"
      :
      : "s"(lds_wave_base)
      : "memory");
}
template <int INST_OFF>
__device__ __forceinline__ void load16_to_lds_at(buffer_rsrc r, uint32_t voffset, uint32_t soffset) {
  asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:%3 lds"
               :
               : "v"(voffset), "s"(r), "s"(soffset), "n"(INST_OFF)
               : "memory");
}

// The LDS write of a global->LDS load is complete when the wavefront's vector-memory counter has
// drained past it; a workgroup barrier alone does not wait for it.  N = loads allowed in flight.
template <int N>
__device__ __forceinline__ void wait_vmem() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

}  // namespace gmlp
