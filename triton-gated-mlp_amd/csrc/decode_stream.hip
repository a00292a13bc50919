// Skinny-M (M <= 32) weight-streaming kernels, HBM-bound: every weight byte is fetched once, in
// 512-byte (or 256-byte) row segments moved global -> LDS without passing through registers.
//
// One persistent workgroup of three wavefronts per CU.  The workgroup takes blocks of weight rows
// that share one set of token operands: rows r..r+15 of W_gate and of W_up (GATED), or 32
// consecutive rows of W_down (16 when a CU's share is no more than that); twice as many rows with
// 256-byte segments.  Whole blocks go round-robin over the workgroups, the rows that do not fill a
// last round are shared out evenly as one partly empty block each.  Its wavefronts split the
// reduction range in near-equal runs of chunks (256 or 128 elements) and combine their partial
// sums through LDS at the end of each block (fixed order, so the result is deterministic).  Each
// wavefront runs a private ring of 3 or 4 LDS slots; a slot holds one stage = one chunk of the
// block's weight rows, 8 KiB per matrix.  The matching token-row operands (x or H, L2-resident)
// are fetched straight into registers, as many stages ahead: one 16-token tile for M <= 16, two
// beyond (MT; the weight fragment read from LDS then feeds two MFMAs).  Achieved HBM bandwidth
// follows the bytes in flight per CU, and LDS capacity bounds those: wavefronts x 3 slots x 16 KiB
// fill 144 of the 160 KiB.  The stream of stages runs on across block boundaries, so the ring
// never drains; loads past the end re-fetch the last stage into a free slot, which keeps the
// in-flight count constant.
//
//   GATED:   H[m, r] = act(x.W_gate[r] + b_gate[r]) * (x.W_up[r] + b_up[r])      (r over N)
//   !GATED:  Y[m, r] = H.W_down[r] + b_down[r]                                   (r over K)
//
// LDS layout of a slot: regions of 16 rows x SEGB bytes (SEGB = 512 or 256); the 16-byte chunk c
// of row r is stored at position c ^ r, so the 16 lanes that read one chunk index of 16 different
// rows for v_mfma_f32_16x16x32 hit 16 different bank groups.
//
// All vector-memory loads of the main loop are written as assembly and ordered by explicit
// s_waitcnt vmcnt(N): the compiler does not see them, so it cannot serialise them either (the
// build checks the generated assembly for uses of a load's destination ahead of its wait).
#include "launch.hpp"
#include "lds_dma.hpp"

namespace gmlp {

typedef float f32x4v __attribute__((ext_vector_type(4)));

template <typename T>
struct Mfma16x;
template <>
struct Mfma16x<f16> {
  static __device__ __forceinline__ f32x4v run(f16x8 a, f16x8 b, f32x4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mfma16x<bf16> {
  static __device__ __forceinline__ f32x4v run(bf16x8 a, bf16x8 b, f32x4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};

constexpr int DS_CH = 256;            // reduction elements per stage
constexpr int DS_REGION = 16 * 512;   // bytes of one 16-row region
// ring slots per wavefront (and stages in flight): 3 slots of two matrices, or 4 of one (3 where
// two token tiles go with 512-byte segments: the token operands in flight are bounded by the
// registers, see the kernel)
constexpr int ds_ring_depth(int nmat, int mt, int segb) { return nmat == 2 || (mt == 2 && segb == 512) ? 3 : 4; }
constexpr int DS_WAVES = 3;           // wavefronts per workgroup
// buffers for the partial sums that change hands at the end of a block: two (alternating) where
// LDS holds them beside the rings, else one
constexpr int ds_part_buffers(int nmat, int mt, int segb) {
  return DS_WAVES * ds_ring_depth(nmat, mt, segb) * nmat * DS_REGION + 2 * (DS_WAVES - 1) * nmat * (512 / segb) * mt * 1024 <=
                 160 * 1024
             ? 2
             : 1;
}
constexpr uint32_t DS_NOWHERE = 0x80000000u;  // voffset beyond any operand (operands are < 2 GiB)
constexpr int DS_WIDE_SEGMENT_MAX_M = 20;     // two token tiles: 512-byte row segments up to here, 256 beyond
constexpr int DS_H_TILED_MIN_M = 10;           // H goes out in fragment order above this many token rows

struct StreamArgs {
  const void* x;      // [M, ldx] token rows (x or H)
  const void* w[2];   // [R, red] weight matrices
  const void* bias[2];
  void* out;          // [M, ldo]
  int M, R, red, ldx, ldo;
  int act;            // Act code (GATED only)
  int tiled;          // H (GATED: out, otherwise: x) is in fragment order, see ds_h_tiled()
};

typedef int i32x4 __attribute__((ext_vector_type(4)));

// 16 bytes per lane into registers; completion is tracked by the caller (wait_vmem_keep).
__device__ __forceinline__ i32x4 load16_async(buffer_rsrc r, uint32_t voffset, uint32_t soffset) {
  i32x4 v;
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"
               : "=v"(v)
               : "v"(voffset), "s"(r), "s"(soffset)
               : "memory");
  return v;
}
// s_waitcnt vmcnt(N) that also "defines" the registers a stage's token operands arrive in (8 per
// token tile), so no use of them can be scheduled above the wait.  The second statement issues no
// instruction: volatile asm statements keep their order, so it ties the second tile's registers
// to the same point.
template <int N, int NX>
__device__ __forceinline__ void wait_vmem_keep(i32x4 (&x)[NX]) {
  static_assert(NX == 8 || NX == 16, "one or two token tiles");
  asm volatile("s_waitcnt vmcnt(%8)"
               : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]),
                 "+v"(x[7])
               : "n"(N)
               : "memory");
  if constexpr (NX == 16)
    asm volatile(""
                 : "+v"(x[8]), "+v"(x[9]), "+v"(x[10]), "+v"(x[11]), "+v"(x[12]), "+v"(x[13]),
                   "+v"(x[14]), "+v"(x[15])
                 :
                 : "memory");
}

// NMAT: weight matrices / runs of rows per stage (GATED: W_gate and W_up; otherwise 1 or 2 runs of
//       W_down rows).
// MT:   tiles of 16 token slots (M <= 16 * MT).
// SEGB: bytes of a weight row per stage, 512 or 256.  A stage always moves 8 KiB per matrix: 16
//       rows x 512 bytes, or 32 rows x 256 bytes as two 16-row regions.  The second form halves
//       the token operands fetched per weight byte (a stage spans half the reduction elements for
//       twice the rows), which is what two token tiles need: with 16-row blocks their token
//       operands cost as much L2 traffic as the weights cost HBM traffic.
template <typename T, bool GATED, int NMAT, int MT, int SEGB>
__global__ void __launch_bounds__(DS_WAVES * 64) decode_stream_kernel(StreamArgs a) {
  typedef typename Traits<T>::vec8 vec8;
  static_assert(NMAT == 2 || (NMAT == 1 && !GATED), "gated blocks stream two matrices");
  static_assert(SEGB == 512 || SEGB == 256, "row segment of a stage");
  constexpr int DS_RD = ds_ring_depth(NMAT, MT, SEGB);
  constexpr int HALVES = 512 / SEGB;          // 16-row regions per matrix and stage
  constexpr int NREG = NMAT * HALVES;         // 16-row regions per stage
  constexpr int REGION = 16 * SEGB;           // bytes of a region
  constexpr int CH = SEGB / 2;                // reduction elements per stage
  constexpr int KS = CH / 32;                 // MFMA steps per stage
  constexpr int CPR = SEGB / 16;              // 16-byte chunks per row segment
  constexpr int LPR = REGION / 1024;          // load instructions per region (64 lanes x 16 bytes each)
  // The token operands in flight live in VGPRs that the loads fill asynchronously.  Were there not
  // enough of the 256 left beside them, the compiler would park them elsewhere right after the
  // load instruction, before the data has arrived.
  static_assert(DS_RD * KS * MT * 4 <= 192, "token operands in flight must leave room in the VGPRs");
  // weight rows (per matrix) a block advances by
  constexpr int BLOCK_ROWS = GATED ? 16 * HALVES : 16 * NREG;
  constexpr int SLOT = NREG * REGION;
  constexpr int LPS = KS * MT + NREG * LPR;  // load instructions per stage (token operands + weights)
  // A stage is complete when no more than the DS_RD - 1 younger stages are in flight.  vmcnt has 6
  // bits: where that count exceeds 63 the wait also covers the first token-operand loads of the
  // next stage (issued right behind the awaited weights, and loads return in order).
  constexpr int YOUNGER = (DS_RD - 1) * LPS < 63 ? (DS_RD - 1) * LPS : 63;
  static_assert((DS_RD - 1) * LPS - YOUNGER <= KS * MT, "the wait may only reach into the next stage's token operands");
  // Partial sums change hands through LDS in two alternating buffers, or, where LDS does not hold
  // two, in one buffer with a second barrier behind its readers.
  constexpr int PART_FLOATS = (DS_WAVES - 1) * NREG * MT * 256;
  constexpr int PARITIES = ds_part_buffers(NMAT, MT, SEGB);

  extern __shared__ __align__(1024) char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void*)smem + wave * (DS_RD * SLOT);
  char* ring = smem + wave * (DS_RD * SLOT);
  float* part = (float*)(smem + DS_WAVES * DS_RD * SLOT);  // [parities][waves-1][NREG][MT][64][4]

  // Blocks of BLOCK_ROWS weight rows go round-robin over the workgroups (block b, b + G, ...: at any
  // time the chip streams one contiguous band of rows) for as many rounds as every workgroup gets a
  // whole block.  The rows left over (the tail) are shared out evenly instead, in multiples of 4
  // (what one lane stores), so that every CU streams the same number of bytes whatever R is: a
  // workgroup's tail share [t_begin, t_end) is one last block with fewer valid rows, the loads of
  // the others go nowhere (an offset beyond the descriptor reads as zero and moves no data) and
  // their results are not stored.
  const int G = (int)gridDim.x;
  const int full = a.R / BLOCK_ROWS / G;
  const int tail0 = full * G * BLOCK_ROWS, tail_rows = a.R - tail0;
  const int t_begin = tail0 + (((int)blockIdx.x * tail_rows / G) & ~3);
  const int t_end = (int)blockIdx.x + 1 == G ? a.R : tail0 + ((((int)blockIdx.x + 1) * tail_rows / G) & ~3);
  // first row and number of existing rows (BLOCK_ROWS or more: all) of this workgroup's j-th block
  auto block_rows = [&](int j, int& row0, int& valid) __attribute__((always_inline)) {
    if (j < full) {
      row0 = ((int)blockIdx.x + j * G) * BLOCK_ROWS;
      valid = BLOCK_ROWS;
    } else {
      row0 = t_begin + (j - full) * BLOCK_ROWS;
      valid = t_end - row0;
    }
  };
  const int chunks = a.red / CH;
  // wavefront w reduces chunks [c0, c0 + spb)
  const int c0 = (chunks * wave) / DS_WAVES;
  const int spb = (chunks * (wave + 1)) / DS_WAVES - c0;
  const int my_blocks = full + (t_end - t_begin + BLOCK_ROWS - 1) / BLOCK_ROWS;
  const int total = my_blocks * spb;
  // Workgroup b starts each block at chunk b % spb of its wavefronts' ranges and wraps around (a
  // sum does not mind the order).  Without it every workgroup on the chip reads the same offset
  // along its rows at the same time, and for a power-of-two row pitch (W_gate, W_up of the usual
  // hidden sizes) those addresses crowd onto a few memory channels: 154 -> 142 us at K = 8192.
  const int rot = (int)blockIdx.x % spb;

  // Per-lane byte offsets: weights, LPR load instructions per region (1024 / SEGB rows each);
  // token operands, the 16 bytes of token row 16 t + lane%16 this lane feeds to the MFMAs of tile t.
  const int r16 = lane & 15, kg = lane >> 4;
  uint32_t woff[LPR], xoff[MT];
  int wrow[LPR];  // row of the region that load q of this lane fetches
#pragma unroll
  for (int q = 0; q < LPR; ++q) {
    int row = (64 / CPR) * q + lane / CPR, pos = lane % CPR;
    wrow[q] = row;
    woff[q] = (uint32_t)(row * a.red + (pos ^ row) * 8) * 2u;
  }
  const bool tiled_x = !GATED && a.tiled;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    if (tiled_x) {
      // [red/8][16 MT token slots][8 elements]: the 8-element group kg of a fragment is 256 MT
      // bytes after the previous one (for MT = 1 a fragment is one contiguous KiB)
      xoff[t] = (uint32_t)(kg * (256 * MT) + t * 256 + r16 * 16);
    } else {
      int xr = 16 * t + r16 < a.M ? 16 * t + r16 : a.M - 1;  // rows past M repeat the last token row
      xoff[t] = (uint32_t)(xr * a.ldx + kg * 8) * 2u;
    }
  }
  const uint32_t xq = tiled_x ? 1024u * MT : 64u;  // from one MFMA's token operand to the next
  // exact size: an offset past the end reads as zero instead of touching memory
  const buffer_rsrc rx = make_rsrc(a.x, tiled_x ? (uint32_t)(16 * MT) * (uint32_t)a.red * 2u
                                                : (uint32_t)a.M * (uint32_t)a.ldx * 2u);
  // exact sizes; region g of a stage: GATED: matrix g / HALVES, rows 16 (g % HALVES) .. +15 of the
  // block; otherwise rows 16 g .. +15 of the block of W_down
  const uint32_t pitch = (uint32_t)a.red * 2u;
  const uint32_t w_bytes = (uint32_t)a.R * pitch;
  const buffer_rsrc rw[2] = {make_rsrc(a.w[0], w_bytes), make_rsrc(GATED ? a.w[1] : a.w[0], w_bytes)};

  i32x4 xf[DS_RD][KS * MT];  // [stage in flight][MFMA step q][token tile]

  // Stage i_req of this wavefront's stream: token operands into xf[u], weights into ring slot u.
  auto issue_stage = [&](int i_req, int u) __attribute__((always_inline)) {
    int i = i_req < total ? i_req : total - 1;
    int j = i / spb, c = i - j * spb;
    c += rot;
    c = c < spb ? c : c - spb;
    int row0, valid;
    block_rows(j, row0, valid);
    uint32_t koff = (uint32_t)((c0 + c) * CH) * 2u;
    // token operand of the stage's q-th MFMA step: 64 bytes further along each row of x, or the
    // next fragment of H (a stage of CH elements x 16 MT token slots)
    const uint32_t xstage = tiled_x ? koff * (16u * MT) : koff;
#pragma unroll
    for (int q = 0; q < KS; ++q)
#pragma unroll
      for (int t = 0; t < MT; ++t) xf[u][q * MT + t] = load16_async(rx, xoff[t], xstage + q * xq);
    uint32_t slot = lds_base + (uint32_t)u * SLOT;
    uint32_t woffs = (uint32_t)row0 * pitch + koff;
#pragma unroll
    for (int g = 0; g < NREG; ++g) {
      const int first = GATED ? 16 * (g % HALVES) : 16 * g;  // region's first row within the block
      const int valid_g = valid - first;
#pragma unroll
      for (int q = 0; q < LPR; ++q)
        load16_to_lds<true>(rw[GATED ? g / HALVES : 0], wrow[q] < valid_g ? woff[q] : DS_NOWHERE,
                            woffs + (uint32_t)first * pitch, slot + g * REGION + q * 1024);
    }
  };

  f32x4v acc[NREG][MT];
#pragma unroll
  for (int g = 0; g < NREG; ++g)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[g][t] = f32x4v{0.f, 0.f, 0.f, 0.f};

#pragma unroll
  for (int p = 0; p < DS_RD; ++p) issue_stage(p, p);

  int in_block = 0, blk = 0;
  for (int i0 = 0; i0 < total; i0 += DS_RD) {
#pragma unroll
    for (int u = 0; u < DS_RD; ++u) {
      const int i = i0 + u;
      if (i < total) {
        wait_vmem_keep<YOUNGER, KS * MT>(xf[u]);
        const char* slot = ring + u * SLOT;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          int pos = ((ks * 4 + kg) ^ r16) << 4;
#pragma unroll
          for (int g = 0; g < NREG; ++g) {
            vec8 wf = *(const vec8*)(slot + g * REGION + r16 * SEGB + pos);
#pragma unroll
            for (int t = 0; t < MT; ++t)
              acc[g][t] = Mfma16x<T>::run(wf, __builtin_bit_cast(vec8, xf[u][ks * MT + t]), acc[g][t]);
          }
        }
        // The MFMAs above consumed every LDS read of this slot, so it can be refilled.
        issue_stage(i + DS_RD, u);

        if (++in_block == spb) {
          // Block finished: wavefronts 1.. hand their partial sums to wavefront 0.  A lane holds,
          // per token tile t, token row 16 t + lane%16 and, per region, weight rows 4*(lane/16) + r
          // of the region.
          in_block = 0;
          float* pp = part + (PARITIES == 2 ? (blk & 1) * PART_FLOATS : 0);
          if (wave > 0) {
#pragma unroll
            for (int g = 0; g < NREG; ++g)
#pragma unroll
              for (int t = 0; t < MT; ++t)
                *(f32x4v*)(pp + (((wave - 1) * NREG + g) * MT + t) * 256 + lane * 4) = acc[g][t];
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
          if (wave == 0) {
            int row0, valid;
            block_rows(blk, row0, valid);
#pragma unroll
            for (int t = 0; t < MT; ++t) {
              const int tok = 16 * t + r16;
              if (!((GATED && a.tiled) || tok < a.M)) continue;
              float v[NREG][4];
#pragma unroll
              for (int g = 0; g < NREG; ++g) {
#pragma unroll
                for (int r = 0; r < 4; ++r) v[g][r] = acc[g][t][r];
#pragma unroll
                for (int w = 0; w < DS_WAVES - 1; ++w) {
                  f32x4v o = *(const f32x4v*)(pp + ((w * NREG + g) * MT + t) * 256 + lane * 4);
#pragma unroll
                  for (int r = 0; r < 4; ++r) v[g][r] += o[r];
                }
                // this lane's four rows of the region, as rows of the block
                const int first = (GATED ? 16 * (g % HALVES) : 16 * g) + 4 * kg;
                const T* bias = (const T*)a.bias[GATED ? g / HALVES : 0];
                if (bias && first < valid) add_w<T, 4>(bias + row0 + first, v[g]);
              }
              if (GATED) {
#pragma unroll
                for (int hf = 0; hf < HALVES; ++hf) {
                  const int first = 16 * hf + 4 * kg;
                  const int r0 = row0 + first;
                  float res[4];
                  act_fwd_w<4>(a.act, v[hf], res);
#pragma unroll
                  for (int r = 0; r < 4; ++r) res[r] *= v[HALVES + hf][r];
                  // Fragment order: H goes out the way the down projection's MFMAs take it in,
                  // [N/8][16 MT token slots][8 elements], so that a token-operand fragment there is
                  // 4 runs of 256 MT bytes (one contiguous KiB for MT = 1) instead of 16 row pieces
                  // of 64 bytes.  All slots are written (slots past M repeat the last token), so
                  // nothing uninitialised is multiplied.
                  if (first < valid) {
                    if (a.tiled)
                      store_w<T, 4>((T*)a.out + ((size_t)(r0 >> 3) * (16 * MT) + tok) * 8 + (r0 & 7), res);
                    else
                      store_w<T, 4>((T*)a.out + (size_t)tok * a.ldo + r0, res);
                  }
                }
              } else {
#pragma unroll
                for (int g = 0; g < NREG; ++g)
                  if (16 * g + 4 * kg < valid)
                    store_w<T, 4>((T*)a.out + (size_t)tok * a.ldo + row0 + 16 * g + 4 * kg, v[g]);
              }
            }
          }
          if (PARITIES == 1) {
            // one buffer: nobody writes the next block's partial sums before wavefront 0 has read these
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
            __builtin_amdgcn_s_barrier();
          }
#pragma unroll
          for (int g = 0; g < NREG; ++g)
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[g][t] = f32x4v{0.f, 0.f, 0.f, 0.f};
          ++blk;
        }
      }
    }
  }
  wait_vmem<0>();
}

template <typename T, bool GATED, int NMAT, int MT, int SEGB>
static hipError_t launch_stream(const StreamArgs& a, int num_cu, hipStream_t s) {
  constexpr int NREG = NMAT * (512 / SEGB);
  constexpr int LDS = DS_WAVES * ds_ring_depth(NMAT, MT, SEGB) * NMAT * DS_REGION +
                      ds_part_buffers(NMAT, MT, SEGB) * (DS_WAVES - 1) * NREG * MT * 256 * 4;
  static_assert(LDS <= 160 * 1024, "a workgroup has 160 KiB of LDS");
  constexpr auto kern = decode_stream_kernel<T, GATED, NMAT, MT, SEGB>;
  if (hipError_t e = allow_dynamic_lds(lds_kernel_of<kern, LDS>, s)) return e;
  // one workgroup per CU, each with its share of the rows (a partly empty block when that is less
  // than a block); fewer workgroups when a share would be under 8 rows
  int grid = a.R / 8 < num_cu ? a.R / 8 : num_cu;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(DS_WAVES * 64), LDS, s, a);
  return hipGetLastError();
}

// Layout of the intermediate H between the two kernels.  Row-major [M, N] costs the down projection
// M pieces of 64 bytes per token-operand fragment, fragment order always one KiB (16 token slots):
// cheaper from about half-full upwards.  Two token tiles always use fragment order.
static int ds_h_tiled(int M) { return M > DS_H_TILED_MIN_M ? 1 : 0; }

bool decode_stream_supported(int M, int K, int N) {
  return M >= 1 && M <= 32 && K % DS_CH == 0 && N % DS_CH == 0 && K >= DS_WAVES * DS_CH && N >= DS_WAVES * DS_CH &&
         (int64_t)K * N * 2 < ((int64_t)1 << 31);
}

template <typename T>
hipError_t launch_decode_stream(const T* x, const T* wg, const T* wu, const T* wd, const T* bg,
                                const T* bu, const T* bd, T* h, T* y, int M, int K, int N,
                                int act, hipStream_t s) {
  int dev = 0, num_cu = 0;
  if (hipError_t e = hipGetDevice(&dev)) return e;
  if (hipError_t e = hipDeviceGetAttribute(&num_cu, hipDeviceAttributeMultiprocessorCount, dev)) return e;
  if (num_cu <= 0) num_cu = 256;
  const int tiled = ds_h_tiled(M);
  StreamArgs a1 = {x, {wg, wu}, {bg, bu}, h, M, N, K, K, N, act, tiled};
  StreamArgs a2 = {h, {wd, wd}, {bd, bd}, y, M, K, N, N, K, ACT_IDENTITY, tiled};
  // two runs of W_down rows per token-operand fetch halve the L2 traffic for H; worth it when a
  // CU's share of the rows exceeds one run
  const bool wide = K > 16 * num_cu;
  if (M <= 16) {
    if (hipError_t e = launch_stream<T, true, 2, 1, 512>(a1, num_cu, s)) return e;
    return wide ? launch_stream<T, false, 2, 1, 512>(a2, num_cu, s) : launch_stream<T, false, 1, 1, 512>(a2, num_cu, s);
  }
  // Two token tiles.  With 512-byte row segments the token operands cost as much L2 traffic as
  // the weights cost HBM traffic, and the time grows by about 2 us per token at the 70B widths;
  // 256-byte segments over twice the rows halve that but stream a few per cent slower from HBM.
  // The two cross between M = 20 and M = 24 at every width measured.
  if (M <= DS_WIDE_SEGMENT_MAX_M) {
    if (hipError_t e = launch_stream<T, true, 2, 2, 512>(a1, num_cu, s)) return e;
    return wide ? launch_stream<T, false, 2, 2, 512>(a2, num_cu, s) : launch_stream<T, false, 1, 2, 512>(a2, num_cu, s);
  }
  if (hipError_t e = launch_stream<T, true, 2, 2, 256>(a1, num_cu, s)) return e;
  return wide ? launch_stream<T, false, 2, 2, 256>(a2, num_cu, s) : launch_stream<T, false, 1, 2, 256>(a2, num_cu, s);
}

template hipError_t launch_decode_stream<f16>(const f16*, const f16*, const f16*, const f16*,
                                              const f16*, const f16*, const f16*, f16*, f16*, int,
                                              int, int, int, hipStream_t);
template hipError_t launch_decode_stream<bf16>(const bf16*, const bf16*, const bf16*, const bf16*,
                                               const bf16*, const bf16*, const bf16*, bf16*, bf16*,
                                               int, int, int, int, hipStream_t);

}  // namespace gmlp
