// Large-tile GEMM kernel for gfx950: one wavefront per SIMD, accumulators in the AGPR half of the
// register file, 16-bit operands and outputs.
//
//   C[M,N] = epilogue(A[M,K] * B[N,K]^T)   (both operands K-contiguous, 16-byte aligned, K a multiple of 128 elements)
//
// A workgroup of four wavefronts (2 x 2) owns a 256 x BN tile (BN = 256 or 192); each wavefront owns
// 128 x BN/2 of it: 256 (192) fp32 accumulators per lane, which only fit because a lone wavefront on a
// SIMD may use all 512 registers of a lane.  Per 16 bytes of K a wavefront then reads 0.5 (0.58) LDS
// operand fragments per 32x32 MFMA instead of the 0.75 of the 8-wavefront tiling.
//
// K advances in steps of 128 bytes per row through a two-stage LDS ring filled by
// `buffer_load_dwordx4 ... lds` DMA loads (no VGPR staging).  The workgroup is persistent: it walks a
// list of tiles, and the sequence of (tile, K step) pairs is one flat stream, so that the DMA runs two K
// steps ahead of the MFMAs also across tile boundaries and a tile's epilogue runs with the next tile's
// first K steps already landing in LDS.  The instruction order of a K step is written out MFMA by MFMA
// (LDS reads and DMA loads at fixed slots between the MFMAs, a scheduling fence after each): what
// limits the K loop is how evenly the DMA loads reach the memory pipeline and how long they have to land
// before the stage barrier, not the LDS or the matrix pipe.
//
// The MFMA operands are swapped (the weight fragment is the matrix instruction's A operand), which leaves
// every lane with runs of four consecutive COLUMNS of one output row; one v_permlane32_swap per register
// pairs lanes up so that a lane holds eight consecutive columns.  Bias and activation are applied there,
// the eight values are rounded to the output type and staged, 32 rows at a time, in a strip of LDS private
// to the wavefront (no workgroup barrier), from which they leave as whole 256-byte row segments; stores
// straight from the accumulator layout would touch 32 different rows per instruction.  Epilogues with a
// column pass (V kept transposed by the QKV split) run the tiles of that column range unswapped: a lane
// then holds eight consecutive ROWS of one column, which is what store_col8 wants.
#pragma once

#include <cstdlib>

#include "gemm_impl.h"

namespace ttmi {

typedef float floatx4 __attribute__((ext_vector_type(4)));
// 16 bytes in flight between a global load and its LDS write: a first-class vector value, so that arrays of it
// are promoted to registers.
typedef uint32_t __attribute__((ext_vector_type(4), may_alias)) Quad;
template <int V>
using template_int = std::integral_constant<int, V>;

// One MF x MF block of the output: the matrix instruction and its accumulator.
template <typename T, int MF>
struct MmaBlock;
template <>
struct MmaBlock<f16, 32> {
  using Acc = floatx16;
  static __device__ __forceinline__ void run(const Chunk& a, const Chunk& b, Acc& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, a), __builtin_bit_cast(halfx8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ void run_zero(const Chunk& a, const Chunk& b, Acc& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, a), __builtin_bit_cast(halfx8, b), Acc{}, 0, 0, 0);
  }
};
template <>
struct MmaBlock<bf16, 32> {
  using Acc = floatx16;
  static __device__ __forceinline__ void run(const Chunk& a, const Chunk& b, Acc& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ void run_zero(const Chunk& a, const Chunk& b, Acc& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), Acc{}, 0, 0, 0);
  }
};
template <>
struct MmaBlock<int8_t, 32> {
  using Acc = intx16;
  static __device__ __forceinline__ void run(const Chunk& a, const Chunk& b, Acc& c) {
    c = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(intx4, a), __builtin_bit_cast(intx4, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ void run_zero(const Chunk& a, const Chunk& b, Acc& c) {
    c = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(intx4, a), __builtin_bit_cast(intx4, b), Acc{}, 0, 0, 0);
  }
};
template <>
struct MmaBlock<f16, 16> {
  using Acc = floatx4;
  // Written as an instruction with the accumulator pinned to the AGPR half ("+a"): through the builtin the compiler
  // keeps part of the 192 accumulator registers of the 16-wide blocks in ordinary registers and moves them back and
  // forth around every matrix instruction (two copies per MFMA in the K loop).
  static __device__ __forceinline__ void run(const Chunk& a, const Chunk& b, Acc& c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(__builtin_bit_cast(halfx8, a)), "v"(__builtin_bit_cast(halfx8, b)));
  }
  // The first product of a tile: C = A.B with the constant 0 as the addend, so the accumulator is only written.
  // Zeroing it beforehand would cost a register write per accumulator, and (the matrix instruction being inline asm)
  // the compiler does not know to keep the wait states between such a write and the instruction that reads it.
  static __device__ __forceinline__ void run_zero(const Chunk& a, const Chunk& b, Acc& c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(c) : "v"(__builtin_bit_cast(halfx8, a)), "v"(__builtin_bit_cast(halfx8, b)));
  }
};
template <>
struct MmaBlock<bf16, 16> {
  using Acc = floatx4;
  // Written as an instruction with the accumulator pinned to the AGPR half ("+a"): through the builtin the compiler
  // keeps part of the 192 accumulator registers of the 16-wide blocks in ordinary registers and moves them back and
  // forth around every matrix instruction (two copies per MFMA in the K loop).
  static __device__ __forceinline__ void run(const Chunk& a, const Chunk& b, Acc& c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(__builtin_bit_cast(bf16x8, a)), "v"(__builtin_bit_cast(bf16x8, b)));
  }
  static __device__ __forceinline__ void run_zero(const Chunk& a, const Chunk& b, Acc& c) {  // see the fp16 form
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(c) : "v"(__builtin_bit_cast(bf16x8, a)), "v"(__builtin_bit_cast(bf16x8, b)));
  }
};
template <>
struct MmaBlock<int8_t, 16> {
  using Acc = intx4;
  static __device__ __forceinline__ void run(const Chunk& a, const Chunk& b, Acc& c) {
    c = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(intx4, a), __builtin_bit_cast(intx4, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ void run_zero(const Chunk& a, const Chunk& b, Acc& c) {
    c = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(intx4, a), __builtin_bit_cast(intx4, b), Acc{}, 0, 0, 0);
  }
};

// Lanes of the lower half of each lane pair (MF = 32: lanes 0..31 with 32..63; MF = 16: 16-lane rows 0 with 1,
// 2 with 3) keep `a` and receive the partner's `a` in `b`; the upper ones keep `b` and receive the partner's `b`
// in `a`.  Afterwards {a, b} of every lane are neighbours in the output.
template <int MF, typename S>
__device__ __forceinline__ void pair_swap(S& a, S& b) {
  static_assert(sizeof(S) == 4, "one register");
#if defined(__HIP_DEVICE_COMPILE__)
  const unsigned ua = __builtin_bit_cast(unsigned, a), ub = __builtin_bit_cast(unsigned, b);
  if constexpr (MF == 32) {
    const auto r = __builtin_amdgcn_permlane32_swap(ua, ub, false, false);
    a = __builtin_bit_cast(S, (unsigned)r[0]);
    b = __builtin_bit_cast(S, (unsigned)r[1]);
  } else {
    const auto r = __builtin_amdgcn_permlane16_swap(ua, ub, false, false);
    a = __builtin_bit_cast(S, (unsigned)r[0]);
    b = __builtin_bit_cast(S, (unsigned)r[1]);
  }
#endif
}

// One accumulator register into an ordinary one, here and now: without it the compiler copies every accumulator of a
// tile out of the AGPR half at the end of the K loop, 192 or 256 live registers at once.
template <typename S>
__device__ __forceinline__ S acc_read(S v) {
  S r;
  asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(r) : "a"(v));
  return r;
}

// 16 bytes into the wavefront's own epilogue strip.  Written as an instruction rather than as a C++ store: with
// global->LDS DMA loads in flight (the next tile's first K steps) the compiler guards every LDS store it knows of
// with a wait for ALL outstanding vector memory operations, i.e. also for the global stores of the previous row
// block, one HBM round trip per block.  The strip is disjoint from the DMA stages, and LDS operations of one
// wavefront complete in order, so the reads that follow need no more than their usual counter wait.
__device__ __forceinline__ void strip_write(uint32_t lds_addr, Quad x) {
  asm volatile("ds_write_b128 %0, %1" : : "v"(lds_addr), "v"(x) : "memory");
}

// Bias of eight consecutive columns, kept in storage precision (16 bytes for 2-byte types) until it is added.
template <typename BT>
struct BiasVec {
  static constexpr int kPer = 16 / sizeof(BT), kChunksPerVec = 8 / kPer;
  Chunk raw[kChunksPerVec];
  bool present;
  // `fallback`: any readable, 16-byte aligned address with 32 bytes behind it.  Without a bias the loads go there
  // (and are ignored): a load under a branch would be waited for at the end of its block, one round trip each.
  __device__ __forceinline__ void load(const BT* bias, int ncol, const void* fallback) {
    present = bias != nullptr;
    const BT* src = present ? bias + ncol : static_cast<const BT*>(fallback);
#pragma unroll
    for (int c = 0; c < kChunksPerVec; ++c) raw[c] = *reinterpret_cast<const Chunk*>(src + c * kPer);
  }
  __device__ __forceinline__ void widen(float (&out)[8]) const {
#pragma unroll
    for (int c = 0; c < kChunksPerVec; ++c) {
      const Vec<BT, kPer> v = __builtin_bit_cast(Vec<BT, kPer>, raw[c]);
#pragma unroll
      for (int e = 0; e < kPer; ++e) out[c * kPer + e] = to_float(v.v[e]);
    }
  }
  template <typename S>
  __device__ __forceinline__ void add_to(S (&out)[8]) const {
    if (!present) return;
#pragma unroll
    for (int c = 0; c < kChunksPerVec; ++c) {
      const Vec<BT, kPer> v = __builtin_bit_cast(Vec<BT, kPer>, raw[c]);
#pragma unroll
      for (int e = 0; e < kPer; ++e) out[c * kPer + e] += (S)to_float(v.v[e]);
    }
  }
};

constexpr int kW4Threads = 256;
// Block size of the matrix instruction the launchers use: 16 (v_mfma_f32_16x16x32) moves a quarter of the accumulator
// bits per FLOP of the 32x32x16 form, and on a chip that runs its matrix loops at the power limit that is clock rate:
// the same K loop runs 5-10 % faster with it.
constexpr int kW4Block = 16;

// Epilogues whose output is one row-major matrix: base address and leading dimension, so that the kernel can
// store through a buffer resource (32-bit offsets; rows past M are predicated off by the kernel itself).
template <typename Epi>
struct LinearDest : std::false_type {
  static __device__ __forceinline__ void* base(const Epi&) { return nullptr; }
  static __device__ __forceinline__ int64_t ldc(const Epi&) { return 0; }
};
template <typename T, int ACT, bool HAS_ACT>
struct LinearDest<EpiBias<T, ACT, HAS_ACT, false>> : std::true_type {
  static __device__ __forceinline__ void* base(const EpiBias<T, ACT, HAS_ACT, false>& e) { return e.c; }
  static __device__ __forceinline__ int64_t ldc(const EpiBias<T, ACT, HAS_ACT, false>& e) { return e.ldc; }
};
template <typename T>
struct LinearDest<EpiAlphaBeta<T>> : std::true_type {
  static __device__ __forceinline__ void* base(const EpiAlphaBeta<T>& e) { return e.c; }
  static __device__ __forceinline__ int64_t ldc(const EpiAlphaBeta<T>& e) { return e.ldc; }
};

#ifdef TTMI_W4_TRACE
__device__ unsigned long long w4_trace[4][16][8][2];
#define W4_STAMP(slot)                                                                    \
  if (blockIdx.x == TTMI_W4_TRACE && lane == 0 && t < 16) {                               \
    w4_trace[wave][t][slot][0] = __builtin_readcyclecounter();                            \
    w4_trace[wave][t][slot][1] = wall_clock64();                                          \
  }
#else
#define W4_STAMP(slot)
#endif

// LDS of the kernel: two K-loop stages plus one private epilogue strip per wavefront (MF rows x BN/2 columns of
// the 2-byte output type; rows padded by 16 bytes when that does not fit a power-of-two swizzle).
template <int BN, int MF>
constexpr int w4_strip_pitch() { return BN == 256 ? 256 : BN + 16; }  // bytes per staged row (BN/2 columns of 2 bytes)
// AS = stages of the A operand's ring (B always has two).  With three, the epilogue strips hold 16 rows instead of 32
// so that everything still fits the 160 KB of a CU.
// DIRECT: no strips at all (row-major outputs stored straight from the accumulator layout).
template <int BN, int MF, int AS = 2, bool DIRECT = false>
constexpr int w4_lds_bytes() {
  return (AS * 256 + 2 * BN) * kRowBytes + (DIRECT ? 0 : 4 * (AS == 3 ? 16 : 32) * w4_strip_pitch<BN, MF>());
}

// What the kernel needs from an epilogue besides bias_ptr(): finish(x) applied to acc + bias in fp32, and
// dest8(m, n), the address of the 16 bytes that hold columns n..n+7 of output row m.
//
// AS = 3: the A operand (the activations: the matrix that comes from HBM or the memory-side cache, while the weights
// stay in L2) gets a THIRD stage, so that its DMA loads are issued two K steps before the barrier that waits for them
// instead of one.  With two stages a load has between half a K step and one K step (0.6-1.3 us) to land, which is
// what an L2 hit takes and less than a fetch from HBM: the product whose A operand does not fit the memory-side
// cache (the second FFN product: 201 MB) ran 20 % slower inside the forward than on a cache-resident operand.
// The loads of a K step go out B first, A last; loads of one wavefront return in order, so the barrier waits for
// all but the A_LOADS youngest (vmcnt(A_LOADS)): the weights of the next step and the activations of the next step
// have landed, the activations of the step after it may still be in flight.  Global STORES return out of order with
// loads, so the first barrier of a tile, which may still have the previous tile's stores in flight, waits for
// everything.  Epilogues with a column pass keep two stages (their transposed unit needs the larger strip).
// DIRECT: a row-major 16-bit output leaves straight from the accumulator layout, without the trip through a strip: after
// the pair swap a lane holds 16 contiguous bytes of one row and the four lanes that share a row 64 contiguous bytes
// between them, so a store instruction writes sixteen 64-byte segments instead of four 256-byte ones, and the LDS
// round trip and its waits are gone.  The launcher uses it for the 256-wide tile (measured 1 % faster on the whole
// BERT-base forward there, level at 192 wide), where the freed LDS also makes room for the third A stage.
template <typename T, int BN, int MF, typename Epi, int AS = 2, bool DIRECT = false>
__global__ __launch_bounds__(kW4Threads) void gemm_w4_kernel(const GemmArgs g, const Epi epi) {
  static_assert(!DIRECT || ((LinearDest<Epi>::value || HasColumnPass<Epi>::value) && MF == 16),
                "direct stores: row-major 16-bit outputs or the head split, 16-wide blocks");
  static_assert(sizeof(T) == 2, "16-bit operands");
  static_assert(MF == 32 || MF == 16, "block sizes of the matrix instructions");
  static_assert(AS == 2 || (AS == 3 && MF == 16 && !HasColumnPass<Epi>::value), "three A stages: 16-wide blocks, row-major epilogues");
  constexpr int BM = 256;
  constexpr int BK = kRowBytes / sizeof(T);
  constexpr int RB = 128 / MF, CB = BN / 2 / MF;   // blocks per wavefront: rows, columns
  constexpr int SUB = MF == 32 ? 4 : 2;            // K substeps per 128-byte K step
  constexpr int CPS = kChunks / SUB;               // 16-byte chunks of a row per substep; lane / MF picks one
  constexpr int ACC = MF * MF / kWave;             // accumulator registers per block
  constexpr int A_BYTES = BM * kRowBytes, B_BYTES = BN * kRowBytes, STAGE = A_BYTES + B_BYTES;
  constexpr int A_LOADS = BM / 8 / 4, B_LOADS = BN / 8 / 4;  // 16-byte loads per lane and K step
  constexpr int LOADS = A_LOADS + B_LOADS;
  constexpr int PITCH = w4_strip_pitch<BN, MF>(), CPR = BN / 2 / 8;  // staged row: bytes, 16-byte chunks
  constexpr bool XOR_STRIP = (CPR & (CPR - 1)) == 0;
  static_assert(BN % (2 * MF) == 0 && BN % 32 == 0, "tile width");
  static_assert(CB % 2 == 0 || MF == 32, "16-wide blocks are stored in pairs");
  static_assert(A_LOADS % 2 == 0 && B_LOADS % 2 == 0, "the LDS swizzle of a load depends on its parity only");
  using MB = MmaBlock<T, MF>;
  using Acc = typename MB::Acc;

  extern __shared__ __align__(16) char smem[];

  // Tiles of this workgroup: XCD x owns [x*per_xcd, (x+1)*per_xcd); its workgroups stride through it together.
  // K slices (fp32 outputs only): with g.k_chunk > 0 the work items are (slice, tile) pairs, slice-major; slice z
  // multiplies columns [z*k_chunk, (z+1)*k_chunk) of both operands and stores its partial product as rows
  // [z*M, (z+1)*M) of the output, for a reduction pass to sum.
  const int tiles_mn = g.tiles_m * g.tiles_n;
  int slices = 1;
  if constexpr (StoresF32<Epi>::value) {
    if (g.k_chunk > 0) slices = g.k / g.k_chunk;
  }
  const int tiles = tiles_mn * slices;
  auto locate = [&](int item, int& tile_m, int& tile_n) __attribute__((always_inline)) {
    int z = 0;
    if constexpr (StoresF32<Epi>::value) {
      if (slices > 1) {
        z = item / tiles_mn;
        item -= z * tiles_mn;
      }
    }
    tile_coords(item, g.tiles_m, g.tiles_n, tile_m, tile_n);
    return z;
  };
  const int per_xcd = (tiles + kNumXcd - 1) / kNumXcd;
  const int xcd = (int)(blockIdx.x % kNumXcd), stride = (int)(gridDim.x / kNumXcd);
  const int xcd_end = min((xcd + 1) * per_xcd, tiles);
  const int first = xcd * per_xcd + (int)(blockIdx.x / kNumXcd);
  if (first >= xcd_end) return;
  const int my_tiles = (xcd_end - first + stride - 1) / stride;
  const int ksteps = (slices > 1 ? g.k_chunk : g.k) / BK;  // even (checked by the launcher)
  const uint32_t slice_bytes = (uint32_t)g.k_chunk * (uint32_t)sizeof(T);  // K offset of slice 1 inside an operand row
  const int total_steps = my_tiles * ksteps;

  const int64_t lda_bytes = g.lda * (int64_t)sizeof(T), ldb_bytes = g.ldb * (int64_t)sizeof(T);

  const int tid = threadIdx.x;
  const int lane = tid % kWave, wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm0 = (wave / 2) * 128, wn0 = (wave % 2) * (BN / 2);
  const int lrow = lane % MF, lgrp = lane / MF;
  // LDS: [A stage 0 .. AS-1][B stage 0][B stage 1][epilogue strips]; the stage of an operand is an immediate offset
  // (with three A stages the A stage is a run-time offset)
  const int a_row0 = (wm0 + lrow) * kRowBytes, b_row0 = AS * A_BYTES + (wn0 + lrow) * kRowBytes;
  const int swz = (lrow >> 1) & 7;

  // ---- DMA cursor.  `buffer_load_dwordx4 ... lds` copies 8 tile rows (64 lanes x 16 bytes) straight into LDS; the
  //      LDS side is linear in the lane id, so the XOR swizzle is applied on the global side: lane l fills physical
  //      chunk l%8 of row l/8 and therefore fetches logical chunk (l%8) ^ ((row>>1)&7).  The LOADS loads of one K
  //      step are not issued as a burst: the memory pipeline takes about 20 cycles per load and serves the four
  //      wavefronts in turn, and a wavefront that finds its queue full stops issuing MFMAs.
  // first column of tile column tile_n: a second run of tiles may start at g.split_col (see GemmArgs)
  auto first_column = [&](int tile_n) __attribute__((always_inline)) {
    return tile_n < g.split_tiles ? tile_n * BN : g.split_col + (tile_n - g.split_tiles) * BN;
  };
  int dma_step = 0, dma_k = 0, dma_tile = first;
  uint32_t voa[A_LOADS], vob[B_LOADS];  // per-lane byte offsets from the tile's first row (row clamp and swizzle inside)
  uint32_t a_soff = 0, b_soff = 0;  // byte offset of the cursor's tile in A and in B (matrices below 2 GiB, checked by the launcher)
  auto dma_point = [&](int tile) __attribute__((always_inline)) {
    int tile_m, tile_n;
    const int z = locate(tile, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = first_column(tile_n);
    const int sub = lane >> 3, p = lane & 7;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int row = (wave * A_LOADS + i) * 8 + sub;
      voa[i] = (uint32_t)(min(m0 + row, g.m - 1) - m0) * (uint32_t)lda_bytes + ((p ^ ((row >> 1) & 7)) << 4);
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      const int row = (wave * B_LOADS + i) * 8 + sub;
      vob[i] = (uint32_t)(min(n0 + row, g.n - 1) - n0) * (uint32_t)ldb_bytes + ((p ^ ((row >> 1) & 7)) << 4);
    }
    a_soff = (uint32_t)m0 * (uint32_t)lda_bytes + (uint32_t)z * slice_bytes;
    b_soff = (uint32_t)n0 * (uint32_t)ldb_bytes + (uint32_t)z * slice_bytes;
  };
  // load i of K step `dma_step` into stage dma_step & 1
#if defined(__HIP_DEVICE_COMPILE__)
  typedef __attribute__((address_space(3))) char lds_char;
  lds_char* lds0 = reinterpret_cast<lds_char*>(reinterpret_cast<uintptr_t>(smem));
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(g.a), 0, (int)min((int64_t)g.m * lda_bytes, (int64_t)0x7fffffff), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(g.b), 0, (int)min((int64_t)g.n * ldb_bytes, (int64_t)0x7fffffff), 0x00020000);
  auto dma_issue_one = [&](int i) __attribute__((always_inline)) {
    if (i < A_LOADS) {
      lds_char* as = lds0 + (dma_step & 1) * A_BYTES + wave * (A_LOADS * 1024);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, as + i * 1024, 16, voa[i], a_soff + dma_k * kRowBytes, 0, 0);
    } else {
      lds_char* bs = lds0 + AS * A_BYTES + (dma_step & 1) * B_BYTES + wave * (B_LOADS * 1024);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, bs + (i - A_LOADS) * 1024, 16, vob[i - A_LOADS], b_soff + dma_k * kRowBytes, 0, 0);
    }
  };
  // the output matrix of a linear epilogue (the resource ends at row M; the stores are predicated on the row as well)
  const uint32_t ldc_bytes = (uint32_t)LinearDest<Epi>::ldc(epi) * (uint32_t)sizeof(T);
  const __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(LinearDest<Epi>::base(epi), 0, (int)min((int64_t)g.m * ldc_bytes, (int64_t)0x7fffffff), 0x00020000);
  auto store_c = [&](Quad x, uint32_t voff, uint32_t soff) __attribute__((always_inline)) {
    __builtin_amdgcn_raw_buffer_store_b128(x, rsrc_c, (int)voff, (int)soff, 0);
  };
  // direct stores of the head split: one resource per destination tensor, each [B, heads, S, d] = M x hidden elements
  // (the launcher checks that this is below 2 GiB and that 16 consecutive rows share a sequence)
  auto head_split_store = [&](Quad x, int which, uint32_t voff, uint32_t soff) __attribute__((always_inline)) {
    if constexpr (DIRECT && HasColumnPass<Epi>::value) {
      T* base = which == 0 ? epi.q : (which == 1 ? epi.k : epi.v);
      const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(base, 0, (int)((int64_t)g.m * epi.hidden * (int64_t)sizeof(T)), 0x00020000);
      __builtin_amdgcn_raw_buffer_store_b128(x, rsrc, (int)voff, (int)soff, 0);
    }
  };
#else
  auto head_split_store = [&](Quad, int, uint32_t, uint32_t) {};
  auto dma_issue_one = [&](int) {};
  const uint32_t ldc_bytes = 0;
  auto store_c = [&](Quad, uint32_t, uint32_t) {};
#endif
  auto dma_issue = [&](auto lo_tag, auto hi_tag) __attribute__((always_inline)) {
    constexpr int LO = decltype(lo_tag)::value, HI = decltype(hi_tag)::value;
#pragma unroll
    for (int i = LO; i < HI; ++i) dma_issue_one(i);
  };
  // Move the cursor to the next K step of the flat sequence.  Past its end it stays on the last step: the surplus
  // loads at the end of the kernel re-fetch that step into stages nobody reads any more.
  auto dma_advance = [&]() __attribute__((always_inline)) {
    ++dma_step;
    if (dma_step < total_steps && ++dma_k == ksteps) {
      dma_k = 0;
      dma_tile += stride;
      dma_point(dma_tile);
    }
  };

  // ---- three A stages: one cursor per operand; the A cursor runs one K step ahead of the B cursor.  (voa / vob and
  //      a_soff / b_soff above are then maintained by these, each at its own pace.)
  int a_step = 0, a_k = 0, a_tile = first, a_st = 0;  // a_st = a_step % 3: the stage the cursor's step is loaded into
  int b_step = 0, b_k = 0, b_tile = first;
  auto a_point = [&](int tile) __attribute__((always_inline)) {
    int tile_m, tile_n;
    const int z = locate(tile, tile_m, tile_n);
    const int m0 = tile_m * BM;
    const int sub = lane >> 3, p = lane & 7;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int row = (wave * A_LOADS + i) * 8 + sub;
      voa[i] = (uint32_t)(min(m0 + row, g.m - 1) - m0) * (uint32_t)lda_bytes + ((p ^ ((row >> 1) & 7)) << 4);
    }
    a_soff = (uint32_t)m0 * (uint32_t)lda_bytes + (uint32_t)z * slice_bytes;
  };
  auto b_point = [&](int tile) __attribute__((always_inline)) {
    int tile_m, tile_n;
    const int z = locate(tile, tile_m, tile_n);
    const int n0 = first_column(tile_n);
    const int sub = lane >> 3, p = lane & 7;
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      const int row = (wave * B_LOADS + i) * 8 + sub;
      vob[i] = (uint32_t)(min(n0 + row, g.n - 1) - n0) * (uint32_t)ldb_bytes + ((p ^ ((row >> 1) & 7)) << 4);
    }
    b_soff = (uint32_t)n0 * (uint32_t)ldb_bytes + (uint32_t)z * slice_bytes;
  };
#if defined(__HIP_DEVICE_COMPILE__)
  // load i of the split cursors: 0 .. B_LOADS-1 are the B loads (issued first), the rest the A loads
  auto split_issue_one = [&](int i) __attribute__((always_inline)) {
    if (i < B_LOADS) {
      lds_char* bs = lds0 + AS * A_BYTES + (b_step & 1) * B_BYTES + wave * (B_LOADS * 1024);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, bs + i * 1024, 16, vob[i], b_soff + b_k * kRowBytes, 0, 0);
    } else {
      lds_char* as = lds0 + a_st * A_BYTES + wave * (A_LOADS * 1024);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, as + (i - B_LOADS) * 1024, 16, voa[i - B_LOADS], a_soff + a_k * kRowBytes, 0, 0);
    }
  };
#else
  auto split_issue_one = [&](int) {};
#endif
  auto a_advance = [&]() __attribute__((always_inline)) {
    ++a_step;
    a_st = a_st == 2 ? 0 : a_st + 1;
    if (a_step < total_steps && ++a_k == ksteps) {
      a_k = 0;
      a_tile += stride;
      a_point(a_tile);
    }
  };
  auto b_advance = [&]() __attribute__((always_inline)) {
    ++b_step;
    if (b_step < total_steps && ++b_k == ksteps) {
      b_k = 0;
      b_tile += stride;
      b_point(b_tile);
    }
  };

  Chunk fa[2][RB], fb[2][CB];
  auto read_frags = [&](int stage, int sub, Chunk (&a)[RB], Chunk (&b)[CB]) __attribute__((always_inline)) {
    const int off = ((sub * CPS + lgrp) ^ swz) << 4;
#pragma unroll
    for (int i = 0; i < RB; ++i) a[i] = *reinterpret_cast<const Chunk*>(smem + (a_row0 + off) + (stage * A_BYTES + i * MF * kRowBytes));
#pragma unroll
    for (int j = 0; j < CB; ++j) b[j] = *reinterpret_cast<const Chunk*>(smem + (b_row0 + off) + (stage * B_BYTES + j * MF * kRowBytes));
  };

  Acc acc[RB][CB];
  // SWAP: the weight fragment is the instruction's A operand -> a lane owns one output ROW of a block.
  // One substep in exact instruction order: MFMA m of this substep, then LDS read m of the next one (m < READS, so
  // the reads have landed long before their use and before the barrier), then a DMA load when m is one of NL evenly
  // spaced slots (the memory pipeline takes about 20 cycles per DMA load and serves the four wavefronts in turn: a
  // wavefront that issues them faster than one per three MFMAs blocks at the queue with the matrix pipe idle).
  // A scheduling fence after every MFMA keeps the compiler from regrouping them.
  // rd_stage/rd_sub: what the reads fetch; DLO: index of the first DMA load issued here.
  constexpr int READS = RB + CB, MMAS = RB * CB;
  auto substep = [&](auto swap_tag, auto cur_tag, auto rd_stage_tag, auto rd_sub_tag, auto dlo_tag, auto nl_tag, auto ext_tag, auto zero_tag) __attribute__((always_inline)) {
    constexpr bool SWAP = decltype(swap_tag)::value;
    constexpr bool ZERO = decltype(zero_tag)::value;  // first substep of a tile: the accumulators are written, not added to
    constexpr int CUR = decltype(cur_tag)::value, RS = decltype(rd_stage_tag)::value, RSUB = decltype(rd_sub_tag)::value;
    constexpr int DLO = decltype(dlo_tag)::value, NL = decltype(nl_tag)::value, EXT = decltype(ext_tag)::value;  // NL loads over the first EXT MFMAs
    static_assert(NL <= EXT && EXT <= MMAS, "at most one DMA load per MFMA");
    const int off = ((RSUB * CPS + lgrp) ^ swz) << 4;
#pragma unroll
    for (int m = 0; m < MMAS; ++m) {
      const int i = m / CB, j = m % CB;
      if constexpr (ZERO) {
        if constexpr (SWAP) MB::run_zero(fb[CUR][j], fa[CUR][i], acc[i][j]);
        else MB::run_zero(fa[CUR][i], fb[CUR][j], acc[i][j]);
      } else {
        if constexpr (SWAP) MB::run(fb[CUR][j], fa[CUR][i], acc[i][j]);
        else MB::run(fa[CUR][i], fb[CUR][j], acc[i][j]);
      }
      if (m < RB) fa[CUR ^ 1][m] = *reinterpret_cast<const Chunk*>(smem + (a_row0 + off) + (RS * A_BYTES + m * MF * kRowBytes));
      else if (m < READS) fb[CUR ^ 1][m - RB] = *reinterpret_cast<const Chunk*>(smem + (b_row0 + off) + (RS * B_BYTES + (m - RB) * MF * kRowBytes));
      if (NL > 0 && m < EXT && ((m + 1) * NL) / EXT != (m * NL) / EXT) dma_issue_one(DLO + (m * NL) / EXT);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // How the LOADS loads of one K step are spread: D3 behind the barrier of step s, D0 and D1 in the first two
  // substeps of step s+1; the substep in front of the barrier issues none, so that every load has at least a
  // substep to land.  (SUB = 2: the barrier sits between the two substeps and all loads follow it.)
  constexpr int D3 = SUB == 4 ? LOADS / 2 : LOADS;
  constexpr int D0 = SUB == 4 ? LOADS - D3 : 0;
  constexpr int D1 = 0;
  constexpr int EXT1 = 1;
  static_assert(D3 + D0 + D1 == LOADS && D3 >= 0, "every load of a K step is issued once");
  template_int<0> I0;

  // One K step.  P = parity of the step = its LDS stage.
  // zero_tag: the first K step of a tile (its first substep writes the accumulators instead of adding to them)
  auto k_step = [&](auto parity_tag, auto swap_tag, auto zero_tag) __attribute__((always_inline)) {
    constexpr int P = decltype(parity_tag)::value;
    std::false_type no;
    if constexpr (SUB == 4) {
      substep(swap_tag, template_int<0>{}, template_int<P>{}, template_int<1>{}, template_int<D3>{}, template_int<D0>{}, template_int<MMAS>{}, zero_tag);
      substep(swap_tag, template_int<1>{}, template_int<P>{}, template_int<2>{}, template_int<D3 + D0>{}, template_int<D1>{}, template_int<EXT1>{}, no);
      dma_advance();
      __builtin_amdgcn_sched_barrier(0);
      substep(swap_tag, template_int<0>{}, template_int<P>{}, template_int<3>{}, I0, I0, template_int<MMAS>{}, no);
    } else {
      substep(swap_tag, template_int<0>{}, template_int<P>{}, template_int<1>{}, I0, I0, template_int<MMAS>{}, zero_tag);
      dma_advance();
      __builtin_amdgcn_sched_barrier(0);
    }
    // everyone has read all of this stage (the last reads were issued half a substep ago); the other stage has landed
    dma_landed_barrier();
    __builtin_amdgcn_sched_barrier(0);
    substep(swap_tag, template_int<1>{}, template_int<P ^ 1>{}, template_int<0>{}, I0, template_int<D3>{}, template_int<MMAS>{}, no);
  };

  // ---- the same with three A stages (16-wide blocks, operands swapped).  a_rd: byte offset of the A stage that is
  //      read.  ISSUE: the LOADS loads of the split cursors go out, evenly spread over the substep, B first.
  auto substep3 = [&](auto cur_tag, auto rd_bstage_tag, auto rd_sub_tag, auto issue_tag, auto zero_tag, int a_rd) __attribute__((always_inline)) {
    constexpr int CUR = decltype(cur_tag)::value, RSB = decltype(rd_bstage_tag)::value, RSUB = decltype(rd_sub_tag)::value;
    constexpr bool ISSUE = decltype(issue_tag)::value, ZERO = decltype(zero_tag)::value;
    const int off = ((RSUB * CPS + lgrp) ^ swz) << 4;
    const int a_base = a_row0 + off + a_rd;
#pragma unroll
    for (int m = 0; m < MMAS; ++m) {
      const int i = m / CB, j = m % CB;
      if constexpr (ZERO) MB::run_zero(fb[CUR][j], fa[CUR][i], acc[i][j]);
      else MB::run(fb[CUR][j], fa[CUR][i], acc[i][j]);
      if (m < RB) fa[CUR ^ 1][m] = *reinterpret_cast<const Chunk*>(smem + a_base + m * MF * kRowBytes);
      else if (m < READS) fb[CUR ^ 1][m - RB] = *reinterpret_cast<const Chunk*>(smem + (b_row0 + off) + (RSB * B_BYTES + (m - RB) * MF * kRowBytes));
      if (ISSUE && ((m + 1) * LOADS) / MMAS != (m * LOADS) / MMAS) split_issue_one((m * LOADS) / MMAS);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  int a_cur = 0;  // stage (0..2) of the A operand of the K step being multiplied
  auto k_step3 = [&](auto parity_tag, auto full_tag) __attribute__((always_inline)) {
    constexpr int P = decltype(parity_tag)::value;
    constexpr bool FULL = decltype(full_tag)::value;
    // FULL = the first K step of a tile: its first substep also writes the accumulators instead of adding to them
    substep3(template_int<0>{}, template_int<P>{}, template_int<1>{}, std::false_type{}, full_tag, a_cur * A_BYTES);
    a_advance();
    b_advance();
    __builtin_amdgcn_sched_barrier(0);
    // everyone has read all of this step's stages; the next step's operands have landed, the A loads of the step
    // after it (the A_LOADS youngest of this wavefront) may still be in flight
    if constexpr (FULL) dma_landed_barrier();
    else dma_landed_barrier_but<A_LOADS>();
    __builtin_amdgcn_sched_barrier(0);
    a_cur = a_cur == 2 ? 0 : a_cur + 1;
    substep3(template_int<1>{}, template_int<P ^ 1>{}, template_int<0>{}, std::true_type{}, std::false_type{}, a_cur * A_BYTES);
  };
  auto read_frags3 = [&](int a_rd) __attribute__((always_inline)) {  // sub 0 of (A stage at a_rd, B stage 0)
    const int off = (lgrp ^ swz) << 4;
#pragma unroll
    for (int i = 0; i < RB; ++i) fa[0][i] = *reinterpret_cast<const Chunk*>(smem + (a_row0 + off + a_rd) + i * MF * kRowBytes);
#pragma unroll
    for (int j = 0; j < CB; ++j) fb[0][j] = *reinterpret_cast<const Chunk*>(smem + (b_row0 + off) + j * MF * kRowBytes);
  };

  if constexpr (AS == 3) {
    // ---- prologue: A steps 0 and 1 and B step 0 land; B step 1 and A step 2 are under way ----
    a_point(a_tile);
    b_point(b_tile);
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) split_issue_one(B_LOADS + i);
    a_advance();
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) split_issue_one(B_LOADS + i);
    a_advance();
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) split_issue_one(i);
    b_advance();
    dma_landed_barrier();
#pragma unroll
    for (int i = 0; i < LOADS; ++i) split_issue_one(i);
    read_frags3(0);
  } else {
  // ---- prologue: K step 0 lands, the first loads of K step 1 are under way ----
  dma_point(dma_tile);
  dma_issue(std::integral_constant<int, 0>{}, std::integral_constant<int, LOADS>{});
  dma_advance();
  dma_landed_barrier();
  dma_issue(std::integral_constant<int, 0>{}, std::integral_constant<int, D3>{});
  read_frags(0, 0, fa[0], fb[0]);
  }

  constexpr int STRIP_ROWS = AS == 3 ? 16 : 32;
  char* strip = smem + AS * A_BYTES + 2 * B_BYTES + wave * (STRIP_ROWS * PITCH);
  const uint32_t strip_lds = (uint32_t)reinterpret_cast<uintptr_t>(strip);  // low half of a generic LDS address = LDS offset
  int tile = first;
  for (int t = 0; t < my_tiles; ++t, tile += stride) {
    int tile_m, tile_n;
    const int slice = locate(tile, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = first_column(tile_n);
    bool swap = true;
    if constexpr (HasColumnPass<Epi>::value) swap = !(epi.column_pass() && n0 >= epi.first_column_of_pass());
    W4_STAMP(0)

    // Three A stages: no zeroing, the first substep of the tile writes the accumulators.  Two stages: zeroed here
    // (peeling the first K step off the loop for a zero-addend form costs this variant twenty registers, which its
    // 256-wide forms do not have).  The matrix instructions are inline asm, so the compiler does not know to keep the
    // wait states between these register writes and the instruction that reads them as its addend: every accumulator
    // is pinned as written (an empty asm that names it) before a pause that covers the distance.
    if constexpr (AS != 3) {
#pragma unroll
      for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int j = 0; j < CB; ++j)
#pragma unroll
          for (int e = 0; e < ACC; ++e) acc[i][j][e] = 0;
      // (not in the head-split kernels: pinned, they spill 0.7-1.3 KB of registers per lane; their zeroing stays
      // where the compiler puts it, which the bit-exact parity tests of those kernels watch)
      if constexpr (!HasColumnPass<Epi>::value) {
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
          for (int j = 0; j < CB; ++j) asm volatile("" : "+a"(acc[i][j]));
        asm volatile("s_nop 7");
      }
    }
    const auto* bias = epi.bias_ptr();
    using BiasT = typename std::remove_cv<typename std::remove_pointer<decltype(bias)>::type>::type;
    const int m_lim = g.m, n_lim = tile_n < g.split_tiles ? g.split_col : g.n;  // a tile in front of the split ends there
    // bias of this lane's column groups, requested now so that it has landed when the epilogue wants it
    // The epilogue works on groups of GROUP rows; a lane contributes NV units of eight consecutive columns to each.
    // MF = 32: unit v = (block column v/2, half v%2 of its 32 columns), the lane's row is lrow.  MF = 16: unit v =
    // (16-row block v / (CB/2) of the group, pair of block columns v % (CB/2)), the lane's row is 16*(v / (CB/2)) + lrow.
    // (the widest tile of the 16-wide blocks stages 16 rows at a time: half the registers for the staged pieces, which
    // its head-split epilogue does not have to spare)
    constexpr int GROUP = (AS == 3 || (MF == 16 && BN > 192)) ? 16 : 32;
    constexpr int NV = MF == 32 ? CB * 2 : (GROUP == 32 ? CB : CB / 2);
    constexpr int NBV = MF == 32 ? NV : CB / 2;  // distinct column groups among the units (= bias vectors to hold)
    auto unit_chunk = [&](int v) __attribute__((always_inline)) {  // which group of eight columns of the wavefront's BN/2
      if constexpr (MF == 32) return (v / 2) * 4 + (v % 2) * 2 + lgrp;
      else return 2 * (2 * (v % (CB / 2)) + (lgrp & 1)) + (lgrp >> 1);
    };
    BiasVec<BiasT> bv[NBV];
    if (swap) {
#pragma unroll
      for (int v = 0; v < NBV; ++v) bv[v].load(bias, min(n0 + wn0 + unit_chunk(v) * 8, n_lim - 8), g.b);  // N % 8 == 0
    }
    W4_STAMP(1)
    if (swap) {
      // three A stages: the first two K steps apart; the very first substep writes the accumulators, and the first
      // barrier of a tile, which may have the previous tile's stores in flight, waits for everything
      if constexpr (AS == 3) {
        k_step3(template_int<0>{}, std::true_type{});
        k_step3(template_int<1>{}, std::false_type{});
      }
      for (int kt = AS == 3 ? 2 : 0; kt < ksteps; kt += 2) {
        if constexpr (AS == 3) {
          k_step3(template_int<0>{}, std::false_type{});
          k_step3(template_int<1>{}, std::false_type{});
        } else {
          k_step(std::integral_constant<int, 0>{}, std::true_type{}, std::false_type{});
          k_step(std::integral_constant<int, 1>{}, std::true_type{}, std::false_type{});
        }
      }
      W4_STAMP(2)
      // A lane now owns, per block, runs of four consecutive columns of one row; a pair swap makes them runs of
      // eight: + bias, finish(), round to T, 16 bytes into the wavefront's strip, which leaves row-contiguous, 16
      // bytes per lane.  A lone wavefront on a SIMD hides no latency by itself, so the order is written out: the
      // arithmetic of row block i runs while the strip reads of block i-1 are in flight, then the stores of block
      // i-1 go out back to back, then block i is written to the strip and its reads are issued.
      constexpr int GROUPS = 128 / GROUP;
      constexpr int PASSES = GROUP * CPR / kWave;
      static_assert(GROUP * CPR % kWave == 0, "whole passes over a strip");
      int rd_off[PASSES], st_row[PASSES], st_col[PASSES], wr_off[NV];
#pragma unroll
      for (int pass = 0; pass < PASSES; ++pass) {
        const int idx = pass * kWave + lane;
        const int r = idx / CPR, c = idx % CPR;
        rd_off[pass] = r * PITCH + ((XOR_STRIP ? (c ^ (r & (CPR - 1))) : c) << 4);
        st_row[pass] = r;
        st_col[pass] = c * 8;
      }
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        const int c = unit_chunk(v), row = MF == 32 ? lrow : 16 * (v / (CB / 2)) + lrow;
        wr_off[v] = row * PITCH + ((XOR_STRIP ? (c ^ (row & (CPR - 1))) : c) << 4);
      }
      // The bias is widened to fp32 once per tile when that costs at most 24 registers; the widest tile keeps it in
      // storage precision and widens eight values at each use instead (its epilogue has no registers to spare).
      constexpr bool WIDE_BIAS = NBV * 8 <= 24;
      float bf[WIDE_BIAS ? NBV : 1][8];
      const bool has_bias = bias != nullptr;  // uniform
      if (WIDE_BIAS && has_bias) {
#pragma unroll
        for (int v = 0; v < NBV; ++v) bv[v].widen(bf[v]);
      }
      const bool whole_width = n0 + BN <= n_lim, whole_rows = m0 + BM <= m_lim;  // uniform
      // epilogues that scatter (the QKV split): the column part of a lane's destinations, once per tile
      T* col_ptr[PASSES];
      bool block_in_one_sequence = false;  // uniform: the rows of a group share their batch index
      if constexpr (!LinearDest<Epi>::value && !StoresF32<Epi>::value && !DIRECT) {
        block_in_one_sequence = epi.rows_share_sequence(GROUP);
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
          col_ptr[pass] = epi.col_part((uint32_t)min(n0 + wn0 + st_col[pass], n_lim - 8));
          if (block_in_one_sequence) col_ptr[pass] += st_row[pass] * epi.dim;  // the lane's share of the row part
        }
      }
      // direct stores: row lrow of a 16-row block, the lane's 16 bytes of a 64-byte run (unit_chunk(0) names them)
      const uint32_t direct_voff = (uint32_t)lrow * ldc_bytes + (uint32_t)unit_chunk(0) * 16u;
      uint32_t head_split_voff = 0;  // the same for the head split: rows of a head are `dim` elements apart
      if constexpr (DIRECT && HasColumnPass<Epi>::value)
        head_split_voff = (uint32_t)lrow * (uint32_t)epi.dim * (uint32_t)sizeof(T) + (uint32_t)unit_chunk(0) * 16u;
      Quad landed[PASSES];  // first-class vectors: arrays of a struct type may end up in scratch memory
      // The matrix instructions are inline asm, so the compiler's hazard recogniser does not see that the accumulator
      // reads below depend on them: wait out the longest write-to-read distance of the matrix pipe here.
      asm volatile("s_nop 15\n\ts_nop 15");
#pragma unroll
      for (int i = 0; i <= GROUPS; ++i) {
        Quad packed[NV];
        if (i < GROUPS) {
#pragma unroll
          for (int v = 0; v < NV; ++v) {
            float out[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float a, b;
              if constexpr (MF == 32) {
                a = acc_read(acc[i][v / 2][8 * (v % 2) + e]);
                b = acc_read(acc[i][v / 2][8 * (v % 2) + 4 + e]);
              } else {
                a = acc_read(acc[(GROUP / 16) * i + v / (CB / 2)][2 * (v % (CB / 2))][e]);
                b = acc_read(acc[(GROUP / 16) * i + v / (CB / 2)][2 * (v % (CB / 2)) + 1][e]);
              }
              pair_swap<MF>(a, b);
              out[e] = a;
              out[4 + e] = b;
            }
            if (has_bias) {
              if constexpr (WIDE_BIAS) {
#pragma unroll
                for (int e = 0; e < 8; ++e) out[e] += bf[v % NBV][e];
              } else {
                bv[v % NBV].add_to(out);
              }
            }
            if constexpr (StoresF32<Epi>::value) {
              // fp32 output: the lane's eight columns are 32 contiguous bytes of one row, and the four lanes that share
              // a row cover 128 contiguous bytes between them: stored as they lie, no trip through the strip
              const int m = m0 + wm0 + i * GROUP + (MF == 32 ? lrow : 16 * (v / (CB / 2)) + lrow);
              const int ncol = n0 + wn0 + unit_chunk(v) * 8;
              if ((whole_rows || m < m_lim) && (whole_width || ncol < n_lim)) {
                float* dst = epi.c + ((int64_t)slice * g.m + m) * epi.ldc + ncol;
                *reinterpret_cast<floatx4*>(dst) = floatx4{out[0], out[1], out[2], out[3]};
                *reinterpret_cast<floatx4*>(dst + 4) = floatx4{out[4], out[5], out[6], out[7]};
              }
              packed[v] = Quad{0, 0, 0, 0};
            } else {
              T rounded[8];
#pragma unroll
              for (int e = 0; e < 8; ++e) rounded[e] = from_float<T>(epi.finish(out[e]));
              packed[v] = __builtin_bit_cast(Quad, pack_chunk(rounded));
              if constexpr (DIRECT) {
                // one per-lane offset for all stores of the tile (the lane's row and its share of the column); the
                // 16-row block goes into the scalar offset, the pair of block columns into the immediate
                const int rblk = i * GROUP + 16 * (v / (CB / 2));  // first row of the unit's 16-row block inside the wavefront's 128
                const int ncol = wn0 + unit_chunk(v) * 8;
                if constexpr (LinearDest<Epi>::value) {
                  if ((whole_rows || m0 + wm0 + rblk + lrow < m_lim) && (whole_width || n0 + ncol < n_lim))
                    store_c(packed[v], direct_voff + (uint32_t)(v % (CB / 2)) * 64u,
                            (uint32_t)(m0 + wm0 + rblk) * ldc_bytes + (uint32_t)(n0 + wn0) * (uint32_t)sizeof(T));
                } else if constexpr (HasColumnPass<Epi>::value) {
                  // Head split: the unit's 32 columns lie in one head of one of q, k, v and its 16 rows in one
                  // sequence (both uniform), so the destination is a scalar offset plus the lane's row and column
                  // share: element ((b * heads + head) * seq + s) * dim + i of that tensor.
                  const uint32_t c32 = (uint32_t)(n0 + wn0 + 32 * (v % (CB / 2)));  // first of the unit's 32 columns
                  const uint32_t which = epi.div_hidden.div(c32), rem = c32 - which * (uint32_t)epi.hidden;
                  const uint32_t head = epi.div_dim.div(rem), i0 = rem - head * (uint32_t)epi.dim;
                  const uint32_t r16 = (uint32_t)(m0 + wm0 + rblk);                 // first of the unit's 16 rows
                  const uint32_t b = epi.div_seq.div(min(r16, (uint32_t)m_lim - 1u)), s16 = r16 - b * (uint32_t)epi.seq;
                  const uint32_t soff = (((b * (uint32_t)epi.heads + head) * (uint32_t)epi.seq + s16) * (uint32_t)epi.dim + i0) * (uint32_t)sizeof(T);
                  if ((whole_rows || m0 + wm0 + rblk + lrow < m_lim) && (whole_width || n0 + ncol < n_lim))
                    head_split_store(packed[v], (int)which, head_split_voff, soff);
                }
              }
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (i > 0 && !StoresF32<Epi>::value && !DIRECT) {
          const int row0 = m0 + wm0 + (i - 1) * GROUP;
          if constexpr (StoresF32<Epi>::value) {
          } else if constexpr (LinearDest<Epi>::value) {
            const uint32_t soff = (uint32_t)row0 * ldc_bytes + (uint32_t)(n0 + wn0) * (uint32_t)sizeof(T);
#pragma unroll
            for (int pass = 0; pass < PASSES; ++pass)
              // rows at and past M are skipped here: the scalar offset of a buffer store takes no part in the
              // resource's range check, so the check alone would not drop a row group that lies wholly past M
              if ((whole_rows || row0 + st_row[pass] < m_lim) && (whole_width || n0 + wn0 + st_col[pass] < n_lim))
                store_c(landed[pass], (uint32_t)st_row[pass] * ldc_bytes + (uint32_t)st_col[pass] * (uint32_t)sizeof(T), soff);
          } else {
            const int64_t block_part = epi.row_part(min(row0, m_lim - 1));  // uniform
#pragma unroll
            for (int pass = 0; pass < PASSES; ++pass) {
              const int m = row0 + st_row[pass];
              if ((whole_rows || m < m_lim) && (whole_width || n0 + wn0 + st_col[pass] < n_lim))
                *reinterpret_cast<Quad*>(col_ptr[pass] + (block_in_one_sequence ? block_part : epi.row_part(m))) = landed[pass];
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (i < GROUPS && !StoresF32<Epi>::value && !DIRECT) {
          // same wavefront, LDS operations complete in order: no barrier between the writes and the reads
#pragma unroll
          for (int v = 0; v < NV; ++v) strip_write(strip_lds + (uint32_t)wr_off[v], packed[v]);
#pragma unroll
          for (int pass = 0; pass < PASSES; ++pass) landed[pass] = *reinterpret_cast<const Quad*>(strip + rd_off[pass]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
      if constexpr (HasColumnPass<Epi>::value) {
        for (int kt = 0; kt < ksteps; kt += 2) {
          k_step(std::integral_constant<int, 0>{}, std::false_type{}, std::false_type{});
          k_step(std::integral_constant<int, 1>{}, std::false_type{}, std::false_type{});
        }
        W4_STAMP(2)
        // A lane owns column lrow of every block and, after the pair swap, eight consecutive rows of it: one 16-byte
        // piece of a V^T row.  Stored as they lie, the 64 lanes of an instruction would touch 64 different rows of
        // V^T.  So the pieces of 32 columns x 64 rows go through the wavefront's strip ([column][64 rows], column
        // pitch 144 bytes: the 16 lanes the LDS serves together land in 16 different 16-byte slots) and come back with
        // eight adjacent lanes holding the 128 contiguous bytes of one column.  As in the row path, the arithmetic
        // of unit u runs while the strip reads of unit u-1 are in flight.
        constexpr int VT_PITCH = 144, UNITS = (BN / 2 / 32) * 2, VP = 4;  // unit = (32 columns, half of the 128 rows)
        static_assert(32 * VT_PITCH <= STRIP_ROWS * PITCH, "the transposed unit fits the strip");
        float bj[CB];
        load_bias_columns_stride<CB, MF>(epi, n0 + wn0 + lrow, n_lim, bj);
        const int rd_col = lane >> 3, rd_chunk = lane & 7;  // pass p returns rows 8*rd_chunk.. of column 8*p + rd_col
        const bool rows_whole = m0 + BM <= m_lim && epi.seq % 8 == 0;  // uniform: every group of eight is one store
        T* const vt_base = epi.vt_col_part((uint32_t)min(n0 + wn0 + rd_col, n_lim - 1));
        Quad vt_landed[VP];
        asm volatile("s_nop 15\n\ts_nop 15");  // as in the row path: the accumulator reads follow inline-asm matrix instructions
#pragma unroll
        for (int u = 0; u <= UNITS; ++u) {
          Quad piece[4];
          if (u < UNITS) {
            const int j = u / 2, hf = u % 2;  // columns 32j.., rows 64hf..
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              float out[8];
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                float a, b, bias_q;
                if constexpr (MF == 32) {  // piece q: rows 32*(q/2) + 16*(q%2) + 8*lgrp.. of column lrow
                  a = acc_read(acc[2 * hf + q / 2][j][8 * (q % 2) + e]);
                  b = acc_read(acc[2 * hf + q / 2][j][8 * (q % 2) + 4 + e]);
                  bias_q = bj[j];
                } else {  // piece q: column 16*(q/2) + lrow, rows 32*(q%2) + 16*(lgrp&1) + 8*(lgrp>>1)..
                  a = acc_read(acc[4 * hf + 2 * (q % 2)][2 * j + q / 2][e]);
                  b = acc_read(acc[4 * hf + 2 * (q % 2) + 1][2 * j + q / 2][e]);
                  bias_q = bj[2 * j + q / 2];
                }
                pair_swap<MF>(a, b);
                out[e] = a + bias_q;
                out[4 + e] = b + bias_q;
              }
              T rounded[8];
#pragma unroll
              for (int e = 0; e < 8; ++e) rounded[e] = from_float<T>(out[e]);
              piece[q] = __builtin_bit_cast(Quad, pack_chunk(rounded));
            }
          }
          __builtin_amdgcn_sched_barrier(0);
          if (u > 0) {
            const int j = (u - 1) / 2, hf = (u - 1) % 2;
            const int m = m0 + wm0 + hf * 64 + rd_chunk * 8;
            uint32_t seq_pos = 0;
            const int64_t row_off = epi.vt_row_part(min(m, m_lim - 1), seq_pos);
            // the eight rows are eight positions of one sequence: still one store, though off the 16-byte grid where
            // the sequence length is no multiple of 8
            const bool in_sequence = m + 8 <= m_lim && seq_pos + 8 <= (uint32_t)epi.seq;
#pragma unroll
            for (int p = 0; p < VP; ++p) {
              const int ncol = n0 + wn0 + j * 32 + p * 8 + rd_col;
              T* dst = vt_base + (int64_t)(j * 32 + p * 8) * epi.v_pitch + row_off;
              if (rows_whole) {
                if (ncol < n_lim) *reinterpret_cast<Quad*>(dst) = vt_landed[p];
              } else if (in_sequence) {
                if (ncol < n_lim) store_vec_unaligned<T, 8>(dst, __builtin_bit_cast(Vec<T, 8>, vt_landed[p]));
              } else if (m < m_lim && ncol < n_lim) {
                // the group runs over the end of its sequence into the next one, hidden * v_pitch elements further
                // on (sequences of fewer than 8 positions off the 8-grid never come here, see wanted()), or over
                // the end of the matrix: element by element, no division.  A rolled loop that picks its element
                // with selects: unrolled, the epilogue grows past what the compiler unrolls of the loop over the
                // units, and the accumulators would be indexed at run time.
                const Vec<T, 8> x = __builtin_bit_cast(Vec<T, 8>, vt_landed[p]);
                const int hop = (int)epi.vt_hop();
#pragma unroll
                for (int e = 0; e < 8; ++e)
                  if (m + e < m_lim) dst[e + (seq_pos + e >= (uint32_t)epi.seq ? hop : 0)] = x.v[e];
              }
            }
          }
          __builtin_amdgcn_sched_barrier(0);
          if (u < UNITS) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              // [column of the unit][group of eight rows of the half]
              const int col = MF == 32 ? lrow : 16 * (q / 2) + lrow;
              const int rows8 = MF == 32 ? (q / 2) * 4 + (q % 2) * 2 + lgrp : (q % 2) * 4 + (lgrp & 1) * 2 + (lgrp >> 1);
              strip_write(strip_lds + (uint32_t)(col * VT_PITCH + rows8 * 16), piece[q]);
            }
#pragma unroll
            for (int p = 0; p < VP; ++p)
              vt_landed[p] = *reinterpret_cast<const Quad*>(strip + (p * 8 + rd_col) * VT_PITCH + rd_chunk * 16);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    W4_STAMP(3)
    // The last substep of the K loop has already fetched the first fragments of the next tile.  Fetching them again
    // here (K step 0 of the next tile sits untouched in stage 0 until that tile's own loads overwrite it) ends the
    // life of those registers at the end of the K loop, so the epilogue has them: up to 64 with 16-wide blocks.
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (AS == 3) read_frags3(a_cur * A_BYTES);
    else read_frags(0, 0, fa[0], fb[0]);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // surplus DMA loads have landed before the LDS is given back
}

// Whether a problem may take this kernel: 16-bit type, one problem, aligned operands, an even number of K steps,
// columns in groups of eight, operands below 2 GiB (32-bit buffer offsets).
template <typename T>
static bool w4_eligible(const GemmArgs& g, int batch, bool aligned) {
  if (sizeof(T) != 2 || batch != 1 || !aligned || g.k_chunk != 0) return false;
  constexpr int BK = kRowBytes / (int)sizeof(T);
  if (g.k % (2 * BK) != 0 || g.n % 8 != 0) return false;
  const int64_t limit = (int64_t)1 << 31;
  return (int64_t)g.m * g.lda * (int64_t)sizeof(T) < limit && (int64_t)g.n * g.ldb * (int64_t)sizeof(T) < limit;
}
// The output of a linear epilogue is addressed with 32-bit offsets as well.
template <typename T>
static bool w4_output_fits(const GemmArgs& g, int64_t ldc) {
  return (int64_t)g.m * ldc * (int64_t)sizeof(T) < ((int64_t)1 << 31);
}

// split_col: a column (multiple of 8) at which a fresh tile has to start whatever BN is (0 = none).
// Three A stages where they fit (192-wide tiles, row-major epilogues).  Switch TTMI_W4_A_STAGES = 2 keeps two.
// (fp32 outputs never use the strips, so they have the room at either width)
template <int BN, typename Epi>
constexpr bool w4_three_stages_fit() { return (BN == 192 && !HasColumnPass<Epi>::value) || StoresF32<Epi>::value; }

template <typename T, int BN, typename Epi, int AS = 2, bool DIRECT = false>
static int launch_w4(GemmArgs g, const Epi& epi, hipStream_t s, int split_col = 0) {
  if constexpr (AS == 2 && !DIRECT && w4_three_stages_fit<BN, Epi>()) {
    if (kernel_switch(kSwitchW4AStages) != 2) return launch_w4<T, BN, Epi, 3>(g, epi, s, split_col);
  }
  // The 256-wide tile has no room for a third stage beside its strips; its row-major 16-bit outputs leave without
  // them (direct stores measured 1 % faster on the BERT-base forward than the strips at this width, level at 192), and
  // the third stage then fills the 160 KB to the last byte (another 0.5 % on the BERT-base and BERT-large forwards,
  // once the direct stores share one per-lane offset: with an offset per store this variant spilled and lost 4 %).
  if constexpr (AS == 2 && !DIRECT && BN == 256 && LinearDest<Epi>::value) {
    if (kernel_switch(kSwitchW4AStages) != 2) return launch_w4<T, BN, Epi, 3, true>(g, epi, s, split_col);
    return launch_w4<T, BN, Epi, 2, true>(g, epi, s, split_col);
  }
  // (the head split keeps its strips with direct stores too: its transposed-V tiles leave through them)
  constexpr int LDS = w4_lds_bytes<BN, kW4Block, AS, (DIRECT && !HasColumnPass<Epi>::value) || StoresF32<Epi>::value>();
  static_assert(LDS <= kLdsPerCu, "tile does not fit in LDS");
  const int slices = g.k_chunk > 0 ? g.k / g.k_chunk : 1;  // K slices: fp32 outputs only (launch_w4_splitk)
  if (describe_only(AS == 3 ? "dma3_agpr" : "dma_agpr", 4, 256, BN, slices)) return 0;
  g.tiles_m = (g.m + 255) / 256;
  g.split_col = split_col;
  g.split_tiles = split_col > 0 ? (split_col + BN - 1) / BN : 0;
  g.tiles_n = g.split_tiles + (g.n - split_col + BN - 1) / BN;
  const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n * slices;
  TTMI_REQUIRE(tiles < (1ll << 30), "GEMM grid too large");
  // one persistent workgroup per CU (the LDS allows no second one), a multiple of the XCD count
  const unsigned grid = (unsigned)(std::min<int64_t>(ceil_div(tiles, kNumXcd), std::max(1, compute_units() / kNumXcd)) * kNumXcd);
  auto kern = gemm_w4_kernel<T, BN, kW4Block, Epi, AS, DIRECT>;
  const int rc = allow_large_lds(reinterpret_cast<const void*>(kern), LDS);
  if (rc != 0) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kW4Threads), LDS, s, g, epi);
  return launch_status("gemm_w4_kernel");
}

// The 256 x 192 tile against the tile configurations of the 8-wavefront kernels: the same cost model, with the
// efficiency this kernel measured against them on the encoder shapes.
constexpr TileConfig kW4Tile192{256, 192, 1, 1.06f};
// The 256 x 256 tile of the same kernel (all 256 AGPRs of a lane are accumulators): a quarter fewer LDS fragment reads
// and DMA bytes per FLOP, for widths that 192 does not divide well (1024 and 4096 of the BERT-large shapes).  Only the
// epilogues with one row-major output have it; the head split needs more registers than are left.
constexpr TileConfig kW4Tile256{256, 256, 1, 1.10f};

// TTMI_LARGE_TILE=0 keeps every problem on the 8-wavefront kernels, =1 sends every eligible problem here whatever
// the cost model says (for A/B timing and for tests of small and ragged shapes); unset: the cost model decides.
template <typename T, typename Epi>
static bool w4_wanted(const GemmArgs& g, const Epi& epi, int batch, bool aligned) {
  if (!epi.vec || !w4_eligible<T>(g, batch, aligned)) return false;
  const int force = kernel_switch(kSwitchLargeTile);
  if (force == 0) return false;
  if (force == 1) return true;
  double other = 0;
  (void)pick_tile(g.m, g.n, batch, &other);
  const double mine = (LinearDest<Epi>::value || StoresF32<Epi>::value) ? std::min(tile_cost(kW4Tile192, g.m, g.n, batch), tile_cost(kW4Tile256, g.m, g.n, batch))
                                             : tile_cost(kW4Tile192, g.m, g.n, batch);
  return mine < other;
}
// Which of the two tile widths a linear epilogue takes.
template <typename T, typename Epi>
static int launch_w4_linear(const GemmArgs& g, const Epi& epi, hipStream_t s) {
  if (tile_cost(kW4Tile256, g.m, g.n, 1) < tile_cost(kW4Tile192, g.m, g.n, 1)) return launch_w4<T, 256>(g, epi, s);
  return launch_w4<T, 192>(g, epi, s);
}

// A product cut along K on this kernel: the work items are (slice, tile) pairs, every slice leaves its partial product
// in fp32 (rows [z*M, (z+1)*M) of the workspace) and `reduce(ws, slices, vec, stream)` sums them and applies the
// epilogue.  For a few thousand rows by a narrow output and a long K (the second FFN product of a 20-request batch:
// 6275 x 768 x 3072), where whole tiles are too few for the CUs whatever their size: 100 tiles of 256 x 192 with 48 K
// steps each become 200 items of 24 steps.  Every slice has the same, even number of K steps.
template <typename T>
static bool w4_splitk_ok(const GemmArgs& g, int splits, bool aligned) {
  constexpr int BK = kRowBytes / (int)sizeof(T);
  return splits > 1 && w4_eligible<T>(g, 1, aligned) && g.k % (splits * 2 * BK) == 0 && g.n % 8 == 0 &&
         (int64_t)splits * g.m * g.n * 4 < ((int64_t)1 << 31);
}
// How many K slices such a product gets on this kernel (0 or 1 = it is not taken).  Switch TTMI_W4_SPLITK: 0 = never,
// n >= 2 = n slices for every product that can be cut that way.
template <typename T>
static int w4_splitk_slices(const GemmArgs& g, bool aligned) {
  const int force = kernel_switch(kSwitchW4SplitK);
  if (force == 0 || kernel_switch(kSwitchLargeTile) == 0) return 0;
  if (force >= 2) return w4_splitk_ok<T>(g, force, aligned) ? force : 0;
  // Two slices where they turn 0.35-0.5 rounds of whole tiles into 0.7-1 round of items and K is long enough to
  // pay for the fp32 partial products (measured, LayerNorm included: 6275 x 768 x 3072 54 -> 46 us; at 4924 and at
  // 10000 rows, where the 8-wavefront kernels' own tiles fill the chip better, level, and not taken).
  constexpr int BK = kRowBytes / (int)sizeof(T);
  if (g.k / BK < 32 || !w4_splitk_ok<T>(g, 2, aligned)) return 0;
  const bool wide = tile_cost(kW4Tile256, g.m, g.n, 2) < tile_cost(kW4Tile192, g.m, g.n, 2);  // as launch_w4_splitk picks
  const int64_t tiles = ceil_div(g.m, 256) * ceil_div(g.n, wide ? 256 : 192);
  const int64_t cus = compute_units();
  return (2 * tiles <= cus && 2 * tiles * 10 > cus * 7) ? 2 : 0;
}
template <typename T, typename Reduce>
static int launch_w4_splitk(GemmArgs g, int splits, hipStream_t s, const Reduce& reduce) {
  float* ws = nullptr;
  if (tl_describe == nullptr) {
    const int rc = splitk_workspace((size_t)splits * g.m * g.n * sizeof(float), s, &ws);
    if (rc != 0) return rc;
  }
  g.k_chunk = g.k / splits;
  const EpiF32<T> part{ws, nullptr, g.n, true};
  const int rc = tile_cost(kW4Tile256, g.m, g.n, splits) < tile_cost(kW4Tile192, g.m, g.n, splits) ? launch_w4<T, 256>(g, part, s)
                                                                                                  : launch_w4<T, 192>(g, part, s);
  if (rc != 0 || tl_describe != nullptr) return rc;
  reduce(ws, splits, true, s);
  return launch_status("gemm_w4_splitk");
}

// Bias, and bias + activation.  With an activation the epilogue is a long stretch of VALU work (two transcendentals
// per element: about a third of the FFN1 product's time) that nothing overlaps when a SIMD holds a single wavefront;
// the 8-wavefront kernel pays the same arithmetic, so the faster K loop still decides.
template <typename T, int ACT, bool HAS_ACT>
struct LargeTileKernel<T, EpiBias<T, ACT, HAS_ACT, false>, typename std::enable_if<sizeof(T) == 2>::type> {
  using Epi = EpiBias<T, ACT, HAS_ACT, false>;
  static bool wanted(const GemmArgs& g, const Epi& epi, int batch, bool aligned) {
    return w4_output_fits<T>(g, epi.ldc) && w4_wanted<T>(g, epi, batch, aligned);
  }
  static int launch(const GemmArgs& g, const Epi& epi, hipStream_t s) { return launch_w4_linear<T>(g, epi, s); }
};
// Bias + head split of a dense (not packed) batch.  With V kept transposed the tiles of the V third run unswapped, so
// that third starts on a tile boundary: where 2 * hidden is no multiple of the tile width, the tile in front of it is
// cut short and a new run of tiles begins (GemmArgs::split_col).
template <typename T>
struct LargeTileKernel<T, EpiQkvSplit<T, false>, typename std::enable_if<sizeof(T) == 2>::type> {
  using Epi = EpiQkvSplit<T, false>;
  // a transposed V third that does not start on a multiple of the tile width starts a run of tiles of its own
  static bool split_run(const GemmArgs& g, const Epi& epi) {
    return epi.v_pitch > 0 && g.n == 3 * epi.hidden && (2 * epi.hidden) % 192 != 0;
  }
  // cost of the 192-wide tiles with the tile columns the two runs really have (one or two of them ragged)
  static double cost192(const GemmArgs& g, const Epi& epi, int batch) {
    const int64_t columns = split_run(g, epi) ? ceil_div(2 * epi.hidden, 192) + ceil_div(epi.hidden, 192) : ceil_div(g.n, 192);
    return tile_cost(kW4Tile192, g.m, columns * 192, batch);
  }
  // the 256-wide tile serves widths it divides, V third included; its head-split epilogue spills some registers, so
  // it is rated a little below the 256-wide tile of the row-major epilogues
  static constexpr TileConfig kTile256{256, 256, 1, 1.07f};
  static bool fits256(const GemmArgs& g, const Epi& epi) { return g.n % 256 == 0 && (epi.v_pitch == 0 || (2 * epi.hidden) % 256 == 0); }
  static double cost(const GemmArgs& g, const Epi& epi, int batch) {
    return std::min(cost192(g, epi, batch), fits256(g, epi) ? tile_cost(kTile256, g.m, g.n, batch) : 1e300);
  }
  static bool wanted(const GemmArgs& g, const Epi& epi, int batch, bool aligned) {
    if (!epi.vec || !w4_eligible<T>(g, batch, aligned)) return false;
    // eight rows of a transposed V lie in at most two sequences: what the kernel's element-wise store assumes
    // (and steps from one sequence to the next with a 32-bit element offset)
    if (epi.v_pitch > 0 && (epi.seq < 8 || (int64_t)epi.hidden * epi.v_pitch >= (1ll << 31))) return false;
    const int force = kernel_switch(kSwitchLargeTile);
    if (force == 0) return false;
    if (force == 1) return true;
    double other = 0;
    (void)pick_tile(g.m, g.n, batch, &other);
    return cost(g, epi, batch) < other;
  }
  // Q, K (and a row-major V) leave straight from the accumulator layout when every 16-row block lies in one sequence and
  // every 32-column group in one head, and a destination tensor stays below 2 GiB (32-bit buffer offsets).
  static bool direct_ok(const GemmArgs& g, const Epi& epi) {
    return epi.seq % 16 == 0 && epi.dim % 32 == 0 && g.m % epi.seq == 0 && g.n == 3 * epi.hidden &&
           (int64_t)g.m * epi.hidden * (int64_t)sizeof(T) < ((int64_t)1 << 31);
  }
  static int launch(const GemmArgs& g, const Epi& epi, hipStream_t s) {
    const bool direct = direct_ok(g, epi);
    if (fits256(g, epi) && tile_cost(kTile256, g.m, g.n, 1) < cost192(g, epi, 1))
      return direct ? launch_w4<T, 256, Epi, 2, true>(g, epi, s) : launch_w4<T, 256>(g, epi, s);
    const int split_col = split_run(g, epi) ? 2 * epi.hidden : 0;
    return direct ? launch_w4<T, 192, Epi, 2, true>(g, epi, s, split_col) : launch_w4<T, 192>(g, epi, s, split_col);
  }
};
// fp32 output of a 16-bit product (the projections in front of a LayerNorm in bfloat16 models).
template <typename T>
struct LargeTileKernel<T, EpiF32<T>, typename std::enable_if<sizeof(T) == 2>::type> {
  using Epi = EpiF32<T>;
  static bool wanted(const GemmArgs& g, const Epi& epi, int batch, bool aligned) { return w4_wanted<T>(g, epi, batch, aligned); }
  static int launch(const GemmArgs& g, const Epi& epi, hipStream_t s) {
    if (tile_cost(kW4Tile256, g.m, g.n, 1) < tile_cost(kW4Tile192, g.m, g.n, 1)) return launch_w4<T, 256>(g, epi, s);
    return launch_w4<T, 192>(g, epi, s);
  }
};
template <typename T>
struct LargeTileKernel<T, EpiAlphaBeta<T>, typename std::enable_if<sizeof(T) == 2>::type> {
  using Epi = EpiAlphaBeta<T>;
  static bool wanted(const GemmArgs& g, const Epi& epi, int batch, bool aligned) {
    return epi.beta == 0.f && w4_output_fits<T>(g, epi.ldc) && w4_wanted<T>(g, epi, batch, aligned);
  }
  static int launch(const GemmArgs& g, const Epi& epi, hipStream_t s) { return launch_w4_linear<T>(g, epi, s); }
};

}  // namespace ttmi
