// BF16 GEMM for MI355X (gfx950 / CDNA4): kernels and the C ABI declared in include/neogemm.h.
//
// What is computed is what the reference's kernel computes (v01.cu:189-270): every output element is
// the fp32-accumulated dot product of a row of A with a row/column of B, rounded once to bf16 with
// round-to-nearest-even.  How it is computed shares nothing with it: the reference stages 64x64 tiles
// with TMA and issues WGMMA from one warpgroup (v01.cu:215-237); here a workgroup of wave64s owns a
// 256x256 (or smaller) macro-tile, stages K with direct-to-LDS buffer loads into a ring of three or four
// XOR-swizzled LDS images per operand (64-deep tiles of a K-major operand, 32-deep slabs of an MN-major
// one), and feeds v_mfma_f32_16x16x32_bf16 from ds_read_b128 / ds_read_b64_tr_b16.  The large unsplit shapes run a
// second 256x256 kernel (gemm_chain_kernel) that issues both K steps of an accumulator tile back to back: same sums in
// the same order, less power per MFMA on a chip whose clock is set by its power limit.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <atomic>
#include <map>
#include <mutex>
#include <type_traits>
#include <string>
#include <utility>
#include <vector>

#include "neogemm.h"

// Split build: compiling this one file takes minutes because of the many instances of the tile kernel, so setup.py
// compiles it NEOGEMM_PARTS times in parallel with -DNEOGEMM_PART=0..NEOGEMM_PARTS-1 and links the objects.  Part 0
// holds everything but the tile kernels; part k > 0 instantiates its share of launch_tile<> (listed behind
// launch_tile) or, the last one, launch_chain, and nothing else.  Without NEOGEMM_PART the file is one self-contained translation unit.
#ifdef NEOGEMM_PART
#define NEOGEMM_HAS_PART(p) (NEOGEMM_PART == (p))
#else
#define NEOGEMM_HAS_PART(p) 1
#endif
#define NEOGEMM_PARTS 9

namespace neogemm {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(4))) short i16x4;
typedef __attribute__((ext_vector_type(8))) short i16x8;

#define NEOGEMM_AS3 __attribute__((address_space(3)))

static constexpr int KT = 32;                        // K depth of one MFMA step / one slab (bf16 elements)
static constexpr int KTILE = 64;                     // K depth of a K-major LDS image, and the split-K unit
static constexpr uint32_t OOB_OFFSET = 0x80000000u;  // >= every num_records this file builds
// Load j of a run of four carries the instruction offset (j & 3) * 1024, which moves the global and the LDS
// address alike; the lane offsets are lowered by it and raised by VOFF_BIAS (so that they cannot go negative,
// whatever the leading dimension), and the resource base is lowered by VOFF_BIAS in turn.
static constexpr uint32_t VOFF_BIAS = 3 * 1024;

// ---------------------------------------------------------------------------------------------
// LDS images and their swizzles.  K is consumed in slabs of 32 (one v_mfma_f32_16x16x32_bf16 step).
//
// K-major operand (rows of the matrix are K-contiguous: A[M,K], B[N,K]) — image of a 64-deep TILE:
//   ROWS x 128 B, row r at r*128, eight 16-byte chunks per row, slab s of the tile in chunks 4s..4s+3;
//   logical chunk c of row r lives at physical chunk c ^ swz_k(r).  64 deep, not 32, so that one
//   direct-to-LDS instruction (8 rows x 128 B) asks the L2 for whole 128-byte lines: with 64-byte
//   pieces the vector L1 issues twice the requests and the wave that issues the load is held up
//   roughly in proportion to the number of requests.  Three images per operand (two for B of the largest
//   tiles when both operands are K-major).
// MN-major operand (the K index is the slow one: B[K,N]) — image of a 32-deep SLAB:
//   32 x (ROWS*2) B, k-row at k*ROWS*2; logical chunk c (8 columns) of k-row k lives at physical
//   chunk c ^ swz_mn(k).  Rows are whole lines already.  Read back with ds_read_b64_tr_b16: in each
//   group of 16 lanes, lanes 4r..4r+3 address k-row r (16 columns, 8 bytes per lane) and lane j
//   receives the 4 k-values of column j.  A half-wave touches k-rows {0..3} and {8..11} (+4, +16),
//   32 bytes of each: swz_mn spreads those eight pieces over the 64 banks.  Four images (ring).
// Either way an operand owns ROWS*256 bytes of LDS.  Direct-to-LDS loads write 64 lanes x 16 B
// contiguously, so a swizzle is applied by choosing which global chunk each lane fetches.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t swz_k(uint32_t row) {
  // bits: row2 | (row0^row2) << 1 | (row0^row1) << 2 — the fastest of the 4096 XOR-linear 3-bit
  // functions of the row number for the 16-row x 4-chunk ds_read_b128 pattern, timed on the hardware
  // (246 B/clk/CU; no swizzle: 77)
  return ((row >> 2) & 1u) | (((row ^ (row >> 2)) & 1u) << 1) | (((row ^ (row >> 1)) & 1u) << 2);
}
__device__ __forceinline__ uint32_t swz_mn(uint32_t krow) {
  // even values 0..14: (k & 3) picks the 32-byte pair, bit 3 of k the 128-byte half
  return ((krow & 3u) << 1) | (((krow >> 3) & 1u) << 3);
}

// Direct-to-LDS loads.  One instruction moves 1 KiB: lane i's 16 bytes at (rsrc.base + voff + OFF)
// land at LDS address M0 + OFF + 16*i.  M0 is written once per run of loads (a scalar write, a wait
// state, then up to four loads told apart by the 12-bit instruction offset, which moves the global
// and the LDS address alike — the per-lane offsets are built with that in mind): a load then costs
// the wave one issue slot, which fits behind a 16-cycle MFMA, where m0-write + nop + load does not.
// The compiler is not told that these touch LDS; ordering against ds_read is done by hand with
// s_waitcnt vmcnt + s_barrier (a builtin load would make the compiler wait vmcnt(0) before every
// LDS read and serialise the pipeline).
__device__ __forceinline__ void dma_set_m0(uint32_t lds) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" : : "s"(lds) : "memory");
}
template <int OFF>
__device__ __forceinline__ void dma16(i32x4 rsrc, uint32_t voff) {
  static_assert(OFF >= 0 && OFF < 4096, "12-bit instruction offset");
  // sc1: device-scope load, i.e. do not keep the line in the CU's 32 KiB vector L1 — the data goes
  // straight to LDS and is never re-read through L1; measured +4.6 % on N(0,1) data at 8192^3.
  asm volatile("buffer_load_dwordx4 %0, %1, 0 offen offset:%2 sc1 lds" : : "v"(voff), "s"(rsrc), "n"(OFF) : "memory");
}

// acc += A(16x32) * B(32x16) with the accumulator pinned in AGPRs and written in place.  Written as
// asm because the builtin lets the register allocator pick a destination different from the source
// accumulator; with all 256 AGPRs holding accumulators that ends in a storm of v_accvgpr copies at
// the loop back-edge.  Being opaque to the compiler, no hazard NOPs are inserted for it: the caller
// keeps reads of an accumulator away from the MFMA that wrote it (see the s_nop before the epilogue).
__device__ __forceinline__ void mfma_16x16x32(f32x4& acc, bf16x8 a, bf16x8 b) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

__device__ __forceinline__ bf16x8 lds_read_b128(uint32_t addr) {
  return *((NEOGEMM_AS3 bf16x8*)(uintptr_t)addr);
}
__device__ __forceinline__ i16x4 lds_read_tr16(uint32_t addr) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((NEOGEMM_AS3 i16x4*)(uintptr_t)addr);
}

template <int N, class Fn, int... I>
__device__ __forceinline__ void static_for_impl(Fn&& fn, std::integer_sequence<int, I...>) {
  (fn(std::integral_constant<int, I>{}), ...);
}
template <int N, class Fn>
__device__ __forceinline__ void static_for(Fn&& fn) {
  static_for_impl<N>(fn, std::make_integer_sequence<int, N>{});
}

struct TileArgs {
  const char* A;  // operand whose rows become output rows
  const char* B;  // operand whose rows/columns become output columns
  char* C;        // bf16 output, row-major [M][ldc]
  float* ws;      // split-K partials [ksplit][M][N] fp32 (ksplit > 1 only)
  int M, N, K;
  long lda, ldb, ldc;  // elements
  int ntm, ntn, group_m;
  int ksplit, ktiles_per_split;  // K is cut in tiles of KTILE; a split is a run of tiles
  unsigned long long* prof;      // phase timers, 4 per wave (profiling instantiation only)
  float alpha, beta;             // C = alpha * A*B + beta * C (beta == 0: C is not read)
  long bsa, bsb, bsc;            // batch strides in elements; blockIdx.z is the batch index
  int early_stores;              // gemm_chain_kernel: stage the epilogue a quarter wave tile at a time (see launch_chain)
  int batch;
};

// Workgroup id -> (K split, output tile).  Consecutive ids land on different XCDs (round-robin over the 8
// dies, each with its own L2), so id%8 selects a contiguous slice of the work order, and the work
// order walks, split by split, group_m tile-rows at a time: a slice is a compact block of C for one
// range of K (with 8 splits every XCD owns one of them and fetches its share of A and B once:
// 1024x1024x32768 went from 70 to 62 us).
template <int BM, int BN>
__device__ __forceinline__ void tile_of_workgroup(const TileArgs& p, int& m0, int& n0, int& kz) {
  const int total = p.ntm * p.ntn;
  const int work = total * p.ksplit;
  const int pid = blockIdx.x;
  const int q = work >> 3, r = work & 7, x = pid & 7;
  const int w = x * q + (x < r ? x : r) + (pid >> 3);
  kz = w / total;
  const int lin = w - kz * total;
  const int per_group = p.group_m * p.ntn;
  const int g = lin / per_group;
  const int first = g * p.group_m;
  const int gsz = (p.ntm - first) < p.group_m ? (p.ntm - first) : p.group_m;
  const int rem = lin - g * per_group;
  m0 = (first + rem % gsz) * BM;
  n0 = (rem / gsz) * BN;
}

// Global -> LDS side of one operand: which 16 bytes each lane fetches for each of this wave's
// 1 KiB loads of a unit (a 64-deep tile if K-major, a 32-deep slab if MN-major), and the buffer
// resource that walks along K.
template <int ROWS, bool KMAJOR, int NW, int NIMG>
struct Operand {
  static constexpr int UNIT_K = KMAJOR ? KTILE : KT;       // K depth of one unit
  static constexpr int UNITS = NIMG;                       // images in LDS
  static constexpr uint32_t IMG = ROWS * UNIT_K * 2;       // bytes per image
  static constexpr int NINSTR = IMG / 1024;                // 1 KiB wave-loads per unit
  static constexpr int IPW = NINSTR / NW;                  // per wave
  static constexpr int ROWB = ROWS * 2;                    // bytes per k-row of an MN-major image
  static constexpr int CPR = ROWS / 8;                     // 16-byte chunks per k-row (MN-major)
  static constexpr int KR = 64 / CPR;                      // k-rows per wave-load (MN-major)
  static_assert(NINSTR % NW == 0 && IPW >= 1 && IPW <= 8, "unit loads must divide evenly over the waves");
  static_assert(KMAJOR || (ROWS >= 128 && (ROWS & (ROWS - 1)) == 0),
                "MN-major: >= 16 chunks per k-row for the swizzle, a power of two so that a wave-load covers whole k-rows");

  uint32_t voff[IPW];
  uint64_t base;
  uint32_t kadv;
  uint32_t lds_w;

  // Every lane offset that would leave the matrix is replaced by OOB_OFFSET, which the buffer range
  // check (num_records = 2 GiB, constant) turns into a zero fill without a memory access; all other
  // offsets address bytes inside the matrix, so the resource needs no exact size and only its base
  // moves along K.  (See VOFF_BIAS for the instruction offsets.)
  __device__ __forceinline__ void init(const char* ptr, long ld, int rows_total, int r0, int k_begin, int wave,
                                       int lane) {
    if constexpr (KMAJOR) {
      base = (uint64_t)ptr + ((uint64_t)r0 * ld + k_begin) * 2;
      kadv = KTILE * 2;
#pragma unroll
      for (int j = 0; j < IPW; ++j) {
        uint32_t row = (wave * IPW + j) * 8 + (lane >> 3);
        uint32_t c = (lane & 7) ^ swz_k(row);
        voff[j] = row * (uint32_t)ld * 2 + c * 16 + VOFF_BIAS - (j & 3) * 1024;
        if (r0 + (int)row >= rows_total) voff[j] = OOB_OFFSET;
      }
    } else {
      base = (uint64_t)ptr + ((uint64_t)k_begin * ld + r0) * 2;
      kadv = KT * (uint32_t)ld * 2;
#pragma unroll
      for (int j = 0; j < IPW; ++j) {
        uint32_t krow = (wave * IPW + j) * KR + lane / CPR;
        uint32_t c = (lane % CPR) ^ swz_mn(krow);
        voff[j] = krow * (uint32_t)ld * 2 + c * 16 + VOFF_BIAS - (j & 3) * 1024;
        // a chunk past the last column would wrap into the next k-row (rows_total % 8 == 0: no straddling)
        if (r0 + (int)c * 8 >= rows_total) voff[j] = OOB_OFFSET;
      }
    }
    lds_w = wave * IPW * 1024;
  }

  // Drop what lies at or past depth krem of the unit about to be loaded (K-major: chunks, which would
  // wrap into the next row; MN-major: whole k-rows).  krem may be <= 0 (a unit entirely past K).
  // Masks only ever grow along K, so they are applied in place.
  __device__ __forceinline__ void mask_k_tail(int krem, int wave, int lane) {
#pragma unroll
    for (int j = 0; j < IPW; ++j) {
      if constexpr (KMAJOR) {
        uint32_t row = (wave * IPW + j) * 8 + (lane >> 3);
        uint32_t c = (lane & 7) ^ swz_k(row);
        if ((int)c * 8 >= krem) voff[j] = OOB_OFFSET;
      } else {
        uint32_t krow = (wave * IPW + j) * KR + lane / CPR;
        if ((int)krow >= krem) voff[j] = OOB_OFFSET;
      }
    }
  }

  // live == false: a resource of size zero, every lane out of range: the loads fill their LDS bytes with zeros and
  // touch no memory (a unit past the end of K)
  __device__ __forceinline__ i32x4 rsrc(bool live = true) const {
    i32x4 r;
    const uint64_t b = base - VOFF_BIAS;
    r[0] = (int)(uint32_t)b;
    r[1] = (int)(uint32_t)(b >> 32);  // a 48-bit address: bits 16.. (stride, swizzle) stay 0
    r[2] = live ? (int)0x80000000u : 0;
    r[3] = 0x00020000;
    return r;
  }
  // load J of this wave; M0 must hold image + lds_w + (J / 4) * 4096 (dma_set_m0)
  template <int J>
  __device__ __forceinline__ void issue_one(i32x4 r) const {
    dma16<(J & 3) * 1024>(r, voff[J]);
  }
  __device__ __forceinline__ void advance() { base += kadv; }
};

// Order of the TM x TN MFMAs of a slab (see slab_step): step m -> column c of B and row i of A.
constexpr int mfma_walk_c(int tm, int tn, int m) {
  if ((tm | tn) & 1) return m / tm;
  return ((m / 4) / (tm / 2)) * 2 + ((m % 4) >> 1);
}
constexpr int mfma_walk_i(int tm, int tn, int m) {
  if ((tm | tn) & 1) return m % tm;
  const int blk = m / 4, in = m % 4, nbi = tm / 2, bc = blk / nbi;
  const int bi = (bc & 1) ? nbi - 1 - blk % nbi : blk % nbi;
  return bi * 2 + ((in & 1) ^ (in >> 1));
}

// Per-lane constants for reading MFMA operand fragments out of an image.  A fragment is the
// 16 rows x 32 k operand of v_mfma_f32_16x16x32_bf16: lane l holds row (l & 15), k = 8*(l >> 4) .. +7.
template <int ROWS, bool KMAJOR, int NT>
struct FragReader {
  static constexpr int ROWB = ROWS * 2;
  // LDS address of this lane's piece in image 0 of the operand's region: K-major, one per slab of the
  // tile (fragment t is t * 2048 further); MN-major, one per fragment.  Image and fragment offsets are
  // compile-time constants wherever possible so that they end up in the 16-bit offset field of ds_read.
  uint32_t lane_off[KMAJOR ? 2 : NT];

  __device__ __forceinline__ void init(uint32_t region, int wrow0, int lane) {
    if constexpr (KMAJOR) {
      const uint32_t row = lane & 15;
#pragma unroll
      for (int s = 0; s < 2; ++s)
        lane_off[s] = region + (uint32_t)(wrow0 + row) * 128 + (((4 * s + ((uint32_t)lane >> 4)) ^ swz_k(row)) << 4);
    } else {
      const uint32_t i = lane & 15, q = lane >> 4;
      const uint32_t tr_r = i >> 2, tr_c = i & 3;
      const uint32_t krow = 8 * q + tr_r;  // the second read adds 4: same swizzle
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        uint32_t chunk = (uint32_t)(wrow0 >> 3) + 2 * t + (tr_c >> 1);
        lane_off[t] = region + krow * ROWB + ((chunk ^ swz_mn(krow)) << 4) + ((tr_c & 1) << 3);
      }
    }
  }
  // MN-major: the two halves (k 0..3 and 4..7 of each lane's eight) of fragment t in the image at `img`
  // (byte offset within the region)
  __device__ __forceinline__ i16x4 read_half(uint32_t img, int t, int h) const {
    return lds_read_tr16(lane_off[t] + img + h * 4 * ROWB);
  }
  // K-major: this lane's address for slab `slab` (its parity picks the half of the tile image) in
  // the image at `img`.  When img is not a compile-time constant the sum is pinned in a VGPR, so that
  // the fragment offsets t * 2048 go into the offset field of the reads instead of being added, one
  // scalar and one vector instruction per read, to the image offset first.
  __device__ __forceinline__ uint32_t base(uint32_t img, int slab) const {
    uint32_t b = lane_off[slab & 1] + img;
    if (!__builtin_constant_p(img)) asm volatile("" : "+v"(b));
    return b;
  }
  __device__ __forceinline__ bf16x8 read_at(uint32_t b, int t) const { return lds_read_b128(b + t * 2048); }
  // fragment t (16 rows) of slab `slab`
  __device__ __forceinline__ bf16x8 read(uint32_t img, int t, int slab) const {
    if constexpr (KMAJOR) {
      return lds_read_b128(lane_off[slab & 1] + img + t * 2048);
    } else {
      i16x8 v = __builtin_shufflevector(read_half(img, t, 0), read_half(img, t, 1), 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(bf16x8, v);
    }
  }
};
__device__ __forceinline__ bf16x8 with_half(bf16x8 f, i16x4 h, int which) {
  const i16x8 v = __builtin_bit_cast(i16x8, f);
  const i16x8 w = __builtin_shufflevector(h, h, 0, 1, 2, 3, 0, 1, 2, 3);
  const i16x8 r = which == 0 ? __builtin_shufflevector(w, v, 0, 1, 2, 3, 12, 13, 14, 15)
                             : __builtin_shufflevector(v, w, 0, 1, 2, 3, 8, 9, 10, 11);
  return __builtin_bit_cast(bf16x8, r);
}

// Where the accumulator tile of a wave lies in C: local (row, column) of the wave tile -> global.  Within an aligned
// run of 16 local rows / 8 local columns the global ones are consecutive.
struct BlockMap {  // one block
  int r0, c0;
  __device__ __forceinline__ int row(int l) const { return r0 + l; }
  __device__ __forceinline__ int col(int l) const { return c0 + l; }
};

// Epilogue of the tile kernels: the TM x TN accumulator tiles of a wave (NW waves per workgroup, LDS_BYTES of LDS
// that the main loop is done with) go to C as bf16, or to the split-K partials as fp32.
// STAGE_TM: row tiles of the wave tile that go through LDS at a time (TM: all of it at once).
template <int TM, int TN, int NW, uint32_t LDS_BYTES, int STAGE_TM = TM, class Map>
__device__ __forceinline__ void store_wave_tile(f32x4 (&acc)[TM][TN], const TileArgs& p, char* gC, int kz, int lane,
                                                int wave, uint32_t lds0, const Map map) {
  constexpr int WTM = TM * 16, WTN = TN * 16;
  static_assert(TM % STAGE_TM == 0, "staging chunks are whole row tiles");
  // Epilogue: lane holds, per 16x16 tile, output row (lane & 15) and 4 consecutive columns 4*(lane >> 4)..+3.
  const int row_l = lane & 15, colq = (lane >> 4) * 4;
  // An accumulator element is read out of its AGPR where it is used: left to itself the compiler copies
  // all 256 accumulators to VGPRs ahead of the three epilogue variants below, and spills.
  auto acc_get = [](float a) -> float {
    float v;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
    return v;
  };
  // Coalesced path: the wave parks its bf16 tile in LDS (the slab ring is dead by now) and reads it back
  // row-wise, so that a store instruction writes whole rows of the wave tile, 16 bytes per lane, instead of
  // sixteen 32-byte pieces.  The staging tile is WTM x WTN bf16, 16-byte chunks XOR-ed with the row number
  // so that neither the 8-byte writes (16 rows per instruction) nor the 16-byte reads collide on banks.
  constexpr int CH = WTN / 8;        // 16-byte chunks per staged row
  constexpr int RPI = 64 / CH;       // rows one store instruction covers
  constexpr bool CAN_STAGE = (size_t)NW * WTM * WTN * 2 <= (size_t)LDS_BYTES && CH >= 4 && CH <= 64;
  const bool stage = CAN_STAGE && p.ksplit == 1 && p.beta == 0.f && (((uintptr_t)gC | (uintptr_t)(p.ldc * 2)) & 15) == 0;
  if (stage) {
    if constexpr (CAN_STAGE) {
      // every wave is done with the slab images (its LDS reads have returned: the MFMAs that used them
      // were issued; wait anyway) before any wave overwrites them; so are its direct-to-LDS loads (when K is
      // short the prologue's fully masked zero fills of later images may still be in flight)
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      const uint32_t region = lds0 + (uint32_t)wave * (WTM * WTN * 2);
      const int colc = lane % CH;
      const int col = map.col(colc * 8);
#pragma unroll
      for (int i0 = 0; i0 < TM; i0 += STAGE_TM) {
        // rows i0*16 .. of the wave tile are rows 0 .. of the staging region
        auto park = [&](auto scaled) {
#pragma unroll
          for (int i = i0; i < i0 + STAGE_TM; ++i) {
            const uint32_t row = (i - i0) * 16 + row_l;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
              bf16x4 o;
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                float v = acc_get(acc[i][j][r]);
                if constexpr (decltype(scaled)::value) v *= p.alpha;
                o[r] = (__bf16)v;
              }
              const uint32_t c = 2 * j + (lane >> 5);
              const uint32_t addr = region + row * (WTN * 2) + ((c ^ (row & (CH - 1))) << 4) + (((lane >> 4) & 1) << 3);
              *((NEOGEMM_AS3 bf16x4*)(uintptr_t)addr) = o;
            }
          }
        };
        if (p.alpha == 1.f) park(std::false_type{});
        else park(std::true_type{});
        // same wave wrote and reads: LDS operations of a wave complete in order; the compiler orders them
#pragma unroll
        for (int st = 0; st < STAGE_TM * 16 / RPI; ++st) {
          const uint32_t row = st * RPI + lane / CH;
          const uint32_t addr = region + row * (WTN * 2) + (((uint32_t)colc ^ (row & (CH - 1))) << 4);
          const bf16x8 v = *((NEOGEMM_AS3 bf16x8*)(uintptr_t)addr);
          const int grow = map.row(i0 * 16 + (int)row);
          if (grow < p.M) {
            char* dst = gC + ((size_t)grow * p.ldc + col) * 2;
            if (col + 7 < p.N) {
              // C is written once and not read again here: streaming stores leave the L2 to A and B
              __builtin_nontemporal_store(v, (bf16x8*)dst);
            } else {
#pragma unroll
              for (int e = 0; e < 8; ++e)
                if (col + e < p.N) ((__bf16*)dst)[e] = v[e];
            }
          }
        }
      }
    }
  } else if (p.ksplit == 1) {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = map.row(i * 16 + row_l);
      if (row >= p.M) continue;
      char* crow = gC + (size_t)row * p.ldc * 2;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = map.col(j * 16 + colq);
        f32x4 v;
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = acc_get(acc[i][j][r]) * p.alpha;
        if (p.beta != 0.f) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (col + r < p.N) v[r] = __builtin_fmaf(p.beta, (float)*(const __bf16*)(crow + (size_t)(col + r) * 2), v[r]);
        }
        const bf16x4 o = {(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
        if (col + 3 < p.N) {
          __builtin_nontemporal_store(o, (bf16x4*)(crow + (size_t)col * 2));
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (col + r < p.N) *(__bf16*)(crow + (size_t)(col + r) * 2) = o[r];
        }
      }
    }
  } else {
    float* wsz = p.ws + ((size_t)blockIdx.z * p.ksplit + kz) * p.M * p.N;
    const bool vec = (p.N & 3) == 0;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = map.row(i * 16 + row_l);
      if (row >= p.M) continue;
      float* wrow = wsz + (size_t)row * p.N;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = map.col(j * 16 + colq);
        f32x4 o;
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = acc_get(acc[i][j][r]);
        if (vec && col + 3 < p.N) {
          *(f32x4*)(wrow + col) = o;
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (col + r < p.N) wrow[col + r] = o[r];
        }
      }
    }
  }
}

// PROF adds s_memtime stamps around the two waits of the main loop and writes, per wave,
// {total, waiting for own loads, waiting at the barrier, epilogue} shader-clock cycles to p.prof — the
// per-phase cycle buffer idea of the reference's harness (cublass/matmul.cu:99-106,149-165).
// Images of B when both operands are K-major: three where the LDS has the room (one more tile of B in
// flight: 64x128 tile -7 % at 1024^3, 128x256 -2.4 % at 8192^3), two for the 256x256 and 192x256 tiles, whose
// A images and two of B fill the 160 KiB.  The 128x128 tile has both instances: three images make it 96 KiB,
// one workgroup per CU, which pays when there is no second workgroup for the CU anyway (-10 % at 1536^3) and
// costs when there is (+5..8 % at 4096^3 and 8192^3 with that tile).
constexpr int b_images_both_kmajor(int bm, int bn) { return (bm + bn) * 384 <= 160 * 1024 ? 3 : 2; }
template <int BM, int BN, int WGM, int WGN, bool AK, bool BK, bool PROF = false, int NB_KK = b_images_both_kmajor(BM, BN)>
__global__ __launch_bounds__(WGM* WGN * 64) void gemm_tile_kernel(TileArgs p) {
  constexpr int NW = WGM * WGN;
  constexpr int WTM = BM / WGM, WTN = BN / WGN;
  constexpr int TM = WTM / 16, TN = WTN / 16;
  static_assert(WTM % 16 == 0 && WTN % 16 == 0, "wave tile must be a multiple of the 16x16 MFMA tile");
  static_assert(AK || BK, "at least one operand is K-major");
  // images per operand: four 32-deep slabs if MN-major; three 64-deep tiles if K-major, except that
  // B gets by with NB_KK = two when both are K-major and the tile is large (160 KiB of LDS for a 256x256 tile either way)
  using OpA = Operand<BM, AK, NW, AK ? 3 : 4>;
  using OpB = Operand<BN, BK, NW, BK ? (AK ? NB_KK : 3) : 4>;
  constexpr uint32_t A_BYTES = OpA::UNITS * OpA::IMG, LDS_BYTES = A_BYTES + OpB::UNITS * OpB::IMG;
  constexpr int IA = OpA::IPW, IB = OpB::IPW;  // this wave's loads per unit of A / of B

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(NEOGEMM_AS3 char*)smem;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;

  int m0, n0, kz;
  tile_of_workgroup<BM, BN>(p, m0, n0, kz);
  const int k_begin = kz * p.ktiles_per_split * KTILE;
  int k_end = k_begin + p.ktiles_per_split * KTILE;
  if (k_end > p.K) k_end = p.K;
  const int klen = k_end - k_begin;
  const int ntile = (klen + KTILE - 1) / KTILE;
  const int nslab = 2 * ntile;  // the last slab of a K-major tile may lie entirely past K: it is loaded as zeros

  unsigned long long t_start = 0, t_loads = 0, t_barrier = 0;
  if constexpr (PROF) t_start = __builtin_readcyclecounter();

  OpA opa;
  OpB opb;
  // problem blockIdx.z of the batch
  const char* gA = p.A + (size_t)blockIdx.z * p.bsa * 2;
  const char* gB = p.B + (size_t)blockIdx.z * p.bsb * 2;
  char* gC = p.C + (size_t)blockIdx.z * p.bsc * 2;
  opa.init(gA, p.lda, p.M, m0, k_begin, wave, lane);
  opb.init(gB, p.ldb, p.N, n0, k_begin, wave, lane);
  FragReader<BM, AK, TM> fa;
  FragReader<BN, BK, TN> fb;
  fa.init(lds0, wm * WTM, lane);
  fb.init(lds0 + A_BYTES, wn * WTN, lane);

  f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;

  // Two copies of every fragment: slab j is computed from copy j & 1 while the fragments of slab j+1
  // are read into the other one.  The accumulators live in the 256 AGPRs, so the VGPRs have room.
  bf16x8 af[2][TM] = {}, bfr[2][TN] = {};

  // LDS image that holds slab j of an operand
  // (byte offset within the operand's region)
  auto img_a = [&](int j) -> uint32_t { return ((uint32_t)(AK ? j >> 1 : j) % OpA::UNITS) * OpA::IMG; };
  auto img_b = [&](int j) -> uint32_t { return ((uint32_t)(BK ? j >> 1 : j) % OpB::UNITS) * OpB::IMG; };

  // Which of this wave's loads go under which half of a slab step.  The schedule has a period of two
  // slabs (four halves P0..P3, starting with an odd slab):
  //   next to an MN-major operand, a K-major one loads a 64-deep tile in P0 and P1, the MN-major one a
  //   slab in P2 and one in P3; if both are K-major, B loads its tile in P0 and A over P1..P3.
  // Segment = loads [lo, hi) of operand A (op 1) or B (op 2); a half carries up to two segments.
  struct Seg { int op, lo, hi; };
  auto plan = [](int phase, int which) constexpr -> Seg {
    if (AK && BK) {
      // B, with two images only, has the least time to land: all of it in P0; A over P1..P3
      if (which == 1) return Seg{0, 0, 0};
      if (phase == 0) return Seg{2, 0, IB};
      return Seg{1, (phase - 1) * IA / 3, phase * IA / 3};
    } else if (AK) {
      if (which == 1) return Seg{0, 0, 0};
      if (phase == 0) return Seg{1, 0, IA / 2};
      if (phase == 1) return Seg{1, IA / 2, IA};
      return Seg{2, 0, IB};
    } else {
      if (which == 1) return Seg{0, 0, 0};
      if (phase == 0) return Seg{2, 0, IB / 2};
      if (phase == 1) return Seg{2, IB / 2, IB};
      return Seg{1, 0, IA};
    }
  };

  // One slab step: the TM x TN MFMAs of the slab whose fragments are in copy PAR, with the LDS reads
  // that fetch the next slab's fragments into the other copy (READ) and the loads the schedule puts
  // under the two halves of this step (phases PH0, PH1; -1: none).  The wave issues in order, about
  // one instruction every four cycles, and whatever sits between two MFMAs beyond the 16 cycles the
  // first one occupies the pipe is lost.  The four waves run in lockstep and share one LDS pipe, which
  // takes longer than those 16 cycles over their four simultaneous 1 KiB reads: so the reads go into
  // every other gap between MFMAs (the first three quarters of the step), the loads into gaps between.
  //   slab_rd: the slab read from LDS (its parity picks the half of a K-major tile image);
  //   ia / ib: image (offset in the operand's region) the fragments are read from;
  //   dst_*0 / dst_*1: LDS address of the image the A / B loads of the first / second half go to.
  auto slab_step = [&](auto par, auto do_read, int slab_rd, uint32_t ia, uint32_t ib, auto ph0, auto ph1,
                       uint32_t dst_a0, uint32_t dst_b0, uint32_t dst_a1, uint32_t dst_b1) {
    constexpr int PAR = decltype(par)::value, PH0 = decltype(ph0)::value, PH1 = decltype(ph1)::value;
    constexpr bool READ = decltype(do_read)::value;
    constexpr int NM = TM * TN;
    // LDS read operations: a K-major fragment is one 16-byte read, an MN-major one two transposing
    // 8-byte reads; A and B alternate as long as both last
    constexpr int RA = AK ? 1 : 2, RB = BK ? 1 : 2, NRA = TM * RA, NRB = TN * RB, NR = READ ? NRA + NRB : 0;
    constexpr int RSPAN = NM - NM / 4;
    uint32_t base_a = 0, base_b = 0;
    if constexpr (READ && AK) base_a = fa.base(ia, slab_rd);
    if constexpr (READ && BK) base_b = fb.base(ib, slab_rd);
    auto read_op = [&](auto kc) {
      constexpr int k = decltype(kc)::value;
      // k-th read: alternate B, A, B, A ... until one list runs out
      constexpr int pairs = NRA < NRB ? NRA : NRB;
      constexpr bool is_b = k < 2 * pairs ? (k % 2 == 0) : (NRB > NRA);
      constexpr int idx = k < 2 * pairs ? k / 2 : k - pairs;
      if constexpr (is_b) {
        if constexpr (BK) bfr[PAR ^ 1][idx] = fb.read_at(base_b, idx);
        else bfr[PAR ^ 1][idx / 2] = with_half(bfr[PAR ^ 1][idx / 2], fb.read_half(ib, idx / 2, idx % 2), idx % 2);
      } else {
        if constexpr (AK) af[PAR ^ 1][idx] = fa.read_at(base_a, idx);
        else af[PAR ^ 1][idx / 2] = with_half(af[PAR ^ 1][idx / 2], fa.read_half(ia, idx / 2, idx % 2), idx % 2);
      }
    };
    auto load_ops = [&](auto phc, auto mc, uint32_t dst_a, uint32_t dst_b, int half) {
      constexpr int PHASE = decltype(phc)::value, m = decltype(mc)::value;  // m: gap index within the half
      if constexpr (PHASE >= 0) {
        constexpr Seg s0 = plan(PHASE, 0), s1 = plan(PHASE, 1);
        constexpr int n0l = s0.hi - s0.lo, n1l = s1.hi - s1.lo, NL = n0l + n1l;
        static_for<NL>([&](auto lc) {
          constexpr int l = decltype(lc)::value;
          // spread over the half, on odd gaps (the reads take the even ones)
          constexpr int gap = (((NM / 2) * (2 * l + 1) / (2 * NL)) | 1) < NM / 2 ? (((NM / 2) * (2 * l + 1) / (2 * NL)) | 1) : NM / 2 - 1;
          if constexpr (gap == m) {
            constexpr Seg sg = l < n0l ? s0 : s1;
            constexpr int J = l < n0l ? s0.lo + l : s1.lo + (l - n0l);
            constexpr bool first = (l == 0) || (l == n0l) || (J % 4 == 0);
            if constexpr (sg.op == 1) {
              if constexpr (first) dma_set_m0(dst_a + opa.lds_w + (J / 4) * 4096);
              opa.template issue_one<J>(opa.rsrc());
              if constexpr (J == IA - 1) opa.advance();  // the unit is complete: move along K
            } else {
              if constexpr (first) dma_set_m0(dst_b + opb.lds_w + (J / 4) * 4096);
              opb.template issue_one<J>(opb.rsrc());
              if constexpr (J == IB - 1) opb.advance();
            }
          }
        });
      }
    };
    static_for<NM>([&](auto mc) {
      constexpr int m = decltype(mc)::value;
      // Which tile MFMA m of the slab works on: 2x2 blocks of (column c of B, row i of A), the blocks row by row in
      // alternating direction.  The order changes nothing in the result (every tile gets one MFMA per slab); it
      // is a matter of power: the matrix cores alone sustain 2.8 % more on N(0,1) operands with this walk than with
      // all rows for one column after the other, and 6 % more than when both operands change with every instruction.
      constexpr int c = mfma_walk_c(TM, TN, m), i = mfma_walk_i(TM, TN, m);
      // B fragment first: D rows index n, D columns index m, so a lane ends up with 4
      // consecutive n of one output row (an 8-byte piece) instead of 4 rows of one column.
      mfma_16x16x32(acc[i][c], bfr[PAR][c], af[PAR][i]);
      static_for<NR>([&](auto kc) {
        constexpr int k = decltype(kc)::value;
        if constexpr (k * RSPAN / (NR > 0 ? NR : 1) == m) read_op(kc);
      });
      if constexpr (m < NM / 2) load_ops(ph0, std::integral_constant<int, m>{}, dst_a0, dst_b0, 0);
      else load_ops(ph1, std::integral_constant<int, m - NM / 2>{}, dst_a1, dst_b1, 1);
    });
  };

  // All loads of one unit of an operand in a burst (prologue and tail).  `unit` counts tiles for a
  // K-major operand and slabs for an MN-major one; the last units get their K tail masked.
  auto burst_a = [&](int unit) {
    const int krem = klen - unit * OpA::UNIT_K;
    if (krem < OpA::UNIT_K) opa.mask_k_tail(krem, wave, lane);
    const i32x4 r = opa.rsrc();
    const uint32_t dst = lds0 + (uint32_t)(unit % OpA::UNITS) * OpA::IMG + opa.lds_w;
    static_for<IA>([&](auto lc) {
      constexpr int J = decltype(lc)::value;
      if constexpr (J % 4 == 0) dma_set_m0(dst + (J / 4) * 4096);
      opa.template issue_one<J>(r);
    });
    opa.advance();
  };
  auto burst_b = [&](int unit) {
    const int krem = klen - unit * OpB::UNIT_K;
    if (krem < OpB::UNIT_K) opb.mask_k_tail(krem, wave, lane);
    const i32x4 r = opb.rsrc();
    const uint32_t dst = lds0 + A_BYTES + (uint32_t)(unit % OpB::UNITS) * OpB::IMG + opb.lds_w;
    static_for<IB>([&](auto lc) {
      constexpr int J = decltype(lc)::value;
      if constexpr (J % 4 == 0) dma_set_m0(dst + (J / 4) * 4096);
      opb.template issue_one<J>(r);
    });
    opb.advance();
  };

  // Wait until this wave's loads of the slab about to be read have landed (all but the `keep` most
  // recent loads), and its own LDS reads are done; then meet the other waves.
  auto sync = [&](auto keep) {
    constexpr int KEEP = decltype(keep)::value;
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (PROF) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      const unsigned long long t0 = __builtin_readcyclecounter();
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(KEEP), "s"(t0) : "memory");
      const unsigned long long t1 = __builtin_readcyclecounter();
      asm volatile("s_waitcnt lgkmcnt(0)" ::"s"(t1) : "memory");
      __builtin_amdgcn_s_barrier();
      const unsigned long long t2 = __builtin_readcyclecounter();
      asm volatile("s_waitcnt lgkmcnt(0)" ::"s"(t2) : "memory");
      t_loads += t1 - t0;
      t_barrier += t2 - t1;
    } else {
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(KEEP) : "memory");
      __builtin_amdgcn_s_barrier();
    }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };
  using T = std::true_type;
  using F = std::false_type;

  // One iteration j of the main loop is: sync, then the MFMAs of slab j while the fragments of slab j+1 are read.
  // After the sync every wave holds all fragments of slab j in registers and slab j+1 has landed, so
  //   an MN-major slab image j & 3 is dead and takes slab j+4;
  //   for odd j the K-major tile image (j >> 1) % U (U images) is dead and takes tile (j >> 1) + U.
  // Steady state, period t (iterations j = 2t+1 and 2t+2; P0, P1 are the halves of the first, P2, P3 of the
  // second), what is issued and what each sync keeps in flight (loads complete in issue order):
  //   one K-major operand X (three images), the other Y MN-major:
  //     P0: first half of X tile t+3      P1: the rest of it      P2: Y slab 2t+5      P3: Y slab 2t+6
  //     the sync before P0 needs X tile t+1 and Y slab 2t+2: all but the loads of the period before
  //     the sync before P2 needs Y slab 2t+3: all but Y slab 2t+4 and X tile t+3
  //   both K-major (A three images, B two): P0: B tile t+2, P1..P3: A tile t+3
  //     the sync before P0 needs A tile t+1 and B tile t+1: all but A tile t+2
  //   (B three images: P0: B tile t+3; the sync before P0 keeps B tile t+2 and A tile t+2 in flight)
  //     no loads land between the sync before P0 and the reads of slab 2t+3: no second sync
  constexpr int KEEP_ODD = (AK && BK) ? IA + (NB_KK == 3 ? IB : 0) : (IA + IB + (AK ? IB : IA));
  constexpr int KEEP_EVEN = (AK && BK) ? -1 : IA + IB;

  // prologue: every image of both operands is requested, what slabs 0 and 1 need first, and only that
  // is waited for (units past K are requested too, fully masked: the counts below hold for any K).
  //   K-major A next to MN-major B: A0 B0 B1 | A1 B2 B3 A2      (mirrored if B is the K-major one)
  //   both K-major:                 A0 B0 | A1 B1 A2 (B2)
  constexpr int KEEP_PRO = (AK && BK) ? 2 * IA + IB + (NB_KK == 3 ? IB : 0) : 2 * IA + 2 * IB;
  if constexpr (AK && BK) {
    burst_a(0); burst_b(0); burst_a(1); burst_b(1); burst_a(2);
    if constexpr (NB_KK == 3) burst_b(2);
  } else if constexpr (AK) {
    burst_a(0); burst_b(0); burst_b(1); burst_a(1); burst_b(2); burst_b(3); burst_a(2);
  } else {
    burst_b(0); burst_a(0); burst_a(1); burst_b(1); burst_a(2); burst_a(3); burst_b(2);
  }
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(KEEP_PRO) : "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
#pragma unroll
  for (int t = 0; t < TM; ++t) af[0][t] = fa.read(img_a(0), t, 0);
#pragma unroll
  for (int t = 0; t < TN; ++t) bfr[0][t] = fb.read(img_b(0), t, 0);

  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  using NoLoads = std::integral_constant<int, -1>;
  // iteration with loads in a burst and full waits: j = 0, and the tail
  auto slow_iteration = [&](auto par, auto keep, int j) {
    sync(keep);
    if constexpr (!AK) { if (j + 4 < nslab) burst_a(j + 4); }
    if constexpr (!BK) { if (j + 4 < nslab) burst_b(j + 4); }
    if (j & 1) {
      if constexpr (AK) { if ((j >> 1) + OpA::UNITS < ntile) burst_a((j >> 1) + OpA::UNITS); }
      if constexpr (BK) { if ((j >> 1) + OpB::UNITS < ntile) burst_b((j >> 1) + OpB::UNITS); }
    }
    slab_step(par, T{}, j + 1, img_a(j + 1), img_b(j + 1), NoLoads{}, NoLoads{}, 0, 0, 0, 0);
  };
  slow_iteration(P0{}, std::integral_constant<int, KEEP_PRO>{}, 0);  // nothing was issued since the prologue's wait

  int j = 1;
  // steady: four periods per trip (the MN-major slab images repeat every four slabs, the K-major tile
  // images rotate at run time; two periods would do, four halve the cost of the loop branch: +0.5 %);
  // every unit loaded here exists and is full
  uint32_t x_ld = 0, x_rd = 1;  // of three tile images: the one that takes tile t+3 (= image of tile t) / that holds tile t+1
  for (; (j >> 1) + 6 < ntile - 1; j += 8) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      // period t = (j >> 1) + u, t & 1 == (u & 1) since j == 1 (mod 8)
      const int jo = j + 2 * u;  // the odd slab 2t+1
      // image index for loads in the first / second half of the period and for reads of slabs 2t+2 / 2t+3:
      //   four slab images: slabs 2t+5, 2t+6 go to (2t+1) & 3, (2t+2) & 3
      //   three tile images: rotate at run time; two: tile t+2 goes to t & 1, tile t+1 is read
      auto idx = [&](int units, int ld_or_rd, int second) -> uint32_t {
        if (units == 4) return (uint32_t)((2 * u + 1 + ld_or_rd + second) & 3);
        if (units == 3) return ld_or_rd ? x_rd : x_ld;
        return (uint32_t)((u + ld_or_rd) & 1);
      };
      const uint32_t da0 = lds0 + idx(OpA::UNITS, 0, 0) * OpA::IMG, da1 = lds0 + idx(OpA::UNITS, 0, 1) * OpA::IMG;
      const uint32_t db0 = lds0 + A_BYTES + idx(OpB::UNITS, 0, 0) * OpB::IMG,
                     db1 = lds0 + A_BYTES + idx(OpB::UNITS, 0, 1) * OpB::IMG;
      const uint32_t ra0 = idx(OpA::UNITS, 1, 0) * OpA::IMG, ra1 = idx(OpA::UNITS, 1, 1) * OpA::IMG;
      const uint32_t rb0 = idx(OpB::UNITS, 1, 0) * OpB::IMG, rb1 = idx(OpB::UNITS, 1, 1) * OpB::IMG;
      sync(std::integral_constant<int, KEEP_ODD>{});
      slab_step(P1{}, T{}, jo + 1, ra0, rb0, std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{}, da0, db0,
                da0, db0);
      if constexpr (KEEP_EVEN >= 0) sync(std::integral_constant<int, KEEP_EVEN>{});
      slab_step(P0{}, T{}, jo + 2, ra1, rb1, std::integral_constant<int, 2>{}, std::integral_constant<int, 3>{}, da0, db0,
                da1, db1);
      x_ld = x_rd;
      x_rd = x_rd + 1 == 3 ? 0 : x_rd + 1;
    }
  }
  // j is odd and nslab even: the tail is whole pairs of iterations
  for (; j + 1 < nslab; j += 2) {
    slow_iteration(P1{}, std::integral_constant<int, 0>{}, j);
    slow_iteration(P0{}, std::integral_constant<int, 0>{}, j + 1);
  }
  // the last slab (odd): its fragments are in registers or on their way from LDS
  slab_step(P1{}, F{}, 0, 0, 0, NoLoads{}, NoLoads{}, 0, 0, 0, 0);

  // The last MFMAs must have left the pipe before their accumulators are read, and the compiler,
  // which sees neither MFMAs nor hazard here, inserts nothing.  Volatile asm statements keep their
  // order, so the empty ones below, which redefine every accumulator, pin all later reads behind the NOPs.
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int jn = 0; jn < TN; ++jn) asm volatile("" : "+a"(acc[i][jn]));
  unsigned long long t_main = 0;
  if constexpr (PROF) t_main = __builtin_readcyclecounter();

  store_wave_tile<TM, TN, NW, LDS_BYTES>(acc, p, gC, kz, lane, wave, lds0, BlockMap{m0 + wm * WTM, n0 + wn * WTN});
  if constexpr (PROF) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const unsigned long long t_end = __builtin_readcyclecounter();
    if (lane == 0 && p.prof) {
      unsigned long long* o = p.prof + ((size_t)blockIdx.x * NW + wave) * 4;
      o[0] = t_end - t_start;
      o[1] = t_loads;
      o[2] = t_barrier;
      o[3] = t_end - t_main;
    }
  }
}

// CUs of the current device (the runtime is asked once per device)
inline hipError_t current_device_cus(int* out) {
  static std::atomic<int> cus_of[64];
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
  int cus = dev >= 0 && dev < 64 ? cus_of[dev].load(std::memory_order_relaxed) : 0;
  if (cus == 0) {
    if (hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev); e != hipSuccess) return e;
    if (dev >= 0 && dev < 64) cus_of[dev].store(cus, std::memory_order_relaxed);
  }
  *out = cus;
  return hipSuccess;
}

// Raise a kernel's dynamic-LDS limit once per (kernel, device): the attribute belongs to the current device's copy
// of the function.  The registry is keyed on the kernel's address (all instances share one function-pointer type).
template <class Kern>
static hipError_t allow_lds(Kern kern, size_t lds) {
  static std::mutex mu;
  static std::map<const void*, uint64_t> done;  // kernel -> one bit per device index
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = 1ull << (dev & 63);
  std::lock_guard<std::mutex> lock(mu);
  uint64_t& mask = done[(const void*)kern];
  if (dev > 63 || !(mask & bit)) {
    e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    mask |= bit;
  }
  return hipSuccess;
}

template <int BM, int BN, int WGM, int WGN>
hipError_t launch_tile(const TileArgs& a, bool ak, bool bk, hipStream_t st) {
  // A: three 64-deep images if K-major, else four 32-deep ones; B likewise, but two or three 64-deep ones if both are K-major
  size_t lds = (size_t)BM * (ak ? 384 : 256) + (size_t)BN * (bk ? (ak ? b_images_both_kmajor(BM, BN) * 128 : 384) : 256);
  dim3 grid(a.ntm * a.ntn * a.ksplit, 1, a.batch), block(WGM * WGN * 64);
  auto go = [&](auto kern) -> hipError_t {
    if (hipError_t e = allow_lds(kern, lds); e != hipSuccess) return e;
    kern<<<grid, block, lds, st>>>(a);
    return hipGetLastError();
  };
  if (a.prof) {
    if constexpr (BM == 256 && BN == 256) {
      if (ak && bk) return go(gemm_tile_kernel<BM, BN, WGM, WGN, true, true, true>);
      if (ak && !bk) return go(gemm_tile_kernel<BM, BN, WGM, WGN, true, false, true>);
    }
    return hipErrorInvalidValue;
  }
  if (ak && bk) {
    if constexpr (BM == 128 && BN == 128) {
      // more workgroups than CUs: two images of B, 80 KiB, so that two workgroups share a CU
      int cus = 0;
      if (hipError_t e = current_device_cus(&cus); e != hipSuccess) return e;
      if ((int64_t)a.ntm * a.ntn * a.ksplit * a.batch > cus) {
        lds = (size_t)BM * 384 + (size_t)BN * 256;
        return go(gemm_tile_kernel<BM, BN, WGM, WGN, true, true, false, 2>);
      }
    }
    return go(gemm_tile_kernel<BM, BN, WGM, WGN, true, true>);
  }
  if (ak && !bk) {
    if constexpr (BN >= 128 && (BN & (BN - 1)) == 0) return go(gemm_tile_kernel<BM, BN, WGM, WGN, true, false>);
  }
  if (!ak && bk) {
    if constexpr (BM >= 128 && (BM & (BM - 1)) == 0) return go(gemm_tile_kernel<BM, BN, WGM, WGN, false, true>);
  }
  return hipErrorInvalidValue;
}

// ---------------------------------------------------------------------------------------------
// 256x256 tile, K in periods of 64 (two MFMA steps), both steps of an accumulator tile back to back.
// A v_mfma that accumulates into the tile the instruction before it wrote takes that operand from the pipeline
// instead of the register file, and with the walk below every MFMA either does that or shares one operand
// register with the one before it: the matrix cores alone sustain 3 % more on N(0,1) operands than with the walk
// of gemm_tile_kernel (matmul_bench ceiling, rows mfma_order), and under the chip's power limit that is clock.
// Both steps of a tile in a row need the fragments of two K steps in registers at once, so the roles of the operands
// are uneven: A's sixteen fragments (8 row tiles x 2 steps) of the current period sit in registers, double-buffered
// across periods; B streams: the wave goes through its eight column tiles in pairs, four fragments per pair, read
// from LDS while the pair before it is being worked on.  40 fragments live at most.
//     period q:  column pair 0..3 (32 MFMAs each): row blocks of two tiles, in alternating direction;
//                a block (2 columns x 2 rows x 2 steps) goes (c0,i0,k0) (c0,i0,k1) (c0,i1,k0) (c0,i1,k1) (c1,i1,k0) ...
// LDS: A two 64-deep tile images (32 KiB each), B three (K-major: a tile image; MN-major: two 32-deep slab images),
// laid out and swizzled as in gemm_tile_kernel.  During period q a wave loads A tile q+2 over tile q (whose fragments
// it read during the last third of period q-1) and B tile q+2 over tile q-1: one load behind every seventh MFMA, the
// last of the sixteen behind MFMA 107 of 128.
// Two barriers per period: at its start (everyone is done reading what the period's loads overwrite) and before MFMA 88
// (A tile q+1 and B tile q+1, requested during period q-1, have landed: they are read during the rest of the period).
// K is a multiple of 128 and not split; a tile past the end of K is requested all the same, as a zero fill.
// ---------------------------------------------------------------------------------------------
template <bool BK>
__global__ __launch_bounds__(256) void gemm_chain_kernel(TileArgs p) {
  constexpr int BM = 256, BN = 256, NW = 4, TM = 8, TN = 8;
  using OpA = Operand<BM, true, NW, 2>;
  using OpB = Operand<BN, BK, NW, BK ? 3 : 6>;
  constexpr uint32_t A_BYTES = 2 * 32768, B_IMG = 32768, LDS_BYTES = A_BYTES + 3 * B_IMG;
  constexpr int IA = OpA::IPW, IB = OpB::IPW;          // loads of this wave per unit (A: a tile; B: a tile or a slab)
  constexpr int UB = KTILE / OpB::UNIT_K, LB = IB * UB;  // B units, B loads per period
  static_assert(IA == 8 && LB == 8, "eight loads per operand, wave and period");
  constexpr int LOAD_STEP = 7;   // a load behind every LOAD_STEP-th MFMA from the third on: the sixteenth behind MFMA 107
  constexpr int LANDED_AT = 88;  // MFMA of the period before which the barrier for tile q+1 sits (even, 64..96); both tuned on the GPU

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(NEOGEMM_AS3 char*)smem;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  int m0, n0, kz;
  tile_of_workgroup<BM, BN>(p, m0, n0, kz);
  const int klen = p.K;  // not split
  const int ntile = klen / KTILE;

  const char* gA = p.A + (size_t)blockIdx.z * p.bsa * 2;
  const char* gB = p.B + (size_t)blockIdx.z * p.bsb * 2;
  char* gC = p.C + (size_t)blockIdx.z * p.bsc * 2;
  OpA opa;
  OpB opb;
  opa.init(gA, p.lda, p.M, m0, 0, wave, lane);
  opb.init(gB, p.ldb, p.N, n0, 0, wave, lane);
  FragReader<BM, true, TM> fra;
  FragReader<BN, BK, TN> frb;
  fra.init(lds0, wm * 128, lane);
  frb.init(lds0 + A_BYTES, wn * 128, lane);

  f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;

  // load l (0..7) of the tile an operand loads next, into the image at `img` (offset within the operand's region)
  int ta = 0, tb = 0;  // tile the next A / B loads belong to
  auto load_a = [&](auto lc, uint32_t img) {
    constexpr int J = decltype(lc)::value;
    if constexpr (J % 4 == 0) dma_set_m0(lds0 + img + opa.lds_w + (J / 4) * 4096);
    opa.template issue_one<J>(opa.rsrc(ta < ntile));
    if constexpr (J == IA - 1) {
      opa.advance();
      ++ta;
    }
  };
  auto load_b = [&](auto lc, uint32_t img) {
    constexpr int l = decltype(lc)::value, u = l / IB, J = l % IB;
    if constexpr (J % 4 == 0) dma_set_m0(lds0 + A_BYTES + img + u * OpB::IMG + opb.lds_w + (J / 4) * 4096);
    opb.template issue_one<J>(opb.rsrc(tb < ntile));
    if constexpr (J == IB - 1) {
      opb.advance();
      if constexpr (u == UB - 1) ++tb;
    }
  };

  // B fragments of column tile c (0..7), step k, from the B image at region offset `img`
  auto read_b = [&](uint32_t img, int c, int k) -> bf16x8 {
    if constexpr (BK) {
      return lds_read_b128(frb.lane_off[k] + img + (uint32_t)c * 2048);
    } else {
      const uint32_t a = frb.lane_off[c] + img + (uint32_t)k * OpB::IMG;
      const i16x8 v = __builtin_shufflevector(lds_read_tr16(a), lds_read_tr16(a + 4 * FragReader<BN, BK, TN>::ROWB), 0, 1, 2,
                                              3, 4, 5, 6, 7);
      return __builtin_bit_cast(bf16x8, v);
    }
  };

  auto barrier = [&](auto keep, auto lgk) {
    constexpr int KEEP = decltype(keep)::value;
    constexpr bool LGK = decltype(lgk)::value;
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (KEEP >= 0 && LGK) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(KEEP) : "memory");
    else if constexpr (KEEP >= 0) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(KEEP) : "memory");
    else if constexpr (LGK) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };
  using NoVm = std::integral_constant<int, -1>;
  using T = std::true_type;
  using F = std::false_type;

  // fragments: fa[buffer][row tile][step], the buffer is the tile's parity; fb[column pair parity][column][step]
  bf16x8 fa[2][TM][2] = {}, fb[2][2][2] = {};

  // prologue: tiles 0 and 1 of both operands; tile 0 of A and the first column pair of B's tile 0 into registers
  uint32_t b_cur = 0, b_nxt = B_IMG, b_ld = 2 * B_IMG;  // B images: this period's tile, the next one's, the one being loaded
  static_for<IA>([&](auto lc) { load_a(lc, 0); });
  static_for<LB>([&](auto lc) { load_b(lc, b_cur); });
  static_for<IA>([&](auto lc) { load_a(lc, 32768); });
  static_for<LB>([&](auto lc) { load_b(lc, b_nxt); });
  barrier(std::integral_constant<int, IA + LB>{}, F{});
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int k = 0; k < 2; ++k) fa[0][i][k] = fra.read(0, i, k);
#pragma unroll
  for (int c = 0; c < 2; ++c)
#pragma unroll
    for (int k = 0; k < 2; ++k) fb[0][c][k] = read_b(b_cur, c, k);

  for (int q = 0; q < ntile; q += 2) {
    static_for<256>([&](auto mc) {
      constexpr int m2 = decltype(mc)::value, par = m2 / 128, m = m2 % 128;  // par: parity of the tile = A buffer and image
      constexpr int cp = m / 32, e = m % 8;
      constexpr int rb = (cp & 1) ? 3 - (m % 32) / 8 : (m % 32) / 8;
      constexpr int c = e / 4, i = rb * 2 + (((e + 2) >> 2) & 1), k = e & 1;  // k ascending on every tile: the sum's order is that of gemm_tile_kernel
      // ---- barriers
      if constexpr (m == 0) barrier(NoVm{}, T{});                                          // the images this period loads into are free
      if constexpr (m == LANDED_AT) barrier(std::integral_constant<int, (LANDED_AT - 2 + LOAD_STEP - 1) / LOAD_STEP < IA + LB ? (LANDED_AT - 2 + LOAD_STEP - 1) / LOAD_STEP : IA + LB>{}, F{});  // tile q+1 of A and of B has landed
      // ---- the MFMA
      mfma_16x16x32(acc[i][cp * 2 + c], fb[cp & 1][c][k], fa[par][i][k]);
      // ---- LDS reads behind it
      // B: the next column pair's four fragments, early in this one (the last pair reads the first of the next tile,
      // which the barrier before has seen land); a K-major fragment is one 16-byte read, an MN-major one two
      // transposing 8-byte reads, each behind an MFMA of its own
      if constexpr (BK) {
        if constexpr (m % 32 < 16 && (m % 4) == 1) {
          constexpr int j = (m % 32) / 4, cc = j / 2, kk = j % 2;
          if constexpr (cp < 3) fb[(cp + 1) & 1][cc][kk] = read_b(b_cur, (cp + 1) * 2 + cc, kk);
          else fb[0][cc][kk] = read_b(b_nxt, cc, kk);
        }
      } else {
        if constexpr (m % 32 < 16 && (m % 2) == 1) {
          constexpr int idx = (m % 32) / 2, j = idx / 2, h = idx % 2, cc = j / 2, kk = j % 2;
          constexpr int nb = cp < 3 ? (cp + 1) & 1 : 0, ct = cp < 3 ? (cp + 1) * 2 + cc : cc;
          const uint32_t a = frb.lane_off[ct] + (cp < 3 ? b_cur : b_nxt) + (uint32_t)kk * OpB::IMG + h * 4 * FragReader<BN, BK, TN>::ROWB;
          fb[nb][cc][kk] = with_half(fb[nb][cc][kk], lds_read_tr16(a), h);
        }
      }
      // A: the next tile's sixteen fragments behind the even MFMAs LANDED_AT .. LANDED_AT + 30 (B's reads sit behind odd ones); done well
      // before the period ends, where the next one's first barrier waits for them
      if constexpr (m >= LANDED_AT && m < LANDED_AT + 32 && (m % 2) == 0) {
        constexpr int j = (m - LANDED_AT) / 2, ii = j / 2, kk = j % 2;
        fa[par ^ 1][ii][kk] = fra.read((par ^ 1) * 32768, ii, kk);
      }
      // ---- loads behind it: one every LOAD_STEP MFMAs, A's tile q+2 over tile q, then B's over tile q-1
      if constexpr (m >= 2 && (m - 2) % LOAD_STEP == 0 && (m - 2) / LOAD_STEP < IA + LB) {
        constexpr int l = (m - 2) / LOAD_STEP;
        if constexpr (l < IA) load_a(std::integral_constant<int, l>{}, par * 32768);
        else load_b(std::integral_constant<int, l - IA>{}, b_ld);
      }
      // ---- end of the period: the B images change roles
      if constexpr (m == 127) {
        const uint32_t t = b_cur;
        b_cur = b_nxt;
        b_nxt = b_ld;
        b_ld = t;
      }
    });
  }

  // the last MFMAs must have left the pipe before their accumulators are read (see gemm_tile_kernel)
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int jn = 0; jn < TN; ++jn) asm volatile("" : "+a"(acc[i][jn]));
  // With one round of workgroups the whole chip reaches its epilogue at once and nothing overlaps it: staging a quarter
  // of the wave tile at a time gets the first stores on their way after a quarter of the conversions (4096^3 and
  // 3000x5120x3584: -0.5 %); with several rounds the plain staging is 0.5 % ahead (8192^3).
  if (p.early_stores) store_wave_tile<TM, TN, NW, LDS_BYTES, TM / 4>(acc, p, gC, kz, lane, wave, lds0, BlockMap{m0 + wm * 128, n0 + wn * 128});
  else store_wave_tile<TM, TN, NW, LDS_BYTES>(acc, p, gC, kz, lane, wave, lds0, BlockMap{m0 + wm * 128, n0 + wn * 128});
}

hipError_t launch_chain(const TileArgs& a, bool bk, hipStream_t st);
#if NEOGEMM_HAS_PART(8)
hipError_t launch_chain(const TileArgs& a, bool bk, hipStream_t st) {
  const size_t lds = 5 * 32768;
  // one round of workgroups or several (one workgroup per CU)
  int cus = 0;
  if (hipError_t e = current_device_cus(&cus); e != hipSuccess) return e;
  TileArgs b = a;
  b.early_stores = (int64_t)a.ntm * a.ntn * a.batch <= cus;
  dim3 grid(a.ntm * a.ntn, 1, a.batch), block(256);
  auto go = [&](auto kern) -> hipError_t {
    if (hipError_t e = allow_lds(kern, lds); e != hipSuccess) return e;
    kern<<<grid, block, lds, st>>>(b);
    return hipGetLastError();
  };
  return bk ? go(gemm_chain_kernel<true>) : go(gemm_chain_kernel<false>);
}
#endif

// The tile kernels are instantiated through launch_tile.  In a split build each part instantiates its share and
// the others only declare it.
#ifdef NEOGEMM_PART
#define NEOGEMM_TILE(BM, BN, WGM, WGN) \
  template hipError_t launch_tile<BM, BN, WGM, WGN>(const TileArgs&, bool, bool, hipStream_t);
#if NEOGEMM_PART == 1
NEOGEMM_TILE(256, 256, 2, 2)
#else
extern NEOGEMM_TILE(256, 256, 2, 2)
#endif
#if NEOGEMM_PART == 2
NEOGEMM_TILE(64, 128, 1, 4)
#else
extern NEOGEMM_TILE(64, 128, 1, 4)
#endif
#if NEOGEMM_PART == 3
NEOGEMM_TILE(128, 128, 2, 2)
#else
extern NEOGEMM_TILE(128, 128, 2, 2)
#endif
#if NEOGEMM_PART == 4
NEOGEMM_TILE(256, 128, 2, 2)
#else
extern NEOGEMM_TILE(256, 128, 2, 2)
#endif
#if NEOGEMM_PART == 5
NEOGEMM_TILE(128, 256, 2, 2)
#else
extern NEOGEMM_TILE(128, 256, 2, 2)
#endif
#if NEOGEMM_PART == 6
NEOGEMM_TILE(192, 256, 2, 2)
#else
extern NEOGEMM_TILE(192, 256, 2, 2)
#endif
#if NEOGEMM_PART == 7
NEOGEMM_TILE(96, 128, 2, 2)
NEOGEMM_TILE(64, 64, 2, 2)
#else
extern NEOGEMM_TILE(96, 128, 2, 2)
extern NEOGEMM_TILE(64, 64, 2, 2)
#endif
#undef NEOGEMM_TILE
#endif

}  // namespace neogemm

// Everything below — the other kernels, the planner, the launcher and the C ABI — belongs to part 0 of a
// split build (see NEOGEMM_PART at the top of the file).
#if NEOGEMM_HAS_PART(0)
namespace neogemm {

// ---------------------------------------------------------------------------------------------
// Skinny M (decode shapes: M <= 16 * TMF; C row-major or, CCOL, column-major): bound by streaming B from HBM once, so what
// counts is bytes in flight per CU, not MFMA rate.  A workgroup owns a strip of columns of C (64 with B [K,N]; with
// B [N,K] as many, in eights up to 64, as fill the CUs in whole rounds: SkinnyArgs::strip, steps of SW = 16, 32 or 64
// rows of B) and the whole of K; no split-K, no second launch.  Its four waves split K between them in steps of 64,
// each with a private ring of RS steps in LDS that only it fills and reads:
// no barrier until the end, when the four partial sums meet in LDS and are added in wave order.
// One step of one wave: A 16*TMF rows x 128 B (K-major image, swz_k), B 64 k-rows x 128 B if B is [K,N]
// (64 columns are one cache line per k-row; swizzle swz_mn64) or SW rows x 128 B if B is [N,K].
// 4 waves x (RA steps of A at 2 KiB * TMF + RS steps of B at SW * 128 B) of LDS, with SW = 64: TMF = 1 with rings of 4 fills the 160 KiB;
// TMF = 2 with 3 and TMF = 4 with 2 (M <= 64: 30.5 us at 64x14336x4096, the split-K tile path 32.9) are the other
// instances for up to 64 rows.  TMF = 5 .. 8 (up to 128 rows) fit two steps of each at most, or one of A and three of B.
// A wave's loads complete in the order it issued them, so a ring deeper than the other operand's buys little: with one
// step of A, B's third step shortens 96 x 14336 x 4096 by 3 % where a second step of A shortens it by 6 %.
// (Fetching the fragments straight into registers instead, which would hold three steps of both, was slower by 40 %:
// a fragment load touches 16 rows x 64 bytes, half a line each, and the vector L1 charges by the line.)
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t swz_mn64(uint32_t kk) {
  // k-row kk (0..31 within a slab) of a 64-column MN-major image: even values 0..6 XOR-ed into the 16-byte chunk
  // index, chosen so that the sixteen 32-byte pieces of one transposing read spread over the banks
  return ((((kk >> 3) & 3u) ^ (((kk >> 1) & 1u) << 1)) << 1);
}
struct SkinnyArgs {
  const char* A;
  const char* B;
  char* C;
  int M, N, K;
  long lda, ldb, ldc;
  float alpha, beta;
  int rot;    // nonzero: workgroup b starts b (b + 1) / 2 steps into its waves' shares of K and wraps around (gemm_strip_kernel:
              // at a stage of its run that is a hash of the strip's number)
  int strip;  // columns of C per workgroup: 64, or with B [N,K] a smaller multiple of 8 that fills the CUs better
  int ra, rb; // gemm_strip_kernel: stages in the ring of A / of B
  // gemm_strip_kernel with K split over ksplit workgroups per strip (0 or 1: none): runs of stages_per_split 128-deep
  // stages; the partial sums go to ws as fp32, [ksplit] matrices of the shape C has in memory, for splitk_reduce_kernel
  int ksplit, stages_per_split;
  float* ws;
};
// One fragment of partial sums to the split-K workspace: `part` is this split's matrix, dense, laid out as C is in
// memory (row-major M x N, or N x M for a column-major C).
template <bool CCOL>
__device__ __forceinline__ void skinny_store_partial(f32x4 sum, int t, int f, const SkinnyArgs& p, int n0, int lane, float* part) {
  const uint32_t frow = lane & 15, fq = (uint32_t)lane >> 4;
  const int row = CCOL ? 16 * t + 4 * (int)fq : 16 * t + (int)frow;
  const int col = CCOL ? n0 + 16 * f + (int)frow : n0 + 16 * f + 4 * (int)fq;
  const int col_end = n0 + p.strip < p.N ? n0 + p.strip : p.N;
  if (row >= p.M || col >= col_end) return;
  const int fast = CCOL ? row : col, fast_end = CCOL ? p.M : col_end, ld = CCOL ? p.M : p.N;
  float* wp = part + (CCOL ? (size_t)col * p.M + row : (size_t)row * p.N + col);
  if (fast + 3 < fast_end && (ld & 3) == 0) {
    *(f32x4*)wp = sum;
  } else {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (fast + r < fast_end) wp[r] = sum[r];
  }
}
// One 16x16 fragment of sums (row fragment t, column fragment f of the strip at column n0) scaled and written to C.
// The lane's four elements are consecutive along `fast` (n for a row-major C, m for a column-major one).
template <bool CCOL>
__device__ __forceinline__ void skinny_store_frag(f32x4 sum, int t, int f, const SkinnyArgs& p, int n0, int lane) {
  const uint32_t frow = lane & 15, fq = (uint32_t)lane >> 4;
  const int row = CCOL ? 16 * t + 4 * (int)fq : 16 * t + (int)frow;
  const int col = CCOL ? n0 + 16 * f + (int)frow : n0 + 16 * f + 4 * (int)fq;
  const int col_end = n0 + p.strip < p.N ? n0 + p.strip : p.N;  // a strip may be narrower than its fragments
  if (row >= p.M || col >= col_end) return;
  const int fast = CCOL ? row : col, fast_end = CCOL ? p.M : col_end;
  char* cp = p.C + (CCOL ? (size_t)col * p.ldc + row : (size_t)row * p.ldc + col) * 2;
#pragma unroll
  for (int r = 0; r < 4; ++r) sum[r] *= p.alpha;
  if (p.beta != 0.f) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (fast + r < fast_end) sum[r] = __builtin_fmaf(p.beta, (float)((const __bf16*)cp)[r], sum[r]);
  }
  const bf16x4 o = {(__bf16)sum[0], (__bf16)sum[1], (__bf16)sum[2], (__bf16)sum[3]};
  if (fast + 3 < fast_end) {
    *(bf16x4*)cp = o;
  } else {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (fast + r < fast_end) ((__bf16*)cp)[r] = o[r];
  }
}
// The end of the skinny kernels: the partial sums of the four waves (each over its share of K) meet in LDS (16 KiB * TMF
// from `smem` on, which no wave may still be using) and wave w adds up fragment column w in wave order, scales and stores.
template <int TMF, bool CCOL, int NF>
__device__ __forceinline__ void skinny_reduce_store(f32x4 (&acc)[TMF][NF], const SkinnyArgs& p, int n0, int wave, int lane,
                                                    char* smem) {
  NEOGEMM_AS3 f32x4* red = (NEOGEMM_AS3 f32x4*)smem;
#pragma unroll
  for (int t = 0; t < TMF; ++t)
#pragma unroll
    for (int f = 0; f < NF; ++f) red[((wave * TMF + t) * NF + f) * 64 + lane] = acc[t][f];
  __syncthreads();
  // fragment i = t * NF + f goes to wave i mod 4 (with four fragment columns: column w to wave w)
  for (int i = wave; i < TMF * NF; i += 4) {
    const int t = i / NF, f = i % NF;
    f32x4 sum = red[i * 64 + lane];
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      const f32x4 v = red[(w * TMF * NF + i) * 64 + lane];
#pragma unroll
      for (int r = 0; r < 4; ++r) sum[r] += v[r];
    }
    skinny_store_frag<CCOL>(sum, t, f, p, n0, lane);
  }
}

template <int TMF, int RS, bool BKM, bool CCOL = false, int RA = RS, int SW = 64>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(SkinnyArgs p) {
  constexpr int BM = 16 * TMF, NF = SW / 16;  // rows of A, 16-column fragments of the strip
  constexpr uint32_t A_STEP = BM * 128, B_STEP = SW * 128, WAVE_LDS = RA * A_STEP + RS * B_STEP;
  constexpr int NA = A_STEP / 1024, NB = B_STEP / 1024, LP = NA + NB;  // 1 KiB loads per step
  static_assert(SW == 64 || (BKM && (SW == 32 || SW == 16)), "narrow strips only of a K-major B (whole lines per row)");
  static_assert(RA >= 1 && RA <= RS, "A comes from L2 (every workgroup reads all of it): its ring may be the shorter one");
  static_assert(4u * WAVE_LDS <= 160u * 1024u, "the four waves' rings must fit the LDS");
  static_assert(4u * TMF * NF * 64u * 16u <= 4u * WAVE_LDS, "the rings double as the reduction buffer");
  static_assert((RA - 1) * LP + (RA < RS ? NB : 0) <= 63 && RA * NA + RS * NB <= 64, "the wait counts must fit the counter");
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(NEOGEMM_AS3 char*)smem;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // workgroup -> strip: consecutive workgroup ids land on different XCDs; with a K-major wide operand id % 8 selects a
  // contiguous run of strips (up to 1.5 % at K = 8192; with B [K,N], where neighbouring strips are neighbouring cache
  // lines of every k-row, the plain order is 0.5 % ahead)
  const int per = gridDim.x >> 3, rem = gridDim.x & 7, xcd = blockIdx.x & 7;
  const int strip_id = BKM ? xcd * per + (xcd < rem ? xcd : rem) + (blockIdx.x >> 3) : (int)blockIdx.x;
  const int n0 = strip_id * p.strip;
  const int nsteps = (p.K + KTILE - 1) / KTILE;
  const uint32_t ring_a = lds0 + (uint32_t)wave * WAVE_LDS, ring_b = ring_a + RA * A_STEP;

  // per-lane byte offsets of the loads of one step, relative to the step's first element of A / B; a load
  // carries the instruction offset (j & 3) * 1024 (see Operand::init), OOB_OFFSET where nothing is to be read
  uint32_t voa[NA], vob[NB];
#pragma unroll
  for (int j = 0; j < NA; ++j) {
    const uint32_t row = 8 * j + (lane >> 3), c = (lane & 7) ^ swz_k(row);
    voa[j] = row * (uint32_t)p.lda * 2 + c * 16 + VOFF_BIAS - (j & 3) * 1024;
    if ((int)row >= p.M) voa[j] = OOB_OFFSET;
  }
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    const uint32_t r = 8 * j + (lane >> 3);  // k-row of the step ([K,N]) or column of the strip ([N,K])
    if constexpr (BKM) {
      const uint32_t c = (lane & 7) ^ swz_k(r);
      vob[j] = r * (uint32_t)p.ldb * 2 + c * 16 + VOFF_BIAS - (j & 3) * 1024;
      if (n0 + (int)r >= p.N || (int)r >= p.strip) vob[j] = OOB_OFFSET;  // rows past the strip: still issued, as zero fills
    } else {
      const uint32_t c = (lane & 7) ^ swz_mn64(r & 31);
      vob[j] = r * (uint32_t)p.ldb * 2 + c * 16 + VOFF_BIAS - (j & 3) * 1024;
      if (n0 + (int)c * 8 >= p.N) vob[j] = OOB_OFFSET;
    }
  }
  // Which steps this wave takes: every fourth one if B is [K,N] (the four waves then read neighbouring k-rows),
  // a contiguous quarter of K if B is [N,K] (each wave then walks along the rows of B: 9 % faster, measured;
  // the other way round is 2 % slower for [K,N]).
  const int qsteps = (nsteps + 3) / 4;
  const int s_begin = BKM ? wave * qsteps : wave, s_stride = BKM ? 1 : 4;
  const int s_end = BKM ? (s_begin + qsteps < nsteps ? s_begin + qsteps : nsteps) : nsteps;
  auto rsrc = [](uint64_t base) {
    i32x4 r;
    base -= VOFF_BIAS;
    r[0] = (int)(uint32_t)base;
    r[1] = (int)(uint32_t)(base >> 32);
    r[2] = (int)0x80000000u;
    r[3] = 0x00020000;
    return r;
  };
  // all loads of A / of B of step s of this wave into slot `slot` of that operand's ring; past K everything is
  // masked (the loads are still issued, as zero fills, so that the count of loads in flight does not depend on K)
  // Rows of a K-major B that lie a multiple of 16 KiB apart (K a multiple of 8192) and are all read at the same depth
  // crowd onto a few memory channels: 16 x 14336 x 8192 runs 20 % faster, K = 16384 44 %, when every workgroup starts
  // at another depth (other K: -3 .. +2 %, B [K,N]: -1 .. -5 %, so only there).  Strip b starts b (b + 1) / 2 steps in,
  // not b: a fixed number of steps per strip can cancel against the distance between the strips in the address hash of
  // the memory channels (b steps: 16 x 8192 x 8192, strips 512 KiB apart, 29.1 us; this way 25.8; 14336 and 28672 columns
  // 1 % slower).  The order of a wave's sums then depends on the strip, not on anything that varies from run to run.
  const int n_mine = s_end > s_begin ? (s_end - s_begin + s_stride - 1) / s_stride : 0;
  const int rot0 = p.rot && n_mine > 0 ? (int)((((unsigned)strip_id * ((unsigned)strip_id + 1u)) >> 1) % (unsigned)n_mine) : 0;
  auto turn = [&](int s) {  // the step taken at the place of step s
    if (!p.rot || s >= s_end) return s;
    int i = (s - s_begin) / s_stride + rot0;
    if (i >= n_mine) i -= n_mine;
    return s_begin + i * s_stride;
  };
  auto issue_a = [&](int s0, int slot) {
    const int s = turn(s0);
    const int krem = s < s_end ? p.K - s * KTILE : 0;  // depth left from this step on (<= 0: nothing)
    const uint32_t dst = ring_a + (uint32_t)slot * A_STEP;
    const i32x4 ra = rsrc((uint64_t)p.A + (uint64_t)s * KTILE * 2);
    static_for<NA>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      uint32_t v = voa[j];
      const uint32_t c = (lane & 7) ^ swz_k(8 * j + (lane >> 3));
      if ((int)c * 8 >= krem) v = OOB_OFFSET;
      if constexpr (j % 4 == 0) dma_set_m0(dst + (j / 4) * 4096);
      dma16<(j & 3) * 1024>(ra, v);
    });
  };
  auto issue_b = [&](int s0, int slot) {
    const int s = turn(s0);
    const int krem = s < s_end ? p.K - s * KTILE : 0;
    const uint32_t dst = ring_b + (uint32_t)slot * B_STEP;
    const i32x4 rb = rsrc((uint64_t)p.B + (BKM ? ((uint64_t)n0 * p.ldb + (uint64_t)s * KTILE) * 2
                                                : ((uint64_t)s * KTILE * p.ldb + n0) * 2));
    static_for<NB>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      uint32_t v = vob[j];
      const uint32_t r = 8 * j + (lane >> 3);
      if constexpr (BKM) {
        const uint32_t c = (lane & 7) ^ swz_k(r);
        if ((int)c * 8 >= krem) v = OOB_OFFSET;
      } else {
        if ((int)r >= krem) v = OOB_OFFSET;
      }
      if constexpr (j % 4 == 0) dma_set_m0(dst + (j / 4) * 4096);
      dma16<(j & 3) * 1024>(rb, v);
    });
  };

  f32x4 acc[TMF][NF];
#pragma unroll
  for (int t = 0; t < TMF; ++t)
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[t][f][v] = 0.f;

  // fragment addresses within a step image (see FragReader)
  const uint32_t frow = lane & 15, fq = (uint32_t)lane >> 4;
  uint32_t a_off[2];  // B [N,K]: the same image shape, 64 rows
#pragma unroll
  for (int sl = 0; sl < 2; ++sl) a_off[sl] = frow * 128 + (((4 * sl + fq) ^ swz_k(frow)) << 4);
  const uint32_t tr_r = frow >> 2, tr_c = frow & 3, kk = 8 * fq + tr_r;  // B [K,N]: k-row within a slab, the second read adds 4

  // Trip t of the loop asks for A of step t + RA, then for B of step t + RS; the prologue is trips -RS .. -1 of that
  // order.  At the top of trip t everything up to A of step t must have landed: behind it in the queue are the B loads
  // issued in the same trip as that A (none if RA == RS: that B is step t's own) and RA - 1 whole trips.
  static_for<RS>([&](auto rc) {
    constexpr int r = decltype(rc)::value;
    if constexpr (r + RA >= RS) issue_a(s_begin + s_stride * (r + RA - RS), r + RA - RS);
    issue_b(s_begin + s_stride * r, r);
  });
  int slot_a = 0, slot_b = 0;
  for (int s = s_begin; s < s_end; s += s_stride) {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((RA - 1) * LP + (RA < RS ? NB : 0)) : "memory");
    const uint32_t img_a = ring_a + (uint32_t)slot_a * A_STEP, img_b = ring_b + (uint32_t)slot_b * B_STEP;
    bf16x8 af[2][TMF], bf[2][NF];
#pragma unroll
    for (int sl = 0; sl < 2; ++sl) {
#pragma unroll
      for (int t = 0; t < TMF; ++t) af[sl][t] = lds_read_b128(img_a + a_off[sl] + t * 2048);
#pragma unroll
      for (int f = 0; f < NF; ++f) {
        if constexpr (BKM) {
          bf[sl][f] = lds_read_b128(img_b + a_off[sl] + f * 2048);
        } else {
          const uint32_t chunk = (2 * f + (tr_c >> 1)) ^ swz_mn64(kk);
          const uint32_t ad = img_b + (32 * sl + kk) * 128 + (chunk << 4) + ((tr_c & 1) << 3);
          const i16x4 lo = lds_read_tr16(ad), hi = lds_read_tr16(ad + 4 * 128);
          bf[sl][f] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
      }
    }
    // the fragments must be in registers before the next loads overwrite these slots
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    issue_a(s + s_stride * RA, slot_a);
    issue_b(s + s_stride * RS, slot_b);
    slot_a = slot_a + 1 == RA ? 0 : slot_a + 1;
    slot_b = slot_b + 1 == RS ? 0 : slot_b + 1;
#pragma unroll
    for (int sl = 0; sl < 2; ++sl)
#pragma unroll
      for (int t = 0; t < TMF; ++t)
#pragma unroll
        for (int f = 0; f < NF; ++f)
          // B fragment first: a lane ends up with 4 consecutive n of one output row (see gemm_tile_kernel);
          // for a column-major C the other way round: 4 consecutive m of one output column
          if constexpr (CCOL) acc[t][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[sl][t], bf[sl][f], acc[t][f], 0, 0, 0);
          else acc[t][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bf[sl][f], af[sl][t], acc[t][f], 0, 0, 0);
  }
  // drain the loads still in flight (zero fills past K included) before the rings become the reduction buffer
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  skinny_reduce_store<TMF, CCOL, NF>(acc, p, n0, wave, lane, smem);
}

// ---------------------------------------------------------------------------------------------
// 65 to 128 rows again: the same strips, with rings that the waves share and eight waves to fill them.
// What bounds these shapes is the path into the CU, not the matrix cores: every workgroup reads its strip of B once
// from HBM and all of A from L2 (at 128 rows twice the bytes of its strip), and at 256 strips the L2s hand out A 256
// times.  Requesting nothing but that, with no arithmetic at all, takes about 31 us at 128 x 14336 x 4096 with B [N,K]
// (B alone: 22), however many requests are in flight; hipBLASLt runs the shape in 30.5.  gemm_skinny_kernel loses
// another 3 us there for two reasons that this kernel removes: a wave gets one 1 KiB request accepted every ~56 cycles
// while the CU's vector memory path takes one every ~20, so four waves that each request 24 KiB per step of 64 are
// held up at issue; and the four partial sums of its K split meet in LDS at the end (128 KiB written, read back and
// added while nothing else runs).
// Here K is consumed in stages of 128 and a workgroup has eight waves.  Waves 0..3 compute: wave w owns a quarter of
// the rows (whole 16-row fragments; TMF not a multiple of 4: the first TMF % 4 waves take one more, the others work on
// their last one twice and drop the copy, so that the loop has no branches), all columns of the strip and all of K,
// so there is nothing to add up at the end.  They also request B, a quarter of each stage per wave.  Waves 4..7
// request A, a quarter of each stage per wave, and do nothing else.
// One barrier per stage: behind it stage t has landed (each wave has waited for its own requests) and every wave is
// past its reads of stage t - 1, whose slots are requested anew, R - 1 stages ahead, between the MFMAs of stage t.
// LDS: [RA stages of A: two 64-deep K-major images of 16*TMF rows each][RB stages of B: two 64-deep images of 64 rows
// (B [N,K]) or 128 k-rows of 64 columns (B [K,N])], laid out and swizzled as gemm_skinny_kernel's steps.
// Stages past the end of K are requested as zero fills (resource size 0) so that the wait counts hold for every K.
// Strips are handed out so that an XCD (workgroup id mod 8) owns a contiguous run of them, and with a K-major B every
// strip starts at another stage of K and wraps around (see SkinnyArgs::rot).
// ---------------------------------------------------------------------------------------------
template <int N>
__device__ __forceinline__ void wait_vmcnt_upto(int stages) {
  // at most stages * N of this wave's loads may stay in flight (stages is wave-uniform; the count is an immediate)
  switch (stages) {
    case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    case 1: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N <= 63 ? N : 63) : "memory"); break;
    case 2: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * N <= 63 ? 2 * N : 63) : "memory"); break;
    case 3: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * N <= 63 ? 3 * N : 63) : "memory"); break;
    case 4: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(4 * N <= 63 ? 4 * N : 63) : "memory"); break;
    case 5: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(5 * N <= 63 ? 5 * N : 63) : "memory"); break;
    case 6: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(6 * N <= 63 ? 6 * N : 63) : "memory"); break;
    default: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(7 * N <= 63 ? 7 * N : 63) : "memory"); break;
  }
}
template <int TMF, bool BKM, bool CCOL>
__global__ __launch_bounds__(512) void gemm_strip_kernel(SkinnyArgs p) {
  static_assert(TMF >= 4 && TMF <= 8, "at least one row fragment per compute wave; 128 rows at most");
  constexpr int NF = 4, STAGE_K = 128, RWF = (TMF + 3) / 4, NM = 4 * NF * RWF;  // row fragments, MFMAs per wave and stage
  constexpr uint32_t A_SUB = TMF * 2048, A_STAGE = 2 * A_SUB, B_SUB = 8192, B_STAGE = 2 * B_SUB;
  constexpr int NLA = TMF, NLB = 4;  // 1 KiB loads per stage of a wave that loads A / B: a quarter of the stage
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(NEOGEMM_AS3 char*)smem;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int quarter = wave & 3;  // the quarter of a stage of its operand this wave loads
  // workgroup -> (split of K, strip): consecutive workgroup ids land on different XCDs; id % 8 selects a contiguous run
  // of the work order, which walks the strips split by split
  const int per = gridDim.x >> 3, rem = gridDim.x & 7, xcd = blockIdx.x & 7;
  const int work = xcd * per + (xcd < rem ? xcd : rem) + (blockIdx.x >> 3);
  const int ksplit = p.ksplit > 1 ? p.ksplit : 1, nstrips = (int)gridDim.x / ksplit;
  const int kz = work / nstrips, strip_id = work - kz * nstrips;
  const int n0 = strip_id * p.strip;
  // this workgroup's stages of K: [st0, st0 + nst) (the host leaves no split empty)
  const int nst_all = (p.K + STAGE_K - 1) / STAGE_K;
  const int st0 = ksplit > 1 ? kz * p.stages_per_split : 0;
  const int nst = ksplit > 1 ? (p.stages_per_split < nst_all - st0 ? p.stages_per_split : nst_all - st0) : nst_all;
  const int RA = p.ra, RB = p.rb;
  const uint32_t ring_a = lds0, ring_b = lds0 + (uint32_t)RA * A_STAGE;
  // the stage of its run this workgroup starts at: scattered over the strips (see launch_strip)
  const int rot0 = p.rot ? (int)((((unsigned)strip_id * 0x9E3779B1u) >> 12) % (unsigned)nst) : 0;

  f32x4 acc[RWF][NF];
#pragma unroll
  for (int t = 0; t < RWF; ++t)
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[t][f][v] = 0.f;
  // a compute wave's row fragments are rf0 .. rf0 + nrf - 1
  const int nrf = TMF / 4 + (quarter < TMF % 4 ? 1 : 0), rf0 = quarter * (TMF / 4) + (quarter < TMF % 4 ? quarter : TMF % 4);

  auto run = [&](auto role) {
    constexpr bool ROLE_A = decltype(role)::value;
    constexpr bool KMAJ = ROLE_A || BKM;  // this wave's operand has K-contiguous rows
    constexpr int NLOAD = ROLE_A ? NLA : NLB;
    constexpr uint32_t STAGE = ROLE_A ? A_STAGE : B_STAGE, SUB = ROLE_A ? A_SUB : B_SUB;
    const int R = ROLE_A ? RA : RB;
    // A quarter of a stage.  K-major operand: half the rows (NLOAD * 8) of one 64-deep image; B [K,N]: 32 k-rows.
    const int kq = KMAJ ? (quarter >> 1) * 64 : quarter * 32;  // depth of the quarter's first element within the stage
    const int row0 = KMAJ ? (quarter & 1) * NLOAD * 8 : 0;    // its first row of the operand
    const uint32_t ring = (ROLE_A ? ring_a : ring_b) + (KMAJ ? (uint32_t)(quarter >> 1) * SUB + (uint32_t)(quarter & 1) * NLOAD * 1024
                                                             : (uint32_t)quarter * 4096);
    // per-lane byte offsets of this wave's loads of a stage, relative to the first element of its quarter
    // (instruction offsets and OOB_OFFSET as in Operand::init)
    uint32_t vo[NLOAD];
    const uint32_t ld = (uint32_t)(ROLE_A ? p.lda : p.ldb);
#pragma unroll
    for (int j = 0; j < NLOAD; ++j) {
      const uint32_t r = 8 * j + (lane >> 3);  // row of the quarter (K-major) or its k-row (B [K,N])
      const uint32_t c = (lane & 7) ^ (KMAJ ? swz_k(row0 + r) : swz_mn64(r));
      vo[j] = r * ld * 2 + c * 16 + VOFF_BIAS - (j & 3) * 1024;
      if constexpr (ROLE_A) {
        if (row0 + (int)r >= p.M) vo[j] = OOB_OFFSET;
      } else if constexpr (BKM) {
        if (n0 + row0 + (int)r >= p.N || row0 + (int)r >= p.strip) vo[j] = OOB_OFFSET;  // rows past the strip: still issued, as zero fills
      } else {
        if (n0 + (int)c * 8 >= p.N || (int)c * 8 >= p.strip) vo[j] = OOB_OFFSET;
      }
    }
    const uint64_t base0 = ROLE_A ? (uint64_t)p.A + ((uint64_t)row0 * p.lda + kq) * 2
                           : BKM  ? (uint64_t)p.B + ((uint64_t)(n0 + row0) * p.ldb + kq) * 2
                                  : (uint64_t)p.B + ((uint64_t)kq * p.ldb + n0) * 2;
    const uint64_t kadv = KMAJ ? (uint64_t)STAGE_K * 2 : (uint64_t)STAGE_K * p.ldb * 2;
    // all loads of this wave for stage s into the ring slot at `dst`: the first quarter of them at once, the others
    // between the MFMAs of `mfmas` (none for a wave that only loads)
    auto stage_loads = [&](int s, uint32_t dst, auto&& mfmas) {
      const bool live = s < nst;
      int ps = live ? s + rot0 : 0;
      if (ps >= nst) ps -= nst;
      ps += st0;
      // depth left from the quarter's first element on (K-major: < 64 is the K tail of its image; B [K,N]: < 32)
      const int krem = live ? p.K - (ps * STAGE_K + kq) : 64;
      const uint64_t b = base0 + (uint64_t)ps * kadv - VOFF_BIAS;
      const i32x4 rs = {(int)(uint32_t)b, (int)(uint32_t)(b >> 32), live ? (int)0x80000000u : 0, 0x00020000};
      constexpr int EARLY = (NLOAD + 3) / 4;
      constexpr int NMF = ROLE_A ? 0 : NM;  // MFMAs of this wave per stage
      static_for<NMF + 1>([&](auto mc) {
        constexpr int m = decltype(mc)::value - 1;  // -1: ahead of the MFMAs
        if constexpr (m >= 0) mfmas(std::integral_constant<int, (m >= 0 ? m : 0)>{});
        static_for<NLOAD>([&](auto jc) {
          constexpr int j = decltype(jc)::value;
          if constexpr ((j < EARLY || NMF == 0 ? -1 : (j - EARLY) * NMF / (NLOAD - EARLY)) == m) {
            uint32_t v = vo[j];
            if (krem < 64) {
              const uint32_t r = 8 * j + (lane >> 3);
              if constexpr (KMAJ) {
                const uint32_t c = (lane & 7) ^ swz_k(row0 + r);
                if ((int)c * 8 >= krem) v = OOB_OFFSET;
              } else {
                if ((int)r >= krem) v = OOB_OFFSET;
              }
            }
            if constexpr (j % 4 == 0) dma_set_m0(dst + (j / 4) * 4096);
            dma16<(j & 3) * 1024>(rs, v);
          }
        });
      });
    };
    // prologue: all but one stage of the ring
    for (int s = 0; s < R - 1; ++s) stage_loads(s, ring + (uint32_t)s * STAGE, [](auto) {});
    int slot_a = 0, slot_b = 0;  // slots of stage t in the two rings
    int slot_ld = R - 1;         // slot of this wave's ring that takes the stage requested next
    if constexpr (ROLE_A) {
      for (int t = 0; t < nst; ++t) {
        wait_vmcnt_upto<NLOAD>(R - 2);
        __builtin_amdgcn_s_barrier();
        stage_loads(t + R - 1, ring + (uint32_t)slot_ld * STAGE, [](auto) {});
        slot_ld = slot_ld + 1 == R ? 0 : slot_ld + 1;
      }
    } else {
      // fragment addresses within a stage (see FragReader and gemm_skinny_kernel): slab sl is the (sl & 1)-th half of the
      // (sl >> 1)-th 64-deep image
      const uint32_t frow = lane & 15, fq = (uint32_t)lane >> 4;
      const uint32_t tr_r = frow >> 2, tr_c = frow & 3, kk = 8 * fq + tr_r;  // B [K,N]: k-row within the slab, the second read adds 4
      auto k_off = [&](int sl) { return frow * 128 + (((4 * (uint32_t)(sl & 1) + fq) ^ swz_k(frow)) << 4); };
      auto fa_off = [&](int sl) { return (uint32_t)(sl >> 1) * A_SUB + k_off(sl); };
      auto fb_off = [&](int sl) { return BKM ? (uint32_t)(sl >> 1) * B_SUB + k_off(sl) : (32 * (uint32_t)sl + kk) * 128 + ((tr_c & 1) << 3); };
      auto read_b = [&](uint32_t img_b, int f) -> bf16x8 {
        if constexpr (BKM) {
          return lds_read_b128(img_b + f * 2048);
        } else {
          const uint32_t ad = img_b + (((2 * f + (tr_c >> 1)) ^ swz_mn64(kk)) << 4);
          const i16x4 lo = lds_read_tr16(ad), hi = lds_read_tr16(ad + 4 * 128);
          return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
      };
      for (int t = 0; t < nst; ++t) {
        // stage t has landed: this wave's requests for it (the R - 2 stages behind it may stay in flight), then everyone's;
        // every wave is past its reads of stage t - 1, whose slot takes stage t + R - 1
        wait_vmcnt_upto<NLOAD>(R - 2);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const uint32_t st_a = ring_a + (uint32_t)slot_a * A_STAGE, st_b = ring_b + (uint32_t)slot_b * B_STAGE;
        bf16x8 af[4][RWF], bf[4][NF];
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
#pragma unroll
          for (int f = 0; f < NF; ++f) bf[sl][f] = read_b(st_b + fb_off(sl), f);
#pragma unroll
          for (int i = 0; i < RWF; ++i) af[sl][i] = lds_read_b128(st_a + fa_off(sl) + (uint32_t)(rf0 + (i < nrf ? i : nrf - 1)) * 2048);
        }
        stage_loads(t + R - 1, ring + (uint32_t)slot_ld * STAGE, [&](auto mc) {
          constexpr int m = decltype(mc)::value, sl = m / (NF * RWF), f = (m / RWF) % NF, i = m % RWF;
          // B fragment first: a lane ends up with 4 consecutive n of one output row; for a column-major C the other way round
          if constexpr (CCOL) acc[i][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[sl][i], bf[sl][f], acc[i][f], 0, 0, 0);
          else acc[i][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bf[sl][f], af[sl][i], acc[i][f], 0, 0, 0);
        });
        // the fragments are in registers before this wave arrives at the next barrier, behind which their slots are rewritten
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        slot_a = slot_a + 1 == RA ? 0 : slot_a + 1;
        slot_b = slot_b + 1 == RB ? 0 : slot_b + 1;
        slot_ld = slot_ld + 1 == R ? 0 : slot_ld + 1;
      }
    }
  };
  if (wave >= 4) {
    run(std::true_type{});
    // the zero fills past the end of K have landed before the wave ends (nobody reads them)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    return;
  }
  run(std::false_type{});
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int i = 0; i < RWF; ++i)
#pragma unroll
    for (int f = 0; f < NF; ++f)
      if (i < nrf) {
        if (ksplit > 1) skinny_store_partial<CCOL>(acc[i][f], rf0 + i, f, p, n0, lane, p.ws + (size_t)kz * p.M * p.N);
        else skinny_store_frag<CCOL>(acc[i][f], rf0 + i, f, p, n0, lane);
      }
}

// Sum the split-K partials in split order (deterministic) and round once to bf16.
// Then C = alpha * sum + beta * C.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws, char* C, int M, int N,
                                                            long ldc, int ksplit, float alpha, float beta,
                                                            long bsc) {
  const size_t MN = (size_t)M * N;
  ws += (size_t)blockIdx.y * ksplit * MN;  // problem blockIdx.y of the batch
  C += (size_t)blockIdx.y * bsc * 2;
  const size_t idx = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (idx >= MN) return;
  if ((N & 3) == 0) {
    // up to four splits are fetched at a time (the loads of one trip are independent; one at a time the
    // kernel would spend a memory latency per split) and added in split order
    f32x4 s = *(const f32x4*)(ws + idx);
    for (int z = 1; z < ksplit; z += 4) {
      f32x4 t[4];
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (z + k < ksplit) t[k] = *(const f32x4*)(ws + (size_t)(z + k) * MN + idx);
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (z + k < ksplit) {
#pragma unroll
          for (int e = 0; e < 4; ++e) s[e] += t[k][e];
        }
    }
    const size_t row = idx / N, col = idx - row * N;
    bf16x4* dst = (bf16x4*)(C + (row * ldc + col) * 2);
#pragma unroll
    for (int e = 0; e < 4; ++e) s[e] *= alpha;
    if (beta != 0.f) {
      const bf16x4 c = *dst;
#pragma unroll
      for (int e = 0; e < 4; ++e) s[e] = __builtin_fmaf(beta, (float)c[e], s[e]);
    }
    bf16x4 o = {(__bf16)s[0], (__bf16)s[1], (__bf16)s[2], (__bf16)s[3]};
    *dst = o;
  } else {
    for (int e = 0; e < 4 && idx + e < MN; ++e) {
      float s = ws[idx + e];
      for (int z = 1; z < ksplit; ++z) s += ws[z * MN + idx + e];
      const size_t row = (idx + e) / N, col = (idx + e) - row * N;
      __bf16* dst = (__bf16*)(C + (row * ldc + col) * 2);
      s *= alpha;
      if (beta != 0.f) s = __builtin_fmaf(beta, (float)*dst, s);
      *dst = (__bf16)s;
    }
  }
}

// Fallback for anything the tile kernels do not take: arbitrary element strides, no alignment needs.
// One thread per output element, 16x16 outputs per workgroup, K walked 16 at a time through LDS.
__global__ __launch_bounds__(256) void gemm_generic_kernel(const __bf16* __restrict__ A, const __bf16* __restrict__ B,
                                                           __bf16* C, int M, int N, int K, long sam, long sak,
                                                           long sbk, long sbn, long scm, long scn, float alpha,
                                                           float beta, long bsa, long bsb, long bsc, unsigned nbx) {
  A += (size_t)blockIdx.z * bsa;  // problem blockIdx.z of the batch
  B += (size_t)blockIdx.z * bsb;
  C += (size_t)blockIdx.z * bsc;
  __shared__ float sa[16][17];
  __shared__ float sb[16][17];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  // blockIdx.x counts 16x16 output blocks row by row (nbx per block row): grid.y is limited to 65535
  const unsigned by = blockIdx.x / nbx, bx = blockIdx.x - by * nbx;
  const long row = (long)by * 16 + ty, col = (long)bx * 16 + tx;
  float acc = 0.f;
  for (int k0 = 0; k0 < K; k0 += 16) {
    // sa[ty][tx] = A(row, k0+tx); sb[ty][tx] = B(k0+ty, col)
    sa[ty][tx] = (row < M && k0 + tx < K) ? (float)A[row * sam + (long)(k0 + tx) * sak] : 0.f;
    sb[ty][tx] = (col < N && k0 + ty < K) ? (float)B[(long)(k0 + ty) * sbk + col * sbn] : 0.f;
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; ++k) acc = __builtin_fmaf(sa[ty][k], sb[k][tx], acc);
    __syncthreads();
  }
  if (row < M && col < N) {
    __bf16* dst = C + row * scm + col * scn;
    acc *= alpha;
    if (beta != 0.f) acc = __builtin_fmaf(beta, (float)*dst, acc);
    *dst = (__bf16)acc;
  }
}

// ---------------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------------
struct VariantInfo {
  int bm, bn, nwaves;
};
static const VariantInfo kVariants[NEOGEMM_VARIANT_COUNT] = {
    {0, 0, 0}, {16, 16, 4}, {0, 0, 0}, {256, 256, 4}, {128, 128, 4}, {256, 128, 4}, {128, 256, 4}, {64, 128, 4}, {0, 0, 0},
    {16, 64, 4}, {32, 64, 4}, {64, 64, 4}, {192, 256, 4}, {96, 128, 4}, {64, 64, 4}, {256, 256, 4}, {128, 64, 4},
    {128, 64, 4},
};
// Two identifiers of earlier builds (a 256x256 tile with eight waves, a 128x128 tile with a 1x4 wave grid) never won
// a shape against the kernels above in any sweep; their numbers stay reserved and a call that names one is refused.
static bool variant_retired(int v) { return v == NEOGEMM_VARIANT_RETIRED_2 || v == NEOGEMM_VARIANT_RETIRED_8; }

static bool is_aligned(const void* A, const void* B, const void* C, int64_t K, int64_t lda, int64_t ldb,
                       int64_t ldc) {
  return (((uintptr_t)A | (uintptr_t)B) & 15) == 0 && ((uintptr_t)C & 7) == 0 && (K & 7) == 0 && (lda & 7) == 0 &&
         (ldb & 7) == 0 && (ldc & 3) == 0;
}

static int ceil_div(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

// Shape -> (variant, split_k) by a small cost model, in microseconds, fitted to timings on one MI355X
// (256 CUs).  A workgroup of variant v spends `ktile_us` of its CU per 64-deep K tile and `fixed_us` on
// prologue + epilogue; the CUs work through ceil(workgroups / 256) of them one after the other (variants
// with small tiles put `per_cu` on a CU at once, which hides their fixed part).  Nothing runs faster than
// the operands stream from HBM (about 5 TB/s in practice).  Splitting K costs a second launch that reads
// the fp32 partials back (about 5 TB/s as well) plus a few microseconds, and a slower, fp32 epilogue.
// (M, N) as the caller states them; c_layout tells which of the two the kernel will see as its rows.
// A workgroup has about 2.5 K tiles of loads in flight, so it cannot finish a K tile faster than 1/2.5 of
// the round trip to where the operands come from: ~0.7 us per K tile when they stream from HBM, ~0.3 us
// when the whole problem stays in the L2s and the last-level cache.
struct PlanCand {
  int variant;
  double ktile_us, fixed_us, split_fixed_us;
  int per_cu;
};
static const PlanCand kPlanCands[] = {
    {NEOGEMM_VARIANT_T256x256_W4, 1.33, 9.0, 12.0, 1}, {NEOGEMM_VARIANT_T128x256_W4, 0.78, 6.0, 5.0, 1},
    {NEOGEMM_VARIANT_T256x128_W4, 0.78, 6.0, 5.0, 1},  {NEOGEMM_VARIANT_T128x128_W4, 0.50, 3.0, 2.0, 2},
    {NEOGEMM_VARIANT_T64x128_W4, 0.35, 2.5, 1.0, 2},    {NEOGEMM_VARIANT_T192x256_W4, 1.04, 7.0, 9.0, 1},
    {NEOGEMM_VARIANT_T96x128_W4, 0.42, 2.8, 1.8, 1},    {NEOGEMM_VARIANT_T64x64_W4, 0.20, 2.0, 1.0, 2},
};
// CUs the model plans for: those of the current device, or 256 (one MI355X) where no device can be asked, as in a
// host-only workspace query
static int planning_cus() {
  static std::atomic<bool> no_device{false};
  if (no_device.load(std::memory_order_relaxed)) return 256;
  int cus = 0;
  if (current_device_cus(&cus) != hipSuccess || cus <= 0) {
    (void)hipGetLastError();  // the failed query must not surface in a later call
    no_device.store(true, std::memory_order_relaxed);
    cus = 256;
  }
  return cus;
}
static void plan_model(int64_t M, int64_t N, int64_t K, bool aligned, int c_layout, int* variant, int* split_k,
                       int64_t batch = 1, int b_layout = NEOGEMM_B_KN, int ncus = 256) {
  if (!aligned || K == 0) {
    *variant = NEOGEMM_VARIANT_GENERIC;
    *split_k = 1;
    return;
  }
  const int64_t rows = c_layout == NEOGEMM_C_ROW ? M : N, cols = c_layout == NEOGEMM_C_ROW ? N : M;
  const int64_t ktiles = ceil_div(K, KTILE);
  const double cus = (double)ncus;
  const double bytes = 2.0 * ((double)rows * K + (double)K * cols + (double)rows * cols) * (double)batch;
  const double stream_us = bytes / 5.0e6, lat_us = bytes > 32e6 ? 0.7 : 0.3;
  static const int kSplits[] = {1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64};
  double best = 1e300;
  int bv = NEOGEMM_VARIANT_T128x128_W4, bs = 1;
  for (const PlanCand& c : kPlanCands) {
    // the 64x128 tile has too little in flight to stream from HBM: only for problems that stay in cache
    if (c.variant == NEOGEMM_VARIANT_T64x128_W4 && bytes > 32e6) continue;
    // 192 rows only of a K-major operand (an MN-major image needs a power of two)
    if ((c.variant == NEOGEMM_VARIANT_T192x256_W4 || c.variant == NEOGEMM_VARIANT_T96x128_W4) && c_layout == NEOGEMM_C_COL &&
        b_layout != NEOGEMM_B_NK)
      continue;
    // the small tiles have too little in flight to stream from HBM; 64x64 takes K-major operands only
    if ((c.variant == NEOGEMM_VARIANT_T96x128_W4 || c.variant == NEOGEMM_VARIANT_T64x64_W4) && bytes > 32e6) continue;
    if (c.variant == NEOGEMM_VARIANT_T64x64_W4 && b_layout != NEOGEMM_B_NK) continue;
    const double tiles = (double)ceil_div(rows, kVariants[c.variant].bm) * (double)ceil_div(cols, kVariants[c.variant].bn);
    for (int sp : kSplits) {
      if (sp > 1 && ktiles / sp < 2) break;  // at least 128 deep per split
      const double ktps = (double)ceil_div(ktiles, sp), wgs = tiles * sp * (double)batch;
      // a partial round runs on an emptier chip (more power and bandwidth per CU): measured at 0.7 of a round
      // when nearly empty, rising to 1 when full
      auto rounds_of = [](double x) {
        const double full = __builtin_floor(x), frac = x - full;
        return full + (frac > 0.0 ? 0.7 + 0.3 * frac : 0.0);
      };
      const double per_cu_wgs = rounds_of(wgs / cus);
      const double rounds = rounds_of(wgs / (cus * c.per_cu));
      double t = per_cu_wgs * ktps * c.ktile_us;
      // both operands K-major: the tall tile runs a little ahead of the wide one (2560^3: 33.8 against 35.0 us)
      if (c.variant == NEOGEMM_VARIANT_T128x256_W4 && b_layout == NEOGEMM_B_NK) t *= 1.02;
      // latency knows no discount, and two latency-bound workgroups on one CU were measured to take turns
      // (with both operands K-major the 128x128 tile has three tiles of each in flight when it streams: 256 x 14336 x 4096
      // unsplit, 224 workgroups, runs its 64 K tiles in 32.3 us; with far fewer workgroups than CUs a K tile takes longer,
      // and with more than CUs the second workgroup of a CU goes at the pace of the first: 128 x 5120 x 27648 with split 6,
      // 240 workgroups, 69 us; split 8, 320 of them, 98; split 12, 480, 76)
      const double lat_v =
          c.variant == NEOGEMM_VARIANT_T128x128_W4 && bytes > 32e6 && b_layout == NEOGEMM_B_NK && wgs >= 0.6 * cus && wgs <= cus ? 0.46 : lat_us;
      const double lat_floor = __builtin_ceil(wgs / cus) * ktps * lat_v;
      if (t < lat_floor) t = lat_floor;
      t += rounds * (c.fixed_us + (sp > 1 ? c.split_fixed_us : 0.0));
      // fewer workgroups than CUs pull less from HBM: 112 of them 4.0 TB/s, 224 and more 5 and above (64x11008x14336
      // with split 3, 129 workgroups: 87 us; split 4, 172: 73; 128x28672x14336 unsplit, 112: 230; split 2: 173)
      const double fill = wgs < cus ? wgs / cus : 1.0;
      const double floor_us = stream_us / (0.55 + 0.45 * fill);
      if (t < floor_us) t = floor_us;
      // Few rows against weights that stream from HBM: every further tile along the short side requests the weights again,
      // from the L2s, which is not free when the launch lives on its loads: 50 ns per MB (512 x 7168 x 7168 with B [N,K]:
      // four row tiles of 128, 72 us; two of 256, 62).  Fitted to the candidate timings of 16 to 512 rows with cold weights,
      // where it takes the plan's mean loss against the best candidate from 6.0 % to 3.6 %.
      if (bytes > 32e6 && (rows <= 512 || cols <= 512)) {
        const double again = cols >= rows ? (double)(ceil_div(rows, kVariants[c.variant].bm) - 1) * (double)cols
                                          : (double)(ceil_div(cols, kVariants[c.variant].bn) - 1) * (double)rows;
        t += again * (double)K * 2.0 * (double)batch * 5.0e-8;
      }
      if (sp > 1) t += 4.0 + (4.0 * sp + 2.0) * (double)rows * (double)cols * (double)batch / 5.0e6;
      if (t < best) {
        best = t;
        bv = c.variant;
        bs = sp;
      }
    }
  }
  // the skinny-M streaming kernel: one strip of up to 64 columns and all of K per workgroup, 128 KiB
  // (M <= 16), 96 KiB (M <= 32) or 64 KiB (M <= 64) of B in flight each at ~2.5 us per round trip; no split-K,
  // one launch
  // With B [N,K] and N <= 64 < M the same kernel runs the transposed problem (the wide operand is A then).
  // Both operands K-major with rows a multiple of 16 KiB apart: the tiles of all workgroups walk along K in step and crowd
  // onto a few memory channels (128 x 8192 x 8192 streams at 3.6 TB/s where 128 x 4096 x 14336 reaches 4.4), which the
  // estimates above do not know; the strip kernels start every strip at another depth for this reason.  So against them
  // the tiles' estimate counts for a fifth more there.
  const double best_tile = best * (b_layout == NEOGEMM_B_NK && K % 8192 == 0 && bytes > 32e6 ? 1.2 : 1.0);
  // The strip kernel with K split over s workgroups per strip, for few strips and deep K (128 x 8192 x 8192: 128 strips,
  // two splits, 38.0 us against 44.0 for split-K tiles; 112 x 4096 x 16384: four, 37 against 47): the unsplit kernel's
  // estimate with a workgroup's bytes divided by s, plus the reduction as for the tiles; 1024 to 8192 deep per split
  // (deeper, tiles with more splits win: 112 x 8192 x 28672 104 us against 111) and one round of workgroups (in two
  // rounds the measured times are up to half above this estimate).  Returns the best split and its estimate.
  auto strip_split = [&](int64_t srows, int64_t scols, int* split_at) {
    double split_best = 1e300;
    for (int sp : {2, 3, 4, 6, 8}) {
      if (K / sp < 1024 || (double)ceil_div(scols, 64) * sp > cus) break;
      if (K / sp > 8192) continue;
      const int rounds_i = ceil_div((int64_t)ceil_div(scols, 64) * sp, (int64_t)cus);
      int ws = 64;  // strip width: see launch_strip
      const int ww = 8 * ceil_div(scols * sp, 8 * (int64_t)rounds_i * (int64_t)cus);
      if (ww >= 40 && ww < 64) ws = ww;
      const double wgs_s = (double)ceil_div(scols, ws) * sp, full_s = __builtin_floor(wgs_s / cus), frac_s = wgs_s / cus - full_s;
      const double rounds_s = full_s + (frac_s > 0.0 ? 0.7 + 0.3 * frac_s : 0.0);
      const double bytes_s = ((double)K * 2.0 * ws + (double)ceil_div(srows, 16) * 16.0 * K * 2.0) / sp;
      double ts = 4.7 + rounds_s * bytes_s / 58.0e3;
      if (ts < stream_us) ts = stream_us;
      ts += 4.0 + (4.0 * sp + 2.0) * (double)srows * (double)scols / 5.0e6;
      if (ts < split_best) {
        split_best = ts;
        *split_at = sp;
      }
    }
    return split_best;
  };
  const bool skinny_m = M <= 64, skinny_n = !skinny_m && N <= 64 && b_layout == NEOGEMM_B_NK;
  if ((skinny_m || skinny_n) && batch == 1 && K >= 4 * KTILE) {
    const int64_t rows = skinny_m ? M : N, cols = skinny_m ? N : M;  // the kernel's own terms, whatever the layout of C
    double t;
    if (b_layout == NEOGEMM_B_NK) {
      // K-major wide operand: strips as wide as fills the CUs in whole rounds (see the launcher).  A workgroup pays
      // for the bytes of its strip (from HBM) and, less, for those of the small operand (from L2); fitted to timings
      // of 16 to 64 rows x 4096 .. 20480 columns x 4096 .. 14336 deep, all within 6 % but K = 8192 (-20 %).
      const int rounds = ceil_div(ceil_div(cols, 64), (int64_t)cus);
      int w = 8 * ceil_div(cols, 8 * (int64_t)rounds * (int64_t)cus);
      w = w < 16 ? 16 : w > 64 ? 64 : w;
      const double frags = (double)ceil_div(rows, 16) * 16.0;
      t = (double)ceil_div(ceil_div(cols, w), (int64_t)cus) * ((double)w * K * 2.0 / 26.9e3 + frags * K * 2.0 / 90.0e3);
      if (t < bytes / 5.9e6) t = bytes / 5.9e6;
    } else {
      // B [K,N]: strips of 64 columns.  A workgroup streams its strip at the rate its loads in flight allow, however few
      // workgroups there are (16 rows x 4096 .. 28672 columns x 3584 .. 28672 deep with weights from HBM: 27 to 35 GB/s per
      // workgroup from 32 strips to 224; 64 rows: 35 to 46), so a partial round takes as long as a full one, and all of
      // them together no less than the bytes take at 5 TB/s.
      // (A problem that stays in the caches streams faster and fills partial rounds better: the earlier fit.)
      if (bytes > 32e6) {
        const double wg_us =
            ((double)K * 128.0 + (double)ceil_div(rows, 16) * 16.0 * K * 2.0) / (rows <= 16 ? 33.0e3 : rows <= 32 ? 34.0e3 : 42.0e3);
        const int rounds_kn = ceil_div(ceil_div(cols, 64), (int64_t)cus);
        // (in a second round the strips stream a tenth slower: 24 x 27648 x 5120 in 432 strips 67.4 us, 40 x 28672 x 8192 109)
        t = (double)rounds_kn * wg_us * (rounds_kn > 1 ? 1.09 : 1.0);
      } else {
        const double wgs = (double)ceil_div(cols, 64), full = __builtin_floor(wgs / cus), frac = wgs / cus - full;
        const double rounds = full + (frac > 0.0 ? 0.7 + 0.3 * frac : 0.0);
        t = rounds * ((double)K * 128.0 + (double)rows * K * 2.0) / (rows <= 16 ? 51.0e3 : rows <= 32 ? 43.0e3 : 39.0e3);
      }
      if (t < stream_us) t = stream_us;
    }
    t += 3.0;
    // (the tile estimates come out a little low for shapes that stream from HBM with few rows, see below)
    bool took_skinny = false;
    if (t < best_tile * (b_layout == NEOGEMM_B_NK && bytes > 32e6 ? 1.04 : 1.0)) {
      best = t;
      bv = rows <= 16 ? NEOGEMM_VARIANT_SKINNY16 : rows <= 32 ? NEOGEMM_VARIANT_SKINNY32 : NEOGEMM_VARIANT_SKINNY64;
      bs = 1;
      took_skinny = true;
    }
    // 33 to 64 rows of a K-major wide operand, few strips, deep K: the strip kernel with K split (64 x 4096 x 16384: four
    // splits, 30.6 us against 38.1 for the tiles; 64 x 8192 x 8192: two, 31.7 against 33.7 for the skinny kernel); with
    // fewer rows it loses to the skinny kernel (16 x 8192 x 8192: 29.6 against 27.4) but not to the tiles where the
    // skinny kernel is out (24 x 4096 x 11008: 24.1 us against 28.5).  With B [K,N] from 33 rows on, against the tiles
    // (56 x 4096 x 11008: 26.1 us against 29.3, 64 x 4096 x 12288: 27.8 against 29.4; 16 x 4096 x 12288: 37 against 27).
    if ((b_layout == NEOGEMM_B_NK && (rows > 32 || !took_skinny)) || (b_layout == NEOGEMM_B_KN && skinny_m && rows > 32 && !took_skinny)) {
      int sp = 1;
      const double ts = strip_split(rows, cols, &sp) * (b_layout == NEOGEMM_B_KN ? 1.08 : 1.0);
      const double against_tiles = best_tile > best * 1.12 ? best_tile : best * 1.12;
      if (ts < (took_skinny ? best : against_tiles)) {
        best = ts;
        bv = NEOGEMM_VARIANT_STRIP;
        bs = sp;
      }
    }
  }
  // 65 to 128 rows (of M, or of N with B [N,K]): strips again, one launch, no workspace.  Up to 96 rows, and with
  // B [K,N], gemm_skinny_kernel with five to eight row fragments per wave; its rings hold two steps at most then, so it
  // is only the better choice where one round of strips about fills the CUs and K is a few thousand deep (with B [K,N]
  // 39.4 us against 36.9 for split-K tiles at 128 x 14336 x 4096, 37.5 against 41.2 at 112 rows).  From 97 rows on with a
  // K-major wide operand, gemm_strip_kernel (eight waves, shared rings, rows split between the waves): 4.7 us + the
  // bytes a workgroup requests at 58 GB/s per round of strips (within 4 % of 100 and 128 rows x 8192 .. 28672 columns x
  // 2048 .. 14336 deep; 128 x 14336 x 4096: 31.4 us against 34.0 for gemm_skinny_kernel, 18.2 against 20.8 at K = 2048).
  // Fitted to such timings; the tile estimates above come out about an eighth below what those shapes measure, hence
  // the factor.
  const bool wide_m = !skinny_m && !skinny_n && M <= 128;
  const bool wide_n = !skinny_m && !skinny_n && !wide_m && N <= 128 && b_layout == NEOGEMM_B_NK;
  if ((wide_m || wide_n) && batch == 1 && K >= 2048) {
    const int64_t rows = wide_m ? M : N, cols = wide_m ? N : M;
    const bool strip_kernel = b_layout == NEOGEMM_B_NK && rows > 96;
    int w = 64;  // strip width: see launch_strip
    if (strip_kernel) {
      const int rounds = ceil_div(ceil_div(cols, 64), (int64_t)cus), ww = 8 * ceil_div(cols, 8 * (int64_t)rounds * (int64_t)cus);
      if (ww >= 40 && ww < 64) w = ww;
    }
    const double wgs = (double)ceil_div(cols, w), full = __builtin_floor(wgs / cus), frac = wgs / cus - full;
    // (gemm_skinny_kernel with weights from HBM: a partial round of strips takes as long as a full one, 72 x 27648 x 5120
    // in 432 strips 69 us)
    const double rounds = !strip_kernel && bytes > 32e6 ? __builtin_ceil(wgs / cus) : full + (frac > 0.0 ? 0.7 + 0.3 * frac : 0.0);
    const double wg_bytes = (double)K * 2.0 * w + (double)ceil_div(rows, 16) * 16.0 * K * 2.0;
    double t = strip_kernel ? 4.7 + rounds * wg_bytes / 58.0e3
                            : 7.0 + rounds * wg_bytes / (b_layout == NEOGEMM_B_NK ? 52.0e3 : 46.0e3);
    if (t < stream_us) t = stream_us;
    // (with more than one round of strips the tile estimates are about right: 128 x 28672 x 4096 55 us for the tiles,
    // 59.5 for the strips; 72 x 27648 x 5120 58 us for the tiles, 69 for gemm_skinny_kernel)
    // (in more than one round of strips the tiles keep their plain estimate: 128 x 28672 x 8192 105 us against 114)
    if (t < (wgs > cus ? best : best_tile) * (wgs > cus ? 1.0 : 1.12)) {
      best = t;
      bv = strip_kernel ? NEOGEMM_VARIANT_STRIP : NEOGEMM_VARIANT_SKINNY128;
      bs = 1;
    }
    // K split over the workgroups of a strip (see strip_split above).  Against the tiles' estimate it gets the same
    // eighth as the unsplit strips (112 x 4096 x 11008: 27.9 us against 33.5 for the tiles, 5120 x 5120: 21.6 against
    // 25.9).  With 65 to 96 rows the time falls less with the rows than the estimate does (72 x 8192 x 8192: 36.6 us,
    // 128 rows 37.5), so it counts for an eighth more there; it still beats the tiles (72 x 4096 x 16384: 35.8 us
    // against 44.9).
    if (b_layout == NEOGEMM_B_NK) {
      // (problems under 80 MB, from 97 rows on: the tiles' estimates with split K come out lower still, 120 x 5120 x 5120 26.5 us
      // measured for 128x128 with split 6 against 22.0 for the strips with split 3, 104 x 6144 x 4096 23.6 against 20.8; with
      // 96 rows the two are level, 6144 x 4096 22.8 against 23.7)
      const double low = bytes < 80e6 && rows > 96 ? 1.3 : 1.12;
      const double against_tiles = best_tile > best * low ? best_tile : best * low;
      // the unsplit strips' estimate if they were taken
      const double limit = bv == NEOGEMM_VARIANT_STRIP || bv == NEOGEMM_VARIANT_SKINNY128 ? best : against_tiles;
      int sp = 1;
      const double ts = strip_split(rows, cols, &sp) * (rows > 96 ? 1.0 : 1.12);
      if (ts < limit) {
        best = ts;
        bv = NEOGEMM_VARIANT_STRIP;
        bs = sp;
      }
    }
  }
  // the 256x256 tile unsplit, K in whole periods of 128, rows from a K-major operand: the kernel that accumulates twice
  // in a row into each tile does the same work on less power (8192^3 +1.3 %, 4096^3 +1.2 %, bit-identical results)
  if (bv == NEOGEMM_VARIANT_T256x256_W4 && bs == 1 && K % (2 * KTILE) == 0 &&
      (c_layout == NEOGEMM_C_ROW || b_layout == NEOGEMM_B_NK))
    bv = NEOGEMM_VARIANT_C256x256_W4;
  *variant = bv;
  *split_k = bs;
}

// Tuned choices override the model: the file named by the environment variable NEOGEMM_PLAN_TABLE, read
// once, holds a JSON array of objects {"M":..,"N":..,"K":..,"b_layout":..,"c_layout":..,"variant":..,"split_k":..}
// (what gemm_amd/tune.py writes; b_layout and c_layout default to 0); an entry applies to calls with exactly
// its shape and layouts, since the kernels behind the layouts differ.  The reference fixes tile and stage counts at
// compile time (v01.cu:275-278); this is the run-time counterpart.  Entries with an unknown variant or a
// split below 1 are ignored, and so is an unreadable file.
struct PlanEntry {
  int64_t M, N, K;
  int b_layout, c_layout, variant, split_k;
};
static const std::vector<PlanEntry>& plan_table() {
  static const std::vector<PlanEntry> table = [] {
    std::vector<PlanEntry> t;
    const char* path = getenv("NEOGEMM_PLAN_TABLE");
    FILE* f = path && *path ? fopen(path, "rb") : nullptr;
    if (!f) return t;
    std::string text;
    char buf[4096];
    size_t n;
    while ((n = fread(buf, 1, sizeof buf, f)) > 0) text.append(buf, n);
    fclose(f);
    // one object at a time: the text between '{' and the next '}' (the objects are flat)
    size_t pos = 0;
    while ((pos = text.find('{', pos)) != std::string::npos) {
      const size_t end = text.find('}', pos);
      if (end == std::string::npos) break;
      const std::string obj = text.substr(pos, end - pos);
      auto field = [&](const char* key, long long dflt) -> long long {
        const std::string k = std::string("\"") + key + "\"";
        size_t at = obj.find(k);
        if (at == std::string::npos) return dflt;
        at = obj.find(':', at + k.size());
        if (at == std::string::npos) return dflt;
        return strtoll(obj.c_str() + at + 1, nullptr, 10);
      };
      PlanEntry e{field("M", -1), field("N", -1), field("K", -1), (int)field("b_layout", 0), (int)field("c_layout", 0),
                  (int)field("variant", -1), (int)field("split_k", 0)};
      if (e.M > 0 && e.N > 0 && e.K > 0 && e.variant > NEOGEMM_VARIANT_AUTO && e.variant < NEOGEMM_VARIANT_COUNT &&
          !variant_retired(e.variant) && e.split_k >= 1 && e.split_k <= 64 && (e.c_layout == NEOGEMM_C_ROW || e.c_layout == NEOGEMM_C_COL) &&
          (e.b_layout == NEOGEMM_B_KN || e.b_layout == NEOGEMM_B_NK))
        t.push_back(e);
      pos = end + 1;
    }
    return t;
  }();
  return table;
}
static void plan_uncached(int64_t M, int64_t N, int64_t K, bool aligned, int c_layout, int* variant, int* split_k,
                          int64_t batch, int b_layout, int ncus);
// The cost model walks every (tile, split) candidate: a few microseconds on the host, as long as a small GEMM takes
// on the GPU.  A caller in a loop repeats a handful of shapes, so each thread remembers its last few answers.
static void plan(int64_t M, int64_t N, int64_t K, bool aligned, int c_layout, int* variant, int* split_k,
                 int64_t batch = 1, int b_layout = NEOGEMM_B_KN) {
  struct Memo {
    int64_t M = -1, N = -1, K = -1, batch = -1;
    int b_layout = -1, c_layout = -1, aligned = -1, ncus = -1, variant = 0, split_k = 0;
  };
  static thread_local Memo memo[32];  // the workspace query alone asks for four layouts of a shape
  static thread_local unsigned next = 0;
  const int ncus = planning_cus();
  for (const Memo& m : memo)
    if (m.M == M && m.N == N && m.K == K && m.batch == batch && m.b_layout == b_layout && m.c_layout == c_layout &&
        m.aligned == (int)aligned && m.ncus == ncus) {
      *variant = m.variant;
      *split_k = m.split_k;
      return;
    }
  plan_uncached(M, N, K, aligned, c_layout, variant, split_k, batch, b_layout, ncus);
  Memo& m = memo[next++ & 31];
  m.M = M, m.N = N, m.K = K, m.batch = batch, m.b_layout = b_layout, m.c_layout = c_layout, m.aligned = (int)aligned;
  m.ncus = ncus;
  m.variant = *variant, m.split_k = *split_k;
}
// Tuned choices that ship with the library: shapes of a sweep (gemm_amd/tune.py over M in 256 .. 8192 x the (N, K) pairs of
// common transformer layers, three layout pairs, one MI355X) where the best measured (variant, split) beat the model's
// choice by more than 3 %.  A table named by NEOGEMM_PLAN_TABLE is looked up first; these apply on a device with the
// CU count they were measured on.
static const int kDefaultPlanCus = 256;
static const PlanEntry kDefaultPlan[] = {
#include "neogemm_default_plan.inc"
};
static void plan_uncached(int64_t M, int64_t N, int64_t K, bool aligned, int c_layout, int* variant, int* split_k,
                          int64_t batch, int b_layout, int ncus) {
  if (aligned && K > 0 && batch == 1) {
    auto match = [&](const PlanEntry& e) {
      return e.M == M && e.N == N && e.K == K && e.c_layout == c_layout && e.b_layout == b_layout;
    };
    for (const PlanEntry& e : plan_table())
      if (match(e)) {
        *variant = e.variant;
        *split_k = e.variant == NEOGEMM_VARIANT_GENERIC ? 1 : e.split_k;
        return;
      }
    if (ncus == kDefaultPlanCus)
      for (const PlanEntry& e : kDefaultPlan)
        if (match(e)) {
          *variant = e.variant;
          *split_k = e.split_k;
          return;
        }
  }
  plan_model(M, N, K, aligned, c_layout, variant, split_k, batch, b_layout, ncus);
}

// The largest split-K factor plan() returns for this shape over the four (b_layout, c_layout) combinations a call can
// name (the kernels, and so the plans, differ between them): the workspace queries bound every call for the shape,
// the reference's own (B [N,K], column-major C: nemgemmV03.cu:346, v01.cu:246,252) included.
static int max_planned_split(int64_t M, int64_t N, int64_t K, int64_t batch) {
  int best = 1;
  for (int bl : {NEOGEMM_B_KN, NEOGEMM_B_NK})
    for (int cl : {NEOGEMM_C_ROW, NEOGEMM_C_COL}) {
      int v, s;
      plan(M, N, K, true, cl, &v, &s, batch, bl);
      if (s > best) best = s;
    }
  return best;
}

// Launch of gemm_strip_kernel (65 to 128 rows).  `rings` = 16 * RA + RB forces the ring depths (0: the defaults below).
// split_k > 1: that many workgroups per strip, each with a run of 128-deep stages; `ws` takes the partial sums and the
// reduction kernel follows.
static int launch_strip(SkinnyArgs sa, bool bkm, bool ccol, int rings, hipStream_t st, int split_k = 1, void* ws = nullptr,
                        size_t ws_bytes = 0) {
  int cus = 0;
  if (hipError_t e = current_device_cus(&cus); e != hipSuccess) {
    fprintf(stderr, "neogemm: device query failed: %s\n", hipGetErrorString(e));
    return NEOGEMM_ERR_LAUNCH;
  }
  // Strips of 64 columns; of a K-major B (a strip is a set of whole rows then) the multiple of 8 from 40 up that fills
  // the CUs in whole rounds (N = 14336: 256 strips of 56).  Strips of B [K,N] that are not 64 wide would share the cache
  // lines at their edges with their neighbours: 128 x 14336 x 4096 takes 47 us with strips of 56 against 38 with 64.
  // split K: no empty split, and a workspace of one fp32 matrix per split
  const int stages = ceil_div(sa.K, 128);
  if (split_k > stages) split_k = stages;
  sa.ksplit = 1;
  if (split_k > 1) {
    sa.stages_per_split = ceil_div(stages, split_k);
    sa.ksplit = ceil_div(stages, sa.stages_per_split);
  }
  if (sa.ksplit > 1) {
    if (!ws || ws_bytes < (size_t)sa.ksplit * (size_t)sa.M * (size_t)sa.N * sizeof(float)) return NEOGEMM_ERR_WORKSPACE;
    if (((uintptr_t)ws & 15) != 0) return NEOGEMM_ERR_BAD_ARG;
    sa.ws = (float*)ws;
  }
  sa.strip = 64;
  if (bkm) {
    // (with K split, the strips of all splits together make the rounds)
    const int rounds = ceil_div((int64_t)ceil_div(sa.N, 64) * sa.ksplit, cus);
    const int w = 8 * ceil_div((int64_t)sa.N * sa.ksplit, 8 * (int64_t)rounds * cus);
    if (w >= 40 && w < 64) sa.strip = w;
    // Every strip starts at another stage of K (and wraps around): measured 3 to 5 % at K = 4096 against all strips at one
    // depth.  Which stage is a multiplicative hash of the strip's number, not a multiple of it: with one stage (256 bytes)
    // further per strip the requests of all strips meet on few memory channels where the strips lie 512 KiB apart
    // (128 x 16384 x 4096: 46.5 us against 34), with two stages at 1 MiB apart (128 x 8192 x 8192 in two splits: 50.5 against
    // 39), with seven at 448 KiB; the hash measured level with the best multiple at twelve shapes, strips 160 KiB to 2 MiB apart.
    sa.rot = 1;
  }
  // row fragments of 16: five to eight, or four for up to 64 rows when K is split (unsplit, gemm_skinny_kernel is the
  // kernel for those; rows past M are zero fills that touch no memory)
  int tmf = ceil_div(sa.M, 16);
  if (tmf < 4 && sa.ksplit > 1) tmf = 4;
  if (tmf < (sa.ksplit > 1 ? 4 : 5) || tmf > 8) return NEOGEMM_ERR_UNSUPPORTED;
  // ring depths: three stages of A (4 KiB * tmf each: two in flight cover the way to L2 and back) and what the 160 KiB
  // leave for B (16 KiB a stage)
  static const int kRings[9][2] = {{0, 0}, {0, 0}, {0, 0}, {0, 0}, {3, 6}, {3, 6}, {3, 5}, {3, 4}, {3, 4}};
  sa.ra = kRings[tmf][0];
  sa.rb = kRings[tmf][1];
  if (rings > 0) {
    sa.ra = rings / 16;
    sa.rb = rings % 16;
  }
  const size_t lds = (size_t)sa.ra * tmf * 4096 + (size_t)sa.rb * 16384;
  // what the kernel assumes: a stage being read besides those in flight, wait counts within the counter's 6 bits,
  // rings that fit the LDS
  if (sa.ra < 2 || sa.rb < 2 || sa.ra > 9 || sa.rb > 9 || (sa.ra - 2) * tmf > 63 || (sa.rb - 2) * 4 > 63 || lds > 160 * 1024)
    return NEOGEMM_ERR_UNSUPPORTED;
  auto go = [&](auto kern) -> hipError_t {
    if (hipError_t e = allow_lds(kern, lds); e != hipSuccess) return e;
    kern<<<dim3(ceil_div(sa.N, sa.strip) * sa.ksplit), 512, lds, st>>>(sa);
    return hipGetLastError();
  };
  auto pick = [&](auto tc) -> hipError_t {
    constexpr int TMF = decltype(tc)::value;
    if (bkm) return ccol ? go(gemm_strip_kernel<TMF, true, true>) : go(gemm_strip_kernel<TMF, true, false>);
    return ccol ? go(gemm_strip_kernel<TMF, false, true>) : go(gemm_strip_kernel<TMF, false, false>);
  };
  hipError_t e = hipErrorInvalidValue;
  switch (tmf) {
    case 4: e = pick(std::integral_constant<int, 4>{}); break;
    case 5: e = pick(std::integral_constant<int, 5>{}); break;
    case 6: e = pick(std::integral_constant<int, 6>{}); break;
    case 7: e = pick(std::integral_constant<int, 7>{}); break;
    default: e = pick(std::integral_constant<int, 8>{}); break;
  }
  if (e != hipSuccess) {
    fprintf(stderr, "neogemm: strip kernel launch failed: %s\n", hipGetErrorString(e));
    return NEOGEMM_ERR_LAUNCH;
  }
  if (sa.ksplit > 1) {
    // C as it lies in memory: M x N row-major, or N x M for a column-major C
    const int rows_mem = ccol ? sa.N : sa.M, cols_mem = ccol ? sa.M : sa.N;
    const size_t MN = (size_t)sa.M * sa.N;
    splitk_reduce_kernel<<<dim3((unsigned)((MN + 1023) / 1024), 1), 256, 0, st>>>(sa.ws, sa.C, rows_mem, cols_mem, sa.ldc, sa.ksplit,
                                                                                sa.alpha, sa.beta, 0);
    if (hipError_t e2 = hipGetLastError(); e2 != hipSuccess) {
      fprintf(stderr, "neogemm: split-K reduction launch failed: %s\n", hipGetErrorString(e2));
      return NEOGEMM_ERR_LAUNCH;
    }
  }
  return NEOGEMM_OK;
}

// A batch of `count` problems of one shape; strides in elements between consecutive problems (0: shared operand).
struct BatchArgs {
  int64_t count = 1, sa = 0, sb = 0, sc = 0;
};

static int run(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
               int64_t ldc, int b_layout, int c_layout, void* workspace, size_t workspace_bytes, void* hip_stream,
               int variant, int split_k, int group_m, unsigned long long* prof = nullptr, float alpha = 1.f,
               float beta = 0.f, const BatchArgs& bt = BatchArgs()) {
  if (M < 0 || N < 0 || K < 0) return NEOGEMM_ERR_BAD_ARG;
  if (bt.count < 1 || bt.count > 65535 || bt.sa < 0 || bt.sb < 0 || bt.sc < 0) return NEOGEMM_ERR_BAD_ARG;
  if (bt.count > 1 && M > 0 && N > 0) {
    // the outputs of the batch must not overlap
    const int64_t c_extent = c_layout == NEOGEMM_C_ROW ? (M - 1) * ldc + N : (N - 1) * ldc + M;
    if (bt.sc < c_extent) return NEOGEMM_ERR_BAD_ARG;
  }
  if ((b_layout != NEOGEMM_B_KN && b_layout != NEOGEMM_B_NK) || (c_layout != NEOGEMM_C_ROW && c_layout != NEOGEMM_C_COL))
    return NEOGEMM_ERR_BAD_ARG;
  if (variant < 0 || variant >= NEOGEMM_VARIANT_COUNT || split_k < 0 || group_m < 0) return NEOGEMM_ERR_BAD_ARG;
  if (variant_retired(variant)) return NEOGEMM_ERR_UNSUPPORTED;
  if (M == 0 || N == 0) return NEOGEMM_OK;
  if (!C || (K > 0 && (!A || !B))) return NEOGEMM_ERR_BAD_ARG;
  if (lda < K || ldb < (b_layout == NEOGEMM_B_KN ? N : K) || ldc < (c_layout == NEOGEMM_C_ROW ? N : M))
    return NEOGEMM_ERR_BAD_ARG;
  if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return NEOGEMM_ERR_BAD_ARG;
  hipStream_t st = (hipStream_t)hip_stream;

  // ld limits keep every in-tile byte offset below 2^31 (the buffer range check uses 32-bit offsets)
  const bool aligned = is_aligned(A, B, C, K, lda, ldb, ldc) && lda < (1 << 21) && ldb < (1 << 21) && K > 0 &&
                       (bt.sa & 7) == 0 && (bt.sb & 7) == 0 && (bt.sc & 3) == 0;
  int v = variant, s = split_k;
  if (v == NEOGEMM_VARIANT_AUTO) {
    int pv, ps;
    plan(M, N, K, aligned, c_layout, &pv, &ps, bt.count, b_layout);
    v = pv;
    if (s == 0) s = ps;
  }
  if (s == 0) s = 1;

  if (v == NEOGEMM_VARIANT_GENERIC) {
    const long sbk = b_layout == NEOGEMM_B_KN ? ldb : 1, sbn = b_layout == NEOGEMM_B_KN ? 1 : ldb;
    const long scm = c_layout == NEOGEMM_C_ROW ? ldc : 1, scn = c_layout == NEOGEMM_C_ROW ? 1 : ldc;
    const int64_t nbx = ceil_div(N, 16), nblocks = nbx * ceil_div(M, 16);
    if (nblocks > 0x7fffffff) return NEOGEMM_ERR_UNSUPPORTED;
    dim3 grid((unsigned)nblocks, 1, (unsigned)bt.count);
    gemm_generic_kernel<<<grid, 256, 0, st>>>((const __bf16*)A, (const __bf16*)B, (__bf16*)C, (int)M, (int)N, (int)K,
                                              lda, 1, sbk, sbn, scm, scn, alpha, beta, bt.sa, bt.sb, bt.sc,
                                              (unsigned)nbx);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
      fprintf(stderr, "neogemm: generic kernel launch failed: %s\n", hipGetErrorString(e));
      return NEOGEMM_ERR_LAUNCH;
    }
    return NEOGEMM_OK;
  }

  if (!aligned) return NEOGEMM_ERR_UNSUPPORTED;

  if (v == NEOGEMM_VARIANT_SKINNY16 || v == NEOGEMM_VARIANT_SKINNY32 || v == NEOGEMM_VARIANT_SKINNY64 ||
      v == NEOGEMM_VARIANT_SKINNY128 || v == NEOGEMM_VARIANT_STRIP) {
    // what the skinny kernel assumes: M within its rows, whole 16-byte chunks of B [K,N] inside the matrix,
    // one problem.  If M is too large but N fits and B is [N,K], it runs the transposed problem
    // C^T = B * A^T: its small operand is B then, its wide one A, and the layout of C flips.
    const bool swap = M > kVariants[v].bm && N <= kVariants[v].bm && b_layout == NEOGEMM_B_NK;
    const bool ok = bt.count == 1 && (M <= kVariants[v].bm || swap) &&
                    (b_layout == NEOGEMM_B_NK || (N & 7) == 0) &&
                    (split_k <= 1 || variant == NEOGEMM_VARIANT_AUTO || v == NEOGEMM_VARIANT_STRIP) && !prof;
    if (!ok) {
      if (variant != NEOGEMM_VARIANT_AUTO) return NEOGEMM_ERR_UNSUPPORTED;
      // the 128x128 tile needs the least of the tile kernels, then the generic kernel
      int st2 = run(A, B, C, M, N, K, lda, ldb, ldc, b_layout, c_layout, workspace, workspace_bytes, hip_stream,
                    NEOGEMM_VARIANT_T128x128_W4, 1, 0, nullptr, alpha, beta, bt);
      if (st2 == NEOGEMM_ERR_UNSUPPORTED)
        st2 = run(A, B, C, M, N, K, lda, ldb, ldc, b_layout, c_layout, workspace, workspace_bytes, hip_stream,
                  NEOGEMM_VARIANT_GENERIC, 1, 0, nullptr, alpha, beta, bt);
      return st2;
    }
    SkinnyArgs sa{(const char*)A, (const char*)B, (char*)C, (int)M, (int)N, (int)K, (long)lda, (long)ldb, (long)ldc, alpha, beta, 0, 64};
    bool bkm = b_layout == NEOGEMM_B_NK, ccol = c_layout == NEOGEMM_C_COL;
    if (swap) {
      sa = SkinnyArgs{(const char*)B, (const char*)A, (char*)C, (int)N, (int)M, (int)K, (long)ldb, (long)lda, (long)ldc, alpha, beta, 0, 64};
      bkm = true;    // A [M,K] takes the place of a B [N,K]
      ccol = !ccol;  // a row-major C[m][n] is the column-major C^T
    }
    const bool wide = v == NEOGEMM_VARIANT_SKINNY128;
    sa.rot = bkm && sa.ldb % 8192 == 0;  // rows of the wide operand a multiple of 16 KiB apart
    if (v == NEOGEMM_VARIANT_STRIP) return launch_strip(sa, bkm, ccol, group_m, st, s, workspace, workspace_bytes);
    if (bkm) {
      // A strip of a K-major B may start at any row of it and be of any width that is a multiple of 8: the width is
      // chosen so that whole rounds of strips fill the CUs (N = 14336: 256 strips of 56 columns instead of 224 of 64,
      // +1 to 3 %; N = 4096: 256 of 16 instead of 64 of 64, 50 -> 32 us at K = 14336 before the rings were deepened).
      int cus = 0;
      if (hipError_t e = current_device_cus(&cus); e != hipSuccess) {
        fprintf(stderr, "neogemm: device query failed: %s\n", hipGetErrorString(e));
        return NEOGEMM_ERR_LAUNCH;
      }
      const int rounds = ceil_div(ceil_div(sa.N, 64), cus), w = 8 * ceil_div(sa.N, 8 * (int64_t)rounds * cus);
      if (w < 64 && w >= (wide ? 48 : 16)) sa.strip = w;
      else if (w < 16 && !wide) sa.strip = 16;
    }
    auto go = [&](auto kern, size_t lds) -> hipError_t {
      if (hipError_t e = allow_lds(kern, lds); e != hipSuccess) return e;
      kern<<<dim3(ceil_div(sa.N, sa.strip)), 256, lds, st>>>(sa);
      return hipGetLastError();
    };
    auto pick = [&](auto tmf, auto rs, auto ra) -> hipError_t {
      constexpr int TMF = decltype(tmf)::value, RS = decltype(rs)::value, RA = decltype(ra)::value;
      constexpr size_t lds = (size_t)4 * (RA * TMF * 2048 + RS * 8192);
      if (bkm) return ccol ? go(gemm_skinny_kernel<TMF, RS, true, true, RA>, lds) : go(gemm_skinny_kernel<TMF, RS, true, false, RA>, lds);
      return ccol ? go(gemm_skinny_kernel<TMF, RS, false, true, RA>, lds) : go(gemm_skinny_kernel<TMF, RS, false, false, RA>, lds);
    };
    // strips of at most 32 / 16 columns of a K-major B: smaller steps of B, deeper rings
    auto pick_narrow = [&](auto tmf, auto rs, auto sw) -> hipError_t {
      constexpr int TMF = decltype(tmf)::value, RS = decltype(rs)::value, SW = decltype(sw)::value;
      constexpr size_t lds = (size_t)4 * RS * (TMF * 2048 + SW * 128);
      return ccol ? go(gemm_skinny_kernel<TMF, RS, true, true, RS, SW>, lds) : go(gemm_skinny_kernel<TMF, RS, true, false, RS, SW>, lds);
    };
    using std::integral_constant;
    hipError_t e;
    using I1 = integral_constant<int, 1>;
    using I2 = integral_constant<int, 2>;
    using I3 = integral_constant<int, 3>;
    using I4 = integral_constant<int, 4>;
    using I5 = integral_constant<int, 5>;
    using I6 = integral_constant<int, 6>;
    using I10 = integral_constant<int, 10>;
    using W16 = integral_constant<int, 16>;
    using W32 = integral_constant<int, 32>;
    const int sw = sa.strip <= 16 ? 16 : sa.strip <= 32 ? 32 : 64;
    if (v == NEOGEMM_VARIANT_SKINNY16) e = sw == 16 ? pick_narrow(I1{}, I10{}, W16{}) : sw == 32 ? pick_narrow(I1{}, I6{}, W32{}) : pick(I1{}, I4{}, I4{});
    else if (v == NEOGEMM_VARIANT_SKINNY32) e = sw == 16 ? pick_narrow(I2{}, I6{}, W16{}) : sw == 32 ? pick_narrow(I2{}, I5{}, W32{}) : pick(I2{}, I3{}, I3{});
    else if (v == NEOGEMM_VARIANT_SKINNY64) e = sw == 16 ? pick_narrow(I4{}, I4{}, W16{}) : sw == 32 ? pick_narrow(I4{}, I3{}, W32{}) : pick(I4{}, I2{}, I2{});
    // 65 to 128 rows, in sixteens: two steps of A and of B in the rings while they fit, else one of A and three of B
    else if (sa.M <= 80) e = pick(I5{}, I2{}, I2{});
    else if (sa.M <= 96) e = pick(I6{}, I2{}, I2{});
    else if (sa.M <= 112) e = pick(integral_constant<int, 7>{}, I3{}, I1{});
    else e = pick(integral_constant<int, 8>{}, I3{}, I1{});
    if (e != hipSuccess) {
      fprintf(stderr, "neogemm: skinny kernel launch failed (variant %d): %s\n", v, hipGetErrorString(e));
      return NEOGEMM_ERR_LAUNCH;
    }
    return NEOGEMM_OK;
  }

  // The tile kernels write row-major output.  Column-major C is the row-major transpose, i.e. the
  // product with the operands' roles exchanged.
  TileArgs a;
  bool ak, bk;
  if (c_layout == NEOGEMM_C_ROW) {
    a.A = (const char*)A; a.lda = lda; ak = true; a.M = (int)M; a.bsa = bt.sa;
    a.B = (const char*)B; a.ldb = ldb; bk = (b_layout == NEOGEMM_B_NK); a.N = (int)N; a.bsb = bt.sb;
  } else {
    a.A = (const char*)B; a.lda = ldb; ak = (b_layout == NEOGEMM_B_NK); a.M = (int)N; a.bsa = bt.sb;
    a.B = (const char*)A; a.ldb = lda; bk = true; a.N = (int)M; a.bsb = bt.sa;
  }
  a.C = (char*)C;
  a.ldc = ldc;
  a.bsc = bt.sc;
  a.batch = (int)bt.count;
  a.K = (int)K;
  const VariantInfo& vi = kVariants[v];
  // What the tile kernels assume about an MN-major operand (see Operand::init): a tile of >= 128 rows, a power
  // of two, for its swizzle and a row count that is a multiple of 8 (16-byte chunks must not straddle the
  // matrix edge).
  auto mn_ok = [](int tile, int rows) { return tile >= 128 && (tile & (tile - 1)) == 0 && (rows & 7) == 0; };
  // (the chained 256x256 kernel takes its rows from a K-major operand only, K in whole periods of 128 and no split)
  const bool fits = (ak || mn_ok(vi.bm, a.M)) && (bk || mn_ok(vi.bn, a.N)) &&
                    (v != NEOGEMM_VARIANT_C256x256_W4 || (ak && K % (2 * KTILE) == 0 && s <= 1));
  if (!fits) {
    if (variant != NEOGEMM_VARIANT_AUTO) return NEOGEMM_ERR_UNSUPPORTED;
    // the planned tile is too wide for an MN-major operand: the 128x128 tile needs the least, then generic
    const int next = v != NEOGEMM_VARIANT_T128x128_W4 ? NEOGEMM_VARIANT_T128x128_W4 : NEOGEMM_VARIANT_GENERIC;
    int st = run(A, B, C, M, N, K, lda, ldb, ldc, b_layout, c_layout, workspace, workspace_bytes, hip_stream, next,
                 next == NEOGEMM_VARIANT_GENERIC ? 1 : s, 0, nullptr, alpha, beta, bt);
    if (st == NEOGEMM_ERR_UNSUPPORTED && next != NEOGEMM_VARIANT_GENERIC)
      st = run(A, B, C, M, N, K, lda, ldb, ldc, b_layout, c_layout, workspace, workspace_bytes, hip_stream,
               NEOGEMM_VARIANT_GENERIC, 1, 0, nullptr, alpha, beta, bt);
    return st;
  }
  a.ntm = ceil_div(a.M, vi.bm);
  a.ntn = ceil_div(a.N, vi.bn);
  a.group_m = group_m > 0 ? group_m : 8;
  const int ktiles = ceil_div(K, KTILE);
  if (s > ktiles) s = ktiles;
  a.ktiles_per_split = ceil_div(ktiles, s);
  a.ksplit = ceil_div(ktiles, a.ktiles_per_split);  // no empty split
  if ((int64_t)a.ntm * a.ntn * a.ksplit > 0x7fffffff) return NEOGEMM_ERR_UNSUPPORTED;  // grid.x counts (split, tile) pairs
  a.ws = nullptr;
  a.prof = prof;
  a.alpha = alpha;
  a.early_stores = 0;
  a.beta = beta;
  if (prof && (bt.count > 1 || a.ksplit > 1 || vi.bm != 256 || vi.bn != 256 || !ak || v == NEOGEMM_VARIANT_C256x256_W4))
    return NEOGEMM_ERR_UNSUPPORTED;
  if (a.ksplit > 1) {
    const size_t need = (size_t)a.ksplit * (size_t)M * (size_t)N * sizeof(float) * (size_t)bt.count;
    if (!workspace || workspace_bytes < need) return NEOGEMM_ERR_WORKSPACE;
    if (((uintptr_t)workspace & 15) != 0) return NEOGEMM_ERR_BAD_ARG;
    a.ws = (float*)workspace;
  }

  hipError_t e;
  switch (v) {
    case NEOGEMM_VARIANT_T256x256_W4: e = launch_tile<256, 256, 2, 2>(a, ak, bk, st); break;
    case NEOGEMM_VARIANT_T128x128_W4: e = launch_tile<128, 128, 2, 2>(a, ak, bk, st); break;
    case NEOGEMM_VARIANT_T256x128_W4: e = launch_tile<256, 128, 2, 2>(a, ak, bk, st); break;
    case NEOGEMM_VARIANT_T128x256_W4: e = launch_tile<128, 256, 2, 2>(a, ak, bk, st); break;
    case NEOGEMM_VARIANT_T64x128_W4: e = launch_tile<64, 128, 1, 4>(a, ak, bk, st); break;
    case NEOGEMM_VARIANT_T192x256_W4: e = launch_tile<192, 256, 2, 2>(a, ak, bk, st); break;
    case NEOGEMM_VARIANT_T96x128_W4: e = launch_tile<96, 128, 2, 2>(a, ak, bk, st); break;
    case NEOGEMM_VARIANT_T64x64_W4: e = launch_tile<64, 64, 2, 2>(a, ak, bk, st); break;
    case NEOGEMM_VARIANT_C256x256_W4: e = launch_chain(a, bk, st); break;
    default: return NEOGEMM_ERR_BAD_ARG;
  }
  if (e != hipSuccess) {
    fprintf(stderr, "neogemm: tile kernel launch failed (variant %d): %s\n", v, hipGetErrorString(e));
    return NEOGEMM_ERR_LAUNCH;
  }
  if (a.ksplit > 1) {
    const size_t MN = (size_t)a.M * a.N;
    const unsigned blocks = (unsigned)((MN + 1023) / 1024);
    splitk_reduce_kernel<<<dim3(blocks, (unsigned)bt.count), 256, 0, st>>>(a.ws, a.C, a.M, a.N, a.ldc, a.ksplit, alpha, beta,
                                                                           a.bsc);
    e = hipGetLastError();
    if (e != hipSuccess) {
      fprintf(stderr, "neogemm: split-K reduce launch failed: %s\n", hipGetErrorString(e));
      return NEOGEMM_ERR_LAUNCH;
    }
  }
  return NEOGEMM_OK;
}

// Split-K partials of the entry point that allocates nothing (neogemm_bf16_noalloc): one array per GPU, laid out
// by the code object, held until the process ends.  In host code the name `scratch` only stands for the symbol;
// the device address is asked for once per device (scratch_on_current_device) and that pointer is what the kernels get.
static __device__ __align__(256) unsigned char scratch[NEOGEMM_NOALLOC_SCRATCH_BYTES];

static int scratch_on_current_device(void** out) {
  static std::mutex mu;
  static void* ptrs[64] = {};
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return NEOGEMM_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      fprintf(stderr, "neogemm: hipGetSymbolAddress(scratch) failed on device %d: %s\n", dev, hipGetErrorString(e));
      return NEOGEMM_ERR_LAUNCH;
    }
    ptrs[dev] = p;
  }
  *out = ptrs[dev];
  return NEOGEMM_OK;
}

}  // namespace neogemm

extern "C" {

int neogemm_bf16_noalloc(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda,
                         int64_t ldb, int64_t ldc, int b_layout, int c_layout, void* hip_stream) {
  // what neogemm_bf16 would be handed as a workspace for this shape, taken from the built-in array instead
  size_t need = 0;
  if (M > 0 && N > 0 && K > 0 && M <= 0x7fffffff && N <= 0x7fffffff && K <= 0x7fffffff)
    need = neogemm_bf16_workspace_bytes(M, N, K);
  if (need > (size_t)NEOGEMM_NOALLOC_SCRATCH_BYTES) return NEOGEMM_ERR_SCRATCH_LIMIT;
  void* ws = nullptr;
  if (need) {
    const int st = neogemm::scratch_on_current_device(&ws);
    if (st != NEOGEMM_OK) return st;
  }
  return neogemm::run(A, B, C, M, N, K, lda, ldb, ldc, b_layout, c_layout, ws, need, hip_stream, NEOGEMM_VARIANT_AUTO, 0,
                      0);
}

int neogemm_bf16(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                 int64_t ldc, int b_layout, int c_layout, void* workspace, size_t workspace_bytes, void* hip_stream) {
  return neogemm::run(A, B, C, M, N, K, lda, ldb, ldc, b_layout, c_layout, workspace, workspace_bytes, hip_stream,
                      NEOGEMM_VARIANT_AUTO, 0, 0);
}

int neogemm_bf16_scaled(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda,
                        int64_t ldb, int64_t ldc, int b_layout, int c_layout, float alpha, float beta, void* workspace,
                        size_t workspace_bytes, void* hip_stream) {
  if (!(alpha == alpha) || !(beta == beta)) return NEOGEMM_ERR_BAD_ARG;  // NaN scale factors
  return neogemm::run(A, B, C, M, N, K, lda, ldb, ldc, b_layout, c_layout, workspace, workspace_bytes, hip_stream,
                      NEOGEMM_VARIANT_AUTO, 0, 0, nullptr, alpha, beta);
}

int neogemm_bf16_batched(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda,
                         int64_t ldb, int64_t ldc, int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch,
                         int b_layout, int c_layout, void* workspace, size_t workspace_bytes, void* hip_stream) {
  if (batch == 0) return (M < 0 || N < 0 || K < 0) ? NEOGEMM_ERR_BAD_ARG : NEOGEMM_OK;
  neogemm::BatchArgs bt;
  bt.count = batch;
  bt.sa = stride_a;
  bt.sb = stride_b;
  bt.sc = stride_c;
  return neogemm::run(A, B, C, M, N, K, lda, ldb, ldc, b_layout, c_layout, workspace, workspace_bytes, hip_stream,
                      NEOGEMM_VARIANT_AUTO, 0, 0, nullptr, 1.f, 0.f, bt);
}

size_t neogemm_bf16_batched_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t batch) {
  if (M <= 0 || N <= 0 || K <= 0 || batch <= 0) return 0;
  const int s = neogemm::max_planned_split(M, N, K, batch);
  return s > 1 ? (size_t)s * (size_t)M * (size_t)N * sizeof(float) * (size_t)batch : 0;
}

int neogemm_bf16_variant(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda,
                         int64_t ldb, int64_t ldc, int b_layout, int c_layout, void* workspace,
                         size_t workspace_bytes, void* hip_stream, int variant, int split_k, int group_m) {
  return neogemm::run(A, B, C, M, N, K, lda, ldb, ldc, b_layout, c_layout, workspace, workspace_bytes, hip_stream,
                      variant, split_k, group_m);
}

int neogemm_bf16_profile(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda,
                         int64_t ldb, int64_t ldc, int b_layout, void* hip_stream, int variant, int group_m,
                         unsigned long long* phase_cycles, size_t phase_cycles_bytes) {
  if (!phase_cycles) return NEOGEMM_ERR_BAD_ARG;
  if (variant != NEOGEMM_VARIANT_T256x256_W4) return NEOGEMM_ERR_UNSUPPORTED;
  if (phase_cycles_bytes < neogemm_bf16_profile_bytes(M, N, variant)) return NEOGEMM_ERR_WORKSPACE;
  return neogemm::run(A, B, C, M, N, K, lda, ldb, ldc, b_layout, NEOGEMM_C_ROW, nullptr, 0, hip_stream, variant, 1,
                      group_m, phase_cycles);
}

size_t neogemm_bf16_profile_bytes(int64_t M, int64_t N, int variant) {
  if (M <= 0 || N <= 0) return 0;
  if (variant != NEOGEMM_VARIANT_T256x256_W4) return 0;
  return (size_t)neogemm::ceil_div(M, 256) * neogemm::ceil_div(N, 256) * 4 * 4 * sizeof(unsigned long long);
}

size_t neogemm_bf16_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const int s = neogemm::max_planned_split(M, N, K, 1);
  return s > 1 ? (size_t)s * (size_t)M * (size_t)N * sizeof(float) : 0;
}

int neogemm_bf16_plan(int64_t M, int64_t N, int64_t K, int b_layout, int c_layout, int aligned, int* variant,
                      int* split_k) {
  if (!variant || !split_k || M < 0 || N < 0 || K < 0) return NEOGEMM_ERR_BAD_ARG;
  if (c_layout != NEOGEMM_C_ROW && c_layout != NEOGEMM_C_COL) return NEOGEMM_ERR_BAD_ARG;
  if (b_layout != NEOGEMM_B_KN && b_layout != NEOGEMM_B_NK) return NEOGEMM_ERR_BAD_ARG;
  neogemm::plan(M, N, K, aligned != 0, c_layout, variant, split_k, 1, b_layout);
  return NEOGEMM_OK;
}

const char* neogemm_strerror(int status) {
  switch (status) {
    case NEOGEMM_OK: return "success";
    case NEOGEMM_ERR_BAD_ARG: return "bad argument (null pointer, negative size, leading dimension too small or unknown layout)";
    case NEOGEMM_ERR_WORKSPACE: return "workspace missing or too small (see neogemm_bf16_workspace_bytes)";
    case NEOGEMM_ERR_UNSUPPORTED: return "the requested kernel variant cannot run this shape or alignment";
    case NEOGEMM_ERR_LAUNCH: return "HIP kernel launch failed";
    case NEOGEMM_ERR_SCRATCH_LIMIT:
      return "the shape needs more split-K scratch than the built-in NEOGEMM_NOALLOC_SCRATCH_BYTES (32 MiB): "
             "call neogemm_bf16 with a workspace instead";
    default: return "unknown neogemm status";
  }
}

const char* neogemm_version(void) { return "neogemm 0.2 gfx950"; }

}  // extern "C"

#endif  // NEOGEMM_HAS_PART(0)
