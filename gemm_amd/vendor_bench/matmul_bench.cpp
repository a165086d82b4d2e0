// Stand-alone timing harness: hipBLASLt and rocBLAS beside libneogemm on the same device buffers.
//
// Takes the role of the reference's cuBLAS harness (cublass/matmul.cu:82-196: N(0,1) host init,
// cublasGemmEx bf16 with fp32 compute :33-43, event-timed repetitions :169-183, TFLOPS print) with
// the vendor libraries of this platform.  Unlike the reference it takes the shape from the command
// line, handles non-square shapes (the reference's lda/ldc only work for squares, matmul.cu:36-37),
// scales the inputs by 1/sqrt(K), rotates the weight buffer for shapes whose working set fits the
// last-level cache, and cross-checks the libraries against each other.
//
//   matmul_bench M N K [reps=100] [b_layout=0|1] [variant=0] [split_k=0] [group_m=0] [nbuf=1]
//   matmul_bench ceiling [preheat_ms=1000]
//   matmul_bench loadpath M N K [b_layout=1] [strip=64] [row_tiles=1] [wide=0] [k_parts=1] [step_depth=128]
//
// One line of JSON per library on stdout.  Lines of timed runs carry "t0" / "t1", CLOCK_MONOTONIC seconds around the
// timed batches, so that a parent process that samples the board's power and clocks can tell which samples belong to
// which run.
//
// `ceiling` measures what the matrix cores sustain with nothing else going on: every wave runs the MFMA
// sequence of a 128x128 wave tile (the 256x256 GEMM tile's share of one wave) from registers, no memory
// traffic at all, one wave per SIMD on all 256 CUs, with all-zero operands and with N(0,1)/sqrt(8192) bf16
// operands (two register sets alternating, so that the operand buses toggle as they do on fresh data).  On
// zeros the chip holds its top clock; on random data it is power-limited and the clock drops: that rate, not
// the data-sheet peak, bounds any GEMM kernel on such inputs on this chip.
// It then runs the 128 MFMAs of a wave tile in four different orders (mfma_order_kernel) and the sequence next to the
// other activities of a GEMM main loop (gemm_like_kernel): what each costs at the power limit.
//
// `loadpath` measures the path into the CUs of a decode-shaped GEMM (few rows M, all of B read once) with the arithmetic
// taken away: every workgroup requests its strip of B (from HBM; B rotates through buffers larger than the last-level
// cache) and all of A (from L2), by global->LDS loads of whole 128-byte lines, and nothing else: no LDS reads, no MFMAs,
// no C.  What that takes bounds every kernel that gives a workgroup a strip of columns and all of K.
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>
#include <rocblas/rocblas.h>

#include <time.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <utility>
#include <vector>

#include "neogemm.h"

#define HIP_OK(x)                                                                          \
  do {                                                                                     \
    hipError_t e_ = (x);                                                                   \
    if (e_ != hipSuccess) {                                                                \
      fprintf(stderr, "%s:%d %s -> %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_)); \
      exit(1);                                                                             \
    }                                                                                      \
  } while (0)
#define BLT_OK(x)                                                          \
  do {                                                                     \
    hipblasStatus_t s_ = (x);                                              \
    if (s_ != HIPBLAS_STATUS_SUCCESS) {                                    \
      fprintf(stderr, "%s:%d %s -> %d\n", __FILE__, __LINE__, #x, (int)s_); \
      exit(1);                                                             \
    }                                                                      \
  } while (0)

static uint16_t f2bf(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float bf2f(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

// MATMUL_BENCH_PREHEAT_MS (environment, default 0): before timing a library, run it for that long, so that the
// chip's clocks have settled under that very load (the first launches after an idle period run slower).
static double preheat_ms_from_env() {
  const char* e = getenv("MATMUL_BENCH_PREHEAT_MS");
  return e ? atof(e) : 0.0;
}

static double monotonic_s() {
  timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}
static double g_t0 = 0.0, g_t1 = 0.0;  // CLOCK_MONOTONIC around the timed batches of the last time_ms()

template <class F>
static double time_ms(F&& launch, int reps, hipStream_t st) {
  hipEvent_t a, b;
  HIP_OK(hipEventCreate(&a));
  HIP_OK(hipEventCreate(&b));
  const int warm = std::max(3, reps / 10);
  for (int i = 0; i < warm; ++i) launch(i);
  HIP_OK(hipStreamSynchronize(st));
  static const double preheat = preheat_ms_from_env();
  for (double heated = 0.0; heated < preheat;) {
    HIP_OK(hipEventRecord(a, st));
    for (int i = 0; i < warm; ++i) launch(i);
    HIP_OK(hipEventRecord(b, st));
    HIP_OK(hipEventSynchronize(b));
    float t;
    HIP_OK(hipEventElapsedTime(&t, a, b));
    heated += t > 0.f ? t : 1.0;
  }
  // median of 5 batches
  std::vector<double> ms;
  g_t0 = monotonic_s();
  for (int batch = 0; batch < 5; ++batch) {
    HIP_OK(hipEventRecord(a, st));
    for (int i = 0; i < reps; ++i) launch(i);
    HIP_OK(hipEventRecord(b, st));
    HIP_OK(hipEventSynchronize(b));
    float t;
    HIP_OK(hipEventElapsedTime(&t, a, b));
    ms.push_back(t / reps);
  }
  g_t1 = monotonic_s();
  std::sort(ms.begin(), ms.end());
  HIP_OK(hipEventDestroy(a));
  HIP_OK(hipEventDestroy(b));
  return ms[ms.size() / 2];
}

static void report(const char* lib, int64_t M, int64_t N, int64_t K, int bl, double ms, const char* extra) {
  const double flop = 2.0 * M * N * K, bytes = 2.0 * (M * K + K * N + M * N);
  printf("{\"lib\": \"%s\", \"M\": %lld, \"N\": %lld, \"K\": %lld, \"b_layout\": %d, \"ms\": %.5f, \"tflops\": %.2f, "
         "\"pct_of_2500\": %.2f, \"gbps\": %.1f, \"pct_of_8000\": %.2f, \"t0\": %.4f, \"t1\": %.4f%s}\n",
         lib, (long long)M, (long long)N, (long long)K, bl, ms, flop / ms / 1e9, flop / ms / 1e9 / 25.0,
         bytes / ms / 1e6, bytes / ms / 1e6 / 80.0, g_t0, g_t1, extra);
  fflush(stdout);
}

// ---- MFMA-only power ceiling -------------------------------------------------------------------
typedef __attribute__((ext_vector_type(8))) __bf16 cbf16x8;
typedef __attribute__((ext_vector_type(4))) float cf32x4;
typedef __attribute__((ext_vector_type(16))) float cf32x16;

// frags: [set 2][operand 2][8][256 threads] bf16x8.  One pass = the MFMAs of a 128x128x32 wave-tile step:
// 64 x v_mfma_f32_16x16x32_bf16 (8x8 tiles of 16x16), or 32 x v_mfma_f32_32x32x16_bf16 (4x4 tiles of 32x32, two
// 16-deep steps).  Accumulators sit in the 256 AGPRs and are written in place, as in the GEMM kernel.
template <bool BIG>
__global__ __launch_bounds__(256) void mfma_ceiling_kernel(const cbf16x8* frags, float* out, int passes) {
  cbf16x8 a[2][8], b[2][8];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      a[s][i] = frags[((s * 2 + 0) * 8 + i) * 256 + threadIdx.x];
      b[s][i] = frags[((s * 2 + 1) * 8 + i) * 256 + threadIdx.x];
    }
  float total = 0.f;
  if constexpr (!BIG) {
    cf32x4 acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] = cf32x4{0.f, 0.f, 0.f, 0.f};
    for (int p = 0; p < passes; p += 2) {
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int c = 0; c < 8; ++c)
#pragma unroll
          for (int i = 0; i < 8; ++i)
            asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][c]) : "v"(b[s][c]), "v"(a[s][i]));
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        asm volatile("" : "+a"(acc[i][j]));
        total += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
      }
  } else {
    cf32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    for (int p = 0; p < passes; p += 2) {
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int h = 0; h < 2; ++h)  // the two 16-deep halves of the 32-deep step
#pragma unroll
          for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int i = 0; i < 4; ++i)
              asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0"
                           : "+a"(acc[i][c])
                           : "v"(b[s][4 * h + c]), "v"(a[s][4 * h + i]));
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        asm volatile("" : "+a"(acc[i][j]));
#pragma unroll
        for (int v = 0; v < 16; ++v) total += acc[i][j][v];
      }
  }
  out[blockIdx.x * 256 + threadIdx.x] = total;
}

// The same MFMA sequence (16x16x32) with, one by one, the other activities of a GEMM main loop at the rates of the
// 256x256 tile kernel, none of which changes what is computed — so the drop in rate is what the activity costs at
// the chip's power limit:
//   PARTS & 1  operand fragments are read from LDS every pass (16 x ds_read_b128 per wave: 64 KiB per CU and pass)
//              into a second register copy, as the kernel's double-buffered fragments are
//   PARTS & 2  direct-to-LDS loads, 8 KiB per wave and pass (32 KiB per CU and pass: a 64-deep tile of A and of B per
//              two passes), from a 64 KiB region per workgroup that stays in the L2
//   PARTS & 4  a workgroup barrier per pass
//   PARTS & 8  the matrix cores idle a fifth of the time (s_sleep after every pass): same work, lower utilisation
template <int PARTS>
__global__ __launch_bounds__(256) void gemm_like_kernel(const cbf16x8* frags, const char* src, float* out, int passes) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];  // 128 KiB of fragments + 32 KiB load ring
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  typedef __attribute__((address_space(3))) cbf16x8 lds_frag;
  lds_frag* myfr = (lds_frag*)(__attribute__((address_space(3))) char*)smem + wave * 2048 + lane;  // [set][16][64 lanes]
  cbf16x8 a[2][8], b[2][8];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      a[s][i] = frags[((s * 2 + 0) * 8 + i) * 256 + threadIdx.x];
      b[s][i] = frags[((s * 2 + 1) * 8 + i) * 256 + threadIdx.x];
      myfr[(s * 16 + i) * 64] = a[s][i];
      myfr[(s * 16 + 8 + i) * 64] = b[s][i];
    }
  __syncthreads();
  const uint32_t ring = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem + 131072 + wave * 8192;
  const uint64_t base = (uint64_t)src + (uint64_t)blockIdx.x * 65536;
  typedef __attribute__((ext_vector_type(4))) int ci32x4;
  const ci32x4 rsrc = {(int)(uint32_t)base, (int)(uint32_t)(base >> 32), 65536, 0x00020000};
  const uint32_t voff = lane * 16;
  cf32x4 acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = cf32x4{0.f, 0.f, 0.f, 0.f};
  for (int p = 0; p < passes; p += 2) {
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      asm volatile("" ::: "memory");  // the LDS reads of a pass stay in that pass
      if constexpr ((PARTS & 2) != 0) {
        // at most the 8 loads of the pass before stay in flight
        asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        const uint32_t soff = (uint32_t)((wave * 16384 + ((p + s) & 1) * 8192) & 65535);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" ::"s"(ring) : "memory");
#pragma unroll
        for (int j = 0; j < 4; ++j)
          asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:%3 sc1 lds" ::"v"(voff), "s"(rsrc), "s"(soff), "n"(j * 1024)
                       : "memory");
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" ::"s"(ring + 4096) : "memory");
#pragma unroll
        for (int j = 0; j < 4; ++j)
          asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:%3 sc1 lds" ::"v"(voff), "s"(rsrc), "s"(soff + 4096),
                       "n"(j * 1024)
                       : "memory");
      }
#pragma unroll
      for (int c = 0; c < 8; ++c) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
          asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][c]) : "v"(b[s][c]), "v"(a[s][i]));
        if constexpr ((PARTS & 1) != 0) {
          // two fragment reads per eight MFMAs: the other copy is refilled while this one is in use
          a[s ^ 1][c] = myfr[((s ^ 1) * 16 + c) * 64];
          b[s ^ 1][c] = myfr[((s ^ 1) * 16 + 8 + c) * 64];
        }
      }
      if constexpr ((PARTS & 4) != 0) __builtin_amdgcn_s_barrier();
      if constexpr ((PARTS & 8) != 0) __builtin_amdgcn_s_sleep(4);  // 256 cycles after 1024 cycles of MFMAs
    }
  }
  asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  float total = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      asm volatile("" : "+a"(acc[i][j]));
      total += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
    }
  out[blockIdx.x * 256 + threadIdx.x] = total;
}

// The order in which a wave visits its 8x8 accumulator tiles over two K steps (128 MFMAs, the same instructions on
// the same operands every time): what changes is how many operand registers and accumulators differ from one MFMA
// to the next, and with it the power the sequence draws.
//   ORDER 0  column by column: the B fragment is held for eight MFMAs, the A fragment changes every time
//   ORDER 1  2x2 blocks of tiles, the blocks in rows of alternating direction: one of the two operands is held at
//            every step (the walk of neogemm's tile kernel)
//   ORDER 2  along diagonals: both operands change at every step
//   ORDER 3  the walk of ORDER 1, but both K steps of a tile back to back: every second MFMA accumulates into the
//            tile the one before it wrote (both operands change at every step)
template <class F, int... I>
__device__ __forceinline__ void order_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
constexpr int order_c(int order, int m) {  // m: 0..63, position in the walk over the tiles
  if (order == 0) return m / 8;
  if (order == 2) return (m / 8 + m % 8) % 8;
  return ((m / 4) / 4) * 2 + ((m % 4) >> 1);
}
constexpr int order_i(int order, int m) {
  if (order == 0 || order == 2) return m % 8;
  const int blk = m / 4, in = m % 4, bc = blk / 4;
  const int bi = (bc & 1) ? 3 - blk % 4 : blk % 4;
  return bi * 2 + ((in & 1) ^ (in >> 1));
}
__device__ __forceinline__ void order_mfma(cf32x4& acc, cbf16x8 x, cbf16x8 y) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(x), "v"(y));
}
template <int ORDER>
__global__ __launch_bounds__(256) void mfma_order_kernel(const cbf16x8* frags, float* out, int passes) {
  cbf16x8 a[2][8], b[2][8];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      a[s][i] = frags[((s * 2 + 0) * 8 + i) * 256 + threadIdx.x];
      b[s][i] = frags[((s * 2 + 1) * 8 + i) * 256 + threadIdx.x];
    }
  cf32x4 acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = cf32x4{0.f, 0.f, 0.f, 0.f};
  for (int p = 0; p < passes; p += 2) {
    order_for_impl(
        [&](auto mc) {
          constexpr int m = decltype(mc)::value;
          constexpr int s = ORDER == 3 ? m % 2 : m / 64, t = ORDER == 3 ? m / 2 : m % 64;
          constexpr int c = order_c(ORDER, t), i = order_i(ORDER, t);
          order_mfma(acc[i][c], b[s][c], a[s][i]);
        },
        std::make_integer_sequence<int, 128>{});
  }
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  float total = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      asm volatile("" : "+a"(acc[i][j]));
      total += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
    }
  out[blockIdx.x * 256 + threadIdx.x] = total;
}

static int run_ceiling(int preheat_ms) {
  hipStream_t st;
  HIP_OK(hipStreamCreate(&st));
  const size_t nfrag = 2 * 2 * 8 * 256;
  std::vector<uint16_t> h(nfrag * 8), z(nfrag * 8, 0);
  std::mt19937 rng(7);
  std::normal_distribution<float> nd(0.f, 1.f);
  const float sc = 1.0f / std::sqrt(8192.f);
  for (auto& v : h) v = f2bf(nd(rng) * sc);
  void *dfr, *dz, *dout;
  HIP_OK(hipMalloc(&dfr, h.size() * 2));
  HIP_OK(hipMalloc(&dz, z.size() * 2));
  HIP_OK(hipMalloc(&dout, 256 * 256 * 4));
  HIP_OK(hipMemcpy(dfr, h.data(), h.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dz, z.data(), z.size() * 2, hipMemcpyHostToDevice));
  const int passes = 2048, wgs = 256;  // one workgroup of four waves per CU: one wave per SIMD, as in the 256x256 GEMM tile
  const double flop = (double)wgs * 4 * passes * 64.0 * 16384.0;  // per launch, either instruction
  struct Case { const char* insn; const char* data; bool big; const void* fr; };
  const Case cases[] = {{"v_mfma_f32_16x16x32_bf16", "zeros", false, dz}, {"v_mfma_f32_16x16x32_bf16", "randn", false, dfr},
                        {"v_mfma_f32_32x32x16_bf16", "zeros", true, dz},  {"v_mfma_f32_32x32x16_bf16", "randn", true, dfr}};
  for (const Case& c : cases) {
    auto launch = [&](int) {
      if (c.big) mfma_ceiling_kernel<true><<<wgs, 256, 0, st>>>((const cbf16x8*)c.fr, (float*)dout, passes);
      else mfma_ceiling_kernel<false><<<wgs, 256, 0, st>>>((const cbf16x8*)c.fr, (float*)dout, passes);
    };
    // time-based preheat: clocks and power settle under this very load before anything is timed
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    float heated = 0.f;
    while (heated < (float)preheat_ms) {
      HIP_OK(hipEventRecord(e0, st));
      for (int i = 0; i < 20; ++i) launch(i);
      HIP_OK(hipEventRecord(e1, st));
      HIP_OK(hipEventSynchronize(e1));
      float t;
      HIP_OK(hipEventElapsedTime(&t, e0, e1));
      heated += t;
    }
    HIP_OK(hipGetLastError());
    const double ms = time_ms(launch, 40, st);
    const double tflops = flop / ms / 1e9;
    // with 64 (16) independent accumulators a wave issues MFMAs back to back: 16 (32) cycles each, 1024 flop per
    // cycle and SIMD, so the rate implies the clock the chip held
    printf("{\"ceiling\": \"%s\", \"operands\": \"%s\", \"ms\": %.5f, \"tflops\": %.1f, \"pct_of_2500\": %.2f, "
           "\"implied_mhz\": %.0f, \"workgroups\": %d, \"waves_per_simd\": 1, \"t0\": %.4f, \"t1\": %.4f}\n",
           c.insn, c.data, ms, tflops, tflops / 25.0, tflops * 1e12 / (256.0 * 4 * 1024.0) / 1e6, wgs, g_t0, g_t1);
    fflush(stdout);
  }
  // the order of the MFMAs of a wave tile, N(0,1) operands
  {
    struct Ord { const char* name; void (*kern)(const cbf16x8*, float*, int); };
    const Ord ords[] = {{"column by column", mfma_order_kernel<0>}, {"2x2 blocks, serpentine", mfma_order_kernel<1>},
                        {"diagonals (both operands change)", mfma_order_kernel<2>},
                        {"2x2 blocks, both K steps of a tile back to back", mfma_order_kernel<3>}};
    for (int zero = 0; zero < 2; ++zero)
    for (const Ord& o : ords) {
      const void* fr = zero ? dz : dfr;  // on zeros the clock is not limited: a slower row there is issue stalls
      auto launch = [&](int) { o.kern<<<wgs, 256, 0, st>>>((const cbf16x8*)fr, (float*)dout, passes); };
      hipEvent_t e0, e1;
      HIP_OK(hipEventCreate(&e0));
      HIP_OK(hipEventCreate(&e1));
      for (float heated = 0.f; heated < (float)preheat_ms;) {
        HIP_OK(hipEventRecord(e0, st));
        for (int i = 0; i < 20; ++i) launch(i);
        HIP_OK(hipEventRecord(e1, st));
        HIP_OK(hipEventSynchronize(e1));
        float t;
        HIP_OK(hipEventElapsedTime(&t, e0, e1));
        heated += t;
      }
      HIP_OK(hipGetLastError());
      const double ms = time_ms(launch, 40, st);
      const double tflops = flop / ms / 1e9;
      printf("{\"ceiling\": \"mfma_order\", \"order\": \"%s\", \"operands\": \"%s\", \"ms\": %.5f, \"tflops\": %.1f, "
             "\"pct_of_2500\": %.2f, \"t0\": %.4f, \"t1\": %.4f}\n", o.name, zero ? "zeros" : "randn", ms, tflops, tflops / 25.0,
             g_t0, g_t1);
      fflush(stdout);
    }
  }
  // the MFMA sequence next to the other parts of a GEMM main loop, N(0,1) operands
  {
    void* dsrc;
    const size_t src_bytes = (size_t)wgs * 65536;
    std::vector<uint16_t> hs(src_bytes / 2);
    for (auto& v : hs) v = f2bf(nd(rng) * sc);
    HIP_OK(hipMalloc(&dsrc, src_bytes));
    HIP_OK(hipMemcpy(dsrc, hs.data(), src_bytes, hipMemcpyHostToDevice));
    const size_t lds = 131072 + 32768;
    struct Like { int parts; const char* name; void (*kern)(const cbf16x8*, const char*, float*, int); };
    const Like likes[] = {{0, "mfma", gemm_like_kernel<0>},
                          {8, "mfma at 80% duty", gemm_like_kernel<8>},
                          {1, "mfma+lds_reads", gemm_like_kernel<1>},
                          {2, "mfma+l2_to_lds_loads", gemm_like_kernel<2>},
                          {3, "mfma+lds_reads+l2_to_lds_loads", gemm_like_kernel<3>},
                          {7, "mfma+lds_reads+l2_to_lds_loads+barrier", gemm_like_kernel<7>}};
    for (int zero = 0; zero < 2; ++zero)
    for (const Like& l : likes) {
      // on all-zero operands the chip is not power-limited: what an activity costs there is issue slots and stalls
      if (zero) HIP_OK(hipMemset(dsrc, 0, src_bytes));
      const void* fr = zero ? dz : dfr;
      HIP_OK(hipFuncSetAttribute((const void*)l.kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
      auto launch = [&](int) { l.kern<<<wgs, 256, lds, st>>>((const cbf16x8*)fr, (const char*)dsrc, (float*)dout, passes); };
      hipEvent_t e0, e1;
      HIP_OK(hipEventCreate(&e0));
      HIP_OK(hipEventCreate(&e1));
      for (float heated = 0.f; heated < (float)preheat_ms;) {
        HIP_OK(hipEventRecord(e0, st));
        for (int i = 0; i < 20; ++i) launch(i);
        HIP_OK(hipEventRecord(e1, st));
        HIP_OK(hipEventSynchronize(e1));
        float t;
        HIP_OK(hipEventElapsedTime(&t, e0, e1));
        heated += t;
      }
      HIP_OK(hipGetLastError());
      const double ms = time_ms(launch, 40, st);
      const double tflops = flop / ms / 1e9;
      printf("{\"ceiling\": \"gemm_like\", \"parts\": \"%s\", \"operands\": \"%s\", \"ms\": %.5f, \"tflops\": %.1f, "
             "\"pct_of_2500\": %.2f, \"t0\": %.4f, \"t1\": %.4f}\n", l.name, zero ? "zeros" : "randn", ms, tflops, tflops / 25.0,
             g_t0, g_t1);
      fflush(stdout);
    }
  }
  return 0;
}

// ---- load path of a decode-shaped GEMM, arithmetic taken away ---------------------------------------
// One 128-deep step of a workgroup: B 2 * strip / 8 requests (8 rows x 128 B each; B [K,N]: 16 requests of 8 k-rows x
// 128 B per 64 columns), A 2 * rows / 8 requests.  The NW waves take the requests of a step round-robin; each keeps at
// most D in flight.  With row_tiles > 1 a strip belongs to that many workgroups, each with its share of A's rows (the
// decomposition of a stream-K library kernel with a 64-row tile: B is requested row_tiles times, once from HBM).
typedef __attribute__((ext_vector_type(4))) int ci32x4b;
template <int D>
__global__ __launch_bounds__(512) void loadpath_kernel(const char* A, const char* B, float* out, int M, int K, int N, int strip,
                                                       int with_a, int b_kn, int row_tiles, int wide, int k_parts, int pshift) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const uint32_t l0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), nw = blockDim.x >> 6;
  const int lane = threadIdx.x & 63;
  // one buffer resource per operand; a request is told apart by a scalar offset.  Lanes past the end of A (rows beyond
  // M) are out of the resource's range: they read as zeros and touch no memory.
  // the workgroups of one strip sit on one XCD (workgroup id mod 8), next to each other in dispatch order, so that the
  // strip's B comes out of HBM once and out of that XCD's L2 for the others; the host rounds the strip count to eights
  // With k_parts > 1 (and row_tiles 1) a strip belongs to that many workgroups, each with its range of K (a split-K or
  // stream-K decomposition: B is requested once, A's bytes per workgroup shrink); part p of every strip runs on the
  // XCDs p, p + k_parts, ..., so an XCD's L2 holds one range of A.
  const int kp = k_parts > 1 ? (blockIdx.x & 7) % k_parts : 0;
  const int rt = k_parts > 1 ? 0 : (blockIdx.x >> 3) % row_tiles;
  const int strip_id = k_parts > 1 ? (blockIdx.x >> 3) * (8 / k_parts) + (blockIdx.x & 7) / k_parts
                                   : (blockIdx.x / (8 * row_tiles)) * 8 + (blockIdx.x & 7);
  const int tile_rows = (M + row_tiles - 1) / row_tiles;
  const int rows = min(tile_rows, M - rt * tile_rows);   // the host checked that every tile has rows
  const uint64_t bb = b_kn ? (uint64_t)B + (uint64_t)strip_id * strip * 2 : (uint64_t)B + (uint64_t)strip_id * strip * K * 2;
  const uint64_t ab = (uint64_t)A + (uint64_t)rt * tile_rows * K * 2;
  const uint32_t ldb = b_kn ? (uint32_t)N * 2 : (uint32_t)K * 2;
  const ci32x4b ra = {(int)(uint32_t)ab, (int)((ab >> 32) & 0xffff), (int)((uint32_t)rows * K * 2), 0x00020000};
  // a request is 8 rows x 128 bytes, or (wide) 4 rows x 256 bytes: the same eight cache lines, in half as many rows
  // (wide: bit 0 for A's requests, bit 1 for B's)
  const bool wide_a = wide & 1, wide_b = wide & 2;
  const uint32_t voff_b = wide_b ? (lane >> 4) * ldb + (lane & 15) * 16 : (lane >> 3) * ldb + (lane & 7) * 16;
  const uint32_t voff_a = wide_a ? (lane >> 4) * (uint32_t)K * 2 + (lane & 15) * 16 : (lane >> 3) * (uint32_t)K * 2 + (lane & 7) * 16;
  asm volatile("s_mov_b32 m0, %0" ::"s"(l0 + wave * 1024) : "memory");
  const int halves = strip / 64;   // B [K,N]: 128-byte pieces of a k-row
  // K-major operands: a step is 64 << pshift deep (pshift 1: 128), i.e. 1 << pshift pieces of 128 bytes per row, requested
  // back to back; the deeper the step, the longer the run of consecutive bytes a row contributes at a time
  const int pieces = 1 << pshift;
  const int nb = b_kn ? 16 * halves : strip / 8 * pieces, na = with_a ? (rows + 7) / 8 * pieces : 0;
  const int steps = b_kn ? K / 128 / k_parts : K / (64 << pshift) / k_parts;
  for (int s = kp * steps; s < (kp + 1) * steps; ++s) {
    // B [N,K]: the strip's rows, 256 bytes further along K per step; B [K,N]: 128 k-rows further down per step
    const uint64_t bs = b_kn ? bb + (uint64_t)s * 128 * ldb : bb + (uint64_t)s * (128u << pshift);
    const ci32x4b rb = {(int)(uint32_t)bs, (int)((bs >> 32) & 0xffff), (int)0x7fffffff, 0x00020000};
    for (int r = wave; r < nb + na; r += nw) {
      if (r < nb) {
        const uint32_t soff = wide_b ? (uint32_t)r * 4 * ldb   // B [K,N]: the host asked for a strip of 128 columns
                              : b_kn ? (uint32_t)(r / halves) * 8 * ldb + (r % halves) * 128 : (uint32_t)(r >> pshift) * 8 * ldb + (r & (pieces - 1)) * 128;
        asm volatile("buffer_load_dwordx4 %0, %1, %2 offen sc1 lds" ::"v"(voff_b), "s"(rb), "s"(soff) : "memory");
      } else {
        const int q = r - nb;
        const uint32_t soff = wide_a ? (uint32_t)q * 4 * K * 2 + (uint32_t)s * 256 : (uint32_t)(q >> pshift) * 8 * K * 2 + (q & (pieces - 1)) * 128 + (uint32_t)s * (b_kn ? 256u : 128u << pshift);
        asm volatile("buffer_load_dwordx4 %0, %1, %2 offen sc1 lds" ::"v"(voff_a), "s"(ra), "s"(soff) : "memory");
      }
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(D) : "memory");
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  out[blockIdx.x * blockDim.x + threadIdx.x] = ((float*)smem)[threadIdx.x];
}

static int run_loadpath(int64_t M, int64_t N, int64_t K, int b_layout, int strip, int row_tiles, int wide, int k_parts, int depth) {
  if (M < 1 || N < strip || K < 128 || K % 128 || N % strip || strip % 8 || strip < 8 || strip > 128 || (b_layout == 0 && strip % 64) ||
      (k_parts != 1 && k_parts != 2 && k_parts != 4 && k_parts != 8) || (k_parts > 1 && (row_tiles != 1 || (N / strip) % (8 / k_parts) ||
                                                                                    K / 128 % k_parts)) ||
      (depth != 128 && depth != 256 && depth != 512 && depth != 1024) || (depth != 128 && (b_layout == 0 || wide)) ||
      K % (depth * k_parts) || wide < 0 || wide > 3 || ((wide & 2) && b_layout == 0 && strip != 128) || ((wide & 2) && strip % 4) || row_tiles < 1 || (row_tiles > 1 && (N / strip) % 8) || (M + row_tiles - 1) / row_tiles * (row_tiles - 1) >= M || (uint64_t)M * K * 2 > 0x7fffffffull ||
      (uint64_t)strip * K * 2 > 0x7fffffffull || (uint64_t)K * N * 2 > 0x7fffffffull * 2) {
    fprintf(stderr, "loadpath: K a multiple of 128, N a multiple of the strip (a multiple of 8 up to 128; 64 or 128 with B [K,N]), "
                    "row_tiles >= 1 with rows in every tile (and then a strip count that is a multiple of 8)\n");
    return 2;
  }
  hipStream_t st;
  HIP_OK(hipStreamCreate(&st));
  const size_t b_bytes = (size_t)N * K * 2;
  const int nbuf = (int)std::min<size_t>(8, (1ull << 30) / b_bytes + 1);
  void *dA, *dout;
  std::vector<void*> dB(nbuf);
  HIP_OK(hipMalloc(&dA, (size_t)M * K * 2));
  HIP_OK(hipMemset(dA, 1, (size_t)M * K * 2));
  for (auto& p : dB) {
    HIP_OK(hipMalloc(&p, b_bytes));
    HIP_OK(hipMemset(p, 1, b_bytes));
  }
  const int wgs = (int)(N / strip) * row_tiles * k_parts;
  HIP_OK(hipMalloc(&dout, (size_t)wgs * 512 * 4));
  HIP_OK(hipFuncSetAttribute((const void*)loadpath_kernel<16>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
  for (int with_a = 0; with_a < 2; ++with_a)
    for (int threads : {256, 512}) {
      auto launch = [&](int i) {
        loadpath_kernel<16><<<wgs, threads, 65536, st>>>((const char*)dA, (const char*)dB[i % nbuf], (float*)dout, (int)M, (int)K, (int)N, strip,
                                                         with_a, b_layout == 0, row_tiles, wide, k_parts, depth == 1024 ? 4 : depth == 512 ? 3 : depth == 256 ? 2 : 1);
      };
      const double ms = time_ms(launch, 100, st);
      HIP_OK(hipGetLastError());
      printf("{\"loadpath\": \"%s\", \"M\": %lld, \"N\": %lld, \"K\": %lld, \"b_layout\": %d, \"strip\": %d, \"row_tiles\": %d, \"k_parts\": %d, \"step_depth\": %d, \"request\": \"%s\", \"workgroups\": %d, "
             "\"waves\": %d, \"requests_in_flight_per_wave\": 16, \"us\": %.2f, \"b_tbps\": %.2f, \"a_from_l2_mb\": %.1f}\n",
             with_a ? "B from HBM + all of A from L2 per workgroup" : "B from HBM only", (long long)M, (long long)N, (long long)K,
             b_layout, strip, row_tiles, k_parts, depth, wide == 3 ? "4 rows x 256 B" : wide == 1 ? "A 4 rows x 256 B, B 8 rows x 128 B" : wide == 2 ? "A 8 rows x 128 B, B 4 rows x 256 B" : "8 rows x 128 B", wgs, threads / 64, ms * 1e3, (double)b_bytes / ms / 1e9,
             with_a ? (double)(N / strip) * M * K * 2 / 1e6 : 0.0);   // (each of k_parts workgroups takes its share of these)
      fflush(stdout);
    }
  return 0;
}

int main(int argc, char** argv) {
  if (argc >= 2 && strcmp(argv[1], "ceiling") == 0) return run_ceiling(argc > 2 ? atoi(argv[2]) : 1000);
  if (argc >= 5 && strcmp(argv[1], "loadpath") == 0)
    return run_loadpath(atoll(argv[2]), atoll(argv[3]), atoll(argv[4]), argc > 5 ? atoi(argv[5]) : 1, argc > 6 ? atoi(argv[6]) : 64,
                        argc > 7 ? atoi(argv[7]) : 1, argc > 8 ? atoi(argv[8]) : 0,
                        argc > 9 ? atoi(argv[9]) : 1, argc > 10 ? atoi(argv[10]) : 128);
  if (argc < 4) {
    fprintf(stderr, "usage: %s M N K [reps] [b_layout] [variant] [split_k] [group_m] [nbuf]\n       %s ceiling [preheat_ms]\n"
            "       %s loadpath M N K [b_layout] [strip] [row_tiles] [wide] [k_parts] [step_depth]\n", argv[0], argv[0], argv[0]);
    return 2;
  }
  const int64_t M = atoll(argv[1]), N = atoll(argv[2]), K = atoll(argv[3]);
  const int reps = argc > 4 ? atoi(argv[4]) : 100;
  const int bl = argc > 5 ? atoi(argv[5]) : 0;
  const int variant = argc > 6 ? atoi(argv[6]) : 0;
  const int split_k = argc > 7 ? atoi(argv[7]) : 0;
  const int group_m = argc > 8 ? atoi(argv[8]) : 0;
  const int nbuf = argc > 9 ? std::max(1, atoi(argv[9])) : 1;
  const bool only_ours = getenv("NEOGEMM_ONLY") != nullptr;

  hipStream_t st;
  HIP_OK(hipStreamCreate(&st));

  // N(0,1)/sqrt(K) inputs (cf. matmul.cu:53-59, which leaves them unscaled)
  std::mt19937 rng(69);
  std::normal_distribution<float> nd(0.f, 1.f);
  const float sc = 1.0f / std::sqrt((float)K);
  std::vector<uint16_t> hA((size_t)M * K), hB((size_t)K * N);
  for (auto& v : hA) v = f2bf(nd(rng) * sc);
  for (auto& v : hB) v = f2bf(nd(rng) * sc);  // stored as given: [K,N] for b_layout 0, [N,K] for 1
  if (getenv("NEOGEMM_ZERO_INPUTS")) {  // power experiment only: zeros switch far fewer wires
    std::fill(hA.begin(), hA.end(), 0);
    std::fill(hB.begin(), hB.end(), 0);
  }
  void *dA, *dC, *dC2;
  std::vector<void*> dB(nbuf);
  HIP_OK(hipMalloc(&dA, hA.size() * 2));
  HIP_OK(hipMalloc(&dC, (size_t)M * N * 2));
  HIP_OK(hipMalloc(&dC2, (size_t)M * N * 2));
  HIP_OK(hipMemcpy(dA, hA.data(), hA.size() * 2, hipMemcpyHostToDevice));
  for (int i = 0; i < nbuf; ++i) {
    HIP_OK(hipMalloc(&dB[i], hB.size() * 2));
    HIP_OK(hipMemcpy(dB[i], hB.data(), hB.size() * 2, hipMemcpyHostToDevice));
  }
  const int64_t ldb = bl == 0 ? N : K;

  // ---- libneogemm
  size_t ws_bytes = neogemm_bf16_workspace_bytes(M, N, K);
  if (split_k > 1) ws_bytes = std::max(ws_bytes, (size_t)split_k * M * N * 4);
  void* ws = nullptr;
  if (ws_bytes) HIP_OK(hipMalloc(&ws, ws_bytes));
  int pv = 0, ps = 0;
  neogemm_bf16_plan(M, N, K, bl, 0, 1, &pv, &ps);
  auto ours = [&](int i) {
    int s = neogemm_bf16_variant(dA, dB[i % nbuf], dC, M, N, K, K, ldb, N, bl, NEOGEMM_C_ROW, ws, ws_bytes, st,
                                 variant, split_k, group_m);
    if (s != NEOGEMM_OK) {
      fprintf(stderr, "neogemm: %s\n", neogemm_strerror(s));
      exit(1);
    }
  };
  {
    double ms = time_ms(ours, reps, st);
    char extra[128];
    snprintf(extra, sizeof extra, ", \"variant\": %d, \"split_k\": %d, \"group_m\": %d", variant ? variant : pv,
             split_k ? split_k : ps, group_m);
    report("neogemm", M, N, K, bl, ms, extra);
  }
  if (only_ours) return 0;

  // ---- hipBLASLt: row-major C[M,N] = A.B is column-major C'[N,M] = op(B') . A'
  hipblasLtHandle_t lt;
  BLT_OK(hipblasLtCreate(&lt));
  hipblasLtMatmulDesc_t desc;
  BLT_OK(hipblasLtMatmulDescCreate(&desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  hipblasOperation_t opB = bl == 0 ? HIPBLAS_OP_N : HIPBLAS_OP_T, opA = HIPBLAS_OP_N;
  BLT_OK(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSA, &opB, sizeof opB));
  BLT_OK(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSB, &opA, sizeof opA));
  hipblasLtMatrixLayout_t lB, lA, lC;
  if (bl == 0) BLT_OK(hipblasLtMatrixLayoutCreate(&lB, HIP_R_16BF, N, K, N));
  else BLT_OK(hipblasLtMatrixLayoutCreate(&lB, HIP_R_16BF, K, N, K));
  BLT_OK(hipblasLtMatrixLayoutCreate(&lA, HIP_R_16BF, K, M, K));
  BLT_OK(hipblasLtMatrixLayoutCreate(&lC, HIP_R_16BF, N, M, N));
  hipblasLtMatmulPreference_t pref;
  BLT_OK(hipblasLtMatmulPreferenceCreate(&pref));
  size_t lt_ws_bytes = 256ull << 20;
  void* lt_ws;
  HIP_OK(hipMalloc(&lt_ws, lt_ws_bytes));
  BLT_OK(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &lt_ws_bytes,
                                               sizeof lt_ws_bytes));
  const int want = 8;
  hipblasLtMatmulHeuristicResult_t res[want];
  int found = 0;
  BLT_OK(hipblasLtMatmulAlgoGetHeuristic(lt, desc, lB, lA, lC, lC, pref, want, res, &found));
  const float alpha = 1.f, beta = 0.f;
  double best = 1e30;
  int best_i = -1;
  for (int a = 0; a < found; ++a) {
    auto fn = [&](int i) {
      BLT_OK(hipblasLtMatmul(lt, desc, &alpha, dB[i % nbuf], lB, dA, lA, &beta, dC2, lC, dC2, lC, &res[a].algo, lt_ws,
                             lt_ws_bytes, st));
    };
    double ms = time_ms(fn, std::max(10, reps / 4), st);
    if (ms < best) best = ms, best_i = a;
  }
  if (best_i >= 0) {
    auto fn = [&](int i) {
      BLT_OK(hipblasLtMatmul(lt, desc, &alpha, dB[i % nbuf], lB, dA, lA, &beta, dC2, lC, dC2, lC, &res[best_i].algo,
                             lt_ws, lt_ws_bytes, st));
    };
    double ms = time_ms(fn, reps, st);
    char extra[96];
    snprintf(extra, sizeof extra, ", \"algo_rank\": %d, \"algos_tried\": %d", best_i, found);
    report("hipblaslt", M, N, K, bl, ms, extra);
  } else {
    fprintf(stderr, "hipblaslt: no algorithm found\n");
  }

  // ---- rocBLAS gemm_ex
  {
    rocblas_handle rb;
    if (rocblas_create_handle(&rb) == rocblas_status_success) {
      rocblas_set_stream(rb, st);
      auto fn = [&](int i) {
        rocblas_gemm_ex(rb, bl == 0 ? rocblas_operation_none : rocblas_operation_transpose, rocblas_operation_none,
                        (rocblas_int)N, (rocblas_int)M, (rocblas_int)K, &alpha, dB[i % nbuf], rocblas_datatype_bf16_r,
                        (rocblas_int)ldb, dA, rocblas_datatype_bf16_r, (rocblas_int)K, &beta, dC2,
                        rocblas_datatype_bf16_r, (rocblas_int)N, dC2, rocblas_datatype_bf16_r, (rocblas_int)N,
                        rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
      };
      double ms = time_ms(fn, reps, st);
      report("rocblas", M, N, K, bl, ms, "");
      rocblas_destroy_handle(rb);
    }
  }

  // ---- cross-check ours against the vendor result left in dC2 (cf. matmul.cu:61-75, abs 0.1 there)
  {
    ours(0);
    HIP_OK(hipStreamSynchronize(st));
    std::vector<uint16_t> c1((size_t)M * N), c2((size_t)M * N);
    HIP_OK(hipMemcpy(c1.data(), dC, c1.size() * 2, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(c2.data(), dC2, c2.size() * 2, hipMemcpyDeviceToHost));
    double num = 0, den = 0, maxabs = 0;
    for (size_t i = 0; i < c1.size(); ++i) {
      double a = bf2f(c1[i]), b = bf2f(c2[i]);
      num += (a - b) * (a - b);
      den += b * b;
      maxabs = std::max(maxabs, std::fabs(a - b));
    }
    printf("{\"check\": \"neogemm_vs_vendor\", \"rel_fro\": %.3e, \"max_abs\": %.3e}\n", std::sqrt(num / std::max(den, 1e-300)),
           maxabs);
  }
  return 0;
}
