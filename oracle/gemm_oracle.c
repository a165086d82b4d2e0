/*
 * TEST INFRASTRUCTURE — CPU restatement of the reference's BF16 GEMM path in plain C.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may call this; the product
 * (gemm_amd/, neoGEMM) never does.
 *
 * What is restated (the reference cannot be compiled here: it is CUDA with sm_90a/sm_100a PTX):
 *   oracle_gemm_bf16       the mathematical contract of gemmkernel (v01.cu:189-270): every output is
 *                          sum_k float(A[i,k]) * float(B[..]) accumulated in fp32, rounded once to
 *                          bf16 with round-to-nearest-even (__float2bfloat16, v01.cu:254-262);
 *                          layouts as flags so that it covers both the reference call
 *                          (B [N,K], C column-major: v01.cu:232-235,246,252; N = B.size(0),
 *                          nemgemmV03.cu:346) and C = gemm(A, B) with B [K,N].
 *   oracle_gemm_v1_tiles   the same product walked the way the reference walks it: one 64x64 output
 *                          tile per block, tile id -> (n = id % (N/64), m = id / (N/64))
 *                          (v01.cu:201-202), K in slabs of 64 (v01.cu:200,215) each consumed as four
 *                          16-deep MMAs that accumulate into the same fp32 registers
 *                          (v01.cu:232-235), epilogue C[col*M + row] (v01.cu:246,252).  Needs
 *                          M, N, K % 64 == 0 like the reference (nemgemmV03.cu:375).
 *   oracle_f32_to_bf16     the rounding itself, written with integer arithmetic.
 *
 * Pinned by tests/test_oracle.py against: a table of hand-derived bf16 roundings (ties, carries,
 * subnormals, inf/nan); exact-integer products whose result does not depend on summation order;
 * identity / one-hot selections; an independent fp64 triple loop; torch.matmul in fp32.
 *
 * A bf16 x bf16 product has at most 16 significant bits and is exact in fp32, so fused and unfused
 * multiply-add give the same fp32 sum here; only the order of additions can change the result.
 */
#include <stdint.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet the NaN, keep sign */
  /* round to nearest, ties to even: add 0x7fff plus the lsb of the part that is kept */
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

float oracle_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }

/* b_layout: 0 = B[K,N] (ldb >= N), 1 = B[N,K] (ldb >= K).  c_layout: 0 = row-major, 1 = column-major. */
void oracle_gemm_bf16(const uint16_t* A, const uint16_t* B, uint16_t* C, int64_t M, int64_t N, int64_t K,
                      int64_t lda, int64_t ldb, int64_t ldc, int b_layout, int c_layout) {
  for (int64_t i = 0; i < M; ++i) {
    for (int64_t j = 0; j < N; ++j) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        float a = bf16_to_f32(A[i * lda + k]);
        float b = b_layout ? bf16_to_f32(B[j * ldb + k]) : bf16_to_f32(B[k * ldb + j]);
        acc += a * b;
      }
      uint16_t r = oracle_f32_to_bf16(acc);
      if (c_layout) C[j * ldc + i] = r; else C[i * ldc + j] = r;
    }
  }
}

/* Reference walk: A[M,K], B[N,K], C column-major with ld = M.  Returns 0, or -1 if a size is not a
 * multiple of 64 (the reference asserts this, nemgemmV03.cu:375). */
int oracle_gemm_v1_tiles(const uint16_t* A, const uint16_t* B, uint16_t* C, int64_t M, int64_t N, int64_t K) {
  enum { BM = 64, BN = 64, BK = 64, MMA_K = 16 };
  if (M % BM || N % BN || K % BK) return -1;
  const int64_t blocks_n = N / BN, nblocks = (M / BM) * blocks_n;
  static float d[BM][BN];
  for (int64_t bid = 0; bid < nblocks; ++bid) {
    const int64_t bn = bid % blocks_n, bm = bid / blocks_n; /* v01.cu:201-202 */
    memset(d, 0, sizeof d);
    for (int64_t kb = 0; kb < K / BK; ++kb) {   /* v01.cu:215 */
      for (int s = 0; s < BK / MMA_K; ++s) {    /* four wgmma m64n64k16, v01.cu:232-235 */
        for (int i = 0; i < BM; ++i)
          for (int j = 0; j < BN; ++j) {
            float t = d[i][j];
            for (int k = 0; k < MMA_K; ++k) {
              const int64_t kk = kb * BK + s * MMA_K + k;
              t += bf16_to_f32(A[(bm * BM + i) * K + kk]) * bf16_to_f32(B[(bn * BN + j) * K + kk]);
            }
            d[i][j] = t;
          }
      }
    }
    for (int i = 0; i < BM; ++i)   /* epilogue: block_C = C + bn*BN*M + bm*BM, IDX(i,j) = j*M + i */
      for (int j = 0; j < BN; ++j) C[(bn * BN + j) * M + (bm * BM + i)] = oracle_f32_to_bf16(d[i][j]);
  }
  return 0;
}
