/*
 * neogemm.h — C ABI of the MI355X (gfx950) BF16 GEMM library `libneogemm.so`.
 *
 * This is the boundary a replacement for the reference's extension binds to.
 * The reference has no C layer of its own: its pybind11 functions take
 * torch::Tensor directly (nemgemmV03.cu:343-399, v01.cu:272-317).  Every entry
 * point below therefore cites the reference interface whose work it carries out.
 *
 * All pointers are DEVICE pointers unless stated otherwise; all matrices are
 * bf16 (IEEE bfloat16, 2 bytes).  The product is accumulated in fp32 and
 * rounded once to bf16 with round-to-nearest-even, as the reference's epilogue
 * does (v01.cu:254-262, __float2bfloat16).
 *
 * Calls are asynchronous on `hip_stream` (a hipStream_t passed as void*; NULL
 * is the default stream).  No entry point synchronises the host.
 */
#ifndef NEOGEMM_H
#define NEOGEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes (0 = success, negative = failure; never a HIP error enum). */
#define NEOGEMM_OK 0
#define NEOGEMM_ERR_BAD_ARG (-1)      /* null pointer, negative size, ld too small, unknown layout */
#define NEOGEMM_ERR_WORKSPACE (-2)    /* workspace missing or smaller than neogemm_bf16_workspace_bytes */
#define NEOGEMM_ERR_UNSUPPORTED (-3)  /* the forced variant cannot run this shape / alignment */
#define NEOGEMM_ERR_LAUNCH (-4)       /* HIP refused the launch (see stderr for hipGetErrorString) */
#define NEOGEMM_ERR_SCRATCH_LIMIT (-5) /* neogemm_bf16_noalloc: the shape needs more than NEOGEMM_NOALLOC_SCRATCH_BYTES */

/* b_layout values */
#define NEOGEMM_B_KN 0 /* B is [K,N] row-major (N contiguous): the layout `C = gemm(A, B)` is quoted on */
#define NEOGEMM_B_NK 1 /* B is [N,K] row-major (K contiguous): the reference's layout, N = B.size(0)
                          (nemgemmV03.cu:346), C = A * B^T (v01.cu:232-235) */
/* c_layout values */
#define NEOGEMM_C_ROW 0 /* C(i,j) at C[i*ldc + j] */
#define NEOGEMM_C_COL 1 /* C(i,j) at C[j*ldc + i]: what the reference's epilogue writes (v01.cu:246,252) */

/* Kernel variants for neogemm_bf16_variant(); 0 lets the library choose. */
#define NEOGEMM_VARIANT_AUTO 0
#define NEOGEMM_VARIANT_GENERIC 1   /* scalar-load fallback: any shape, stride, alignment */
/* Tile variants: BM x BN macro-tile per workgroup, K in steps of 64, 16x16x32 MFMA; (r x c) = wave grid. */
#define NEOGEMM_VARIANT_RETIRED_2 2   /* was 256x256 with 8 wave64: never the fastest on any shape; calls naming it are refused */
#define NEOGEMM_VARIANT_T256x256_W4 3 /* 256x256, 4 wave64 (2x2): the default for large shapes */
#define NEOGEMM_VARIANT_T128x128_W4 4 /* 128x128, 4 wave64 (2x2) */
#define NEOGEMM_VARIANT_T256x128_W4 5 /* 256x128, 4 wave64 (2x2) */
#define NEOGEMM_VARIANT_T128x256_W4 6 /* 128x256, 4 wave64 (2x2) */
#define NEOGEMM_VARIANT_T64x128_W4 7  /* 64x128, 4 wave64 (1x4) */
#define NEOGEMM_VARIANT_RETIRED_8 8   /* was 128x128 with a 1x4 wave grid: likewise */
/* Skinny M (or, with B [N,K], skinny N): a strip of 64 columns and all of K per workgroup, no split-K (decode shapes). */
#define NEOGEMM_VARIANT_SKINNY16 9  /* M <= 16 */
#define NEOGEMM_VARIANT_SKINNY32 10 /* M <= 32 */
#define NEOGEMM_VARIANT_SKINNY64 11 /* M <= 64 */
/* 192x256, 4 wave64 (2x2): 3/4 of the 256x256 tile, for tile counts that fill the 256 CUs better (3072, 6144 ...);
   the operand that supplies the 192 rows must be K-major (A for row-major C; B [N,K] for column-major C). */
#define NEOGEMM_VARIANT_T192x256_W4 12
/* 96x128, 4 wave64 (2x2): three quarters of the 128x128 tile (1536 = 16 x 96: 192 workgroups where 128x128 gives 144);
   the 96 rows must come from a K-major operand, as for 192x256. */
#define NEOGEMM_VARIANT_T96x128_W4 13
/* 64x64, 4 wave64 (2x2), both operands K-major (B [N,K]): small problems that would leave most CUs idle otherwise. */
#define NEOGEMM_VARIANT_T64x64_W4 14
/* 256x256, 4 wave64 (2x2), K in periods of 64 with both MFMA steps of an accumulator tile back to back (less
   register-file traffic per flop: what the chip's power limit rewards); the operand that supplies the rows must be
   K-major, K a multiple of 128, no split-K. */
#define NEOGEMM_VARIANT_C256x256_W4 15
/* M <= 128 by the same kernel (five to eight row fragments of 16 per wave, shorter rings): one launch, no workspace;
   chosen for 65 to 96 rows (to 128 with B [K,N]) where one round of strips about fills the CUs and K is a few thousand deep */
#define NEOGEMM_VARIANT_SKINNY128 16
/* 65 <= M <= 128 (or, with B [N,K], 65 <= N <= 128 < M): strips of up to 64 columns and all of K per workgroup like
   the skinny variants, but eight waves per workgroup and K in stages of 128 held in rings that the waves share: four
   waves compute (a quarter of the rows each, so no partial sums meet at the end) and request B, four request A and do
   nothing else.  One launch, no workspace; chosen from 97 rows on when the wide operand is K-major and one round of
   strips about fills the CUs.  With split_k > 1 that many workgroups share a strip, each with a run of 128-deep stages
   of K, the partial sums go through the workspace (split_k * M * N floats) and the reduction kernel follows: chosen
   when there are too few strips for the CUs and K is deep (128 x 8192 x 8192: two splits), from 33 rows on: split, the
   variant also takes fewer than 65 rows.  For this variant the group_m
   argument of neogemm_bf16_variant carries the ring depths, 16 * stages of A + stages of B (0: the defaults); rings that
   do not fit the 160 KiB of LDS are refused. */
#define NEOGEMM_VARIANT_STRIP 17
#define NEOGEMM_VARIANT_COUNT 18

/*
 * C = A * op(B), bf16 in, fp32 accumulate, bf16 out.
 * Replaces the host launcher neoGemmV1(A,B,C) (nemgemmV03.cu:343-391; v1/v2: neogemm(),
 * v01.cu:272-313) together with the kernel it launches (v01.cu:189-270).  The reference call is
 * neogemm_bf16(A,B,C, M,N,K, K,K,M, NEOGEMM_B_NK, NEOGEMM_C_COL, ws, ws_bytes, stream).
 *
 *   A          [M,K] row-major, leading dimension lda >= K (elements)
 *   B          [K,N] with ldb >= N (b_layout 0) or [N,K] with ldb >= K (b_layout 1)
 *   C          [M,N] row-major with ldc >= N (c_layout 0) or column-major with ldc >= M (c_layout 1)
 *   workspace  device scratch of at least neogemm_bf16_workspace_bytes(M,N,K) bytes, or NULL when
 *              that function returns 0 for the shape.  Only split-K paths use it (fp32 partials).
 *
 * Unlike the reference (M,N,K % 64 == 0, nemgemmV03.cu:375) every M,N,K >= 0 is accepted; shapes or
 * pointers that the MFMA path cannot take (K % 8, ld % 8, 16-byte alignment) run the generic kernel.
 * M == 0 or N == 0 is a no-op; K == 0 writes zeros.
 */
int neogemm_bf16(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda,
                 int64_t ldb, int64_t ldc, int b_layout, int c_layout, void* workspace,
                 size_t workspace_bytes, void* hip_stream);

/*
 * C = alpha * A * op(B) + beta * C: the epilogue the reference's latest kernel declares
 * ("D = alpha*A*B + beta*C", neogemmv4.cu:166,266) and never reaches (its launch omits both
 * factors, neogemmv4.cu:322-323).  Arguments as for neogemm_bf16.  In fp32:
 * t = alpha * acc; if beta != 0: t = fma(beta, float(C), t); C = RNE_bf16(t).  With beta == 0 the
 * old contents of C are not read (they may be NaN); alpha == 1, beta == 0 is neogemm_bf16 bit for bit.
 * NaN factors are refused with NEOGEMM_ERR_BAD_ARG.
 */
int neogemm_bf16_scaled(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda,
                        int64_t ldb, int64_t ldc, int b_layout, int c_layout, float alpha, float beta,
                        void* workspace, size_t workspace_bytes, void* hip_stream);

/*
 * `batch` problems of one shape in one launch: problem b uses A + b*stride_a, B + b*stride_b,
 * C + b*stride_c (strides in elements; 0 for A or B shares that operand across the batch; the outputs
 * must not overlap).  Everything else as for neogemm_bf16.  The reference has no batched call — its
 * launcher takes one (A,B,C) triple (nemgemmV03.cu:343-351); this is the same launcher over a third grid
 * dimension.  1 <= batch <= 65535 (0 is a no-op); the workspace bound is
 * neogemm_bf16_batched_workspace_bytes(M,N,K,batch).
 */
int neogemm_bf16_batched(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda,
                         int64_t ldb, int64_t ldc, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                         int64_t batch, int b_layout, int c_layout, void* workspace, size_t workspace_bytes,
                         void* hip_stream);
size_t neogemm_bf16_batched_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t batch);

/*
 * neogemm_bf16 for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments and
 * result as neogemm_bf16 (bit for bit: the same kernels run), minus the workspace: split-K partials go to
 * an array of NEOGEMM_NOALLOC_SCRATCH_BYTES that the library's code object holds on each GPU it runs on,
 * until the process ends.  The call makes no hipMalloc/hipFree and no other allocating call; the first call on a
 * device (it resolves the array's address, which loads the code object) and the first launch of a kernel instance (it
 * raises that kernel's dynamic-LDS limit) make host-side set-up calls that a capturing stream does not allow: warm the
 * shapes up once outside the capture, then capture.  A shape whose
 * neogemm_bf16_workspace_bytes(M,N,K) exceeds NEOGEMM_NOALLOC_SCRATCH_BYTES is refused with
 * NEOGEMM_ERR_SCRATCH_LIMIT and nothing is launched.  All calls on one GPU share that GPU's array: calls on
 * one stream are ordered and safe (every partial is rewritten before it is read, nothing has to start at
 * zero); calls that overlap in time on one GPU (different streams or threads) race on it.
 */
#define NEOGEMM_NOALLOC_SCRATCH_BYTES (32u * 1024u * 1024u)
int neogemm_bf16_noalloc(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda,
                         int64_t ldb, int64_t ldc, int b_layout, int c_layout, void* hip_stream);

/*
 * Upper bound of the scratch neogemm_bf16 may use for (M,N,K), in bytes, whatever the layouts of B and C
 * (the bound is the largest need over the four combinations).  Host-only arithmetic.
 * Counterpart of the per-call device allocations the reference's launcher makes for its TMA
 * descriptors (v01.cu:153-160, nemgemmV03.cu:60-68): here the caller owns the scratch.
 */
size_t neogemm_bf16_workspace_bytes(int64_t M, int64_t N, int64_t K);

/*
 * Same as neogemm_bf16 but with the kernel variant, the split-K factor (>= 1; 0 = choose) and the
 * tile-order group height (0 = default) forced.  The reference fixes these at compile time
 * (template arguments at v01.cu:304-311); this entry point exists for tuning, tests and the bench.
 * Returns NEOGEMM_ERR_UNSUPPORTED if the variant cannot run the shape.  With split_k > 1 the
 * workspace must hold split_k * M * N floats.
 */
int neogemm_bf16_variant(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K,
                         int64_t lda, int64_t ldb, int64_t ldc, int b_layout, int c_layout,
                         void* workspace, size_t workspace_bytes, void* hip_stream, int variant,
                         int split_k, int group_m);

/*
 * What neogemm_bf16 would pick for this call: writes the variant id and split-K factor.  Host only.
 * `aligned` is nonzero when pointers and leading dimensions satisfy the MFMA path (16-byte / 8-element).
 * The choice comes from a cost model over the tile variants; if the environment variable
 * NEOGEMM_PLAN_TABLE names a JSON file of tuned choices (an array of objects with the integer fields
 * "M","N","K","b_layout","c_layout","variant","split_k"; the layouts default to 0; gemm_amd/tune.py writes one), an
 * entry for the exact shape and layouts wins.  The file is read once per process.
 */
int neogemm_bf16_plan(int64_t M, int64_t N, int64_t K, int b_layout, int c_layout, int aligned,
                      int* variant, int* split_k);

/*
 * Instrumented run of NEOGEMM_VARIANT_T256x256_W4 (row-major C, no split-K): besides computing C, every
 * wave writes four shader-clock cycle counts {whole kernel, waiting for its own global->LDS loads, waiting
 * at the workgroup barrier, epilogue} to phase_cycles[(workgroup * 4 + wave) * 4 + i], workgroup = launch
 * order; other variants are refused with NEOGEMM_ERR_UNSUPPORTED.  This is the per-phase cycle buffer of the
 * reference's harness (the `DB` array: cublass/matmul.cu:99-106 allocation, :149-165 decode), which
 * no kernel in the reference fills in.  phase_cycles is device memory of at least
 * neogemm_bf16_profile_bytes(M, N, variant) bytes.  The timers cost a few percent; never time with it.
 */
int neogemm_bf16_profile(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda,
                         int64_t ldb, int64_t ldc, int b_layout, void* hip_stream, int variant, int group_m,
                         unsigned long long* phase_cycles, size_t phase_cycles_bytes);
size_t neogemm_bf16_profile_bytes(int64_t M, int64_t N, int variant);

/* Text for a status code; replaces the std::cerr print at nemgemmV03.cu:387-390. Never NULL. */
const char* neogemm_strerror(int status);

/* Library version string, e.g. "neogemm 0.2 gfx950". */
const char* neogemm_version(void);

#ifdef __cplusplus
}
#endif
#endif /* NEOGEMM_H */
