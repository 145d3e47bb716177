/*
 * cmk.h - C ABI of libcmk.so, the gfx950 (MI355X) fused batched-matmul library.
 *
 * Every entry point enqueues work on the caller's HIP stream and returns
 * without synchronising.  All data pointers are device pointers owned by the
 * caller; the library never allocates or frees device memory.  Scratch space,
 * where an operation needs it, is a caller-provided workspace whose size is
 * reported by cmk_workspace_bytes().
 *
 * Matrices are fp32.  An operand is described by a pointer, a leading
 * dimension `ld` (in elements), a batch stride (in elements) and a transpose
 * flag:
 *     transA == 0 : A[b][m][k] lives at  A + b*strideA + m*lda + k   ("n")
 *     transA == 1 : A[b][m][k] lives at  A + b*strideA + k*lda + m   ("t")
 *     transB == 0 : B[b][k][n] lives at  B + b*strideB + k*ldb + n   ("n")
 *     transB == 1 : B[b][k][n] lives at  B + b*strideB + n*ldb + k   ("t")
 * These are the four layouts the reference infers from tensor strides
 * (reference bmm.py:56-66) and compiles as separate kernels
 * (reference kernels/bmm.cu:1,93,184,276).
 *
 * Return value: 0 on success, otherwise a negative CMK_ERR_* code or a
 * positive hipError_t; cmk_last_error() then holds a message for the calling
 * thread.
 */
#ifndef CMK_H_
#define CMK_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CMK_ABI_VERSION 1

#define CMK_OK                 0
#define CMK_ERR_INVALID_ARG   -1   /* bad shape / dim / k / null pointer          */
#define CMK_ERR_UNSUPPORTED   -2   /* valid request that this build does not do   */
#define CMK_ERR_WORKSPACE     -3   /* workspace missing or too small              */

/* operation ids for cmk_workspace_bytes() */
#define CMK_OP_BMM      0
#define CMK_OP_MBMM     1
#define CMK_OP_MIN_BMM  2
#define CMK_OP_TOPK_BMM 3
#define CMK_OP_TOPK_1D  4
#define CMK_OP_MIN_BMM_L2 5   /* cmk_min_bmm_f32 with CMK_DIST_L2 on the matrix pipe */

/* accumulate functions of min_bmm / topk_bmm (reference kernels/bmm_helpers.cu:20-60;
 * selected by the `distance` constructor argument, minbmm.py:12-19, topkbmm.py:15-22).
 * INNER runs on the matrix pipe; L2 and L1 have no matrix form and run on the
 * vector unit, in the reference's order of operations (d = a - b, then
 * fmaf(d, d, c) or c + fabsf(d), k ascending), a few times slower.
 * cmk_min_bmm_f32 has a second route for L2 that gives the same bits from the
 * matrix pipe (see there).  cmk_topk_bmm_f32 with L2 / L1 runs about 40 % faster
 * when the operand of the reduced axis is stored with that axis contiguous (A
 * with transA = 1 for dim 1, B with transB = 0 for dim 2); the Python wrapper
 * copies a large operand into that form. */
#define CMK_DIST_INNER 0   /* c += a*b        ("madd")       */
#define CMK_DIST_L2    1   /* c += (a-b)^2    ("squared_l2") */
#define CMK_DIST_L1    2   /* c += |a-b|      ("l1")         */

/* Operand description shared by all GEMM-family entry points. */
typedef struct cmk_gemm_desc {
  int L, M, N, K;            /* batch, rows of C, cols of C, contraction length */
  int transA, transB;        /* 0 = "n", 1 = "t" (see above)                    */
  long long lda, ldb;        /* leading dimensions, elements                    */
  long long strideA, strideB;/* batch strides, elements                         */
} cmk_gemm_desc;

/*
 * C[b][m][n] = sum_k A[b][m][k] * B[b][k][n]; C is dense row-major
 * [L][M][N] and every element is written (no pre-zeroing needed).
 * Replaces the launch of bmm_{nn,nt,tn,tt}
 * (reference bmm.py:115-125, kernels/bmm.cu:184-274).
 */
int cmk_bmm_f32(const float* A, const float* B, float* C,
                const cmk_gemm_desc* d, void* stream);

/*
 * The same product for callers that can lend a workspace of
 * cmk_workspace_bytes(CMK_OP_BMM, L, M, N, K, 0) bytes.  When C has too few
 * tiles to occupy the GPU and the contraction is long (say 512x512 with
 * K = 4096), the contraction is cut into ranges whose partial products go to
 * the workspace and are summed in ascending order of k by a second kernel:
 * results are reproducible from run to run, and differ from cmk_bmm_f32's by
 * fp32 rounding only.  With a workspace size of 0 reported, or given, for
 * shapes that need none, this is cmk_bmm_f32.  The reference walks the whole
 * contraction in one block per tile (kernels/bmm.cu:184-274) and has no
 * counterpart; the Python class calls this entry point (reference
 * bmm.py:68-129 allocates its result through PyTorch at every call, as this
 * workspace is).
 */
int cmk_bmm_ws_f32(const float* A, const float* B, float* C,
                   const cmk_gemm_desc* d,
                   void* workspace, size_t workspace_bytes, void* stream);

/*
 * Masked product: C = (A@B) * element_mask where the 128x128 tile's
 * block_mask and the 8x8 micro-tile's thread_mask are both non-zero, else 0.
 * Tiles whose block_mask is 0 are not computed (only zeros are written).
 * Masks are uint8: block_mask [Lm][ceil(M/128)][ceil(N/128)], thread_mask
 * [Lm][ceil(M/8)][ceil(N/8)], element_mask [Lm][M][N] with Lm = 1 when
 * share_mask != 0 and Lm = L otherwise.  All four operand layouts are
 * accepted (the reference implements "nn" only; its mbmm_tn / mbmm_nt /
 * mbmm_tt are empty).  The element mask is a 0/1 multiplier, as in the
 * reference (kernels/mbmm.cu:127-128): a non-finite product under a zero
 * element-mask byte gives NaN, not 0; block- and thread-masked positions are
 * exact zeros whatever the operands hold.  Replaces the launch of mbmm_nn
 * (reference mbmm.py:84-97, kernels/mbmm.cu:208-374) and stands in for
 * mbmm_tn, mbmm_nt, mbmm_tt (kernels/mbmm.cu:184-206, 376-385).
 */
int cmk_mbmm_f32(const float* A, const float* B, float* C,
                 const uint8_t* block_mask, const uint8_t* thread_mask,
                 const uint8_t* element_mask, int share_mask,
                 const cmk_gemm_desc* d, void* stream);

/*
 * Derives mbmm's coarse masks from an element mask [Lm][M][N] (uint8, any
 * non-zero byte = kept; a torch.bool tensor's storage qualifies):
 * thread_mask[Lm][ceil(M/8)][ceil(N/8)] = kept elements per 8x8 micro-tile
 * (0..64), block_mask[Lm][ceil(M/128)][ceil(N/128)] = 1 where the 128x128 tile
 * keeps any.  Elements beyond M or N count as dropped.  The reference has no
 * kernel for this: its callers derive the masks with tensor reductions
 * (reference colab/test_mbmm.ipynb:1295-1313), which this entry point replaces.
 */
int cmk_derive_masks_u8(const uint8_t* element_mask, uint8_t* block_mask,
                        uint8_t* thread_mask, int Lm, int M, int N, void* stream);

/*
 * Fused min/argmin of C = A@B (or of the accumulated distance CMK_DIST_*
 * between the rows of A and the columns of B) along `dim` of C[L][M][N] (1 =
 * over m, output [L][N]; 2 = over n, output [L][M]) without storing C.  `values` is fp32,
 * `indices` int64; every output element is written; exact ties resolve to
 * the lowest index.  Replaces the launch of min_bmm_{nn,nt,tn,tt}
 * (reference minbmm.py:132-143, kernels/minbmm.cu:347-440).
 *
 * `workspace` must hold cmk_workspace_bytes(CMK_OP_MIN_BMM, ...) bytes (0 for
 * many shapes).  With CMK_DIST_L2 and a 256-byte aligned workspace of at
 * least cmk_workspace_bytes(CMK_OP_MIN_BMM_L2, ...) bytes (non-zero whenever
 * K > 0) the call takes the matrix pipe instead of the vector unit: the pipe
 * computes |x|^2 - 2 x.y for all pairs, the kernel keeps per output the two
 * smallest of these and a bound on the rest, and the exact fmaf sum is
 * evaluated only for the candidates that the rounding error cannot rule out;
 * outputs that stay undecided (ties among duplicated points, heavy
 * cancellation, non-finite input) are recomputed exactly, a few of them one by
 * one, many of them by the vector-unit kernel over the whole problem.  Values
 * and indices are bit-equal to the vector route's in every case; on random
 * data the call takes about a third of the vector route's time.
 */
int cmk_min_bmm_f32(const float* A, const float* B,
                    float* values, long long* indices,
                    const cmk_gemm_desc* d, int dim, int distance,
                    void* workspace, size_t workspace_bytes, void* stream);

/*
 * cmk_min_bmm_f32 for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
 * same arguments without the workspace, same results.  The partial results of
 * a split reduction go to a static device array of CMK_STATIC_SCRATCH_BYTES
 * that each GPU holds from library load until the process ends; the call
 * allocates and frees nothing.  Problems whose cmk_workspace_bytes() exceeds
 * that size are refused with CMK_ERR_WORKSPACE.  All calls on one GPU share
 * the array: calls that may overlap on one GPU (different streams) race and
 * must be serialised by the caller.  The first call on a device looks up the
 * array's address, which is not a stream operation: make one call outside any
 * graph capture before capturing it.  No counterpart in the reference, which
 * allocates through PyTorch at every call (minbmm.py:116-122).
 */
#define CMK_STATIC_SCRATCH_BYTES (4u << 20)
int cmk_min_bmm_f32_static(const float* A, const float* B,
                           float* values, long long* indices,
                           const cmk_gemm_desc* d, int dim, int distance,
                           void* stream);

/*
 * Fused top-k (largest, sorted descending, 0 < k <= 128) of C = A@B (or of
 * the accumulated distance CMK_DIST_*; still the largest k) along `dim` of
 * C[L][M][N]: dim == 2 gives [L][M][k], dim == 1 gives [L][N][k].
 * `values` fp32 and `indices` int64 are dense with row pitch k.  When fewer
 * than k candidates exist the trailing slots hold -inf / -1.  Replaces the
 * launch of topk_bmm_{nn,nt,tn,tt}
 * (reference topkbmm.py:137-149, kernels/topkbmm.cu:499-594).
 */
int cmk_topk_bmm_f32(const float* A, const float* B,
                     float* values, long long* indices,
                     const cmk_gemm_desc* d, int dim, int k, int distance,
                     void* workspace, size_t workspace_bytes, void* stream);

/*
 * Top-k (largest, sorted descending, 0 < k <= 128) of a 1-D fp32 array of
 * length n.  Replaces the launch of bitonic_sort
 * (reference kernels/bitonic_sort.cu:182-216).
 */
int cmk_topk_1d_f32(const float* arr, long long n,
                    float* values, long long* indices, int k,
                    void* workspace, size_t workspace_bytes, void* stream);

/* Bytes of device workspace an operation needs (0 = none).  For
 * CMK_OP_TOPK_1D pass the array length in M (L = 1).  The work is cut for the
 * GPU that is current when this is called (its compute-unit count): call it
 * with the device current on which the operation will be launched, or the
 * launch may refuse the workspace as too small (CMK_ERR_WORKSPACE). */
size_t cmk_workspace_bytes(int op, int L, int M, int N, int K, int dim);

/* Message describing the last failure on the calling thread ("" if none). */
const char* cmk_last_error(void);

int cmk_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* CMK_H_ */
