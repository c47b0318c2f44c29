/* qmm_hip.h -- C ABI of libqmm_hip.so: quantized matmul for MI355X (gfx950).
 *
 * The library serves the fused op that the reference's quantized-matmul
 * recognizer emits.  Every entry point takes raw DEVICE pointers and explicit
 * shapes; the caller owns every buffer (including the optional workspace); no
 * entry point allocates, frees or synchronizes; work is enqueued on the given
 * HIP stream (a hipStream_t passed as void*, NULL = the default stream).
 *
 * Return value: 0 on success, else one of the QMM_ERR_* codes; the message of
 * the calling thread's last failure is available from qmm_last_error().
 * A non-zero status means nothing was launched, so a caller can run the
 * literal (unfused) chain instead, which is what the reference's handler does
 * on any exception (reference src/metaljax/qmm.py:2348-2355).
 *
 * Layouts (identical to what the reference hands mx.quantized_matmul,
 * reference src/metaljax/qmm.py:2469-2501 and :206-282):
 *   x        [batch, M, K] row-major, dtype x_dtype (bf16, or float16 / float32:
 *            those are split, exactly, into two / three bf16 terms that are
 *            multiplied like bf16 activations and added in float32 -- the
 *            workspace queries take x_dtype for that)
 *   w        affine: uint32 [batch, N, K*bits/32]; element i of a row at bits
 *            [i*bits, (i+1)*bits) of the row's little-endian stream.
 *            mxfp4:  the same stream of 4-bit E2M1 codes (uint32 [N, K/8] ==
 *            uint8 [N, K/2], low nibble = even element)
 *   scales   affine: [batch, N, K/group_size] in table_dtype;
 *            mxfp4:  uint8 E8M0 [batch, N, K/32]
 *   biases   affine: like scales; mxfp4: NULL
 *   y        [batch, M, N] row-major, dtype y_dtype
 * Semantics: y = x . dequant(w)^T with float32 accumulation, where
 *   affine  w = scales*q + biases          (one fused multiply-add)
 *   mxfp4   w = E2M1[code] * 2^(scale-127)
 */
#ifndef QMM_HIP_H_
#define QMM_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  QMM_OK = 0,
  QMM_ERR_BAD_ARGUMENT = 1,  /* null pointer, negative size, misaligned pointer */
  QMM_ERR_BAD_SHAPE = 2,     /* K % group_size, K % 32, ... */
  QMM_ERR_UNSUPPORTED = 3,   /* a dtype / bits / group_size combination not built */
  QMM_ERR_WORKSPACE = 4,     /* workspace missing or too small */
  QMM_ERR_HIP = 5            /* a HIP runtime call failed */
};

enum { QMM_F32 = 0, QMM_BF16 = 1, QMM_F16 = 2 };
enum { QMM_MODE_AFFINE = 0, QMM_MODE_MXFP4 = 1 };

/* Which kernel family a shape is routed to (returned by qmm_plan). */
enum { QMM_KERNEL_GEMV = 1, QMM_KERNEL_GEMM = 2, QMM_KERNEL_MXFP4_MFMA = 3 };

int qmm_abi_version(void);
const char* qmm_last_error(void);

/* Replaces mx.quantized_matmul(x, w, scales, biases, transpose=True,
 * group_size, bits, mode) -- reference src/metaljax/qmm.py:2491.
 * `batch` > 1 multiplies batch independent [M,K] x [N,K] pairs (the batched
 * dot of reference src/metaljax/qmm.py:65-69).  `workspace` may be NULL when
 * qmm_workspace_bytes() returns 0 for the same arguments. */
int qmm_quantized_matmul(const void* x, int x_dtype, const void* w, const void* scales,
                         const void* biases, int table_dtype, void* y, int y_dtype,
                         int64_t batch, int64_t M, int64_t N, int64_t K, int group_size,
                         int bits, int mode, void* workspace, size_t workspace_bytes,
                         void* stream);

/* Scratch bytes qmm_quantized_matmul / qmm_grouped_qmm need for these
 * arguments (M = total rows for the grouped form). */
size_t qmm_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K, int group_size,
                           int bits, int mode, int x_dtype);

/* Scratch bytes qmm_gather_qmm wants for P pairs over E experts of [N, K]
 * weights (0 below four pairs, which run as independent decode products): the
 * expert sort's arrays, plus the segment list of the grouped decode (up to
 * 16 pairs an expert on average: one decode product per expert and sixteen
 * pairs) or the re-laid activation copy of the prefill kernel (more pairs).
 * With less the call still runs, on a slower kernel (bf16 activations; float16
 * and float32 activations need the whole of it). */
size_t qmm_gather_workspace_bytes(int64_t P, int64_t E, int64_t N, int64_t K, int x_dtype);

/* The kernel family and launch geometry the dispatcher would choose. */
int qmm_plan(int64_t M, int64_t N, int64_t K, int group_size, int bits, int mode,
             int* kernel, int* grid, int* block);

/* Replaces mx.gather_qmm(x, w, scales, biases, lhs_idx, rhs_idx, transpose=True, ...)
 * with one row per pair -- reference src/metaljax/moe.py:1320:
 *   y[p, :] = x[lhs_idx[p], :] . dequant(w[rhs_idx[p]])^T     p in [0, P)
 * x [T, K]; w/scales/biases carry a leading expert axis [E, N, ...];
 * lhs_idx, rhs_idx int32 [P] on the device, in any order; y [P, N].
 * lhs_idx may be NULL (identity). */
int qmm_gather_qmm(const void* x, int x_dtype, const void* w, const void* scales,
                   const void* biases, int table_dtype, void* y, int y_dtype,
                   const int32_t* lhs_idx, const int32_t* rhs_idx, int64_t P, int64_t T,
                   int64_t E, int64_t N, int64_t K, int group_size, int bits, int mode,
                   void* workspace, size_t workspace_bytes, void* stream);

/* qmm_gather_qmm for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * No counterpart in the reference.  Same arguments and results as
 * qmm_gather_qmm without the workspace pair: the expert sort's arrays, the
 * segment list and the re-laid activation copy live in a device array of
 * QMM_STATIC_SCRATCH_BYTES that is part of the library's code object (every
 * GPU the library runs on holds one until the process ends).  A call whose
 * qmm_gather_workspace_bytes(P, E, N, K, x_dtype) exceeds that size fails with
 * QMM_ERR_WORKSPACE and launches nothing.  The call allocates and frees
 * nothing.  Every call on a GPU uses that GPU's one array: calls that overlap
 * on one GPU (different streams, or threads) race; calls in stream order do
 * not, and each call initialises what it reads.  The first call on a device
 * looks up the array's address and sets kernel attributes: make it outside a
 * stream capture (any call, of any size); later calls only launch kernels. */
#define QMM_STATIC_SCRATCH_BYTES (16u << 20)
int qmm_gather_qmm_static(const void* x, int x_dtype, const void* w, const void* scales,
                          const void* biases, int table_dtype, void* y, int y_dtype,
                          const int32_t* lhs_idx, const int32_t* rhs_idx, int64_t P, int64_t T,
                          int64_t E, int64_t N, int64_t K, int group_size, int bits, int mode,
                          void* stream);

/* The sorted-rows form of the same product (rows of x already grouped by
 * expert): rows [row_offsets[e], row_offsets[e+1]) use expert e's weight.
 * row_offsets int32 [E+1] on the device, non-decreasing, row_offsets[0] = 0,
 * row_offsets[E] = R.  Empty experts are legal.  No host synchronization.
 * Serves the per-expert product of reference src/metaljax/moe.py:1283-1340. */
int qmm_grouped_qmm(const void* x, int x_dtype, const void* w, const void* scales,
                    const void* biases, int table_dtype, void* y, int y_dtype,
                    const int32_t* row_offsets, int64_t R, int64_t E, int64_t N, int64_t K,
                    int group_size, int bits, int mode, void* workspace,
                    size_t workspace_bytes, void* stream);

/* Replaces mx.dequantize(w, scales, biases, group_size, bits[, mode]) --
 * used by the reference's layout tests (tests/test_qmm.py:121;
 * tests/test_qmm_mxfp4.py:192).  rows = product of the leading dims; out
 * [rows, K] in out_dtype.  Bit-exact: float32 out is fma(scale, q, bias);
 * bf16 / f16 out is one round-to-nearest-even of that. */
int qmm_dequantize(const void* w, const void* scales, const void* biases, int table_dtype,
                   void* out, int out_dtype, int64_t rows, int64_t K, int group_size,
                   int bits, int mode, void* stream);

/* uint32 words [rows, K*bits/32] -> uint8 codes [rows, K]; inverse of the
 * reference's pack_codes (src/metaljax/qmm.py:206-232).  bits in {2, 4, 8}. */
int qmm_unpack_codes(const void* w, void* codes, int64_t rows, int64_t K, int bits,
                     void* stream);

/* uint8 codes [rows, K] -> uint32 words [rows, K*bits/32], masking each code
 * to `bits` -- reference pack_codes, src/metaljax/qmm.py:206-232. */
int qmm_pack_codes(const void* codes, void* w, int64_t rows, int64_t K, int bits,
                   void* stream);

/* out[r, j] = x[r, perm[j]]: the activation gather applied when a weight was
 * packed with a permuted contraction axis (mx.take(x, perm, -1), reference
 * src/metaljax/qmm.py:2486-2490).  perm int32 [K] on the device. */
int qmm_take_k(const void* x, int x_dtype, const int32_t* perm, void* out, int64_t rows,
               int64_t K, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* QMM_HIP_H_ */
