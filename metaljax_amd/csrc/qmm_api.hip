// C ABI of libqmm_hip.so: argument validation and regime dispatch.
// See include/qmm_hip.h for the contract of every entry point.
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <mutex>

#include "qmm_common.hpp"

namespace qmm {

void gemv_dispatch(const void* x, const void* w, const void* s, const void* b, int tab, void* y,
                   int y_dtype, int64_t batch, int64_t M, int64_t N, int64_t K, int gs, int bits,
                   int mode, const int32_t* lhs_idx, const int32_t* rhs_idx, int64_t n_experts,
                   int64_t n_xrows, hipStream_t st);
void gemv_geometry(int64_t M, int64_t N, int64_t K, int* t, int* waves);
void skinny_geometry(int64_t N, int64_t K, int bits, int* waves, int* rows_per_wg);
bool skinny2_plan(int64_t M, int64_t N, int64_t K, int bits, int* rows_per_wg);
bool skinny2_mx_plan(int64_t N, int64_t K, int* rows_per_wg);
bool skinny2_grouped_supported(int64_t N, int64_t K, int gs, int bits, int mode, int tab,
                               const void* s, const void* b, int64_t E);
void skinny2_grouped_dispatch(const void* x, const void* w, const void* s, const void* b, void* y,
                              int y_dtype, const int32_t* segments, const int32_t* src_row,
                              const int32_t* out_row, int64_t P, int64_t T, int64_t E, int64_t N,
                              int64_t K, int gs, int bits, int mode, int tab, hipStream_t st);
int64_t skinny2_max_segments(int64_t P, int64_t E);
void gemm_dispatch(const void* x, const void* w, const void* s, const void* b, int tab, void* y,
                   int y_dtype, const int32_t* row_offsets, const int32_t* lhs_idx,
                   const int32_t* out_idx, int64_t R, int64_t x_rows, int64_t E, int64_t N,
                   int64_t K, int gs, int bits, int mode, hipStream_t st);
int64_t gemm_row_tile(int64_t R, int64_t E);
bool gemv_runs_general(int64_t N, int64_t K, int gs, int bits, int mode, int tab, const void* s, const void* b);
void gemv_grouped_dispatch(const void* x, const void* w, const void* s, const void* b, int tab, void* y,
                           int y_dtype, const int32_t* segments, const int32_t* src_row,
                           const int32_t* out_row, int64_t max_segments, int64_t x_rows, int64_t N,
                           int64_t K, int gs, int bits, int mode, hipStream_t st);
bool gemm2_supported(int64_t R, int64_t N, int64_t K);
size_t gemm2_workspace_bytes(int64_t R, int64_t K);
void gemm2_dispatch(const void* x, const void* w, const void* s, const void* b, int tab, void* y,
                    int y_dtype, const int32_t* row_offsets, const int32_t* lhs_idx,
                    const int32_t* out_idx, int64_t R, int64_t x_rows, int64_t E, int64_t N,
                    int64_t K, int gs, int bits, int mode, int row_tile, void* workspace,
                    hipStream_t st);
bool mxfp4_mfma_supported(int64_t R, int64_t N, int64_t K);
size_t mxfp4_workspace_bytes(int64_t R, int64_t K);
void mxfp4_geometry(int64_t R, int64_t N, int64_t K, int* grid, int* block);
void mxfp4_mfma_dispatch(const void* x, const void* w, const void* s, void* y, int y_dtype,
                         const int32_t* row_offsets, const int32_t* lhs_idx,
                         const int32_t* out_idx, int64_t R, int64_t x_rows, int64_t E, int64_t N,
                         int64_t K, void* workspace, hipStream_t st);
void unpack_dispatch(const void* w, void* codes, int64_t rows, int64_t K, int bits, hipStream_t st);
void pack_dispatch(const void* codes, void* w, int64_t rows, int64_t K, int bits, hipStream_t st);
void dequant_dispatch(const void* w, const void* s, const void* b, int tab, void* out,
                      int out_dtype, int64_t rows, int64_t K, int gs, int bits, int mode,
                      hipStream_t st);
void take_dispatch(const void* x, int x_dtype, const int32_t* perm, void* out, int64_t rows,
                   int64_t K, hipStream_t st);
void split_terms_dispatch(const void* x, int x_dtype, void* out, int64_t batch, int64_t rows,
                          int64_t K, const int32_t* src_row, int64_t x_rows, hipStream_t st);
void sum_terms_dispatch(const void* part, int terms, void* y, int y_dtype, int64_t batch,
                        int64_t rows, int64_t N, const int32_t* offsets,
                        const int32_t* expert_of_row, int64_t E, hipStream_t st);

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = setup_error();                   // a failed launch set-up (nothing was launched)
  setup_error() = hipSuccess;
  if (e == hipSuccess) e = hipGetLastError();
  if (e != hipSuccess) return fail(QMM_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
  return QMM_OK;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Largest M served by the decode kernel.
constexpr int64_t kGemvMaxM = 16;
// Pairs at or below which the gather form runs one decode launch per pair
// instead of sorting rows by expert.
constexpr int64_t kGatherGemvMaxPairs = 64;
// From this many pairs on (and up to kGatherGemvMaxPairs) the pairs are sorted
// by expert and every expert's weight is streamed once (grouped decode); below
// it the sort's launch costs more than a shared expert saves.
constexpr int64_t kGroupedDecodeMinPairs = 4;

int check_quant(int64_t N, int64_t K, int gs, int bits, int mode, int tab, const void* w,
                const void* s, const void* b) {
  if (!w || !s) return fail(QMM_ERR_BAD_ARGUMENT, "null weight or scale pointer");
  if (N < 0 || K < 0) return fail(QMM_ERR_BAD_ARGUMENT, "negative shape");
  if (mode == QMM_MODE_MXFP4) {
    if (bits != 4) return fail(QMM_ERR_UNSUPPORTED, "mxfp4 requires bits=4, got %d", bits);
    if (gs != 32) return fail(QMM_ERR_UNSUPPORTED, "mxfp4 requires group_size=32, got %d", gs);
    if (b) return fail(QMM_ERR_BAD_ARGUMENT, "mxfp4 takes no biases");
  } else if (mode == QMM_MODE_AFFINE) {
    if (bits != 4 && bits != 8) return fail(QMM_ERR_UNSUPPORTED, "affine bits=%d (4 or 8 built)", bits);
    if (gs != 32 && gs != 64 && gs != 128)
      return fail(QMM_ERR_UNSUPPORTED, "group_size=%d (32, 64 or 128)", gs);
    if (!b) return fail(QMM_ERR_BAD_ARGUMENT, "affine mode needs biases");
    if (tab != QMM_F32 && tab != QMM_BF16 && tab != QMM_F16)
      return fail(QMM_ERR_UNSUPPORTED, "table dtype %d", tab);
  } else {
    return fail(QMM_ERR_UNSUPPORTED, "mode %d", mode);
  }
  if (K % 32) return fail(QMM_ERR_BAD_SHAPE, "K=%lld is not a multiple of 32", (long long)K);
  if (K % gs) return fail(QMM_ERR_BAD_SHAPE, "K=%lld is not a multiple of group_size=%d", (long long)K, gs);
  if (!aligned16(w)) return fail(QMM_ERR_BAD_ARGUMENT, "weight pointer not 16-byte aligned");
  return QMM_OK;
}

int check_io(const void* x, int x_dtype, void* y, int y_dtype) {
  if (!x || !y) return fail(QMM_ERR_BAD_ARGUMENT, "null activation or output pointer");
  if (x_dtype != QMM_BF16 && x_dtype != QMM_F16 && x_dtype != QMM_F32)
    return fail(QMM_ERR_UNSUPPORTED, "activation dtype %d", x_dtype);
  if (y_dtype != QMM_BF16 && y_dtype != QMM_F32 && y_dtype != QMM_F16)
    return fail(QMM_ERR_UNSUPPORTED, "output dtype %d", y_dtype);
  if (!aligned16(x)) return fail(QMM_ERR_BAD_ARGUMENT, "activation pointer not 16-byte aligned");
  return QMM_OK;
}

// ---- routing for the gather form: pairs -> rows sorted by expert -----------
// workspace layout (int32): row_offsets[E+1] | cursor[E] | src_row[P] | out_row[P] | segments
// segments (grouped decode only): [0] = count, then (expert, first sorted
// position, rows <= 16) per chunk of sixteen rows of every expert that has rows
__global__ __launch_bounds__(1024) void route_kernel(const int32_t* __restrict__ lhs_idx,
                                                     const int32_t* __restrict__ rhs_idx, int P,
                                                     int E, int32_t* __restrict__ row_offsets,
                                                     int32_t* __restrict__ cursor,
                                                     int32_t* __restrict__ src_row,
                                                     int32_t* __restrict__ out_row,
                                                     int32_t* __restrict__ segments) {
  for (int e = threadIdx.x; e <= E; e += blockDim.x) {
    row_offsets[e] = 0;
    if (e < E) cursor[e] = 0;
  }
  // slots that no valid pair lands in (pairs naming an expert outside [0, E)) gather nothing
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    src_row[p] = -1;
    out_row[p] = -1;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = rhs_idx[p];
    if (e >= 0 && e < E) atomicAdd(&cursor[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      const int c = cursor[e];
      row_offsets[e] = run;
      cursor[e] = run;
      run += c;
    }
    row_offsets[E] = run;
    if (segments) {
      int n = 0;
      for (int e = 0; e < E; ++e) {
        const int lo = row_offsets[e], cnt = row_offsets[e + 1] - lo;
        for (int c = 0; c * 16 < cnt; ++c) {
          segments[1 + 3 * n] = e;
          segments[2 + 3 * n] = lo + 16 * c;
          segments[3 + 3 * n] = cnt - 16 * c < 16 ? cnt - 16 * c : 16;
          ++n;
        }
      }
      segments[0] = n;
    }
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = rhs_idx[p];
    if (e < 0 || e >= E) continue;
    const int pos = atomicAdd(&cursor[e], 1);
    // (the indices are read twice, to count and to place: were the caller to change them meanwhile, a
    // slot past the expert's counted range would run into the next array -- such a pair is dropped)
    if (pos >= row_offsets[e + 1]) continue;
    src_row[pos] = lhs_idx ? lhs_idx[p] : p;
    out_row[pos] = p;
  }
}

size_t route_bytes(int64_t P, int64_t E) {     // a multiple of 256: what follows stays aligned
  return ((size_t)(2 * E + 1 + 2 * P) * sizeof(int32_t) + 255) / 256 * 256;
}

// the sort's arrays plus the segment list of the grouped decode
size_t route_bytes_segments(int64_t P, int64_t E) {
  return ((size_t)(2 * E + 1 + 2 * P + 1 + 3 * skinny2_max_segments(P, E)) * sizeof(int32_t) + 255) / 256 * 256;
}

// Pairs up to which the grouped decode (one decode product per expert and
// sixteen pairs) beats the grouped prefill kernel: measured on 8 experts of
// 14336 x 4096: 128 pairs 151 against 235 us, 256 pairs 239 against 244 us, 512
// pairs 436 against 237 us.
bool grouped_decode_pairs(int64_t P, int64_t E) {
  static const int64_t gd_max = experiment_env("QMM_GD_MAX") ? atoll(experiment_env("QMM_GD_MAX")) : 0;
  if (P < kGroupedDecodeMinPairs) return false;
  return gd_max ? P <= gd_max : P <= 16 * E && P <= 4096;
}

// ---- float16 / float32 activations ---------------------------------------------
// The kernels multiply bf16 operands.  Wider activations are split, exactly,
// into bf16 terms (float16: two, float32: three), every term is multiplied
// like a bf16 activation (products exact, float32 accumulate) and the terms'
// float32 results are added, largest first, before the one rounding to the
// output type.  In the dense decode case the terms ride as extra rows of the
// same launch (terms x M <= 16: the weight is still streamed once).
int act_terms(int x_dtype) { return x_dtype == QMM_F32 ? 3 : x_dtype == QMM_F16 ? 2 : 1; }

size_t align256(size_t n) { return (n + 255) / 256 * 256; }

// Scratch of the bf16 dense / grouped product over `rows` rows.  `exact`: the
// activation terms must stay exact, so MXFP4 weights take the bf16 kernels
// (their FP6 activation terms would round).
size_t dense_scratch(int64_t rows, int64_t N, int64_t K, int mode, bool exact) {
  if (mode == QMM_MODE_MXFP4 && !exact && rows > kGemvMaxM && mxfp4_mfma_supported(rows, N, K))
    return mxfp4_workspace_bytes(rows, K);
  if (rows > kGemvMaxM && gemm2_supported(rows, N, K)) return gemm2_workspace_bytes(rows, K);
  return 0;
}

size_t gather_scratch(int64_t P, int64_t E, int64_t N, int64_t K, bool exact) {
  if (P < kGroupedDecodeMinPairs) return 0;
  const size_t decode = grouped_decode_pairs(P, E) ? route_bytes_segments(P, E) : 0;
  if (P <= kGatherGemvMaxPairs) return decode;    // the expert sort of the grouped decode
  // the expert sort's arrays, then (when the register-operand kernel serves
  // the shape) the re-laid copy of the gathered activation rows
  size_t relaid = gemm2_supported(P, N, K) ? gemm2_workspace_bytes(P, K) : 0;
  if (!exact && mxfp4_mfma_supported(P, N, K) && mxfp4_workspace_bytes(P, K) > relaid)
    relaid = mxfp4_workspace_bytes(P, K);          // the mode is not known here: the larger of the two
  const size_t gemm = route_bytes(P, E) + relaid;
  return gemm > decode ? gemm : decode;
}

// ---- scratch of the allocation-free entry point ------------------------------
// Part of the code object: each GPU that loads the library holds its own copy
// at its own address.  In host code the name is only a handle for
// hipGetSymbolAddress; the address it yields is what kernels are given.
__device__ __align__(256) unsigned char scratch[QMM_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// The current device's scratch address (looked up once per device).
int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(QMM_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(QMM_ERR_HIP, "device ordinal %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return fail(QMM_ERR_HIP, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return QMM_OK;
}

}  // namespace
}  // namespace qmm

using namespace qmm;

extern "C" {

int qmm_abi_version(void) { return 2; }

const char* qmm_last_error(void) { return g_err; }

size_t qmm_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K, int, int, int mode,
                           int x_dtype) {
  const int terms = act_terms(x_dtype);
  if (terms == 1) return dense_scratch(M, N, K, mode, false);
  // terms as bf16 rows, their float32 products, then the scratch of the bf16
  // product: over terms x M stacked rows (dense) or over M rows (grouped)
  if (batch < 1) batch = 1;
  const size_t stacked = dense_scratch(terms * M, N, K, mode, true), plain = dense_scratch(M, N, K, mode, true);
  return align256((size_t)(batch * terms * M * K) * 2) + align256((size_t)(batch * terms * M * N) * 4) +
         (stacked > plain ? stacked : plain);
}

size_t qmm_gather_workspace_bytes(int64_t P, int64_t E, int64_t N, int64_t K, int x_dtype) {
  const int terms = act_terms(x_dtype);
  if (terms == 1) return gather_scratch(P, E, N, K, false);
  // the gathered rows' terms, their float32 products, the bf16 product's scratch
  return align256((size_t)(terms * P * K) * 2) + align256((size_t)(terms * P * N) * 4) +
         gather_scratch(P, E, N, K, true);
}

int qmm_plan(int64_t M, int64_t N, int64_t K, int group_size, int bits, int mode, int* kernel,
             int* grid, int* block) {
  if (mode == QMM_MODE_MXFP4 && M > kGemvMaxM && mxfp4_mfma_supported(M, N, K)) {
    int g, b;
    mxfp4_geometry(M, N, K, &g, &b);
    if (kernel) *kernel = QMM_KERNEL_MXFP4_MFMA;
    if (grid) *grid = g;
    if (block) *block = b;
    return QMM_OK;
  }
  if (M <= kGemvMaxM && mode == QMM_MODE_MXFP4) {
    // the loader-wavefront kernel from three K-slices a row on, its ragged one-pass form for a K that
    // is no whole number of slices
    int rows;
    if (skinny2_mx_plan(N, K, &rows)) {
      if (kernel) *kernel = QMM_KERNEL_GEMV;
      if (grid) *grid = (int)ceil_div(N, (int64_t)rows);
      if (block) *block = 64 * 12;
      return QMM_OK;
    }
  }
  if (M <= kGemvMaxM && mode == QMM_MODE_AFFINE && (group_size == 64 || group_size == 128) &&
      (bits == 4 || bits == 8) && K % (2048 / bits) == 0) {
    // the staged decode kernel (bf16 tables assumed): contiguous row ranges
    int waves, rows, rows2;
    skinny_geometry(N, K, bits, &waves, &rows);
    // eight compute + four loader wavefronts where the loader kernel serves the shape
    const bool loaders = !experiment_env("QMM_SKINNY_V1") && skinny2_plan(M, N, K, bits, &rows2);
    if (loaders) rows = rows2;
    if (kernel) *kernel = QMM_KERNEL_GEMV;
    if (grid) *grid = (int)ceil_div(N, rows);
    if (block) *block = loaders ? 64 * 12 : 64 * waves;
    return QMM_OK;
  }
  if (M <= kGemvMaxM) {
    int t, waves;
    gemv_geometry(M, N, K, &t, &waves);
    if (kernel) *kernel = QMM_KERNEL_GEMV;
    if (grid) *grid = (int)ceil_div(N, 16 * t);
    if (block) *block = 64 * waves;
  } else if (K % 256 == 0 && (mode == QMM_MODE_MXFP4 || bits == 4 || bits == 8)) {
    // the split-role kernel (bf16 tables assumed): 256-row tiles, four
    // multiplying and four dequantizing wavefronts
    if (kernel) *kernel = QMM_KERNEL_GEMM;
    if (grid) *grid = (int)(ceil_div(N, 128) * ceil_div(M, 256));
    if (block) *block = 512;
  } else {
    const int64_t bm = gemm_row_tile(M, 1);
    if (kernel) *kernel = QMM_KERNEL_GEMM;
    if (grid) *grid = (int)(ceil_div(N, 128) * ceil_div(M, bm));
    if (block) *block = 256;
  }
  return QMM_OK;
}

// The three products on bf16 activations.  `exact`: the activations are exact
// terms of a wider type (MXFP4 weights then take the bf16 kernels).
static int dense_bf16(const void* x, int x_dtype, const void* w, const void* scales,
                      const void* biases, int table_dtype, void* y, int y_dtype, int64_t batch,
                      int64_t M, int64_t N, int64_t K, int group_size, int bits, int mode,
                      void* workspace, size_t workspace_bytes, void* stream, bool exact) {
  if (batch < 0 || M < 0) return fail(QMM_ERR_BAD_ARGUMENT, "negative shape");
  if (batch == 0 || M == 0 || N == 0) return QMM_OK;
  if (K == 0) return fail(QMM_ERR_BAD_SHAPE, "K=0");
  int rc = check_quant(N, K, group_size, bits, mode, table_dtype, w, scales, biases);
  if (rc) return rc;
  rc = check_io(x, x_dtype, y, y_dtype);
  if (rc) return rc;
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX || batch > 65535 || M * K >= (1ll << 30))
    return fail(QMM_ERR_BAD_SHAPE, "shape exceeds kernel index range");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (M <= kGemvMaxM) {
    gemv_dispatch(x, w, scales, biases, table_dtype, y, y_dtype, batch, M, N, K, group_size,
                  bits, mode, nullptr, nullptr, 0, 0, st);
    return check_launch("gemv launch");
  }
  const int wbits = mode == QMM_MODE_MXFP4 ? 4 : bits;
  const int64_t wpr = K * wbits / 32;
  const int64_t ng = mode == QMM_MODE_MXFP4 ? K / 32 : K / group_size;
  const int tabsz = mode == QMM_MODE_MXFP4 ? 1 : (table_dtype == QMM_F32 ? 4 : 2);
  const int ysz = y_dtype == QMM_F32 ? 4 : 2;
  if (mode == QMM_MODE_MXFP4 && !exact && mxfp4_mfma_supported(M, N, K)) {
    // block-scaled matrix cores; the activations are split into the workspace first
    const size_t need = mxfp4_workspace_bytes(M, K);
    if (!workspace || workspace_bytes < need)
      return fail(QMM_ERR_WORKSPACE, "mxfp4 needs %zu workspace bytes, got %zu", need,
                  workspace ? workspace_bytes : (size_t)0);
    if (!aligned16(workspace) || !aligned16(scales))
      return fail(QMM_ERR_BAD_ARGUMENT, "workspace / scale pointer not 16-byte aligned");
    for (int64_t z = 0; z < batch; ++z) {
      mxfp4_mfma_dispatch(static_cast<const char*>(x) + z * M * K * 2,
                          static_cast<const uint32_t*>(w) + z * N * wpr,
                          static_cast<const char*>(scales) + z * N * ng,
                          static_cast<char*>(y) + z * M * N * ysz, y_dtype, nullptr, nullptr,
                          nullptr, M, M, 1, N, K, workspace, st);
      rc = check_launch("mxfp4 launch");
      if (rc) return rc;
    }
    return QMM_OK;
  }
  if (gemm2_supported(M, N, K)) {
    const size_t need = gemm2_workspace_bytes(M, K);
    if (!workspace || workspace_bytes < need)
      return fail(QMM_ERR_WORKSPACE, "the prefill kernel needs %zu workspace bytes, got %zu", need,
                  workspace ? workspace_bytes : (size_t)0);
    if (!aligned16(workspace) || !aligned16(scales))
      return fail(QMM_ERR_BAD_ARGUMENT, "workspace / table pointer not 16-byte aligned");
    const int bm = (int)gemm_row_tile(M, 1);
    for (int64_t z = 0; z < batch; ++z) {
      gemm2_dispatch(static_cast<const char*>(x) + z * M * K * 2,
                     static_cast<const uint32_t*>(w) + z * N * wpr,
                     static_cast<const char*>(scales) + z * N * ng * tabsz,
                     biases ? static_cast<const char*>(biases) + z * N * ng * tabsz : nullptr,
                     table_dtype, static_cast<char*>(y) + z * M * N * ysz, y_dtype, nullptr, nullptr,
                     nullptr, M, M, 1, N, K, group_size, bits, mode, bm, workspace, st);
      rc = check_launch("gemm launch");
      if (rc) return rc;
    }
    return QMM_OK;
  }
  for (int64_t z = 0; z < batch; ++z) {
    gemm_dispatch(static_cast<const char*>(x) + z * M * K * 2,
                  static_cast<const uint32_t*>(w) + z * N * wpr,
                  static_cast<const char*>(scales) + z * N * ng * tabsz,
                  biases ? static_cast<const char*>(biases) + z * N * ng * tabsz : nullptr,
                  table_dtype, static_cast<char*>(y) + z * M * N * ysz, y_dtype, nullptr, nullptr,
                  nullptr, M, M, 1, N, K, group_size, bits, mode, st);
    rc = check_launch("gemm launch");
    if (rc) return rc;
  }
  return QMM_OK;
}

static int grouped_bf16(const void* x, int x_dtype, const void* w, const void* scales,
                        const void* biases, int table_dtype, void* y, int y_dtype,
                        const int32_t* row_offsets, int64_t R, int64_t E, int64_t N, int64_t K,
                        int group_size, int bits, int mode, void* workspace, size_t workspace_bytes,
                        void* stream, bool exact) {
  if (R < 0 || E < 0) return fail(QMM_ERR_BAD_ARGUMENT, "negative shape");
  if (R == 0 || N == 0 || E == 0) return QMM_OK;
  if (!row_offsets) return fail(QMM_ERR_BAD_ARGUMENT, "null row_offsets");
  int rc = check_quant(N, K, group_size, bits, mode, table_dtype, w, scales, biases);
  if (rc) return rc;
  rc = check_io(x, x_dtype, y, y_dtype);
  if (rc) return rc;
  if (R > INT32_MAX || N > INT32_MAX || K > INT32_MAX || E > 65535 || R * K >= (1ll << 30))
    return fail(QMM_ERR_BAD_SHAPE, "shape exceeds kernel index range");
  if (mode == QMM_MODE_MXFP4 && !exact && mxfp4_mfma_supported(R, N, K) && workspace &&
      workspace_bytes >= mxfp4_workspace_bytes(R, K) && aligned16(workspace) && aligned16(scales)) {
    // MXFP4 experts on the block-scaled matrix cores
    mxfp4_mfma_dispatch(x, w, scales, y, y_dtype, row_offsets, nullptr, nullptr, R, R, E, N, K,
                        workspace, static_cast<hipStream_t>(stream));
    return check_launch("grouped mxfp4 launch");
  }
  if (gemm2_supported(R, N, K) && workspace && workspace_bytes >= gemm2_workspace_bytes(R, K) &&
      aligned16(workspace)) {
    gemm2_dispatch(x, w, scales, biases, table_dtype, y, y_dtype, row_offsets, nullptr, nullptr, R,
                   R, E, N, K, group_size, bits, mode, (int)gemm_row_tile(R, E), workspace,
                   static_cast<hipStream_t>(stream));
    return check_launch("grouped gemm launch");
  }
  // without a workspace the grouped product runs on the LDS-staged kernel
  gemm_dispatch(x, w, scales, biases, table_dtype, y, y_dtype, row_offsets, nullptr, nullptr, R,
                R, E, N, K, group_size, bits, mode, static_cast<hipStream_t>(stream));
  return check_launch("grouped gemm launch");
}

static int gather_bf16(const void* x, int x_dtype, const void* w, const void* scales,
                       const void* biases, int table_dtype, void* y, int y_dtype,
                       const int32_t* lhs_idx, const int32_t* rhs_idx, int64_t P, int64_t T,
                       int64_t E, int64_t N, int64_t K, int group_size, int bits, int mode,
                       void* workspace, size_t workspace_bytes, void* stream, bool exact) {
  if (P < 0 || T < 0 || E < 0) return fail(QMM_ERR_BAD_ARGUMENT, "negative shape");
  if (P == 0 || N == 0) return QMM_OK;
  if (!rhs_idx) return fail(QMM_ERR_BAD_ARGUMENT, "null rhs_idx");
  int rc = check_quant(N, K, group_size, bits, mode, table_dtype, w, scales, biases);
  if (rc) return rc;
  rc = check_io(x, x_dtype, y, y_dtype);
  if (rc) return rc;
  if (P > INT32_MAX / 2 || N > INT32_MAX || K > INT32_MAX || E > 65535 || T * K >= (1ll << 30))
    return fail(QMM_ERR_BAD_SHAPE, "shape exceeds kernel index range");
  hipStream_t st = static_cast<hipStream_t>(stream);
  static const bool no_grouped_decode = experiment_env("QMM_NO_GROUPED_DECODE") != nullptr;
  if (grouped_decode_pairs(P, E) && !no_grouped_decode && workspace &&
      workspace_bytes >= route_bytes_segments(P, E) &&
      skinny2_grouped_supported(N, K, group_size, bits, mode, table_dtype, scales, biases, E)) {
    int32_t* ro = static_cast<int32_t*>(workspace);
    int32_t* cursor = ro + E + 1;
    int32_t* src_row = cursor + E;
    int32_t* out_row = src_row + P;
    int32_t* segments = out_row + P;
    hipLaunchKernelGGL(route_kernel, dim3(1), dim3(1024), 0, st, lhs_idx, rhs_idx, (int)P, (int)E,
                       ro, cursor, src_row, out_row, segments);
    rc = check_launch("route launch");
    if (rc) return rc;
    skinny2_grouped_dispatch(x, w, scales, biases, y, y_dtype, segments, src_row, out_row, P, T, E, N, K,
                             group_size, bits, mode, table_dtype, st);
    return check_launch("grouped decode launch");
  }
  if (P <= kGatherGemvMaxPairs) {
    // From sixteen pairs on, and half a pair an expert, shapes that only the
    // general decode kernels serve are grouped by expert as well: an expert's
    // weights are then read once for up to sixteen of its pairs instead of
    // once per pair.  (The sort costs a launch of its own, and with fewer
    // pairs than that few of them share an expert.  Measured on 32 MXFP4
    // experts of [5760, 2880]: 16 pairs 61 against 60 us, 32 pairs 86 against
    // 110, 64 pairs 109 against 216; on 128 experts: 32 pairs 128 against 110,
    // 64 pairs 194 against 217; 8 experts of [4096, 11008] with four-bit
    // codes: 16 pairs 108 against 206 us, 32 pairs 110 against 397.)
    if (P >= 16 && 2 * P >= E && grouped_decode_pairs(P, E) && workspace &&
        workspace_bytes >= route_bytes_segments(P, E) &&
        gemv_runs_general(N, K, group_size, bits, mode, table_dtype, scales, biases) &&
        !experiment_env("QMM_NO_GROUPED_GEMV")) {
      int32_t* ro = static_cast<int32_t*>(workspace);
      int32_t* cursor = ro + E + 1;
      int32_t* src_row = cursor + E;
      int32_t* out_row = src_row + P;
      int32_t* segments = out_row + P;
      hipLaunchKernelGGL(route_kernel, dim3(1), dim3(1024), 0, st, lhs_idx, rhs_idx, (int)P, (int)E,
                         ro, cursor, src_row, out_row, segments);
      rc = check_launch("route launch");
      if (rc) return rc;
      gemv_grouped_dispatch(x, w, scales, biases, table_dtype, y, y_dtype, segments, src_row, out_row,
                            skinny2_max_segments(P, E), T, N, K, group_size, bits, mode, st);
      return check_launch("grouped gemv launch");
    }
    gemv_dispatch(x, w, scales, biases, table_dtype, y, y_dtype, P, 1, N, K, group_size, bits,
                  mode, lhs_idx, rhs_idx, E, T, st);
    return check_launch("gather gemv launch");
  }
  const size_t need = route_bytes(P, E);
  if (!workspace || workspace_bytes < need)
    return fail(QMM_ERR_WORKSPACE, "gather_qmm needs %zu workspace bytes, got %zu", need,
                workspace_bytes);
  int32_t* ro = static_cast<int32_t*>(workspace);
  int32_t* cursor = ro + E + 1;
  int32_t* src_row = cursor + E;
  int32_t* out_row = src_row + P;
  hipLaunchKernelGGL(route_kernel, dim3(1), dim3(1024), 0, st, lhs_idx, rhs_idx, (int)P, (int)E,
                     ro, cursor, src_row, out_row, static_cast<int32_t*>(nullptr));
  rc = check_launch("route launch");
  if (rc) return rc;
  if (mode == QMM_MODE_MXFP4 && !exact && mxfp4_mfma_supported(P, N, K) &&
      workspace_bytes >= need + mxfp4_workspace_bytes(P, K) && aligned16(workspace) &&
      aligned16(scales)) {
    mxfp4_mfma_dispatch(x, w, scales, y, y_dtype, ro, src_row, out_row, P, T, E, N, K,
                        static_cast<char*>(workspace) + need, st);
    return check_launch("gather mxfp4 launch");
  }
  if (gemm2_supported(P, N, K) && workspace_bytes >= need + gemm2_workspace_bytes(P, K) &&
      aligned16(workspace)) {
    // rows gathered in expert order into the re-laid copy, results scattered back to pair order
    gemm2_dispatch(x, w, scales, biases, table_dtype, y, y_dtype, ro, src_row, out_row, P, T, E, N, K,
                   group_size, bits, mode, (int)gemm_row_tile(P, E),
                   static_cast<char*>(workspace) + need, st);
    return check_launch("gather gemm launch");
  }
  gemm_dispatch(x, w, scales, biases, table_dtype, y, y_dtype, ro, src_row, out_row, P, T, E, N, K,
                group_size, bits, mode, st);
  return check_launch("gather gemm launch");
}

int qmm_quantized_matmul(const void* x, int x_dtype, const void* w, const void* scales,
                         const void* biases, int table_dtype, void* y, int y_dtype,
                         int64_t batch, int64_t M, int64_t N, int64_t K, int group_size,
                         int bits, int mode, void* workspace, size_t workspace_bytes,
                         void* stream) {
  const int terms = act_terms(x_dtype);
  if (terms == 1 || batch <= 0 || M <= 0 || N <= 0 || K <= 0 || !x)
    return dense_bf16(x, x_dtype, w, scales, biases, table_dtype, y, y_dtype, batch, M, N, K,
                      group_size, bits, mode, workspace, workspace_bytes, stream, false);
  // bf16 terms as extra rows: x2 [batch, terms * M, K] -> p2 [batch, terms * M, N] -> y
  if (!aligned16(x)) return fail(QMM_ERR_BAD_ARGUMENT, "activation pointer not 16-byte aligned");
  if (batch * terms * M * K >= (1ll << 30))
    return fail(QMM_ERR_BAD_SHAPE, "shape exceeds kernel index range");
  const size_t xs = align256((size_t)(batch * terms * M * K) * 2);
  const size_t ps = align256((size_t)(batch * terms * M * N) * 4);
  const size_t inner = dense_scratch(terms * M, N, K, mode, true);
  if (!workspace || workspace_bytes < xs + ps + inner || !aligned16(workspace))
    return fail(QMM_ERR_WORKSPACE, "float16 / float32 activations need %zu aligned workspace bytes, got %zu",
                xs + ps + inner, workspace ? workspace_bytes : (size_t)0);
  char* ws = static_cast<char*>(workspace);
  hipStream_t st = static_cast<hipStream_t>(stream);
  split_terms_dispatch(x, x_dtype, ws, batch, M, K, nullptr, -1, st);
  int rc = check_launch("activation split launch");
  if (rc) return rc;
  rc = dense_bf16(ws, QMM_BF16, w, scales, biases, table_dtype, ws + xs, QMM_F32, batch, terms * M, N, K,
                  group_size, bits, mode, inner ? ws + xs + ps : nullptr, inner, stream, true);
  if (rc) return rc;
  if (!y) return fail(QMM_ERR_BAD_ARGUMENT, "null output pointer");
  sum_terms_dispatch(ws + xs, terms, y, y_dtype, batch, M, N, nullptr, nullptr, 0, st);
  return check_launch("term sum launch");
}

int qmm_grouped_qmm(const void* x, int x_dtype, const void* w, const void* scales,
                    const void* biases, int table_dtype, void* y, int y_dtype,
                    const int32_t* row_offsets, int64_t R, int64_t E, int64_t N, int64_t K,
                    int group_size, int bits, int mode, void* workspace, size_t workspace_bytes,
                    void* stream) {
  const int terms = act_terms(x_dtype);
  if (terms == 1 || R <= 0 || E <= 0 || N <= 0 || K <= 0 || !x || !row_offsets || !y)
    return grouped_bf16(x, x_dtype, w, scales, biases, table_dtype, y, y_dtype, row_offsets, R, E, N, K,
                        group_size, bits, mode, workspace, workspace_bytes, stream, false);
  // one grouped product per bf16 term (the rows keep their expert order)
  if (!aligned16(x)) return fail(QMM_ERR_BAD_ARGUMENT, "activation pointer not 16-byte aligned");
  const size_t xs = align256((size_t)(terms * R * K) * 2), ps = align256((size_t)(terms * R * N) * 4);
  const size_t inner = dense_scratch(R, N, K, mode, true);
  if (!workspace || workspace_bytes < xs + ps + inner || !aligned16(workspace))
    return fail(QMM_ERR_WORKSPACE, "float16 / float32 activations need %zu aligned workspace bytes, got %zu",
                xs + ps + inner, workspace ? workspace_bytes : (size_t)0);
  char* ws = static_cast<char*>(workspace);
  hipStream_t st = static_cast<hipStream_t>(stream);
  split_terms_dispatch(x, x_dtype, ws, 1, R, K, nullptr, -1, st);
  int rc = check_launch("activation split launch");
  for (int t = 0; t < terms && !rc; ++t)
    rc = grouped_bf16(ws + (size_t)t * R * K * 2, QMM_BF16, w, scales, biases, table_dtype,
                      ws + xs + (size_t)t * R * N * 4, QMM_F32, row_offsets, R, E, N, K, group_size, bits,
                      mode, inner ? ws + xs + ps : nullptr, inner, stream, true);
  if (rc) return rc;
  sum_terms_dispatch(ws + xs, terms, y, y_dtype, 1, R, N, row_offsets, nullptr, E, st);
  return check_launch("term sum launch");
}

int qmm_gather_qmm(const void* x, int x_dtype, const void* w, const void* scales,
                   const void* biases, int table_dtype, void* y, int y_dtype,
                   const int32_t* lhs_idx, const int32_t* rhs_idx, int64_t P, int64_t T,
                   int64_t E, int64_t N, int64_t K, int group_size, int bits, int mode,
                   void* workspace, size_t workspace_bytes, void* stream) {
  const int terms = act_terms(x_dtype);
  if (terms == 1 || P <= 0 || T < 0 || E < 0 || N <= 0 || K <= 0 || !x || !rhs_idx || !y)
    return gather_bf16(x, x_dtype, w, scales, biases, table_dtype, y, y_dtype, lhs_idx, rhs_idx, P, T, E,
                       N, K, group_size, bits, mode, workspace, workspace_bytes, stream, false);
  // the pairs' rows are gathered while they are split; every term is then a
  // gathered product over rows already in pair order
  const size_t xs = align256((size_t)(terms * P * K) * 2), ps = align256((size_t)(terms * P * N) * 4);
  const size_t inner = gather_scratch(P, E, N, K, true);
  if (!workspace || workspace_bytes < xs + ps + inner || !aligned16(workspace))
    return fail(QMM_ERR_WORKSPACE, "float16 / float32 activations need %zu aligned workspace bytes, got %zu",
                xs + ps + inner, workspace ? workspace_bytes : (size_t)0);
  if (terms * P * K >= (1ll << 30)) return fail(QMM_ERR_BAD_SHAPE, "shape exceeds kernel index range");
  char* ws = static_cast<char*>(workspace);
  hipStream_t st = static_cast<hipStream_t>(stream);
  split_terms_dispatch(x, x_dtype, ws, 1, P, K, lhs_idx, T, st);      // lhs_idx null: row p of x
  int rc = check_launch("activation split launch");
  for (int t = 0; t < terms && !rc; ++t)
    rc = gather_bf16(ws + (size_t)t * P * K * 2, QMM_BF16, w, scales, biases, table_dtype,
                     ws + xs + (size_t)t * P * N * 4, QMM_F32, nullptr, rhs_idx, P, P, E, N, K, group_size,
                     bits, mode, inner ? ws + xs + ps : nullptr, inner, stream, true);
  if (rc) return rc;
  sum_terms_dispatch(ws + xs, terms, y, y_dtype, 1, P, N, nullptr, rhs_idx, E, st);
  return check_launch("term sum launch");
}

int qmm_gather_qmm_static(const void* x, int x_dtype, const void* w, const void* scales,
                          const void* biases, int table_dtype, void* y, int y_dtype,
                          const int32_t* lhs_idx, const int32_t* rhs_idx, int64_t P, int64_t T,
                          int64_t E, int64_t N, int64_t K, int group_size, int bits, int mode,
                          void* stream) {
  if (P < 0 || T < 0 || E < 0 || N < 0 || K < 0) return fail(QMM_ERR_BAD_ARGUMENT, "negative shape");
  const size_t need = qmm_gather_workspace_bytes(P, E, N, K, x_dtype);
  if (need > (size_t)QMM_STATIC_SCRATCH_BYTES)
    return fail(QMM_ERR_WORKSPACE,
                "gather_qmm_static: %lld pairs over %lld experts of [%lld, %lld] need %zu scratch "
                "bytes, the static scratch holds %zu (use qmm_gather_qmm with a workspace)",
                (long long)P, (long long)E, (long long)N, (long long)K, need,
                (size_t)QMM_STATIC_SCRATCH_BYTES);
  void* ptr = nullptr;
  if (need) {
    const int rc = static_scratch(&ptr);
    if (rc) return rc;
  }
  return qmm_gather_qmm(x, x_dtype, w, scales, biases, table_dtype, y, y_dtype, lhs_idx, rhs_idx, P,
                        T, E, N, K, group_size, bits, mode, ptr, need ? (size_t)QMM_STATIC_SCRATCH_BYTES : 0,
                        stream);
}

int qmm_dequantize(const void* w, const void* scales, const void* biases, int table_dtype,
                   void* out, int out_dtype, int64_t rows, int64_t K, int group_size, int bits,
                   int mode, void* stream) {
  if (rows < 0) return fail(QMM_ERR_BAD_ARGUMENT, "negative shape");
  if (rows == 0 || K == 0) return QMM_OK;
  int rc = check_quant(rows, K, group_size, bits, mode, table_dtype, w, scales, biases);
  if (rc) return rc;
  if (!out) return fail(QMM_ERR_BAD_ARGUMENT, "null output pointer");
  if (out_dtype != QMM_F32 && out_dtype != QMM_BF16 && out_dtype != QMM_F16)
    return fail(QMM_ERR_UNSUPPORTED, "output dtype %d", out_dtype);
  if (!aligned16(out)) return fail(QMM_ERR_BAD_ARGUMENT, "output pointer not 16-byte aligned");
  dequant_dispatch(w, scales, biases, table_dtype, out, out_dtype, rows, K, group_size, bits,
                   mode, static_cast<hipStream_t>(stream));
  return check_launch("dequantize launch");
}

static int check_codes(const void* a, const void* b, int64_t rows, int64_t K, int bits) {
  if (rows < 0 || K < 0) return fail(QMM_ERR_BAD_ARGUMENT, "negative shape");
  if (bits != 2 && bits != 4 && bits != 8) return fail(QMM_ERR_UNSUPPORTED, "bits=%d (2, 4 or 8)", bits);
  if (K % (32 / bits)) return fail(QMM_ERR_BAD_SHAPE, "K=%lld not a multiple of %d", (long long)K, 32 / bits);
  if (rows * K == 0) return QMM_OK;
  if (!a || !b) return fail(QMM_ERR_BAD_ARGUMENT, "null pointer");
  if (!aligned16(a) || !aligned16(b)) return fail(QMM_ERR_BAD_ARGUMENT, "pointer not 16-byte aligned");
  return QMM_OK;
}

int qmm_unpack_codes(const void* w, void* codes, int64_t rows, int64_t K, int bits, void* stream) {
  int rc = check_codes(w, codes, rows, K, bits);
  if (rc || rows * K == 0) return rc;
  unpack_dispatch(w, codes, rows, K, bits, static_cast<hipStream_t>(stream));
  return check_launch("unpack launch");
}

int qmm_pack_codes(const void* codes, void* w, int64_t rows, int64_t K, int bits, void* stream) {
  int rc = check_codes(codes, w, rows, K, bits);
  if (rc || rows * K == 0) return rc;
  pack_dispatch(codes, w, rows, K, bits, static_cast<hipStream_t>(stream));
  return check_launch("pack launch");
}

int qmm_take_k(const void* x, int x_dtype, const int32_t* perm, void* out, int64_t rows,
               int64_t K, void* stream) {
  if (rows < 0 || K < 0) return fail(QMM_ERR_BAD_ARGUMENT, "negative shape");
  if (rows * K == 0) return QMM_OK;
  if (!x || !perm || !out) return fail(QMM_ERR_BAD_ARGUMENT, "null pointer");
  if (x_dtype != QMM_F32 && x_dtype != QMM_BF16 && x_dtype != QMM_F16)
    return fail(QMM_ERR_UNSUPPORTED, "dtype %d", x_dtype);
  take_dispatch(x, x_dtype, perm, out, rows, K, static_cast<hipStream_t>(stream));
  return check_launch("take launch");
}

}  // extern "C"
