// Layout utilities: unpack / pack codes, dequantize, activation gather.
// All are elementwise and HBM-bound; each thread handles one packed word (or
// one 16-byte run of the output) so loads and stores are coalesced.
#include "qmm_common.hpp"

namespace qmm {

namespace {

constexpr int kBlock = 256;

template <int BITS>
__global__ __launch_bounds__(kBlock) void unpack_kernel(const uint32_t* __restrict__ w,
                                                       uint8_t* __restrict__ codes,
                                                       int64_t words) {
  constexpr int PER = 32 / BITS;
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= words) return;
  const uint32_t v = w[i];
  uint8_t out[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) out[j] = (uint8_t)((v >> (j * BITS)) & ((1u << BITS) - 1u));
  if constexpr (PER == 4) {
    *reinterpret_cast<uint32_t*>(codes + i * 4) = *reinterpret_cast<uint32_t*>(out);
  } else if constexpr (PER == 8) {
    *reinterpret_cast<u32x2*>(codes + i * 8) = *reinterpret_cast<u32x2*>(out);
  } else {
    *reinterpret_cast<u32x4*>(codes + i * 16) = *reinterpret_cast<u32x4*>(out);
  }
}

template <int BITS>
__global__ __launch_bounds__(kBlock) void pack_kernel(const uint8_t* __restrict__ codes,
                                                     uint32_t* __restrict__ w, int64_t words) {
  constexpr int PER = 32 / BITS;
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= words) return;
  uint8_t in[PER];
  if constexpr (PER == 4) {
    *reinterpret_cast<uint32_t*>(in) = *reinterpret_cast<const uint32_t*>(codes + i * 4);
  } else if constexpr (PER == 8) {
    *reinterpret_cast<u32x2*>(in) = *reinterpret_cast<const u32x2*>(codes + i * 8);
  } else {
    *reinterpret_cast<u32x4*>(in) = *reinterpret_cast<const u32x4*>(codes + i * 16);
  }
  uint32_t v = 0;
#pragma unroll
  for (int j = 0; j < PER; ++j) v |= ((uint32_t)in[j] & ((1u << BITS) - 1u)) << (j * BITS);
  w[i] = v;
}

// One thread per packed word; MODE 0 affine, 1 mxfp4 (BITS = 4, group 32).
template <int MODE, int BITS>
__global__ __launch_bounds__(kBlock) void dequant_kernel(const uint32_t* __restrict__ w,
                                                        const void* __restrict__ s,
                                                        const void* __restrict__ b, int tab,
                                                        void* __restrict__ out, int out_dtype,
                                                        int64_t words, int64_t wpr, int gs) {
  constexpr int PER = 32 / BITS;
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= words) return;
  const int64_t row = i / wpr, col = (i - row * wpr) * PER;      // first element index
  const int64_t k = wpr * PER;
  const uint32_t v = w[i];
  float f[PER];
  if constexpr (MODE == 1) {
    const float sc = e8m0_to_f32(static_cast<const uint8_t*>(s)[row * (k / 32) + col / 32]);
#pragma unroll
    for (int j = 0; j < PER; ++j) f[j] = e2m1_to_f32((v >> (4 * j)) & 15u) * sc;
  } else {
    const int64_t ti = row * (k / gs) + col / gs;                // PER divides gs
    const float sc = load_table_rt(s, ti, tab), bi = load_table_rt(b, ti, tab);
#pragma unroll
    for (int j = 0; j < PER; ++j)
      f[j] = fmaf(sc, (float)((v >> (j * BITS)) & ((1u << BITS) - 1u)), bi);
  }
  const int64_t o = i * PER;
  if (out_dtype == QMM_F32) {
    float* p = static_cast<float*>(out) + o;
#pragma unroll
    for (int j = 0; j < PER; j += 4) *reinterpret_cast<f32x4*>(p + j) = f32x4{f[j], f[j + 1], f[j + 2], f[j + 3]};
  } else {
    uint32_t h[PER / 2];
#pragma unroll
    for (int j = 0; j < PER / 2; ++j) {
      if (out_dtype == QMM_BF16) h[j] = pack_bf16x2(f[2 * j], f[2 * j + 1]);
      else h[j] = f32_to_f16_bits(f[2 * j]) | (f32_to_f16_bits(f[2 * j + 1]) << 16);
    }
    uint32_t* p = reinterpret_cast<uint32_t*>(static_cast<uint16_t*>(out) + o);
    if constexpr (PER == 8) *reinterpret_cast<u32x4*>(p) = u32x4{h[0], h[1], h[2], h[3]};
    else *reinterpret_cast<u32x2*>(p) = u32x2{h[0], h[1]};
  }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void take_kernel(const T* __restrict__ x,
                                                     const int32_t* __restrict__ perm,
                                                     T* __restrict__ out, int64_t rows, int64_t k) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= rows * k) return;
  const int64_t r = i / k, j = i - r * k;
  out[i] = x[r * k + perm[j]];
}

// float16 / float32 activations as exact sums of bf16 terms (float16: 11
// significant bits = 8 + 3; float32: 24 = 8 + 8 + 8), term t of batch entry z,
// row m at out[z][t][m][:]: the matrix cores then multiply bf16 operands and
// every product stays exact.  x [batch, rows, K]; out bf16 [batch, TERMS, rows, K].
template <int TERMS, typename T>
__global__ void split_terms_kernel(const T* __restrict__ x, uint16_t* __restrict__ out,
                                   int64_t rows_k, int64_t k, int64_t total,
                                   const int32_t* __restrict__ src_row, int64_t x_rows) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int64_t z = i / rows_k, j = i - z * rows_k;
  int64_t src = i;
  bool ok = true;
  if (src_row) {                                   // rows gathered: out row j / k is x row src_row[j / k]
    const int64_t row = j / k, sr = src_row[row];
    ok = sr >= 0 && sr < x_rows;                   // a row outside x gathers zeros
    src = sr * k + (j - row * k);
  } else if (x_rows >= 0) {                        // pair p reads row p of x: rows past the end read as zeros
    ok = j / k < x_rows;
  }
  float v = 0.f;
  if (ok) {
    if constexpr (sizeof(T) == 4) v = x[src];
    else v = f16_bits_to_f32(x[src]);
  }
  uint16_t* o = out + z * TERMS * rows_k + j;
#pragma unroll
  for (int t = 0; t < TERMS; ++t) {
    uint32_t hi = __float_as_uint(v) & 0xFFFF0000u;             // truncation: the remainder is exact
    if (v != v) hi |= 0x00400000u;                              // a NaN stays a NaN when its payload is cut
    o[(int64_t)t * rows_k] = (uint16_t)(hi >> 16);
    // inf / NaN stay in the first term alone (inf - inf would put NaN into the others)
    v = (hi & 0x7F800000u) == 0x7F800000u ? 0.f : v - __uint_as_float(hi);
  }
}

// y[z][m][n] = sum_t part[z][t][m][n] (float32 partial products, added in term
// order: largest first), rounded once to the output type.  Rows that the
// product did not compute are left alone: rows outside [offsets[0], offsets[E])
// of a grouped product, pairs whose expert index is outside [0, E) of a
// gathered one.
template <int TERMS>
__global__ void sum_terms_kernel(const float* __restrict__ part, void* __restrict__ y, int y_dtype,
                                 int64_t rows_n, int64_t n, int64_t total,
                                 const int32_t* __restrict__ offsets,
                                 const int32_t* __restrict__ expert_of_row, int E) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int64_t z = i / rows_n, j = i - z * rows_n;
  if (offsets || expert_of_row) {
    const int64_t row = j / n;
    if (offsets && (row < offsets[0] || row >= offsets[E])) return;
    if (expert_of_row && (expert_of_row[row] < 0 || expert_of_row[row] >= E)) return;
  }
  const float* p = part + z * TERMS * rows_n + j;
  float v = p[0];
#pragma unroll
  for (int t = 1; t < TERMS; ++t) v += p[(int64_t)t * rows_n];
  store_out(y, i, v, y_dtype);
}

inline unsigned blocks_for(int64_t n) { return (unsigned)ceil_div(n, kBlock); }

}  // namespace

void unpack_dispatch(const void* w, void* codes, int64_t rows, int64_t K, int bits,
                     hipStream_t st) {
  const int64_t words = rows * (K * bits / 32);
  if (words == 0) return;
  const uint32_t* wp = static_cast<const uint32_t*>(w);
  uint8_t* cp = static_cast<uint8_t*>(codes);
  if (bits == 4) hipLaunchKernelGGL(unpack_kernel<4>, dim3(blocks_for(words)), dim3(kBlock), 0, st, wp, cp, words);
  else if (bits == 8) hipLaunchKernelGGL(unpack_kernel<8>, dim3(blocks_for(words)), dim3(kBlock), 0, st, wp, cp, words);
  else hipLaunchKernelGGL(unpack_kernel<2>, dim3(blocks_for(words)), dim3(kBlock), 0, st, wp, cp, words);
}

void pack_dispatch(const void* codes, void* w, int64_t rows, int64_t K, int bits, hipStream_t st) {
  const int64_t words = rows * (K * bits / 32);
  if (words == 0) return;
  const uint8_t* cp = static_cast<const uint8_t*>(codes);
  uint32_t* wp = static_cast<uint32_t*>(w);
  if (bits == 4) hipLaunchKernelGGL(pack_kernel<4>, dim3(blocks_for(words)), dim3(kBlock), 0, st, cp, wp, words);
  else if (bits == 8) hipLaunchKernelGGL(pack_kernel<8>, dim3(blocks_for(words)), dim3(kBlock), 0, st, cp, wp, words);
  else hipLaunchKernelGGL(pack_kernel<2>, dim3(blocks_for(words)), dim3(kBlock), 0, st, cp, wp, words);
}

void dequant_dispatch(const void* w, const void* s, const void* b, int tab, void* out,
                      int out_dtype, int64_t rows, int64_t K, int gs, int bits, int mode,
                      hipStream_t st) {
  const uint32_t* wp = static_cast<const uint32_t*>(w);
  if (mode == QMM_MODE_MXFP4) {
    const int64_t wpr = K / 8, words = rows * wpr;
    if (words == 0) return;
    hipLaunchKernelGGL((dequant_kernel<1, 4>), dim3(blocks_for(words)), dim3(kBlock), 0, st, wp, s, b, tab, out, out_dtype, words, wpr, 32);
    return;
  }
  const int64_t wpr = K * bits / 32, words = rows * wpr;
  if (words == 0) return;
  if (bits == 4) hipLaunchKernelGGL((dequant_kernel<0, 4>), dim3(blocks_for(words)), dim3(kBlock), 0, st, wp, s, b, tab, out, out_dtype, words, wpr, gs);
  else hipLaunchKernelGGL((dequant_kernel<0, 8>), dim3(blocks_for(words)), dim3(kBlock), 0, st, wp, s, b, tab, out, out_dtype, words, wpr, gs);
}

// x (float16 / float32) [batch, rows, K] -> bf16 terms [batch, terms, rows, K];
// with src_row (batch = 1): out row r = x row src_row[r] of x [x_rows, K]; without it and x_rows >= 0:
// out row r = x row r, rows past x_rows read as zeros; x_rows < 0: no gather, rows is what x holds
void split_terms_dispatch(const void* x, int x_dtype, void* out, int64_t batch, int64_t rows,
                          int64_t K, const int32_t* src_row, int64_t x_rows, hipStream_t st) {
  const int64_t total = batch * rows * K;
  if (total == 0) return;
  uint16_t* o = static_cast<uint16_t*>(out);
  if (x_dtype == QMM_F32)
    hipLaunchKernelGGL((split_terms_kernel<3, float>), dim3(blocks_for(total)), dim3(kBlock), 0, st,
                       static_cast<const float*>(x), o, rows * K, K, total, src_row, x_rows);
  else
    hipLaunchKernelGGL((split_terms_kernel<2, uint16_t>), dim3(blocks_for(total)), dim3(kBlock), 0, st,
                       static_cast<const uint16_t*>(x), o, rows * K, K, total, src_row, x_rows);
}

// part float32 [batch, terms, rows, N] -> y [batch, rows, N]; `offsets` ([E+1],
// grouped form) / `expert_of_row` ([rows], gathered form) name the rows that
// were computed (null: all of them)
void sum_terms_dispatch(const void* part, int terms, void* y, int y_dtype, int64_t batch,
                        int64_t rows, int64_t N, const int32_t* offsets,
                        const int32_t* expert_of_row, int64_t E, hipStream_t st) {
  const int64_t total = batch * rows * N;
  if (total == 0) return;
  const float* p = static_cast<const float*>(part);
  if (terms == 3)
    hipLaunchKernelGGL(sum_terms_kernel<3>, dim3(blocks_for(total)), dim3(kBlock), 0, st, p, y, y_dtype,
                       rows * N, N, total, offsets, expert_of_row, (int)E);
  else
    hipLaunchKernelGGL(sum_terms_kernel<2>, dim3(blocks_for(total)), dim3(kBlock), 0, st, p, y, y_dtype,
                       rows * N, N, total, offsets, expert_of_row, (int)E);
}

void take_dispatch(const void* x, int x_dtype, const int32_t* perm, void* out, int64_t rows,
                   int64_t K, hipStream_t st) {
  const int64_t n = rows * K;
  if (n == 0) return;
  if (x_dtype == QMM_F32)
    hipLaunchKernelGGL(take_kernel<uint32_t>, dim3(blocks_for(n)), dim3(kBlock), 0, st, static_cast<const uint32_t*>(x), perm, static_cast<uint32_t*>(out), rows, K);
  else
    hipLaunchKernelGGL(take_kernel<uint16_t>, dim3(blocks_for(n)), dim3(kBlock), 0, st, static_cast<const uint16_t*>(x), perm, static_cast<uint16_t*>(out), rows, K);
}

}  // namespace qmm
