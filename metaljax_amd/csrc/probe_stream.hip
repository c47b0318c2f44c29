// Measuring kernels for the decode roofline: what one launch can reach on this
// machine whatever the arithmetic.  Built into libqmm_probe.so (not part of the
// quantized-matmul ABI); driven by `python bench.py --probe`.
//
//   probe_read   a launch that only reads `bytes` (16 bytes a lane, every
//                workgroup a contiguous share, `unroll` loads in flight a
//                lane) and keeps an XOR so that nothing is elided
//   probe_empty  a launch of the same geometry and LDS size that does nothing
//   probe_mfma_feed  a stream of matrix instructions with and without operand
//                loads beside it (what bounds the prefill kernels)
//   probe_loaders  the decode kernel's way of asking: only the first `active`
//                wavefronts of a workgroup request the workgroup's share, 1 KB
//                an instruction, everything before the first wait, into
//                registers or straight into LDS (`dma`)
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace {

typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

template <int U>
__global__ void read_kernel(const u32x4* __restrict__ p, int64_t pieces_per_wg, uint32_t* sink) {
  extern __shared__ unsigned char lds[];
  const u32x4* base = p + (int64_t)blockIdx.x * pieces_per_wg;
  u32x4 acc = {0u, 0u, 0u, 0u};
  for (int64_t i = threadIdx.x; i < pieces_per_wg; i += (int64_t)blockDim.x * U) {
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t j = i + (int64_t)u * blockDim.x;
      v[u] = j < pieces_per_wg ? __builtin_nontemporal_load(base + j) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u];
  }
  const uint32_t x = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
  if (x == 0x9E3779B9u && sink) sink[threadIdx.x] = x + lds[0];    // practically never: keeps the loads alive
}

typedef __attribute__((address_space(3))) void lds_void;

// U requests a wavefront: chunk (1 KB) c = wave + u * active of the workgroup's share.
template <int U, bool DMA, int AUX>
__global__ void loaders_kernel(const unsigned char* __restrict__ p, int chunks_per_wg, int active,
                               uint32_t* sink) {
  extern __shared__ unsigned char lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (wave >= active) return;
  const unsigned char* base = p + (int64_t)blockIdx.x * chunks_per_wg * 1024;
  const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<unsigned char*>(base), 0, (uint32_t)chunks_per_wg * 1024u, 0x00020000);
  uint32_t x = 0;
  if constexpr (DMA) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = wave + u * active;
      const uint32_t off = c < chunks_per_wg ? (uint32_t)c * 1024u + lane * 16u : 0x80000000u;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void*)(lds + (c < chunks_per_wg ? c : 0) * 1024),
                                               16, off, 0u, 0, AUX);
    }
    __builtin_amdgcn_s_waitcnt(0x0070);     // vmcnt(0)
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    x = reinterpret_cast<const uint32_t*>(lds)[wave * 256 + lane];
  } else {
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = wave + u * active;
      const uint32_t off = c < chunks_per_wg ? (uint32_t)c * 1024u + lane * 16u : 0x80000000u;
      v[u] = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0u, AUX);
    }
    u32x4 acc = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u];
    x = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
  }
  if (x == 0x9E3779B9u && sink) sink[threadIdx.x] = x;
}

// The loaders' request with clock stamps (constant 100 MHz clock, lane 0 of
// every asking wavefront): start, all 32 requests issued, then a quarter, a
// half, three quarters and all of them landed.  pattern 0: 1 KB runs as above;
// 1: the decode kernel's tiles (a request = 256 bytes of each of four rows
// 2 KB apart, the 16-byte pieces of a row permuted by its row number; a
// wavefront's eight consecutive requests walk along its four rows).
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

// What the other eight wavefronts of the workgroup do meanwhile (`busy`): 0 nothing, 1 sleep in a loop, 2 matrix
// instructions, 3 vector ALU work, 4 LDS reads, 5 all three, 6 / 7 an activation fetch first (below); about `iters` rounds of 16 instructions of each kind.
__device__ __forceinline__ void bystander(int busy, int iters, unsigned char* lds, int lane, uint32_t* sink) {
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  bf16x8_t a, b;
  for (int i = 0; i < 8; ++i) { a[i] = (__bf16)(float)(lane + i); b[i] = (__bf16)1.0f; }
  float v = (float)lane;
  uint32_t x = 0;
  for (int it = 0; it < iters; ++it) {
    if (busy == 1) __builtin_amdgcn_s_sleep(8);
    if (busy == 2 || busy == 5) {
#pragma unroll
      for (int k = 0; k < 16; ++k) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
    }
    if (busy == 3 || busy == 5) {
#pragma unroll
      for (int k = 0; k < 64; ++k) v = __builtin_fmaf(v, 1.0001f, 0.5f);
    }
    if (busy == 4 || busy == 5) {
#pragma unroll
      for (int k = 0; k < 8; ++k)
        x ^= *reinterpret_cast<volatile uint32_t*>(lds + 135168 + ((lane * 8 + k * 512 + it * 64) & 8191));
    }
  }
  if (acc[0] + v == 12345.678f && x == 77u) sink[0] = 1u;
}

template <int PATTERN>
__global__ void stamped_loaders_kernel(const unsigned char* __restrict__ p, uint64_t* stamps, int busy, int iters) {
  extern __shared__ unsigned char lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (wave >= 4) {
    if (busy >= 6) {
      // the decode kernel's activation fetch ahead of the stream: sixteen loads a wavefront from one 128 KB array
      // that every workgroup reads (busy 6: one live row, i.e. four live lanes an instruction; 7: sixteen rows,
      // whole lines), then `iters` rounds of arithmetic
      const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(p), 0, 131072u, 0x00020000);
      u32x4 v[16];
      const int w8 = wave - 4;
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        uint32_t off;
        if (busy == 6) off = (lane & 15) == 0 ? (uint32_t)(w8 * 1024 + (u >> 1) * 128 + (lane >> 4) * 32 + (u & 1) * 16) : 0x80000000u;
        else off = (uint32_t)(((u & 1) * 8 + (lane >> 3)) * 8192 + w8 * 1024 + (u >> 1) * 128 + (lane & 7) * 16);
        v[u] = __builtin_amdgcn_raw_buffer_load_b128(rx, off, 0u, 0);
      }
      uint32_t x = 0;
#pragma unroll
      for (int u = 0; u < 16; ++u) x ^= v[u][0] ^ v[u][3];
      if (x == 0x12345u) reinterpret_cast<uint32_t*>(stamps)[65536 * 2 + 1] = x;
      bystander(5, iters, lds, lane, reinterpret_cast<uint32_t*>(stamps) + 65536 * 2);
      return;
    }
    if (busy) bystander(busy, iters, lds, lane, reinterpret_cast<uint32_t*>(stamps) + 65536 * 2);
    return;
  }
  if (busy >= 6) __builtin_amdgcn_s_sleep(32);     // (the loaders start about 0.4 us after the first wavefronts)
  if (busy == -1) {
    // 256 scalar instructions of eight bytes each (2 KB of straight-line code) ahead of the first request: what a
    // preamble of that length costs when the instructions have to be fetched first
    uint32_t k = (uint32_t)iters;
    asm volatile(".rept 256\n\ts_add_u32 %0, %0, 0x12345\n\t.endr" : "+s"(k));
    if (k == 77u) stamps[1 << 17] = k;
  }
  uint64_t t[6];
  t[0] = __builtin_amdgcn_s_memrealtime();
  const unsigned char* base = p + (int64_t)blockIdx.x * 131072;
  const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<unsigned char*>(base), 0, 131072u, 0x00020000);
  uint32_t lane_off;
  if (PATTERN == 0) {
    lane_off = (uint32_t)wave * 1024u + lane * 16u;
  } else {
    const int row = 4 * wave + (lane >> 4);
    lane_off = (uint32_t)row * 2048u + (uint32_t)(((lane & 15) ^ (row & 15)) * 16);
  }
  uint64_t ti[4];
#pragma unroll
  for (int u = 0; u < 32; ++u) {
    const uint32_t so = PATTERN == 0 ? (uint32_t)u * 4096u : (uint32_t)(u >> 3) * 32768u + (uint32_t)(u & 7) * 256u;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void*)(lds + (wave + 4 * u) * 1024), 16, lane_off, so, 0, 2);
    if (u == 0) ti[0] = __builtin_amdgcn_s_memrealtime();
    if (u == 1) ti[1] = __builtin_amdgcn_s_memrealtime();
    if (u == 7) ti[2] = __builtin_amdgcn_s_memrealtime();
    if (u == 15) ti[3] = __builtin_amdgcn_s_memrealtime();
  }
  t[1] = __builtin_amdgcn_s_memrealtime();
  __builtin_amdgcn_s_waitcnt(0x4F78);       // vmcnt(24)
  t[2] = __builtin_amdgcn_s_memrealtime();
  __builtin_amdgcn_s_waitcnt(0x4F70);       // vmcnt(16)
  t[3] = __builtin_amdgcn_s_memrealtime();
  __builtin_amdgcn_s_waitcnt(0x0F78);       // vmcnt(8)
  t[4] = __builtin_amdgcn_s_memrealtime();
  __builtin_amdgcn_s_waitcnt(0x0F70);       // vmcnt(0)
  t[5] = __builtin_amdgcn_s_memrealtime();
  if (lane == 0) {
    for (int i = 0; i < 6; ++i) stamps[((int64_t)blockIdx.x * 4 + wave) * 10 + i] = t[i];
    for (int i = 0; i < 4; ++i) stamps[((int64_t)blockIdx.x * 4 + wave) * 10 + 6 + i] = ti[i];
  }
}

// What feeding the matrix cores costs (the prefill kernels' bound): a
// wavefront runs `iters` groups of eight MFMAs; per group it also issues LOADS
// 1 KB loads into registers (16 bytes a lane, from a window that stays in L2)
// and LDSR 1 KB LDS reads.  The loaded registers are the A operands of a group
// five groups later, as in a kernel that prefetches.  KIND 0: bf16 32x32x16;
// 1: the block-scaled 32x32x64 FP6 x FP4 form.  Lane 0 of every wavefront
// reports the constant-clock (100 MHz) and shader-clock time of the loop.
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(8))) int i32x8_t;

template <int LOADS, int LDSR, int KIND, int DMA = 0>
__global__ void mfma_feed_kernel(const unsigned char* __restrict__ p, uint64_t* out, int iters, uint32_t* sink) {
  extern __shared__ unsigned char lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<unsigned char*>(p) + (int64_t)(blockIdx.x & 63) * 262144, 0, 262144u, 0x00020000);
  constexpr int NB = LOADS > 0 ? LOADS : 1;
  // The loaded registers are used DEPTH - 1 groups after they were asked for
  // (about 1300 clocks of matrix work: more than L2's latency), in a loop
  // unrolled DEPTH times so that the buffers keep static names.
  constexpr int DEPTH = 6;
  u32x4 buf[DEPTH][NB];
  for (int d = 0; d < DEPTH; ++d)
    for (int j = 0; j < NB; ++j) buf[d][j] = u32x4{0x3f803f80u + (uint32_t)lane, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
  u32x4 lv = {0u, 0u, 0u, 0u};
  f32x16_t acc[2];
  for (int t = 0; t < 2; ++t)
    for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;
  bf16x8_t bop;
  for (int i = 0; i < 8; ++i) bop[i] = (__bf16)1.0f;
  const i32x8_t b8 = {0x22222222 + lane, 0x22222222, 0x22222222, 0x22222222, 0, 0, 0, 0};
  const uint32_t lane_off = (uint32_t)wave * 65536u + (uint32_t)lane * 16u;
  const uint64_t c0 = __builtin_amdgcn_s_memtime(), t0 = __builtin_amdgcn_s_memrealtime();
  // (the loop has no side effects of its own: tie it between the two clock reads)
  asm volatile("" : "+v"(acc[0][0]), "+v"(acc[1][0]) : "s"(c0), "s"(t0));
  for (int it = 0; it < iters; it += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
#pragma unroll
      for (int j = 0; j < LOADS; ++j)
        buf[d][j] = __builtin_amdgcn_raw_buffer_load_b128(r, lane_off + (uint32_t)(j * 1024), (uint32_t)(((it + d) & 7) * 8192), 0);
      // (DMA: as many 1 KB loads straight into LDS instead, at most three
      // groups' worth outstanding)
#pragma unroll
      for (int j = 0; j < DMA; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void*)(lds + ((wave * 16 + (d & 3) * 4 + (j & 3)) * 1024) % 65536), 16,
                                                 lane_off + (uint32_t)(j * 1024), (uint32_t)(((it + d) & 7) * 8192), 0, 0);
      if (DMA) __builtin_amdgcn_s_waitcnt(0x0F70 | ((3 * DMA) & 0xF) | (((3 * DMA) >> 4) << 14));
#pragma unroll
      for (int m = 0; m < 8; ++m) {
        const u32x4 a = buf[(d + 1) % DEPTH][m % NB];             // the oldest buffer
        if constexpr (KIND == 0) {
          acc[m & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), bop, acc[m & 1], 0, 0, 0);
        } else {
          // (the eight-register operand is two loads' registers side by side: no copies)
          const u32x4 a2 = buf[(d + 1) % DEPTH][(m + 1) % NB];
          const i32x8_t a8 = {(int)a[0], (int)a[1], (int)a[2], (int)a[3], (int)a2[0], (int)a2[1], (int)a2[2], (int)a2[3]};
          acc[m & 1] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, acc[m & 1], 2, 4, 0, 127, 0, 127);
        }
        if (m < LDSR / 2) {
#pragma unroll
          for (int q = 0; q < 2; ++q)
            lv ^= *reinterpret_cast<const u32x4*>(lds + ((wave * 16 + m * 2 + q) * 1024 + lane * 16) % 65536);
        }
      }
    }
  }
  asm volatile("" : "+v"(acc[0][0]), "+v"(acc[1][0]), "+v"(buf[0][0][0]), "+v"(buf[DEPTH - 1][0][0]));
  const uint64_t c1 = __builtin_amdgcn_s_memtime(), t1 = __builtin_amdgcn_s_memrealtime();
  float v = 0.f;
  for (int t = 0; t < 2; ++t)
    for (int i = 0; i < 16; ++i) v += acc[t][i];
  if (v == 12345.678f && (lv[0] ^ lv[3]) == 77u) sink[0] = 1u;
  if (lane == 0) {
    out[((int64_t)blockIdx.x * (blockDim.x >> 6) + wave) * 2] = t1 - t0;
    out[((int64_t)blockIdx.x * (blockDim.x >> 6) + wave) * 2 + 1] = c1 - c0;
  }
}

__global__ void empty_kernel(uint32_t* sink) {
  extern __shared__ unsigned char lds[];
  if (sink && threadIdx.x == 0xFFFFFF) sink[0] = lds[0];
}

}  // namespace

extern "C" {

// 0 on success, else the hipError_t.  bytes must be a multiple of 16 * blocks.
int probe_read(const void* p, int64_t bytes, void* sink, int blocks, int threads, int unroll,
               int lds_bytes, void* stream) {
  const int64_t pieces = bytes / 16 / blocks;
  hipStream_t st = static_cast<hipStream_t>(stream);
  auto launch = [&](auto kern) {
    if (lds_bytes > 65536)
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(threads), lds_bytes, st,
                       static_cast<const u32x4*>(p), pieces, static_cast<uint32_t*>(sink));
  };
  if (unroll >= 8) launch(read_kernel<8>);
  else if (unroll >= 4) launch(read_kernel<4>);
  else if (unroll >= 2) launch(read_kernel<2>);
  else launch(read_kernel<1>);
  return (int)hipGetLastError();
}

// The workgroup's share (bytes / blocks, a multiple of 1 KB, at most 128 KB and, with dma, at most
// lds_bytes) requested by `active` in {4, 8, 12} wavefronts.  nt = the loads carry the non-temporal hint.
int probe_loaders(const void* p, int64_t bytes, void* sink, int blocks, int threads, int active, int dma,
                  int nt, int lds_bytes, void* stream) {
  const int chunks = (int)(bytes / blocks / 1024);
  if (chunks > 128 || (dma && chunks * 1024 > lds_bytes) || active * 64 > threads) return -1;
  hipStream_t st = static_cast<hipStream_t>(stream);
  auto launch = [&](auto kern) {
    if (lds_bytes > 65536)
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(threads), lds_bytes, st,
                       static_cast<const unsigned char*>(p), chunks, active, static_cast<uint32_t*>(sink));
  };
  auto pick = [&](auto u) {
    constexpr int U = decltype(u)::value;
    if (dma) { if (nt) launch(loaders_kernel<U, true, 2>); else launch(loaders_kernel<U, true, 0>); }
    else     { if (nt) launch(loaders_kernel<U, false, 2>); else launch(loaders_kernel<U, false, 0>); }
  };
  if (active == 4) pick(std::integral_constant<int, 32>());
  else if (active == 8) pick(std::integral_constant<int, 16>());
  else if (active == 12) pick(std::integral_constant<int, 11>());
  else return -1;
  return (int)hipGetLastError();
}

// 256 workgroups of 768 threads over 32 MiB at p; stamps: uint64 [256][4][10] (the six above, then after the
// 1st, 2nd, 8th and 16th request was issued); at least 1 MiB, its tail is the bystanders' sink.
int probe_stamped_loaders(const void* p, void* stamps, int pattern, int busy, int iters, void* stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  auto launch = [&](auto kern) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                              147456);
    hipLaunchKernelGGL(kern, dim3(256), dim3(768), 147456, st, static_cast<const unsigned char*>(p),
                       static_cast<uint64_t*>(stamps), busy, iters);
  };
  if (pattern) launch(stamped_loaders_kernel<1>); else launch(stamped_loaders_kernel<0>);
  return (int)hipGetLastError();
}

// 256 workgroups of `waves` wavefronts (4: one a SIMD, 8: two); `loads` in {0, 2, 4, 8} register loads and
// `lds_reads` in {0, 8, 16} LDS reads of 1 KB per group of eight MFMAs of `kind` (0 bf16, 1 block-scaled FP6 x FP4;
// + 100: the loads go straight into LDS, with 8 LDS reads);
// p: at least 16 MiB; out: uint64 [256 * waves][2] = (10 ns ticks, shader clocks) of the loop.
int probe_mfma_feed(const void* p, void* out, void* sink, int waves, int loads, int lds_reads, int kind, int iters,
                    void* stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (waves != 4 && waves != 8) return -1;
  auto launch = [&](auto kern) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
    hipLaunchKernelGGL(kern, dim3(256), dim3(64 * waves), 65536, st, static_cast<const unsigned char*>(p),
                       static_cast<uint64_t*>(out), iters, static_cast<uint32_t*>(sink));
  };
  const int key = (kind >= 100 ? 1000000 : 0) + (kind % 100) * 10000 + loads * 100 + lds_reads;
  switch (key) {
    case 0: launch(mfma_feed_kernel<0, 0, 0>); break;
    case 200: launch(mfma_feed_kernel<2, 0, 0>); break;
    case 400: launch(mfma_feed_kernel<4, 0, 0>); break;
    case 800: launch(mfma_feed_kernel<8, 0, 0>); break;
    case 8: launch(mfma_feed_kernel<0, 8, 0>); break;
    case 16: launch(mfma_feed_kernel<0, 16, 0>); break;
    case 816: launch(mfma_feed_kernel<8, 16, 0>); break;
    case 10000: launch(mfma_feed_kernel<0, 0, 1>); break;
    case 10200: launch(mfma_feed_kernel<2, 0, 1>); break;
    case 10400: launch(mfma_feed_kernel<4, 0, 1>); break;
    case 10800: launch(mfma_feed_kernel<8, 0, 1>); break;
    case 10008: launch(mfma_feed_kernel<0, 8, 1>); break;
    case 1000208: launch(mfma_feed_kernel<0, 8, 0, 2>); break;      // + 1000000: the loads go straight into LDS
    case 1000408: launch(mfma_feed_kernel<0, 8, 0, 4>); break;
    case 1000808: launch(mfma_feed_kernel<0, 8, 0, 8>); break;
    case 1010208: launch(mfma_feed_kernel<0, 8, 1, 2>); break;
    case 1010408: launch(mfma_feed_kernel<0, 8, 1, 4>); break;
    default: return -1;
  }
  return (int)hipGetLastError();
}

int probe_empty(void* sink, int blocks, int threads, int lds_bytes, void* stream) {
  if (lds_bytes > 65536)
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(empty_kernel),
                              hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
  hipLaunchKernelGGL(empty_kernel, dim3(blocks), dim3(threads), lds_bytes,
                     static_cast<hipStream_t>(stream), static_cast<uint32_t*>(sink));
  return (int)hipGetLastError();
}

}  // extern "C"
