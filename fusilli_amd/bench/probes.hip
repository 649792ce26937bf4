// Stand-alone probes of two gfx950 facts the kernels are built around:
//
//  1. the per-CU rate of the three ways of bringing global memory into a
//     workgroup (LDS-DMA buffer loads, loads to registers, loads to registers
//     followed by LDS writes), on a cache-resident and on an HBM-sized window;
//  2. how matrix (MFMA) and vector instructions share a SIMD: from two
//     wavefronts of one SIMD, and inside ONE wavefront's instruction stream
//     (softmax-like arithmetic placed between MFMAs, with and without LDS
//     reads).
//
// Build: `make -C fusilli_amd/bench` (bin/probes); needs no library.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <vector>

#define AS3 __attribute__((address_space(3)))
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t mk_rsrc(const void *base, uint32_t bytes) {
  const uint64_t b64 = (uint64_t)base;
  const uint32_t blo = __builtin_amdgcn_readfirstlane((uint32_t)b64);
  const uint32_t bhi = __builtin_amdgcn_readfirstlane((uint32_t)(b64 >> 32));
  return __builtin_amdgcn_make_buffer_rsrc((void *)(((uint64_t)bhi << 32) | blo), 0,
                                           (int)__builtin_amdgcn_readfirstlane(bytes), 0x00020000);
}
constexpr int wait_imm(int vm) { return (vm & 0xF) | ((vm >> 4) << 14) | (0x7 << 4) | (0x0 << 8); }

// ---- 1. load paths -----------------------------------------------------------
// MODE 0: LDS-DMA, 1: loads to registers, 2: loads to registers + LDS writes.
// Every wavefront instruction moves 1 KB of contiguous memory; a workgroup
// cycles through `region` bytes.
template <int MODE, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void load_probe(const char *src, uint32_t region, int iters,
                                                         uint64_t *clk, uint32_t *sink) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int l = threadIdx.x & 63;
  const uint32_t slice = region / WAVES;
  const __amdgpu_buffer_rsrc_t rs = mk_rsrc(src + (size_t)blockIdx.x * region + wave * slice, slice);
  const uint32_t wlds = lds0 + wave * 8192;
  u32x4 acc = {0, 0, 0, 0};
  __syncthreads();
  const uint64_t t0 = __builtin_amdgcn_s_memtime();
  uint32_t off = 0;
  for (int it = 0; it < iters; ++it) {
    if (MODE == 0) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rs, (AS3 char *)__builtin_amdgcn_readfirstlane(wlds + j * 1024), 16, l * 16,
            off + j * 1024, 0, 0);
      __builtin_amdgcn_s_waitcnt(wait_imm(8));
    } else {
      u32x4 v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        v[j] = __builtin_amdgcn_raw_buffer_load_b128(rs, l * 16, off + j * 1024, 0);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (MODE == 2)
          *(AS3 u32x4 *)(uintptr_t)(wlds + j * 1024 + l * 16) = v[j];
        else
          acc ^= v[j];
      }
    }
    off += 8192;
    if (off >= slice)
      off = 0;
  }
  __builtin_amdgcn_s_waitcnt(wait_imm(0));
  __syncthreads();
  const uint64_t t1 = __builtin_amdgcn_s_memtime();
  if (threadIdx.x == 0)
    clk[blockIdx.x] = t1 - t0;
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u)
    sink[0] = acc[0];
}

template <int MODE, int WAVES>
void run_load(const char *name, const char *src, uint32_t region, uint64_t *clk, uint32_t *sink) {
  const int iters = 400;
  hipFuncSetAttribute((const void *)load_probe<MODE, WAVES>,
                      hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
  hipEvent_t e0, e1;
  hipEventCreate(&e0);
  hipEventCreate(&e1);
  for (int rep = 0; rep < 3; ++rep) {
    hipEventRecord(e0);
    hipLaunchKernelGGL((load_probe<MODE, WAVES>), dim3(256), dim3(WAVES * 64), 65536, 0, src, region,
                       iters, clk, sink);
    hipEventRecord(e1);
    hipEventSynchronize(e1);
  }
  float ms;
  hipEventElapsedTime(&ms, e0, e1);
  std::vector<uint64_t> h(256);
  hipMemcpy(h.data(), clk, 256 * 8, hipMemcpyDeviceToHost);
  double avg = 0;
  for (auto c : h)
    avg += c;
  avg /= 256;
  const double bytes_cu = (double)iters * 8192 * WAVES;
  printf("load path %-24s %d wavefronts, window %5u KB per CU: %6.1f B/clk per CU, %6.2f TB/s\n", name,
         WAVES, region / 1024, bytes_cu / avg, bytes_cu * 256 / (ms * 1e-3) / 1e12);
}

// ---- 2a. two wavefronts of a SIMD: A issues MFMAs, B softmax-like arithmetic ----
template <int RA, int RB>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void
pair_probe(int iters, uint64_t *clk, float *sink, float seed) {
  const int wave = threadIdx.x >> 6;
  const bool mfma = wave < 4 ? RA == 1 : RB == 2;
  const bool valu = wave >= 4 && RB == 1;
  f32x16 acc0 = {}, acc1 = {};
  u32x4 a = {0x3f803f80u + threadIdx.x, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
  u32x4 b = {0x3f803f80u, 0x3f803f80u + threadIdx.x, 0x3f803f80u, 0x3f803f80u};
  float s[32];
#pragma unroll
  for (int i = 0; i < 32; ++i)
    s[i] = seed * (i + 1) + threadIdx.x * 1e-3f;
  float sum = 0.f, mx = -1e30f;
  uint32_t pk = 0;
  __syncthreads();
  const uint64_t t0 = __builtin_amdgcn_s_memtime();
  if (mfma) {
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                      __builtin_bit_cast(bf16x8, b), acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, b),
                                                      __builtin_bit_cast(bf16x8, a), acc1, 0, 0, 0);
      }
    }
  } else if (valu) {
    // 32 scores: maximum, scale-and-shift, exp2, sum, pairs packed to bf16
    for (int it = 0; it < iters; ++it) {
      float p[32];
#pragma unroll
      for (int i = 0; i < 32; i += 2)
        mx = __builtin_fmaxf(mx, __builtin_fmaxf(s[i], s[i + 1]));
      const float m2 = mx * 0.125f;
#pragma unroll
      for (int i = 0; i < 32; ++i) {
        p[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], 0.125f, -m2));
        sum += p[i];
      }
#pragma unroll
      for (int i = 0; i < 32; i += 2) {
        typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
        typedef float f2 __attribute__((ext_vector_type(2)));
        const bf2 c = __builtin_convertvector(f2{p[i], p[i + 1]}, bf2);
        pk ^= __builtin_bit_cast(uint32_t, c);
      }
#pragma unroll
      for (int i = 0; i < 32; ++i)
        s[i] = p[i] * 0.5f;
    }
  }
  const uint64_t t1 = __builtin_amdgcn_s_memtime();
  if ((threadIdx.x & 63) == 0)
    clk[blockIdx.x * 8 + wave] = t1 - t0;
  float r = sum + mx + __builtin_bit_cast(float, pk & 0x3fffffffu);
#pragma unroll
  for (int i = 0; i < 16; ++i)
    r += acc0[i] + acc1[i];
#pragma unroll
  for (int i = 0; i < 32; ++i)
    r += s[i];
  if (r == 12345.678f)
    sink[0] = r;
}

template <int RA, int RB> void run_pair(const char *name, uint64_t *clk, float *sink) {
  const int iters = 2000;
  for (int rep = 0; rep < 2; ++rep) {
    hipLaunchKernelGGL((pair_probe<RA, RB>), dim3(256), dim3(512), 0, 0, iters, clk, sink, 0.37f);
    hipDeviceSynchronize();
  }
  std::vector<uint64_t> h(256 * 8);
  hipMemcpy(h.data(), clk, h.size() * 8, hipMemcpyDeviceToHost);
  double a = 0, b = 0;
  for (int g = 0; g < 256; ++g)
    for (int w = 0; w < 8; ++w)
      (w < 4 ? a : b) += h[g * 8 + w];
  printf("two wavefronts per SIMD, %-34s A %7.1f clk per 32 MFMAs, B %7.1f clk per 32 scores\n", name,
         a / 1024 / iters, b / 1024 / iters);
}

// ---- 2b. one wavefront per SIMD: NE exponentials (scale, exp2, sum, half a pack;
// stages 8 elements apart, so nothing waits for the instruction before it)
// between consecutive MFMAs, optionally one 16-byte LDS read per MFMA ----------
template <int NE, bool MFMA, bool LDSR>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void
stream_probe(int iters, uint64_t *clk, float *sink, float seed) {
  __shared__ __attribute__((aligned(16))) char smem[16384];
  f32x16 acc[4] = {};
  u32x4 a = {0x3f803f80u + threadIdx.x, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
  u32x4 b = {0x3f803f80u, 0x3f803f80u + threadIdx.x, 0x3f803f80u, 0x3f803f80u};
  float s[64], p[64];
#pragma unroll
  for (int i = 0; i < 64; ++i) {
    s[i] = seed * (i + 1) + threadIdx.x * 1e-3f;
    p[i] = 0.f;
  }
  float sum0 = 0.f, sum1 = 0.f;
  uint32_t pk = 0;
  u32x4 fr[4] = {};
  const uint32_t laddr = (uint32_t)(uintptr_t)smem + (threadIdx.x & 63) * 16;
  __syncthreads();
  const uint64_t t0 = __builtin_amdgcn_s_memtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int m = 0; m < 32; ++m) {
      if (LDSR) {
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(fr[m & 3]) : "v"(laddr), "n"(1024));
        asm volatile("s_waitcnt lgkmcnt(3)" ::: "memory");
      }
      if (MFMA) {
        const u32x4 aa = LDSR ? fr[(m + 1) & 3] : a;
        acc[m & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            __builtin_bit_cast(bf16x8, aa), __builtin_bit_cast(bf16x8, b), acc[m & 3], 0, 0, 0);
      }
#pragma unroll
      for (int u = 0; u < NE; ++u) {
        const int i = (m * NE + u) & 63, j = (m * NE + u + 56) & 63, k = (m * NE + u + 48) & 63;
        s[i] = __builtin_fmaf(s[i], 0.125f, -seed);
        p[j] = __builtin_amdgcn_exp2f(s[j]);
        if (u & 1) {
          sum1 += p[k];
          typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
          typedef float f2 __attribute__((ext_vector_type(2)));
          const bf2 c = __builtin_convertvector(f2{p[k], p[(k + 63) & 63]}, bf2);
          pk ^= __builtin_bit_cast(uint32_t, c);
        } else {
          sum0 += p[k];
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  const uint64_t t1 = __builtin_amdgcn_s_memtime();
  if ((threadIdx.x & 63) == 0)
    clk[blockIdx.x * 4 + (threadIdx.x >> 6)] = t1 - t0;
  float r = sum0 + sum1 + __builtin_bit_cast(float, pk & 0x3fffffffu) +
            __builtin_bit_cast(float, fr[0].x & 0x3fffffffu);
#pragma unroll
  for (int i = 0; i < 16; ++i)
    r += acc[0][i] + acc[1][i] + acc[2][i] + acc[3][i];
#pragma unroll
  for (int i = 0; i < 64; ++i)
    r += s[i] + p[i];
  if (r == 12345.678f)
    sink[0] = r;
}

template <int NE, bool MFMA, bool LDSR> void run_stream(uint64_t *clk, float *sink) {
  const int iters = 1000;
  for (int rep = 0; rep < 2; ++rep) {
    hipLaunchKernelGGL((stream_probe<NE, MFMA, LDSR>), dim3(256), dim3(256), 0, 0, iters, clk, sink,
                       0.37f);
    hipDeviceSynchronize();
  }
  std::vector<uint64_t> h(256 * 4);
  hipMemcpy(h.data(), clk, h.size() * 8, hipMemcpyDeviceToHost);
  double a = 0;
  for (auto c : h)
    a += c;
  printf("one wavefront per SIMD, per slot: %d exponentials%s%s: %6.1f clk\n", NE,
         MFMA ? " + 1 MFMA 32x32x16" : "", LDSR ? " + 1 LDS read" : "", a / 1024 / iters / 32);
}

int main() {
  const size_t total = (size_t)256 * (4 << 20);
  char *src;
  uint64_t *clk;
  uint32_t *sink;
  hipMalloc(&src, total);
  hipMemset(src, 1, total);
  hipMalloc(&clk, 256 * 8 * 8);
  hipMalloc(&sink, 64);
  for (uint32_t region : {65536u, 4u << 20}) {
    run_load<0, 8>("LDS-DMA", src, region, clk, sink);
    run_load<1, 8>("loads to registers", src, region, clk, sink);
    run_load<2, 8>("loads + LDS writes", src, region, clk, sink);
  }
  run_pair<1, 0>("A: MFMA, B: idle", clk, (float *)sink);
  run_pair<0, 1>("A: idle, B: softmax", clk, (float *)sink);
  run_pair<1, 1>("A: MFMA, B: softmax", clk, (float *)sink);
  run_pair<1, 2>("A: MFMA, B: MFMA", clk, (float *)sink);
  run_stream<1, false, false>(clk, (float *)sink);
  run_stream<1, true, false>(clk, (float *)sink);
  run_stream<2, false, false>(clk, (float *)sink);
  run_stream<2, true, false>(clk, (float *)sink);
  run_stream<0, true, true>(clk, (float *)sink);
  run_stream<2, true, true>(clk, (float *)sink);
  return 0;
}
