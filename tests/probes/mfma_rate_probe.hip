// Probe: the sustained full-chip rate of v_mfma_f32_32x32x16_bf16 issued from registers (2 waves per SIMD, 4
// independent accumulators per wave, no LDS, no memory traffic, no vector arithmetic), as a function of the operand
// DATA: constants, one random fragment pair, rotating random fragments. It measures the ceiling that any bf16
// attention kernel on this device works under: the chip is power-limited, and the power of a matrix instruction
// depends on how many operand bits toggle. Output: one line per (data, fragments, workgroups) with milliseconds,
// TFLOP/s, cycles per instruction as seen by one wave, and the shader clock derived from it.
// Built by tests/probes/build_probes.py, run by tests/test_probes_gpu.py; never part of the library.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cstdint>
#include <vector>
#include <cmath>
#include <cstring>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("HIP error %s at %d\n", hipGetErrorString(e), __LINE__); exit(1);} }while(0)
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

// NF = number of distinct A / B fragments cycled through; data from `src` (per-lane distinct)
template <int NF>
__global__ __launch_bounds__(512) void k_mfma(const bf16x8* __restrict__ src, float* out, long long* cyc, int iters) {
  bf16x8 a[NF], b[NF];
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    a[f] = src[(f * 2) * 64 + lane + (threadIdx.x >> 6) * 1024];
    b[f] = src[(f * 2 + 1) * 64 + lane + (threadIdx.x >> 6) * 1024];
  }
  f32x16 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
  const long long t0 = __builtin_readcyclecounter();
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[f], b[f], c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(f + 1) % NF], b[f], c1, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[f], b[(f + 1) % NF], c2, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(f + 1) % NF], b[(f + 1) % NF], c3, 0, 0, 0);
    }
  }
  const long long t1 = __builtin_readcyclecounter();
  float s = 0;
  for (int v = 0; v < 16; ++v) s += c0[v] + c1[v] + c2[v] + c3[v];
  if (s == 1.2345f) out[0] = s;
  if (threadIdx.x == 0 && blockIdx.x == 0) cyc[0] = t1 - t0;
}

static uint16_t f2bf(float f) { uint32_t u; memcpy(&u, &f, 4); u += 0x7fff + ((u >> 16) & 1); return u >> 16; }

int main() {
  const size_t n = 8 * 1024 * 8;  // 8 waves x 1024 fragments-slots x 8 elems
  std::vector<uint16_t> h(n);
  float* out; long long* cyc; uint16_t* d;
  CK(hipMalloc(&out, 64)); CK(hipMalloc(&cyc, 64)); CK(hipMalloc(&d, n * 2));
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  const char* names[3] = {"constants (1.0 / 0.5)", "random normal * 0.1", "random normal (unit)"};
  for (int mode = 0; mode < 3; ++mode) {
    srand(1);
    for (size_t i = 0; i < n; ++i) {
      float u1 = (rand() + 1.0f) / (RAND_MAX + 2.0f), u2 = (rand() + 1.0f) / (RAND_MAX + 2.0f);
      float g = sqrtf(-2 * logf(u1)) * cosf(6.2831853f * u2);
      h[i] = mode == 0 ? f2bf((i / 512) % 2 ? 0.5f : 1.0f) : f2bf(mode == 1 ? g * 0.1f : g);
    }
    CK(hipMemcpy(d, h.data(), n * 2, hipMemcpyHostToDevice));
    for (int nf : {1, 4, 8}) {
      for (int blocks : {256, 512}) {
        const int iters = 20000 / nf;
        auto launch = [&]() {
          if (nf == 1) hipLaunchKernelGGL(k_mfma<1>, dim3(blocks), dim3(512), 0, 0, (const bf16x8*)d, out, cyc, iters);
          else if (nf == 4) hipLaunchKernelGGL(k_mfma<4>, dim3(blocks), dim3(512), 0, 0, (const bf16x8*)d, out, cyc, iters);
          else hipLaunchKernelGGL(k_mfma<8>, dim3(blocks), dim3(512), 0, 0, (const bf16x8*)d, out, cyc, iters);
        };
        launch(); CK(hipDeviceSynchronize());
        CK(hipEventRecord(e0)); launch(); launch(); launch(); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
        float ms; CK(hipEventElapsedTime(&ms, e0, e1)); ms /= 3;
        long long c; CK(hipMemcpy(&c, cyc, 8, hipMemcpyDeviceToHost));
        const double flops = (double)blocks * 8 * 4.0 * nf * iters * 32768.0;
        // one block per CU when blocks == 256: 8 waves, 2 per SIMD -> 8 * 4 * nf * iters MFMAs / 4 SIMDs * 32 cycles
        printf("%-24s fragments %d blocks %d: %.3f ms  %.0f TFLOP/s  (wave 0: %.1f cycles per MFMA of its SIMD, clock %.2f GHz)\n", names[mode], nf, blocks, ms,
               flops / ms * 1e-9, (double)c / (2.0 * 4 * nf * iters), blocks == 256 ? (double)c / (ms * 1e6) : 0.0);
        fflush(stdout);
      }
    }
  }
  return 0;
}
