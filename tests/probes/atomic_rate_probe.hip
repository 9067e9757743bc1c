// Probe: throughput of fp32 global atomic adds (vector memory instructions, no return value) for the access
// pattern a single-kernel attention backward would have: every workgroup (512 threads = 8 waves) adds, per
// interval, a 64 x 128 fp32 dQ tile (each wave one 32 x 32 block, 16 instructions) into dQ[Sq, Hq, 128] fp32, with
// the dK/dV kernel's workgroup -> (key block, kv head, head part) mapping, alone and next to that kernel's matrix
// load. The sums are verified. It answers whether accumulating dQ by atomics could replace the second backward
// kernel: the recomputation such a kernel would save takes 0.45 ms per launch at this shape.
// Built by tests/probes/build_probes.py, run by tests/test_probes_gpu.py; never part of the library.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <vector>
#include <cstring>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("HIP error %s at %d\n", hipGetErrorString(e), __LINE__); exit(1);} }while(0)

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

struct P {
  float* dq;       // [Sq][Hq][128]
  unsigned* xcc;   // [grid] XCC id seen by each block
  int Sq, Hq, Hkv, split, group, n_tiles;
  int mapping;     // 0: linear = n_tile*per_level + (hk*split+part) (dkdv kernel's), 1: linear = (hk*split+part)*n_tiles + n_tile
  int stagger;     // start q tile rotated by n_tile
  int n_mfma;      // filler MFMAs per wave and interval
  int do_atomic;
  int q_rows;      // rows per interval (64 or 128)
};

template <int SC1>
__device__ __forceinline__ void atomic_add_f32(float* base, int byte_off, float v) {
  if (SC1) asm volatile("global_atomic_add_f32 %0, %1, %2 sc1" : : "v"(byte_off), "v"(v), "s"(base) : "memory");
  else asm volatile("global_atomic_add_f32 %0, %1, %2" : : "v"(byte_off), "v"(v), "s"(base) : "memory");
}

template <int SC1>
__global__ __launch_bounds__(512) void probe(P p) {
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, g = lane >> 5;
  const int per_level = p.Hkv * p.split;
  int n_tile, pos;
  if (p.mapping == 0) { n_tile = blockIdx.x / per_level; pos = blockIdx.x % per_level; }
  else { pos = blockIdx.x / p.n_tiles; n_tile = blockIdx.x % p.n_tiles; }
  const int part = pos % p.split, hk = pos / p.split;
  const int heads_per_part = p.group / p.split;
  const int hq0 = hk * p.group + part * heads_per_part;
  if (tid == 0) p.xcc[blockIdx.x] = __builtin_amdgcn_s_getreg((31 << 11) | 20);
  const int m_tiles = p.Sq / p.q_rows;
  const int row_bytes = p.Hq * 128 * 4;
  // wave's 32x32 block of the (q_rows x 128) tile: q_rows=64 -> 2x4 blocks, one per wave;
  // q_rows=128 -> 4x4 blocks, two per wave
  f32x16 acc;
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;
  bf16x8 a, b;
  for (int e = 0; e < 8; ++e) { a[e] = (__bf16)(0.001f * (lane + e)); b[e] = (__bf16)(0.002f * (lane - e)); }
  const int m0 = p.stagger ? (n_tile * 4) % m_tiles : 0;
  for (int h = 0; h < heads_per_part; ++h) {
    const int hq = hq0 + h;
    for (int mi = 0; mi < m_tiles; ++mi) {
      int mt = mi + m0; if (mt >= m_tiles) mt -= m_tiles;
      for (int i = 0; i < p.n_mfma; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
      if (p.do_atomic) {
        const int blocks = p.q_rows / 64;
        for (int bb = 0; bb < blocks; ++bb) {
          const int rb = (wave >> 2) + 2 * bb, ob = wave & 3;
          float* base = p.dq + ((size_t)(mt * p.q_rows + rb * 32) * p.Hq + hq) * 128 + ob * 32;
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int row = 8 * (v >> 2) + 4 * g + (v & 3);
            atomic_add_f32<SC1>(base, row * row_bytes + c * 4, 1.0f);
          }
        }
      }
    }
  }
  if (acc[0] == 123.456f) p.dq[0] = acc[1];  // keep the MFMAs alive
}

int main(int argc, char** argv) {
  const int Sq = 8192, Hq = 32, Hkv = 4, group = 8, split = 4, Skv = 4096;
  float* dq; unsigned* xcc;
  const size_t n = (size_t)Sq * Hq * 128;
  CK(hipMalloc(&dq, n * 4));
  std::vector<float> host(n);
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  struct Cfg { const char* name; int sc1, mapping, stagger, n_mfma, do_atomic, kv_per_wg, q_rows; };
  const Cfg cfgs[] = {
    {"atomics only, system scope, dkdv mapping", 1, 0, 0, 0, 1, 128, 64},
    {"atomics only, device scope, dkdv mapping", 0, 0, 0, 0, 1, 128, 64},
    {"atomics only, device scope, staggered start", 0, 0, 1, 0, 1, 128, 64},
    {"atomics only, system scope, scattered mapping", 1, 1, 0, 0, 1, 128, 64},
    {"mfma only (40 per wave-interval)", 0, 0, 0, 40, 0, 128, 64},
    {"mfma 40 + atomics, device scope", 0, 0, 0, 40, 1, 128, 64},
    {"256 keys per workgroup: atomics only, device scope", 0, 0, 1, 0, 1, 256, 64},
    {"256 keys per workgroup: mfma 80 + atomics, device scope", 0, 0, 1, 80, 1, 256, 64},
  };
  for (const Cfg& c : cfgs) {
    P p; p.dq = dq; p.Sq = Sq; p.Hq = Hq; p.Hkv = Hkv; p.split = split; p.group = group;
    p.n_tiles = Skv / c.kv_per_wg; p.mapping = c.mapping; p.stagger = c.stagger; p.n_mfma = c.n_mfma;
    p.do_atomic = c.do_atomic; p.q_rows = c.q_rows;
    const int grid = p.n_tiles * Hkv * split;
    CK(hipMalloc(&xcc, grid * 4));
    p.xcc = xcc;
    float best = 1e9;
    const int reps = 3;
    CK(hipMemset(dq, 0, n * 4));
    for (int r = 0; r < reps + 1; ++r) {
      if (r == 1) CK(hipMemset(dq, 0, n * 4));
      CK(hipEventRecord(e0));
      if (c.sc1) hipLaunchKernelGGL(probe<1>, dim3(grid), dim3(512), 0, 0, p);
      else hipLaunchKernelGGL(probe<0>, dim3(grid), dim3(512), 0, 0, p);
      CK(hipEventRecord(e1));
      CK(hipEventSynchronize(e1));
      float ms; CK(hipEventElapsedTime(&ms, e0, e1));
      if (r > 0 && ms < best) best = ms;
    }
    CK(hipMemcpy(host.data(), dq, n * 4, hipMemcpyDeviceToHost));
    // every element receives n_tiles adds per launch, `reps` timed launches
    const float want = c.do_atomic ? (float)(p.n_tiles * reps) : 0.f;
    size_t bad = 0; for (size_t i = 0; i < n; ++i) bad += host[i] != want;
    std::vector<unsigned> hx(grid); CK(hipMemcpy(hx.data(), xcc, grid * 4, hipMemcpyDeviceToHost));
    int rr = 0; for (int i = 0; i < grid; ++i) rr += (hx[i] & 15) == (unsigned)(i % 8);
    const double bytes = c.do_atomic ? (double)grid * (group / split) * (Sq / c.q_rows) * c.q_rows * 128 * 4 : 0;
    printf("%-58s grid %4d  %8.3f ms  atomic %7.1f GB/s  wrong elements %zu  blocks with xcc==id%%8: %d/%d\n", c.name, grid, best,
           bytes / best * 1e-6, bad, rr, grid);
    fflush(stdout);
    CK(hipFree(xcc));
  }
  return 0;
}
