// Query-gradient kernel for head dims (128, 128) on gfx950 that reads dS instead of recomputing it:
// dQ = scale * dS K (pithtrain/operators/mla/triton.py:205-266, the last product of the loop body),
// with dS = P*(dP - delta) taken, already rounded to bf16, from the images that the dK/dV kernel of
// attn_bwd_dkdv_d128.hip leaves in p.ds (layout documented there). The two score products that the
// other dQ kernels repeat are gone; the price is one trip of dS through memory, so this kernel is
// bound by the rate at which it can stream the images, not by the matrix pipe.
//
// Work split: a workgroup of 8 wavefronts owns 512 query rows of one (batch, head), wave w the 64-row
// query tile 8*m_tile + w. Keys are visited in steps of 32 (one wave pair of the writer). Per step the
// K tile (shared, packed and swizzled like everywhere else, 8 KB) and, per wave, the 4 KB image of its
// tile for that pair (copied verbatim) go global -> LDS directly into a ring of four stages (160 KB),
// requested three steps ahead (two steps in flight while one is in use): what bounds the kernel is how many bytes each compute unit keeps in
// flight, so the stages are sized to spend the LDS on dS rather than on K. dQ^T += K^T dS^T: K^T
// fragments come from transposing reads of the K tile and serve both 32-row blocks of the wave's
// tile, dS^T fragments from transposing reads of the image, in the same key slot order.
#include <type_traits>

#include "attn_bwd_common.h"

namespace pith {
namespace {

constexpr int kThreads = 512;
constexpr int kBM = 512;  // query rows per workgroup (64 per wave)
constexpr int kBN = 32;   // keys per step
constexpr int kD = 128;
constexpr int kStages = 4;                       // power of two; steps s (in use), s+1 .. s+3 (in flight)
constexpr int kKTile = kBN * kRowBytes128;       // 8 KB
constexpr int kDsWave = 4096;                    // per wave and step
constexpr int kStage = kKTile + 8 * kDsWave;     // 40 KB
constexpr int kLoadsK = kBN * 16 / kThreads;     // K tile loads per wave and step (1)
constexpr int kLoadsDs = 4;

// s_waitcnt with vmcnt = n, the other counters left at their maxima (gfx9 encoding: vmcnt in bits
// 3:0 and 15:14).
template <int N>
__device__ __forceinline__ void wait_vector_loads_but() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

template <bool CAUSAL, typename OutT>
__global__ __launch_bounds__(kThreads) void attn_bwd_dq_ds_kernel(BwdParams p) {
  constexpr int DB = kD / 32;
  static_assert(kStages * kStage <= 160 * 1024, "the ring must fit the LDS");
  __shared__ __attribute__((aligned(1024))) char smem[kStages * kStage];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, g = lane >> 5;
  int m_tile, h, b;
  decode_block(blockIdx.x, p.Hq, p.B, p.tiles, m_tile, h, b);
  const int hk = h / p.group;
  const int m0 = m_tile * kBM;
  const int mt = m_tile * 8 + wave;  // this wave's 64-row query tile
  const int q_wave0 = mt * 64;

  const int kv_row_bytes = p.Hkv * kD * 2;
  const char* kh = reinterpret_cast<const char*>(p.k + b * p.k_bs + (int64_t)hk * kD);

  // key steps: all of them, or up to the diagonal; a wave whose query tile does not exist (ragged
  // Sq) has no images and visits nothing
  const int n_steps_all = (p.Skv + kBN - 1) / kBN;
  int n_steps_wg = n_steps_all, n_steps_wave = mt < p.ds_qt ? n_steps_all : 0;
  if (CAUSAL) {
    n_steps_wg = min(n_steps_all, (m0 + kBM - 1) / kBN + 1);
    n_steps_wave = mt < p.ds_qt ? min(n_steps_all, (q_wave0 + 63) / kBN + 1) : 0;
  }

  // images of this wave's query tile: key step s = pair s&3 of key block s>>2, 4 KB each, consecutive in s
  const char* ds_wave = p.ds + (((int64_t)(b * p.Hq + h) * p.ds_qt + (mt < p.ds_qt ? mt : 0)) * p.ds_kb) * (4 * 4096);

  DirectTile128<kBN, kThreads> mover;
  mover.init(kv_row_bytes, wave, lane);
  auto request = [&](int s) __attribute__((always_inline)) {
    char* stage = smem + (s & (kStages - 1)) * kStage;
    mover.issue(kh + (int64_t)s * kBN * kv_row_bytes, p.Skv - s * kBN, stage, wave, lane);
    if (s < n_steps_wave) {
      const char* src = ds_wave + (int64_t)s * 4096;
      char* dst = stage + kKTile + wave * kDsWave;
      int off = lane << 4;
      asm volatile("" : "+v"(off));
#pragma unroll
      for (int j = 0; j < 4; ++j) load_lds16(src + j * 1024, off, dst + j * 1024);
    }
  };
  // loads this wave issued for step t
  auto loads_of = [&](int t) __attribute__((always_inline)) { return t >= n_steps_wg ? 0 : (t < n_steps_wave ? kLoadsK + kLoadsDs : kLoadsK); };
  // waits until this wave's loads for step s have landed. At that point steps s+1 .. s+kStages-2 have
  // been requested as well (step s+kStages-1 follows after the barrier) and may stay in flight.
  auto wait_step = [&](int s) __attribute__((always_inline)) {
    static_assert(kStages == 4, "the list of counts below is for two steps in flight");
    const int n = loads_of(s + 1) + loads_of(s + 2);  // one of 0, 1, 2, 5, 6, 10
    if (n >= 10) wait_vector_loads_but<10>();
    else if (n >= 6) wait_vector_loads_but<6>();
    else if (n >= 5) wait_vector_loads_but<5>();
    else if (n >= 2) wait_vector_loads_but<2>();
    else if (n >= 1) wait_vector_loads_but<1>();
    else wait_vector_loads_but<0>();
  };

  f32x16 acc[2][DB];  // [32-row block of the tile][feature block]
#pragma unroll
  for (int rb = 0; rb < 2; ++rb)
#pragma unroll
    for (int o = 0; o < DB; ++o)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[rb][o][v] = 0.f;

  // per-lane read offsets. K tile: transposing reads of feature block o, lower / upper 8 keys of a
  // 16-key step. Image: this lane supplies, for its 16-lane block (g, chalf) and r = 4i + m, the 8
  // bytes that hold key 4g + i (+ 8 for the upper read) at queries 16*chalf + 4m .. +3 of a 32-row
  // block: 16-row step chalf of the block, writer lane group m&1, fragment half m>>1.
  int t_off[DB][2];
#pragma unroll
  for (int o = 0; o < DB; ++o)
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) t_off[o][hh] = transposed_offset128(0, hh, 32 * o, lane);
  int ds_off[2];
  {
    const int r = lane & 15, chalf = (lane >> 4) & 1;
    const int i = r >> 2, m = r & 3, gl = m & 1;
    const int key = 4 * g + i;
    ds_off[0] = chalf * 1024 + gl * 512 + ((key ^ (gl << 3) ^ (chalf << 2)) << 4) + (m >> 1) * 8;
    ds_off[1] = ds_off[0] ^ 128;  // key + 8: bit 3 of the key index
  }

  auto compute = [&](const char* stage) __attribute__((always_inline)) {
    const char* img = stage + kKTile + wave * kDsWave;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {  // 16 keys each
      bf16x8 dsf[2];
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
        const char* d = img + rb * 2048 + ks * 256;
        dsf[rb] = lds_read_transposed_at(d + ds_off[0], d + ds_off[1]);
      }
      const char* kt = stage + ks * 16 * kRowBytes128;
#pragma unroll
      for (int o = 0; o < DB; ++o) {
        const bf16x8 a = lds_read_transposed_at(kt + t_off[o][0], kt + t_off[o][1]);
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) acc[rb][o] = mfma32(a, dsf[rb], acc[rb][o]);
      }
    }
  };

#pragma unroll
  for (int d = 0; d < kStages - 1; ++d)
    if (d < n_steps_wg) request(d);
  auto step = [&](int s, auto compute_tag) __attribute__((always_inline)) {
    wait_step(s);
    __syncthreads();  // every wave's part of step s has landed; everyone is done with step s-1
    if (s + kStages - 1 < n_steps_wg) request(s + kStages - 1);
    if constexpr (decltype(compute_tag)::value) compute(smem + (s & (kStages - 1)) * kStage);
  };
  int s = 0;
  for (; s < n_steps_wave; ++s) step(s, std::true_type{});
  // other waves of the workgroup may still have steps to visit: keep moving K tiles, keep in step
  for (; s < n_steps_wg; ++s) step(s, std::false_type{});

  OutT* dqh = reinterpret_cast<OutT*>(p.dq) + b * p.dq_bs + (int64_t)h * kD;
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) {
    const int qrow = q_wave0 + 32 * rb + c;
    if (qrow < p.Sq) {
      OutT* dst = dqh + qrow * ((int64_t)p.Hq * kD);
#pragma unroll
      for (int o = 0; o < DB; ++o)
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4)
          store4<OutT>(dst + 32 * o + 8 * b4 + 4 * g, acc[rb][o][4 * b4] * p.scale, acc[rb][o][4 * b4 + 1] * p.scale,
                       acc[rb][o][4 * b4 + 2] * p.scale, acc[rb][o][4 * b4 + 3] * p.scale, p.accumulate != 0);
    }
  }
}

}  // namespace

void launch_dq_from_ds(const BwdParams& p, bool causal, bool f32_out, hipStream_t st) {
  const dim3 grid((unsigned)(p.tiles * p.Hq * p.B)), block(kThreads);
  if (causal) {
    if (f32_out) hipLaunchKernelGGL((attn_bwd_dq_ds_kernel<true, float>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((attn_bwd_dq_ds_kernel<true, __bf16>), grid, block, 0, st, p);
  } else {
    if (f32_out) hipLaunchKernelGGL((attn_bwd_dq_ds_kernel<false, float>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((attn_bwd_dq_ds_kernel<false, __bf16>), grid, block, 0, st, p);
  }
}

}  // namespace pith
