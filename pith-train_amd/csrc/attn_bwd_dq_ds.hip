// Query-gradient kernel for head dims (128, 128) on gfx950 that reads dS instead of recomputing it:
// dQ = scale * dS K (pithtrain/operators/mla/triton.py:205-266, the last product of the loop body),
// with dS = P*(dP - delta) taken, already rounded to bf16 and with its sign flipped, from the images
// that the dK/dV kernel of attn_bwd_dkdv_d128.hip leaves in p.ds (layout documented there). The two score products that the
// other dQ kernels repeat are gone; the price is one trip of dS through memory, so this kernel is
// bound by the rate at which it can stream the images, not by the matrix pipe.
//
// Work split: a workgroup of 8 wavefronts owns 512 query rows of one (batch, head), wave w the 64-row
// query tile 8*m_tile + w of the writer. Keys are visited in steps of 32 (one wave pair of the
// writer). Per step the K tile (shared, packed and swizzled like everywhere else, 8 KB) and, per
// wave, the 4 KB image of its tile for that pair (copied verbatim) go global -> LDS directly. What
// bounds the kernel is how many bytes of dS each compute unit keeps in flight (a compute unit's
// vector cache holds about 64 outstanding 128-byte requests, i.e. ~8 KB per ~650 cycles of latency, so
// every unit must stay busy and spend its requests on dS), so the LDS goes to dS: K tiles live in a
// ring of 3 stages (they come from L2), the images in a ring of 4 stages of 32 KB. A wave's vector
// loads complete in issue order, so one wave cannot wait for a K tile requested two steps ago without
// also waiting for every image it requested before that tile; therefore waves 0..3 request the K
// tiles and nothing else, and waves 4..7 request the images of all eight waves (each its own and that
// of wave w - 4). Every wave waits for its own requests and the step's barrier publishes them.
// dQ += dS K: K fragments (B operands: 32 features x 16 keys) come from transposing reads of the K tile
// and serve both 32-row blocks of the wave's tile, dS fragments (A operands: 32 query rows x 16 keys)
// from transposing reads of the image, in the same key slot order. The accumulators therefore hold
// dQ untransposed (a lane owns one feature column of 16 rows) and the epilogue reads and writes whole
// 128-byte lines (store_rows32).
// With 192-feature keys the same scheme was measured not to pay: a workgroup then holds accumulators
// for 256 rows only, K is 43 % of the bytes a compute unit requests, and the kernel is no faster than
// recomputing the scores.
#include <type_traits>

#include "attn_bwd_common.h"

namespace pith {
namespace {

constexpr int kThreads = 512;
constexpr int kBN = 32;      // keys per step
constexpr int kRingK = 3;    // K tiles: step s in use, s+1 and s+2 requested

// s_waitcnt with vmcnt = N, the other counters left at their maxima (gfx9 encoding: vmcnt in bits
// 3:0 and 15:14).
template <int N>
__device__ __forceinline__ void wait_vector_loads_but() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}
// the same for a wave-uniform run-time count LO <= n <= HI, as a binary decision tree (a switch over
// the counts compiles to a chain of one compare and branch per case, a few hundred cycles per call)
template <int LO, int HI>
__device__ __forceinline__ void wait_vector_loads_but(int n) {
  if constexpr (LO == HI) {
    wait_vector_loads_but<LO>();
  } else {
    constexpr int MID = (LO + HI) / 2;
    if (n <= MID) wait_vector_loads_but<LO, MID>(n);
    else wait_vector_loads_but<MID + 1, HI>(n);
  }
}

template <bool CAUSAL, typename OutT>
__global__ __launch_bounds__(kThreads) void attn_bwd_dq_ds_kernel(BwdParams p) {
  constexpr int DQK = 128, DB = DQK / 32;
  constexpr int QW = 64;                    // query rows per wave
  constexpr int RBW = QW / 32;              // 32-row blocks per wave
  constexpr int kBM = 8 * QW;               // query rows per workgroup
  constexpr int kKStage = kBN * kRowBytes128;                        // 8 KB
  constexpr int kDsWave = RBW * 2048;                                // per wave and step
  constexpr int kDsStage = 8 * kDsWave;                              // 32 KB
  constexpr int kRingD = 4;                                          // images: step s in use, the next three requested
  constexpr int kOffDs = kRingK * kKStage;
  constexpr int kLoadsDs = 2 * RBW;                                  // per image
  constexpr int kLoadsK = 2;                                         // per K-moving wave and step
  static_assert(kOffDs + kRingD * kDsStage <= 160 * 1024, "the rings must fit the LDS");
  __shared__ __attribute__((aligned(1024))) char smem[kOffDs + kRingD * kDsStage];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, g = lane >> 5;
  int m_tile, h, b;
  decode_block(blockIdx.x, p.Hq, p.B, p.tiles, p.group, m_tile, h, b);
  const int hk = h / p.group;
  const int m0 = m_tile * kBM;
  const int q_wave0 = m0 + wave * QW;

  const int kv_row_bytes = p.HkvT * DQK * 2;
  const char* kh = reinterpret_cast<const char*>(p.k + b * p.k_bs + (int64_t)hk * DQK);

  // key steps: all of them, or up to the diagonal; a wave whose query tile does not exist (ragged
  // Sq) has no images and visits nothing. Rows q0 .. q0+QW-1 lie in the writer's 64-row tile q0 >> 6.
  const int n_steps_all = (p.Skv + kBN - 1) / kBN;
  const int n_steps_wg = CAUSAL ? min(n_steps_all, (m0 + kBM - 1) / kBN + 1) : n_steps_all;
  auto steps_of = [&](int q0) __attribute__((always_inline)) {
    if ((q0 >> 6) >= p.ds_qt) return 0;
    return CAUSAL ? min(n_steps_all, (q0 + QW - 1) / kBN + 1) : n_steps_all;
  };
  const int n_steps_wave = steps_of(q_wave0);
  // images of the query tile of rows q0..: key step s = pair s&3 of key block s>>2, 4 KB each,
  // consecutive in s; the rows' part starts 1 KB per 16 rows into each image
  auto images_of = [&](int q0) __attribute__((always_inline)) {
    const int mt = min(q0 >> 6, p.ds_qt - 1);
    return p.ds + (int64_t)(b * p.Hq + h) * p.ds_hs + ds_tile_start<CAUSAL>(mt, p.ds_kb) * kDsBlockBytes + (q0 & 63) * 64;
  };

  // ---- requests. Waves 0..3: K tiles. Waves 4..7: the dS parts of waves w-4 and w.
  const bool k_mover = wave < 4;
  DirectTile128<kBN, 256> mover;
  mover.init(kv_row_bytes, wave & 3, lane);
  const char* ds_src[2] = {images_of(q_wave0 - 4 * QW), images_of(q_wave0)};        // only used by waves 4..7
  const int ds_steps[2] = {k_mover ? 0 : steps_of(q_wave0 - 4 * QW), k_mover ? 0 : n_steps_wave};
  auto request_k = [&](int s, int slot) __attribute__((always_inline)) {
    char* stage = smem + slot * kKStage;
    const char* k_src = kh + (int64_t)s * kBN * kv_row_bytes;
    mover.issue(k_src, p.Skv - s * kBN, stage, wave & 3, lane);
  };
  auto request_ds = [&](int s, int slot) __attribute__((always_inline)) {
    int off = lane << 4;
    asm volatile("" : "+v"(off));
#pragma unroll
    for (int r = 0; r < 2; ++r)
      if (s < ds_steps[r]) {
        const char* src = ds_src[r] + (int64_t)s * 4096;
        char* dst = smem + kOffDs + slot * kDsStage + (wave - 4 + 4 * r) * kDsWave;
#pragma unroll
        for (int j = 0; j < kLoadsDs; ++j) load_lds16(src + j * 1024, off, dst + j * 1024);
      }
  };
  // loads this wave issued for step t
  auto loads_of = [&](int t) __attribute__((always_inline)) {
    if (t >= n_steps_wg) return 0;
    if (k_mover) return kLoadsK;
    return (t < ds_steps[0] ? kLoadsDs : 0) + (t < ds_steps[1] ? kLoadsDs : 0);
  };
  // ring slots of step s (K tiles, dS parts) and of the steps to request next; advanced by one per step
  int k_slot = 0, k_next = kRingK - 1, d_slot = 0, d_next = kRingD - 1;
  auto advance = [&]() __attribute__((always_inline)) {
    k_slot = k_slot + 1 == kRingK ? 0 : k_slot + 1;
    k_next = k_next + 1 == kRingK ? 0 : k_next + 1;
    d_slot = d_slot + 1 == kRingD ? 0 : d_slot + 1;
    d_next = d_next + 1 == kRingD ? 0 : d_next + 1;
  };
  // waits until this wave's loads for step s have landed: the steps requested after it (all but the
  // last of the ring, which follows after the barrier) may stay in flight. Away from the end of the key
  // range that is a constant number of loads.
  constexpr int kSteadyDs = (kRingD - 2) * 2 * kLoadsDs;
  static_assert(kRingK == 3 && kSteadyDs < 32, "one K step in flight; dS loads in flight fit the decision tree");
  const int ds_steady_end = min(min(ds_steps[0], ds_steps[1]), n_steps_wg) - (kRingD - 2);  // steps below: steady state
  auto wait_step = [&](int s) __attribute__((always_inline)) {
    if (k_mover) {
      if (s + 1 < n_steps_wg) wait_vector_loads_but<kLoadsK>();
      else wait_vector_loads_but<0>();
    } else if (s < ds_steady_end) {
      wait_vector_loads_but<kSteadyDs>();
    } else {
      int n = 0;
#pragma unroll
      for (int d = 1; d < kRingD - 1; ++d) n += loads_of(s + d);
      wait_vector_loads_but<0, 31>(n);
    }
  };

  f32x16 acc[RBW][DB];  // [32-row block][feature block]
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
    for (int o = 0; o < DB; ++o)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[rb][o][v] = 0.f;

  // per-lane read offsets. K tile: transposing reads of the lower / upper 8 keys of a 16-key step at
  // feature block 0; block o follows by XOR with o << 6 (the swizzle is an XOR of the piece index).
  // Image: this lane supplies, for its 16-lane block (g, chalf) and r = 4i + m, the 8 bytes that hold
  // key 4g + i (+ 8 for the upper read) at queries 16*chalf + 4m .. +3 of a 32-row block: 16-row step
  // chalf of the block, writer lane group m&1, fragment half m>>1.
  const int t_base[2] = {transposed_offset128(0, 0, 0, lane), transposed_offset128(0, 1, 0, lane)};
  int ds_off[2];
  {
    const int r = lane & 15, chalf = (lane >> 4) & 1;
    const int i = r >> 2, m = r & 3, gl = m & 1;
    const int key = 4 * g + i;
    ds_off[0] = chalf * 1024 + gl * 512 + ((key ^ (gl << 3) ^ (chalf << 2)) << 4) + (m >> 1) * 8;
    ds_off[1] = ds_off[0] ^ 128;  // key + 8: bit 3 of the key index
  }

  auto compute = [&](const char* stage, const char* img) __attribute__((always_inline)) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {  // 16 keys each
      bf16x8 dsf[RBW];
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb) {
        const char* d = img + rb * 2048 + ks * 256;
        dsf[rb] = lds_read_transposed_at(d + ds_off[0], d + ds_off[1]);
      }
#pragma unroll
      for (int o = 0; o < DB; ++o) {
        const char* kt = stage + ks * 16 * kRowBytes128;
        const bf16x8 a = lds_read_transposed_at(kt + (t_base[0] ^ (o << 6)), kt + (t_base[1] ^ (o << 6)));
#pragma unroll
        for (int rb = 0; rb < RBW; ++rb) acc[rb][o] = mfma32(dsf[rb], a, acc[rb][o]);
      }
    }
  };

  if (k_mover) {
#pragma unroll
    for (int d = 0; d < kRingK - 1; ++d)
      if (d < n_steps_wg) request_k(d, d);
  } else {
#pragma unroll
    for (int d = 0; d < kRingD - 1; ++d)
      if (d < n_steps_wg) request_ds(d, d);
  }
  auto step = [&](int s, auto compute_tag) __attribute__((always_inline)) {
    wait_step(s);
    __syncthreads();  // every wave's requests for step s have landed; everyone is done with step s-1
    if (k_mover) {
      if (s + kRingK - 1 < n_steps_wg) request_k(s + kRingK - 1, k_next);
    } else {
      if (s + kRingD - 1 < n_steps_wg) request_ds(s + kRingD - 1, d_next);
    }
    if constexpr (decltype(compute_tag)::value)
      compute(smem + k_slot * kKStage, smem + kOffDs + d_slot * kDsStage + wave * kDsWave);
    advance();
  };
  int s = 0;
  for (; s < n_steps_wave; ++s) step(s, std::true_type{});
  // other waves of the workgroup may still have steps to visit: keep moving tiles, keep in step
  for (; s < n_steps_wg; ++s) step(s, std::false_type{});

  OutT* dqh = reinterpret_cast<OutT*>(p.dq) + b * p.dq_bs + (int64_t)h * DQK;
  const float sc = -p.scale;  // the images hold -dS (the writer forms delta - dP)
  const int64_t row_stride = (int64_t)p.HqT * DQK;
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb) {
    const int row0 = q_wave0 + 32 * rb;
    __bf16* fin = nullptr;  // rows whose gradient is complete with this call go out as bf16
    if (p.dq_final != nullptr && row0 >= p.final_r0 && row0 < p.final_r1)
      fin = p.dq_final + b * p.dq_final_bs + (int64_t)h * DQK + row0 * row_stride;
    store_rows32<OutT, DB>(dqh + row0 * row_stride, row_stride, p.Sq - row0, acc[rb], sc, p.accumulate != 0, c, g, fin);
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
