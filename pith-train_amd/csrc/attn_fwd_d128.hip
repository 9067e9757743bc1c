// Chunk attention forward for head dims (128, 128) on gfx950. Same function and numerics as the
// general kernel in attn_fwd.hip (pithtrain/operators/mla/triton.py:32-93, :274-323: fp32
// scores from bf16 MFMA, P = exp2(kappa*(s - m)) in fp32, row sum from the fp32 P, P rounded to
// bf16 for P V, base-2 LSE, lazily refreshed running maximum), organised around two facts
// measured on the device:
//   - the two wavefronts that share a SIMD overlap matrix and vector work only while they are in
//     DIFFERENT phases; left alone they fall into lock step (both in MFMA, then both in VALU);
//   - moving K/V tiles through registers into LDS costs several hundred cycles per tile of
//     vector-issue time in which no MFMA runs.
// So (1) K/V tiles go global -> LDS directly (global_load_lds, packed swizzled tiles, a ring of
// four per operand), requested two intervals ahead, and (2) the 8 wavefronts of a workgroup are split into
// "early" (0-3) and "late" (4-7) ones, wave w and w+4 sharing a SIMD. Per interval every wave
// runs one matrix block  [O^T += V(i)^T P(i)^T ; S(i+1)^T = K(i+1) Q^T]  and one vector block
// [P = softmax(S)]; early waves run matrix then vector, late waves vector then matrix, so on
// each SIMD one wave's MFMAs coincide with the other's softmax. In its matrix block a wave has
// no help in hiding LDS latency, so the fragment reads run a few products ahead of their use.
#include <type_traits>

#include "attn_fwd_common.h"

namespace pith {
namespace {

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kBM = kWaves * 32;  // query rows per workgroup
constexpr int kBN = kFwdBlockN;   // keys per tile
constexpr int kD = 128;
constexpr int kDist = 2;   // a tile is requested kDist intervals before the interval that reads it
constexpr int kSlots = 4;  // ring depth per operand, > kDist; a power of two (the slot index is a mask)
static_assert(kSlots > kDist && (kSlots & (kSlots - 1)) == 0, "ring depth");
constexpr int kAhead = 4;  // fragment reads run this many products ahead in the matrix block
constexpr int kTile = kBN * kRowBytes128;

template <bool CAUSAL>
__global__ __launch_bounds__(kThreads) void attn_fwd_d128_kernel(FwdParams p) {
  constexpr int KS = kD / 16;   // contraction steps of Q K^T
  constexpr int DVB = kD / 32;  // 32-row blocks of O^T
  __shared__ __attribute__((aligned(1024))) char smem[2 * kSlots * kTile];
  char* const kbuf = smem;
  char* const vbuf = smem + kSlots * kTile;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, g = lane >> 5;
  const bool late = wave >= kWaves / 2;  // shares its SIMD with wave - kWaves/2

  int m_tile, h, b;
  decode_block(blockIdx.x, p.Hq, p.B, p.m_tiles, m_tile, h, b);
  const int hk = h / p.group;
  const int m0 = m_tile * kBM;
  const int q_wave0 = m0 + wave * 32;
  const int qrow = q_wave0 + c;

  const int64_t q_row_stride = (int64_t)p.Hq * kD;
  const int64_t o_row_stride = (int64_t)p.Hq * kD;
  const int kv_row_bytes = p.Hkv * kD * 2;
  const __bf16* qh = p.q + b * p.q_bs + (int64_t)h * kD;
  const char* kh = reinterpret_cast<const char*>(p.k + b * p.k_bs + (int64_t)hk * kD);
  const char* vh = reinterpret_cast<const char*>(p.v + b * p.v_bs + (int64_t)hk * kD);

  // Number of key tiles this workgroup / this wavefront has to visit.
  const int n_tiles_all = (p.Skv + kBN - 1) / kBN;
  int n_tiles_wg = n_tiles_all, n_tiles_wave = n_tiles_all;
  if (CAUSAL) {
    n_tiles_wg = min(n_tiles_all, (m0 + kBM - 1) / kBN + 1);
    n_tiles_wave = min(n_tiles_all, (q_wave0 + 31) / kBN + 1);
  }

  DirectTile128<kBN, kThreads> mover;
  mover.init(kv_row_bytes, wave, lane);
  auto issue_k = [&](int t) __attribute__((always_inline)) {
    mover.issue(kh + (int64_t)t * kBN * kv_row_bytes, p.Skv - t * kBN, kbuf + (t & (kSlots - 1)) * kTile, wave, lane);
  };
  auto issue_v = [&](int t) __attribute__((always_inline)) {
    mover.issue(vh + (int64_t)t * kBN * kv_row_bytes, p.Skv - t * kBN, vbuf + (t & (kSlots - 1)) * kTile, wave, lane);
  };
  // tiles needed by the prologue (K 0), interval 0 (K 1, V 0) and interval 1 (K 2, V 1)
  issue_k(0);
#pragma unroll
  for (int t = 0; t < kDist; ++t) {
    if (t + 1 < n_tiles_wg) issue_k(t + 1);
    if (t < n_tiles_wg) issue_v(t);
  }

  // Q^T fragments (B operand): column = query row, slots = 8 consecutive features.
  bf16x8 qf[KS];
  {
    const int row = qrow < p.Sq ? qrow : p.Sq - 1;
    const __bf16* src = qh + row * q_row_stride + g * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(src + ks * 16);
  }

  // per-lane read offsets inside a tile
  int k_off[KS];      // straight fragment of key row c, contraction step ks (+ 32 rows: + 8192 bytes)
  int v_off[DVB][2];  // transposing reads of feature block i, lower / upper 8 keys (+ 16 keys: + 4096 bytes)
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) k_off[ks] = straight_offset128(c, 2 * ks + g);
#pragma unroll
  for (int i = 0; i < DVB; ++i)
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) v_off[i][hh] = transposed_offset128(0, hh, 32 * i, lane);

  f32x16 oacc[DVB];
#pragma unroll
  for (int i = 0; i < DVB; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[i][v] = 0.f;
  float m_run = -INFINITY;
  float l_run = 0.f;  // this lane's share of the row sum (the partner lane holds the rest)

  f32x16 s[2];   // S^T of one key tile: [64 keys] x [32 queries] as two 32 x 32 tiles
  bf16x8 pf[4];  // P^T of one key tile as B operand, one fragment per 16 keys

  // ---- S^T = K Q^T
  auto scores = [&](const char* ktile) __attribute__((always_inline)) {
#pragma unroll
    for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
      for (int v = 0; v < 16; ++v) s[kvb][v] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(ktile + k_off[ks] + kvb * 32 * kRowBytes128);
        s[kvb] = mfma32(a, qf[ks], s[kvb]);
      }
  };

  // ---- mask, online softmax (one query column per lane pair), P^T fragments
  auto softmax = [&](int t) __attribute__((always_inline)) {
    const int n0 = t * kBN;
    if ((CAUSAL && (n0 + kBN - 1 > q_wave0)) || (n0 + kBN > p.Skv)) {
      // tile crossing the diagonal of a causal chunk, or a ragged last tile
      const int limit = CAUSAL ? min(qrow, p.Skv - 1) : p.Skv - 1;  // last visible key
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int key = n0 + kvb * 32 + acc_row(v, g);
          if (key > limit) s[kvb][v] = -INFINITY;
        }
    }
    float x = s[0][0];
#pragma unroll
    for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
      for (int v = 0; v < 16; ++v) x = fmaxf(x, s[kvb][v]);
    const float mx = pair_max(x);
    const bool refresh = (mx - m_run) * p.kappa > kRescaleThreshold;  // true on the first tile (m = -inf)
    if (__builtin_amdgcn_ballot_w64(refresh) != 0) {                   // wave-uniform
      const float m_new = fmaxf(m_run, mx);
      // a row with no visible key so far keeps m = -inf; exp2 of (-inf - -inf) is avoided
      const float alpha = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f((m_run - m_new) * p.kappa);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int i = 0; i < DVB; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[i][v] *= alpha;
    }
    const float mk = (m_run == -INFINITY) ? 0.f : m_run * p.kappa;
    float rs = 0.f;
#pragma unroll
    for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float e = __builtin_amdgcn_exp2f(s[kvb][v] * p.kappa - mk);
        s[kvb][v] = e;
        rs += e;
      }
    l_run += rs;
#pragma unroll
    for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        const f32x16& x16 = s[kvb];
        pf[2 * kvb + jj] = to_bf16x8(x16[8 * jj], x16[8 * jj + 1], x16[8 * jj + 2], x16[8 * jj + 3], x16[8 * jj + 4],
                                     x16[8 * jj + 5], x16[8 * jj + 6], x16[8 * jj + 7]);
      }
  };

  // ---- O^T += V^T P^T
  auto accumulate = [&](const char* vtile) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < DVB; ++i) {
        const bf16x8 a = lds_read_transposed_at(vtile + v_off[i][0] + j * 16 * kRowBytes128,
                                                vtile + v_off[i][1] + j * 16 * kRowBytes128);
        oacc[i] = mfma32(a, pf[j], oacc[i]);
      }
  };

  // ---- matrix block of one interval: O^T += V^T P^T of one tile, then S^T of the next, with
  // the fragment reads pinned kAhead products ahead of their use.
  auto matrix_block = [&](const char* vtile, const char* ktile) __attribute__((always_inline)) {
    constexpr int NPV = 4 * DVB, NQK = 2 * KS;
    bf16x8 av[4][DVB], ak[KS][2];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < DVB; ++i)
        av[j][i] = lds_read_transposed_at(vtile + v_off[i][0] + j * 16 * kRowBytes128,
                                          vtile + v_off[i][1] + j * 16 * kRowBytes128);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb)
        ak[ks][kvb] = *reinterpret_cast<const bf16x8*>(ktile + k_off[ks] + kvb * 32 * kRowBytes128);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < DVB; ++i) oacc[i] = mfma32(av[j][i], pf[j], oacc[i]);
#pragma unroll
    for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
      for (int v = 0; v < 16; ++v) s[kvb][v] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb) s[kvb] = mfma32(ak[ks][kvb], qf[ks], s[kvb]);
    // a transposed fragment takes two LDS reads, a straight one a single read
    __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);
#pragma unroll
    for (int m = 0; m < NPV - kAhead; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
#pragma unroll
    for (int m = 0; m < NQK; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 0);
  };

  // Every interval ends by waiting until at most the loads of the last kDist - 1 intervals are
  // still in flight (the tiles of the next interval have landed), and a workgroup barrier.
  constexpr int kPerInterval = 2 * DirectTile128<kBN, kThreads>::kPerThread;
  static_assert((kDist - 1) * kPerInterval < 16, "vmcnt immediate below assumes a 4-bit low field");
  auto land_and_sync = [&](bool steady) __attribute__((always_inline)) {
    if (steady) __builtin_amdgcn_s_waitcnt(0x0F70 | ((kDist - 1) * kPerInterval));
    else __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
  };

  // ---- prologue: S(0) (and P(0) in the early waves) from K tile 0
  __builtin_amdgcn_s_waitcnt(0x0F70);  // everything issued so far, Q fragments included
  __syncthreads();
  scores(kbuf);
  __syncthreads();  // K tile 0 has been read by every wave: its slot may be refilled
  if (!late) softmax(0);

  // One interval; FULL: this wave has both a tile to accumulate and a next tile to score.
  auto interval = [&](int i, auto late_tag, auto full_tag) __attribute__((always_inline)) {
    constexpr bool LATE = decltype(late_tag)::value, FULL = decltype(full_tag)::value;
    const char* vtile = vbuf + (i & (kSlots - 1)) * kTile;
    const char* ktile = kbuf + ((i + 1) & (kSlots - 1)) * kTile;
    const bool steady = i + 1 + kDist < n_tiles_wg;  // both a K and a V tile are requested in this interval
    // Requests are placed where no LDS read of the same wave follows closely: after the matrix
    // block in the early waves, before the vector block in the late ones.
    auto request = [&]() __attribute__((always_inline)) {
      if (i + 1 + kDist < n_tiles_wg) issue_k(i + 1 + kDist);
      if (i + kDist < n_tiles_wg) issue_v(i + kDist);
    };
    if (!LATE) {
      if (FULL) {
        matrix_block(vtile, ktile);
        __builtin_amdgcn_sched_barrier(0);
        request();
        softmax(i + 1);
      } else {
        if (i < n_tiles_wave) accumulate(vtile);
        request();
      }
    } else {
      request();
      if (FULL || i < n_tiles_wave) softmax(i);
      __builtin_amdgcn_sched_barrier(0);
      if (FULL) matrix_block(vtile, ktile);
      else if (i < n_tiles_wave) accumulate(vtile);
    }
    land_and_sync(steady);
  };
  // Every wave passes the same number of barriers; the two roles run separate loops so that
  // each loop body is straight-line code around one accumulator set.
  if (!late) {
    int i = 0;
    for (; i + 1 < n_tiles_wave; ++i) interval(i, std::false_type{}, std::true_type{});
    for (; i < n_tiles_wg; ++i) interval(i, std::false_type{}, std::false_type{});
  } else {
    int i = 0;
    for (; i + 1 < n_tiles_wave; ++i) interval(i, std::true_type{}, std::true_type{});
    for (; i < n_tiles_wg; ++i) interval(i, std::true_type{}, std::false_type{});
  }

  // ---- epilogue: normalise, store O (bf16) and LSE2
  __bf16* oh = p.o + b * p.o_bs + (int64_t)h * kD;
  float* lse = p.lse + b * p.lse_bs + (int64_t)h * p.lse_hs;
  const float l = pair_sum(l_run);
  const float inv = l > 0.f ? 1.f / l : 0.f;
  if (qrow < p.Sq) {
    __bf16* dst = oh + qrow * o_row_stride;
#pragma unroll
    for (int i = 0; i < DVB; ++i)
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) {
        u32x2 w;
        w[0] = pack_bf16x2(oacc[i][4 * b4] * inv, oacc[i][4 * b4 + 1] * inv);
        w[1] = pack_bf16x2(oacc[i][4 * b4 + 2] * inv, oacc[i][4 * b4 + 3] * inv);
        *reinterpret_cast<u32x2*>(dst + 32 * i + 8 * b4 + 4 * g) = w;
      }
    if (g == 0) lse[qrow] = (l > 0.f) ? __builtin_amdgcn_logf(l) + m_run * p.kappa : -INFINITY;
  }
}

}  // namespace

void launch_fwd_d128(FwdParams p, bool causal, hipStream_t st) {
  p.m_tiles = (p.Sq + kBM - 1) / kBM;
  const dim3 grid((unsigned)(p.m_tiles * p.Hq * p.B)), block(kThreads);
  if (causal)
    hipLaunchKernelGGL((attn_fwd_d128_kernel<true>), grid, block, 0, st, p);
  else
    hipLaunchKernelGGL((attn_fwd_d128_kernel<false>), grid, block, 0, st, p);
}

}  // namespace pith
