// Query-gradient kernel for head dims (128, 128) and (192, 128) on gfx950, organised like the
// direct-load forward kernel (256-row workgroups, or 128-row ones whose wave pairs split the keys).
// Same function and numerics as the other dQ kernels (pithtrain/operators/mla/triton.py:205-266,
// :392-441: P = exp2(kappa*s - lse2) in fp32, masked entries 0, dS = P*(dP - delta)*scale rounded
// to bf16, fp32 accumulation of dQ += dS K; `scale` is applied once to the accumulated dQ).
//
// Organisation: that of the direct-load forward kernel (attn_fwd_direct.hip). K/V tiles go
// global -> LDS directly into packed swizzled tiles (rings of four, requested two intervals ahead).
// Wave w and wave w + 4 of a workgroup share a SIMD. Per interval a wave runs one matrix block
//     dQ^T += K(i)^T dS(i)^T ;  S(i+1)^T = K(i+1) Q^T ;  dP(i+1)^T = V(i+1) dO^T
// and one vector block  dS(i+1) = P o (dP - delta);  early waves (0-3) run matrix then vector, late
// waves (4-7) vector then matrix, so that on every SIMD one wave's MFMAs coincide with the other's
// arithmetic. Q^T and dO^T fragments, lse and delta of a wave's 32 query rows are stationary.
// FULL: a workgroup owns 256 query rows, every wave 32 of them and all 64 keys of each tile (48
// matrix instructions per wave and interval against some 110 vector instructions: the vector block
// hides completely behind the sibling's matrix block).
// HALF: a workgroup owns 128 query rows; wave w and w + 4 own the SAME 32 rows, the early wave keys
// 0-31 and the late wave keys 32-63 of every tile; at the end the late wave hands its partial dQ to
// the early wave through LDS.
//
// With 192-feature queries the stationary fragments alone (Q^T 48 + dO^T 32 registers) push a wave
// past 256 registers, and spilled fragments are reloaded from scratch memory in every interval. The
// last four Q^T fragments (features 128..191) and the last four dO^T fragments are therefore kept
// in LDS (written once, 8 KB per pair of waves) and read as B operands when needed; tiles are
// requested ONE interval ahead there (K ring of 4, V ring of 2) to make the room.
//
// Why this form: with 192-feature queries a wave that owned all 64 keys of a tile would need more
// than 256 registers (Q^T 48 + dO^T 32 + dQ 96 + S, dP 64 + dS 16); owning half the keys brings
// the tile-width dependent part down to 40. And launches with few query rows (the MLA ring share:
// 16 heads x 4096 rows) get twice as many workgroups.
#include <type_traits>

#include "attn_bwd_common.h"

namespace pith {
namespace {

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kBN = 64;    // keys per tile
constexpr int kDv = 128;
constexpr int kSlots = 4;  // K ring depth (tiles i, i+1 in use, later ones landing); a power of two
constexpr int kAhead = 4;  // fragment reads run this many products ahead in the matrix block
constexpr int kTile = kBN * kRowBytes128;

template <int DQK, bool HALF, bool CAUSAL, typename OutT>
__global__ __launch_bounds__(kThreads) void attn_bwd_dq_direct_kernel(BwdParams p) {
  static_assert(DQK == 128 || (DQK == 192 && HALF), "head dims (192-feature queries need the HALF form)");
  constexpr int KVB = HALF ? 1 : 2;      // 32-key blocks of a tile this wave owns
  constexpr int kBM = HALF ? 128 : 256;  // query rows per workgroup
  // kDist: a tile is requested kDist intervals before the interval that first reads it.
  // kLdsQ / kLdsDo: trailing Q^T / dO^T fragments kept in LDS instead of registers.
  constexpr int kDist = DQK == 192 ? 1 : 2;
  constexpr int kVSlots = kDist + 1 == 2 ? 2 : 4;
  constexpr int kLdsQ = DQK == 192 ? 4 : 0, kLdsDo = DQK == 192 ? 4 : 0;
  constexpr int kStatPair = (kLdsQ + kLdsDo) * 1024;  // bytes of LDS-resident fragments per pair of waves
  constexpr int KS = DQK / 16;   // contraction steps of S = Q K^T
  constexpr int VS = kDv / 16;   // contraction steps of dP = dO V^T
  constexpr int DB = DQK / 32;   // 32-feature blocks of dQ^T
  constexpr int kKTile = kTile + (DQK == 192 ? kExtraTileBytes : 0);
  __shared__ __attribute__((aligned(1024))) char smem[kSlots * kKTile + kVSlots * kTile + 4 * kStatPair];
  char* const kbuf = smem;
  char* const vbuf = smem + kSlots * kKTile;
  const char* const stat = smem + kSlots * kKTile + kVSlots * kTile + (threadIdx.x >> 6 & 3) * kStatPair + (threadIdx.x & 63) * 16;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, g = lane >> 5;
  const bool late = wave >= kWaves / 2;
  const int kvb0 = HALF ? wave >> 2 : 0;  // the first 32-key block of every tile this wave owns

  int m_tile, h, b;
  decode_block(blockIdx.x, p.Hq, p.B, p.tiles, p.group, m_tile, h, b);
  const int hk = h / p.group;
  const int m0 = m_tile * kBM;
  const int q_wave0 = m0 + (HALF ? (wave & 3) : wave) * 32;
  const int qrow = q_wave0 + c;

  const int64_t q_row_stride = (int64_t)p.HqT * DQK;
  const int64_t do_row_stride = (int64_t)p.HqT * kDv;
  // keys in two parts: K rows hold 128 features per head, the last 64 come from k_pe (no head offset)
  const bool two_part = DQK == 192 && p.k_pe != nullptr;
  const int k_head_elems = two_part ? 128 : DQK;
  const int k_row_bytes = p.HkvT * k_head_elems * 2, v_row_bytes = p.HkvT * kDv * 2;
  const char* kh = reinterpret_cast<const char*>(p.k + b * p.k_bs + (int64_t)hk * k_head_elems);
  const char* kx = two_part ? reinterpret_cast<const char*>(p.k_pe + b * p.k_pe_bs) : kh;  // source of features 128..
  const int kx_row_bytes = two_part ? (int)p.k_pe_rs * 2 : k_row_bytes;
  const char* vh = reinterpret_cast<const char*>(p.v + b * p.v_bs + (int64_t)hk * kDv);

  const int n_tiles_all = (p.Skv + kBN - 1) / kBN;
  int n_tiles_wg = n_tiles_all, n_tiles_wave = n_tiles_all;
  if (CAUSAL) {
    n_tiles_wg = min(n_tiles_all, (m0 + kBM - 1) / kBN + 1);
    n_tiles_wave = min(n_tiles_all, (q_wave0 + 31) / kBN + 1);
  }

  DirectTile128<kBN, kThreads> mover, kmover;  // V tiles (and K tiles when the row pitches agree); K tiles otherwise
  DirectExtra64 xmover;
  mover.init(v_row_bytes, wave, lane);
  if constexpr (DQK != kDv) {
    kmover.init(k_row_bytes, wave, lane);
    xmover.init(kx_row_bytes, two_part ? 0 : 256, wave, lane);
  }
  auto request = [&](int t) __attribute__((always_inline)) {
    char* kslot = kbuf + (t & (kSlots - 1)) * kKTile;
    const char* ksrc = kh + (int64_t)t * kBN * k_row_bytes;
    if constexpr (DQK != kDv) {
      kmover.issue(ksrc, p.Skv - t * kBN, kslot, wave, lane);
      xmover.issue(kx + (int64_t)t * kBN * kx_row_bytes, p.Skv - t * kBN, kslot + kTile, wave, lane);
    } else {
      mover.issue(ksrc, p.Skv - t * kBN, kslot, wave, lane);
    }
    mover.issue(vh + (int64_t)t * kBN * v_row_bytes, p.Skv - t * kBN, vbuf + (t & (kVSlots - 1)) * kTile, wave, lane);
  };
  // tiles of the prologue (0) and of the first kDist intervals
#pragma unroll
  for (int t = 0; t <= kDist; ++t)
    if (t < n_tiles_wg) request(t);

  // stationary side: Q^T and dO^T fragments (B operands), lse and delta of this lane's query row
  constexpr int KSR = KS - kLdsQ, VSR = VS - kLdsDo;  // fragments held in registers
  bf16x8 qf[KSR], dof[VSR];
  float lse_q, delta_q;
  {
    const int row = qrow < p.Sq ? qrow : p.Sq - 1;
    const __bf16* src = p.q + b * p.q_bs + (int64_t)h * DQK + row * q_row_stride + g * 8;
    const __bf16* dsrc = p.dout + b * p.dout_bs + (int64_t)h * kDv + row * do_row_stride + g * 8;
#pragma unroll
    for (int ks = 0; ks < KSR; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(src + ks * 16);
#pragma unroll
    for (int ks = 0; ks < VSR; ++ks) dof[ks] = *reinterpret_cast<const bf16x8*>(dsrc + ks * 16);
    if (!late) {  // the two waves of a pair hold the same rows: the early one fills the pair's LDS copy
#pragma unroll
      for (int ks = 0; ks < kLdsQ; ++ks)
        *reinterpret_cast<bf16x8*>(const_cast<char*>(stat) + ks * 1024) = *reinterpret_cast<const bf16x8*>(src + (KSR + ks) * 16);
#pragma unroll
      for (int ks = 0; ks < kLdsDo; ++ks)
        *reinterpret_cast<bf16x8*>(const_cast<char*>(stat) + (kLdsQ + ks) * 1024) = *reinterpret_cast<const bf16x8*>(dsrc + (VSR + ks) * 16);
    }
    lse_q = (p.lse + b * p.lse_bs + (int64_t)h * p.lse_hs)[row];
    delta_q = (p.delta + b * p.lse_bs + (int64_t)h * p.lse_hs)[row];
  }
  // B operand of contraction step ks of S / of dP
  auto q_frag = [&](int ks) __attribute__((always_inline)) {
    return ks < KSR ? qf[ks < KSR ? ks : 0] : *reinterpret_cast<const bf16x8*>(stat + (ks - KSR) * 1024);
  };
  auto do_frag = [&](int ks) __attribute__((always_inline)) {
    return ks < VSR ? dof[ks < VSR ? ks : 0] : *reinterpret_cast<const bf16x8*>(stat + (kLdsQ + ks - VSR) * 1024);
  };

  // per-lane read offsets inside a tile, for this wave's key block. The swizzle is an XOR on the
  // 16-byte piece index, so the offsets of all contraction steps / feature blocks of one tile part
  // differ from the first one by an XOR with a constant: only the first ones are kept in registers
  // (s_base / t_base: 128-feature tile, sx_base / tx_base: the extra tile behind a K tile).
  //   straight fragment of key row c, contraction step ks:  s_base ^ (ks << 5)      (ks < 8)
  //                                                          sx_base ^ ((ks-8) << 5) (ks >= 8)
  //   transposing reads of K feature block o, lower / upper 8 keys of a 16-key step (+ 16 keys:
  //   + 4096 bytes):  t_base[hh] ^ (o << 6)  (o < 4),  tx_base[hh] ^ ((o-4) << 6)  (o >= 4)
  int s_base = straight_offset128(c, g) + kvb0 * 32 * kRowBytes128;
  int sx_base = kTile + straight_offset128(c, g + 8 * kvb0);
  int t_base[2], tx_base[2];
#pragma unroll
  for (int hh = 0; hh < 2; ++hh) {
    t_base[hh] = transposed_offset128(0, hh, 0, lane) + kvb0 * 32 * kRowBytes128;
    tx_base[hh] = kTile + transposed_offset128(0, hh, 64 * kvb0, lane);
  }
  // Called once per interval: the compiler must take the base offsets as new values each time, or it
  // would compute all derived offsets once, keep them in registers across the loop and spill others.
  auto refresh_offsets = [&]() __attribute__((always_inline)) {
    if constexpr (DQK == 192) asm volatile("" : "+v"(s_base), "+v"(sx_base), "+v"(t_base[0]), "+v"(t_base[1]), "+v"(tx_base[0]), "+v"(tx_base[1]));
    else if constexpr (!HALF) asm volatile("" : "+v"(s_base), "+v"(t_base[0]), "+v"(t_base[1]));
  };
  auto s_off = [&](int ks) __attribute__((always_inline)) { return ks < 8 ? s_base ^ (ks << 5) : sx_base ^ ((ks - 8) << 5); };
  auto t_off = [&](int o, int hh) __attribute__((always_inline)) {
    return o < 4 ? t_base[hh] ^ (o << 6) : tx_base[hh] ^ ((o - 4) << 6);
  };

  f32x16 acc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;

  f32x16 s[KVB], dp[KVB];  // S^T and dP^T of this wave's keys of one tile: 32 x 32 tiles [keys] x [queries]
  bf16x8 dsf[2 * KVB];     // dS^T / scale of the same keys as B operand, one fragment per 16 keys
  // straight fragment of key block kvb: the 128-feature tile steps 32 rows on, the extra tile (192
  // features, HALF only) is never asked for a second block
  auto a_frag = [&](const char* tile, int ks, int kvb) __attribute__((always_inline)) {
    return *reinterpret_cast<const bf16x8*>(tile + s_off(ks) + kvb * 32 * kRowBytes128);
  };

  // ---- S^T = K Q^T and dP^T = V dO^T
  auto scores = [&](const char* ktile, const char* vtile) __attribute__((always_inline)) {
#pragma unroll
    for (int kvb = 0; kvb < KVB; ++kvb)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        s[kvb][v] = 0.f;
        dp[kvb][v] = 0.f;
      }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int kvb = 0; kvb < KVB; ++kvb) s[kvb] = mfma32(a_frag(ktile, ks, kvb), q_frag(ks), s[kvb]);
#pragma unroll
    for (int ks = 0; ks < VS; ++ks)
#pragma unroll
      for (int kvb = 0; kvb < KVB; ++kvb) dp[kvb] = mfma32(a_frag(vtile, ks, kvb), do_frag(ks), dp[kvb]);
  };
  // ---- dQ^T += K^T dS^T
  auto accumulate = [&](const char* ktile) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 2 * KVB; ++j)
#pragma unroll
      for (int o = 0; o < DB; ++o) {
        const char* base = ktile + j * 16 * kRowBytes128;
        acc[o] = mfma32(lds_read_transposed_at(base + t_off(o, 0), base + t_off(o, 1)), dsf[j], acc[o]);
      }
  };
  // ---- matrix block: the gradient product of tile `kprev`, then both score products of the next
  // tile: first the contraction steps whose B operand sits in registers, then those whose B operand
  // is read from LDS (two reads per product, like the transposed fragments).
  auto matrix_block = [&](const char* kprev, const char* ktile, const char* vtile) __attribute__((always_inline)) {
    constexpr int NT = 2 * KVB * DB, N1 = KVB * (KSR + VSR), N2 = kLdsQ + kLdsDo;
    static_assert(kAhead <= NT && kAhead <= N1 && (N2 == 0 || kAhead <= N2), "look-ahead segments");
    static_assert(N2 == 0 || KVB == 1, "LDS-resident B operands only in the HALF form");
    bf16x8 at[2 * KVB][DB], ak[KS][KVB], av[VS][KVB], bq[kLdsQ + 1], bd[kLdsDo + 1];
#pragma unroll
    for (int j = 0; j < 2 * KVB; ++j)
#pragma unroll
      for (int o = 0; o < DB; ++o) {
        const char* base = kprev + j * 16 * kRowBytes128;
        at[j][o] = lds_read_transposed_at(base + t_off(o, 0), base + t_off(o, 1));
      }
#pragma unroll
    for (int ks = 0; ks < KSR; ++ks)
#pragma unroll
      for (int kvb = 0; kvb < KVB; ++kvb) ak[ks][kvb] = a_frag(ktile, ks, kvb);
#pragma unroll
    for (int ks = 0; ks < VSR; ++ks)
#pragma unroll
      for (int kvb = 0; kvb < KVB; ++kvb) av[ks][kvb] = a_frag(vtile, ks, kvb);
#pragma unroll
    for (int ks = 0; ks < kLdsQ; ++ks) {
      ak[KSR + ks][0] = a_frag(ktile, KSR + ks, 0);
      bq[ks] = *reinterpret_cast<const bf16x8*>(stat + ks * 1024);
    }
#pragma unroll
    for (int ks = 0; ks < kLdsDo; ++ks) {
      av[VSR + ks][0] = a_frag(vtile, VSR + ks, 0);
      bd[ks] = *reinterpret_cast<const bf16x8*>(stat + (kLdsQ + ks) * 1024);
    }
#pragma unroll
    for (int j = 0; j < 2 * KVB; ++j)
#pragma unroll
      for (int o = 0; o < DB; ++o) acc[o] = mfma32(at[j][o], dsf[j], acc[o]);
#pragma unroll
    for (int kvb = 0; kvb < KVB; ++kvb)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        s[kvb][v] = 0.f;
        dp[kvb][v] = 0.f;
      }
#pragma unroll
    for (int ks = 0; ks < KSR; ++ks)
#pragma unroll
      for (int kvb = 0; kvb < KVB; ++kvb) s[kvb] = mfma32(ak[ks][kvb], qf[ks], s[kvb]);
#pragma unroll
    for (int ks = 0; ks < VSR; ++ks)
#pragma unroll
      for (int kvb = 0; kvb < KVB; ++kvb) dp[kvb] = mfma32(av[ks][kvb], dof[ks], dp[kvb]);
#pragma unroll
    for (int ks = 0; ks < kLdsQ; ++ks) s[0] = mfma32(ak[KSR + ks][0], bq[ks], s[0]);
#pragma unroll
    for (int ks = 0; ks < kLdsDo; ++ks) dp[0] = mfma32(av[VSR + ks][0], bd[ks], dp[0]);
    // Reads run kAhead products ahead: after product m come the reads of product m + kAhead.
    // Products 0 .. NT-1 and the last N2 take two LDS reads each, the N1 in between one.
    __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);
#pragma unroll
    for (int m = 0; m < NT - kAhead; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
#pragma unroll
    for (int m = 0; m < N1; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
#pragma unroll
    for (int m = 0; m < N2; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 0);
  };
  // ---- s, dp of tile t -> dS / scale as bf16 fragments
  // MASKED = false: the caller knows that tile t lies entirely below this wave's diagonal and inside
  // the key range (no mask code, and nothing it needs stays live in the loop that uses it)
  auto make_ds = [&](int t, auto masked_tag) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    const int n0 = t * kBN;
#pragma unroll
    for (int kvb = 0; kvb < KVB; ++kvb)
#pragma unroll
      for (int v = 0; v < 16; ++v) s[kvb][v] = __builtin_amdgcn_exp2f(s[kvb][v] * p.kappa - lse_q);
    if (MASKED && ((CAUSAL && (n0 + kBN - 1 > q_wave0)) || (n0 + kBN > p.Skv))) {
      // tile crossing the diagonal of a causal chunk, or a ragged last tile (wave-uniform branch)
      const int limit = CAUSAL ? min(qrow, p.Skv - 1) : p.Skv - 1;  // last visible key
#pragma unroll
      for (int kvb = 0; kvb < KVB; ++kvb)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          if (n0 + (kvb0 + kvb) * 32 + acc_row(v, g) > limit) s[kvb][v] = 0.f;
    }
#pragma unroll
    for (int kvb = 0; kvb < KVB; ++kvb) {
#pragma unroll
      for (int v = 0; v < 16; ++v) s[kvb][v] *= dp[kvb][v] - delta_q;
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
        dsf[2 * kvb + jj] = to_bf16x8(s[kvb][8 * jj], s[kvb][8 * jj + 1], s[kvb][8 * jj + 2], s[kvb][8 * jj + 3],
                                      s[kvb][8 * jj + 4], s[kvb][8 * jj + 5], s[kvb][8 * jj + 6], s[kvb][8 * jj + 7]);
    }
  };

  // Every interval ends by waiting until at most the loads of the last kDist - 1 intervals are
  // still in flight (the tiles of the next interval have landed), and a workgroup barrier.
  constexpr int kPerInterval = 2 * DirectTile128<kBN, kThreads>::kPerThread + (DQK == 192 ? 1 : 0);
  static_assert((kDist - 1) * kPerInterval < 16, "vmcnt immediate below assumes a 4-bit low field");
  auto land_and_sync = [&](bool steady) __attribute__((always_inline)) {
    if (steady) __builtin_amdgcn_s_waitcnt(0x0F70 | ((kDist - 1) * kPerInterval));
    else __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
  };
  auto kslot = [&](int t) __attribute__((always_inline)) { return kbuf + (t & (kSlots - 1)) * kKTile; };
  auto vslot = [&](int t) __attribute__((always_inline)) { return vbuf + (t & (kVSlots - 1)) * kTile; };

  // ---- prologue: S(0), dP(0) (and dS(0) in the early waves)
  __builtin_amdgcn_s_waitcnt(0x0F70);  // everything issued so far, the stationary fragments included
  __syncthreads();
  scores(kslot(0), vslot(0));
  if (!late) make_ds(0, std::true_type{});

  // Interval i = 0 .. n_tiles_wg - 1 reads K(i) (gradient product), K(i+1) and V(i+1) (scores) and
  // requests tile i + 1 + kDist, whose slots were last read in interval i - 1 (kDist 2: they held
  // tile i - 1) or hold nothing that is still needed (kDist 1: K slot of tile i - 2, V slot of tile i,
  // read in interval i - 1).
  // FULL: this wave has both a tile to accumulate and a next tile to score.
  // MASKED: the tile whose dS this interval makes (i + 1 in the early waves, i in the late ones) may
  // need the mask.
  auto interval = [&](int i, auto late_tag, auto full_tag, auto masked_tag) __attribute__((always_inline)) {
    constexpr bool LATE = decltype(late_tag)::value, FULL = decltype(full_tag)::value;
    const bool will_request = i + 1 + kDist < n_tiles_wg;
    refresh_offsets();
    if (!LATE) {
      if (FULL) {
        matrix_block(kslot(i), kslot(i + 1), vslot(i + 1));
        __builtin_amdgcn_sched_barrier(0);
        if (will_request) request(i + 1 + kDist);
        make_ds(i + 1, masked_tag);
      } else {
        if (i < n_tiles_wave) accumulate(kslot(i));
        if (will_request) request(i + 1 + kDist);
      }
    } else {
      if (will_request) request(i + 1 + kDist);
      if (FULL || i < n_tiles_wave) make_ds(i, masked_tag);
      __builtin_amdgcn_sched_barrier(0);
      if (FULL) matrix_block(kslot(i), kslot(i + 1), vslot(i + 1));
      else if (i < n_tiles_wave) accumulate(kslot(i));
    }
    land_and_sync(will_request);
  };
  // tiles [0, first_masked) need no mask for this wave: they lie below its diagonal and inside Skv
  int first_masked = p.Skv / kBN;
  if (CAUSAL) first_masked = min(first_masked, q_wave0 >= kBN - 1 ? (q_wave0 - (kBN - 1)) / kBN + 1 : 0);
  constexpr std::false_type no;
  constexpr std::true_type yes;
  if (!late) {
    int i = 0;
    for (; i + 1 < min(n_tiles_wave, first_masked); ++i) interval(i, no, yes, no);  // makes dS(i + 1)
    for (; i + 1 < n_tiles_wave; ++i) interval(i, no, yes, yes);
    for (; i < n_tiles_wg; ++i) interval(i, no, no, yes);
  } else {
    int i = 0;
    for (; i + 1 < n_tiles_wave && i < first_masked; ++i) interval(i, yes, yes, no);  // makes dS(i)
    for (; i + 1 < n_tiles_wave; ++i) interval(i, yes, yes, yes);
    for (; i < n_tiles_wg; ++i) interval(i, yes, no, yes);
  }

  // ---- the late wave of a pair hands its partial dQ to the early wave (the tile ring is free: every
  // wave passed the barrier that ends the last interval)
  // one area per wave pair; with 128 features it is used twice: for the late wave's partial dQ, then to turn the
  // early wave's result tile (the 192-feature kernel keeps the direct stores: it has no register to spare, and any
  // longer epilogue pushes spills into its main loop)
  constexpr bool kTurn = DQK == 128;
  constexpr int kExch = kTurn ? kRowsViaLdsBytes<DB> : DB * 4 * 64 * 16;
  static_assert(kExch >= DB * 4 * 64 * 16 && 4 * kExch <= (int)sizeof(smem), "exchange area");
  char* const exch = smem + (wave & 3) * kExch;
  if constexpr (!HALF) {
    OutT* dqh = reinterpret_cast<OutT*>(p.dq) + b * p.dq_bs + (int64_t)h * DQK;
    if (qrow < p.Sq) {
      OutT* dst = dqh + qrow * q_row_stride;
#pragma unroll
      for (int o = 0; o < DB; ++o)
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4)
          store4<OutT>(dst + 32 * o + 8 * b4 + 4 * g, acc[o][4 * b4] * p.scale, acc[o][4 * b4 + 1] * p.scale,
                       acc[o][4 * b4 + 2] * p.scale, acc[o][4 * b4 + 3] * p.scale, p.accumulate != 0);
    }
    return;
  }
  if (late) {
#pragma unroll
    for (int o = 0; o < DB; ++o)
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) {
        const f32x4 v4 = {acc[o][4 * b4], acc[o][4 * b4 + 1], acc[o][4 * b4 + 2], acc[o][4 * b4 + 3]};
        *reinterpret_cast<f32x4*>(exch + ((o * 4 + b4) * 64 + lane) * 16) = v4;
      }
  }
  __syncthreads();
  if (late) return;

  OutT* dqh = reinterpret_cast<OutT*>(p.dq) + b * p.dq_bs + (int64_t)h * DQK;
  if constexpr (kTurn) {
    // the pair's dQ^T (a lane owns one query row) is turned through LDS - the same area, once the partner's values
    // are in registers - so that the epilogue reads and writes whole rows
#pragma unroll
    for (int o = 0; o < DB; ++o)
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) {
        const f32x4 v4 = *reinterpret_cast<const f32x4*>(exch + ((o * 4 + b4) * 64 + lane) * 16);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[o][4 * b4 + e] += v4[e];
      }
    __bf16* fin = nullptr;  // rows whose gradient is complete with this call go out as bf16
    if (p.dq_final != nullptr && q_wave0 >= p.final_r0 && q_wave0 < p.final_r1)
      fin = p.dq_final + b * p.dq_final_bs + (int64_t)h * DQK + q_wave0 * q_row_stride;
    store_rows32_via_lds<OutT, DB>(exch, dqh + q_wave0 * q_row_stride, q_row_stride, p.Sq - q_wave0, acc, p.scale, p.accumulate != 0, lane, fin);
  } else if (qrow < p.Sq) {
    OutT* dst = dqh + qrow * q_row_stride;
    // rows whose gradient is complete with this call go out as bf16 (an fp32 dq only; the same for the whole wave)
    const bool fin = sizeof(OutT) == 4 && p.dq_final != nullptr && q_wave0 >= p.final_r0 && q_wave0 < p.final_r1;
    __bf16* fdst = p.dq_final + b * p.dq_final_bs + (int64_t)h * DQK + qrow * q_row_stride;
#pragma unroll
    for (int o = 0; o < DB; ++o)
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) {
        const f32x4 v4 = *reinterpret_cast<const f32x4*>(exch + ((o * 4 + b4) * 64 + lane) * 16);
        const int col = 32 * o + 8 * b4 + 4 * g;
        if (fin) {
          f32x4 x = {(acc[o][4 * b4] + v4[0]) * p.scale, (acc[o][4 * b4 + 1] + v4[1]) * p.scale,
                     (acc[o][4 * b4 + 2] + v4[2]) * p.scale, (acc[o][4 * b4 + 3] + v4[3]) * p.scale};
          if (p.accumulate) x += *reinterpret_cast<const f32x4*>(dst + col);
          store4<__bf16>(fdst + col, x[0], x[1], x[2], x[3], false);
        } else {
          store4<OutT>(dst + col, (acc[o][4 * b4] + v4[0]) * p.scale, (acc[o][4 * b4 + 1] + v4[1]) * p.scale,
                       (acc[o][4 * b4 + 2] + v4[2]) * p.scale, (acc[o][4 * b4 + 3] + v4[3]) * p.scale, p.accumulate != 0);
        }
      }
  }
}

template <int DQK, bool HALF>
void launch_one(const BwdParams& p, bool causal, bool f32_out, hipStream_t st) {
  const dim3 grid((unsigned)(p.tiles * p.Hq * p.B)), block(kThreads);
  if (causal) {
    if (f32_out) hipLaunchKernelGGL((attn_bwd_dq_direct_kernel<DQK, HALF, true, float>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((attn_bwd_dq_direct_kernel<DQK, HALF, true, __bf16>), grid, block, 0, st, p);
  } else {
    if (f32_out) hipLaunchKernelGGL((attn_bwd_dq_direct_kernel<DQK, HALF, false, float>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((attn_bwd_dq_direct_kernel<DQK, HALF, false, __bf16>), grid, block, 0, st, p);
  }
}

}  // namespace

void launch_dq_direct(const BwdParams& p, int dqk, bool causal, bool f32_out, hipStream_t st) {
  // only the HALF form is built: with all 64 keys of a tile per wave this organisation needs some 300
  // registers (the 256-row kernel for 128 features is attn_bwd_dq_d128.hip, organised differently)
  if (dqk == 192) launch_one<192, true>(p, causal, f32_out, st);
  else launch_one<128, true>(p, causal, f32_out, st);
}

}  // namespace pith
