// Chunk attention forward for head dims (128, 128) and (192, 128) on gfx950. Same function and
// numerics as the general kernel in attn_fwd.hip (pithtrain/operators/mla/triton.py:32-93,
// :274-323: fp32 scores from bf16 MFMA, P = exp2(kappa*(s - m)) in fp32, row sum from the fp32 P,
// P rounded to bf16 for P V, base-2 LSE, lazily refreshed running maximum), organised around two
// facts measured on the device:
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
//
// Head dim 192 (the MLA key: 128 + 64 features): a K tile is the packed 128-feature tile plus a
// second packed tile for features 128..191 that holds TWO keys per 256-byte row (key r in pieces
// 0-7, key r+32 in pieces 8-15 of row r), so that both are read with the same conflict-free
// swizzle.
//
// Two work splits. FULL: a workgroup owns 256 query rows, a wave 32 of them and all 64 keys of
// every tile. HALF: a workgroup owns 128 query rows; the two waves of a SIMD own the SAME 32 rows,
// the early one keys 0-31 and the late one keys 32-63 of every tile, each with its own running
// maximum, sum and accumulator, merged through LDS at the end. HALF doubles the number of
// workgroups (for launches that would leave compute units idle or badly balanced under the
// causal mask) and halves the registers per wave that depend on the tile width, at the price of
// half as many matrix instructions between two barriers.
#include <type_traits>

#include "attn_fwd_common.h"

namespace pith {
namespace {

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kBN = kFwdBlockN;   // keys per tile
constexpr int kDv = 128;
constexpr int kDist = 2;   // a tile is requested kDist intervals before the interval that reads it
constexpr int kSlots = 4;  // ring depth per operand, > kDist; a power of two (the slot index is a mask)
static_assert(kSlots > kDist && (kSlots & (kSlots - 1)) == 0, "ring depth");
constexpr int kAhead = 4;  // fragment reads run this many products ahead in the matrix block
constexpr int kTile = kBN * kRowBytes128;  // a packed 128-feature tile of 64 rows
constexpr int kExtraTile = kExtraTileBytes;  // features 128..191 of 64 keys, two keys per row

template <int DQK, bool HALF, bool CAUSAL>
__global__ __launch_bounds__(kThreads) void attn_fwd_direct_kernel(FwdParams p) {
  constexpr int KS = DQK / 16;    // contraction steps of Q K^T
  constexpr int DVB = kDv / 32;   // 32-row blocks of O^T
  constexpr int KVB = HALF ? 1 : 2;          // 32-key blocks of a tile this wave owns
  constexpr int kBM = HALF ? 128 : 256;      // query rows per workgroup
  constexpr int kKTile = kTile + (DQK == 192 ? kExtraTile : 0);
  static_assert(DQK == 128 || DQK == 192, "head dims");
  constexpr bool kSumTest = !(DQK == 192 && !HALF);  // how the softmax decides to refresh its running maximum
  // the tile rings; the epilogue reuses them to turn the output tile (one area per storing wave)
  constexpr int kRings = kSlots * (kKTile + kTile), kTurn = (HALF ? kWaves / 2 : kWaves) * kRowsViaLdsBytes<DVB>;
  // 256-row workgroups for 128 features fetch their query block through LDS as well (four 64-row tiles into the three
  // ring slots that are still empty while the first tiles land, and one more tile behind the rings): whole-row direct
  // loads instead of 32-byte pieces of 32 different rows per instruction
  constexpr bool kQViaLds = DQK == 128 && !HALF;
  constexpr int kQSpill = kRings;  // where the fourth query tile goes
  constexpr int kNeed = kQViaLds ? kRings + kTile : kRings;
  __shared__ __attribute__((aligned(1024))) char smem[kNeed > kTurn ? kNeed : kTurn];
  char* const kbuf = smem;
  char* const vbuf = smem + kSlots * kKTile;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, g = lane >> 5;
  const bool late = wave >= kWaves / 2;  // shares its SIMD with wave - kWaves/2
  const int kvb0 = HALF ? (wave >> 2) : 0;  // first 32-key block of a tile this wave owns

  int m_tile, h, b;
  decode_block(blockIdx.x, p.Hq, p.B, p.m_tiles, p.group, m_tile, h, b);
  const int hk = h / p.group;
  const int m0 = m_tile * kBM;
  const int q_wave0 = m0 + (HALF ? (wave & 3) : wave) * 32;
  const int qrow = q_wave0 + c;

  const int64_t q_row_stride = (int64_t)p.Hq * DQK;
  const int64_t o_row_stride = (int64_t)p.Hq * kDv;
  // keys in two parts: K rows hold 128 features per head, the last 64 come from k_pe (no head offset)
  const bool two_part = DQK == 192 && p.k_pe != nullptr;
  const int k_head_elems = two_part ? 128 : DQK;
  const int k_row_bytes = p.Hkv * k_head_elems * 2, v_row_bytes = p.Hkv * kDv * 2;
  const __bf16* qh = p.q + b * p.q_bs + (int64_t)h * DQK;
  const char* kh = reinterpret_cast<const char*>(p.k + b * p.k_bs + (int64_t)hk * k_head_elems);
  const char* kx = two_part ? reinterpret_cast<const char*>(p.k_pe + b * p.k_pe_bs) : kh;  // source of features 128..
  const int kx_row_bytes = two_part ? (int)p.k_pe_rs * 2 : k_row_bytes;
  const char* vh = reinterpret_cast<const char*>(p.v + b * p.v_bs + (int64_t)hk * kDv);

  // Number of key tiles this workgroup / this wavefront has to visit.
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
  auto issue_k = [&](int t) __attribute__((always_inline)) {
    char* slot = kbuf + (t & (kSlots - 1)) * kKTile;
    const char* src = kh + (int64_t)t * kBN * k_row_bytes;
    if constexpr (DQK != kDv) {
      kmover.issue(src, p.Skv - t * kBN, slot, wave, lane);
      xmover.issue(kx + (int64_t)t * kBN * kx_row_bytes, p.Skv - t * kBN, slot + kTile, wave, lane);
    } else {
      mover.issue(src, p.Skv - t * kBN, slot, wave, lane);
    }
  };
  auto issue_v = [&](int t) __attribute__((always_inline)) {
    mover.issue(vh + (int64_t)t * kBN * v_row_bytes, p.Skv - t * kBN, vbuf + (t & (kSlots - 1)) * kTile, wave, lane);
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
  // LDS homes of the workgroup's four 64-row query tiles (kQViaLds): K slot 3, V slots 2 and 3, behind the rings
  auto q_home = [&](int t) __attribute__((always_inline)) -> char* {
    return t == 0 ? kbuf + 3 * kKTile : t == 1 ? vbuf + 2 * kTile : t == 2 ? vbuf + 3 * kTile : smem + kQSpill;
  };
  if constexpr (kQViaLds) {
    DirectTile128<kBN, kThreads> qmover;
    qmover.init((int)(q_row_stride * 2), wave, lane);
    const char* qsrc = reinterpret_cast<const char*>(qh);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      // rows beyond Sq repeat the last row (their results are never stored); a tile wholly beyond Sq is skipped by
      // clamping its first row, which keeps the number of load instructions per wave fixed
      const int row0 = min(m0 + t * kBN, p.Sq - 1);
      qmover.issue(qsrc + (int64_t)row0 * q_row_stride * 2, p.Sq - row0, q_home(t), wave, lane);
    }
  } else {
    const int row = qrow < p.Sq ? qrow : p.Sq - 1;
    const __bf16* src = qh + row * q_row_stride + g * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(src + ks * 16);
  }

  // per-lane read offsets inside a tile. The swizzle is an XOR, so every offset is one base XOR a constant; only the
  // bases live in registers across the loop (refresh_offsets keeps the compiler from hoisting all derived values
  // back into registers, where they would push accumulators into scratch memory):
  //   k_off(ks): straight fragment of this wave's first key block, row c, contraction step ks. Steps 0..7 lie in
  //     the 128-feature tile (the next key block: + 32 rows = + 8192 bytes); steps 8.. in the extra tile behind it,
  //     whose row c holds key c in pieces 0-7 and key c + 32 in pieces 8-15 (the next key block: piece + 8, i.e.
  //     the offset with bit 7 flipped);
  //   v_off(i, hh): transposing reads of feature block i, lower / upper 8 keys (+ 16 keys: + 4096 bytes).
  int k_base = straight_offset128(c, g) + kvb0 * 32 * kRowBytes128;
  int x_base = kTile + straight_offset128(c, g + 8 * kvb0);
  int v_base[2] = {transposed_offset128(0, 0, 0, lane) + kvb0 * 32 * kRowBytes128,
                   transposed_offset128(0, 1, 0, lane) + kvb0 * 32 * kRowBytes128};
  // Only the variants that would spill otherwise pay the extra XOR per read (the 256-row causal kernels); the
  // others let the compiler keep every derived offset in a register.
  constexpr bool kDeriveOffsets = !HALF && CAUSAL;
  auto refresh_offsets = [&]() __attribute__((always_inline)) {
    if constexpr (kDeriveOffsets) {
      asm volatile("" : "+v"(k_base), "+v"(v_base[0]), "+v"(v_base[1]));
      if constexpr (DQK == 192) asm volatile("" : "+v"(x_base));
    }
  };
  auto k_off = [&](int ks) __attribute__((always_inline)) { return ks < 8 ? k_base ^ (ks << 5) : x_base ^ ((ks - 8) << 5); };
  auto v_off = [&](int i, int hh) __attribute__((always_inline)) { return v_base[hh] ^ (i << 6); };
  auto k_frag = [&](const char* ktile, int ks, int kvb) __attribute__((always_inline)) {
    const int off = ks < 8 ? k_off(ks) + kvb * 32 * kRowBytes128 : (kvb ? k_off(ks) ^ 128 : k_off(ks));
    return *reinterpret_cast<const bf16x8*>(ktile + off);
  };

  f32x16 oacc[DVB];
#pragma unroll
  for (int i = 0; i < DVB; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[i][v] = 0.f;
  float m_run = -INFINITY;
  float l_run = 0.f;  // this lane's share of the row sum (the partner lane holds the rest)

  f32x16 s[KVB];       // S^T of this wave's keys of one tile: 32 x 32 tiles [keys] x [queries]
  bf16x8 pf[2 * KVB];  // P^T of the same keys as B operand, one fragment per 16 keys

  // ---- S^T = K Q^T
  auto scores = [&](const char* ktile) __attribute__((always_inline)) {
#pragma unroll
    for (int kvb = 0; kvb < KVB; ++kvb)
#pragma unroll
      for (int v = 0; v < 16; ++v) s[kvb][v] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int kvb = 0; kvb < KVB; ++kvb) s[kvb] = mfma32(k_frag(ktile, ks, kvb), qf[ks], s[kvb]);
  };

  // ---- mask, online softmax (one query column per lane pair), P^T fragments
  auto softmax = [&](int t) __attribute__((always_inline)) {
    const int n0 = t * kBN;
    if ((CAUSAL && (n0 + kBN - 1 > q_wave0)) || (n0 + kBN > p.Skv)) {
      // tile crossing the diagonal of a causal chunk, or a ragged last tile
      const int limit = CAUSAL ? min(qrow, p.Skv - 1) : p.Skv - 1;  // last visible key
#pragma unroll
      for (int kvb = 0; kvb < KVB; ++kvb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int key = n0 + (kvb0 + kvb) * 32 + acc_row(v, g);
          if (key > limit) s[kvb][v] = -INFINITY;
        }
    }
    f32x16 e[KVB];
    float rs = 0.f;
    if constexpr (kSumTest) {
      // The running maximum is refreshed lazily, and whether a refresh is due is read off the row sum instead of a
      // maximum over the tile: every term of the sum is >= 0, so a lane's partial sum within kRescaleLimit means that
      // none of its P values exceeds kRescaleLimit either. The common tile then costs no maximum at all (24 of the
      // ~140 vector instructions per tile); a tile that fails the test (the first tile of a row, tiles where the scores
      // still climb, and any overflow or NaN) is redone from the scores, which are kept until the test has passed.
      const bool fresh = m_run == -INFINITY;
      float mk = fresh ? 0.f : m_run * p.kappa;
#pragma unroll
      for (int kvb = 0; kvb < KVB; ++kvb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          e[kvb][v] = __builtin_amdgcn_exp2f(s[kvb][v] * p.kappa - mk);
          rs += e[kvb][v];
        }
      if (__builtin_amdgcn_ballot_w64(fresh || !(rs <= kRescaleLimit)) != 0) {  // wave-uniform, rare
        float x = s[0][0];
#pragma unroll
        for (int kvb = 0; kvb < KVB; ++kvb)
#pragma unroll
          for (int v = 0; v < 16; ++v) x = fmaxf(x, s[kvb][v]);
        const float m_new = fmaxf(m_run, pair_max(x));
        // a row with no visible key so far keeps m = -inf; exp2 of (-inf - -inf) is avoided
        const float alpha = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f((m_run - m_new) * p.kappa);
        m_run = m_new;
        l_run *= alpha;
#pragma unroll
        for (int i = 0; i < DVB; ++i)
#pragma unroll
          for (int v = 0; v < 16; ++v) oacc[i][v] *= alpha;
        mk = (m_run == -INFINITY) ? 0.f : m_run * p.kappa;
        rs = 0.f;
#pragma unroll
        for (int kvb = 0; kvb < KVB; ++kvb)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            e[kvb][v] = __builtin_amdgcn_exp2f(s[kvb][v] * p.kappa - mk);
            rs += e[kvb][v];
          }
      }
    } else {
      // the 256-row kernels for 192-feature keys have no registers for a second score tile: tile maximum first
      float x = s[0][0];
#pragma unroll
      for (int kvb = 0; kvb < KVB; ++kvb)
#pragma unroll
        for (int v = 0; v < 16; ++v) x = fmaxf(x, s[kvb][v]);
      const float mx = pair_max(x);
      const bool refresh = (mx - m_run) * p.kappa > kRescaleThreshold;  // true on the first tile (m = -inf)
      if (__builtin_amdgcn_ballot_w64(refresh) != 0) {                   // wave-uniform
        const float m_new = fmaxf(m_run, mx);
        const float alpha = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f((m_run - m_new) * p.kappa);
        m_run = m_new;
        l_run *= alpha;
#pragma unroll
        for (int i = 0; i < DVB; ++i)
#pragma unroll
          for (int v = 0; v < 16; ++v) oacc[i][v] *= alpha;
      }
      const float mk = (m_run == -INFINITY) ? 0.f : m_run * p.kappa;
#pragma unroll
      for (int kvb = 0; kvb < KVB; ++kvb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          e[kvb][v] = __builtin_amdgcn_exp2f(s[kvb][v] * p.kappa - mk);
          rs += e[kvb][v];
        }
    }
    l_run += rs;
#pragma unroll
    for (int kvb = 0; kvb < KVB; ++kvb)
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        const f32x16& x16 = e[kvb];
        pf[2 * kvb + jj] = to_bf16x8(x16[8 * jj], x16[8 * jj + 1], x16[8 * jj + 2], x16[8 * jj + 3], x16[8 * jj + 4],
                                     x16[8 * jj + 5], x16[8 * jj + 6], x16[8 * jj + 7]);
      }
  };

  // ---- O^T += V^T P^T
  auto accumulate = [&](const char* vtile) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 2 * KVB; ++j)
#pragma unroll
      for (int i = 0; i < DVB; ++i) {
        const bf16x8 a = lds_read_transposed_at(vtile + v_off(i, 0) + j * 16 * kRowBytes128,
                                                vtile + v_off(i, 1) + j * 16 * kRowBytes128);
        oacc[i] = mfma32(a, pf[j], oacc[i]);
      }
  };

  // ---- matrix block of one interval: O^T += V^T P^T of one tile, then S^T of the next, with
  // the fragment reads pinned kAhead products ahead of their use.
  auto matrix_block = [&](const char* vtile, const char* ktile) __attribute__((always_inline)) {
    constexpr int NPV = 2 * KVB * DVB, NQK = KVB * KS;
    static_assert(kAhead <= NPV, "look-ahead assumes it starts inside the P V product");
    __builtin_amdgcn_s_setprio(2);  // the wave that owns the matrix pipe issues first
    bf16x8 av[2 * KVB][DVB], ak[KS][KVB];
#pragma unroll
    for (int j = 0; j < 2 * KVB; ++j)
#pragma unroll
      for (int i = 0; i < DVB; ++i)
        av[j][i] = lds_read_transposed_at(vtile + v_off(i, 0) + j * 16 * kRowBytes128,
                                          vtile + v_off(i, 1) + j * 16 * kRowBytes128);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int kvb = 0; kvb < KVB; ++kvb) ak[ks][kvb] = k_frag(ktile, ks, kvb);
#pragma unroll
    for (int j = 0; j < 2 * KVB; ++j)
#pragma unroll
      for (int i = 0; i < DVB; ++i) oacc[i] = mfma32(av[j][i], pf[j], oacc[i]);
#pragma unroll
    for (int kvb = 0; kvb < KVB; ++kvb)
#pragma unroll
      for (int v = 0; v < 16; ++v) s[kvb][v] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int kvb = 0; kvb < KVB; ++kvb) s[kvb] = mfma32(ak[ks][kvb], qf[ks], s[kvb]);
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
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_setprio(0);
  };

  // ---- prologue: S(0) (and P(0) in the early waves) from K tile 0
  __builtin_amdgcn_s_waitcnt(0x0F70);  // everything issued so far, Q fragments included
  __syncthreads();
  if constexpr (kQViaLds) {
    // this wave's 32 rows: tile wave / 2, row block wave % 2 (the slots are refilled only after the next barrier)
    const char* qt = q_home(wave >> 1) + (wave & 1) * 32 * kRowBytes128;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qt + straight_offset128(c, 2 * ks + g));
  }
  scores(kbuf);
  __syncthreads();  // K tile 0 has been read by every wave: its slot may be refilled
  if (!late) softmax(0);

  // One interval; FULL: this wave has both a tile to accumulate and a next tile to score.
  // Intervals come in pairs (even, odd): the even one requests the tiles of BOTH intervals of the pair after next
  // (K i+3, i+4 and V i+2, i+3), the odd one ends with the wait for those loads and the workgroup barrier. A slot
  // that is refilled was last read before the barrier that precedes the request, and everything an interval reads
  // had landed before the barrier that precedes the pair. PAIR: 1 = even, 2 = odd, 0 = decided from i at run time.
  auto interval = [&](int i, auto late_tag, auto full_tag, auto pair_tag) __attribute__((always_inline)) {
    constexpr bool LATE = decltype(late_tag)::value, FULL = decltype(full_tag)::value;
    constexpr int PAIR = decltype(pair_tag)::value;
    const bool even = PAIR == 1 || (PAIR == 0 && !(i & 1));
    const char* vtile = vbuf + (i & (kSlots - 1)) * kTile;
    const char* ktile = kbuf + ((i + 1) & (kSlots - 1)) * kKTile;
    refresh_offsets();
    // Requests are placed where no LDS read of the same wave follows closely: after the matrix
    // block in the early waves, before the vector block in the late ones.
    auto request = [&]() __attribute__((always_inline)) {
      if constexpr (PAIR != 2) {
        if (even) {
          if (i + 3 < n_tiles_wg) issue_k(i + 3);
          if (i + 2 < n_tiles_wg) issue_v(i + 2);
          if (i + 4 < n_tiles_wg) issue_k(i + 4);
          if (i + 3 < n_tiles_wg) issue_v(i + 3);
        }
      }
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
    if (PAIR == 2 || !even || i + 1 == n_tiles_wg) {  // the same decision in every wave of the workgroup
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
    }
  };
  // A merging launch reads 8-16 KB of running output per wave in its epilogue, every compute unit of the device at
  // the same moment, from memory that nothing has touched since the previous launch. One or two intervals before the
  // end every lane therefore touches one 128-byte line of its wave's rows (the 4 bytes land in the LDS area behind the
  // rings, which nobody reads any more), so that the epilogue finds the rows in L2. The loads complete, like the tile
  // loads, before the wait that ends the next pair of intervals.
  auto warm_previous_rows = [&]() __attribute__((always_inline)) {
    if (p.prev_o == nullptr) return;
    const int row_bytes = p.prev_f32 ? kDv * 4 : kDv * 2;               // 4 or 2 lines per row
    const int per_row = row_bytes >> 7;
    const int64_t prev_rs = o_row_stride * (p.prev_f32 ? 4 : 2);
    const char* base = reinterpret_cast<const char*>(p.prev_o) + (b * p.prev_bs + (int64_t)h * kDv) * (p.prev_f32 ? 4 : 2);
    char* const dump = smem + kQSpill + wave * 256;
    for (int idx = lane; idx < 32 * per_row; idx += 64) {  // wave-uniform trip count: 1 or 2
      const int row = min(q_wave0 + idx / per_row, p.Sq - 1);
      load_lds4(base + row * prev_rs + (idx % per_row) * 128, dump);
    }
  };
  // Every wave passes the same number of barriers; the two roles run separate loops so that
  // each loop body is straight-line code around one accumulator set.
  auto run = [&](auto late_tag) __attribute__((always_inline)) {
    using Full = std::true_type;
    using Part = std::false_type;
    int i = 0;
    // the pair as one loop body (no parity tests, the odd interval without request code) wherever two copies of the
    // interval still fit the registers
    if constexpr (!(DQK == 192 && !HALF)) {
      for (; i + 2 < n_tiles_wave; i += 2) {
        interval(i, late_tag, Full{}, std::integral_constant<int, 1>{});
        interval(i + 1, late_tag, Full{}, std::integral_constant<int, 2>{});
      }
    }
    if constexpr (kQViaLds && !CAUSAL) warm_previous_rows();
    for (; i + 1 < n_tiles_wave; ++i) interval(i, late_tag, Full{}, std::integral_constant<int, 0>{});
    for (; i < n_tiles_wg; ++i) interval(i, late_tag, Part{}, std::integral_constant<int, 0>{});
  };
  if (!late) run(std::false_type{});
  else run(std::true_type{});

  // ---- HALF: the late wave of a pair hands its accumulator, maximum and sum to the early wave,
  // which rescales both to the common maximum and adds them. The tile ring is free by now (every
  // wave passed the barrier that ends the last interval).
  if constexpr (HALF) {
    constexpr int kExch = 16 * 64 * 16 + 64 * 8;  // 64 accumulator values and (m, l) per lane
    char* const exch = smem + (wave & 3) * kExch;
    if (late) {
#pragma unroll
      for (int i = 0; i < DVB; ++i)
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4) {
          const f32x4 v4 = {oacc[i][4 * b4], oacc[i][4 * b4 + 1], oacc[i][4 * b4 + 2], oacc[i][4 * b4 + 3]};
          *reinterpret_cast<f32x4*>(exch + ((i * 4 + b4) * 64 + lane) * 16) = v4;
        }
      const f32x2 ml = {m_run, l_run};
      *reinterpret_cast<f32x2*>(exch + 16 * 64 * 16 + lane * 8) = ml;
    }
    __syncthreads();
    if (late) return;
    const f32x2 ml = *reinterpret_cast<const f32x2*>(exch + 16 * 64 * 16 + lane * 8);
    const float m_new = fmaxf(m_run, ml[0]);
    // a side that saw no key has m = -inf, l = 0 and a zero accumulator: weight 0
    const float a_e = (m_run == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m_run - m_new) * p.kappa);
    const float a_l = (ml[0] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((ml[0] - m_new) * p.kappa);
    m_run = m_new;
    l_run = l_run * a_e + ml[1] * a_l;
#pragma unroll
    for (int i = 0; i < DVB; ++i)
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) {
        const f32x4 v4 = *reinterpret_cast<const f32x4*>(exch + ((i * 4 + b4) * 64 + lane) * 16);
#pragma unroll
        for (int e = 0; e < 4; ++e) oacc[i][4 * b4 + e] = oacc[i][4 * b4 + e] * a_e + v4[e] * a_l;
      }
  }

  // ---- epilogue: normalise, store O (bf16) and LSE2
  __bf16* oh = p.o + b * p.o_bs + (int64_t)h * kDv;
  float* lse = p.lse + b * p.lse_bs + (int64_t)h * p.lse_hs;
  const float l = pair_sum(l_run);
  const float inv = l > 0.f ? 1.f / l : 0.f;
  if constexpr (!CAUSAL) {
    if (p.prev_o != nullptr) {  // the same for the whole launch
      // ---- merging epilogue: the ring's log2-domain online-softmax combine of this chunk's (O, LSE2) with the running
      // (prev_o, lse) of the rows: M = max(l1, l2), w = 2^(l - M), out = (w1 o1 + w2 o2) / (w1 + w2),
      // lse = M + log2(w1 + w2). The chunk's O is acc / l, so its weight and 1 / l fold into one factor per row.
      const float lse_new = l > 0.f ? __builtin_amdgcn_logf(l) + m_run * p.kappa : -INFINITY;
      const float lse_old = qrow < p.Sq ? lse[qrow] : -INFINITY;
      const float big = fmaxf(lse_old, lse_new);
      // both sides empty (-inf): weights 0, result (0, -inf); the ring never gets there (it starts from finfo.min)
      const float w_old = big == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(lse_old - big);
      const float w_new = big == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(lse_new - big);
      const float den = w_old + w_new;
      const float rden = den > 0.f ? 1.f / den : 0.f;
      char* const turn = smem + (HALF ? (wave & 3) : wave) * kRowsViaLdsBytes<DVB>;
      const int64_t prev_rs = o_row_stride;  // the three tensors share the [.., Hq, 128] row layout
      const char* prev = reinterpret_cast<const char*>(p.prev_o) +
                         (b * p.prev_bs + (int64_t)h * kDv + q_wave0 * prev_rs) * (p.prev_f32 ? 4 : 2);
      // which of the two outputs this wave's 32 rows go to (the ranges lie on multiples of 32 rows)
      const bool to_o = p.o && q_wave0 >= p.o_r0 && q_wave0 < p.o_r1;
      const bool to_acc = p.acc_o && q_wave0 >= p.acc_r0 && q_wave0 < p.acc_r1;
      merge_rows32_via_lds<DVB>(turn, prev, p.prev_f32 != 0, prev_rs, to_o ? oh + q_wave0 * o_row_stride : nullptr, o_row_stride,
                                to_acc ? p.acc_o + b * p.acc_bs + (int64_t)h * kDv + q_wave0 * o_row_stride : nullptr,
                                o_row_stride, p.Sq - q_wave0, oacc, w_new * inv * rden, w_old * rden, lane);
      if (qrow < p.Sq && g == 0) lse[qrow] = den > 0.f ? big + __builtin_amdgcn_logf(den) : -INFINITY;
      return;
    }
  }
  // O^T sits in the accumulators (a lane owns one query row): turned through LDS so that the stores
  // cover whole rows. Every wave is past the barrier behind the last tile read (HALF: past the merge).
  // (Not in the 256-row causal kernel for 192-feature keys, which has no register to spare: the extra
  // live values of the turned epilogue push spills into its main loop.)
  if constexpr (!(DQK == 192 && !HALF && CAUSAL)) {
    char* const turn = smem + (HALF ? (wave & 3) : wave) * kRowsViaLdsBytes<DVB>;
    store_rows32_via_lds<__bf16, DVB>(turn, oh + q_wave0 * o_row_stride, o_row_stride, p.Sq - q_wave0, oacc, inv, false, lane);
  } else if (qrow < p.Sq) {
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
  }
  if (qrow < p.Sq && g == 0) lse[qrow] = (l > 0.f) ? __builtin_amdgcn_logf(l) + m_run * p.kappa : -INFINITY;
}

template <int DQK, bool HALF>
void launch_one(FwdParams p, bool causal, hipStream_t st) {
  constexpr int kBM = HALF ? 128 : 256;
  p.m_tiles = (p.Sq + kBM - 1) / kBM;
  const dim3 grid((unsigned)(p.m_tiles * p.Hq * p.B)), block(kThreads);
  if (causal) hipLaunchKernelGGL((attn_fwd_direct_kernel<DQK, HALF, true>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((attn_fwd_direct_kernel<DQK, HALF, false>), grid, block, 0, st, p);
}

}  // namespace

void launch_fwd_direct(const FwdParams& p, int dqk, bool causal, bool half, hipStream_t st) {
  if (dqk == 128) {
    if (half) launch_one<128, true>(p, causal, st);
    else launch_one<128, false>(p, causal, st);
  } else {
    if (half) launch_one<192, true>(p, causal, st);
    else launch_one<192, false>(p, causal, st);
  }
}

}  // namespace pith
