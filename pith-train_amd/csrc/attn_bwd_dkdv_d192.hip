// Key/value-gradient kernel for head dims (192, 128) on gfx950 (the MLA shape). Same function and
// numerics as the 128-dim kernel of attn_bwd_dkdv_d128.hip (pithtrain/operators/mla/triton.py:130-197,
// :331-384: P = exp2(kappa*s - lse2) in fp32, masked entries 0, P rounded to bf16 for dV += P^T dO,
// dS = P*(dP - delta) rounded to bf16 for dK += dS^T Q, the factor `scale` applied once to the
// accumulated dK, fp32 accumulation) and the same design:
//   - a workgroup of 8 wavefronts owns 128 key rows of one (batch, kv head); the wavefronts form 4
//     pairs (SIMD siblings), one per 32 keys; wave A of a pair holds K and dV, wave B holds V and dK;
//   - Q / dO tiles and the lse / delta rows go global -> LDS directly into a ring of three stages,
//     requested one interval ahead; tiles are packed and swizzled;
//   - B runs one tile behind A: in interval i wave A computes dV(i-1), S(i), P(i), wave B computes
//     dS(i-1), dK(i-1), dP(i); A runs [matrix block | vector block], B [vector block | matrix block]
//     with a workgroup barrier at "|" and at the end of the interval; A hands the fp32 P tile to B
//     through an LDS buffer per pair.
// What the 192 features change: a wave's stationary fragments and accumulators are 12 + 4x16
// (A: K, dV) and 8 + 6x16 (B: V, dK) registers, 32 more in B than at 128 features. Query tiles of
// 64 rows still fit 256 registers because the per-lane tile offsets are derived by XOR from five
// bases and B forms dS one 32-row block at a time; both waves issue 40 MFMAs per interval
// (A: 16 + 24, B: 24 + 16). The kernel is written for tiles of 32 * TB rows, TB = 1 or 2. The
// trailing 64 features of a Q tile form a second packed tile with two tile rows per 256-byte LDS
// row (row r in pieces 0-7, row r + 16*TB in pieces 8-15), so the swizzle and both read patterns of
// the 128-feature tiles apply to it.
// Keys in two parts (p.k_pe): K's trailing 64 features come from k_pe, their gradient goes per head
// to p.ws_dkpe (the caller adds the heads), dk has 128 features per head.
#include <type_traits>

#include "attn_bwd_common.h"

namespace pith {
namespace {

constexpr int kThreads = 512;
constexpr int kBN = kDkdvBlockN;    // key rows per workgroup
constexpr int kDQ = 192, kDV = 128;
constexpr int kStages = 3;          // tiles i-1, i (in use) and i+1 (landing)
constexpr int kAhead = 4;           // fragment reads run this many products ahead

// LDS layout for query tiles of 32 * TB rows
template <int TB>
struct Layout {
  static constexpr int kBM = 32 * TB;
  static constexpr int kQMain = kBM * kRowBytes128;         // features 0..127 of the Q tile
  static constexpr int kQExtra = (kBM / 2) * kRowBytes128;  // features 128..191, two tile rows per LDS row
  static constexpr int kOTile = kBM * kRowBytes128;
  static constexpr int kStat = 2 * kBM * 4;                 // lse[kBM], delta[kBM]
  static constexpr int kOffExtra = kQMain, kOffO = kQMain + kQExtra, kOffStat = kOffO + kOTile;
  static constexpr int kStage = kOffStat + kStat;
  static constexpr int kExchPair = kBM * 32 * 4;            // one kBM x 32 fp32 P tile
  static constexpr int kSmem = kStages * kStage + 4 * kExchPair;
};

// Position of a query tile in the stream of (query head, tile) pairs a workgroup visits.
struct TileCursor {
  int hq, mt;
  __device__ __forceinline__ void advance(int m_first, int m_end) {
    if (++mt == m_end) {
      mt = m_first;
      ++hq;
    }
  }
};

// Features 128..191 of a tile of 2*H rows, global memory -> LDS: H LDS rows of 256 bytes, LDS row r
// holding tile row r in pieces 0-7 and tile row r + H in pieces 8-15; one global_load_lds per lane of
// the wavefronts 0 .. H/4-1 (wave w fills LDS rows 4w .. 4w+3).
template <int H>
struct DirectExtra {
  static constexpr int kWaves = H / 4;
  int src_off, row_bytes;
  __device__ __forceinline__ static int source(int row_bytes, int wave, int lane, int rows_left) {
    const int row = 4 * wave + (lane >> 4);
    const int piece = (lane & 15) ^ tile_swizzle(row);
    int r = row + H * (piece >> 3);
    r = r < rows_left ? r : rows_left - 1;
    return r * row_bytes + 256 + ((piece & 7) << 4);
  }
  __device__ __forceinline__ void init(int row_bytes_, int wave, int lane) {
    row_bytes = row_bytes_;
    src_off = source(row_bytes_, wave & (kWaves - 1), lane, 2 * H);
  }
  __device__ __forceinline__ void issue(const char* tile_src, int rows_left, char* slot, int wave, int lane) const {
    if (rows_left >= 2 * H) load_lds16(tile_src, src_off, slot + wave * 1024);
    else load_lds16(tile_src, source(row_bytes, wave, lane, rows_left), slot + wave * 1024);
  }
};

template <int TB, bool CAUSAL, typename OutT>
__global__ __launch_bounds__(kThreads) void attn_bwd_dkdv_d192_kernel(BwdParams p) {
  using L = Layout<TB>;
  constexpr int kBM = L::kBM, kStage = L::kStage, kOffExtra = L::kOffExtra, kOffO = L::kOffO, kOffStat = L::kOffStat;
  constexpr int kExchPair = L::kExchPair;
  constexpr int KS = kDQ / 16, VS = kDV / 16, DB = kDQ / 32, DVB = kDV / 32;
  __shared__ __attribute__((aligned(1024))) char smem[L::kSmem];

  const int tid = threadIdx.x;
  if ((int)blockIdx.x >= p.main_blocks) {  // workgroups appended to the grid: clear the rows behind the chunk's visible part
    zero_tail_block<OutT>(p, (int)blockIdx.x - p.main_blocks, p.k_pe ? 128 : kDQ, kDV, tid, kThreads);
    return;
  }
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, g = lane >> 5;
  const int pair = wave & 3;
  const bool role_b = wave >= 4;

  // linear block id -> (key tile, kv head, batch, head part)
  const int per_level = p.Hkv * p.B * p.split;
  int n_tile, pos;
  decode_dkdv_block(blockIdx.x, per_level, p.tiles, n_tile, pos);
  const int part = pos % p.split;
  pos /= p.split;
  const int hk = pos % p.Hkv, b = pos / p.Hkv;
  const int heads_per_part = p.group / p.split;
  const int hq0 = hk * p.group + part * heads_per_part;

  const int kv_wg0 = n_tile * kBN;
  const int kv_pair0 = kv_wg0 + pair * 32;
  const int key = kv_pair0 + c;

  const int q_row_bytes = p.HqT * kDQ * 2, do_row_bytes = p.HqT * kDV * 2;
  const bool two_part = p.k_pe != nullptr;
  const int k_head = two_part ? 128 : kDQ;
  const int64_t k_row_stride = (int64_t)p.HkvT * k_head;
  const int64_t v_row_stride = (int64_t)p.HkvT * kDV;

  // Query tiles to visit: all of them, or from the diagonal down under the causal mask.
  const int m_end = (p.Sq + kBM - 1) / kBM;
  const int m_first = CAUSAL ? min(kv_wg0 / kBM, m_end) : 0;
  const int n_iter = (m_end - m_first) * heads_per_part;

  // ---- requests: issued by the four B waves only (their vector block, dS, is the shorter one)
  using Extra = DirectExtra<kBM / 2>;
  DirectTile128<kBM, kThreads / 2> q_mover, o_mover;
  Extra e_mover[2];  // LDS rows 4*pair .. +3 and, where the extra tile has them, 4*(pair + 4) .. +3
  q_mover.init(q_row_bytes, pair, lane);
  o_mover.init(do_row_bytes, pair, lane);
  e_mover[0].init(q_row_bytes, pair, lane);
  e_mover[1].init(q_row_bytes, pair + 4, lane);
  const char* q_base = reinterpret_cast<const char*>(p.q + b * p.q_bs);
  const char* do_base = reinterpret_cast<const char*>(p.dout + b * p.dout_bs);
  TileCursor req = {hq0, m_first};
  auto request = [&](char* stage) __attribute__((always_inline)) {
    const int row0 = req.mt * kBM;
    const char* q_src = q_base + (int64_t)req.hq * kDQ * 2 + (int64_t)row0 * q_row_bytes;
    q_mover.issue(q_src, p.Sq - row0, stage, pair, lane);
    o_mover.issue(do_base + (int64_t)req.hq * kDV * 2 + (int64_t)row0 * do_row_bytes, p.Sq - row0, stage + kOffO, pair, lane);
    e_mover[0].issue(q_src, p.Sq - row0, stage + kOffExtra, pair, lane);
    if constexpr (Extra::kWaves > 4) e_mover[1].issue(q_src, p.Sq - row0, stage + kOffExtra, pair + 4, lane);
    // the tile's lse and delta rows: [lse kBM | delta kBM] floats, 64 per wavefront instruction
    if (TB == 1 ? pair == 0 : pair < 2) {
      const int idx = TB == 1 ? lane : pair * 64 + lane;  // position in the stats area
      int row = row0 + (idx & (kBM - 1));
      row = row < p.Sq ? row : p.Sq - 1;
      const float* src = (idx < kBM ? p.lse : p.delta) + b * p.lse_bs + (int64_t)req.hq * p.lse_hs + row;
      load_lds4(src, stage + kOffStat + (TB == 1 ? 0 : pair * 256));
    }
    req.advance(m_first, m_end);
  };
  if (n_iter > 0 && role_b) request(smem);

  // stationary fragments: K rows for wave A (12), V rows for wave B (8)
  bf16x8 stat[KS];
  {
    const int row = key < p.Skv ? key : p.Skv - 1;
    if (!role_b) {
      const __bf16* src = p.k + b * p.k_bs + row * k_row_stride + (int64_t)hk * k_head + g * 8;
      const __bf16* src_pe = two_part ? p.k_pe + b * p.k_pe_bs + row * p.k_pe_rs + g * 8 : src + 128;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        stat[ks] = *reinterpret_cast<const bf16x8*>(ks < 8 ? src + ks * 16 : src_pe + (ks - 8) * 16);
    } else {
      const __bf16* src = p.v + b * p.v_bs + row * v_row_stride + (int64_t)hk * kDV + g * 8;
#pragma unroll
      for (int ks = 0; ks < VS; ++ks) stat[ks] = *reinterpret_cast<const bf16x8*>(src + ks * 16);
      // wave B works with -V: its score-type product then starts from delta and yields delta - dP,
      // i.e. -(dP - delta) without a subtraction per element; the factor -scale on the accumulated dK
      // undoes the sign
#pragma unroll
      for (int ks = 0; ks < VS; ++ks) stat[ks] = __builtin_bit_cast(bf16x8, __builtin_bit_cast(u32x4, stat[ks]) ^ 0x80008000u);
    }
  }
  f32x16 acc[DB];  // A uses the first DVB of them
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;

  // per-lane read offsets inside the tiles; the others follow by XOR with a constant (the swizzle is
  // an XOR of the piece index): straight fragment of contraction step ks = s_base ^ (ks << 5),
  // transposing read of feature block o = t_base[hh] ^ (o << 6).
  const int s_base = straight_offset128(c, g);                              // 128-feature tiles, row c
  // extra tile, tile row 32*rb + c: with 32-row tiles rows c and c + 16 share LDS row c % 16, with
  // 64-row tiles rows c and c + 32 share LDS row c (then the 32-row block rb selects pieces 8*rb ..)
  const int se_base = TB == 1 ? straight_offset128(c & 15, g + 8 * (c >> 4)) : s_base;
  const int t_base[2] = {transposed_offset128(0, 0, 0, lane), transposed_offset128(0, 1, 0, lane)};

  char* const exch = smem + kStages * kStage + pair * kExchPair;

  f32x16 x[TB];         // [32-row block] A: S, then P of the current tile. B: dP, kept into the next interval
  bf16x8 frag[2 * TB];  // [16-row step] A: P(i) as B operand of dV(i) in the next interval. B: dS(i-1) for dK(i-1)

  // fragment (contraction step ks, 32-row block rb) of the score-type product of the tile in `stage`
  // (A: Q straight, 12 steps; B: dO straight, 8 steps)
  auto straight_frag = [&](const char* stage, int ks, int rb, auto role_tag) __attribute__((always_inline)) -> bf16x8 {
    if constexpr (decltype(role_tag)::value)
      return *reinterpret_cast<const bf16x8*>(stage + kOffO + rb * 32 * kRowBytes128 + (s_base ^ (ks << 5)));
    else if (ks < 8) return *reinterpret_cast<const bf16x8*>(stage + rb * 32 * kRowBytes128 + (s_base ^ (ks << 5)));
    else return *reinterpret_cast<const bf16x8*>(stage + kOffExtra + (se_base ^ ((ks - 8) << 5) ^ (TB == 1 ? 0 : rb << 7)));
  };
  // fragment (16-row step j, feature block o) of the gradient-type product (A: dO transposed, 4
  // blocks; B: Q transposed, 6 blocks, the last two from the extra tile, where 16-row step j sits in
  // LDS rows 16*(j % TB) .. and pieces 8*(j / TB) .. 8*(j / TB) + 7)
  auto transposed_frag = [&](const char* stage, int j, int o, auto role_tag) __attribute__((always_inline)) -> bf16x8 {
    if constexpr (!decltype(role_tag)::value) {
      const char* base = stage + kOffO + j * 16 * kRowBytes128;
      return lds_read_transposed_at(base + (t_base[0] ^ (o << 6)), base + (t_base[1] ^ (o << 6)));
    } else if (o < 4) {
      const char* base = stage + j * 16 * kRowBytes128;
      return lds_read_transposed_at(base + (t_base[0] ^ (o << 6)), base + (t_base[1] ^ (o << 6)));
    } else {
      const char* base = stage + kOffExtra + (j % TB) * 16 * kRowBytes128;
      const int piece_bits = (8 * (j / TB) + 4 * (o - 4)) << 4;
      return lds_read_transposed_at(base + (t_base[0] ^ piece_bits), base + (t_base[1] ^ piece_bits));
    }
  };

  // x starts from 0 in wave A and from the delta values of the tile's rows in wave B
  auto start_x = [&](const char* stage, auto role_tag) __attribute__((always_inline)) {
    if constexpr (decltype(role_tag)::value) {
      const float* delta_s = reinterpret_cast<const float*>(stage + kOffStat) + kBM;
#pragma unroll
      for (int rb = 0; rb < TB; ++rb)
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4) {
          const f32x4 d = *reinterpret_cast<const f32x4*>(delta_s + 32 * rb + 8 * b4 + 4 * g);
#pragma unroll
          for (int e = 0; e < 4; ++e) x[rb][4 * b4 + e] = d[e];
        }
    } else {
#pragma unroll
      for (int rb = 0; rb < TB; ++rb)
#pragma unroll
        for (int v = 0; v < 16; ++v) x[rb][v] = 0.f;
    }
  };
  auto straight_product = [&](const char* stage, auto role_tag) __attribute__((always_inline)) {
    constexpr int NS = decltype(role_tag)::value ? VS : KS;
    start_x(stage, role_tag);
#pragma unroll
    for (int ks = 0; ks < NS; ++ks)
#pragma unroll
      for (int rb = 0; rb < TB; ++rb) x[rb] = mfma32(straight_frag(stage, ks, rb, role_tag), stat[ks], x[rb]);
  };
  auto transposed_product = [&](const char* stage, auto role_tag) __attribute__((always_inline)) {
    constexpr int NO = decltype(role_tag)::value ? DB : DVB;
#pragma unroll
    for (int j = 0; j < 2 * TB; ++j)
#pragma unroll
      for (int o = 0; o < NO; ++o) acc[o] = mfma32(transposed_frag(stage, j, o, role_tag), frag[j], acc[o]);
  };
  // both (gradient product of `stage_prev`, then score product of `stage_cur`), with the fragment
  // reads kAhead products ahead
  auto matrix_block = [&](const char* stage_prev, const char* stage_cur, auto role_tag) __attribute__((always_inline)) {
    constexpr bool RB = decltype(role_tag)::value;
    constexpr int NO = RB ? DB : DVB, NT = 2 * TB * NO, NS0 = RB ? VS : KS, NS = TB * NS0;
    static_assert(kAhead <= NT, "look-ahead assumes it starts inside the gradient product");
    __builtin_amdgcn_s_setprio(2);  // the wave that owns the matrix pipe issues first
    bf16x8 at[2 * TB][NO], as[NS0][TB];
#pragma unroll
    for (int j = 0; j < 2 * TB; ++j)
#pragma unroll
      for (int o = 0; o < NO; ++o) at[j][o] = transposed_frag(stage_prev, j, o, role_tag);
    start_x(stage_cur, role_tag);
#pragma unroll
    for (int ks = 0; ks < NS0; ++ks)
#pragma unroll
      for (int rb = 0; rb < TB; ++rb) as[ks][rb] = straight_frag(stage_cur, ks, rb, role_tag);
#pragma unroll
    for (int j = 0; j < 2 * TB; ++j)
#pragma unroll
      for (int o = 0; o < NO; ++o) acc[o] = mfma32(at[j][o], frag[j], acc[o]);
#pragma unroll
    for (int ks = 0; ks < NS0; ++ks)
#pragma unroll
      for (int rb = 0; rb < TB; ++rb) x[rb] = mfma32(as[ks][rb], stat[ks], x[rb]);
    // a transposed fragment takes two LDS reads, a straight one a single read
    __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);
#pragma unroll
    for (int m = 0; m < NT - kAhead; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    // wave B: the reads of delta, the start of x, follow the last fragment of the gradient product
    if constexpr (RB) __builtin_amdgcn_sched_group_barrier(0x100, 4 * TB, 0);
#pragma unroll
    for (int m = 0; m < NS; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 0);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_setprio(0);
  };

  // A: x = S of query tile mt -> P, left in the exchange buffer (fp32) and in frag (bf16).
  // Rows of the tile are queries q0 + 32*rb + acc_row(v, g); this lane's column is `key`.
  auto make_p = [&](const char* stage, int mt) __attribute__((always_inline)) {
    const float* lse_s = reinterpret_cast<const float*>(stage + kOffStat);
    const int q0 = mt * kBM;
    const bool masked = (CAUSAL && q0 < kv_pair0 + 31) || (q0 + kBM > p.Sq);  // wave-uniform: diagonal or ragged tile
#pragma unroll
    for (int rb = 0; rb < TB; ++rb) {
      f32x4 l4[4];
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) l4[b4] = *reinterpret_cast<const f32x4*>(lse_s + 32 * rb + 8 * b4 + 4 * g);
#pragma unroll
      for (int v = 0; v < 16; ++v) x[rb][v] = __builtin_amdgcn_exp2f(x[rb][v] * p.kappa - l4[v >> 2][v & 3]);
      if (masked) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int qrow = q0 + 32 * rb + acc_row(v, g);
          if ((CAUSAL && key > qrow) || qrow >= p.Sq) x[rb][v] = 0.f;
        }
      }
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) {
        const f32x4 pr = {x[rb][4 * b4], x[rb][4 * b4 + 1], x[rb][4 * b4 + 2], x[rb][4 * b4 + 3]};
        *reinterpret_cast<f32x4*>(exch + ((rb * 4 + b4) * 64 + lane) * 16) = pr;
      }
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
        frag[2 * rb + jj] = to_bf16x8(x[rb][8 * jj], x[rb][8 * jj + 1], x[rb][8 * jj + 2], x[rb][8 * jj + 3],
                                      x[rb][8 * jj + 4], x[rb][8 * jj + 5], x[rb][8 * jj + 6], x[rb][8 * jj + 7]);
    }
  };
  // B: x = delta - dP of the tile in `stage`, P from the exchange buffer -> -dS / scale in frag (bf16),
  // one 32-row block at a time (the temporaries of a block are dead before the next one is read).
  auto make_ds = [&](const char* stage) __attribute__((always_inline)) {
#pragma unroll
    for (int rb = 0; rb < TB; ++rb) {
      f32x4 pr[4];
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) pr[b4] = *reinterpret_cast<const f32x4*>(exch + ((rb * 4 + b4) * 64 + lane) * 16);
#pragma unroll
      for (int v = 0; v < 16; ++v) x[rb][v] = pr[v >> 2][v & 3] * x[rb][v];
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
        frag[2 * rb + jj] = to_bf16x8(x[rb][8 * jj], x[rb][8 * jj + 1], x[rb][8 * jj + 2], x[rb][8 * jj + 3],
                                      x[rb][8 * jj + 4], x[rb][8 * jj + 5], x[rb][8 * jj + 6], x[rb][8 * jj + 7]);
    }
  };

  __builtin_amdgcn_s_waitcnt(0x0F70);  // everything issued so far: tile 0, stationary fragments
  __syncthreads();

  // Interval i = 0 .. n_iter touches tiles i-1 and i; tile -1 and tile n_iter do not exist, so the
  // first and the last interval are peeled and the loop body in between is straight-line code.
  // Under the causal mask a tile that lies entirely above a pair's diagonal is processed like any
  // other: its P is all zeros. Ring stages rotate: prev <- cur <- next <- (the stage prev used to be).
  auto run = [&](auto role_tag) __attribute__((always_inline)) {
    constexpr bool ROLE_B = decltype(role_tag)::value;
    TileCursor cur = {hq0, m_first};
    int off_prev = 2 * kStage, off_cur = 0, off_next = kStage;
    auto end_interval = [&]() __attribute__((always_inline)) {
      __builtin_amdgcn_s_waitcnt(0x0F70);  // the tile requested in this interval has landed
      __syncthreads();
      cur.advance(m_first, m_end);
      const int t = off_prev;
      off_prev = off_cur;
      off_cur = off_next;
      off_next = t;
    };
    // interval 0
    if (!ROLE_B) {
      straight_product(smem + off_cur, role_tag);
      __syncthreads();
      make_p(smem + off_cur, cur.mt);
    } else {
      if (n_iter > 1) request(smem + off_next);
      __syncthreads();
      straight_product(smem + off_cur, role_tag);
    }
    end_interval();
    for (int i = 1; i < n_iter; ++i) {
      const char* stage_cur = smem + off_cur;
      const char* stage_prev = smem + off_prev;
      const bool will_request = i + 1 < n_iter;
      if (!ROLE_B) {
        matrix_block(stage_prev, stage_cur, role_tag);
        __syncthreads();  // B has read P(i-1); the matrix pipe passes to B
        make_p(stage_cur, cur.mt);
      } else {
        if (will_request) request(smem + off_next);
        make_ds(stage_prev);
        __syncthreads();
        matrix_block(stage_prev, stage_cur, role_tag);
      }
      end_interval();
    }
    // interval n_iter
    if (!ROLE_B) {
      transposed_product(smem + off_prev, role_tag);
      __syncthreads();
    } else {
      make_ds(smem + off_prev);
      __syncthreads();
      transposed_product(smem + off_prev, role_tag);
    }
  };
  // Both roles pass the same barriers; separate code keeps each loop body straight-line.
  if (n_iter > 0) {
    if (!role_b) run(std::false_type{});
    else run(std::true_type{});
  }

  // ---- epilogue: wave A stores dV, wave B stores dK (times scale), for key row `key`, features
  // 32*o + 8*b4 + 4*g ..+3
  if (key < p.Skv) {
    const float f = role_b ? -p.scale : 1.f;  // wave B accumulated -dK / scale
    const int d = role_b ? k_head : kDV;
    const int nblk = role_b ? k_head / 32 : DVB;
    const int64_t row_stride = role_b ? k_row_stride : v_row_stride;
    if (two_part && role_b) {  // this head's gradient of the shared rotary part: [Hkv][B][Skv][64] fp32
      float* ws = p.ws_dkpe + (((int64_t)hk * p.B + b) * p.Skv + key) * 64;
#pragma unroll
      for (int o = 4; o < DB; ++o)
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4)
          store4<float>(ws + 32 * (o - 4) + 8 * b4 + 4 * g, acc[o][4 * b4] * f, acc[o][4 * b4 + 1] * f, acc[o][4 * b4 + 2] * f,
                        acc[o][4 * b4 + 3] * f, false);
    }
    if (p.split > 1) {
      // the partials are packed: exactly the Hkv heads of this call per row
      float* ws = (role_b ? p.ws_dk : p.ws_dv) + (((int64_t)part * p.B + b) * p.Skv + key) * ((int64_t)p.Hkv * d) + (int64_t)hk * d;
#pragma unroll
      for (int o = 0; o < DB; ++o)
        if (o < nblk)
#pragma unroll
          for (int b4 = 0; b4 < 4; ++b4)
            store4<float>(ws + 32 * o + 8 * b4 + 4 * g, acc[o][4 * b4] * f, acc[o][4 * b4 + 1] * f, acc[o][4 * b4 + 2] * f,
                          acc[o][4 * b4 + 3] * f, false);
    } else {
      OutT* out = reinterpret_cast<OutT*>(role_b ? p.dk : p.dv) + b * (role_b ? p.dk_bs : p.dv_bs) + key * row_stride +
                  (int64_t)hk * d;
#pragma unroll
      for (int o = 0; o < DB; ++o)
        if (o < nblk)
#pragma unroll
          for (int b4 = 0; b4 < 4; ++b4)
            store4<OutT>(out + 32 * o + 8 * b4 + 4 * g, acc[o][4 * b4] * f, acc[o][4 * b4 + 1] * f, acc[o][4 * b4 + 2] * f,
                         acc[o][4 * b4 + 3] * f, p.accumulate != 0);
    }
  }
}

}  // namespace

void launch_dkdv_d192(const BwdParams& p, bool causal, bool f32_out, unsigned grid, hipStream_t st) {
  constexpr int TB = 2;  // 64-row query tiles (32-row tiles, TB = 1, measured 3 % slower)
  const dim3 g(grid), block(kThreads);
  if (causal) {
    if (f32_out) hipLaunchKernelGGL((attn_bwd_dkdv_d192_kernel<TB, true, float>), g, block, 0, st, p);
    else hipLaunchKernelGGL((attn_bwd_dkdv_d192_kernel<TB, true, __bf16>), g, block, 0, st, p);
  } else {
    if (f32_out) hipLaunchKernelGGL((attn_bwd_dkdv_d192_kernel<TB, false, float>), g, block, 0, st, p);
    else hipLaunchKernelGGL((attn_bwd_dkdv_d192_kernel<TB, false, __bf16>), g, block, 0, st, p);
  }
}

}  // namespace pith
