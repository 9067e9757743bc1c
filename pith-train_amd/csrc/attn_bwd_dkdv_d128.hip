// Key/value-gradient kernel for head dims (128, 128) on gfx950. Same function and numerics as the
// general kernel in attn_bwd_dkdv.hip (pithtrain/operators/mla/triton.py:130-197, :331-384:
// P = exp2(kappa*s - lse2) in fp32, masked entries 0, P rounded to bf16 for dV += P^T dO,
// dS = P*(dP - delta)*scale rounded to bf16 for dK += dS^T Q, fp32 accumulation), same work split:
// a workgroup of 8 wavefronts owns 128 key rows of one (batch, kv head) and streams query tiles
// of its query heads; the wavefronts form 4 pairs, one per 32 keys, wave A of a pair holds K and
// dV, wave B holds V and dK, and A hands the fp32 P tile to B through an LDS buffer.
//
// What differs from the general kernel (all of it measured to matter on the device):
//   - query tiles are 64 rows, so a wave issues 32 MFMAs between synchronisations;
//   - Q / dO tiles and the lse / delta rows go global -> LDS directly (global_load_lds) into a
//     ring of three stages, requested one interval ahead by the B waves; tiles are packed and swizzled;
//   - B runs ONE TILE BEHIND A. In interval i wave A computes dV(i-1), S(i), P(i); wave B
//     computes dS(i-1), dK(i-1), dP(i);
//   - A runs [matrix block | vector block], B runs [vector block | matrix block], with a
//     workgroup barrier at "|" and at the end of the interval. The two waves of a pair share a
//     SIMD, so the matrix pipe is always owned by exactly one of them while the other does its
//     exp / dS arithmetic, tile requests and bookkeeping. The middle barrier also orders B's read
//     of P(i-1) before A's write of P(i): one P buffer per pair is enough;
//   - inside a matrix block the LDS fragment reads run kAhead products ahead of their use.
#include <type_traits>

#include "attn_bwd_common.h"

namespace pith {
namespace {

constexpr int kThreads = 512;
constexpr int kBM = 64;             // query rows per tile
constexpr int kBN = kDkdvBlockN;    // key rows per workgroup
constexpr int kD = 128;
constexpr int kStages = 3;          // tiles i-1, i (in use) and i+1 (landing)
constexpr int kAhead = 4;           // fragment reads run this many products ahead
constexpr int kTile = kBM * kRowBytes128;        // 16 KB
constexpr int kStat = 2 * kBM * 4;               // lse[64], delta[64]
constexpr int kStage = 2 * kTile + kStat;        // Q tile, dO tile, stats
constexpr int kExchPair = kBM * 32 * 4;          // one 64 x 32 fp32 P tile
constexpr int kSmem = kStages * kStage + 4 * kExchPair;
// dS hand-over: vector-memory stores a B wave issues per interval (one 16-byte store per lane and 16-row step of
// the 64-row tile). The wait that ends an interval lets exactly this many operations stay in flight, which is
// right only while they are the LAST vector-memory operations the wave issued (tests/test_cabi.py checks that on
// the compiler's output: loads first, then these stores, no spill traffic in the loop).
constexpr int kDsStoresPerInterval = kBM / 16;
static_assert(kDsStoresPerInterval == 4, "make_ds stores frag[0..3]; the vmcnt immediate below has a 4-bit low field");

// Position of a query tile in the stream of (query head, tile) pairs a workgroup visits, and the order of that
// stream. Ascending: head by head, tiles upwards. Descending (DESC): tiles from the last one down with the heads
// innermost. Under the mask a workgroup starts at its diagonal, so in ascending order the workgroups of an XCD stand
// on different tiles of the Q / dO stream they share and each fetches it from beyond L2 again; descending, all of
// them start on the last tile together. Measured: the causal launch over 16384 rows x 64 heads (34 GB fetched per launch, Q and dO
// are 537 MB) 5-7 % faster; over 8192 rows x 32 heads (134 MB, which the 256 MB last-level cache holds) 0-2 %
// slower; non-causal launches, whose workgroups walk in step either way, 1-3 % slower. The host picks by size
// (BwdParams::walk_desc selects the DESC instances of the causal kernel).
template <bool DESC>
struct TileCursor {
  int hq, mt;
  __device__ __forceinline__ static TileCursor first(int hq0, int m_first, int m_end) {
    return TileCursor{hq0, DESC ? m_end - 1 : m_first};
  }
  __device__ __forceinline__ void advance(int m_first, int m_end, int hq0, int hq_end) {
    if (DESC) {
      if (++hq == hq_end) {
        hq = hq0;
        --mt;
      }
    } else if (++mt == m_end) {
      mt = m_first;
      ++hq;
    }
  }
};

// EMIT_DS: wave B also stores every dS tile it forms (bf16, as -dS before the factor `scale`) to p.ds for
// the dQ kernel of attn_bwd_dq_ds.hip, which then needs no score recomputation. Layout of p.ds:
// one 4 KB image per (batch, query head, 64-row query tile, 128-key block, wave pair), in that
// order (under the causal mask only the key blocks a query tile can see: ds_tile_start); an image is the four bf16x8 fragments of the pair's B wave as they sit in registers,
// 1 KB per 16-row step j, the 16 bytes of lane (g, c) at g*512 + ((c ^ 8g ^ 4(j&1)) << 4) (the
// XOR terms make the reader's transposing LDS reads conflict-free). Keys at or beyond Skv hold 0
// (their P is masked to 0).
template <bool CAUSAL, typename OutT, bool EMIT_DS, bool DESC = false>
__global__ __launch_bounds__(kThreads) void attn_bwd_dkdv_d128_kernel(BwdParams p) {
  constexpr int KS = kD / 16, DB = kD / 32;
  __shared__ __attribute__((aligned(1024))) char smem[kSmem];

  const int tid = threadIdx.x;
  if ((int)blockIdx.x >= p.main_blocks) {  // workgroups appended to the grid: clear the rows behind the chunk's visible part
    zero_tail_block<OutT>(p, (int)blockIdx.x - p.main_blocks, kD, kD, tid, kThreads);
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

  const int q_row_bytes = p.HqT * kD * 2;  // Q and dO rows
  const int64_t kv_row_stride = (int64_t)p.HkvT * kD;

  // Query tiles to visit: all of them, or from the diagonal down under the causal mask.
  const int m_end = (p.Sq + kBM - 1) / kBM;
  const int m_first = CAUSAL ? min(kv_wg0 / kBM, m_end) : 0;
  const int n_iter = (m_end - m_first) * heads_per_part;

  // ---- requests: issued by the four B waves only (their vector block, dS, is the shorter one: measured
  // 2 % faster than sharing the requests among all eight waves)
  DirectTile128<kBM, kThreads / 2> mover;
  mover.init(q_row_bytes, pair, lane);
  const char* q_base = reinterpret_cast<const char*>(p.q + b * p.q_bs);
  const char* do_base = reinterpret_cast<const char*>(p.dout + b * p.dout_bs);
  using Cursor = TileCursor<DESC>;
  const int hq_end = hq0 + heads_per_part;
  Cursor req = Cursor::first(hq0, m_first, m_end);
  auto request = [&](char* stage) __attribute__((always_inline)) {
    const int row0 = req.mt * kBM;
    const int64_t head_off = (int64_t)req.hq * kD * 2 + (int64_t)row0 * q_row_bytes;
    mover.issue(q_base + head_off, p.Sq - row0, stage, pair, lane);
    mover.issue(do_base + head_off, p.Sq - row0, stage + kTile, pair, lane);
    if (pair < 2) {  // pair 0 fetches the 64 lse values of the tile's rows, pair 1 the 64 delta values
      int row = row0 + lane;
      row = row < p.Sq ? row : p.Sq - 1;
      const float* src = (pair == 0 ? p.lse : p.delta) + b * p.lse_bs + (int64_t)req.hq * p.lse_hs + row;
      load_lds4(src, stage + 2 * kTile + pair * kBM * 4);
    }
    req.advance(m_first, m_end, hq0, hq_end);
  };
  if (n_iter > 0 && role_b) request(smem);

  // stationary fragments: K rows for wave A, V rows for wave B
  bf16x8 stat[KS];
  {
    const int row = key < p.Skv ? key : p.Skv - 1;
    const __bf16* src = (role_b ? p.v + b * p.v_bs : p.k + b * p.k_bs) + row * kv_row_stride + (int64_t)hk * kD + g * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) stat[ks] = *reinterpret_cast<const bf16x8*>(src + ks * 16);
    if (role_b) {
      // wave B works with -V: its score-type product then starts from delta and yields delta - dP,
      // i.e. -(dP - delta) without a subtraction per element; the sign is undone with the factor
      // -scale on the accumulated dK (and by the reader of the dS images)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) stat[ks] = __builtin_bit_cast(bf16x8, __builtin_bit_cast(u32x4, stat[ks]) ^ 0x80008000u);
    }
  }
  f32x16 acc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;

  // per-lane read offsets inside a tile
  int s_off[KS];     // straight fragment of tile row c, contraction step ks (+ 32 rows: + 8192 bytes)
  int t_off[DB][2];  // transposing reads of feature block o, lower / upper 8 rows (+ 16 rows: + 4096 bytes)
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) s_off[ks] = straight_offset128(c, 2 * ks + g);
#pragma unroll
  for (int o = 0; o < DB; ++o)
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) t_off[o][hh] = transposed_offset128(0, hh, 32 * o, lane);

  // Within a stage wave A reads Q straight and dO transposed, wave B dO straight and Q transposed.
  const int straight_tile = role_b ? kTile : 0;
  const int transposed_tile = role_b ? 0 : kTile;
  char* const exch = smem + kStages * kStage + pair * kExchPair;

  f32x16 x[2];      // [32-row block] A: S, then P of the current tile. B: delta - dP, kept into the next interval
  bf16x8 frag[4];   // [16-row step] A: P(i) as B operand of dV(i) in the next interval. B: -dS(i-1) for dK(i-1)

  // score-type product of the tile in `stage`: x = T1 * stat^T
  // x starts from 0 in wave A and from the delta values of the tile's rows in wave B
  auto start_x = [&](const char* stage, auto role_tag) __attribute__((always_inline)) {
    if constexpr (decltype(role_tag)::value) {
      const float* delta_s = reinterpret_cast<const float*>(stage + 2 * kTile) + kBM;
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4) {
          const f32x4 d = *reinterpret_cast<const f32x4*>(delta_s + 32 * rb + 8 * b4 + 4 * g);
#pragma unroll
          for (int e = 0; e < 4; ++e) x[rb][4 * b4 + e] = d[e];
        }
    } else {
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int v = 0; v < 16; ++v) x[rb][v] = 0.f;
    }
  };
  auto straight_product = [&](const char* stage, auto role_tag) __attribute__((always_inline)) {
    start_x(stage, role_tag);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(stage + straight_tile + s_off[ks] + rb * 32 * kRowBytes128);
        x[rb] = mfma32(a, stat[ks], x[rb]);
      }
  };
  // gradient-type product with the tile in `stage`: acc^T += T2^T * frag
  auto transposed_product = [&](const char* stage) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int o = 0; o < DB; ++o) {
        const char* base = stage + transposed_tile + j * 16 * kRowBytes128;
        const bf16x8 a = lds_read_transposed_at(base + t_off[o][0], base + t_off[o][1]);
        acc[o] = mfma32(a, frag[j], acc[o]);
      }
  };
  // both (gradient product of `stage_prev`, then score product of `stage_cur`), with the
  // fragment reads kAhead products ahead
  auto matrix_block = [&](const char* stage_prev, const char* stage_cur, auto role_tag) __attribute__((always_inline)) {
    constexpr int NT = 4 * DB, NS = 2 * KS;
    static_assert(kAhead <= NT, "look-ahead assumes it starts inside the gradient product");
    __builtin_amdgcn_s_setprio(2);  // the wave that owns the matrix pipe issues first
    bf16x8 at[4][DB], as[KS][2];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int o = 0; o < DB; ++o) {
        const char* base = stage_prev + transposed_tile + j * 16 * kRowBytes128;
        at[j][o] = lds_read_transposed_at(base + t_off[o][0], base + t_off[o][1]);
      }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
        as[ks][rb] = *reinterpret_cast<const bf16x8*>(stage_cur + straight_tile + s_off[ks] + rb * 32 * kRowBytes128);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int o = 0; o < DB; ++o) acc[o] = mfma32(at[j][o], frag[j], acc[o]);
    start_x(stage_cur, role_tag);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) x[rb] = mfma32(as[ks][rb], stat[ks], x[rb]);
    // wave B: the eight reads of delta, the start of x, come first (measured: 2 % faster than placing them
    // behind the gradient product, where x would be live for a shorter time)
    if constexpr (decltype(role_tag)::value) __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
    // a transposed fragment takes two LDS reads, a straight one a single read
    __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);
#pragma unroll
    for (int m = 0; m < NT - kAhead; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
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
    const float* lse_s = reinterpret_cast<const float*>(stage + 2 * kTile);
    const int q0 = mt * kBM;
    f32x4 l4[2][4];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) l4[rb][b4] = *reinterpret_cast<const f32x4*>(lse_s + 32 * rb + 8 * b4 + 4 * g);
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int v = 0; v < 16; ++v) x[rb][v] = __builtin_amdgcn_exp2f(x[rb][v] * p.kappa - l4[rb][v >> 2][v & 3]);
    if ((CAUSAL && q0 < kv_pair0 + 31) || (q0 + kBM > p.Sq) || (EMIT_DS && kv_pair0 + 32 > p.Skv)) {
      // tile on the diagonal of a causal chunk, a ragged last tile, or (when dS is handed on, where
      // nonexistent keys must read 0) the ragged last key block (wave-uniform branch)
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int qrow = q0 + 32 * rb + acc_row(v, g);
          if ((CAUSAL && key > qrow) || qrow >= p.Sq || (EMIT_DS && key >= p.Skv)) x[rb][v] = 0.f;
        }
    }
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
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
  // B: x = delta - dP of the tile in `stage`, P from the exchange buffer -> -dS / scale in frag (bf16).
  // The factor `-scale` is applied once to the accumulated dK in the epilogue.
  // `tile` is the (query head, tile) the stage holds (only used to place the dS image).
  // With EMIT_DS the fragments are also stored as the image of query tile `tile` (layout at the top).
  // The stores cost the kernel about 12 % wherever they are issued in the interval (measured: in this
  // vector block, spread over B's matrix block, or at its end): each compute unit then has 16 KB of
  // writes per interval in flight next to 33 KB of tile reads, its vector cache stalls on pending
  // requests three times as often, and the sustained clock drops by 6 % under the write traffic.
  char* const ds_wg = EMIT_DS ? p.ds + ((int64_t)n_tile * 4 + pair) * 4096 : nullptr;
  auto make_ds = [&](const char* stage, const Cursor& tile) __attribute__((always_inline)) {
    f32x4 pr[2][4];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) pr[rb][b4] = *reinterpret_cast<const f32x4*>(exch + ((rb * 4 + b4) * 64 + lane) * 16);
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
      for (int v = 0; v < 16; ++v) x[rb][v] = pr[rb][v >> 2][v & 3] * x[rb][v];  // x = delta - dP
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
        frag[2 * rb + jj] = to_bf16x8(x[rb][8 * jj], x[rb][8 * jj + 1], x[rb][8 * jj + 2], x[rb][8 * jj + 3],
                                      x[rb][8 * jj + 4], x[rb][8 * jj + 5], x[rb][8 * jj + 6], x[rb][8 * jj + 7]);
    }
    if constexpr (EMIT_DS) {
      char* img = ds_wg + (int64_t)(b * p.Hq + tile.hq) * p.ds_hs + ds_tile_start<CAUSAL>(tile.mt, p.ds_kb) * kDsBlockBytes;
      int off = (g << 9) + ((c ^ (g << 3)) << 4);  // recomputed per tile: no register is held across the interval
      asm volatile("" : "+v"(off));
#pragma unroll
      for (int j = 0; j < kDsStoresPerInterval; ++j)
        __builtin_nontemporal_store(frag[j], reinterpret_cast<bf16x8*>(img + j * 1024 + (off ^ ((j & 1) << 6))));
    }
  };

  __builtin_amdgcn_s_waitcnt(0x0F70);  // everything issued so far: tile 0, stationary fragments
  __syncthreads();

  // Interval i = 0 .. n_iter touches tiles i-1 and i; tile -1 and tile n_iter do not exist, so the
  // first and the last interval are peeled and the loop body in between is straight-line code.
  // Under the causal mask a tile that lies entirely above a pair's diagonal is processed like any
  // other: its P is all zeros (at most one tile per query head and pair).
  // Ring stages rotate: prev <- cur <- next <- (the stage prev used to be).
  auto run = [&](auto role_tag) __attribute__((always_inline)) {
    constexpr bool ROLE_B = decltype(role_tag)::value;
    Cursor cur = Cursor::first(hq0, m_first, m_end), done = cur;  // tiles i and i-1 of interval i
    int off_prev = 2 * kStage, off_cur = 0, off_next = kStage;
    auto end_interval = [&](bool stored) __attribute__((always_inline)) {
      // the tile requested in this interval has landed. Vector memory operations complete in issue
      // order, and where wave B issued its four dS stores after the request (every interval but the
      // first) they may stay in flight.
      if (ROLE_B && EMIT_DS && stored) __builtin_amdgcn_s_waitcnt(0x0F70 | kDsStoresPerInterval);
      else __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
      done = cur;
      cur.advance(m_first, m_end, hq0, hq_end);
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
    end_interval(false);
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
        make_ds(stage_prev, done);
        __syncthreads();
        matrix_block(stage_prev, stage_cur, role_tag);
      }
      end_interval(true);
    }
    // interval n_iter
    if (!ROLE_B) {
      transposed_product(smem + off_prev);
      __syncthreads();
    } else {
      make_ds(smem + off_prev, done);
      __syncthreads();
      transposed_product(smem + off_prev);
    }
  };
  // Both roles pass the same barriers; separate code keeps each loop body straight-line.
  if (n_iter > 0) {
    if (!role_b) run(std::false_type{});
    else run(std::true_type{});
  }

  if (role_b) {
#pragma unroll
    for (int o = 0; o < DB; ++o)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[o][v] *= -p.scale;  // wave B accumulated -dK / scale
  }
  // ---- epilogue: wave A stores dV, wave B stores dK, for key row `key`, features 32*o + 8*b4 + 4*g ..+3
  if (key < p.Skv) {
    if (p.split > 1) {
      // the partials are packed: exactly the Hkv heads of this call per row
      float* ws = (role_b ? p.ws_dk : p.ws_dv) + (((int64_t)part * p.B + b) * p.Skv + key) * ((int64_t)p.Hkv * kD) + (int64_t)hk * kD;
#pragma unroll
      for (int o = 0; o < DB; ++o)
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4)
          store4<float>(ws + 32 * o + 8 * b4 + 4 * g, acc[o][4 * b4], acc[o][4 * b4 + 1], acc[o][4 * b4 + 2],
                        acc[o][4 * b4 + 3], false);
    } else {
      OutT* out = reinterpret_cast<OutT*>(role_b ? p.dk : p.dv) + b * (role_b ? p.dk_bs : p.dv_bs) + key * kv_row_stride +
                  (int64_t)hk * kD;
#pragma unroll
      for (int o = 0; o < DB; ++o)
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4)
          store4<OutT>(out + 32 * o + 8 * b4 + 4 * g, acc[o][4 * b4], acc[o][4 * b4 + 1], acc[o][4 * b4 + 2],
                       acc[o][4 * b4 + 3], p.accumulate != 0);
    }
  }
}

}  // namespace

template <bool EMIT_DS>
static void launch_variant(const BwdParams& p, bool causal, bool f32_out, unsigned grid, hipStream_t st) {
  const dim3 g(grid), block(kThreads);
  if (causal) {
    if (p.walk_desc) {
      if (f32_out) hipLaunchKernelGGL((attn_bwd_dkdv_d128_kernel<true, float, EMIT_DS, true>), g, block, 0, st, p);
      else hipLaunchKernelGGL((attn_bwd_dkdv_d128_kernel<true, __bf16, EMIT_DS, true>), g, block, 0, st, p);
    } else if (f32_out) hipLaunchKernelGGL((attn_bwd_dkdv_d128_kernel<true, float, EMIT_DS>), g, block, 0, st, p);
    else hipLaunchKernelGGL((attn_bwd_dkdv_d128_kernel<true, __bf16, EMIT_DS>), g, block, 0, st, p);
  } else {
    if (f32_out) hipLaunchKernelGGL((attn_bwd_dkdv_d128_kernel<false, float, EMIT_DS>), g, block, 0, st, p);
    else hipLaunchKernelGGL((attn_bwd_dkdv_d128_kernel<false, __bf16, EMIT_DS>), g, block, 0, st, p);
  }
}

void launch_dkdv_d128(const BwdParams& p, bool causal, bool f32_out, unsigned grid, hipStream_t st) {
  if (p.ds) launch_variant<true>(p, causal, f32_out, grid, st);
  else launch_variant<false>(p, causal, f32_out, grid, st);
}

}  // namespace pith
