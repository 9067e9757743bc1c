// Key/value-gradient kernel of one chunk attention backward for gfx950 with register-staged tiles
// (used for head dims 64/64; 128/128 and 192/128 have direct-load kernels of their own), the entry
// points of the dK/dV step and the reduction kernel of the head split; against an external
// (ring-combined) base-2 LSE and delta = rowsum(O*dO). Follows
// pithtrain/operators/mla/triton.py:130-197 (non-causal :331-384): P = exp2(kappa*s - lse2) in
// fp32, masked entries 0, P rounded to bf16 for dV += P^T dO, dS = P*(dP - delta)*scale rounded
// to bf16 for dK += dS^T Q, fp32 accumulation.
//
// Work split. A workgroup of 8 wavefronts owns 128 key rows of one (batch, kv head) and loops
// over query tiles of 32 rows of the query heads assigned to it. The 8 wavefronts form 4 PAIRS,
// one per 32 key rows; the two waves of a pair share a SIMD and split the work so that each
// stays below 256 registers (two waves per SIMD, no accumulator spills):
//     wave A:  S = Q K^T  ->  P = exp2(kappa*S - lse)  ->  dV^T += dO^T P      (holds K, dV)
//     wave B:  dP = dO V^T ->  dS = P o (dP - delta) * scale -> dK^T += Q^T dS (holds V, dK)
// B needs A's P: A leaves the fp32 P tile (32 x 32) in an LDS exchange buffer, in the lane order
// both waves share, and B picks it up after the iteration's only barrier. Both waves issue the
// same number of MFMAs.
// The stationary side (K or V rows) sits in registers as B operands, so score tiles have the key
// index as their column; P / dS then feed the products that contract over queries straight from
// registers (slot order, see attn_tiles.h) with dO^T / Q^T read transposed from LDS.
//
// Query tiles stream through a 3-deep LDS ring: the tile for iteration i+1 is committed while
// iteration i computes and becomes visible at iteration i's barrier, its buffer having been
// released by the previous barrier. Global loads run two tiles ahead.
//
// With grouped-query attention the heads of a group may be cut into `split` parts handled by
// different workgroups (more parallelism when there are few key tiles); the parts leave fp32
// partial results in a caller-provided workspace and a second kernel adds them in a fixed
// order, so the result does not depend on scheduling.
#include <mutex>

#include "attn_bwd_common.h"

namespace pith {
namespace {

constexpr int kThreads = 512;
constexpr int kBM = 32;    // query rows per tile
constexpr int kBN = kDkdvBlockN;  // key rows per workgroup
constexpr int kStages = 3;

template <int DQK, int DV>
struct DkdvLayout {
  static constexpr int QP = DQK * 2 + 80;  // tiles are read straight by one wave of a pair, transposed by the other
  static constexpr int OP = DV * 2 + 80;
  static constexpr int kQTile = kBM * QP;
  static constexpr int kOTile = kBM * OP;
  static constexpr int kStat = 2 * kBM * 4;  // lse[32], delta[32]
  static constexpr int kStage = kQTile + kOTile + kStat;
  static constexpr int kExch = 4 * 2 * 4096;  // [pair][parity][32 x 32 fp32]
  static constexpr int kTotal = kStages * kStage + kExch;
};

// One wave's loop. ROLE_B = false: wave A (T1 = Q tile, stationary K, out dV). ROLE_B = true:
// wave B (T1 = dO tile, stationary V, out dK). KDIM = contraction length of the score-type
// product, ODIM = feature length of the gradient this wave accumulates.
template <int DQK, int DV, bool CAUSAL, bool ROLE_B, typename Fetch, typename Commit>
__device__ __forceinline__ void dkdv_wave_loop(const BwdParams& p, char* smem, int lane, int pair, int kv_pair0, int n_iter,
                                               int m_end, int m_start_wg, const bf16x8* stat,
                                               f32x16* acc, Fetch& fetch, Commit& commit) {
  using L = DkdvLayout<DQK, DV>;
  constexpr int KDIM = ROLE_B ? DV : DQK;
  constexpr int ODIM = ROLE_B ? DQK : DV;
  constexpr int T1P = ROLE_B ? L::OP : L::QP;   // pitch of the tile read straight
  constexpr int T2P = ROLE_B ? L::QP : L::OP;   // pitch of the tile read transposed
  constexpr int T1_OFF = ROLE_B ? L::kQTile : 0;
  constexpr int T2_OFF = ROLE_B ? 0 : L::kQTile;
  const int c = lane & 31, g = lane >> 5;
  const int key = kv_pair0 + c;
  const int m_start_pair = CAUSAL ? kv_pair0 / kBM : 0;
  char* exch = smem + kStages * L::kStage + pair * 8192;

  // Ring stages rotate (prev <- cur <- next <- prev) and the tile position advances by increments:
  // no division or modulo in the loop. The body has no branch around its matrix instructions (a
  // tile entirely above this pair's diagonal is processed like any other, its P is all zeros), so
  // the accumulators stay in place from one iteration to the next.
  int off_prev = 2 * L::kStage, off_cur = 0, off_next = L::kStage;
  int mt = m_start_wg;
  for (int i = 0; i < n_iter; ++i) {
    if (i + 1 < n_iter) commit(off_next);
    if (i + 2 < n_iter) fetch();
    const char* stage = smem + off_cur;
    const float* stats = reinterpret_cast<const float*>(stage + L::kQTile + L::kOTile);
    const int q0 = mt * kBM;

    f32x16 x;
    bf16x8 frag[2];
#pragma unroll
    for (int v = 0; v < 16; ++v) x[v] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KDIM / 16; ++ks) {
      const bf16x8 a = lds_read_straight(stage + T1_OFF, T1P, c, ks * 16 + g * 8);
      x = mfma32(a, stat[ks], x);
    }
    if (!ROLE_B) {
      // rows of the tile are queries q0 + acc_row(v, g); this lane's column is `key`
      f32x4 l4[4];
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) l4[b4] = *reinterpret_cast<const f32x4*>(stats + 8 * b4 + 4 * g);
#pragma unroll
      for (int v = 0; v < 16; ++v) x[v] = __builtin_amdgcn_exp2f(x[v] * p.kappa - l4[v >> 2][v & 3]);
      if ((CAUSAL && mt <= m_start_pair) || (q0 + kBM > p.Sq)) {  // wave-uniform
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int qrow = q0 + acc_row(v, g);
          if ((CAUSAL && key > qrow) || qrow >= p.Sq) x[v] = 0.f;
        }
      }
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) {
        const f32x4 pr = {x[4 * b4], x[4 * b4 + 1], x[4 * b4 + 2], x[4 * b4 + 3]};
        *reinterpret_cast<f32x4*>(exch + (i & 1) * 4096 + (b4 * 64 + lane) * 16) = pr;
      }
    }
    __syncthreads();
    if (ROLE_B) {
      const float* delta_s = stats + kBM;
      f32x4 pr[4], d4[4];
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) {
        pr[b4] = *reinterpret_cast<const f32x4*>(exch + (i & 1) * 4096 + (b4 * 64 + lane) * 16);
        d4[b4] = *reinterpret_cast<const f32x4*>(delta_s + 8 * b4 + 4 * g);
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) x[v] = pr[v >> 2][v & 3] * (x[v] - d4[v >> 2][v & 3]) * p.scale;
    }
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
      frag[jj] = to_bf16x8(x[8 * jj], x[8 * jj + 1], x[8 * jj + 2], x[8 * jj + 3], x[8 * jj + 4], x[8 * jj + 5],
                           x[8 * jj + 6], x[8 * jj + 7]);
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int o = 0; o < ODIM / 32; ++o) {
        const bf16x8 a = lds_read_transposed(stage + T2_OFF, T2P, 16 * j, 32 * o, lane);
        acc[o] = mfma32(a, frag[j], acc[o]);
      }
    const int t = off_prev;
    off_prev = off_cur;
    off_cur = off_next;
    off_next = t;
    if (++mt == m_end) mt = m_start_wg;
  }
}

template <int DQK, int DV, bool CAUSAL, typename OutT>
__global__ __launch_bounds__(kThreads) void attn_bwd_dkdv_kernel(BwdParams p) {
  using L = DkdvLayout<DQK, DV>;
  constexpr int KS = DQK / 16, VS = DV / 16, DB = DQK / 32, DVB = DV / 32;
  constexpr int NSTAT = KS > VS ? KS : VS, NACC = DB > DVB ? DB : DVB;
  __shared__ __attribute__((aligned(16))) char smem[L::kTotal];

  const int tid = threadIdx.x;
  if ((int)blockIdx.x >= p.main_blocks) {  // workgroups appended to the grid: clear the rows behind the chunk's visible part
    zero_tail_block<OutT>(p, (int)blockIdx.x - p.main_blocks, DQK, DV, tid, kThreads);
    return;
  }
  const int lane = tid & 63, wave = tid >> 6;
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

  const int64_t q_row_stride = (int64_t)p.HqT * DQK;
  const int64_t do_row_stride = (int64_t)p.HqT * DV;
  const int k_head = DQK;
  const int64_t k_row_stride = (int64_t)p.HkvT * k_head;
  const int64_t v_row_stride = (int64_t)p.HkvT * DV;

  // stationary fragments: K rows for wave A, V rows for wave B
  bf16x8 stat[NSTAT];
  {
    const int row = key < p.Skv ? key : p.Skv - 1;
    if (!role_b) {
      const __bf16* src = p.k + b * p.k_bs + row * k_row_stride + (int64_t)hk * k_head + g * 8;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) stat[ks] = *reinterpret_cast<const bf16x8*>(src + ks * 16);
    } else {
      const __bf16* src = p.v + b * p.v_bs + row * v_row_stride + (int64_t)hk * DV + g * 8;
#pragma unroll
      for (int ks = 0; ks < VS; ++ks) stat[ks] = *reinterpret_cast<const bf16x8*>(src + ks * 16);
    }
  }
  f32x16 acc[NACC];
#pragma unroll
  for (int i = 0; i < NACC; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;

  // Query tiles to visit: all of them, or from the diagonal down under the causal mask.
  const int m_tiles_all = (p.Sq + kBM - 1) / kBM;
  const int m_start_wg = CAUSAL ? min(kv_wg0 / kBM, m_tiles_all) : 0;
  const int n_m = m_tiles_all - m_start_wg;
  const int n_iter = n_m * heads_per_part;

  TileCopy<kBM, DQK, L::QP, kThreads> qcopy;
  TileCopy<kBM, DV, L::OP, kThreads> ocopy;
  float stat_val = 0.f;  // threads 0..31 carry lse, 32..63 carry delta of the tile's rows
  int fetch_hq = hq0, fetch_mt = m_start_wg;  // position of the next tile to fetch
  auto fetch = [&]() {
    const int hq = fetch_hq, mt = fetch_mt;
    if (++fetch_mt == m_tiles_all) {
      fetch_mt = m_start_wg;
      ++fetch_hq;
    }
    qcopy.fetch(p.q + b * p.q_bs + (int64_t)hq * DQK, q_row_stride, mt * kBM, p.Sq, tid);
    ocopy.fetch(p.dout + b * p.dout_bs + (int64_t)hq * DV, do_row_stride, mt * kBM, p.Sq, tid);
    if (tid < 2 * kBM) {
      int row = mt * kBM + (tid & (kBM - 1));
      row = row < p.Sq ? row : p.Sq - 1;
      const float* src = (tid < kBM ? p.lse : p.delta) + b * p.lse_bs + (int64_t)hq * p.lse_hs;
      stat_val = src[row];
    }
  };
  auto commit = [&](int stage_off) {
    char* base = smem + stage_off;
    qcopy.commit(base, tid);
    ocopy.commit(base + L::kQTile, tid);
    if (tid < 2 * kBM) reinterpret_cast<float*>(base + L::kQTile + L::kOTile)[tid] = stat_val;
  };

  if (n_iter > 0) {
    fetch();
    commit(0);
    if (n_iter > 1) fetch();
  }
  wait_all_vector_loads();
  __syncthreads();

  if (!role_b)
    dkdv_wave_loop<DQK, DV, CAUSAL, false>(p, smem, lane, pair, kv_pair0, n_iter, m_tiles_all, m_start_wg, stat, acc, fetch, commit);
  else
    dkdv_wave_loop<DQK, DV, CAUSAL, true>(p, smem, lane, pair, kv_pair0, n_iter, m_tiles_all, m_start_wg, stat, acc, fetch, commit);

  // ---- epilogue: wave A stores dV, wave B stores dK, for key row `key`, features 32*o + 8*b4 + 4*g ..+3
  if (key < p.Skv) {
    const int d = role_b ? k_head : DV;
    const int nblk = role_b ? k_head / 32 : DVB;
    const int64_t row_stride = role_b ? k_row_stride : v_row_stride;
    if (p.split > 1) {
      float* ws = (role_b ? p.ws_dk : p.ws_dv) +
                  (((int64_t)part * p.B + b) * p.Skv + key) * ((int64_t)p.Hkv * d) + (int64_t)hk * d;  // partials are packed
#pragma unroll
      for (int o = 0; o < NACC; ++o)
        if (o < nblk)
#pragma unroll
          for (int b4 = 0; b4 < 4; ++b4)
            store4<float>(ws + 32 * o + 8 * b4 + 4 * g, acc[o][4 * b4], acc[o][4 * b4 + 1], acc[o][4 * b4 + 2],
                          acc[o][4 * b4 + 3], false);
    } else {
      OutT* out = reinterpret_cast<OutT*>(role_b ? p.dk : p.dv) + b * (role_b ? p.dk_bs : p.dv_bs) + key * row_stride +
                  (int64_t)hk * d;
#pragma unroll
      for (int o = 0; o < NACC; ++o)
        if (o < nblk)
#pragma unroll
          for (int b4 = 0; b4 < 4; ++b4)
            store4<OutT>(out + 32 * o + 8 * b4 + 4 * g, acc[o][4 * b4], acc[o][4 * b4 + 1], acc[o][4 * b4 + 2],
                         acc[o][4 * b4 + 3], p.accumulate != 0);
    }
  }
}

// out[b, s, h, :] (+)= sum over parts of ws[part][b][s][h][:], parts added in index order; dK
// (blockIdx.y = 0) and dV (blockIdx.y = 1) in one launch.
struct ReduceParams {
  const float* ws[2];
  void* out[2];
  int64_t part_stride[2], row_elems[2], out_bs[2], n4[2];
  int64_t out_row_elems[2];  // elements between consecutive rows of `out` (>= row_elems: a head range of a wider tensor)
  int64_t rows_per_batch;
  int parts, accumulate;
};

template <typename OutT>
__global__ __launch_bounds__(256) void reduce_parts_kernel(ReduceParams r) {
  const int t = blockIdx.y;
  const float* __restrict__ ws = r.ws[t];
  OutT* out = reinterpret_cast<OutT*>(r.out[t]);
  const int64_t part_stride = r.part_stride[t], n4 = r.n4[t];
  const int64_t per_batch = r.rows_per_batch * r.row_elems[t];
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t e = i * 4;
    f32x4 s = *reinterpret_cast<const f32x4*>(ws + e);
    for (int pidx = 1; pidx < r.parts; ++pidx) s += *reinterpret_cast<const f32x4*>(ws + pidx * part_stride + e);
    const int64_t bb = e / per_batch;
    const int64_t in_batch = e - bb * per_batch;
    const int64_t row = in_batch / r.row_elems[t];
    OutT* dst = out + bb * r.out_bs[t] + row * r.out_row_elems[t] + (in_batch - row * r.row_elems[t]);
    store4<OutT>(dst, s[0], s[1], s[2], s[3], r.accumulate != 0);
  }
}

int pick_split(const pith_attn_bwd_args* a) {
  const int64_t group = a->Hq / a->Hkv;
  const int64_t base = ((a->Skv + kBN - 1) / kBN) * a->Hkv * a->B;
  int split = 1;
  // one workgroup per compute unit is resident; without a causal mask all workgroups carry the same
  // work, so one full round is ideal; under the mask two rounds (heaviest first) balance better
  const int64_t want = (a->causal ? 2 : 1) * (int64_t)compute_units_or_default();
  while (split < group && base * split < want && group % (split * 2) == 0) split *= 2;
  return split;
}

// Workspace layout: [head-split partial dK | partial dV] (split > 1), then the per-head gradients of a
// shared k_pe [Hkv][B][Skv][64] (keys in two parts).
int64_t split_bytes_for(const pith_attn_bwd_args* a, int split) {
  if (split <= 1) return 0;
  return (int64_t)split * a->B * a->Skv * a->Hkv * (a->Dqk + a->Dv) * (int64_t)sizeof(float);
}
int64_t dkpe_bytes_for(const pith_attn_bwd_args* a) {
  return a->k_pe ? a->Hkv * a->B * a->Skv * 64 * (int64_t)sizeof(float) : 0;
}
int64_t workspace_bytes_for(const pith_attn_bwd_args* a, int split) { return split_bytes_for(a, split) + dkpe_bytes_for(a); }

constexpr int64_t kWalkDescBytes = 192ll << 20;

template <int DQK, int DV>
void launch_dkdv(BwdParams p, const pith_attn_bwd_args* a, hipStream_t st) {
  p.tiles = (int)((a->Skv + kBN - 1) / kBN);
  p.accumulate = a->accumulate_dkv;
  p.main_blocks = (int)(p.tiles * a->Hkv * a->B * p.split);
  p.zero_tail = a->accumulate_dkv ? 0 : (int)a->dkv_zero_tail;  // rows that are added to keep what they hold
  const dim3 grid((unsigned)(p.main_blocks + (p.zero_tail + kZeroTailRows - 1) / kZeroTailRows)), block(kThreads);
  const bool f32 = a->dkv_dtype == PITH_F32;
  if constexpr (DQK == 128 && DV == 128) {
    // descending walk under the mask when Q and dO together exceed what the last-level cache (256 MB) keeps
    p.walk_desc = a->causal != 0 && (int64_t)a->B * a->Sq * a->Hq * (DQK + DV) * 2 > kWalkDescBytes;
    launch_dkdv_d128(p, a->causal != 0, f32, grid.x, st);
  } else if constexpr (DQK == 192 && DV == 128) {
    launch_dkdv_d192(p, a->causal != 0, f32, grid.x, st);
  } else {
    if (a->causal) {
      if (f32) hipLaunchKernelGGL((attn_bwd_dkdv_kernel<DQK, DV, true, float>), grid, block, 0, st, p);
      else hipLaunchKernelGGL((attn_bwd_dkdv_kernel<DQK, DV, true, __bf16>), grid, block, 0, st, p);
    } else {
      if (f32) hipLaunchKernelGGL((attn_bwd_dkdv_kernel<DQK, DV, false, float>), grid, block, 0, st, p);
      else hipLaunchKernelGGL((attn_bwd_dkdv_kernel<DQK, DV, false, __bf16>), grid, block, 0, st, p);
    }
  }
  if (p.k_pe) {  // dk_pe (+)= sum over heads, in head order
    ReduceParams r;
    r.row_elems[0] = r.out_row_elems[0] = 64;
    r.part_stride[0] = a->B * a->Skv * 64;
    r.n4[0] = r.part_stride[0] / 4;
    r.ws[0] = p.ws_dkpe;
    r.out[0] = a->dk_pe;
    r.out_bs[0] = a->dk_pe_bs;
    r.row_elems[1] = r.out_row_elems[1] = r.part_stride[1] = r.n4[1] = r.out_bs[1] = 0;
    r.ws[1] = nullptr;
    r.out[1] = nullptr;
    r.rows_per_batch = a->Skv;
    r.parts = (int)a->Hkv;
    r.accumulate = a->accumulate_dkv;
    const int64_t blocks = (r.n4[0] + 255) / 256;
    const dim3 rgrid((unsigned)(blocks < 8192 ? blocks : 8192), 1);
    if (f32) hipLaunchKernelGGL((reduce_parts_kernel<float>), rgrid, dim3(256), 0, st, r);
    else hipLaunchKernelGGL((reduce_parts_kernel<__bf16>), rgrid, dim3(256), 0, st, r);
  }
  if (p.split > 1) {
    ReduceParams r;
    int64_t max_n4 = 0;
    for (int which = 0; which < 2; ++which) {
      const int64_t d = which == 0 ? a->Dqk : a->Dv;
      r.row_elems[which] = a->Hkv * d;
      r.out_row_elems[which] = p.HkvT * d;
      r.part_stride[which] = a->B * a->Skv * r.row_elems[which];
      r.n4[which] = r.part_stride[which] / 4;
      r.ws[which] = which == 0 ? p.ws_dk : p.ws_dv;
      r.out[which] = which == 0 ? a->dk : a->dv;
      r.out_bs[which] = which == 0 ? a->dk_bs : a->dv_bs;
      if (r.n4[which] > max_n4) max_n4 = r.n4[which];
    }
    r.rows_per_batch = a->Skv;
    r.parts = p.split;
    r.accumulate = a->accumulate_dkv;
    const dim3 rgrid((unsigned)((max_n4 + 255) / 256 < 8192 ? (max_n4 + 255) / 256 : 8192), 2);
    if (f32) hipLaunchKernelGGL((reduce_parts_kernel<float>), rgrid, dim3(256), 0, st, r);
    else hipLaunchKernelGGL((reduce_parts_kernel<__bf16>), rgrid, dim3(256), 0, st, r);
  }
}

}  // namespace
}  // namespace pith

using namespace pith;

extern "C" int64_t pith_attn_bwd_dkdv_workspace_bytes(const pith_attn_bwd_args* a) {
  if (!a || a->Hkv <= 0 || a->Hq <= 0 || a->Hq % a->Hkv != 0 || a->B <= 0 || a->Skv <= 0) return 0;
  return workspace_bytes_for(a, pick_split(a));
}

namespace {

// Runs the kernels with the head-split partials in `workspace` (NULL: no head split).
int run_dkdv(const pith_attn_bwd_args* a, int split, void* workspace, hipStream_t st, const char* who) {
  // the grid of this kernel runs over key tiles (validate_bwd bounded the query-side grid)
  if (((a->Skv + kBN - 1) / kBN) * a->Hkv * a->B * (int64_t)split > 0x7fffffffLL)
    return fail(PITH_ERR_UNSUPPORTED, "%s: Skv=%lld x Hkv=%lld x B=%lld exceeds the launch grid limit", who,
                (long long)a->Skv, (long long)a->Hkv, (long long)a->B);
  BwdParams p = make_bwd_params(a);
  if (a->k_pe) {
    if (a->Hq != a->Hkv)
      return fail(PITH_ERR_UNSUPPORTED, "%s: keys in two parts need Hq == Hkv (got %lld, %lld)", who, (long long)a->Hq, (long long)a->Hkv);
    if (!a->dk_pe) return fail(PITH_ERR_NULL_POINTER, "%s: dk_pe is NULL", who);
    if (!aligned16(a->dk_pe) || a->dk_pe_bs % 8) return fail(PITH_ERR_MISALIGNED, "%s: dk_pe pointer / batch stride must keep 16-byte alignment", who);
    if (!workspace) return fail(PITH_ERR_BAD_SHAPE, "%s: keys in two parts need a workspace of %lld bytes", who, (long long)dkpe_bytes_for(a));
    p.ws_dkpe = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + split_bytes_for(a, split));
  }
  begin_launch();
  if (split > 1 && workspace) {
    p.split = split;
    p.ws_dk = reinterpret_cast<float*>(workspace);
    p.ws_dv = p.ws_dk + (int64_t)split * a->B * a->Skv * a->Hkv * a->Dqk;
  }
  // dS hand-over to the dQ call: only when the buffer is usable (otherwise the call behaves as without it)
  if (a->ds && ds_bytes_for(a) > 0 && a->ds_bytes >= ds_bytes_for(a)) {
    if ((uintptr_t)a->ds % 256) return fail(PITH_ERR_MISALIGNED, "%s: ds must be 256-byte aligned", who);
    p.ds = reinterpret_cast<char*>(a->ds);
  }
  if (a->Dqk == 128) launch_dkdv<128, 128>(p, a, st);
  else if (a->Dqk == 192) launch_dkdv<192, 128>(p, a, st);
  else launch_dkdv<64, 64>(p, a, st);
  return check_launch(who);
}

// Scratch of pith_attn_bwd_dkdv_static: device memory that belongs to the library's code object
// (one copy per GPU, held until the process ends). Host code never uses this name as an address;
// it asks the runtime for the array's device address once per device and passes that on.
constexpr int64_t kStaticScratchBytes = PITH_DKDV_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device; resolved at the first call on that device.
int static_scratch(void** out, const char* who) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(PITH_ERR_LAUNCH, "%s: hipGetDevice: %s", who, hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(PITH_ERR_UNSUPPORTED, "%s: device index %d beyond %d", who, dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return fail(PITH_ERR_LAUNCH, "%s: hipGetSymbolAddress(scratch) on device %d: %s", who, dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return PITH_OK;
}

}  // namespace

extern "C" int pith_attn_bwd_dkdv(const pith_attn_bwd_args* a, pith_stream_t stream) {
  const int rc = validate_bwd(a, "pith_attn_bwd_dkdv", false, true);
  if (rc != PITH_OK) return rc;
  // Head groups are split only when the caller brought a workspace that is large enough.
  int split = pick_split(a);
  if (!(split > 1 && a->workspace && a->workspace_bytes >= workspace_bytes_for(a, split))) split = 1;
  if (a->workspace && !aligned16(a->workspace)) return fail(PITH_ERR_MISALIGNED, "pith_attn_bwd_dkdv: workspace must be 16-byte aligned");
  if (a->k_pe && (!a->workspace || a->workspace_bytes < workspace_bytes_for(a, split)))
    return fail(PITH_ERR_BAD_SHAPE, "pith_attn_bwd_dkdv: keys in two parts need a workspace of %lld bytes, %lld given",
                (long long)workspace_bytes_for(a, split), (long long)(a->workspace ? a->workspace_bytes : 0));
  return run_dkdv(a, split, a->workspace, (hipStream_t)stream, "pith_attn_bwd_dkdv");
}

extern "C" int pith_attn_bwd_dkdv_static(const pith_attn_bwd_args* a, pith_stream_t stream) {
  const char* who = "pith_attn_bwd_dkdv_static";
  const int rc = validate_bwd(a, who, false, true);
  if (rc != PITH_OK) return rc;
  const int split = pick_split(a);
  const int64_t need = workspace_bytes_for(a, split);
  if (need > kStaticScratchBytes)
    return fail(PITH_ERR_UNSUPPORTED,
                "%s: the head-split partial sums of this shape need %lld bytes, the built-in scratch holds %lld "
                "(use pith_attn_bwd_dkdv with a caller-provided workspace)",
                who, (long long)need, (long long)kStaticScratchBytes);
  void* ws = nullptr;
  if (need > 0) {
    const int src = static_scratch(&ws, who);
    if (src != PITH_OK) return src;
  }
  return run_dkdv(a, split, ws, (hipStream_t)stream, who);
}
