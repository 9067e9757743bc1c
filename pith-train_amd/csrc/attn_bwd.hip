// One chunk attention backward for gfx950 against an external (ring-combined) base-2 LSE and
// delta = rowsum(O*dO). Two kernels, as in pithtrain/operators/mla/triton.py:
//   dK/dV (:130-197, non-causal :331-384): key-tile stationary, streams Q / dO tiles;
//   dQ    (:205-266, non-causal :392-441): query-tile stationary, streams K / V tiles.
// Numerics as in the reference: P = exp2(kappa*s - lse2) in fp32, masked entries 0, P rounded to
// bf16 for dV, dS = P*(dP - delta)*scale rounded to bf16 for dK and dQ, fp32 accumulation.
//
// Both kernels keep the stationary side in registers as B operands (a lane owns one stationary
// row), stream the other side through LDS as A operands, and produce the score tile with the
// stationary index as its COLUMN. The products that contract over the streamed index then take
// P / dS from registers (slot order, see attn_tiles.h) and the streamed tile through transposing
// LDS reads.
#include "attn_tiles.h"

namespace pith {
namespace {

constexpr int kBwdThreads = 256;

struct BwdParams {
  const __bf16* q;
  const __bf16* k;
  const __bf16* v;
  const __bf16* dout;
  const float* lse;
  const float* delta;
  void* dq;
  void* dk;
  void* dv;
  int Sq, Skv, Hq, Hkv, group;
  int tiles;  // query tiles (dQ kernel) or key tiles (dK/dV kernel) in the grid's x dimension
  int64_t q_bs, k_bs, v_bs, dout_bs, dq_bs, dk_bs, dv_bs, lse_bs, lse_hs;
  float kappa, scale;
  int accumulate;
};

// Stores 4 consecutive output features held by one lane; OutT is __bf16 or float.
template <typename OutT>
__device__ __forceinline__ void store4(OutT* dst, float a0, float a1, float a2, float a3, bool accumulate);

template <>
__device__ __forceinline__ void store4<float>(float* dst, float a0, float a1, float a2, float a3, bool accumulate) {
  f32x4 r = {a0, a1, a2, a3};
  if (accumulate) r += *reinterpret_cast<const f32x4*>(dst);
  *reinterpret_cast<f32x4*>(dst) = r;
}

template <>
__device__ __forceinline__ void store4<__bf16>(__bf16* dst, float a0, float a1, float a2, float a3, bool accumulate) {
  if (accumulate) {
    const u32x2 old = *reinterpret_cast<const u32x2*>(dst);
    a0 += bf16lo_to_f32(old[0]);
    a1 += bf16hi_to_f32(old[0]);
    a2 += bf16lo_to_f32(old[1]);
    a3 += bf16hi_to_f32(old[1]);
  }
  u32x2 w;
  w[0] = pack_bf16x2(a0, a1);
  w[1] = pack_bf16x2(a2, a3);
  *reinterpret_cast<u32x2*>(dst) = w;
}

// =============================================================================================
// dQ kernel. Workgroup = 4 wavefronts x (32*QB) query rows of one (batch, head); key tiles of
// 32*NB keys. Per tile: S^T = K Q^T, dP^T = V dO^T, dS^T = P^T o (dP^T - delta) * scale,
// dQ^T += K^T dS^T.
template <int DQK, int DV, bool CAUSAL, int QB, int NB, typename OutT>
__global__ __launch_bounds__(kBwdThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void attn_bwd_dq_kernel(
    BwdParams p) {
  constexpr int KS = DQK / 16, VS = DV / 16, DB = DQK / 32;
  constexpr int BN = 32 * NB;
  constexpr int ROWS_WAVE = 32 * QB, BM = 4 * ROWS_WAVE;
  constexpr int KP = DQK * 2 + 80;  // read straight and transposed
  constexpr int VP = DV * 2 + 16;   // read straight only
  constexpr int kKTile = BN * KP, kVTile = BN * VP;
  __shared__ __attribute__((aligned(16))) char smem[2 * (kKTile + kVTile)];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, g = lane >> 5;
  const int m_tile = p.tiles - 1 - blockIdx.x;
  const int h = blockIdx.y, b = blockIdx.z;
  const int hk = h / p.group;
  const int m0 = m_tile * BM;
  const int q_wave0 = m0 + wave * ROWS_WAVE;

  const int64_t q_row_stride = (int64_t)p.Hq * DQK;
  const int64_t do_row_stride = (int64_t)p.Hq * DV;
  const int64_t k_row_stride = (int64_t)p.Hkv * DQK;
  const int64_t v_row_stride = (int64_t)p.Hkv * DV;
  const __bf16* qh = p.q + b * p.q_bs + (int64_t)h * DQK;
  const __bf16* doh = p.dout + b * p.dout_bs + (int64_t)h * DV;
  const __bf16* kh = p.k + b * p.k_bs + (int64_t)hk * DQK;
  const __bf16* vh = p.v + b * p.v_bs + (int64_t)hk * DV;
  const float* lse = p.lse + b * p.lse_bs + (int64_t)h * p.lse_hs;
  const float* delta = p.delta + b * p.lse_bs + (int64_t)h * p.lse_hs;

  bf16x8 qf[QB][KS], dof[QB][VS];
  float lse_q[QB], delta_q[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    int row = q_wave0 + qb * 32 + c;
    row = row < p.Sq ? row : p.Sq - 1;
    const __bf16* src = qh + row * q_row_stride + g * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[qb][ks] = *reinterpret_cast<const bf16x8*>(src + ks * 16);
    const __bf16* dsrc = doh + row * do_row_stride + g * 8;
#pragma unroll
    for (int ks = 0; ks < VS; ++ks) dof[qb][ks] = *reinterpret_cast<const bf16x8*>(dsrc + ks * 16);
    lse_q[qb] = lse[row];
    delta_q[qb] = delta[row];
  }

  f32x16 acc[DB][QB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][qb][v] = 0.f;

  const int n_tiles_all = (p.Skv + BN - 1) / BN;
  int n_tiles_wg = n_tiles_all, n_tiles_wave = n_tiles_all;
  if (CAUSAL) {
    n_tiles_wg = min(n_tiles_all, (m0 + BM - 1) / BN + 1);
    n_tiles_wave = min(n_tiles_all, (q_wave0 + ROWS_WAVE - 1) / BN + 1);
  }

  TileCopy<BN, DQK, KP, kBwdThreads> kcopy;
  TileCopy<BN, DV, VP, kBwdThreads> vcopy;
  kcopy.fetch(kh, k_row_stride, 0, p.Skv, tid);
  vcopy.fetch(vh, v_row_stride, 0, p.Skv, tid);
  kcopy.commit(smem, tid);
  vcopy.commit(smem + kKTile, tid);
  __syncthreads();

  for (int t = 0; t < n_tiles_wg; ++t) {
    const char* ktile = smem + (t & 1) * (kKTile + kVTile);
    const char* vtile = ktile + kKTile;
    const bool have_next = t + 1 < n_tiles_wg;
    if (have_next) {
      kcopy.fetch(kh, k_row_stride, (t + 1) * BN, p.Skv, tid);
      vcopy.fetch(vh, v_row_stride, (t + 1) * BN, p.Skv, tid);
    }

    if (t < n_tiles_wave) {
      f32x16 s[NB][QB], dp[NB][QB];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            s[nb][qb][v] = 0.f;
            dp[nb][qb][v] = 0.f;
          }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const bf16x8 a = lds_read_straight(ktile, KP, nb * 32 + c, ks * 16 + g * 8);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) s[nb][qb] = mfma32(a, qf[qb][ks], s[nb][qb]);
        }
#pragma unroll
      for (int ks = 0; ks < VS; ++ks)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const bf16x8 a = lds_read_straight(vtile, VP, nb * 32 + c, ks * 16 + g * 8);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) dp[nb][qb] = mfma32(a, dof[qb][ks], dp[nb][qb]);
        }

      const int n0 = t * BN;
      const bool masked = (CAUSAL && (n0 + BN - 1 > q_wave0)) || (n0 + BN > p.Skv);
      bf16x8 dsf[QB][2 * NB];
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const int qrow = q_wave0 + qb * 32 + c;
        const int limit = CAUSAL ? min(qrow, p.Skv - 1) : p.Skv - 1;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            float pr = __builtin_amdgcn_exp2f(s[nb][qb][v] * p.kappa - lse_q[qb]);
            if (masked && (n0 + nb * 32 + acc_row(v, g) > limit)) pr = 0.f;
            s[nb][qb][v] = pr * (dp[nb][qb][v] - delta_q[qb]) * p.scale;
          }
#pragma unroll
          for (int jj = 0; jj < 2; ++jj) {
            const f32x16& x = s[nb][qb];
            dsf[qb][2 * nb + jj] = to_bf16x8(x[8 * jj], x[8 * jj + 1], x[8 * jj + 2], x[8 * jj + 3], x[8 * jj + 4],
                                             x[8 * jj + 5], x[8 * jj + 6], x[8 * jj + 7]);
          }
        }
      }

#pragma unroll
      for (int j = 0; j < 2 * NB; ++j)
#pragma unroll
        for (int i = 0; i < DB; ++i) {
          const bf16x8 a = lds_read_transposed(ktile, KP, 16 * j, 32 * i, lane);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) acc[i][qb] = mfma32(a, dsf[qb][j], acc[i][qb]);
        }
    }

    if (have_next) {
      char* nk = smem + ((t + 1) & 1) * (kKTile + kVTile);
      kcopy.commit(nk, tid);
      vcopy.commit(nk + kKTile, tid);
    }
    __syncthreads();
  }

  OutT* dqh = reinterpret_cast<OutT*>(p.dq) + b * p.dq_bs + (int64_t)h * DQK;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int qrow = q_wave0 + qb * 32 + c;
    if (qrow < p.Sq) {
      OutT* dst = dqh + qrow * q_row_stride;
#pragma unroll
      for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4)
          store4<OutT>(dst + 32 * i + 8 * b4 + 4 * g, acc[i][qb][4 * b4], acc[i][qb][4 * b4 + 1],
                       acc[i][qb][4 * b4 + 2], acc[i][qb][4 * b4 + 3], p.accumulate != 0);
    }
  }
}

// =============================================================================================
// dK/dV kernel. Workgroup = 4 wavefronts x 32 key rows of one (batch, kv head); it loops over
// the query heads of the kv head's group and over query tiles of 32*MB rows. Per tile:
// S = Q K^T, dP = dO V^T, P = exp2(kappa*S - lse), dV^T += dO^T P, dS = P o (dP - delta) * scale,
// dK^T += Q^T dS.
template <int DQK, int DV, bool CAUSAL, int MB, typename OutT>
__global__ __launch_bounds__(kBwdThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void attn_bwd_dkdv_kernel(
    BwdParams p) {
  constexpr int KS = DQK / 16, VS = DV / 16, DB = DQK / 32, DVB = DV / 32;
  constexpr int BM = 32 * MB;     // query tile rows
  constexpr int BN = 128;         // key rows per workgroup
  constexpr int QP = DQK * 2 + 80, OP = DV * 2 + 80;  // both tiles are read straight and transposed
  constexpr int kQTile = BM * QP, kOTile = BM * OP, kStat = 2 * BM * 4;
  constexpr int kStage = kQTile + kOTile + kStat;
  __shared__ __attribute__((aligned(16))) char smem[2 * kStage];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, g = lane >> 5;
  const int n_tile = blockIdx.x;  // early key tiles see the most query tiles under the causal mask
  const int hk = blockIdx.y, b = blockIdx.z;
  const int kv_wg0 = n_tile * BN;
  const int kv_wave0 = kv_wg0 + wave * 32;
  const int key = kv_wave0 + c;  // the key row this lane owns in score tiles

  const int64_t q_row_stride = (int64_t)p.Hq * DQK;
  const int64_t do_row_stride = (int64_t)p.Hq * DV;
  const int64_t k_row_stride = (int64_t)p.Hkv * DQK;
  const int64_t v_row_stride = (int64_t)p.Hkv * DV;

  bf16x8 kf[KS], vf[VS];
  {
    const int row = key < p.Skv ? key : p.Skv - 1;
    const __bf16* ksrc = p.k + b * p.k_bs + row * k_row_stride + (int64_t)hk * DQK + g * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kf[ks] = *reinterpret_cast<const bf16x8*>(ksrc + ks * 16);
    const __bf16* vsrc = p.v + b * p.v_bs + row * v_row_stride + (int64_t)hk * DV + g * 8;
#pragma unroll
    for (int ks = 0; ks < VS; ++ks) vf[ks] = *reinterpret_cast<const bf16x8*>(vsrc + ks * 16);
  }

  f32x16 dk_acc[DB], dv_acc[DVB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) dk_acc[i][v] = 0.f;
#pragma unroll
  for (int i = 0; i < DVB; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) dv_acc[i][v] = 0.f;

  // Query tiles to visit: all of them, or from the diagonal down under the causal mask.
  const int m_tiles_all = (p.Sq + BM - 1) / BM;
  const int m_start_wg = CAUSAL ? min(kv_wg0 / BM, m_tiles_all) : 0;
  const int m_start_wave = CAUSAL ? kv_wave0 / BM : 0;
  const int n_m = m_tiles_all - m_start_wg;
  const int n_iter = n_m * p.group;

  TileCopy<BM, DQK, QP, kBwdThreads> qcopy;
  TileCopy<BM, DV, OP, kBwdThreads> ocopy;
  float stat = 0.f;  // threads 0..63 carry lse, 64..127 carry delta of the tile's rows
  auto fetch = [&](int it) {
    const int hq = hk * p.group + it / n_m;
    const int mt = m_start_wg + it % n_m;
    qcopy.fetch(p.q + b * p.q_bs + (int64_t)hq * DQK, q_row_stride, mt * BM, p.Sq, tid);
    ocopy.fetch(p.dout + b * p.dout_bs + (int64_t)hq * DV, do_row_stride, mt * BM, p.Sq, tid);
    if (tid < 2 * BM) {
      int row = mt * BM + (tid & (BM - 1));
      row = row < p.Sq ? row : p.Sq - 1;
      const float* src = (tid < BM ? p.lse : p.delta) + b * p.lse_bs + (int64_t)hq * p.lse_hs;
      stat = src[row];
    }
  };
  auto commit = [&](int stage) {
    char* base = smem + stage * kStage;
    qcopy.commit(base, tid);
    ocopy.commit(base + kQTile, tid);
    if (tid < 2 * BM) reinterpret_cast<float*>(base + kQTile + kOTile)[tid] = stat;
  };

  if (n_iter > 0) {
    fetch(0);
    commit(0);
  }
  __syncthreads();

  for (int it = 0; it < n_iter; ++it) {
    const char* qtile = smem + (it & 1) * kStage;
    const char* otile = qtile + kQTile;
    const float* lse_s = reinterpret_cast<const float*>(otile + kOTile);
    const float* delta_s = lse_s + BM;
    const bool have_next = it + 1 < n_iter;
    if (have_next) fetch(it + 1);

    const int mt = m_start_wg + it % n_m;
    if (mt >= m_start_wave) {
      const int q0 = mt * BM;
      f32x16 s[MB], dp[MB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          s[mb][v] = 0.f;
          dp[mb][v] = 0.f;
        }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          const bf16x8 a = lds_read_straight(qtile, QP, mb * 32 + c, ks * 16 + g * 8);
          s[mb] = mfma32(a, kf[ks], s[mb]);
        }
#pragma unroll
      for (int ks = 0; ks < VS; ++ks)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          const bf16x8 a = lds_read_straight(otile, OP, mb * 32 + c, ks * 16 + g * 8);
          dp[mb] = mfma32(a, vf[ks], dp[mb]);
        }

      // Rows of the score tile are queries q0 + mb*32 + acc_row(v, g); the lane's column is `key`.
      const bool masked = (CAUSAL && (q0 < kv_wave0 + 31)) || (q0 + BM > p.Sq);
      bf16x8 pf[2 * MB], dsf[2 * MB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4) {
          const int r0 = mb * 32 + 8 * b4 + 4 * g;
          const f32x4 l4 = *reinterpret_cast<const f32x4*>(lse_s + r0);
          const f32x4 d4 = *reinterpret_cast<const f32x4*>(delta_s + r0);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int v = 4 * b4 + i;
            float pr = __builtin_amdgcn_exp2f(s[mb][v] * p.kappa - l4[i]);
            if (masked) {
              const int qrow = q0 + r0 + i;
              if ((CAUSAL && key > qrow) || qrow >= p.Sq) pr = 0.f;
            }
            s[mb][v] = pr;
            dp[mb][v] = pr * (dp[mb][v] - d4[i]) * p.scale;
          }
        }
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          const f32x16& x = s[mb];
          pf[2 * mb + jj] = to_bf16x8(x[8 * jj], x[8 * jj + 1], x[8 * jj + 2], x[8 * jj + 3], x[8 * jj + 4],
                                      x[8 * jj + 5], x[8 * jj + 6], x[8 * jj + 7]);
          const f32x16& y = dp[mb];
          dsf[2 * mb + jj] = to_bf16x8(y[8 * jj], y[8 * jj + 1], y[8 * jj + 2], y[8 * jj + 3], y[8 * jj + 4],
                                       y[8 * jj + 5], y[8 * jj + 6], y[8 * jj + 7]);
        }
      }

#pragma unroll
      for (int j = 0; j < 2 * MB; ++j) {
#pragma unroll
        for (int i = 0; i < DVB; ++i) {
          const bf16x8 a = lds_read_transposed(otile, OP, 16 * j, 32 * i, lane);
          dv_acc[i] = mfma32(a, pf[j], dv_acc[i]);
        }
#pragma unroll
        for (int i = 0; i < DB; ++i) {
          const bf16x8 a = lds_read_transposed(qtile, QP, 16 * j, 32 * i, lane);
          dk_acc[i] = mfma32(a, dsf[j], dk_acc[i]);
        }
      }
    }

    if (have_next) commit((it + 1) & 1);
    __syncthreads();
  }

  if (key < p.Skv) {
    OutT* dkh = reinterpret_cast<OutT*>(p.dk) + b * p.dk_bs + key * k_row_stride + (int64_t)hk * DQK;
    OutT* dvh = reinterpret_cast<OutT*>(p.dv) + b * p.dv_bs + key * v_row_stride + (int64_t)hk * DV;
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4)
        store4<OutT>(dkh + 32 * i + 8 * b4 + 4 * g, dk_acc[i][4 * b4], dk_acc[i][4 * b4 + 1], dk_acc[i][4 * b4 + 2],
                     dk_acc[i][4 * b4 + 3], p.accumulate != 0);
#pragma unroll
    for (int i = 0; i < DVB; ++i)
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4)
        store4<OutT>(dvh + 32 * i + 8 * b4 + 4 * g, dv_acc[i][4 * b4], dv_acc[i][4 * b4 + 1], dv_acc[i][4 * b4 + 2],
                     dv_acc[i][4 * b4 + 3], p.accumulate != 0);
  }
}

int validate_bwd(const pith_attn_bwd_args* a, const char* who, bool need_dq, bool need_dkv) {
  if (!a) return fail(PITH_ERR_NULL_POINTER, "%s: args is NULL", who);
  if (!a->q || !a->k || !a->v || !a->dout || !a->lse || !a->delta)
    return fail(PITH_ERR_NULL_POINTER, "%s: NULL input tensor pointer", who);
  if (need_dq && !a->dq) return fail(PITH_ERR_NULL_POINTER, "%s: dq is NULL", who);
  if (need_dkv && (!a->dk || !a->dv)) return fail(PITH_ERR_NULL_POINTER, "%s: dk or dv is NULL", who);
  if (a->B <= 0 || a->Sq <= 0 || a->Skv <= 0 || a->Hq <= 0 || a->Hkv <= 0)
    return fail(PITH_ERR_BAD_SHAPE, "%s: B=%lld Sq=%lld Skv=%lld Hq=%lld Hkv=%lld must all be positive", who,
                (long long)a->B, (long long)a->Sq, (long long)a->Skv, (long long)a->Hq, (long long)a->Hkv);
  if (a->Hq % a->Hkv != 0)
    return fail(PITH_ERR_BAD_SHAPE, "%s: Hq=%lld is not a multiple of Hkv=%lld", who, (long long)a->Hq, (long long)a->Hkv);
  if (a->causal && a->Sq != a->Skv)
    return fail(PITH_ERR_UNSUPPORTED, "%s: causal needs Sq == Skv (got %lld, %lld)", who, (long long)a->Sq, (long long)a->Skv);
  if (a->Sq > (1 << 24) || a->Skv > (1 << 24) || a->Hq > 65535 || a->B > 65535)
    return fail(PITH_ERR_UNSUPPORTED, "%s: sequence, head or batch count beyond the launch grid limits", who);
  const int dt = need_dq ? a->dq_dtype : a->dkv_dtype;
  if (dt != PITH_BF16 && dt != PITH_F32) return fail(PITH_ERR_BAD_DTYPE, "%s: output dtype %d is not bf16/fp32", who, dt);
  if (!aligned16(a->q) || !aligned16(a->k) || !aligned16(a->v) || !aligned16(a->dout) || a->q_bs % 8 || a->k_bs % 8 ||
      a->v_bs % 8 || a->dout_bs % 8)
    return fail(PITH_ERR_MISALIGNED, "%s: input pointers / batch strides must keep 16-byte alignment", who);
  if (need_dq && (!aligned16(a->dq) || a->dq_bs % 8))
    return fail(PITH_ERR_MISALIGNED, "%s: dq pointer / batch stride must keep 16-byte alignment", who);
  if (need_dkv && (!aligned16(a->dk) || !aligned16(a->dv) || a->dk_bs % 8 || a->dv_bs % 8))
    return fail(PITH_ERR_MISALIGNED, "%s: dk/dv pointers / batch strides must keep 16-byte alignment", who);
  const bool dims_ok = (a->Dqk == 128 && a->Dv == 128) || (a->Dqk == 192 && a->Dv == 128) || (a->Dqk == 64 && a->Dv == 64);
  if (!dims_ok)
    return fail(PITH_ERR_UNSUPPORTED, "%s: head dims (Dqk=%lld, Dv=%lld) not in {(64,64),(128,128),(192,128)}", who,
                (long long)a->Dqk, (long long)a->Dv);
  return PITH_OK;
}

BwdParams make_params(const pith_attn_bwd_args* a) {
  BwdParams p;
  p.q = (const __bf16*)a->q; p.k = (const __bf16*)a->k; p.v = (const __bf16*)a->v; p.dout = (const __bf16*)a->dout;
  p.lse = a->lse; p.delta = a->delta; p.dq = a->dq; p.dk = a->dk; p.dv = a->dv;
  p.Sq = (int)a->Sq; p.Skv = (int)a->Skv; p.Hq = (int)a->Hq; p.Hkv = (int)a->Hkv; p.group = (int)(a->Hq / a->Hkv);
  p.tiles = 0;
  p.q_bs = a->q_bs; p.k_bs = a->k_bs; p.v_bs = a->v_bs; p.dout_bs = a->dout_bs;
  p.dq_bs = a->dq_bs; p.dk_bs = a->dk_bs; p.dv_bs = a->dv_bs; p.lse_bs = a->lse_bs; p.lse_hs = a->lse_hs;
  p.scale = a->scale;
  p.kappa = a->scale * 1.44269504088896340736f;
  p.accumulate = 0;
  return p;
}

template <int DQK, int DV, int QB, int NB>
void launch_dq(BwdParams p, const pith_attn_bwd_args* a, hipStream_t st) {
  constexpr int BM = 128 * QB;
  p.tiles = (int)((a->Sq + BM - 1) / BM);
  p.accumulate = a->accumulate_dq;
  const dim3 grid((unsigned)p.tiles, (unsigned)a->Hq, (unsigned)a->B), block(kBwdThreads);
  const bool f32 = a->dq_dtype == PITH_F32;
  if (a->causal) {
    if (f32) hipLaunchKernelGGL((attn_bwd_dq_kernel<DQK, DV, true, QB, NB, float>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((attn_bwd_dq_kernel<DQK, DV, true, QB, NB, __bf16>), grid, block, 0, st, p);
  } else {
    if (f32) hipLaunchKernelGGL((attn_bwd_dq_kernel<DQK, DV, false, QB, NB, float>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((attn_bwd_dq_kernel<DQK, DV, false, QB, NB, __bf16>), grid, block, 0, st, p);
  }
}

template <int DQK, int DV, int MB>
void launch_dkdv(BwdParams p, const pith_attn_bwd_args* a, hipStream_t st) {
  p.tiles = (int)((a->Skv + 127) / 128);
  p.accumulate = a->accumulate_dkv;
  const dim3 grid((unsigned)p.tiles, (unsigned)a->Hkv, (unsigned)a->B), block(kBwdThreads);
  const bool f32 = a->dkv_dtype == PITH_F32;
  if (a->causal) {
    if (f32) hipLaunchKernelGGL((attn_bwd_dkdv_kernel<DQK, DV, true, MB, float>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((attn_bwd_dkdv_kernel<DQK, DV, true, MB, __bf16>), grid, block, 0, st, p);
  } else {
    if (f32) hipLaunchKernelGGL((attn_bwd_dkdv_kernel<DQK, DV, false, MB, float>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((attn_bwd_dkdv_kernel<DQK, DV, false, MB, __bf16>), grid, block, 0, st, p);
  }
}

}  // namespace
}  // namespace pith

using namespace pith;

extern "C" int pith_attn_bwd_dq(const pith_attn_bwd_args* a, pith_stream_t stream) {
  const int rc = validate_bwd(a, "pith_attn_bwd_dq", true, false);
  if (rc != PITH_OK) return rc;
  const BwdParams p = make_params(a);
  hipStream_t st = (hipStream_t)stream;
  if (a->Dqk == 128) launch_dq<128, 128, 2, 1>(p, a, st);
  else if (a->Dqk == 192) launch_dq<192, 128, 1, 2>(p, a, st);
  else launch_dq<64, 64, 2, 1>(p, a, st);
  return check_launch("pith_attn_bwd_dq");
}

extern "C" int pith_attn_bwd_dkdv(const pith_attn_bwd_args* a, pith_stream_t stream) {
  const int rc = validate_bwd(a, "pith_attn_bwd_dkdv", false, true);
  if (rc != PITH_OK) return rc;
  const BwdParams p = make_params(a);
  hipStream_t st = (hipStream_t)stream;
  if (a->Dqk == 128) launch_dkdv<128, 128, 2>(p, a, st);
  else if (a->Dqk == 192) launch_dkdv<192, 128, 1>(p, a, st);
  else launch_dkdv<64, 64, 2>(p, a, st);
  return check_launch("pith_attn_bwd_dkdv");
}
