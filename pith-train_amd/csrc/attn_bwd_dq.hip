// Query-gradient kernel of one chunk attention backward for gfx950, against an external
// (ring-combined) base-2 LSE and delta = rowsum(O*dO); plus the argument checks shared with the
// dK/dV kernel. Follows pithtrain/operators/mla/triton.py:205-266 (non-causal :392-441):
// P = exp2(kappa*s - lse2) in fp32, masked entries 0, dS = P*(dP - delta)*scale rounded to bf16,
// fp32 accumulation of dQ += dS K.
//
// The query side is stationary in registers as B operands (a lane owns one query row), K/V tiles
// stream through LDS as A operands, and the score tile is produced with the query index as its
// COLUMN: lse and delta are then per-lane scalars and dS^T feeds dQ^T += K^T dS^T from registers
// (slot order, see attn_tiles.h) with K^T coming from transposing LDS reads.
#include "attn_bwd_common.h"

namespace pith {
namespace {

// =============================================================================================
// dQ kernel. Workgroup = WAVES wavefronts x (32*QB) query rows of one (batch, head); key tiles of
// 32*NB keys. With QB = NB = 1 a wavefront stays below 256 registers and two share a SIMD. Per tile: S^T = K Q^T, dP^T = V dO^T, dS^T = P^T o (dP^T - delta) * scale,
// dQ^T += K^T dS^T.
template <int DQK, int DV, bool CAUSAL, int QB, int NB, int WAVES, typename OutT>
__global__ __launch_bounds__(WAVES * 64) void attn_bwd_dq_kernel(BwdParams p) {
  constexpr int THREADS = WAVES * 64;
  constexpr int KS = DQK / 16, VS = DV / 16, DB = DQK / 32;
  constexpr int BN = 32 * NB;
  constexpr int ROWS_WAVE = 32 * QB, BM = WAVES * ROWS_WAVE;
  constexpr int KP = DQK * 2 + 80;  // read straight and transposed
  constexpr int VP = DV * 2 + 16;   // read straight only
  constexpr int kKTile = BN * KP, kVTile = BN * VP;
  __shared__ __attribute__((aligned(16))) char smem[2 * (kKTile + kVTile)];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, g = lane >> 5;
  int m_tile, h, b;
  decode_block(blockIdx.x, p.Hq, p.B, p.tiles, p.group, m_tile, h, b);
  const int hk = h / p.group;
  const int m0 = m_tile * BM;
  const int q_wave0 = m0 + wave * ROWS_WAVE;

  const int64_t q_row_stride = (int64_t)p.HqT * DQK;
  const int64_t do_row_stride = (int64_t)p.HqT * DV;
  const int64_t k_row_stride = (int64_t)p.HkvT * DQK;
  const int64_t v_row_stride = (int64_t)p.HkvT * DV;
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
  int n_tiles_wg = n_tiles_all;
  if (CAUSAL) n_tiles_wg = min(n_tiles_all, (m0 + BM - 1) / BN + 1);

  TileCopy<BN, DQK, KP, THREADS> kcopy;
  TileCopy<BN, DV, VP, THREADS> vcopy;
  kcopy.fetch(kh, k_row_stride, 0, p.Skv, tid);
  vcopy.fetch(vh, v_row_stride, 0, p.Skv, tid);
  kcopy.commit(smem, tid);
  vcopy.commit(smem + kKTile, tid);
  wait_all_vector_loads();
  __syncthreads();

  for (int t = 0; t < n_tiles_wg; ++t) {
    const char* ktile = smem + (t & 1) * (kKTile + kVTile);
    const char* vtile = ktile + kKTile;
    const bool have_next = t + 1 < n_tiles_wg;
    if (have_next) {
      kcopy.fetch(kh, k_row_stride, (t + 1) * BN, p.Skv, tid);
      vcopy.fetch(vh, v_row_stride, (t + 1) * BN, p.Skv, tid);
    }

    // No branch around the matrix instructions: a wave whose rows lie entirely above this tile
    // under the causal mask processes it like any other (its P is all zeros), which keeps the
    // accumulators in place across iterations; the workgroup waits for its last wave anyway.
    {
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
      const bool masked = (CAUSAL && (n0 + BN - 1 > q_wave0)) || (n0 + BN > p.Skv);  // wave-uniform
      bf16x8 dsf[QB][2 * NB];
      // With registers to spare (small head dims) the mask is a pass of its own under the
      // wave-uniform branch, which saves a compare and a select per element on unmasked tiles;
      // at 192/128 that version spills, and the test stays inside the element loop.
      constexpr bool kMaskPass = DQK + DV <= 192;
      if (kMaskPass) {
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
#pragma unroll
          for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int v = 0; v < 16; ++v) s[nb][qb][v] = __builtin_amdgcn_exp2f(s[nb][qb][v] * p.kappa - lse_q[qb]);
        if (masked) {
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) {
            const int qrow = q_wave0 + qb * 32 + c;
            const int limit = CAUSAL ? min(qrow, p.Skv - 1) : p.Skv - 1;
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
              for (int v = 0; v < 16; ++v)
                if (n0 + nb * 32 + acc_row(v, g) > limit) s[nb][qb][v] = 0.f;
          }
        }
      }
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const int qrow = q_wave0 + qb * 32 + c;
        const int limit = CAUSAL ? min(qrow, p.Skv - 1) : p.Skv - 1;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            float pr = s[nb][qb][v];
            if (!kMaskPass) {
              pr = __builtin_amdgcn_exp2f(pr * p.kappa - lse_q[qb]);
              if (masked && (n0 + nb * 32 + acc_row(v, g) > limit)) pr = 0.f;
            }
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

template <int DQK, int DV, int QB, int NB, int WAVES>
void launch_dq(BwdParams p, const pith_attn_bwd_args* a, hipStream_t st) {
  constexpr int BM = WAVES * 32 * QB;
  p.tiles = (int)((a->Sq + BM - 1) / BM);
  p.accumulate = a->accumulate_dq;
  const dim3 grid((unsigned)(p.tiles * a->Hq * a->B)), block(WAVES * 64);
  const bool f32 = a->dq_dtype == PITH_F32;
  if constexpr (DQK == 128 && DV == 128) {
    static_assert(BM == 256, "the 128-dim kernel owns 256 query rows per workgroup");
    launch_dq_d128(p, a->causal != 0, f32, st);
  } else {
    if (a->causal) {
      if (f32) hipLaunchKernelGGL((attn_bwd_dq_kernel<DQK, DV, true, QB, NB, WAVES, float>), grid, block, 0, st, p);
      else hipLaunchKernelGGL((attn_bwd_dq_kernel<DQK, DV, true, QB, NB, WAVES, __bf16>), grid, block, 0, st, p);
    } else {
      if (f32) hipLaunchKernelGGL((attn_bwd_dq_kernel<DQK, DV, false, QB, NB, WAVES, float>), grid, block, 0, st, p);
      else hipLaunchKernelGGL((attn_bwd_dq_kernel<DQK, DV, false, QB, NB, WAVES, __bf16>), grid, block, 0, st, p);
    }
  }
}

}  // namespace

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
  if ((a->q_row_heads && (a->q_row_heads < a->Hq || a->q_row_heads > 65535)) ||
      (a->kv_row_heads && (a->kv_row_heads < a->Hkv || a->kv_row_heads > 65535)))
    return fail(PITH_ERR_BAD_SHAPE, "%s: q_row_heads=%lld / kv_row_heads=%lld must be 0 or at least Hq=%lld / Hkv=%lld", who,
                (long long)a->q_row_heads, (long long)a->kv_row_heads, (long long)a->Hq, (long long)a->Hkv);
  if (a->k_pe && (a->q_row_heads > a->Hq || a->kv_row_heads > a->Hkv))
    return fail(PITH_ERR_UNSUPPORTED, "%s: keys in two parts cannot be combined with a head range of wider tensors", who);
  if (a->dkv_zero_tail < 0 || a->dkv_zero_tail > (1 << 24))
    return fail(PITH_ERR_BAD_SHAPE, "%s: dkv_zero_tail=%lld out of range", who, (long long)a->dkv_zero_tail);
  if (a->causal && a->Sq != a->Skv)
    return fail(PITH_ERR_UNSUPPORTED, "%s: causal needs Sq == Skv (got %lld, %lld)", who, (long long)a->Sq, (long long)a->Skv);
  if (a->Sq > (1 << 24) || a->Skv > (1 << 24) || a->Hq > 65535 || a->B > 65535 ||
      ((a->Sq + 31) / 32) * a->Hq * a->B > 0x7fffffffLL)
    return fail(PITH_ERR_UNSUPPORTED, "%s: sequence, head or batch count beyond the launch grid limits", who);
  if (!(a->scale > 0.f) || !(a->scale < INFINITY))
    return fail(PITH_ERR_BAD_SHAPE, "%s: scale=%g must be positive and finite", who, (double)a->scale);
  const int dt = need_dq ? a->dq_dtype : a->dkv_dtype;
  if (dt != PITH_BF16 && dt != PITH_F32) return fail(PITH_ERR_BAD_DTYPE, "%s: output dtype %d is not bf16/fp32", who, dt);
  if (!aligned16(a->q) || !aligned16(a->k) || !aligned16(a->v) || !aligned16(a->dout) || a->q_bs % 8 || a->k_bs % 8 ||
      a->v_bs % 8 || a->dout_bs % 8)
    return fail(PITH_ERR_MISALIGNED, "%s: input pointers / batch strides must keep 16-byte alignment", who);
  if (need_dq && (!aligned16(a->dq) || a->dq_bs % 8))
    return fail(PITH_ERR_MISALIGNED, "%s: dq pointer / batch stride must keep 16-byte alignment", who);
  if (need_dkv && (!aligned16(a->dk) || !aligned16(a->dv) || a->dk_bs % 8 || a->dv_bs % 8))
    return fail(PITH_ERR_MISALIGNED, "%s: dk/dv pointers / batch strides must keep 16-byte alignment", who);
  if (a->k_pe) {
    if (a->Dqk != 192 || a->Dv != 128)
      return fail(PITH_ERR_UNSUPPORTED, "%s: keys in two parts (k_pe) need head dims (192, 128), got (%lld, %lld)", who,
                  (long long)a->Dqk, (long long)a->Dv);
    if (!aligned16(a->k_pe) || a->k_pe_bs % 8 || a->k_pe_rs % 8 || a->k_pe_rs < 64)
      return fail(PITH_ERR_MISALIGNED, "%s: k_pe pointer / strides must keep 16-byte alignment (row stride >= 64)", who);
  }
  const bool dims_ok = (a->Dqk == 128 && a->Dv == 128) || (a->Dqk == 192 && a->Dv == 128) || (a->Dqk == 64 && a->Dv == 64);
  if (!dims_ok)
    return fail(PITH_ERR_UNSUPPORTED, "%s: head dims (Dqk=%lld, Dv=%lld) not in {(64,64),(128,128),(192,128)}", who,
                (long long)a->Dqk, (long long)a->Dv);
  return PITH_OK;
}

BwdParams make_bwd_params(const pith_attn_bwd_args* a) {
  BwdParams p;
  p.q = (const __bf16*)a->q; p.k = (const __bf16*)a->k; p.v = (const __bf16*)a->v; p.dout = (const __bf16*)a->dout;
  p.lse = a->lse; p.delta = a->delta; p.dq = a->dq; p.dk = a->dk; p.dv = a->dv;
  p.Sq = (int)a->Sq; p.Skv = (int)a->Skv; p.Hq = (int)a->Hq; p.Hkv = (int)a->Hkv; p.group = (int)(a->Hq / a->Hkv); p.B = (int)a->B;
  p.HqT = (int)(a->q_row_heads ? a->q_row_heads : a->Hq);
  p.HkvT = (int)(a->kv_row_heads ? a->kv_row_heads : a->Hkv);
  p.tiles = 0;
  p.q_bs = a->q_bs; p.k_bs = a->k_bs; p.v_bs = a->v_bs; p.dout_bs = a->dout_bs;
  p.dq_bs = a->dq_bs; p.dk_bs = a->dk_bs; p.dv_bs = a->dv_bs; p.lse_bs = a->lse_bs; p.lse_hs = a->lse_hs;
  p.scale = a->scale;
  p.kappa = a->scale * 1.44269504088896340736f;
  p.accumulate = 0;
  p.split = 1;
  p.ws_dk = nullptr;
  p.ws_dv = nullptr;
  p.k_pe = (const __bf16*)a->k_pe; p.k_pe_bs = a->k_pe_bs; p.k_pe_rs = a->k_pe_rs;
  p.ws_dkpe = nullptr;
  p.ds = nullptr;
  p.ds_qt = (int)((a->Sq + 63) / 64);
  p.ds_kb = (int)((a->Skv + kDkdvBlockN - 1) / kDkdvBlockN);
  p.ds_hs = (a->causal ? ds_tile_start<true>(p.ds_qt, p.ds_kb) : ds_tile_start<false>(p.ds_qt, p.ds_kb)) * kDsBlockBytes;
  p.dq_final = nullptr; p.dq_final_bs = 0; p.final_r0 = p.final_r1 = 0;
  p.zero_tail = 0; p.main_blocks = 0x7fffffff; p.walk_desc = 0;
  return p;
}

int64_t ds_bytes_for(const pith_attn_bwd_args* a) {
  if (!a || a->Dqk != 128 || a->Dv != 128 || a->k_pe || a->B <= 0 || a->Hq <= 0 || a->Sq <= 0 || a->Skv <= 0) return 0;
  const int qt = (int)((a->Sq + 63) / 64), kb = (int)((a->Skv + kDkdvBlockN - 1) / kDkdvBlockN);
  // a causal call (Sq == Skv) keeps only the key blocks at or below the diagonal of every query tile
  const int64_t blocks = a->causal ? ds_tile_start<true>(qt, kb) : ds_tile_start<false>(qt, kb);
  return a->B * a->Hq * blocks * kDsBlockBytes;
}

}  // namespace pith

using namespace pith;

extern "C" int64_t pith_attn_bwd_ds_bytes(const pith_attn_bwd_args* a) { return ds_bytes_for(a); }

extern "C" int pith_attn_bwd_dq(const pith_attn_bwd_args* a, pith_stream_t stream) {
  const int rc = validate_bwd(a, "pith_attn_bwd_dq", true, false);
  if (rc != PITH_OK) return rc;
  BwdParams p = make_bwd_params(a);
  if (a->dq_final) {
    if (a->dq_dtype != PITH_F32 || a->Dv != 128 || (a->Dqk != 128 && a->Dqk != 192))
      return fail(PITH_ERR_UNSUPPORTED, "pith_attn_bwd_dq: dq_final needs an fp32 dq and head dims (128,128) or (192,128)");
    if (!aligned16(a->dq_final) || a->dq_final_bs % 8)
      return fail(PITH_ERR_MISALIGNED, "pith_attn_bwd_dq: dq_final pointer / batch stride must keep 16-byte alignment");
    int64_t r0 = a->dq_final_rows[0], r1 = a->dq_final_rows[1];
    if (r0 == 0 && r1 == 0) r1 = a->Sq;
    if (r0 < 0 || r1 < r0 || r1 > a->Sq || r0 % 32 || (r1 % 32 && r1 != a->Sq))
      return fail(PITH_ERR_BAD_SHAPE, "pith_attn_bwd_dq: dq_final_rows = [%lld, %lld) must lie within the %lld query rows on multiples of 32",
                  (long long)a->dq_final_rows[0], (long long)a->dq_final_rows[1], (long long)a->Sq);
    p.dq_final = reinterpret_cast<__bf16*>(a->dq_final);
    p.dq_final_bs = a->dq_final_bs;
    p.final_r0 = (int)r0;
    p.final_r1 = (int)r1;
  }
  hipStream_t st = (hipStream_t)stream;
  begin_launch();
  if (a->ds && ds_bytes_for(a) > 0 && a->ds_bytes >= ds_bytes_for(a)) {
    // dS was left by the dK/dV call of the same chunk: one product instead of three
    if ((uintptr_t)a->ds % 256) return fail(PITH_ERR_MISALIGNED, "pith_attn_bwd_dq: ds must be 256-byte aligned");
    BwdParams q = p;
    q.ds = reinterpret_cast<char*>(a->ds);
    q.tiles = (int)((a->Sq + 511) / 512);
    q.accumulate = a->accumulate_dq;
    launch_dq_from_ds(q, a->causal != 0, a->dq_dtype == PITH_F32, st);
    return check_launch("pith_attn_bwd_dq");
  }
  const bool half = a->Dqk == 192 || prefer_half_rows(a->Sq, a->Hq, a->B, a->causal != 0);
  if (a->Dqk == 192 || (a->Dqk == 128 && half)) {
    // early / late wave roles with 128-row workgroups whose wave pairs split every tile's keys: the
    // only direct-load form for 192-feature queries, and the better one for 128 features when
    // 256-row workgroups would leave compute units idle
    BwdParams q = p;
    q.tiles = (int)((a->Sq + 127) / 128);
    q.accumulate = a->accumulate_dq;
    launch_dq_direct(q, (int)a->Dqk, a->causal != 0, a->dq_dtype == PITH_F32, st);
  } else if (a->Dqk == 128) {
    launch_dq<128, 128, 1, 2, 8>(p, a, st);
  } else {
    // short query ranges: workgroups of 4 wavefronts x 32 rows, so that no compute unit idles
    const bool few = ((a->Sq + 255) / 256) * a->Hq * a->B * 4 < 3 * (int64_t)compute_units_or_default();
    if (few) launch_dq<64, 64, 1, 1, 4>(p, a, st);
    else launch_dq<64, 64, 1, 1, 8>(p, a, st);
  }
  return check_launch("pith_attn_bwd_dq");
}

