// One chunk attention forward for gfx950: O = softmax(scale * Q K^T [+causal]) V, base-2 LSE.
// Numerics follow pithtrain/operators/mla/triton.py:32-93 (causal) and :274-323 (non-causal):
// fp32 scores from bf16 MFMA, P = exp2(kappa*(s - m)) in fp32, row sum from the fp32 P, P rounded
// to bf16 for P V, O = acc / l rounded to bf16, LSE2 = log2(l) + kappa*m, kappa = scale*log2(e).
// One deviation in rounding only: the running maximum m is refreshed (and O, l rescaled) only when
// a row's tile maximum exceeds it by more than 2^8 in the exp2 domain; P, l and O stay consistent
// with whichever m is in force, so O and LSE2 are the same function of the inputs.
//
// Work split: a workgroup of WAVES wavefronts owns WAVES*32*QB consecutive query rows of one
// (batch, head); each wavefront owns 32*QB of them. With QB = 1 a wavefront needs fewer than 256
// registers, so two wavefronts share a SIMD and one's softmax (VALU) overlaps the other's MFMAs.
// K/V tiles of 64 keys are staged through LDS (double buffered, fetched to registers one tile
// ahead) and shared by all waves. Scores are produced TRANSPOSED, S^T = K Q^T, so that a lane
// holds one query column: the softmax row reductions are in-lane plus one exchange with the
// partner lane, and P^T feeds the second product O^T += V^T P^T straight from registers; V^T
// comes from transposing LDS reads.
#include "attn_fwd_common.h"

namespace pith {
namespace {

template <int DQK, int DV, bool CAUSAL, int QB, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void attn_fwd_kernel(FwdParams p) {
  constexpr int THREADS = WAVES * 64;
  constexpr int ROWS_WAVE = 32 * QB;
  constexpr int BM = WAVES * ROWS_WAVE;
  constexpr int BN = kFwdBlockN;
  constexpr int KS = DQK / 16;         // contraction steps of Q K^T
  constexpr int DVB = DV / 32;         // 32-row blocks of O^T
  constexpr int KP = DQK * 2 + 16;     // K tile pitch: conflict-free 16-byte row reads
  constexpr int VP = DV * 2 + 64;      // V tile pitch: conflict-free transposing reads
  constexpr int kKTile = BN * KP;
  constexpr int kVTile = BN * VP;
  __shared__ __attribute__((aligned(16))) char smem[2 * (kKTile + kVTile)];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, g = lane >> 5;

  int m_tile, h, b;
  decode_block(blockIdx.x, p.Hq, p.B, p.m_tiles, p.group, m_tile, h, b);
  const int hk = h / p.group;
  const int m0 = m_tile * BM;
  const int q_wave0 = m0 + wave * ROWS_WAVE;

  const int64_t q_row_stride = (int64_t)p.Hq * DQK;
  const int64_t k_row_stride = (int64_t)p.Hkv * DQK;
  const int64_t v_row_stride = (int64_t)p.Hkv * DV;
  const int64_t o_row_stride = (int64_t)p.Hq * DV;
  const __bf16* qh = p.q + b * p.q_bs + (int64_t)h * DQK;
  const __bf16* kh = p.k + b * p.k_bs + (int64_t)hk * DQK;
  const __bf16* vh = p.v + b * p.v_bs + (int64_t)hk * DV;

  // Q^T fragments (B operand): column = query row, slots = 8 consecutive features.
  bf16x8 qf[QB][KS];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    int row = q_wave0 + qb * 32 + c;
    row = row < p.Sq ? row : p.Sq - 1;
    const __bf16* src = qh + row * q_row_stride + g * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[qb][ks] = *reinterpret_cast<const bf16x8*>(src + ks * 16);
  }

  f32x16 oacc[DVB][QB];
#pragma unroll
  for (int i = 0; i < DVB; ++i)
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int v = 0; v < 16; ++v) oacc[i][qb][v] = 0.f;
  float m_run[QB], l_run[QB];  // l_run: this lane's share of the row sum (partner lane holds the rest)
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m_run[qb] = -INFINITY;
    l_run[qb] = 0.f;
  }

  // Number of key tiles this workgroup / this wavefront has to visit.
  const int n_tiles_all = (p.Skv + BN - 1) / BN;
  int n_tiles_wg = n_tiles_all, n_tiles_wave = n_tiles_all;
  if (CAUSAL) {
    n_tiles_wg = min(n_tiles_all, (m0 + BM - 1) / BN + 1);
    n_tiles_wave = min(n_tiles_all, (q_wave0 + ROWS_WAVE - 1) / BN + 1);
  }

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

    if (t < n_tiles_wave) {
      // ---- S^T = K Q^T : [64 keys] x [32*QB queries] as 2 x QB tiles of 32 x 32
      f32x16 s[2][QB];
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
#pragma unroll
          for (int v = 0; v < 16; ++v) s[kvb][qb][v] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int kvb = 0; kvb < 2; ++kvb) {
          const bf16x8 a = lds_read_straight(ktile, KP, kvb * 32 + c, ks * 16 + g * 8);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) s[kvb][qb] = mfma32(a, qf[qb][ks], s[kvb][qb]);
        }
      }

      // ---- mask (tiles crossing the diagonal of a causal chunk, or a ragged last tile)
      const int n0 = t * BN;
      if ((CAUSAL && (n0 + BN - 1 > q_wave0)) || (n0 + BN > p.Skv)) {
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          const int qrow = q_wave0 + qb * 32 + c;
          const int limit = CAUSAL ? min(qrow, p.Skv - 1) : p.Skv - 1;  // last visible key
#pragma unroll
          for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              const int key = n0 + kvb * 32 + acc_row(v, g);
              if (key > limit) s[kvb][qb][v] = -INFINITY;
            }
        }
      }

      // ---- online softmax, one query column per lane pair
      float mx[QB];
      bool refresh = false;
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        float x = s[0][qb][0];
#pragma unroll
        for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
          for (int v = 0; v < 16; ++v) x = fmaxf(x, s[kvb][qb][v]);
        mx[qb] = pair_max(x);
        refresh |= (mx[qb] - m_run[qb]) * p.kappa > kRescaleThreshold;  // true on the first tile (m = -inf)
      }
      if (__builtin_amdgcn_ballot_w64(refresh) != 0) {  // wave-uniform
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          const float m_new = fmaxf(m_run[qb], mx[qb]);
          // a row with no visible key so far keeps m = -inf; exp2 of (-inf - -inf) is avoided
          const float alpha = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f((m_run[qb] - m_new) * p.kappa);
          m_run[qb] = m_new;
          l_run[qb] *= alpha;
#pragma unroll
          for (int i = 0; i < DVB; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) oacc[i][qb][v] *= alpha;
        }
      }

      bf16x8 pf[QB][4];  // P^T as B operand: [query block][contraction step of 16 keys]
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const float mk = (m_run[qb] == -INFINITY) ? 0.f : m_run[qb] * p.kappa;
        float rs = 0.f;
#pragma unroll
        for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const float e = __builtin_amdgcn_exp2f(s[kvb][qb][v] * p.kappa - mk);
            s[kvb][qb][v] = e;
            rs += e;
          }
        l_run[qb] += rs;
#pragma unroll
        for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
          for (int jj = 0; jj < 2; ++jj) {
            const f32x16& x = s[kvb][qb];
            pf[qb][2 * kvb + jj] = to_bf16x8(x[8 * jj], x[8 * jj + 1], x[8 * jj + 2], x[8 * jj + 3], x[8 * jj + 4],
                                             x[8 * jj + 5], x[8 * jj + 6], x[8 * jj + 7]);
          }
      }

      // ---- O^T += V^T P^T
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int i = 0; i < DVB; ++i) {
          const bf16x8 a = lds_read_transposed(vtile, VP, 16 * j, 32 * i, lane);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) oacc[i][qb] = mfma32(a, pf[qb][j], oacc[i][qb]);
        }
      }
    }

    if (have_next) {
      char* nk = smem + ((t + 1) & 1) * (kKTile + kVTile);
      kcopy.commit(nk, tid);
      vcopy.commit(nk + kKTile, tid);
    }
    __syncthreads();
  }

  // ---- epilogue: normalise, store O (bf16) and LSE2
  __bf16* oh = p.o + b * p.o_bs + (int64_t)h * DV;
  float* lse = p.lse + b * p.lse_bs + (int64_t)h * p.lse_hs;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int qrow = q_wave0 + qb * 32 + c;
    const float l = pair_sum(l_run[qb]);
    const float inv = l > 0.f ? 1.f / l : 0.f;
    if (qrow < p.Sq) {
      __bf16* dst = oh + qrow * o_row_stride;
#pragma unroll
      for (int i = 0; i < DVB; ++i)
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4) {
          u32x2 w;
          w[0] = pack_bf16x2(oacc[i][qb][4 * b4] * inv, oacc[i][qb][4 * b4 + 1] * inv);
          w[1] = pack_bf16x2(oacc[i][qb][4 * b4 + 2] * inv, oacc[i][qb][4 * b4 + 3] * inv);
          *reinterpret_cast<u32x2*>(dst + 32 * i + 8 * b4 + 4 * g) = w;
        }
      if (g == 0) lse[qrow] = (l > 0.f) ? __builtin_amdgcn_logf(l) + m_run[qb] * p.kappa : -INFINITY;
    }
  }
}

template <int DQK, int DV, int QB, int WAVES>
void launch_fwd(FwdParams p, const pith_attn_fwd_args* a, hipStream_t st) {
  constexpr int BM = WAVES * 32 * QB;
  p.m_tiles = (int)((a->Sq + BM - 1) / BM);
  const dim3 grid((unsigned)(p.m_tiles * a->Hq * a->B)), block(WAVES * 64);
  if (a->causal)
    hipLaunchKernelGGL((attn_fwd_kernel<DQK, DV, true, QB, WAVES>), grid, block, 0, st, p);
  else
    hipLaunchKernelGGL((attn_fwd_kernel<DQK, DV, false, QB, WAVES>), grid, block, 0, st, p);
}

// With 256 query rows per workgroup a short query range leaves compute units idle (one workgroup
// per unit at these LDS sizes): below 3/4 of the device's compute units the launch uses workgroups
// of 4 wavefronts x 32 rows instead, which doubles their number.
bool few_workgroups(int64_t Sq, int64_t Hq, int64_t B) {
  return ((Sq + 255) / 256) * Hq * B * 4 < 3 * (int64_t)compute_units_or_default();
}

}  // namespace
}  // namespace pith

using namespace pith;

extern "C" int pith_attn_fwd(const pith_attn_fwd_args* a, pith_stream_t stream) {
  if (!a) return fail(PITH_ERR_NULL_POINTER, "pith_attn_fwd: args is NULL");
  if (!a->q || !a->k || !a->v || !a->lse || (!a->o && !(a->prev_o && a->acc_o)))
    return fail(PITH_ERR_NULL_POINTER, "pith_attn_fwd: NULL tensor pointer");
  if (a->B <= 0 || a->Sq <= 0 || a->Skv <= 0 || a->Hq <= 0 || a->Hkv <= 0)
    return fail(PITH_ERR_BAD_SHAPE, "pith_attn_fwd: B=%lld Sq=%lld Skv=%lld Hq=%lld Hkv=%lld must all be positive",
                (long long)a->B, (long long)a->Sq, (long long)a->Skv, (long long)a->Hq, (long long)a->Hkv);
  if (a->Hq % a->Hkv != 0)
    return fail(PITH_ERR_BAD_SHAPE, "pith_attn_fwd: Hq=%lld is not a multiple of Hkv=%lld", (long long)a->Hq,
                (long long)a->Hkv);
  if (!(a->scale > 0.f) || !(a->scale < INFINITY))
    return fail(PITH_ERR_BAD_SHAPE, "pith_attn_fwd: scale=%g must be positive and finite", (double)a->scale);
  if (a->causal && a->Sq != a->Skv)
    return fail(PITH_ERR_UNSUPPORTED, "pith_attn_fwd: causal needs Sq == Skv (got %lld, %lld)", (long long)a->Sq,
                (long long)a->Skv);
  if (a->Sq > (1 << 24) || a->Skv > (1 << 24) || a->Hq > 65535 || a->B > 65535 ||
      ((a->Sq + 63) / 64) * a->Hq * a->B > 0x7fffffffLL)
    return fail(PITH_ERR_UNSUPPORTED, "pith_attn_fwd: sequence, head or batch count beyond the launch grid limits");
  if (!aligned16(a->q) || !aligned16(a->k) || !aligned16(a->v) || !aligned16(a->o) || a->q_bs % 8 || a->k_bs % 8 ||
      a->v_bs % 8 || a->o_bs % 8)
    return fail(PITH_ERR_MISALIGNED, "pith_attn_fwd: tensor pointers / batch strides must keep 16-byte alignment");

  FwdParams p;
  p.q = (const __bf16*)a->q; p.k = (const __bf16*)a->k; p.v = (const __bf16*)a->v;
  p.o = (__bf16*)a->o; p.lse = a->lse;
  p.Sq = (int)a->Sq; p.Skv = (int)a->Skv; p.Hq = (int)a->Hq; p.Hkv = (int)a->Hkv; p.group = (int)(a->Hq / a->Hkv);
  p.B = (int)a->B; p.m_tiles = 0;
  p.q_bs = a->q_bs; p.k_bs = a->k_bs; p.v_bs = a->v_bs; p.o_bs = a->o_bs; p.lse_bs = a->lse_bs; p.lse_hs = a->lse_hs;
  p.kappa = a->scale * 1.44269504088896340736f;
  p.k_pe = (const __bf16*)a->k_pe; p.k_pe_bs = a->k_pe_bs; p.k_pe_rs = a->k_pe_rs;
  if (a->k_pe) {
    if (a->Dqk != 192 || a->Dv != 128)
      return fail(PITH_ERR_UNSUPPORTED, "pith_attn_fwd: keys in two parts (k_pe) need head dims (192, 128), got (%lld, %lld)",
                  (long long)a->Dqk, (long long)a->Dv);
    if (!aligned16(a->k_pe) || a->k_pe_bs % 8 || a->k_pe_rs % 8 || a->k_pe_rs < 64)
      return fail(PITH_ERR_MISALIGNED, "pith_attn_fwd: k_pe pointer / strides must keep 16-byte alignment (row stride >= 64)");
  }
  p.prev_o = a->prev_o; p.prev_f32 = a->prev_o_dtype == PITH_F32; p.prev_bs = a->prev_o_bs;
  p.acc_o = a->prev_o ? a->acc_o : nullptr; p.acc_bs = a->acc_o_bs;
  p.o_r0 = p.o_r1 = p.acc_r0 = p.acc_r1 = 0;
  if (a->prev_o) {
    if (a->prev_o_dtype != PITH_BF16 && a->prev_o_dtype != PITH_F32)
      return fail(PITH_ERR_BAD_DTYPE, "pith_attn_fwd: prev_o_dtype %d is not bf16/fp32", a->prev_o_dtype);
    if (a->causal || a->Dv != 128 || (a->Dqk != 128 && a->Dqk != 192))
      return fail(PITH_ERR_UNSUPPORTED, "pith_attn_fwd: merging with a running result needs a non-causal call with head dims "
                  "(128,128) or (192,128); run pith_attn_fwd and pith_combine instead");
    if (!aligned16(a->prev_o) || a->prev_o_bs % 8 || (a->acc_o && (!aligned16(a->acc_o) || a->acc_o_bs % 8)))
      return fail(PITH_ERR_MISALIGNED, "pith_attn_fwd: prev_o / acc_o pointers and batch strides must keep 16-byte alignment");
    const int64_t* ranges[2] = {a->o_rows, a->acc_o_rows};
    int* dst[2][2] = {{&p.o_r0, &p.o_r1}, {&p.acc_r0, &p.acc_r1}};
    for (int i = 0; i < 2; ++i) {
      int64_t r0 = ranges[i][0], r1 = ranges[i][1];
      if (r0 == 0 && r1 == 0) r1 = a->Sq;
      if (r0 < 0 || r1 < r0 || r1 > a->Sq || r0 % 32 || (r1 % 32 && r1 != a->Sq))
        return fail(PITH_ERR_BAD_SHAPE, "pith_attn_fwd: %s = [%lld, %lld) must lie within the %lld query rows on multiples of 32",
                    i ? "acc_o_rows" : "o_rows", (long long)ranges[i][0], (long long)ranges[i][1], (long long)a->Sq);
      *dst[i][0] = (int)r0;
      *dst[i][1] = (int)r1;
    }
  }
  hipStream_t st = (hipStream_t)stream;
  begin_launch();
  if ((a->Dqk == 128 || a->Dqk == 192) && a->Dv == 128) {
    launch_fwd_direct(p, (int)a->Dqk, a->causal != 0, prefer_half_rows(a->Sq, a->Hq, a->B, a->causal != 0), st);
  } else if (a->Dqk == 64 && a->Dv == 64) {
    if (few_workgroups(a->Sq, a->Hq, a->B)) launch_fwd<64, 64, 1, 4>(p, a, st);
    else launch_fwd<64, 64, 1, 8>(p, a, st);
  }
  else
    return fail(PITH_ERR_UNSUPPORTED, "pith_attn_fwd: head dims (Dqk=%lld, Dv=%lld) not in {(64,64),(128,128),(192,128)}",
                (long long)a->Dqk, (long long)a->Dv);
  return check_launch("pith_attn_fwd");
}
