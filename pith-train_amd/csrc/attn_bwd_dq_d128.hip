// Query-gradient kernel for head dims (128, 128) on gfx950. Same function and numerics as the
// general kernel in attn_bwd_dq.hip (pithtrain/operators/mla/triton.py:205-266, :392-441:
// P = exp2(kappa*s - lse2) in fp32, masked entries 0, dS = P*(dP - delta)*scale rounded to bf16,
// fp32 accumulation of dQ += dS K), same work split: a workgroup of 8 wavefronts owns 256 query
// rows of one (batch, head), a wavefront 32 of them, stationary in registers as B operands (Q^T
// and dO^T fragments, per-lane lse and delta); K/V tiles of 64 keys stream through LDS.
//
// What differs from the general kernel:
//   - K/V tiles go global -> LDS directly (global_load_lds) into packed swizzled tiles, requested
//     one interval ahead (ring of 4 K tiles, 2 V tiles);
//   - the gradient product runs ONE TILE BEHIND: interval i issues, as one block of 48 MFMAs,
//     dQ^T += K(i-1)^T dS(i-1)^T, S(i)^T = K(i) Q^T and dP(i)^T = V(i) dO^T, with the LDS fragment
//     reads pinned kAhead products ahead of their use, and then turns S(i), dP(i) into dS(i);
//   - the factor `scale` of dS is applied once to the accumulated dQ (dS / scale is what gets
//     rounded to bf16: the same relative rounding);
//   - first and last interval are peeled, the loop body in between is straight-line code.
#include "attn_bwd_common.h"

namespace pith {
namespace {

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kBM = kWaves * 32;  // query rows per workgroup
constexpr int kBN = 64;           // keys per tile
constexpr int kD = 128;
constexpr int kKSlots = 4;        // K tiles i-1, i in use, i+1 landing; a power of two
constexpr int kVSlots = 2;        // V tiles i in use, i+1 landing
constexpr int kAhead = 4;         // fragment reads run this many products ahead in the matrix block
constexpr int kTile = kBN * kRowBytes128;

template <bool CAUSAL, typename OutT>
__global__ __launch_bounds__(kThreads) void attn_bwd_dq_d128_kernel(BwdParams p) {
  constexpr int KS = kD / 16, DB = kD / 32;
  // the tile rings; the epilogue reuses the memory to turn the result tile (one area per wave)
  constexpr int kRings = (kKSlots + kVSlots) * kTile, kTurn = kThreads / 64 * kRowsViaLdsBytes<DB>;
  __shared__ __attribute__((aligned(1024))) char smem[kRings > kTurn ? kRings : kTurn];
  char* const kbuf = smem;
  char* const vbuf = smem + kKSlots * kTile;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, g = lane >> 5;
  int m_tile, h, b;
  decode_block(blockIdx.x, p.Hq, p.B, p.tiles, p.group, m_tile, h, b);
  const int hk = h / p.group;
  const int m0 = m_tile * kBM;
  const int q_wave0 = m0 + wave * 32;
  const int qrow = q_wave0 + c;

  const int64_t q_row_stride = (int64_t)p.HqT * kD;
  const int kv_row_bytes = p.HkvT * kD * 2;
  const char* kh = reinterpret_cast<const char*>(p.k + b * p.k_bs + (int64_t)hk * kD);
  const char* vh = reinterpret_cast<const char*>(p.v + b * p.v_bs + (int64_t)hk * kD);

  const int n_tiles_all = (p.Skv + kBN - 1) / kBN;
  int n_tiles_wg = n_tiles_all, n_tiles_wave = n_tiles_all;
  if (CAUSAL) {
    n_tiles_wg = min(n_tiles_all, (m0 + kBM - 1) / kBN + 1);
    n_tiles_wave = min(n_tiles_all, (q_wave0 + 31) / kBN + 1);
  }

  DirectTile128<kBN, kThreads> mover;
  mover.init(kv_row_bytes, wave, lane);
  auto request = [&](int t) __attribute__((always_inline)) {
    mover.issue(kh + (int64_t)t * kBN * kv_row_bytes, p.Skv - t * kBN, kbuf + (t & (kKSlots - 1)) * kTile, wave, lane);
    mover.issue(vh + (int64_t)t * kBN * kv_row_bytes, p.Skv - t * kBN, vbuf + (t & (kVSlots - 1)) * kTile, wave, lane);
  };
  request(0);

  // stationary side: Q^T and dO^T fragments (B operands), lse and delta of this lane's query row
  bf16x8 qf[KS], dof[KS];
  float lse_q, delta_q;
  {
    const int row = qrow < p.Sq ? qrow : p.Sq - 1;
    const __bf16* src = p.q + b * p.q_bs + (int64_t)h * kD + row * q_row_stride + g * 8;
    const __bf16* dsrc = p.dout + b * p.dout_bs + (int64_t)h * kD + row * q_row_stride + g * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(src + ks * 16);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) dof[ks] = *reinterpret_cast<const bf16x8*>(dsrc + ks * 16);
    lse_q = (p.lse + b * p.lse_bs + (int64_t)h * p.lse_hs)[row];
    delta_q = (p.delta + b * p.lse_bs + (int64_t)h * p.lse_hs)[row];
  }

  // per-lane read offsets inside a tile. The swizzle is an XOR on the 16-byte piece index, so the
  // offsets of the other contraction steps / feature blocks are the first one XOR a constant; only
  // the first ones live in registers (the kernel sits at the 256-register limit, and a spilled
  // value is reloaded from scratch with a wait that also waits for the tile loads in flight):
  //   straight fragment of tile row c, contraction step ks (+ 32 rows: + 8192 bytes):  s_base ^ (ks << 5)
  //   transposing reads of feature block o, lower / upper 8 rows (+ 16 rows: + 4096 bytes):  t_base[hh] ^ (o << 6)
  int s_base = straight_offset128(c, g);
  int t_base[2] = {transposed_offset128(0, 0, 0, lane), transposed_offset128(0, 1, 0, lane)};
  // called once per interval: the bases are handed to the compiler as new values, or it would
  // compute every derived offset once and keep all of them in registers across the loop
  auto refresh_offsets = [&]() __attribute__((always_inline)) { asm volatile("" : "+v"(s_base), "+v"(t_base[0]), "+v"(t_base[1])); };
  auto s_off = [&](int ks) __attribute__((always_inline)) { return s_base ^ (ks << 5); };
  auto t_off = [&](int o, int hh) __attribute__((always_inline)) { return t_base[hh] ^ (o << 6); };

  f32x16 acc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;

  f32x16 s[2], dp[2];  // S^T and dP^T of one key tile: [64 keys] x [32 queries] as two 32 x 32 tiles
  bf16x8 dsf[4];       // dS^T / scale of one key tile as B operand, one fragment per 16 keys

  // ---- S^T = K Q^T and dP^T = V dO^T of one tile
  auto scores = [&](const char* ktile, const char* vtile) __attribute__((always_inline)) {
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        s[nb][v] = 0.f;
        dp[nb][v] = 0.f;
      }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(ktile + s_off(ks) + nb * 32 * kRowBytes128);
        s[nb] = mfma32(a, qf[ks], s[nb]);
      }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(vtile + s_off(ks) + nb * 32 * kRowBytes128);
        dp[nb] = mfma32(a, dof[ks], dp[nb]);
      }
  };
  // ---- dQ^T += K^T dS^T of one tile
  auto accumulate = [&](const char* ktile) __attribute__((always_inline)) {
    bf16x8 at[4][DB];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int o = 0; o < DB; ++o) {
        const char* base = ktile + j * 16 * kRowBytes128;
        at[j][o] = lds_read_transposed_at(base + t_off(o, 0), base + t_off(o, 1));
      }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int o = 0; o < DB; ++o) acc[o] = mfma32(at[j][o], dsf[j], acc[o]);
    __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);
#pragma unroll
    for (int m = 0; m < 4 * DB - kAhead; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 0);
  };
  // ---- half nb (32 keys) of tile t: s[nb], dp[nb] -> dS / scale as bf16 fragments dsf[2*nb], dsf[2*nb+1]
  auto make_ds_half_masked = [&](int t, int nb) __attribute__((always_inline)) {
    const int n0 = t * kBN;
#pragma unroll
    for (int v = 0; v < 16; ++v) s[nb][v] = __builtin_amdgcn_exp2f(s[nb][v] * p.kappa - lse_q);
    if ((CAUSAL && (n0 + kBN - 1 > q_wave0)) || (n0 + kBN > p.Skv)) {
      // tile crossing the diagonal of a causal chunk, or a ragged last tile (wave-uniform branch)
      const int limit = CAUSAL ? min(qrow, p.Skv - 1) : p.Skv - 1;  // last visible key
#pragma unroll
      for (int v = 0; v < 16; ++v)
        if (n0 + nb * 32 + acc_row(v, g) > limit) s[nb][v] = 0.f;
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) s[nb][v] *= dp[nb][v] - delta_q;
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
      dsf[2 * nb + jj] = to_bf16x8(s[nb][8 * jj], s[nb][8 * jj + 1], s[nb][8 * jj + 2], s[nb][8 * jj + 3],
                                   s[nb][8 * jj + 4], s[nb][8 * jj + 5], s[nb][8 * jj + 6], s[nb][8 * jj + 7]);
  };
  // ---- S^T and dP^T of one half (32 keys) of a tile, with the dS arithmetic of the unmasked
  // half `other` of a tile already scored (-1: none) woven in: after every pair of MFMAs come the
  // exp / multiply / convert of two elements, so that the matrix pipe keeps running while this
  // wave converts scores. The order is pinned with scheduling barriers; the LDS fragment reads
  // run kAhead / 2 contraction steps ahead.
  auto scores_half = [&](const char* ktile, const char* vtile, int nb, int other) __attribute__((always_inline)) {
    constexpr int kPre = kAhead / 2;
    bf16x8 ak[KS], av[KS];
    uint32_t w[8];
#pragma unroll
    for (int ks = 0; ks < kPre; ++ks) {
      ak[ks] = *reinterpret_cast<const bf16x8*>(ktile + s_off(ks) + nb * 32 * kRowBytes128);
      av[ks] = *reinterpret_cast<const bf16x8*>(vtile + s_off(ks) + nb * 32 * kRowBytes128);
    }
    f32x16 sn, dn;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      sn[v] = 0.f;
      dn[v] = 0.f;
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks + kPre < KS) {
        ak[ks + kPre] = *reinterpret_cast<const bf16x8*>(ktile + s_off(ks + kPre) + nb * 32 * kRowBytes128);
        av[ks + kPre] = *reinterpret_cast<const bf16x8*>(vtile + s_off(ks + kPre) + nb * 32 * kRowBytes128);
      }
      sn = mfma32(ak[ks], qf[ks], sn);
      dn = mfma32(av[ks], dof[ks], dn);
      // empty volatile statements pin the program order: the optimiser would otherwise sink the
      // arithmetic below past all MFMAs
      asm volatile("" : "+v"(sn), "+v"(dn));
      if (other >= 0) {
        const float e0 = __builtin_amdgcn_exp2f(s[other][2 * ks] * p.kappa - lse_q) * (dp[other][2 * ks] - delta_q);
        const float e1 = __builtin_amdgcn_exp2f(s[other][2 * ks + 1] * p.kappa - lse_q) * (dp[other][2 * ks + 1] - delta_q);
        w[ks] = pack_bf16x2(e0, e1);
        asm volatile("" : "+v"(w[ks]));
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (other >= 0) {
      const u32x4 lo = {w[0], w[1], w[2], w[3]}, hi = {w[4], w[5], w[6], w[7]};
      dsf[2 * other] = __builtin_bit_cast(bf16x8, lo);
      dsf[2 * other + 1] = __builtin_bit_cast(bf16x8, hi);
    }
    s[nb] = sn;
    dp[nb] = dn;
  };

  __builtin_amdgcn_s_waitcnt(0x0F70);  // tile 0 and the stationary fragments
  __syncthreads();

  // Interval i = 0 .. n_tiles_wg touches tiles i-1 and i. A wave has work up to interval
  // n_tiles_wave; every wave passes all barriers. Between intervals a wave carries S, dP of the
  // upper half (keys 32..63) of the last tile and the dS fragments of its lower half: the vector
  // arithmetic of a half tile is issued between the MFMAs that produce the next half, so that
  // the matrix pipe does not idle while a wave converts scores.
  auto end_interval = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // the tiles requested in this interval have landed
    __syncthreads();
  };
  auto kslot = [&](int t) __attribute__((always_inline)) { return kbuf + (t & (kKSlots - 1)) * kTile; };
  auto vslot = [&](int t) __attribute__((always_inline)) { return vbuf + (t & (kVSlots - 1)) * kTile; };
  // tiles [0, first_masked) need no mask for this wave
  int first_masked = p.Skv / kBN;
  if (CAUSAL) first_masked = min(first_masked, q_wave0 >= kBN - 1 ? (q_wave0 - (kBN - 1)) / kBN + 1 : 0);
  const int n_fast = min(n_tiles_wave, first_masked);

  // interval 0 (every wave has at least one tile)
  scores(kslot(0), vslot(0));
  if (1 < n_tiles_wg) request(1);
  make_ds_half_masked(0, 0);
  end_interval();
  int i = 1;
  for (; i < n_fast; ++i) {  // tiles i-1 and i unmasked
    refresh_offsets();
    // tile i+1 is requested first: its slots were last read in interval i-1, and the load then
    // has the whole interval to land
    if (i + 1 < n_tiles_wg) request(i + 1);
    scores_half(kslot(i), vslot(i), 0, 1);
    __builtin_amdgcn_sched_barrier(0);
    accumulate(kslot(i - 1));
    __builtin_amdgcn_sched_barrier(0);
    scores_half(kslot(i), vslot(i), 1, 0);
    __builtin_amdgcn_sched_barrier(0);
    end_interval();
  }
  for (; i < n_tiles_wave; ++i) {  // near the diagonal / ragged end: plain order, masks applied
    refresh_offsets();
    if (i + 1 < n_tiles_wg) request(i + 1);
    make_ds_half_masked(i - 1, 1);
    accumulate(kslot(i - 1));
    scores(kslot(i), vslot(i));
    make_ds_half_masked(i, 0);
    end_interval();
  }
  // interval n_tiles_wave: the last gradient product of this wave
  make_ds_half_masked(i - 1, 1);
  accumulate(kslot(i - 1));
  // other waves of the workgroup may still have tiles to visit: keep moving them and keep in step
  for (; i < n_tiles_wg; ++i) {
    if (i + 1 < n_tiles_wg) request(i + 1);
    end_interval();
  }

  // dQ^T sits in the accumulators (a lane owns one query row): turned through LDS so that the epilogue
  // reads and writes whole rows. A wave reads its last K tile after the last barrier of the loops above,
  // hence one more barrier before the rings are overwritten.
  __syncthreads();
  OutT* dqh = reinterpret_cast<OutT*>(p.dq) + b * p.dq_bs + (int64_t)h * kD;
  __bf16* fin = nullptr;  // rows whose gradient is complete with this call go out as bf16
  if (p.dq_final != nullptr && q_wave0 >= p.final_r0 && q_wave0 < p.final_r1)
    fin = p.dq_final + b * p.dq_final_bs + (int64_t)h * kD + q_wave0 * q_row_stride;
  store_rows32_via_lds<OutT, DB>(smem + wave * kRowsViaLdsBytes<DB>, dqh + q_wave0 * q_row_stride, q_row_stride, p.Sq - q_wave0,
                                 acc, p.scale, p.accumulate != 0, lane, fin);
}

}  // namespace

void launch_dq_d128(const BwdParams& p, bool causal, bool f32_out, hipStream_t st) {
  const dim3 grid((unsigned)(p.tiles * p.Hq * p.B)), block(kThreads);
  if (causal) {
    if (f32_out) hipLaunchKernelGGL((attn_bwd_dq_d128_kernel<true, float>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((attn_bwd_dq_d128_kernel<true, __bf16>), grid, block, 0, st, p);
  } else {
    if (f32_out) hipLaunchKernelGGL((attn_bwd_dq_d128_kernel<false, float>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((attn_bwd_dq_d128_kernel<false, __bf16>), grid, block, 0, st, p);
  }
}

}  // namespace pith
