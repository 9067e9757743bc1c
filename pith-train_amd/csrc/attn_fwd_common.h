// Declarations shared by the forward kernels.
#pragma once

#include "attn_tiles.h"

namespace pith {

constexpr int kFwdBlockN = 64;            // keys per LDS tile
constexpr float kRescaleThreshold = 8.f;  // log2 units, see attn_fwd.hip
constexpr float kRescaleLimit = 256.f;    // = 2^kRescaleThreshold: the same bound on a P value, tested on row sums (attn_fwd_direct.hip)

struct FwdParams {
  const __bf16* q;
  const __bf16* k;
  const __bf16* v;
  __bf16* o;
  float* lse;
  int Sq, Skv, Hq, Hkv, group;  // group = Hq / Hkv
  int B, m_tiles;
  int64_t q_bs, k_bs, v_bs, o_bs, lse_bs, lse_hs;
  float kappa;  // scale * log2(e)
  // keys in two parts (k_pe != nullptr): k holds the first 128 features per head, k_pe the last 64,
  // one vector per position shared by all heads (batch / row strides in elements)
  const __bf16* k_pe;
  int64_t k_pe_bs, k_pe_rs;
  // merge with the running result of the rows (prev_o != nullptr; non-causal direct-load kernels only): prev_o is
  // bf16 or fp32 (prev_f32), the merged result goes to o (bf16, may be null then) and / or acc_o (fp32, may be null);
  // lse holds the running LSE on entry and the merged LSE on return
  const void* prev_o;
  int prev_f32;
  int64_t prev_bs;
  float* acc_o;
  int64_t acc_bs;
  int o_r0, o_r1, acc_r0, acc_r1;  // query rows [r0, r1) that receive o / acc_o when merging (multiples of 32, or Sq)
};

// Forward for head dims (128, 128) and (192, 128) with tiles loaded global -> LDS directly:
// attn_fwd_direct.hip. dqk = 128 or 192; half = workgroups of 128 query rows whose wave pairs split
// the keys of every tile (see there) instead of 256-row workgroups.
void launch_fwd_direct(const FwdParams& p, int dqk, bool causal, bool half, hipStream_t stream);

}  // namespace pith
