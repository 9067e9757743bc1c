// Declarations shared by the forward kernels.
#pragma once

#include "attn_tiles.h"

namespace pith {

constexpr int kFwdBlockN = 64;            // keys per LDS tile
constexpr float kRescaleThreshold = 8.f;  // log2 units, see attn_fwd.hip

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
};

// Forward for head dims (128, 128) and (192, 128) with tiles loaded global -> LDS directly:
// attn_fwd_direct.hip. dqk = 128 or 192; half = workgroups of 128 query rows whose wave pairs split
// the keys of every tile (see there) instead of 256-row workgroups.
void launch_fwd_direct(const FwdParams& p, int dqk, bool causal, bool half, hipStream_t stream);

}  // namespace pith
