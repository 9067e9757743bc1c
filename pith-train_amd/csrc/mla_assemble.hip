// Attention prologue of the MLA layer: rotary embedding of the rope parts of q and of the shared
// k_pe, and assembly of the three tensors the attention call takes, in one pass; and its backward.
//
// Follows pithtrain/models/deepseek_v2_lite.py:446-454,462 (apply_rotary_pos_emb :173-187,
// rotate_half :165-169):
//     q = [q_nope | q_pe] per head, kv = [k_nope | value] per head, k_pe shared by all heads
//     pe'  = de-interleave(pe):  pe'[j] = pe[2j], pe'[Dr/2 + j] = pe[2j+1]
//     rot  = pe' * cos[pos] + rotate_half(pe') * sin[pos]
//     query_states = [q_nope | rot(q_pe)],  key_states = [k_nope | rot(k_pe) for every head],
//     value_states = value (made contiguous)
// The reference does this with two rotary expressions in eager bf16, four strided slice copies
// into new tensors and a .contiguous(); here every output byte is written once by one kernel and
// the rotation is evaluated in fp32 with a single rounding.
//
// HBM-bound data movement. One thread produces 16-byte pieces of the output tensors: it decodes a
// piece index into (tensor, head, piece), loads what the piece needs (a straight 16-byte copy,
// or two input pieces plus cos/sin for a rotated piece) and stores it; consecutive threads work
// on consecutive pieces, so the accesses of a wavefront are contiguous runs.
#include "pith_common.h"

namespace pith {
namespace {

constexpr int kThreads = 256;

struct AssembleParams {
  const __bf16* q;
  const __bf16* kv;
  const __bf16* k_pe;
  const __bf16* cos;
  const __bf16* sin;
  const int64_t* pos;
  __bf16* q_out;  // forward outputs / backward: dq, dkv, dk_pe
  __bf16* k_out;
  __bf16* v_out;
  const __bf16* dq_out;  // backward inputs
  const __bf16* dk_out;
  const __bf16* dv_out;
  int64_t S, P;
  int H, Dn, Dr, Dv;
  int64_t q_bs, kv_bs, k_pe_bs, k_pe_rs, pos_bs;
};

__device__ __forceinline__ float lo_of(uint32_t w) { return bf16lo_to_f32(w); }
__device__ __forceinline__ float hi_of(uint32_t w) { return bf16hi_to_f32(w); }

__device__ __forceinline__ int64_t table_row(const AssembleParams& p, int b, int64_t s) {
  int64_t pos = p.pos ? p.pos[b * p.pos_bs + s] : s;
  // positions outside the table would be an indexing error in the reference; clamp instead of faulting
  pos = pos < 0 ? 0 : (pos >= p.P ? p.P - 1 : pos);
  return pos * p.Dr;
}

// Rotated output piece `piece` (0 .. Dr/8-1) of one rope vector `src` (Dr interleaved elements).
// Pieces of the first half hold pe'[j] cos[j] - pe'[Dr/2+j] sin[j], pieces of the second half
// pe'[Dr/2+j] cos[Dr/2+j] + pe'[j] sin[Dr/2+j], for the 8 values of j the piece covers; both need
// the interleaved input elements 2j, 2j+1, i.e. two consecutive input pieces.
__device__ __forceinline__ u32x4 rotated_piece(const __bf16* src, const __bf16* cos_row, const __bf16* sin_row, int piece,
                                               int half_pieces) {
  const bool upper = piece >= half_pieces;
  const int jp = upper ? piece - half_pieces : piece;  // which group of 8 pairs
  const u32x4 in0 = *reinterpret_cast<const u32x4*>(src + 16 * jp);
  const u32x4 in1 = *reinterpret_cast<const u32x4*>(src + 16 * jp + 8);
  const u32x4 c = *reinterpret_cast<const u32x4*>(cos_row + 8 * piece);
  const u32x4 s = *reinterpret_cast<const u32x4*>(sin_row + 8 * piece);
  float r[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const uint32_t pair = e < 4 ? in0[e] : in1[e - 4];  // (even, odd) = (pe'[j], pe'[Dr/2+j])
    const float even = lo_of(pair), odd = hi_of(pair);
    const float ce = (e & 1) ? hi_of(c[e >> 1]) : lo_of(c[e >> 1]);
    const float se = (e & 1) ? hi_of(s[e >> 1]) : lo_of(s[e >> 1]);
    r[e] = upper ? odd * ce + even * se : even * ce - odd * se;
  }
  u32x4 out;
#pragma unroll
  for (int e = 0; e < 4; ++e) out[e] = pack_bf16x2(r[2 * e], r[2 * e + 1]);
  return out;
}

__device__ __forceinline__ void store_piece(__bf16* dst, u32x4 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dst));
}

constexpr int kBatch = 4;  // copied pieces a thread has in flight

// Forward. A token's output consists of copied pieces (q_nope, k_nope, value: one 16-byte load
// and store each, issued kBatch loads at a time) and rotated pieces (the rope parts of q_out and,
// identical for every head, of k_out).
__global__ __launch_bounds__(kThreads) void mla_assemble_fwd_kernel(AssembleParams p) {
  const int b = blockIdx.y;
  const int64_t s = blockIdx.x;
  const int qk = p.Dn + p.Dr, kvw = p.Dn + p.Dv;
  const int n8 = p.Dn >> 3, r8 = p.Dr >> 3, v8 = p.Dv >> 3;
  const int64_t row = table_row(p, b, s);
  const __bf16* q = p.q + b * p.q_bs + s * p.H * (int64_t)qk;
  const __bf16* kv = p.kv + b * p.kv_bs + s * p.H * (int64_t)kvw;
  const __bf16* k_pe = p.k_pe + b * p.k_pe_bs + s * p.k_pe_rs;
  const int64_t tok = (int64_t)b * p.S + s;
  __bf16* q_out = p.q_out + tok * p.H * qk;
  __bf16* k_out = p.k_out + tok * p.H * qk;
  __bf16* v_out = p.v_out + tok * p.H * p.Dv;

  // copied pieces, in order: q_nope [H][Dn/8], k_nope [H][Dn/8], value [H][Dv/8]
  const int n_nope = p.H * n8, n_copy = 2 * n_nope + p.H * v8;
  for (int i0 = threadIdx.x; i0 < n_copy; i0 += kThreads * kBatch) {
    u32x4 val[kBatch];
    __bf16* dst[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      int i = i0 + u * kThreads;
      if (i < n_copy) {
        const __bf16* src;
        if (i < 2 * n_nope) {
          const bool is_k = i >= n_nope;
          i -= is_k ? n_nope : 0;
          const int h = i / n8, piece = i - h * n8;
          src = (is_k ? kv + (int64_t)h * kvw : q + (int64_t)h * qk) + 8 * piece;
          dst[u] = (is_k ? k_out : q_out) + (int64_t)h * qk + 8 * piece;
        } else {
          i -= 2 * n_nope;
          const int h = i / v8, piece = i - h * v8;
          src = kv + (int64_t)h * kvw + p.Dn + 8 * piece;
          dst[u] = v_out + (int64_t)i * 8;
        }
        val[u] = *reinterpret_cast<const u32x4*>(src);
      }
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u)
      if (i0 + u * kThreads < n_copy) store_piece(dst[u], val[u]);
  }
  // rotated pieces, in order: q_out rope [H][Dr/8], k_out rope [H][Dr/8]
  const int n_rope = p.H * r8;
  for (int i = threadIdx.x; i < 2 * n_rope; i += kThreads) {
    const bool is_k = i >= n_rope;
    const int j = is_k ? i - n_rope : i;
    const int h = j / r8, piece = j - h * r8;
    const __bf16* src = is_k ? k_pe : q + (int64_t)h * qk + p.Dn;
    __bf16* dst = (is_k ? k_out : q_out) + (int64_t)h * qk + p.Dn + 8 * piece;
    store_piece(dst, rotated_piece(src, p.cos + row, p.sin + row, piece, r8 >> 1));
  }
}

// Gradient of the 8 interleaved input elements 8m .. 8m+7 of a rope vector (pairs j = 4m .. 4m+3)
// from the gradient g of its rotated form:  d even_j = g[j] cos[j] + g[Dr/2+j] sin[Dr/2+j],
// d odd_j = g[Dr/2+j] cos[Dr/2+j] - g[j] sin[j]. `g_lo`, `g_hi` are fp32 values of g at j and Dr/2+j.
__device__ __forceinline__ u32x4 unrotated_piece(const float* g_lo, const float* g_hi, const __bf16* cos_row,
                                                 const __bf16* sin_row, int m, int half) {
  const u32x2 c_lo = *reinterpret_cast<const u32x2*>(cos_row + 4 * m);
  const u32x2 c_hi = *reinterpret_cast<const u32x2*>(cos_row + half + 4 * m);
  const u32x2 s_lo = *reinterpret_cast<const u32x2*>(sin_row + 4 * m);
  const u32x2 s_hi = *reinterpret_cast<const u32x2*>(sin_row + half + 4 * m);
  u32x4 out;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float cl = (e & 1) ? hi_of(c_lo[e >> 1]) : lo_of(c_lo[e >> 1]);
    const float ch = (e & 1) ? hi_of(c_hi[e >> 1]) : lo_of(c_hi[e >> 1]);
    const float sl = (e & 1) ? hi_of(s_lo[e >> 1]) : lo_of(s_lo[e >> 1]);
    const float sh = (e & 1) ? hi_of(s_hi[e >> 1]) : lo_of(s_hi[e >> 1]);
    out[e] = pack_bf16x2(g_lo[e] * cl + g_hi[e] * sh, g_hi[e] * ch - g_lo[e] * sl);
  }
  return out;
}

__device__ __forceinline__ void load4(const __bf16* src, float* dst, bool add) {
  const u32x2 v = *reinterpret_cast<const u32x2*>(src);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float x = (e & 1) ? hi_of(v[e >> 1]) : lo_of(v[e >> 1]);
    dst[e] = add ? dst[e] + x : x;
  }
}

// Backward. dk_pe is a sum over all heads: one thread per (head, piece) loads its share of the rope
// gradient of key_states and leaves it in LDS (all those loads are in flight together), and after
// the block's other work Dr/8 threads add the heads in head order and apply the inverse rotation.
// In between: the copied pieces (dq nope from dq_out, dkv nope from dk_out, dkv value from
// dv_out), kBatch loads at a time, and the rope part of dq.
__global__ __launch_bounds__(kThreads) void mla_assemble_bwd_kernel(AssembleParams p) {
  extern __shared__ float rope_grad[];  // [H][Dr/8][8]: (g[4m..4m+3], g[Dr/2+4m..+3]) of every head
  const int b = blockIdx.y;
  const int64_t s = blockIdx.x;
  const int qk = p.Dn + p.Dr, kvw = p.Dn + p.Dv;
  const int n8 = p.Dn >> 3, r8 = p.Dr >> 3, v8 = p.Dv >> 3;
  const int half = p.Dr >> 1;
  const int64_t row = table_row(p, b, s);
  const int64_t tok = (int64_t)b * p.S + s;
  const __bf16* dq_out = p.dq_out + tok * p.H * qk;
  const __bf16* dk_out = p.dk_out + tok * p.H * qk;
  const __bf16* dv_out = p.dv_out + tok * p.H * p.Dv;
  __bf16* dq = p.q_out + tok * p.H * qk;
  __bf16* dkv = p.k_out + tok * p.H * kvw;
  __bf16* dk_pe = p.v_out + tok * p.Dr;
  const int n_rope = p.H * r8;

  for (int i = threadIdx.x; i < n_rope; i += kThreads) {
    const int h = i / r8, m = i - h * r8;
    float g[8];
    load4(dk_out + (int64_t)h * qk + p.Dn + 4 * m, g, false);
    load4(dk_out + (int64_t)h * qk + p.Dn + half + 4 * m, g + 4, false);
    *reinterpret_cast<f32x4*>(rope_grad + 8 * i) = f32x4{g[0], g[1], g[2], g[3]};
    *reinterpret_cast<f32x4*>(rope_grad + 8 * i + 4) = f32x4{g[4], g[5], g[6], g[7]};
  }

  const int n_nope = p.H * n8, n_copy = 2 * n_nope + p.H * v8;
  for (int i0 = threadIdx.x; i0 < n_copy; i0 += kThreads * kBatch) {
    u32x4 val[kBatch];
    __bf16* dst[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      int i = i0 + u * kThreads;
      if (i < n_copy) {
        const __bf16* src;
        if (i < 2 * n_nope) {
          const bool is_k = i >= n_nope;
          i -= is_k ? n_nope : 0;
          const int h = i / n8, piece = i - h * n8;
          src = (is_k ? dk_out : dq_out) + (int64_t)h * qk + 8 * piece;
          dst[u] = (is_k ? dkv + (int64_t)h * kvw : dq + (int64_t)h * qk) + 8 * piece;
        } else {
          i -= 2 * n_nope;
          const int h = i / v8, piece = i - h * v8;
          src = dv_out + (int64_t)i * 8;
          dst[u] = dkv + (int64_t)h * kvw + p.Dn + 8 * piece;
        }
        val[u] = *reinterpret_cast<const u32x4*>(src);
      }
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u)
      if (i0 + u * kThreads < n_copy) store_piece(dst[u], val[u]);
  }

  for (int i = threadIdx.x; i < n_rope; i += kThreads) {
    const int h = i / r8, m = i - h * r8;
    float g_lo[4], g_hi[4];
    load4(dq_out + (int64_t)h * qk + p.Dn + 4 * m, g_lo, false);
    load4(dq_out + (int64_t)h * qk + p.Dn + half + 4 * m, g_hi, false);
    store_piece(dq + (int64_t)h * qk + p.Dn + 8 * m, unrotated_piece(g_lo, g_hi, p.cos + row, p.sin + row, m, half));
  }

  __syncthreads();
  for (int m = threadIdx.x; m < r8; m += kThreads) {
    float g_lo[4] = {0.f, 0.f, 0.f, 0.f}, g_hi[4] = {0.f, 0.f, 0.f, 0.f};
    for (int h = 0; h < p.H; ++h) {
      const f32x4 lo = *reinterpret_cast<const f32x4*>(rope_grad + 8 * (h * r8 + m));
      const f32x4 hi = *reinterpret_cast<const f32x4*>(rope_grad + 8 * (h * r8 + m) + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        g_lo[e] += lo[e];
        g_hi[e] += hi[e];
      }
    }
    store_piece(dk_pe + 8 * m, unrotated_piece(g_lo, g_hi, p.cos + row, p.sin + row, m, half));
  }
}

int validate(const char* who, const pith_mla_assemble_args* a, bool backward) {
  if (!a) return fail(PITH_ERR_NULL_POINTER, "%s: args is NULL", who);
  if (!a->cos || !a->sin || !a->q_out || !a->k_out || !a->v_out)
    return fail(PITH_ERR_NULL_POINTER, "%s: NULL tensor pointer", who);
  if (!backward && (!a->q || !a->kv || !a->k_pe)) return fail(PITH_ERR_NULL_POINTER, "%s: NULL input pointer", who);
  if (backward && (!a->dq_out || !a->dk_out || !a->dv_out))
    return fail(PITH_ERR_NULL_POINTER, "%s: NULL gradient pointer", who);
  if (a->B <= 0 || a->S <= 0 || a->H <= 0 || a->Dn <= 0 || a->Dr <= 0 || a->Dv <= 0 || a->P <= 0)
    return fail(PITH_ERR_BAD_SHAPE, "%s: B=%lld S=%lld H=%lld Dn=%lld Dr=%lld Dv=%lld P=%lld must all be positive", who,
                (long long)a->B, (long long)a->S, (long long)a->H, (long long)a->Dn, (long long)a->Dr, (long long)a->Dv,
                (long long)a->P);
  if (a->Dn % 8 || a->Dv % 8 || a->Dr % 16)
    return fail(PITH_ERR_UNSUPPORTED, "%s: Dn=%lld and Dv=%lld must be multiples of 8, Dr=%lld of 16", who,
                (long long)a->Dn, (long long)a->Dv, (long long)a->Dr);
  if (a->B > 65535 || a->S > 2147483647LL || a->H * (2 * (a->Dn + a->Dr) + a->Dn + a->Dv) / 8 + a->Dr > (1 << 24))
    return fail(PITH_ERR_UNSUPPORTED, "%s: B=%lld > 65535, S > 2^31-1 or too many heads", who, (long long)a->B);
  uintptr_t bits = reinterpret_cast<uintptr_t>(a->cos) | reinterpret_cast<uintptr_t>(a->sin) |
                   reinterpret_cast<uintptr_t>(a->q_out) | reinterpret_cast<uintptr_t>(a->k_out) |
                   reinterpret_cast<uintptr_t>(a->v_out);
  if (backward)
    bits |= reinterpret_cast<uintptr_t>(a->dq_out) | reinterpret_cast<uintptr_t>(a->dk_out) |
            reinterpret_cast<uintptr_t>(a->dv_out);
  else
    bits |= reinterpret_cast<uintptr_t>(a->q) | reinterpret_cast<uintptr_t>(a->kv) | reinterpret_cast<uintptr_t>(a->k_pe);
  if (bits % 16 || (!backward && (a->q_bs % 8 || a->kv_bs % 8 || a->k_pe_bs % 8 || a->k_pe_rs % 8)))
    return fail(PITH_ERR_MISALIGNED, "%s: pointers and strides must keep 16-byte alignment", who);
  if (a->position_ids && reinterpret_cast<uintptr_t>(a->position_ids) % 8)
    return fail(PITH_ERR_MISALIGNED, "%s: position_ids must be 8-byte aligned", who);
  if (!backward) {
    if (a->B > 1 && (a->q_bs < a->S * a->H * (a->Dn + a->Dr) || a->kv_bs < a->S * a->H * (a->Dn + a->Dv)))
      return fail(PITH_ERR_BAD_SHAPE, "%s: a batch stride is smaller than its tensor", who);
    if (a->k_pe_rs < a->Dr) return fail(PITH_ERR_BAD_SHAPE, "%s: k_pe row stride %lld < Dr", who, (long long)a->k_pe_rs);
  }
  return PITH_OK;
}

AssembleParams make_params(const pith_mla_assemble_args* a) {
  AssembleParams p;
  p.q = (const __bf16*)a->q; p.kv = (const __bf16*)a->kv; p.k_pe = (const __bf16*)a->k_pe;
  p.cos = (const __bf16*)a->cos; p.sin = (const __bf16*)a->sin; p.pos = a->position_ids;
  p.q_out = (__bf16*)a->q_out; p.k_out = (__bf16*)a->k_out; p.v_out = (__bf16*)a->v_out;
  p.dq_out = (const __bf16*)a->dq_out; p.dk_out = (const __bf16*)a->dk_out; p.dv_out = (const __bf16*)a->dv_out;
  p.S = a->S; p.P = a->P; p.H = (int)a->H; p.Dn = (int)a->Dn; p.Dr = (int)a->Dr; p.Dv = (int)a->Dv;
  p.q_bs = a->q_bs; p.kv_bs = a->kv_bs; p.k_pe_bs = a->k_pe_bs; p.k_pe_rs = a->k_pe_rs; p.pos_bs = a->pos_bs;
  return p;
}

}  // namespace
}  // namespace pith

using namespace pith;

extern "C" int pith_mla_assemble_fwd(const pith_mla_assemble_args* a, pith_stream_t stream) {
  if (const int rc = validate("pith_mla_assemble_fwd", a, false)) return rc;
  const AssembleParams p = make_params(a);
  begin_launch();
  hipLaunchKernelGGL(mla_assemble_fwd_kernel, dim3((unsigned)a->S, (unsigned)a->B), dim3(kThreads), 0, (hipStream_t)stream, p);
  return check_launch("pith_mla_assemble_fwd");
}

extern "C" int pith_mla_assemble_bwd(const pith_mla_assemble_args* a, pith_stream_t stream) {
  if (const int rc = validate("pith_mla_assemble_bwd", a, true)) return rc;
  const AssembleParams p = make_params(a);
  const size_t lds = (size_t)a->H * a->Dr * sizeof(float);
  if (lds > 64 * 1024)
    return fail(PITH_ERR_UNSUPPORTED, "pith_mla_assemble_bwd: H*Dr=%lld exceeds 16384", (long long)(a->H * a->Dr));
  begin_launch();
  hipLaunchKernelGGL(mla_assemble_bwd_kernel, dim3((unsigned)a->S, (unsigned)a->B), dim3(kThreads), lds, (hipStream_t)stream, p);
  return check_launch("pith_mla_assemble_bwd");
}
