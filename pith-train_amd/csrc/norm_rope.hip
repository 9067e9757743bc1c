// Attention prologue of the GQA layer: per-head RMSNorm of the projected q / k followed by the
// rotary position embedding, in one pass over the tensor, and its backward.
//
// Follows pithtrain/models/qwen3_30b_a3b.py:417-421 (q_norm / k_norm, then apply_rotary_pos_emb
// :107-136 with rotate_half :100-104):
//     y   = x * rsqrt(mean_d(x^2) + eps) * w                     (per [b, s, h] row of D elements)
//     out = y * cos + rotate_half(y) * sin,   rotate_half(y) = cat(-y[D/2:], y[:D/2])
// The reference evaluates this with a dozen eager bf16 kernels (each rounding to bf16); here the
// row is read once, everything is computed in fp32 and the result rounded to bf16 once.
//
// Both kernels are HBM-bound: x (and dout) are read once and out (dx) written once, 2 bytes per
// element each; cos/sin are read once per token and kept in registers for all heads of the token.
//
// Work split. A row of D elements is owned by D/8 consecutive lanes; a lane holds elements
// [4l, 4l+4) of the first half and the same four of the second half, i.e. both members of the
// four rotation pairs it computes, so the rotation needs no exchange between lanes. A block of
// 256 threads has 2048/D row slots, arranged as tile_s tokens x hg head groups; a slot walks the
// heads g, g + hg, g + 2 hg, ... of its token. Adjacent slots take adjacent heads, so the rows a
// wavefront touches in one instruction are contiguous in memory.
#include "pith_common.h"

namespace pith {
namespace {

constexpr int kThreads = 256;
constexpr int kBatch = 4;  // rows a slot has in flight (forward)
constexpr int kBwdBatch = 2;  // the same in the backward, which holds two tensors per row

struct Quad {  // four consecutive bf16
  u32x2 raw;
  __device__ __forceinline__ void load(const __bf16* p) { raw = *reinterpret_cast<const u32x2*>(p); }
  __device__ __forceinline__ void store(__bf16* p) const { __builtin_nontemporal_store(raw, reinterpret_cast<u32x2*>(p)); }
  __device__ __forceinline__ float get(int i) const {
    const uint32_t w = raw[i >> 1];
    return (i & 1) ? bf16hi_to_f32(w) : bf16lo_to_f32(w);
  }
  __device__ __forceinline__ void set(const float* v) {
    raw[0] = pack_bf16x2(v[0], v[1]);
    raw[1] = pack_bf16x2(v[2], v[3]);
  }
};

struct NormRopeParams {
  const __bf16* x;
  const void* w;  // [D] bf16 or fp32; unused without NORM
  const __bf16* cos;
  const __bf16* sin;
  const __bf16* dout;  // backward only
  __bf16* out;         // forward: out; backward: dx
  float* partial;      // backward with NORM: [blocks][D] partial sums of dw
  int64_t S;
  int H, D;
  int lanes;   // D / 8, a power of two <= 64
  int hg;      // head groups per token, a power of two <= 2048 / D
  int tile_s;  // tokens per block = (2048 / D) / hg
  int n_tiles;  // ceil(S / tile_s)
  int grid_x;  // blocks of this tensor along x (backward: blocks stride over the tiles)
  int64_t x_bs, out_bs, dout_bs, cs_bs;
  float eps, inv_d;
  int w_f32;
};

// One launch serves up to two tensors (q and k of a layer): blocks [0, blocks0) along x work on
// t[0], the rest on t[1].
struct PairParams {
  NormRopeParams t[2];
  int blocks0;
};

__device__ __forceinline__ float row_sum(float v, int lanes) {
  for (int off = lanes >> 1; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

__device__ __forceinline__ void load_gain(const NormRopeParams& p, int l, float* w_lo, float* w_hi) {
  const int half = p.D >> 1;
  if (p.w_f32) {
    const float* w = reinterpret_cast<const float*>(p.w);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      w_lo[j] = w[4 * l + j];
      w_hi[j] = w[half + 4 * l + j];
    }
  } else {
    Quad a, b;
    a.load(reinterpret_cast<const __bf16*>(p.w) + 4 * l);
    b.load(reinterpret_cast<const __bf16*>(p.w) + half + 4 * l);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      w_lo[j] = a.get(j);
      w_hi[j] = b.get(j);
    }
  }
}

template <bool NORM>
__global__ __launch_bounds__(kThreads) void norm_rope_fwd_kernel(PairParams pp) {
  const int which = (int)blockIdx.x >= pp.blocks0;
  const NormRopeParams& p = pp.t[which];
  const int bx = blockIdx.x - (which ? pp.blocks0 : 0);
  const int l = threadIdx.x % p.lanes;
  const int slot = threadIdx.x / p.lanes;
  const int g = slot % p.hg;
  const int b = blockIdx.y;
  const int64_t s = (int64_t)bx * p.tile_s + slot / p.hg;
  if (s >= p.S) return;  // no block-wide synchronisation below
  const int half = p.D >> 1;

  float w_lo[4], w_hi[4];
  if (NORM) load_gain(p, l, w_lo, w_hi);

  const int64_t cs = b * p.cs_bs + s * p.D + 4 * l;
  Quad c_lo, c_hi, s_lo, s_hi;
  c_lo.load(p.cos + cs);
  c_hi.load(p.cos + cs + half);
  s_lo.load(p.sin + cs);
  s_hi.load(p.sin + cs + half);

  const int64_t row0 = s * p.H * (int64_t)p.D + 4 * l;
  const __bf16* x = p.x + b * p.x_bs + row0;
  __bf16* out = p.out + b * p.out_bs + row0;

  for (int h0 = g; h0 < p.H; h0 += kBatch * p.hg) {
    Quad lo[kBatch], hi[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int h = h0 + u * p.hg;
      if (h < p.H) {
        lo[u].load(x + (int64_t)h * p.D);
        hi[u].load(x + (int64_t)h * p.D + half);
      }
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int h = h0 + u * p.hg;
      if (h >= p.H) break;  // the lanes of a row leave together: lanes of a row share h
      float a[4], c[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        a[j] = lo[u].get(j);
        c[j] = hi[u].get(j);
      }
      if (NORM) {
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) ss += a[j] * a[j] + c[j] * c[j];
        const float r = rsqrtf(row_sum(ss, p.lanes) * p.inv_d + p.eps);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          a[j] *= r * w_lo[j];
          c[j] *= r * w_hi[j];
        }
      }
      float o_lo[4], o_hi[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        o_lo[j] = a[j] * c_lo.get(j) - c[j] * s_lo.get(j);
        o_hi[j] = c[j] * c_hi.get(j) + a[j] * s_hi.get(j);
      }
      Quad r_lo, r_hi;
      r_lo.set(o_lo);
      r_hi.set(o_hi);
      r_lo.store(out + (int64_t)h * p.D);
      r_hi.store(out + (int64_t)h * p.D + half);
    }
  }
}

// Backward. With dy = dout * cos + rotate_half^T(dout * sin):
//     dy_lo = g_lo cos_lo + g_hi sin_hi,   dy_hi = g_hi cos_hi - g_lo sin_lo
//     dw   += dy * xhat                    (xhat = x * rstd; summed over every row of the tensor)
//     dxh   = dy * w;  dx = rstd * (dxh - xhat * mean_d(dxh * xhat))
// Blocks walk tiles with a grid stride; a thread keeps its eight dw sums in registers over all
// its rows, the block adds its slots through LDS and writes one [D] partial; a second kernel adds
// the partials in a fixed order, so dw does not depend on scheduling.
template <bool NORM>
__global__ __launch_bounds__(kThreads) void norm_rope_bwd_kernel(PairParams pp) {
  __shared__ float red[2048];  // [slots][D] = 256 threads x 8 sums
  const int which = (int)blockIdx.x >= pp.blocks0;
  const NormRopeParams& p = pp.t[which];
  const int bx = blockIdx.x - (which ? pp.blocks0 : 0);
  const int l = threadIdx.x % p.lanes;
  const int slot = threadIdx.x / p.lanes;
  const int g = slot % p.hg;
  const int b = blockIdx.y;
  const int half = p.D >> 1;

  float w_lo[4], w_hi[4];
  float dw_lo[4] = {0.f, 0.f, 0.f, 0.f}, dw_hi[4] = {0.f, 0.f, 0.f, 0.f};
  if (NORM) load_gain(p, l, w_lo, w_hi);

  for (int tile = bx; tile < p.n_tiles; tile += p.grid_x) {
    const int64_t s = (int64_t)tile * p.tile_s + slot / p.hg;
    if (s >= p.S) continue;
    const int64_t cs = b * p.cs_bs + s * p.D + 4 * l;
    Quad c_lo, c_hi, s_lo, s_hi;
    c_lo.load(p.cos + cs);
    c_hi.load(p.cos + cs + half);
    s_lo.load(p.sin + cs);
    s_hi.load(p.sin + cs + half);

    const int64_t row0 = s * p.H * (int64_t)p.D + 4 * l;
    const __bf16* x = p.x + b * p.x_bs + row0;
    const __bf16* dout = p.dout + b * p.dout_bs + row0;
    __bf16* dx = p.out + b * p.out_bs + row0;

    for (int h0 = g; h0 < p.H; h0 += kBwdBatch * p.hg) {
      Quad lo[kBwdBatch], hi[kBwdBatch], g_lo[kBwdBatch], g_hi[kBwdBatch];
#pragma unroll
      for (int u = 0; u < kBwdBatch; ++u) {
        const int h = h0 + u * p.hg;
        if (h < p.H) {
          if (NORM) {
            lo[u].load(x + (int64_t)h * p.D);
            hi[u].load(x + (int64_t)h * p.D + half);
          }
          g_lo[u].load(dout + (int64_t)h * p.D);
          g_hi[u].load(dout + (int64_t)h * p.D + half);
        }
      }
#pragma unroll
      for (int u = 0; u < kBwdBatch; ++u) {
        const int h = h0 + u * p.hg;
        if (h >= p.H) break;
        float dy_lo[4], dy_hi[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float ga = g_lo[u].get(j), gc = g_hi[u].get(j);
          dy_lo[j] = ga * c_lo.get(j) + gc * s_hi.get(j);
          dy_hi[j] = gc * c_hi.get(j) - ga * s_lo.get(j);
        }
        if (NORM) {
          float a[4], c[4];
          float ss = 0.f;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            a[j] = lo[u].get(j);
            c[j] = hi[u].get(j);
            ss += a[j] * a[j] + c[j] * c[j];
          }
          const float r = rsqrtf(row_sum(ss, p.lanes) * p.inv_d + p.eps);
          float dot = 0.f;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            a[j] *= r;  // xhat
            c[j] *= r;
            dw_lo[j] += dy_lo[j] * a[j];
            dw_hi[j] += dy_hi[j] * c[j];
            dy_lo[j] *= w_lo[j];  // d xhat
            dy_hi[j] *= w_hi[j];
            dot += dy_lo[j] * a[j] + dy_hi[j] * c[j];
          }
          const float m = row_sum(dot, p.lanes) * p.inv_d;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            dy_lo[j] = r * (dy_lo[j] - a[j] * m);
            dy_hi[j] = r * (dy_hi[j] - c[j] * m);
          }
        }
        Quad r_lo, r_hi;
        r_lo.set(dy_lo);
        r_hi.set(dy_hi);
        r_lo.store(dx + (int64_t)h * p.D);
        r_hi.store(dx + (int64_t)h * p.D + half);
      }
    }
  }

  if (NORM) {
    float* mine = red + slot * p.D;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      mine[4 * l + j] = dw_lo[j];
      mine[half + 4 * l + j] = dw_hi[j];
    }
    __syncthreads();
    const int slots = kThreads / p.lanes;
    float* part = p.partial + ((int64_t)blockIdx.y * p.grid_x + bx) * p.D;
    for (int d = threadIdx.x; d < p.D; d += kThreads) {
      float acc = 0.f;
      for (int sl = 0; sl < slots; ++sl) acc += red[sl * p.D + d];
      part[d] = acc;
    }
  }
}

// dw[d] = sum over `n` partial rows. A block owns 16 columns; 16 threads per column each add
// every 16th row (eight loads in flight), then their sums are added in thread order: the order
// of additions is fixed, so the result does not depend on scheduling.
constexpr int kSumCols = 16;

struct SumParams {
  const float* partial[2];
  float* dw[2];
  int n[2];
  int D[2];
};

__global__ __launch_bounds__(kThreads) void sum_partials_kernel(SumParams sp) {
  __shared__ float red[kThreads];
  constexpr int kParts = kThreads / kSumCols;
  const int t = blockIdx.y;  // tensor of the pair
  const int n = sp.n[t], D = sp.D[t];
  const int c = threadIdx.x % kSumCols;
  const int col = blockIdx.x * kSumCols + c;
  const int part = threadIdx.x / kSumCols;
  float acc = 0.f;
  if (col < D) {
    const float* src = sp.partial[t] + col;
    int i = part;
    for (; i + 7 * kParts < n; i += 8 * kParts) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = src[(int64_t)(i + u * kParts) * D];
#pragma unroll
      for (int u = 0; u < 8; ++u) acc += v[u];
    }
    for (; i < n; i += kParts) acc += src[(int64_t)i * D];
  }
  red[threadIdx.x] = acc;
  __syncthreads();
  if (part == 0 && col < D) {
    float total = 0.f;
    for (int i = 0; i < kParts; ++i) total += red[i * kSumCols + c];
    sp.dw[t][col] = total;
  }
}

struct Plan {
  int lanes, hg, tile_s, n_tiles;
};

// Head groups: about eight heads per slot, so cos/sin of a token are reused from registers; fewer
// heads per slot when the tensor is so small that the grid would otherwise not fill the device.
Plan make_plan(int64_t B, int64_t S, int64_t H, int64_t D) {
  Plan pl;
  pl.lanes = (int)(D / 8);
  const int slots = kThreads / pl.lanes;
  int hg = 1;
  while (hg < slots && hg * 8 < H) hg <<= 1;
  const int64_t want = 8 * (int64_t)compute_units_or_default();  // eight resident blocks per compute unit
  while (hg < slots && hg < H && B * ((S * hg + slots - 1) / slots) < want) hg <<= 1;
  pl.hg = hg;
  pl.tile_s = slots / hg;
  pl.n_tiles = (int)((S + pl.tile_s - 1) / pl.tile_s);
  return pl;
}

constexpr int kMaxBwdBlocksX = 1024;

int bwd_blocks_x(const Plan& pl, int64_t B) {
  int64_t cap = kMaxBwdBlocksX / B;
  if (cap < 1) cap = 1;
  return (int)(pl.n_tiles < cap ? pl.n_tiles : cap);
}

int validate(const char* who, const pith_norm_rope_args* a, bool backward) {
  if (!a) return fail(PITH_ERR_NULL_POINTER, "%s: args is NULL", who);
  if (!a->x || !a->cos || !a->sin || !a->out) return fail(PITH_ERR_NULL_POINTER, "%s: NULL tensor pointer", who);
  if (backward && !a->dout) return fail(PITH_ERR_NULL_POINTER, "%s: dout is NULL", who);
  if (backward && a->weight && !a->dweight) return fail(PITH_ERR_NULL_POINTER, "%s: dweight is NULL", who);
  if (a->B <= 0 || a->S <= 0 || a->H <= 0 || a->D <= 0)
    return fail(PITH_ERR_BAD_SHAPE, "%s: B=%lld S=%lld H=%lld D=%lld must all be positive", who, (long long)a->B,
                (long long)a->S, (long long)a->H, (long long)a->D);
  const int64_t lanes = a->D / 8;
  if (a->D % 8 != 0 || lanes > 64 || (lanes & (lanes - 1)) != 0)
    return fail(PITH_ERR_UNSUPPORTED, "%s: D=%lld must be 8 * a power of two, at most 512", who, (long long)a->D);
  if (a->B > 65535 || a->H > (1 << 20) || a->S > (1 << 30))
    return fail(PITH_ERR_UNSUPPORTED, "%s: B=%lld > 65535, H=%lld > 2^20 or S=%lld > 2^30 (launch grid limits)", who,
                (long long)a->B, (long long)a->H, (long long)a->S);
  if (a->weight && a->weight_dtype != PITH_BF16 && a->weight_dtype != PITH_F32)
    return fail(PITH_ERR_BAD_DTYPE, "%s: weight dtype %d is not bf16/fp32", who, a->weight_dtype);
  uintptr_t bits = reinterpret_cast<uintptr_t>(a->x) | reinterpret_cast<uintptr_t>(a->cos) |
                   reinterpret_cast<uintptr_t>(a->sin) | reinterpret_cast<uintptr_t>(a->out) |
                   reinterpret_cast<uintptr_t>(a->weight);
  if (backward) bits |= reinterpret_cast<uintptr_t>(a->dout);
  if (bits % 8 || a->x_bs % 4 || a->out_bs % 4 || (backward && a->dout_bs % 4) || a->cs_bs % 4)
    return fail(PITH_ERR_MISALIGNED, "%s: pointers / batch strides must keep 8-byte alignment", who);
  const int64_t slab = a->S * a->H * a->D;
  if (a->B > 1 && (a->x_bs < slab || a->out_bs < slab || (backward && a->dout_bs < slab)))
    return fail(PITH_ERR_BAD_SHAPE, "%s: a batch stride is smaller than S*H*D", who);
  if (a->cs_bs != 0 && a->B > 1 && a->cs_bs < a->S * a->D)
    return fail(PITH_ERR_BAD_SHAPE, "%s: cos/sin batch stride must be 0 (shared) or at least S*D", who);
  return PITH_OK;
}

NormRopeParams make_params(const pith_norm_rope_args* a, const Plan& pl) {
  NormRopeParams p;
  p.x = (const __bf16*)a->x; p.w = a->weight; p.cos = (const __bf16*)a->cos; p.sin = (const __bf16*)a->sin;
  p.dout = (const __bf16*)a->dout; p.out = (__bf16*)a->out; p.partial = nullptr;
  p.S = a->S; p.H = (int)a->H; p.D = (int)a->D;
  p.lanes = pl.lanes; p.hg = pl.hg; p.tile_s = pl.tile_s; p.n_tiles = pl.n_tiles; p.grid_x = pl.n_tiles;
  p.x_bs = a->x_bs; p.out_bs = a->out_bs; p.dout_bs = a->dout_bs; p.cs_bs = a->cs_bs;
  p.eps = a->eps; p.inv_d = 1.0f / (float)a->D;
  p.w_f32 = a->weight_dtype == PITH_F32;
  return p;
}

}  // namespace
}  // namespace pith

using namespace pith;

namespace {

// What the two tensors of a pair must agree on: the grid's batch dimension and the kernel variant.
int validate_pair(const char* who, const pith_norm_rope_args* a, const pith_norm_rope_args* b) {
  if (a->B != b->B) return fail(PITH_ERR_BAD_SHAPE, "%s: the two tensors differ in B (%lld, %lld)", who, (long long)a->B, (long long)b->B);
  if ((a->weight == nullptr) != (b->weight == nullptr))
    return fail(PITH_ERR_UNSUPPORTED, "%s: either both tensors have a weight or neither", who);
  return PITH_OK;
}

// `b` may be NULL (one tensor).
int launch_fwd(const char* who, const pith_norm_rope_args* a, const pith_norm_rope_args* b, pith_stream_t stream) {
  if (const int rc = validate(who, a, false)) return rc;
  if (b) {
    if (const int rc = validate(who, b, false)) return rc;
    if (const int rc = validate_pair(who, a, b)) return rc;
  }
  PairParams pp;
  const Plan pa = make_plan(a->B, a->S, a->H, a->D);
  pp.t[0] = make_params(a, pa);
  pp.t[1] = pp.t[0];
  pp.blocks0 = pa.n_tiles;
  int64_t blocks = pa.n_tiles;
  if (b) {
    const Plan pb = make_plan(b->B, b->S, b->H, b->D);
    pp.t[1] = make_params(b, pb);
    blocks += pb.n_tiles;
  }
  if (blocks > 0x7fffffffLL) return fail(PITH_ERR_UNSUPPORTED, "%s: %lld row tiles exceed the launch grid limit", who, (long long)blocks);
  const dim3 grid((unsigned)blocks, (unsigned)a->B);
  begin_launch();
  if (a->weight)
    hipLaunchKernelGGL(norm_rope_fwd_kernel<true>, grid, dim3(kThreads), 0, (hipStream_t)stream, pp);
  else
    hipLaunchKernelGGL(norm_rope_fwd_kernel<false>, grid, dim3(kThreads), 0, (hipStream_t)stream, pp);
  return check_launch(who);
}

int prepare_bwd(const char* who, const pith_norm_rope_args* a, NormRopeParams* p) {
  const Plan pl = make_plan(a->B, a->S, a->H, a->D);
  *p = make_params(a, pl);
  p->grid_x = bwd_blocks_x(pl, a->B);
  if (!a->weight) return PITH_OK;
  const int64_t need = (int64_t)p->grid_x * a->B * a->D * (int64_t)sizeof(float);
  if (!a->workspace || a->workspace_bytes < need)
    return fail(PITH_ERR_BAD_SHAPE, "%s: workspace of %lld bytes needed, %lld given", who, (long long)need,
                (long long)(a->workspace ? a->workspace_bytes : 0));
  if (reinterpret_cast<uintptr_t>(a->workspace) % 4 || reinterpret_cast<uintptr_t>(a->dweight) % 4)
    return fail(PITH_ERR_MISALIGNED, "%s: workspace / dweight must be 4-byte aligned", who);
  p->partial = (float*)a->workspace;
  return PITH_OK;
}

int launch_bwd(const char* who, const pith_norm_rope_args* a, const pith_norm_rope_args* b, pith_stream_t stream) {
  if (const int rc = validate(who, a, true)) return rc;
  if (b) {
    if (const int rc = validate(who, b, true)) return rc;
    if (const int rc = validate_pair(who, a, b)) return rc;
  }
  PairParams pp;
  if (const int rc = prepare_bwd(who, a, &pp.t[0])) return rc;
  pp.t[1] = pp.t[0];
  pp.blocks0 = pp.t[0].grid_x;
  int64_t blocks = pp.blocks0;
  if (b) {
    if (const int rc = prepare_bwd(who, b, &pp.t[1])) return rc;
    blocks += pp.t[1].grid_x;
  }
  const dim3 grid((unsigned)blocks, (unsigned)a->B);
  begin_launch();
  hipStream_t st = (hipStream_t)stream;
  if (!a->weight) {
    hipLaunchKernelGGL(norm_rope_bwd_kernel<false>, grid, dim3(kThreads), 0, st, pp);
    return check_launch(who);
  }
  hipLaunchKernelGGL(norm_rope_bwd_kernel<true>, grid, dim3(kThreads), 0, st, pp);
  if (const int rc = check_launch(who)) return rc;
  SumParams sp;
  const pith_norm_rope_args* both[2] = {a, b ? b : a};
  int64_t max_d = 0;
  for (int t = 0; t < 2; ++t) {
    sp.partial[t] = pp.t[t].partial;
    sp.dw[t] = both[t]->dweight;
    sp.n[t] = (int)(pp.t[t].grid_x * both[t]->B);
    sp.D[t] = (int)both[t]->D;
    if (both[t]->D > max_d) max_d = both[t]->D;
  }
  hipLaunchKernelGGL(sum_partials_kernel, dim3((unsigned)((max_d + kSumCols - 1) / kSumCols), b ? 2u : 1u),
                     dim3(kThreads), 0, st, sp);
  return check_launch(who);
}

}  // namespace

extern "C" int pith_norm_rope_fwd(const pith_norm_rope_args* a, pith_stream_t stream) {
  return launch_fwd("pith_norm_rope_fwd", a, nullptr, stream);
}

extern "C" int pith_norm_rope_fwd_pair(const pith_norm_rope_args* a, const pith_norm_rope_args* b, pith_stream_t stream) {
  if (!a || !b) return fail(PITH_ERR_NULL_POINTER, "pith_norm_rope_fwd_pair: args is NULL");
  return launch_fwd("pith_norm_rope_fwd_pair", a, b, stream);
}

extern "C" int64_t pith_norm_rope_bwd_workspace_bytes(const pith_norm_rope_args* a) {
  if (!a || !a->weight || a->B <= 0 || a->S <= 0 || a->H <= 0 || a->D <= 0 || a->D % 8 != 0 || a->D > 512) return 0;
  const Plan pl = make_plan(a->B, a->S, a->H, a->D);
  return (int64_t)bwd_blocks_x(pl, a->B) * a->B * a->D * (int64_t)sizeof(float);
}

extern "C" int pith_norm_rope_bwd(const pith_norm_rope_args* a, pith_stream_t stream) {
  return launch_bwd("pith_norm_rope_bwd", a, nullptr, stream);
}

extern "C" int pith_norm_rope_bwd_pair(const pith_norm_rope_args* a, const pith_norm_rope_args* b, pith_stream_t stream) {
  if (!a || !b) return fail(PITH_ERR_NULL_POINTER, "pith_norm_rope_bwd_pair: args is NULL");
  return launch_bwd("pith_norm_rope_bwd_pair", a, b, stream);
}
