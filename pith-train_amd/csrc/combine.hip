// Online-softmax combine of two partial attention results, plus the two small streaming
// kernels of the path (delta = rowsum(O*dO), fp32 -> bf16 cast). All three are HBM-bound:
// every byte of the operands is read once and every byte of the result written once, with
// accesses that are contiguous across a wavefront; results are written with non-temporal
// stores (measured +12 % on the combine: the output is not read again by this kernel).
//
// Combine follows pithtrain/operators/ring_attention/mla.py:27-40 (base 2) and
// pithtrain/operators/ring_attention/standard.py:53-66 (base e).
//
// Two combine kernels compute the same values bit for bit. combine_front_kernel serves the common
// shapes: one resident block per compute unit, all blocks together walking the tensors as ONE
// moving front (measured: the memory system gives a compact front of a few MB 10-15 % more than
// thousands of independent slabs). combine_kernel (one block per tile) takes every other shape.
#include "pith_common.h"

namespace pith {
namespace {

constexpr int kCombineThreads = 256;

// 8 consecutive elements of a bf16 or fp32 row.
template <typename T>
struct Vec8;

template <>
struct Vec8<__bf16> {
  u32x4 raw;
  __device__ __forceinline__ void load(const __bf16* p) { raw = *reinterpret_cast<const u32x4*>(p); }
  __device__ __forceinline__ void load_nt(const __bf16* p) { raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)); }
  __device__ __forceinline__ void store(__bf16* p) const { __builtin_nontemporal_store(raw, reinterpret_cast<u32x4*>(p)); }
  __device__ __forceinline__ float get(int i) const {
    uint32_t w = raw[i >> 1];
    return (i & 1) ? bf16hi_to_f32(w) : bf16lo_to_f32(w);
  }
  __device__ __forceinline__ void set_pair(int pair, float a, float b) { raw[pair] = pack_bf16x2(a, b); }
};

template <>
struct Vec8<float> {
  f32x4 lo, hi;
  __device__ __forceinline__ void load(const float* p) {
    lo = *reinterpret_cast<const f32x4*>(p);
    hi = *reinterpret_cast<const f32x4*>(p + 4);
  }
  __device__ __forceinline__ void load_nt(const float* p) {
    lo = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
    hi = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p + 4));
  }
  __device__ __forceinline__ void store(float* p) const {
    __builtin_nontemporal_store(lo, reinterpret_cast<f32x4*>(p));
    __builtin_nontemporal_store(hi, reinterpret_cast<f32x4*>(p + 4));
  }
  __device__ __forceinline__ float get(int i) const { return i < 4 ? lo[i] : hi[i - 4]; }
  __device__ __forceinline__ void set_pair(int pair, float a, float b) {
    if (pair < 2) {
      lo[2 * pair] = a;
      lo[2 * pair + 1] = b;
    } else {
      hi[2 * pair - 4] = a;
      hi[2 * pair - 3] = b;
    }
  }
};

// 4 consecutive elements: used when a tensor of the call is fp32, so that every access of a
// wavefront instruction is one contiguous range (16 bytes per lane for fp32, 8 for bf16).
template <typename T>
struct Vec4;

template <>
struct Vec4<__bf16> {
  u32x2 raw;
  __device__ __forceinline__ void load(const __bf16* p) { raw = *reinterpret_cast<const u32x2*>(p); }
  __device__ __forceinline__ void load_nt(const __bf16* p) { raw = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p)); }
  __device__ __forceinline__ void store(__bf16* p) const { __builtin_nontemporal_store(raw, reinterpret_cast<u32x2*>(p)); }
  __device__ __forceinline__ float get(int i) const {
    uint32_t w = raw[i >> 1];
    return (i & 1) ? bf16hi_to_f32(w) : bf16lo_to_f32(w);
  }
  __device__ __forceinline__ void set_pair(int pair, float a, float b) { raw[pair] = pack_bf16x2(a, b); }
};

template <>
struct Vec4<float> {
  f32x4 raw;
  __device__ __forceinline__ void load(const float* p) { raw = *reinterpret_cast<const f32x4*>(p); }
  __device__ __forceinline__ void load_nt(const float* p) { raw = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p)); }
  __device__ __forceinline__ void store(float* p) const { __builtin_nontemporal_store(raw, reinterpret_cast<f32x4*>(p)); }
  __device__ __forceinline__ float get(int i) const { return raw[i]; }
  __device__ __forceinline__ void set_pair(int pair, float a, float b) {
    raw[2 * pair] = a;
    raw[2 * pair + 1] = b;
  }
};

template <typename T, int N>
struct VecSel;
template <typename T>
struct VecSel<T, 8> { typedef Vec8<T> type; };
template <typename T>
struct VecSel<T, 4> { typedef Vec4<T> type; };

// (w1*x + w2*y) * rinv with each product rounded on its own (no fused multiply-add), as the
// reference's eager expression evaluates it: the result is then bit-identical when the two
// partials are swapped.
__device__ __forceinline__ float merge_element(float w1, float x, float w2, float y, float rinv) {
#pragma clang fp contract(off)
  const float a = w1 * x;
  const float b = w2 * y;
  return (a + b) * rinv;
}

// Weights of one (position, head) row from its two lse values: (w1, w2, 1/(w1+w2)) and the
// merged lse. Both partials empty (both lse -inf): the reference yields NaN (-inf - -inf); an
// empty result (weights 0, lse -inf) is returned instead. The ring never produces this case.
__device__ __forceinline__ f32x4 merge_weights(float a, float c, bool base_e) {
  const float m = fmaxf(a, c);
  if (m == -INFINITY) return f32x4{0.f, 0.f, 0.f, -INFINITY};
  float w1, w2;
  if (base_e) {
    w1 = expf(a - m);
    w2 = expf(c - m);
  } else {
    w1 = exp2f(a - m);
    w2 = exp2f(c - m);
  }
  const float sum = w1 + w2;
  return f32x4{w1, w2, 1.f / sum, m + (base_e ? logf(sum) : log2f(sum))};
}

struct CombineParams {
  const void* out1;
  const float* lse1;
  const void* out2;
  const float* lse2;
  void* out;
  float* lse_out;
  int64_t S;
  int H, D8;  // D8 = D / 8 chunks of 16 bytes (bf16) per head row
  int tile_s;
  int base_e;
  int64_t out1_bs, out2_bs, out_bs;
  int64_t lse1_bs, lse1_hs, lse2_bs, lse2_hs, lse_out_bs, lse_out_hs;
};

// One block = `tile_s` consecutive sequence positions of one batch element, all heads.
// Stage 1: the [H, tile_s] patch of both LSE tensors is read (contiguous along s), the two
//          normalised weights are left in LDS and the merged LSE is written.
// Stage 2: the [tile_s, H, D] slab of O, which is one contiguous range of memory, is streamed
//          with 16-byte accesses; thread t owns chunks t, t+256, ...
template <typename T1, typename T2, typename TO, int N>
__global__ __launch_bounds__(kCombineThreads) void combine_kernel(CombineParams p) {
  const int DN = p.D8 * (8 / N);  // chunks of N elements per head row
  extern __shared__ float weights[];  // [rows][3] = (w1, w2, 1/(w1+w2)), rows = tile_s * H, row = s_local * H + h
  const int b = blockIdx.y;
  const int64_t s0 = (int64_t)blockIdx.x * p.tile_s;
  const int ts = (int)min((int64_t)p.tile_s, p.S - s0);
  const int rows = ts * p.H;

  const float* l1 = p.lse1 + b * p.lse1_bs + s0;
  const float* l2 = p.lse2 + b * p.lse2_bs + s0;
  float* lo = p.lse_out + b * p.lse_out_bs + s0;
  for (int i = threadIdx.x; i < rows; i += kCombineThreads) {
    const int h = i / ts, sl = i - h * ts;
    const f32x4 mw = merge_weights(l1[h * p.lse1_hs + sl], l2[h * p.lse2_hs + sl], p.base_e != 0);
    float* w = weights + 3 * (sl * p.H + h);
    w[0] = mw[0];
    w[1] = mw[1];
    w[2] = mw[2];
    lo[h * p.lse_out_hs + sl] = mw[3];
  }
  __syncthreads();

  const int64_t slab = (s0 * p.H) * (int64_t)p.D8 * 8;
  const T1* o1 = reinterpret_cast<const T1*>(p.out1) + b * p.out1_bs + slab;
  const T2* o2 = reinterpret_cast<const T2*>(p.out2) + b * p.out2_bs + slab;
  TO* oo = reinterpret_cast<TO*>(p.out) + b * p.out_bs + slab;
  const int chunks = rows * DN;

  constexpr int kUnroll = 4;
  for (int c0 = threadIdx.x; c0 < chunks; c0 += kCombineThreads * kUnroll) {
    typename VecSel<T1, N>::type x[kUnroll];
    typename VecSel<T2, N>::type y[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int c = c0 + u * kCombineThreads;
      if (c < chunks) {
        x[u].load(o1 + (int64_t)c * N);
        y[u].load(o2 + (int64_t)c * N);
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int c = c0 + u * kCombineThreads;
      if (c < chunks) {
        const int row = c / DN;
        const float w1 = weights[3 * row], w2 = weights[3 * row + 1], rinv = weights[3 * row + 2];
        typename VecSel<TO, N>::type r;
#pragma unroll
        for (int j = 0; j < N / 2; ++j)
          r.set_pair(j, merge_element(w1, x[u].get(2 * j), w2, y[u].get(2 * j), rinv),
                     merge_element(w1, x[u].get(2 * j + 1), w2, y[u].get(2 * j + 1), rinv));
        r.store(oo + (int64_t)c * N);
      }
    }
  }
}

// Front-walking variant. A tile is `tile_s` consecutive positions x all heads = exactly 256 * U
// chunks of N elements, with at most 256 (position, head) rows; the grid is G blocks (G a multiple
// of 8, one block per compute unit) and round k covers tiles [k*G, (k+1)*G): the whole device
// reads and writes one window of G tiles that moves through memory. Within a round block `id`
// takes tile (id % 8) * (G/8) + id / 8: workgroups are dealt to the 8 XCDs round-robin, so the
// blocks of one XCD own G/8 CONSECUTIVE positions and every 128-byte line of the [B,H,S] lse
// tensors is fetched, and every line of lse_out written, through a single L2.
// Per tile: the O loads are issued first, then thread r < rows turns the lse pair it fetched one
// round earlier into weights (LDS, double buffered, one barrier per tile) while the loads are in
// flight, fetches the next round's lse pair, and the tile is merged and stored.
// Aliasing: every O chunk and every lse element is read by the thread that later writes it.
template <typename T1, typename T2, typename TO, int N, int U>
__global__ __launch_bounds__(kCombineThreads) void combine_front_kernel(CombineParams p, int n_tiles, int dn_shift) {
  __shared__ f32x4 wsm[2][kCombineThreads];
  const int b = blockIdx.y;
  const int rows = p.tile_s * p.H;
  const char* o1 = reinterpret_cast<const char*>(reinterpret_cast<const T1*>(p.out1) + b * p.out1_bs);
  const char* o2 = reinterpret_cast<const char*>(reinterpret_cast<const T2*>(p.out2) + b * p.out2_bs);
  char* oo = reinterpret_cast<char*>(reinterpret_cast<TO*>(p.out) + b * p.out_bs);
  const float* l1 = p.lse1 + b * p.lse1_bs;
  const float* l2 = p.lse2 + b * p.lse2_bs;
  float* lo = p.lse_out + b * p.lse_out_bs;
  const int tid = threadIdx.x;
  const int h = tid / p.tile_s, sl = tid - h * p.tile_s;  // the row this thread weighs: lse[h][tile * tile_s + sl]
  const bool has_row = tid < rows;
  constexpr int kTileChunks = kCombineThreads * U;
  const int G = gridDim.x;
  int t = (blockIdx.x & 7) * (G >> 3) + (blockIdx.x >> 3);
  float la = 0.f, lc = 0.f;
  if (t < n_tiles && has_row) {
    la = l1[h * p.lse1_hs + (int64_t)t * p.tile_s + sl];
    lc = l2[h * p.lse2_hs + (int64_t)t * p.tile_s + sl];
  }
  typedef typename VecSel<T1, N>::type V1;
  typedef typename VecSel<T2, N>::type V2;
  typedef typename VecSel<TO, N>::type VO;
  int buf = 0;
  for (; t < n_tiles; t += G, buf ^= 1) {
    V1 x[U];
    V2 y[U];
    const size_t c_base = (size_t)t * kTileChunks + tid;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t c = c_base + u * kCombineThreads;
      x[u].load_nt(reinterpret_cast<const T1*>(o1 + c * (N * sizeof(T1))));
      y[u].load_nt(reinterpret_cast<const T2*>(o2 + c * (N * sizeof(T2))));
    }
    const float a = la, c2 = lc;
    const int tn = t + G;
    if (tn < n_tiles && has_row) {
      la = l1[h * p.lse1_hs + (int64_t)tn * p.tile_s + sl];
      lc = l2[h * p.lse2_hs + (int64_t)tn * p.tile_s + sl];
    }
    if (has_row) {
      const f32x4 mw = merge_weights(a, c2, p.base_e != 0);
      wsm[buf][sl * p.H + h] = mw;
      lo[h * p.lse_out_hs + (int64_t)t * p.tile_s + sl] = mw[3];
    }
    __syncthreads();  // also orders this tile's reads of wsm[buf] before the writes two tiles later
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const f32x4 w = wsm[buf][(tid + u * kCombineThreads) >> dn_shift];
      VO r;
#pragma unroll
      for (int j = 0; j < N / 2; ++j)
        r.set_pair(j, merge_element(w[0], x[u].get(2 * j), w[1], y[u].get(2 * j), w[2]),
                   merge_element(w[0], x[u].get(2 * j + 1), w[1], y[u].get(2 * j + 1), w[2]));
      r.store(reinterpret_cast<TO*>(oo + (c_base + u * kCombineThreads) * (N * sizeof(TO))));
    }
  }
}

// Tile shape for combine_front_kernel, or tile_s = 0 when the shape does not fit its assumptions
// (chunks per head row a power of two, a tile of exactly 256 * U chunks with U in {2, 4, 8} and at
// most 256 rows, S a multiple of the tile).
struct FrontPlan {
  int tile_s, unroll, dn_shift;
};

FrontPlan plan_front(int64_t S, int64_t H, int64_t D, int n) {
  FrontPlan fp = {0, 0, 0};
  const int64_t dn = D / n;
  if (D % n != 0 || (dn & (dn - 1)) != 0 || dn > kCombineThreads) return fp;
  int shift = 0;
  while ((1 << shift) < dn) ++shift;
  const int prefer[3] = {4, 8, 2};
  for (int u : prefer)
    for (int ts = 1; ts <= 8; ts <<= 1)
      if (S % ts == 0 && ts * H <= kCombineThreads && ts * H * dn == (int64_t)kCombineThreads * u &&
          S / ts < (1 << 30)) {
        fp.tile_s = ts;
        fp.unroll = u;
        fp.dn_shift = shift;
        return fp;
      }
  return fp;
}

template <typename T1, typename T2, typename TO, int N>
void launch_front(const CombineParams& p, const FrontPlan& fp, int n_tiles, dim3 grid, hipStream_t st) {
  const dim3 block(kCombineThreads);
  if (fp.unroll == 2) hipLaunchKernelGGL((combine_front_kernel<T1, T2, TO, N, 2>), grid, block, 0, st, p, n_tiles, fp.dn_shift);
  else if (fp.unroll == 4) hipLaunchKernelGGL((combine_front_kernel<T1, T2, TO, N, 4>), grid, block, 0, st, p, n_tiles, fp.dn_shift);
  else hipLaunchKernelGGL((combine_front_kernel<T1, T2, TO, N, 8>), grid, block, 0, st, p, n_tiles, fp.dn_shift);
}

// Elements per chunk of a dtype combination: 4 whenever an fp32 tensor takes part (see Vec4).
template <typename T1, typename T2>
constexpr int chunk_elems(bool out_f32) {
  return (sizeof(T1) == 4 || sizeof(T2) == 4 || out_f32) ? 4 : 8;
}

template <typename T1, typename T2>
void launch_front_t2(const CombineParams& p, int dtype_out, const FrontPlan& fp, int n_tiles, dim3 grid, hipStream_t st) {
  if (dtype_out == PITH_BF16) launch_front<T1, T2, __bf16, chunk_elems<T1, T2>(false)>(p, fp, n_tiles, grid, st);
  else launch_front<T1, T2, float, 4>(p, fp, n_tiles, grid, st);
}

template <typename T1, typename T2>
void launch_combine_t2(const CombineParams& p, int dtype_out, dim3 grid, size_t lds, hipStream_t st) {
  // N = 4 whenever an fp32 tensor takes part (see Vec4)
  constexpr bool in_f32 = sizeof(T1) == 4 || sizeof(T2) == 4;
  if (dtype_out == PITH_BF16)
    hipLaunchKernelGGL((combine_kernel<T1, T2, __bf16, in_f32 ? 4 : 8>), grid, dim3(kCombineThreads), lds, st, p);
  else
    hipLaunchKernelGGL((combine_kernel<T1, T2, float, 4>), grid, dim3(kCombineThreads), lds, st, p);
}

// ---------------------------------------------------------------------------------------------
// delta[b,h,s] = sum_d O*dO (pithtrain/operators/mla/triton.py:101-122). One block handles
// `tile_s` consecutive positions x all heads; the [tile_s, H, D] slabs of O and dO are contiguous.
// D/8 consecutive lanes own one (s,h) row and reduce with DPP-free shuffles; the per-row sums go
// through LDS so the [H, tile_s] patch of delta is written contiguously along s.
struct DeltaParams {
  const __bf16* o;
  const __bf16* dout;
  float* delta;
  int64_t S;
  int H, D8, tile_s;
  int64_t o_bs, dout_bs, delta_bs, delta_hs;
};

constexpr int kDeltaThreads = 256;

__global__ __launch_bounds__(kDeltaThreads) void delta_kernel(DeltaParams p) {
  extern __shared__ float rowsum[];  // [tile_s * H]
  const int b = blockIdx.y;
  const int64_t s0 = (int64_t)blockIdx.x * p.tile_s;
  const int ts = (int)min((int64_t)p.tile_s, p.S - s0);
  const int rows = ts * p.H;
  const int64_t slab = (s0 * p.H) * (int64_t)p.D8 * 8;
  const __bf16* o = p.o + b * p.o_bs + slab;
  const __bf16* g = p.dout + b * p.dout_bs + slab;
  const int chunks = rows * p.D8;
  // D8 is a power of two <= 64 (checked on the host), so the lanes of one row sit inside one wave.
  for (int c0 = 0; c0 < chunks; c0 += kDeltaThreads) {
    const int c = c0 + threadIdx.x;
    float acc = 0.f;
    if (c < chunks) {
      Vec8<__bf16> x, y;
      x.load(o + (int64_t)c * 8);
      y.load(g + (int64_t)c * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc += x.get(j) * y.get(j);
    }
    for (int off = p.D8 >> 1; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
    if (c < chunks && (c & (p.D8 - 1)) == 0) rowsum[c / p.D8] = acc;
  }
  __syncthreads();
  float* d = p.delta + b * p.delta_bs + s0;
  for (int i = threadIdx.x; i < rows; i += kDeltaThreads) {
    const int h = i / ts, sl = i - h * ts;
    d[h * p.delta_hs + sl] = rowsum[sl * p.H + h];
  }
}

__global__ __launch_bounds__(256) void cast_f32_bf16_kernel(const float* __restrict__ src, __bf16* __restrict__ dst,
                                                            int64_t n8) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += (int64_t)gridDim.x * blockDim.x) {
    Vec8<float> x;
    x.load(src + i * 8);
    Vec8<__bf16> y;
#pragma unroll
    for (int j = 0; j < 4; ++j) y.set_pair(j, x.get(2 * j), x.get(2 * j + 1));
    y.store(dst + i * 8);
  }
}

// Rows per block: as many as keep the grid at several blocks per CU and the LDS patch small.
int pick_tile_s(int64_t B, int64_t S, int64_t H, int max_rows) {
  int ts = 16;
  const int64_t want = 8 * (int64_t)compute_units_or_default();  // eight resident blocks per compute unit
  while (ts > 1 && (B * ((S + ts - 1) / ts) < want || ts * H > max_rows)) ts >>= 1;
  return ts;
}

}  // namespace
}  // namespace pith

using namespace pith;

extern "C" int pith_combine(const pith_combine_args* a, pith_stream_t stream) {
  if (!a) return fail(PITH_ERR_NULL_POINTER, "pith_combine: args is NULL");
  if (!a->out1 || !a->lse1 || !a->out2 || !a->lse2 || !a->out || !a->lse_out)
    return fail(PITH_ERR_NULL_POINTER, "pith_combine: NULL tensor pointer");
  if (a->B <= 0 || a->S <= 0 || a->H <= 0 || a->D <= 0)
    return fail(PITH_ERR_BAD_SHAPE, "pith_combine: B=%lld S=%lld H=%lld D=%lld must all be positive", (long long)a->B,
                (long long)a->S, (long long)a->H, (long long)a->D);
  if (a->D % 8 != 0) return fail(PITH_ERR_BAD_SHAPE, "pith_combine: D=%lld is not a multiple of 8", (long long)a->D);
  if (a->H > 4096 || a->B > 65535)
    return fail(PITH_ERR_UNSUPPORTED, "pith_combine: H=%lld > 4096 or B=%lld > 65535", (long long)a->H,
                (long long)a->B);
  const int dts[3] = {a->dtype1, a->dtype2, a->dtype_out};
  for (int dt : dts)
    if (dt != PITH_BF16 && dt != PITH_F32) return fail(PITH_ERR_BAD_DTYPE, "pith_combine: dtype %d is not bf16/fp32", dt);
  if (a->base != PITH_BASE_2 && a->base != PITH_BASE_E)
    return fail(PITH_ERR_BAD_DTYPE, "pith_combine: base %d is not PITH_BASE_2/PITH_BASE_E", a->base);
  if (!aligned16(a->out1) || !aligned16(a->out2) || !aligned16(a->out) || a->out1_bs % 8 || a->out2_bs % 8 ||
      a->out_bs % 8)
    return fail(PITH_ERR_MISALIGNED, "pith_combine: O pointers / batch strides must keep 16-byte alignment");
  const int64_t slab = a->S * a->H * a->D;
  if (a->B > 1 && (a->out1_bs < slab || a->out2_bs < slab || a->out_bs < slab))
    return fail(PITH_ERR_BAD_SHAPE, "pith_combine: an O batch stride is smaller than S*H*D");

  CombineParams p;
  p.out1 = a->out1; p.lse1 = a->lse1; p.out2 = a->out2; p.lse2 = a->lse2; p.out = a->out; p.lse_out = a->lse_out;
  p.S = a->S; p.H = (int)a->H; p.D8 = (int)(a->D / 8);
  p.base_e = a->base == PITH_BASE_E;
  p.out1_bs = a->out1_bs; p.out2_bs = a->out2_bs; p.out_bs = a->out_bs;
  p.lse1_bs = a->lse1_bs; p.lse1_hs = a->lse1_hs; p.lse2_bs = a->lse2_bs; p.lse2_hs = a->lse2_hs;
  p.lse_out_bs = a->lse_out_bs; p.lse_out_hs = a->lse_out_hs;
  hipStream_t st = (hipStream_t)stream;
  const bool any_f32 = a->dtype1 == PITH_F32 || a->dtype2 == PITH_F32 || a->dtype_out == PITH_F32;
  const FrontPlan fp = plan_front(a->S, a->H, a->D, any_f32 ? 4 : 8);
  const int cus = compute_units();
  if (fp.tile_s > 0 && cus >= 8) {
    p.tile_s = fp.tile_s;
    const int n_tiles = (int)(a->S / fp.tile_s);
    int g = cus & ~7;  // one block per compute unit, a multiple of the 8 XCDs
    if (n_tiles < g) g = (n_tiles + 7) & ~7;
    begin_launch();
    const dim3 fgrid((unsigned)g, (unsigned)a->B);
    if (a->dtype1 == PITH_BF16) {
      if (a->dtype2 == PITH_BF16) launch_front_t2<__bf16, __bf16>(p, a->dtype_out, fp, n_tiles, fgrid, st);
      else launch_front_t2<__bf16, float>(p, a->dtype_out, fp, n_tiles, fgrid, st);
    } else {
      if (a->dtype2 == PITH_BF16) launch_front_t2<float, __bf16>(p, a->dtype_out, fp, n_tiles, fgrid, st);
      else launch_front_t2<float, float>(p, a->dtype_out, fp, n_tiles, fgrid, st);
    }
    return check_launch("pith_combine");
  }
  p.tile_s = pick_tile_s(a->B, a->S, a->H, 4096);
  const dim3 grid((unsigned)((a->S + p.tile_s - 1) / p.tile_s), (unsigned)a->B);
  const size_t lds = (size_t)p.tile_s * p.H * 3 * sizeof(float);
  begin_launch();
  if (a->dtype1 == PITH_BF16) {
    if (a->dtype2 == PITH_BF16) launch_combine_t2<__bf16, __bf16>(p, a->dtype_out, grid, lds, st);
    else launch_combine_t2<__bf16, float>(p, a->dtype_out, grid, lds, st);
  } else {
    if (a->dtype2 == PITH_BF16) launch_combine_t2<float, __bf16>(p, a->dtype_out, grid, lds, st);
    else launch_combine_t2<float, float>(p, a->dtype_out, grid, lds, st);
  }
  return check_launch("pith_combine");
}

extern "C" int pith_attn_bwd_delta(const pith_attn_delta_args* a, pith_stream_t stream) {
  if (!a) return fail(PITH_ERR_NULL_POINTER, "pith_attn_bwd_delta: args is NULL");
  if (!a->o || !a->dout || !a->delta) return fail(PITH_ERR_NULL_POINTER, "pith_attn_bwd_delta: NULL tensor pointer");
  if (a->B <= 0 || a->S <= 0 || a->H <= 0 || a->D <= 0)
    return fail(PITH_ERR_BAD_SHAPE, "pith_attn_bwd_delta: B=%lld S=%lld H=%lld D=%lld must all be positive",
                (long long)a->B, (long long)a->S, (long long)a->H, (long long)a->D);
  const int64_t d8 = a->D / 8;
  if (a->D % 8 != 0 || d8 > 64 || (d8 & (d8 - 1)) != 0)
    return fail(PITH_ERR_UNSUPPORTED, "pith_attn_bwd_delta: D=%lld must be 8 * a power of two, at most 512",
                (long long)a->D);
  if (a->H > 4096 || a->B > 65535)
    return fail(PITH_ERR_UNSUPPORTED, "pith_attn_bwd_delta: H=%lld > 4096 or B=%lld > 65535", (long long)a->H,
                (long long)a->B);
  if (!aligned16(a->o) || !aligned16(a->dout) || a->o_bs % 8 || a->dout_bs % 8)
    return fail(PITH_ERR_MISALIGNED, "pith_attn_bwd_delta: O/dO pointers / batch strides must keep 16-byte alignment");
  DeltaParams p;
  p.o = (const __bf16*)a->o; p.dout = (const __bf16*)a->dout; p.delta = a->delta;
  p.S = a->S; p.H = (int)a->H; p.D8 = (int)d8;
  p.o_bs = a->o_bs; p.dout_bs = a->dout_bs; p.delta_bs = a->delta_bs; p.delta_hs = a->delta_hs;
  p.tile_s = pick_tile_s(a->B, a->S, a->H, 8192);
  const dim3 grid((unsigned)((a->S + p.tile_s - 1) / p.tile_s), (unsigned)a->B);
  begin_launch();
  hipLaunchKernelGGL(delta_kernel, grid, dim3(kDeltaThreads), (size_t)p.tile_s * p.H * sizeof(float),
                     (hipStream_t)stream, p);
  return check_launch("pith_attn_bwd_delta");
}

extern "C" int pith_cast_f32_bf16(const float* src, void* dst, int64_t n, pith_stream_t stream) {
  if (!src || !dst) return fail(PITH_ERR_NULL_POINTER, "pith_cast_f32_bf16: NULL pointer");
  if (n <= 0 || n % 8 != 0) return fail(PITH_ERR_BAD_SHAPE, "pith_cast_f32_bf16: n=%lld must be a positive multiple of 8", (long long)n);
  if (!aligned16(src) || !aligned16(dst)) return fail(PITH_ERR_MISALIGNED, "pith_cast_f32_bf16: pointers must be 16-byte aligned");
  const int64_t n8 = n / 8;
  const int64_t blocks = (n8 + 255) / 256;
  begin_launch();
  hipLaunchKernelGGL(cast_f32_bf16_kernel, dim3((unsigned)(blocks < 16384 ? blocks : 16384)), dim3(256), 0,
                     (hipStream_t)stream, src, (__bf16*)dst, n8);
  return check_launch("pith_cast_f32_bf16");
}
