// Declarations shared by the two backward kernels (dQ and dK/dV).
#pragma once

#include "attn_tiles.h"

namespace pith {

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
  int Sq, Skv, Hq, Hkv, group, B;
  // heads per ROW of the query-side tensors (q, dout, dq) and of the key-side tensors (k, v, dk, dv): Hq / Hkv for
  // tensors that hold exactly the heads of this call, larger when the call works on a head range of wider tensors
  int HqT, HkvT;
  int tiles;  // query tiles (dQ kernel) or key tiles (dK/dV kernel) in the grid's x dimension
  int64_t q_bs, k_bs, v_bs, dout_bs, dq_bs, dk_bs, dv_bs, lse_bs, lse_hs;
  float kappa, scale;
  int accumulate;
  int split;        // dK/dV kernel: query-head groups are cut into `split` parts handled by different workgroups
  float* ws_dk;     // dK/dV kernel, split > 1: fp32 partial results [split][B][Skv][Hkv][D]
  float* ws_dv;
  // keys in two parts (k_pe != nullptr): k / dk hold the first 128 features per head; k_pe holds the
  // last 64, one vector per position shared by all heads (batch / row strides in elements);
  // ws_dkpe: dK/dV kernel, fp32 per-head gradients of k_pe [Hkv][B][Skv][64]
  const __bf16* k_pe;
  int64_t k_pe_bs, k_pe_rs;
  float* ws_dkpe;
  // dS hand-over from the dK/dV kernel to the dQ kernel (head dims 128/128): bf16 images, 16 KB per
  // (batch, query head, 64-row query tile, 128-key block); ds_qt / ds_kb = number of such tiles / blocks.
  // Without a causal mask a head holds ds_qt x ds_kb of them, query tile by query tile; under the mask
  // only the blocks a tile can see are kept (tile t: its first t/2 + 1 key blocks, see ds_tile_start).
  // ds_hs = bytes per (batch, head).
  char* ds;
  int ds_qt, ds_kb;
  int64_t ds_hs;
  // dQ kernels, fp32 dq: query rows [final_r0, final_r1) (multiples of 32, or Sq) receive their result, old
  // contents of dq included when accumulating, as bf16 in dq_final instead of dq (nullptr: none do)
  __bf16* dq_final;
  int64_t dq_final_bs;
  int final_r0, final_r1;
  // dK/dV kernels: blocks main_blocks .. of the grid clear rows [Skv, Skv + zero_tail) of dk and dv
  int zero_tail, main_blocks;
  // dK/dV for head dims (128, 128), causal: launch the instance that visits the query tiles from the last one down
  int walk_desc;
};

constexpr int kZeroTailRows = 32;  // rows one such block clears

// The body of a dK/dV workgroup beyond the main grid: zero-fills its share of the rows behind the Skv rows the
// call computes (a ring step that sees only the first rows of a chunk owes the others a zero gradient).
// dk_feats: features per head of dk (128 when the keys come in two parts).
template <typename OutT>
__device__ __forceinline__ void zero_tail_block(const BwdParams& p, int idx, int dk_feats, int dv_feats, int tid, int threads) {
  const int r0 = p.Skv + idx * kZeroTailRows;
  const int rows = min(kZeroTailRows, p.Skv + p.zero_tail - r0);
  const u32x4 zero = {0u, 0u, 0u, 0u};
  constexpr int kPer16 = 16 / (int)sizeof(OutT);  // elements per 16-byte piece
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    OutT* base = reinterpret_cast<OutT*>(t == 0 ? p.dk : p.dv);
    const int64_t bs = t == 0 ? p.dk_bs : p.dv_bs;
    const int feats = t == 0 ? dk_feats : dv_feats;
    const int64_t row_stride = (int64_t)p.HkvT * feats;  // a row holds HkvT heads, Hkv of them belong to this call
    const int pieces = p.Hkv * feats / kPer16;
    const int total = p.B * rows * pieces;
    for (int i = tid; i < total; i += threads) {
      const int piece = i % pieces, rb = i / pieces;
      const int row = r0 + rb % rows, b = rb / rows;
      *reinterpret_cast<u32x4*>(base + b * bs + row * row_stride + (int64_t)piece * kPer16) = zero;
    }
  }
}

constexpr int kDsBlockBytes = 4 * 4096;  // one (query tile, key block): four wave-pair images
// Number of 16 KB blocks that precede query tile t within a head.
template <bool CAUSAL>
__host__ __device__ __forceinline__ int64_t ds_tile_start(int t, int ds_kb) {
  if (!CAUSAL) return (int64_t)t * ds_kb;
  const int64_t a = t >> 1;  // tiles 2a and 2a + 1 see a + 1 key blocks each
  return (t & 1) ? (a + 1) * (a + 1) : a * (a + 1);
}

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

// Stores a 32-row block of a result whose accumulators hold it UNtransposed: acc[o][v] is element
// (row acc_row(v, g), feature 32*o + c) for lane (c, g). For one v the 64 lanes cover two rows x 32 consecutive
// features: every instruction reads or writes whole 128-byte lines (fp32), where the transposed form (a lane owning
// one row and 4 consecutive features per access) touches 32 lines with 32 bytes each. `block` = row 0, feature 0 of
// the block; rows at or beyond `rows_valid` are skipped. With `accumulate` the old values of a batch of rows are all read before
// the batch's first store (row pointers may alias as far as the compiler can tell; it would chain load - store - load
// otherwise).
// With `final_block` (wave-uniform; the same rows of a bf16 tensor laid out like `block`) the result, old values included,
// is rounded to bf16 and written there, and `block` keeps what it held.
template <typename OutT, int NB>
__device__ __forceinline__ void store_rows32(OutT* block, int64_t row_stride, int rows_valid, const f32x16 (&acc)[NB],
                                             float factor, bool accumulate, int c, int g, __bf16* final_block = nullptr) {
#pragma clang fp contract(off)  // product rounded, then added: what accumulating into a separate tensor gives
  constexpr int kBatch = NB > 4 ? 4 : 8;  // accumulator elements per lane and batch: NB * kBatch old values in registers
  // a block wholly beyond the last row (wave-uniform): `block` itself is out of range, so not even the clamped
  // old-value loads may run
  if (rows_valid <= 0) return;
#pragma unroll
  for (int v0 = 0; v0 < 16; v0 += kBatch) {
    float old[kBatch][NB];
    if (accumulate) {
#pragma unroll
      for (int dv = 0; dv < kBatch; ++dv) {
        const int r = acc_row(v0 + dv, g);
        const OutT* src = block + (r < rows_valid ? r : 0) * row_stride + c;
#pragma unroll
        for (int o = 0; o < NB; ++o) old[dv][o] = (float)src[32 * o];
      }
    }
#pragma unroll
    for (int dv = 0; dv < kBatch; ++dv) {
      const int r = acc_row(v0 + dv, g);
      if (r < rows_valid) {
        OutT* dst = block + r * row_stride + c;
        __bf16* fin = final_block + r * row_stride + c;
#pragma unroll
        for (int o = 0; o < NB; ++o) {
          float x = acc[o][v0 + dv] * factor;
          if (accumulate) x += old[dv][o];
          if (final_block != nullptr) fin[32 * o] = (__bf16)x;
          else dst[32 * o] = (OutT)x;
        }
      }
    }
  }
}

// dK/dV kernels: linear block id -> (key tile, position within a level), a level being the `per_level` (kv head,
// batch, head part) combinations of one key tile; early key tiles first: under the causal mask they see the most
// query tiles. Each combination streams its own Q / dO tiles. With more than 8 of them and at least kChunkedTiles
// key tiles they are taken in chunks of 8, all key tiles of a chunk before the next chunk, so that the workgroups
// one XCD holds at a time (block id mod 8) belong to one combination and share its Q / dO stream through that
// XCD's L2 (see decode_block for the measurements behind the threshold).
__device__ __forceinline__ void decode_dkdv_block(int linear, int per_level, int tiles, int& n_tile, int& pos) {
  if (tiles >= kChunkedTiles && per_level > 8 && (per_level & 7) == 0) {
    const int per_chunk = 8 * tiles;
    const int c = linear / per_chunk;
    const int rem = linear - c * per_chunk;
    n_tile = rem >> 3;
    pos = c * 8 + (rem & 7);
  } else {
    n_tile = linear / per_level;
    pos = linear - n_tile * per_level;
  }
}

// dK/dV kernels: a workgroup owns kDkdvBlockN key rows (the grid and the head split depend on it).
constexpr int kDkdvBlockN = 128;
// dK/dV for head dims (128, 128): attn_bwd_dkdv_d128.hip. p.tiles, p.split, p.ws_* are set by the caller.
void launch_dkdv_d128(const BwdParams& p, bool causal, bool f32_out, unsigned grid, hipStream_t stream);

// dK/dV for head dims (192, 128): attn_bwd_dkdv_d192.hip. Same conventions.
void launch_dkdv_d192(const BwdParams& p, bool causal, bool f32_out, unsigned grid, hipStream_t stream);

// dQ for head dims (128, 128): attn_bwd_dq_d128.hip. p.tiles = number of 256-row query tiles.
void launch_dq_d128(const BwdParams& p, bool causal, bool f32_out, hipStream_t stream);

// dQ for head dims (128, 128) and (192, 128) with 128-row workgroups, early / late wave roles:
// attn_bwd_dq_direct.hip. p.tiles = number of 128-row query tiles.
void launch_dq_direct(const BwdParams& p, int dqk, bool causal, bool f32_out, hipStream_t stream);

// dQ for head dims (128, 128) from the dS images the dK/dV kernel left in p.ds: attn_bwd_dq_ds.hip.
// p.tiles = number of 512-row query tiles.
void launch_dq_from_ds(const BwdParams& p, bool causal, bool f32_out, hipStream_t stream);
// Bytes of dS images for a shape (0: the shape has no hand-over path).
int64_t ds_bytes_for(const pith_attn_bwd_args* a);

// Argument checks common to both entry points; returns PITH_OK or records the error.
int validate_bwd(const pith_attn_bwd_args* a, const char* who, bool need_dq, bool need_dkv);
BwdParams make_bwd_params(const pith_attn_bwd_args* a);

}  // namespace pith
