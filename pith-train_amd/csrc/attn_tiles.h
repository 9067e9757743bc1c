// Device building blocks shared by the attention kernels (forward, dQ, dK/dV) on gfx950.
//
// Matrix-core conventions used everywhere (v_mfma_f32_32x32x16_bf16, one wavefront of 64 lanes,
// lane = 32*g + c with c = lane % 32, g = lane / 32):
//   A operand (32 x 16): lane holds row c, contraction slots k = 8*g + e, e = 0..7
//   B operand (16 x 32): lane holds column c, the same contraction slots
//   C/D      (32 x 32): lane holds column c, rows 8*(v/4) + 4*g + v%4, v = 0..15
// A result tile can therefore be fed back as the B operand of a product that contracts over
// its ROW index without leaving registers: slot (g, e) of contraction step j then stands for
// row 16*j + 8*(e/4) + 4*g + e%4 of the tile ("slot order"). The other operand of that product
// is fetched from LDS in the same slot order.
//
// Tiles streamed through LDS are row-major [row][col] bf16 with a padded pitch. They are read
//   - "straight": lane takes 8 consecutive columns of row c            (one ds_read_b128), or
//   - "transposed": lane takes column c at 8 rows in slot order         (two ds_read_b64_tr_b16).
#pragma once

#include "pith_common.h"

namespace pith {

typedef __attribute__((address_space(3))) char lds_char;

__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// Straight A/B fragment: row `row`, columns col0 .. col0+7 (col0 multiple of 8).
__device__ __forceinline__ bf16x8 lds_read_straight(const char* tile, int pitch, int row, int col0) {
  return *reinterpret_cast<const bf16x8*>(tile + row * pitch + col0 * 2);
}

// Transposed fragment in slot order. For a wavefront the result is the A (or B) operand whose
// non-contracted index is the tile COLUMN col_base + c and whose contraction slots (g, e) are
// the tile ROWS row_base + 8*(e/4) + 4*g + e%4.
// ds_read_b64_tr_b16 works on blocks of 16 lanes: lane r of a block supplies the address of 4
// consecutive columns; lanes 4i..4i+3 of the block must cover 16 consecutive columns of row i;
// lane r then receives column r of rows 0..3 of the block.
__device__ __forceinline__ bf16x8 lds_read_transposed(const char* tile, int pitch, int row_base, int col_base,
                                                      int lane) {
  const int r = lane & 15, blk = lane >> 4;
  const int row = row_base + 4 * (blk >> 1) + (r >> 2);
  const int col = col_base + 16 * (blk & 1) + 4 * (r & 3);
  const char* p = tile + row * pitch + col * 2;
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p + 8 * pitch));
  typedef __attribute__((ext_vector_type(8))) short s16x8;
  s16x8 v;
  v[0] = lo[0]; v[1] = lo[1]; v[2] = lo[2]; v[3] = lo[3];
  v[4] = hi[0]; v[5] = hi[1]; v[6] = hi[2]; v[7] = hi[3];
  return __builtin_bit_cast(bf16x8, v);
}

// Row index (0..31) inside a 32x32 result tile of accumulator element v for lane group g.
__device__ __forceinline__ int acc_row(int v, int g) { return 8 * (v >> 2) + 4 * g + (v & 3); }

// max / sum across the two lanes (c, c+32) that share a result column.
__device__ __forceinline__ float pair_max(float x) {
  const int xi = __float_as_int(x);
  const auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
  return fmaxf(__int_as_float(r[0]), __int_as_float(r[1]));
}
__device__ __forceinline__ float pair_sum(float x) {
  const int xi = __float_as_int(x);
  const auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
  return __int_as_float(r[0]) + __int_as_float(r[1]);
}

// Eight fp32 accumulator values -> bf16 fragment (round-to-nearest-even).
__device__ __forceinline__ bf16x8 to_bf16x8(float a0, float a1, float a2, float a3, float a4, float a5, float a6,
                                            float a7) {
  bf16x8 r;
  r[0] = (__bf16)a0; r[1] = (__bf16)a1; r[2] = (__bf16)a2; r[3] = (__bf16)a3;
  r[4] = (__bf16)a4; r[5] = (__bf16)a5; r[6] = (__bf16)a6; r[7] = (__bf16)a7;
  return r;
}

// Waits until every vector-memory load issued so far has returned. Placed once before a main
// loop, after the loop-invariant fragments were fetched: otherwise the compiler keeps the waits
// for those fragments inside the loop, where they also wait for the loads that prefetch the next
// tile and so expose the global-memory latency in every iteration.
__device__ __forceinline__ void wait_all_vector_loads() {
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), expcnt and lgkmcnt left at their maxima
}

// Maps a linear workgroup id to (tile, head, batch) so that
//   - tiles are visited from `tiles-1` down to 0 (under a causal mask the late tiles carry the most work, and
//     the lightest workgroups should be the last ones dispatched);
//   - workgroups are dealt round-robin to the 8 XCDs of the device, each with its own L2: the
//     heads of one level are permuted so that an XCD keeps a contiguous range of heads, i.e. the
//     query heads that share a kv head read their K/V through the same L2;
//   - with more than 8 kv heads per level (`group` = query heads per kv head) and at least kChunkedTiles tiles
//     the heads are taken in chunks of 8 kv heads, all tiles of a chunk before the next chunk: the workgroups an
//     XCD holds at one time then belong to ONE kv head and stream the same K/V tiles at about the same time,
//     instead of one stream per head. Each chunk ends with its light tiles, so the order is no longer
//     heaviest-first over the whole grid: measured 9-14 % faster at 128 heads x 32768 rows, 2-6 % slower at 4096
//     rows (16-32 tiles), hence the threshold.
constexpr int kChunkedTiles = 64;
__device__ __forceinline__ void decode_block(int linear, int heads, int batch, int tiles, int group, int& tile, int& h, int& b) {
  const int per_level = heads * batch;
  const int chunk = 8 * group;
  int level, pos;
  if (tiles >= kChunkedTiles && per_level > chunk && per_level % chunk == 0) {
    const int per_chunk = chunk * tiles;
    const int c = linear / per_chunk;
    const int rem = linear - c * per_chunk;
    level = rem / chunk;
    const int u = rem - level * chunk;
    pos = c * chunk + (u & 7) * group + (u >> 3);
  } else {
    level = linear / per_level;
    pos = linear - level * per_level;
    if ((per_level & 7) == 0) pos = (pos & 7) * (per_level >> 3) + (pos >> 3);
  }
  tile = tiles - 1 - level;
  b = pos / heads;
  h = pos - b * heads;
}

// Cooperative copy of a [ROWS x COLS] bf16 tile between global memory and LDS by THREADS threads,
// split into a "fetch to registers" half and a "store to LDS" half so that the global loads of
// the next tile can be in flight while the current tile is consumed.
template <int ROWS, int COLS, int PITCH, int THREADS>
struct TileCopy {
  static constexpr int kChunksPerRow = COLS / 8;
  static constexpr int kChunks = ROWS * kChunksPerRow;
  static constexpr int kPerThread = (kChunks + THREADS - 1) / THREADS;
  u32x4 regs[kPerThread];

  // src: address of element [row 0][col 0] of the tile's head slice; row_stride in elements;
  // rows at or beyond `valid_rows` are read from the last valid row (their values are masked
  // or discarded by the caller).
  __device__ __forceinline__ void fetch(const __bf16* src, int64_t row_stride, int row0, int valid_rows, int tid) {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const int c = tid + i * THREADS;
      if (kChunks % THREADS == 0 || c < kChunks) {
        const int row = c / kChunksPerRow, col = c - row * kChunksPerRow;
        int grow = row0 + row;
        grow = grow < valid_rows ? grow : valid_rows - 1;
        regs[i] = *reinterpret_cast<const u32x4*>(src + grow * row_stride + col * 8);
      }
    }
  }
  __device__ __forceinline__ void commit(char* tile, int tid) const {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const int c = tid + i * THREADS;
      if (kChunks % THREADS == 0 || c < kChunks) {
        const int row = c / kChunksPerRow, col = c - row * kChunksPerRow;
        *reinterpret_cast<u32x4*>(tile + row * PITCH + col * 16) = regs[i];
      }
    }
  }
};

// ---------------------------------------------------------------------------------------------
// 128-feature tiles moved global memory -> LDS directly (global_load_lds_dwordx4), without
// passing through registers. One wavefront instruction moves 64 pieces of 16 bytes to 1 KB of
// consecutive LDS (lane L -> byte 16*L of the region), so tile rows are packed at 256 bytes
// (16 pieces) with no padding; bank conflicts are avoided by keeping piece q of row r at
// position q ^ tile_swizzle(r). The swizzle is a bijection of r % 16 (16 consecutive rows read
// "straight" at one feature offset hit 16 different positions) and moves rows r..r+3 to four
// different 64-byte groups (what the transposing read touches at once).
constexpr int kRowBytes128 = 256;

__device__ __forceinline__ int tile_swizzle(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }

// Byte offset inside a packed tile of the 16-byte piece `piece` (0..15) of row `row`.
__device__ __forceinline__ int swizzled_offset(int row, int piece) {
  return row * kRowBytes128 + ((piece ^ tile_swizzle(row)) << 4);
}

// 16 bytes per lane from global address `base` + `offset` (base the same for all lanes, offset
// per lane, unsigned) to LDS at `dst_wave` + 16 * lane; `dst_wave` must be the same for all lanes
// of the wavefront. Completion is tracked by vmcnt, in issue order with the other vector loads.
// Written as inline assembly on purpose: the compiler does not see an LDS write, so it places no
// wait between this load and later LDS reads of OTHER tiles; the caller waits (s_waitcnt vmcnt)
// and synchronises the workgroup before anyone reads the destination.
// The statement overwrites M0 behind the compiler's back: M0 is a reserved register that cannot
// be declared as clobbered (clang warns that such a declaration is not honoured). That is sound
// only while the compiler itself emits no M0 use in a kernel that includes this header (dynamic
// register indexing, s_sendmsg, LDS-DMA or GWS builtins would); tests/test_cabi.py compiles every
// source to assembly and fails if M0 appears anywhere outside these inline statements.
__device__ __forceinline__ void load_lds16(const char* base, int offset, char* dst_wave) {
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lds_char*)dst_wave;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(offset), "s"(base)
               : "memory");
}

// 4 bytes per lane from the per-lane global address `src` to LDS at `dst_wave` + 4 * lane (same
// conventions as load_lds16).
__device__ __forceinline__ void load_lds4(const void* src, char* dst_wave) {
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lds_char*)dst_wave;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"
               :
               : "s"(lds_addr), "v"(src)
               : "memory");
}

// Moves a [ROWS x 128] bf16 tile with THREADS threads (THREADS / 64 wavefronts): wavefront w
// moves the 4 tile rows of every 1 KB region n * WAVES + w. With 4 * WAVES a multiple of 16 the
// swizzle of a lane's row is the same in every region, so one per-lane source offset serves all
// regions and the region only moves the (uniform) source address on.
template <int ROWS, int THREADS>
struct DirectTile128 {
  static constexpr int kWaves = THREADS / 64;
  static constexpr int kPerThread = ROWS * 16 / THREADS;
  static_assert(ROWS * 16 % THREADS == 0, "tile must split evenly over the threads");
  static_assert((4 * kWaves) % 16 == 0, "rows of successive regions must share their swizzle");
  static constexpr int kTileBytes = ROWS * kRowBytes128;
  int src_off;  // byte offset of this lane's source piece in region 0 from the tile's first row
  int row_bytes;

  // row_bytes: distance between consecutive rows in global memory, in bytes
  __device__ __forceinline__ void init(int row_bytes_, int wave, int lane) {
    row_bytes = row_bytes_;
    const int row = 4 * wave + (lane >> 4);
    src_off = row * row_bytes + (((lane & 15) ^ tile_swizzle(row)) << 4);
  }
  // tile_src: address of [first row of the tile][feature 0] of the head slice (uniform);
  // rows_left: valid rows from there on (>= 1), rows beyond are read from the last valid row.
  // `slot` is the LDS tile (uniform).
  __device__ __forceinline__ void issue(const char* tile_src, int rows_left, char* slot, int wave, int lane) const {
    if (rows_left >= ROWS) {
      // The offset is pinned in a register BEFORE the first load is issued: were it spilled, the
      // compiler would reload it between two loads and wait for the reload with a counter wait that
      // also waits for every tile load issued before it.
      int off = src_off;
      asm volatile("" : "+v"(off));
#pragma unroll
      for (int n = 0; n < kPerThread; ++n)
        load_lds16(tile_src + (int64_t)n * 4 * kWaves * row_bytes, off, slot + (n * kWaves + wave) * 1024);
    } else {
#pragma unroll
      for (int n = 0; n < kPerThread; ++n) {
        const int row = 4 * (n * kWaves + wave) + (lane >> 4);
        const int src_row = row < rows_left ? row : rows_left - 1;
        load_lds16(tile_src, src_row * row_bytes + (((lane & 15) ^ tile_swizzle(row)) << 4),
                   slot + (n * kWaves + wave) * 1024);
      }
    }
  }
};

// ---------------------------------------------------------------------------------------------
// Features 128..191 of a 64-row tile of a 192-feature operand (the MLA key / query): a second
// packed tile that holds TWO tile rows per 256-byte LDS row, row r in pieces 0-7 and row r + 32
// in pieces 8-15 of LDS row r (r < 32), under the same swizzle. Read like a 32-row, 128-feature
// tile whose features 64..127 are the second 32-row block: a straight fragment of row block kb,
// row c, contraction step x (0..3) is piece 2x + g + 8*kb of LDS row c; a transposed fragment of
// row block kb, feature block f (0..1) uses col_base = 64*kb + 32*f.
constexpr int kExtraTileBytes = 32 * kRowBytes128;

// Moves that part of a tile global memory -> LDS: one global_load_lds per thread of a 512-thread
// workgroup (wave w fills LDS rows 4w .. 4w+3). Source rows are 384 bytes of features per head.
struct DirectExtra64 {
  int src_off, row_bytes, col_bytes;
  __device__ __forceinline__ static int source(int row_bytes, int col_bytes, int wave, int lane, int rows_left) {
    const int row = 4 * wave + (lane >> 4);
    const int piece = (lane & 15) ^ tile_swizzle(row);
    int key = row + 32 * (piece >> 3);
    key = key < rows_left ? key : rows_left - 1;
    return key * row_bytes + col_bytes + ((piece & 7) << 4);
  }
  // row_bytes: distance between consecutive source rows; col_bytes: where the 64 features start
  // within a source row (256 when they follow the first 128 features of the same row, 0 when they
  // are a tensor of their own)
  __device__ __forceinline__ void init(int row_bytes_, int col_bytes_, int wave, int lane) {
    row_bytes = row_bytes_;
    col_bytes = col_bytes_;
    src_off = source(row_bytes_, col_bytes_, wave, lane, 64);
  }
  __device__ __forceinline__ void issue(const char* tile_src, int rows_left, char* slot, int wave, int lane) const {
    if (rows_left >= 64) load_lds16(tile_src, src_off, slot + wave * 1024);
    else load_lds16(tile_src, source(row_bytes, col_bytes, wave, lane, rows_left), slot + wave * 1024);
  }
};

// Per-lane offsets for reading a packed swizzled tile.
// straight_offset(c, piece): fragment of row c (+ a multiple of 16 rows added by the caller as
// rows * 256 bytes), features 8*piece .. 8*piece+7.
__device__ __forceinline__ int straight_offset128(int row, int piece) { return swizzled_offset(row, piece); }

// Offset for one ds_read_b64_tr_b16 of a transposed fragment (see lds_read_transposed): tile
// rows row_base + 8*half + 4*(blk>>1) + (r>>2), features col_base + 16*(blk&1) + 4*(r&3) .. +3.
// row_base must be a multiple of 16, col_base a multiple of 32.
__device__ __forceinline__ int transposed_offset128(int row_base, int half, int col_base, int lane) {
  const int r = lane & 15, blk = lane >> 4;
  const int row = row_base + 8 * half + 4 * (blk >> 1) + (r >> 2);
  const int col = col_base + 16 * (blk & 1) + 4 * (r & 3);  // features
  return swizzled_offset(row, col >> 3) + ((col & 7) << 1);
}

__device__ __forceinline__ bf16x8 lds_read_transposed_at(const char* lo_addr, const char* hi_addr) {
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(lo_addr));
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(hi_addr));
  typedef __attribute__((ext_vector_type(8))) short s16x8;
  s16x8 v;
  v[0] = lo[0]; v[1] = lo[1]; v[2] = lo[2]; v[3] = lo[3];
  v[4] = hi[0]; v[5] = hi[1]; v[6] = hi[2]; v[7] = hi[3];
  return __builtin_bit_cast(bf16x8, v);
}

// ---------------------------------------------------------------------------------------------
// Epilogue of the kernels whose accumulators hold their result TRANSPOSED (a lane owns one result
// row, its registers 4-feature pieces of it: accT[o][v] = R[row c][feature 32*o + acc_row(v, g)] for lane
// (c, g)). Written straight from that layout a store instruction touches 32 rows with 16 or 32 bytes
// each, i.e. 32 memory lines, and a compute unit's vector cache keeps only about 64 requests in flight;
// turned through LDS first, every instruction reads or writes whole rows (2 rows x 512 bytes of fp32 per
// instruction at 128 features). `lds` is a wave-private area of kRowsViaLdsBytes<NB> bytes (the tile
// rings are free by then: the caller has passed the barrier behind their last reader); `factor` is this
// lane's (= this row's) scale; rows at or beyond rows_valid are neither read nor written (rows_valid may be <= 0).
// With `accumulate` all old values are read before the first store. With `final_block` (wave-uniform; the same rows of
// a bf16 tensor laid out like `block`) the result, old values included, is rounded to bf16 and written there, and
// `block` keeps what it held.
template <int NB>
constexpr int kRowsViaLdsBytes = 32 * (NB * 128 + 16);

template <typename OutT, int NB>
__device__ __forceinline__ void store_rows32_via_lds(char* lds, OutT* block, int64_t row_stride, int rows_valid,
                                                     const f32x16 (&accT)[NB], float factor, bool accumulate, int lane,
                                                     __bf16* final_block = nullptr) {
#pragma clang fp contract(off)  // product rounded, then added: what accumulating into a separate tensor gives
  constexpr int kPitch = NB * 128 + 16;  // bytes; the 16 spread the 32 rows of a column over the banks
  constexpr int kPieces = NB * 8;        // 16-byte pieces (4 features) per row
  constexpr int kIters = 32 * kPieces / 64;
  // a block that lies wholly beyond the last row (the same for the whole wave): nothing to store, and the
  // clamped old-value loads below would start from `block`, which is itself out of range then
  if (rows_valid <= 0) return;
  const int c = lane & 31, g = lane >> 5;
#pragma unroll
  for (int o = 0; o < NB; ++o)
#pragma unroll
    for (int b4 = 0; b4 < 4; ++b4) {
      const f32x4 x = {accT[o][4 * b4] * factor, accT[o][4 * b4 + 1] * factor, accT[o][4 * b4 + 2] * factor,
                       accT[o][4 * b4 + 3] * factor};
      *reinterpret_cast<f32x4*>(lds + c * kPitch + (32 * o + 8 * b4 + 4 * g) * 4) = x;
    }
  // the reads below see the writes above: one wave's LDS operations execute in order
  f32x4 val[kIters];
  int row[kIters], piece[kIters];
#pragma unroll
  for (int it = 0; it < kIters; ++it) {
    const int idx = it * 64 + lane;
    row[it] = idx / kPieces;
    piece[it] = idx - row[it] * kPieces;
    val[it] = *reinterpret_cast<const f32x4*>(lds + row[it] * kPitch + piece[it] * 16);
  }
  if (accumulate) {
#pragma unroll
    for (int it = 0; it < kIters; ++it) {
      const OutT* src = block + (row[it] < rows_valid ? row[it] : 0) * row_stride + 4 * piece[it];
      if constexpr (sizeof(OutT) == 4) {
        val[it] += *reinterpret_cast<const f32x4*>(src);
      } else {
        const u32x2 old = *reinterpret_cast<const u32x2*>(src);
        val[it][0] += bf16lo_to_f32(old[0]);
        val[it][1] += bf16hi_to_f32(old[0]);
        val[it][2] += bf16lo_to_f32(old[1]);
        val[it][3] += bf16hi_to_f32(old[1]);
      }
    }
  }
  if (final_block != nullptr) {
#pragma unroll
    for (int it = 0; it < kIters; ++it) {
      if (row[it] < rows_valid) {
        u32x2 w;
        w[0] = pack_bf16x2(val[it][0], val[it][1]);
        w[1] = pack_bf16x2(val[it][2], val[it][3]);
        *reinterpret_cast<u32x2*>(final_block + row[it] * row_stride + 4 * piece[it]) = w;
      }
    }
    return;
  }
#pragma unroll
  for (int it = 0; it < kIters; ++it) {
    if (row[it] < rows_valid) {
      OutT* dst = block + row[it] * row_stride + 4 * piece[it];
      if constexpr (sizeof(OutT) == 4) {
        *reinterpret_cast<f32x4*>(dst) = val[it];
      } else {
        u32x2 w;
        w[0] = pack_bf16x2(val[it][0], val[it][1]);
        w[1] = pack_bf16x2(val[it][2], val[it][3]);
        *reinterpret_cast<u32x2*>(dst) = w;
      }
    }
  }
}

// The same turn through LDS for the forward kernel's merging epilogue: row r of the block becomes
//     f_new[r] * accT[r] + f_old[r] * prev[r]
// (the online-softmax combine of the chunk result in the accumulators with the running result `prev`, bf16 or fp32,
// whose per-row weights the caller has formed from the two LSEs) and is written as bf16 to `out_bf16` and / or as fp32
// to `out_f32` (either may be null, either may alias `prev`: a lane reads the old values of a piece before it writes
// that piece, and no other lane touches it). f_new / f_old are this lane's (= this row's) weights; the old weight
// travels to the lanes that handle the row's pieces through the 16 bytes of padding behind the row in LDS.
// All three tensors are addressed from row 0 of the block, feature 0 of the head.
template <int NB>
__device__ __forceinline__ void merge_rows32_via_lds(char* lds, const void* prev, bool prev_f32, int64_t prev_row_stride,
                                                     __bf16* out_bf16, int64_t out_row_stride, float* out_f32,
                                                     int64_t acc_row_stride, int rows_valid, const f32x16 (&accT)[NB],
                                                     float f_new, float f_old, int lane) {
  constexpr int kPitch = NB * 128 + 16;
  constexpr int kPieces = NB * 8;
  constexpr int kIters = 32 * kPieces / 64;
  if (rows_valid <= 0) return;  // wave-uniform
  const int c = lane & 31, g = lane >> 5;
  // the running values first: their memory latency then overlaps the turn through LDS (the accumulators are still
  // live, which the epilogue can afford)
  f32x4 old[kIters];
  int row[kIters], piece[kIters];
#pragma unroll
  for (int it = 0; it < kIters; ++it) {
    const int idx = it * 64 + lane;
    row[it] = idx / kPieces;
    piece[it] = idx - row[it] * kPieces;
    const int src_row = row[it] < rows_valid ? row[it] : 0;
    if (prev_f32) {
      old[it] = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(prev) + src_row * prev_row_stride + 4 * piece[it]);
    } else {
      const u32x2 w = *reinterpret_cast<const u32x2*>(reinterpret_cast<const __bf16*>(prev) + src_row * prev_row_stride + 4 * piece[it]);
      old[it] = f32x4{bf16lo_to_f32(w[0]), bf16hi_to_f32(w[0]), bf16lo_to_f32(w[1]), bf16hi_to_f32(w[1])};
    }
  }
#pragma unroll
  for (int o = 0; o < NB; ++o)
#pragma unroll
    for (int b4 = 0; b4 < 4; ++b4) {
      const f32x4 x = {accT[o][4 * b4] * f_new, accT[o][4 * b4 + 1] * f_new, accT[o][4 * b4 + 2] * f_new,
                       accT[o][4 * b4 + 3] * f_new};
      *reinterpret_cast<f32x4*>(lds + c * kPitch + (32 * o + 8 * b4 + 4 * g) * 4) = x;
    }
  if (g == 0) *reinterpret_cast<float*>(lds + c * kPitch + NB * 128) = f_old;
  // the reads below see the writes above: one wave's LDS operations execute in order
#pragma unroll
  for (int it = 0; it < kIters; ++it) {
    const f32x4 val = *reinterpret_cast<const f32x4*>(lds + row[it] * kPitch + piece[it] * 16);
    const float fo = *reinterpret_cast<const float*>(lds + row[it] * kPitch + NB * 128);
    if (row[it] >= rows_valid) continue;
    const f32x4 r = val + old[it] * fo;
    if (out_f32) *reinterpret_cast<f32x4*>(out_f32 + row[it] * acc_row_stride + 4 * piece[it]) = r;
    if (out_bf16) {
      u32x2 w;
      w[0] = pack_bf16x2(r[0], r[1]);
      w[1] = pack_bf16x2(r[2], r[3]);
      *reinterpret_cast<u32x2*>(out_bf16 + row[it] * out_row_stride + 4 * piece[it]) = w;
    }
  }
}

}  // namespace pith
