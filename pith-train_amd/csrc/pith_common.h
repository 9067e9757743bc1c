// Shared declarations of libpith_hip.so (host side + small device helpers).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "pith_hip.h"

namespace pith {

// Records `msg` (printf-style) as the calling thread's last error and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// Launch status of an entry point: begin_launch() discards an error an earlier runtime call of
// the host program may have left behind on this thread (it belongs to that call, and would
// otherwise be reported against ours); check_launch() then reads the status of the launches made
// since and returns PITH_OK or PITH_ERR_LAUNCH.
void begin_launch();
int check_launch(const char* what);

// Compute units of the current device (looked up once per device; 0 if the runtime cannot tell).
int compute_units();
// The same for launch heuristics: 256 (an MI355X) when the runtime cannot tell.
inline int compute_units_or_default() {
  const int n = compute_units();
  return n > 0 ? n : 256;
}

// Work split of the query-stationary direct-load kernels (forward, dQ): true = 128-row workgroups.
bool prefer_half_rows(int64_t Sq, int64_t Hq, int64_t B, bool causal);

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;

// bf16 bit pattern -> fp32 (exact).
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }
__device__ __forceinline__ float bf16lo_to_f32(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t packed) { return __uint_as_float(packed & 0xffff0000u); }

// Two fp32 -> packed bf16 pair (lo = a, hi = b), round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  bf16x2 v;
  v[0] = (__bf16)a;
  v[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, v);
}

}  // namespace pith
