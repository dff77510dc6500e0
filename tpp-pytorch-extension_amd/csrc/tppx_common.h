// Shared host/device helpers of the gfx950 quantized-linear library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#include "tppx.h"

namespace tppx {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(16))) int i32x16;

// ---- error plumbing (host) ------------------------------------------------
int set_error(int code, const char* fmt, ...);
int check_hip(hipError_t e, const char* what);

#define TPPX_REQUIRE(cond, code, ...)          \
  do {                                         \
    if (!(cond))                               \
      return ::tppx::set_error(code, __VA_ARGS__); \
  } while (0)

// ---- launch plan recording (host) -------------------------------------------
// While a plan is being recorded (tppx_plan_linear_*), launch sites describe
// the kernel they would run and launch nothing.
bool plan_recording();
void plan_note(const void* kernel_fn, dim3 grid, dim3 block, size_t lds_bytes);
#define TPPX_PLAN_ONLY(kern, grid, block, lds)                                  \
  do {                                                                          \
    if (::tppx::plan_recording()) {                                             \
      ::tppx::plan_note(reinterpret_cast<const void*>(kern), grid, block, lds); \
      return hipSuccess;                                                        \
    }                                                                           \
  } while (0)

static inline bool aligned16(const void* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

// ---- bf16 <-> fp32 (device) -----------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) {
  return __uint_as_float(h << 16);
}

// round to nearest even, NaN kept quiet (same rule as the CPU side)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u)
    return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

__device__ __forceinline__ float round_bf16(float f) {
  return bf16_bits_to_f32(f32_to_bf16_bits(f));
}

// ---- post-ops on the bf16-rounded GEMM result -------------------------------
// `v` is bias + dot product in fp32.  The value is rounded to bf16 first and
// every post-op re-rounds where the CPU path stores its bf16 tile.
__device__ __forceinline__ uint32_t apply_post_bits(float v, int post,
                                                    uint32_t in1, uint32_t in2,
                                                    float scale) {
  uint32_t yb = f32_to_bf16_bits(v);
  float y = bf16_bits_to_f32(yb);
  switch (post) {
    case TPPX_POST_SILU: {
      // hardware exp2 / reciprocal: their error (about 1e-7 relative) is far below the bf16 rounding that follows,
      // and the full-precision expf + divide cost as much as 30 MFMA issue slots per output in the prefill epilogue
      float s = round_bf16(__frcp_rn(1.0f + __expf(-y)));
      return f32_to_bf16_bits(y * s);
    }
    case TPPX_POST_MUL:
      return f32_to_bf16_bits(bf16_bits_to_f32(in1) * y);
    case TPPX_POST_ADD_SCALE:
      return f32_to_bf16_bits(fmaf(bf16_bits_to_f32(in1), scale, y));
    case TPPX_POST_ADD2_SCALE: {
      float t = round_bf16(y + bf16_bits_to_f32(in1));
      return f32_to_bf16_bits(fmaf(bf16_bits_to_f32(in2), scale, t));
    }
    case TPPX_POST_GELU:
      return f32_to_bf16_bits(0.5f * y * (1.0f + erff(y * 0.70710678118654752f)));
    case TPPX_POST_RELU:
      return (yb & 0x8000u) ? 0u : yb;
    default:
      return yb;
  }
}

// E8M0 byte -> fp32 factor used when de-quantising (byte shifted into the
// exponent field; 0 gives 0.0, 255 gives +Inf).
__device__ __forceinline__ float e8m0_to_f32(uint32_t x) {
  return __uint_as_float((x & 0xffu) << 23);
}

// compile-time loop: f(std::integral_constant<int, I>) for I in [B, E)
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(std::integral_constant<int, B>{});
    static_for<B + 1, E>(f);
  }
}

// W4A8 (USE_MXFP4_INT8): the integer the reference multiplies for an E2M1 code = its value times 127 / 6, rounded
// four 4-bit E2M1 codes (one per byte, bits 0..3) -> four int8 values
__device__ __forceinline__ uint32_t w4a8_expand(uint32_t codes) {
  const uint32_t sel = codes & 0x07070707u;
  // v_perm_b32: selector bytes 0..3 pick from the second operand, 4..7 from the first
  const uint32_t pos = __builtin_amdgcn_perm(0x7F55402Au, 0x20150B00u, sel); // 0 11 21 32 | 42 64 85 127
  const uint32_t neg = __builtin_amdgcn_perm(0x81ABC0D6u, 0xE0EBF500u, sel); // the same, negated
  const uint32_t m = ((codes >> 3) & 0x01010101u) * 0xFFu;                   // 0xFF in the bytes with the sign bit
  return (neg & m) | (pos & ~m);
}

} // namespace tppx
