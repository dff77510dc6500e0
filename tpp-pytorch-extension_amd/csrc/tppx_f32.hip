// QINT8-family linear with fp32 output: the path of float / half activations and of pre-quantized activations whose
// compute type is float (fc_plain_wrap's element-type switch, src/csrc/llm/fused_llm_infer.cpp:1526-1545, on
// TppBlockedQInt8LinearW<float, uint8_t, float>, src/csrc/fused_gemm.h:1076-1341).  The caller quantizes the
// activations (int8 [M][K] row-major + f32 [M][K/qbs], quantize_int8sym of fused_gemm.h:1248); this kernel does
//   y[m][n] = bias[n] + sum_b float(sum_{k in b} xq[m][k] * wq[n][k]) * (sa[m][b] * sw[n][b])
// one fused multiply-add per K block in ascending block order, nothing rounded below fp32.
// It is the seldom-used wide-output path, kept simple: one wave owns a 16 x 16 output tile over the whole K (so the
// sum order is the formula's), four waves = 64 rows share a workgroup's weight tile stream through the caches.
#include <hip/hip_runtime.h>

#include "tppx.h"
#include "tppx_common.h"

namespace tppx {

struct F32OutParams {
  const int8_t* xq; // [M][K]
  const float* sa;  // [M][K/qbs]
  const void* qw;   // native tiles [N/16][K/64][64 lanes][16 B]
  const float* sw;  // native scales [N/16][K/qbs][16]
  const float* bias; // [N] or null
  float* y;          // [M][N]
  int M, N, K, qbs;
};

__global__ void __launch_bounds__(256)
linear_qint8_f32_kernel(const F32OutParams p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = blockIdx.x, m0 = (blockIdx.y * 4 + wave) * 16;
  if (m0 >= p.M) // whole waves only; no barrier below
    return;
  const int KT = p.K / 64, NB = p.K / p.qbs, TPB = p.qbs / 64;
  const i32x4* wq = reinterpret_cast<const i32x4*>(p.qw) + (int64_t)tile * KT * 64 + lane;
  const float* sw = p.sw + (int64_t)tile * NB * 16 + (lane & 15);
  // A operand: row lane & 15 (rows past M re-read the last one, never stored), K group lane >> 4
  const int8_t* xr = p.xq + (int64_t)min(m0 + (lane & 15), p.M - 1) * p.K + (lane >> 4) * 16;
  // result rows (lane >> 4) * 4 + r, column lane & 15
  const int n = tile * 16 + (lane & 15);
  float f[4];
  const float* sar[4];
#pragma unroll
  for (int r = 0; r < 4; r++) {
    f[r] = p.bias ? p.bias[n] : 0.f;
    sar[r] = p.sa + (int64_t)min(m0 + (lane >> 4) * 4 + r, p.M - 1) * NB;
  }
  for (int b = 0; b < NB; b++) {
    i32x4 acc = {0, 0, 0, 0};
    for (int t = b * TPB; t < (b + 1) * TPB; t++)
      acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(*reinterpret_cast<const i32x4*>(xr + (int64_t)t * 64), wq[(int64_t)t * 64], acc, 0, 0, 0);
    const float swv = sw[b * 16];
#pragma unroll
    for (int r = 0; r < 4; r++)
      f[r] = fmaf((float)acc[r], sar[r][b] * swv, f[r]);
  }
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const int m = m0 + (lane >> 4) * 4 + r;
    if (m < p.M)
      p.y[(int64_t)m * p.N + n] = f[r];
  }
}

// ---------------------------------------------------------------------------
// float / half activations on MXFP4 or unquantized bf16 weights: TppBlockedLinearW<Tin, uint8_t, Tout> /
// <Tin, bfloat16, Tout> with Tin = float or half (the element-type switch of fc_plain_wrap,
// src/csrc/llm/fused_llm_infer.cpp:1526-1545, dispatched in src/csrc/fused_gemm.h:1519-1523, 1541-1550).  The
// activations keep their own precision (no rounding to bf16): every weight value is exact in fp32 (E2M1 code times a
// power of two, or a bf16), the products run on the fp32 MFMA (16 x 16 x 4) and are summed in fp32:
//   y[m][n] = bias[n] + sum_k x[m][k] * w[n][k]          (fp32; the caller rounds / applies the post-op)
// Both native layouts give lane (g, n) of a 128-channel K tile the 32 weights k = g*32 .. g*32 + 31 of channel n, and
// MFMA step i multiplies the four channels k = g*32 + i (one per K group g).  One wave per 16 x 16 output tile, four
// waves (64 rows) per workgroup share the weight tile through the caches: the seldom-used wide path, kept simple.
// ---------------------------------------------------------------------------
struct WideParams {
  const void* x;     // [M][K] fp32 or fp16
  const void* qw;    // native tiles
  const uint8_t* sw; // MXFP4: native scale bytes [N/16][K/128][64]
  const float* bias; // [N] or null
  float* y;          // [M][N]
  int M, N, K;
};

template <bool XHALF, bool WBF16>
__global__ void __launch_bounds__(256)
linear_wide_kernel(const WideParams p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = blockIdx.x, m0 = (blockIdx.y * 4 + wave) * 16;
  if (m0 >= p.M) // whole waves only; no barrier below
    return;
  const int KT = p.K / 128, g = lane >> 4;
  const int64_t row = min(m0 + (lane & 15), p.M - 1); // rows past M re-read the last one, never stored
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int kt = 0; kt < KT; kt++) {
    float w[32], xv[32];
    if (WBF16) {
      const i32x4* wq = reinterpret_cast<const i32x4*>(p.qw) + ((int64_t)tile * KT + kt) * 256 + lane;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const i32x4 v = wq[j * 64];
#pragma unroll
        for (int d = 0; d < 4; d++) {
          w[j * 8 + 2 * d] = bf16_bits_to_f32((uint32_t)v[d] & 0xffffu);
          w[j * 8 + 2 * d + 1] = bf16_bits_to_f32((uint32_t)v[d] >> 16);
        }
      }
    } else {
      const int64_t slot = ((int64_t)tile * KT + kt) * 64 + lane;
      const i32x4 v = reinterpret_cast<const i32x4*>(p.qw)[slot];
      const float sc = e8m0_to_f32(p.sw[slot]);
      typedef __attribute__((ext_vector_type(2))) float f32x2;
#pragma unroll
      for (int d = 0; d < 4; d++) {
        const uint32_t c = (uint32_t)v[d]; // 8 codes; byte h holds codes 2h and 2h + 1
        const f32x2 p0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, sc, 0);
        const f32x2 p1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, sc, 1);
        const f32x2 p2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, sc, 2);
        const f32x2 p3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, sc, 3);
        w[d * 8 + 0] = p0[0]; w[d * 8 + 1] = p0[1]; w[d * 8 + 2] = p1[0]; w[d * 8 + 3] = p1[1];
        w[d * 8 + 4] = p2[0]; w[d * 8 + 5] = p2[1]; w[d * 8 + 6] = p3[0]; w[d * 8 + 7] = p3[1];
      }
    }
    if (XHALF) {
      const i32x4* xr = reinterpret_cast<const i32x4*>(reinterpret_cast<const _Float16*>(p.x) + row * p.K + kt * 128 + g * 32);
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const i32x4 v = xr[c];
#pragma unroll
        for (int d = 0; d < 4; d++) {
          const uint32_t u = (uint32_t)v[d];
          xv[c * 8 + 2 * d] = (float)__builtin_bit_cast(_Float16, (uint16_t)(u & 0xffffu));
          xv[c * 8 + 2 * d + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(u >> 16));
        }
      }
    } else {
      const f32x4* xr = reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(p.x) + row * p.K + kt * 128 + g * 32);
#pragma unroll
      for (int c = 0; c < 8; c++) {
        const f32x4 v = xr[c];
        xv[c * 4] = v[0]; xv[c * 4 + 1] = v[1]; xv[c * 4 + 2] = v[2]; xv[c * 4 + 3] = v[3];
      }
    }
#pragma unroll
    for (int i = 0; i < 32; i++)
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[i], w[i], acc, 0, 0, 0);
  }
  const int n = tile * 16 + (lane & 15);
  const float b = p.bias ? p.bias[n] : 0.f;
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const int m = m0 + g * 4 + r;
    if (m < p.M)
      p.y[(int64_t)m * p.N + n] = b + acc[r];
  }
}

// Rounds the fp32 GEMM result to the activations' type and applies the post-op there, re-rounding where the CPU path
// stores its tile (src/csrc/fused_gemm.h:1343-1488 on Tout = float or half): for float nothing is rounded.
template <bool HALF>
__device__ __forceinline__ float wide_round(float v) {
  return HALF ? (float)(_Float16)v : v;
}
template <bool HALF>
__global__ void __launch_bounds__(256)
post_op_wide_kernel(const float* __restrict__ acc, const void* __restrict__ in1, const void* __restrict__ in2,
                    void* __restrict__ out, int64_t n, int post, float scale) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n)
    return;
  auto ld = [&](const void* p) {
    return p == nullptr ? 0.f : HALF ? (float)reinterpret_cast<const _Float16*>(p)[i] : reinterpret_cast<const float*>(p)[i];
  };
  const float y = wide_round<HALF>(acc[i]);
  float o = y;
  switch (post) {
    case TPPX_POST_SILU:
      o = wide_round<HALF>(y * wide_round<HALF>(1.0f / (1.0f + __expf(-y))));
      break;
    case TPPX_POST_MUL:
      o = wide_round<HALF>(ld(in1) * y);
      break;
    case TPPX_POST_ADD_SCALE:
      o = wide_round<HALF>(fmaf(ld(in1), scale, y));
      break;
    case TPPX_POST_ADD2_SCALE:
      o = wide_round<HALF>(fmaf(ld(in2), scale, wide_round<HALF>(y + ld(in1))));
      break;
    case TPPX_POST_GELU:
      o = wide_round<HALF>(0.5f * y * (1.0f + erff(y * 0.70710678118654752f)));
      break;
    case TPPX_POST_RELU:
      o = y < 0.f ? 0.f : y;
      break;
    default:
      break;
  }
  if (HALF)
    reinterpret_cast<_Float16*>(out)[i] = (_Float16)o;
  else
    reinterpret_cast<float*>(out)[i] = o;
}

} // namespace tppx

using namespace tppx;

extern "C" int tppx_linear_wide(const void* x, int x_dtype, const void* w, const void* sw, int w_kind, const void* bias_f32,
                                void* y_f32, int64_t M, int64_t N, int64_t K, tppx_stream_t stream) {
  const char* who = "tppx_linear_wide";
  TPPX_REQUIRE(x && w && y_f32, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(x_dtype == TPPX_DT_F32 || x_dtype == TPPX_DT_F16, TPPX_EINVAL, "%s: activations must be fp32 or fp16 (dtype id %d)", who, x_dtype);
  TPPX_REQUIRE(w_kind == TPPX_W_MXFP4 || w_kind == TPPX_W_BF16, TPPX_EINVAL, "%s: weight kind %d is neither MXFP4 nor bf16", who, w_kind);
  TPPX_REQUIRE(w_kind == TPPX_W_BF16 || sw, TPPX_EINVAL, "%s: MXFP4 weights need their scale bytes", who);
  TPPX_REQUIRE(aligned16(x) && aligned16(w), TPPX_EINVAL, "%s: activation / weight pointer not 16-byte aligned", who);
  TPPX_REQUIRE(M >= 0 && M < (1 << 22), TPPX_ESHAPE, "%s: M=%ld out of range", who, (long)M);
  TPPX_REQUIRE(N > 0 && N % (w_kind == TPPX_W_MXFP4 ? 32 : 16) == 0, TPPX_ESHAPE, "%s: N=%ld must be a positive multiple of %d", who, (long)N, w_kind == TPPX_W_MXFP4 ? 32 : 16);
  TPPX_REQUIRE(K > 0 && K % 128 == 0, TPPX_ESHAPE, "%s: K=%ld must be a positive multiple of 128 (native tiles span 128 input channels)", who, (long)K);
  TPPX_REQUIRE(N / 16 < (1 << 30), TPPX_ESHAPE, "%s: N=%ld too large", who, (long)N);
  if (M == 0)
    return TPPX_OK;
  WideParams p;
  p.x = x;
  p.qw = w;
  p.sw = (const uint8_t*)sw;
  p.bias = (const float*)bias_f32;
  p.y = (float*)y_f32;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  const dim3 grid((unsigned)(N / 16), (unsigned)((M + 63) / 64)), block(256);
  const hipStream_t st = (hipStream_t)stream;
  if (x_dtype == TPPX_DT_F16) {
    if (w_kind == TPPX_W_BF16)
      linear_wide_kernel<true, true><<<grid, block, 0, st>>>(p);
    else
      linear_wide_kernel<true, false><<<grid, block, 0, st>>>(p);
  } else {
    if (w_kind == TPPX_W_BF16)
      linear_wide_kernel<false, true><<<grid, block, 0, st>>>(p);
    else
      linear_wide_kernel<false, false><<<grid, block, 0, st>>>(p);
  }
  return check_hip(hipGetLastError(), who);
}

extern "C" int tppx_post_op_wide(const void* acc_f32, int out_dtype, int post_op, const void* post_in, const void* post_in2,
                                 float post_scale, void* out, int64_t count, tppx_stream_t stream) {
  const char* who = "tppx_post_op_wide";
  TPPX_REQUIRE(acc_f32 && out, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(out_dtype == TPPX_DT_F32 || out_dtype == TPPX_DT_F16, TPPX_EINVAL, "%s: output must be fp32 or fp16 (dtype id %d)", who, out_dtype);
  TPPX_REQUIRE(post_op >= TPPX_POST_NONE && post_op <= TPPX_POST_RELU, TPPX_EINVAL, "%s: unknown post-op id %d", who, post_op);
  const bool need1 = post_op == TPPX_POST_MUL || post_op == TPPX_POST_ADD_SCALE || post_op == TPPX_POST_ADD2_SCALE;
  TPPX_REQUIRE(!need1 || post_in, TPPX_EINVAL, "%s: post-op %d needs post_in", who, post_op);
  TPPX_REQUIRE(post_op != TPPX_POST_ADD2_SCALE || post_in2, TPPX_EINVAL, "%s: post-op %d needs post_in2", who, post_op);
  TPPX_REQUIRE(count >= 0 && count < ((int64_t)1 << 40), TPPX_ESHAPE, "%s: count %ld out of range", who, (long)count);
  if (count == 0)
    return TPPX_OK;
  const unsigned blocks = (unsigned)((count + 255) / 256);
  if (out_dtype == TPPX_DT_F16)
    post_op_wide_kernel<true><<<blocks, 256, 0, (hipStream_t)stream>>>((const float*)acc_f32, post_in, post_in2, out, count, post_op, post_scale);
  else
    post_op_wide_kernel<false><<<blocks, 256, 0, (hipStream_t)stream>>>((const float*)acc_f32, post_in, post_in2, out, count, post_op, post_scale);
  return check_hip(hipGetLastError(), who);
}

extern "C" int tppx_linear_qint8_f32(const void* xq, const void* sa, const void* qw, const void* sw, const void* bias_f32,
                                     void* y_f32, int64_t M, int64_t N, int64_t K, int64_t qbs, tppx_stream_t stream) {
  const char* who = "tppx_linear_qint8_f32";
  TPPX_REQUIRE(xq && sa && qw && sw && y_f32, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(aligned16(xq) && aligned16(qw), TPPX_EINVAL, "%s: activation / weight pointer not 16-byte aligned", who);
  TPPX_REQUIRE(M >= 0 && M < (1 << 30), TPPX_ESHAPE, "%s: M=%ld out of range", who, (long)M);
  TPPX_REQUIRE(N > 0 && N % 16 == 0, TPPX_ESHAPE, "%s: N=%ld must be a positive multiple of 16", who, (long)N);
  TPPX_REQUIRE(qbs >= 64 && qbs % 64 == 0, TPPX_ESHAPE, "%s: block size %ld must be a multiple of 64", who, (long)qbs);
  TPPX_REQUIRE(K > 0 && K % qbs == 0, TPPX_ESHAPE, "%s: K=%ld must be a positive multiple of the block size %ld", who, (long)K, (long)qbs);
  TPPX_REQUIRE(M * N < ((int64_t)1 << 40) && N / 16 < 65536 * 32768ll, TPPX_ESHAPE, "%s: problem too large", who);
  if (M == 0)
    return TPPX_OK;
  F32OutParams p;
  p.xq = (const int8_t*)xq;
  p.sa = (const float*)sa;
  p.qw = qw;
  p.sw = (const float*)sw;
  p.bias = (const float*)bias_f32;
  p.y = (float*)y_f32;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.qbs = (int)qbs;
  const int64_t by = (M + 63) / 64;
  TPPX_REQUIRE(by <= 65535, TPPX_ESHAPE, "%s: M=%ld exceeds the grid (at most 65535 blocks of 64 rows)", who, (long)M);
  linear_qint8_f32_kernel<<<dim3((unsigned)(N / 16), (unsigned)by), dim3(256), 0, (hipStream_t)stream>>>(p);
  return check_hip(hipGetLastError(), who);
}
