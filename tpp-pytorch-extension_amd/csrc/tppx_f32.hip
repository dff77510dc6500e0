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

} // namespace tppx

using namespace tppx;

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
