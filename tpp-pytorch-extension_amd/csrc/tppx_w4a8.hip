// W4A8: MXFP4 weights in the VNNI8-interleaved layout that remap_and_quantize_mxfp4 produces under USE_MXFP4_INT8
// (src/csrc/qtypes.cpp:787-790, 840-861) against int8 activations quantized over blocks of 32
// (TppBlockedLinearW<int8_t, uint8_t, Tout>, src/csrc/fused_gemm.h:965-978, 1523-1526), on the K = 32 int8 MFMA:
//   y = post( bf16( bias + sum_b float(sum_{k in b} xq[m][k] * wi[n][k]) * (sa[m][b] * 2^(e[n][b] - 127)) ) )
// with wi = the E2M1 value times 127/6 as an integer, {0, 11, 21, 32, 42, 64, 85, 127} with sign (the activation
// scales arrive multiplied by 6/127, fused_gemm.h:975-977; the table itself lives inside the reference's JIT
// library and is restated, not copied: results agree with the reference only within that table's rounding).
// Weight bytes are read where the reference keeps them, no repacking: q u8 [N/8][K/bc][bc/8][8][4], byte j of a
// group (channel n8, 8 K values) = K value j | K value 4 + j << 4 -- the low nibbles of a lane's four bytes are the
// first four of its eight MFMA operand bytes, the high nibbles the last four; scales u8 [N/8][K/bc][bc/32][8].
// A workgroup owns a 16 x 16 output tile; its four waves split the MX blocks of K and add their partial sums in
// wave order: the simple shape of the calls the decode kernel (skinny_w4a8_kernel) does not take, not a tuned kernel.
#include <hip/hip_runtime.h>

#include "tppx.h"
#include "tppx_common.h"

namespace tppx {

struct W4A8Params {
  const int8_t* xq; // [M][K]
  const float* sa;  // [M][K/32], already times 6/127
  const uint8_t* q;
  const uint8_t* sc;
  const uint16_t* bias;
  const uint16_t* post_in;
  const uint16_t* post_in2;
  uint16_t* y;
  int M, N, K, bc, post_op;
  float post_scale;
};

__global__ void __launch_bounds__(256)
linear_w4a8_kernel(const W4A8Params p) {
  __shared__ float part[4][64][4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m0 = blockIdx.y * 16;
  const int n = blockIdx.x * 16 + (lane & 15), kg = lane >> 4;
  const int n8b = n >> 3, n8 = n & 7;
  const int C1 = p.K / p.bc, G = p.bc / 8, SB = p.bc / 32, NB = p.K / 32;
  const int8_t* xr = p.xq + (int64_t)min(m0 + (lane & 15), p.M - 1) * p.K + kg * 8;
  float f[4] = {0.f, 0.f, 0.f, 0.f};
  const float* sar[4];
#pragma unroll
  for (int r = 0; r < 4; r++)
    sar[r] = p.sa + (int64_t)min(m0 + kg * 4 + r, p.M - 1) * NB;
  // the four waves split the MX blocks of K (ascending ranges), their partial sums meet in LDS in wave order
  const int b0 = (wave * NB) / 4, b1 = ((wave + 1) * NB) / 4;
  for (int b = b0; b < b1; b++) {
    const int c1 = (b * 32) / p.bc, kb = (b * 32) % p.bc;
    const int64_t blk = (int64_t)n8b * C1 + c1;
    const uint32_t codes = *reinterpret_cast<const uint32_t*>(p.q + ((blk * G + (kb >> 3) + kg) * 8 + n8) * 4);
    const uint32_t lo = w4a8_expand(codes & 0x0F0F0F0Fu), hi = w4a8_expand((codes >> 4) & 0x0F0F0F0Fu);
    const long wb = (long)(((uint64_t)hi << 32) | lo);
    const long xa = *reinterpret_cast<const long*>(xr + (int64_t)b * 32);
    const i32x4 acc = __builtin_amdgcn_mfma_i32_16x16x32_i8(xa, wb, i32x4{0, 0, 0, 0}, 0, 0, 0);
    const float wsc = e8m0_to_f32(p.sc[(blk * SB + (kb >> 5)) * 8 + n8]);
#pragma unroll
    for (int r = 0; r < 4; r++)
      f[r] = fmaf((float)acc[r], sar[r][b] * wsc, f[r]);
  }
#pragma unroll
  for (int r = 0; r < 4; r++)
    part[wave][lane][r] = f[r];
  __syncthreads();
  if (wave != 0)
    return;
  const float bias = p.bias ? bf16_bits_to_f32(p.bias[n]) : 0.f;
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const int m = m0 + kg * 4 + r;
    const float v = bias + (((part[0][lane][r] + part[1][lane][r]) + part[2][lane][r]) + part[3][lane][r]);
    if (m < p.M) {
      const int64_t o = (int64_t)m * p.N + n;
      p.y[o] = (uint16_t)apply_post_bits(v, p.post_op, p.post_in ? p.post_in[o] : 0, p.post_in2 ? p.post_in2[o] : 0,
                                         p.post_scale);
    }
  }
}

} // namespace tppx

using namespace tppx;

extern "C" int tppx_linear_mxfp4_int8(const void* xq, const void* sa, const void* q, const void* sc, const void* bias,
                                      const void* post_in, const void* post_in2, void* y, int64_t M, int64_t N, int64_t K,
                                      int64_t bc, int post_op, float post_scale, tppx_stream_t stream) {
  const char* who = "tppx_linear_mxfp4_int8";
  TPPX_REQUIRE(xq && sa && q && sc && y, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(((uintptr_t)xq & 7) == 0 && ((uintptr_t)q & 3) == 0, TPPX_EINVAL, "%s: activation / weight pointer misaligned", who);
  TPPX_REQUIRE(post_op >= TPPX_POST_NONE && post_op <= TPPX_POST_RELU, TPPX_EINVAL, "%s: unknown post-op id %d", who, post_op);
  TPPX_REQUIRE(M >= 0 && M < (1 << 30), TPPX_ESHAPE, "%s: M=%ld out of range", who, (long)M);
  TPPX_REQUIRE(N > 0 && N % 16 == 0, TPPX_ESHAPE, "%s: N=%ld must be a positive multiple of 16", who, (long)N);
  TPPX_REQUIRE(bc >= 32 && bc % 32 == 0, TPPX_ESHAPE, "%s: input-channel block %ld must be a multiple of 32", who, (long)bc);
  TPPX_REQUIRE(K > 0 && K % bc == 0, TPPX_ESHAPE, "%s: K=%ld must be a positive multiple of the block %ld", who, (long)K, (long)bc);
  const int64_t by = (M + 15) / 16;
  TPPX_REQUIRE(by <= 65535 && M * N < ((int64_t)1 << 40), TPPX_ESHAPE, "%s: problem too large", who);
  if (M == 0)
    return TPPX_OK;
  W4A8Params p;
  p.xq = (const int8_t*)xq;
  p.sa = (const float*)sa;
  p.q = (const uint8_t*)q;
  p.sc = (const uint8_t*)sc;
  p.bias = (const uint16_t*)bias;
  p.post_in = (const uint16_t*)post_in;
  p.post_in2 = (const uint16_t*)post_in2;
  p.y = (uint16_t*)y;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.bc = (int)bc;
  p.post_op = post_op;
  p.post_scale = post_scale;
  linear_w4a8_kernel<<<dim3((unsigned)(N / 16), (unsigned)by), dim3(256), 0, (hipStream_t)stream>>>(p);
  return check_hip(hipGetLastError(), who);
}
