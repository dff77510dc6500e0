// Quantize / de-quantize / re-layout kernels (HBM-bound byte work, one-time per
// weight except for the activation quantizer which runs on every QINT8 call).
#include "tppx_common.h"
#include "tppx_launch.h"

namespace tppx {

// offset of element (n,k) of a blocked weight (see tppx_quantize_mxfp4 in tppx.h)
__device__ __forceinline__ int64_t blocked_off(int64_t n, int64_t k, int64_t K,
                                               int64_t bk, int64_t bc,
                                               int64_t vnni) {
  int64_t kb = k % bc;
  return ((n / bk) * (K / bc) + k / bc) * bk * bc + (kb / vnni) * bk * vnni +
      (n % bk) * vnni + kb % vnni;
}

template <typename T>
__device__ __forceinline__ float load_as_f32(const T* p, int64_t i);
template <>
__device__ __forceinline__ float load_as_f32<float>(const float* p, int64_t i) {
  return p[i];
}
template <>
__device__ __forceinline__ float load_as_f32<uint16_t>(const uint16_t* p,
                                                      int64_t i) {
  return bf16_bits_to_f32(p[i]);
}

// E2M1 code of an already scaled value: nearest, ties to even mantissa,
// saturating at 6, +-0 -> 0, NaN -> 0.
__device__ __forceinline__ uint32_t e2m1_encode(float v) {
  if (v != v)
    return 0;
  float a = fabsf(v);
  uint32_t c = a <= 0.25f ? 0u
      : a < 0.75f         ? 1u
      : a <= 1.25f        ? 2u
      : a < 1.75f         ? 3u
      : a <= 2.5f         ? 4u
      : a < 3.5f          ? 5u
      : a <= 5.0f         ? 6u
                          : 7u;
  if (c != 0 && (__float_as_uint(v) >> 31))
    c |= 8u;
  return c;
}

// One thread per MX block (one output channel x 32 consecutive K).
// Threads are ordered with the channel-in-32 index fastest so that the byte
// and scale stores of a wave fall into contiguous 32-byte runs.
template <typename T>
__global__ void __launch_bounds__(256)
quantize_mxfp4_kernel(const T* __restrict__ w, int64_t N, int64_t K, int64_t bk,
                      int64_t bc, int64_t vnni, uint8_t* __restrict__ qdata,
                      uint8_t* __restrict__ scales) {
  int64_t nblk = (N / 32) * (K / 64) * 2 * 32;
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= nblk)
    return;
  int64_t k2 = t & 31;
  int64_t h = (t >> 5) & 1;
  int64_t rest = t >> 6;
  int64_t Nc = K / 64;
  int64_t nc = rest % Nc, nk = rest / Nc;
  int64_t n = nk * 32 + k2, k0 = nc * 64 + h * 32;
  float v[32];
#pragma unroll
  for (int j = 0; j < 32; j++)
    v[j] = load_as_f32<T>(w, blocked_off(n, k0 + j, K, bk, bc, vnni));
  // max = |first|, then std::max(max, |v|) as the CPU path has it: a NaN in the first slot stays (scale byte 255),
  // a NaN anywhere else never wins the comparison
  float amax = fabsf(v[0]);
#pragma unroll
  for (int j = 1; j < 32; j++) {
    float a = fabsf(v[j]);
    amax = a > amax ? a : amax;
  }
  int e = (int)((__float_as_uint(amax) >> 23) & 0xffu);
  bool flush = (e == 0);
  int x = (e == 255) ? 255 : (e - 2 < 0 ? 0 : e - 2);
  scales[((nk * Nc + nc) * 2 + h) * 32 + k2] = (uint8_t)x;
  // division by the power-of-two scale is an exact exponent shift; x == 0
  // stands for 2^-127, x == 255 for NaN (all codes 0)
  int sh = 127 - x;
#pragma unroll
  for (int p = 0; p < 16; p++) {
    uint32_t c0 = 0, c1 = 0;
    if (!flush && x != 255) {
      c0 = e2m1_encode(ldexpf(v[2 * p], sh));
      c1 = e2m1_encode(ldexpf(v[2 * p + 1], sh));
    }
    qdata[((nk * Nc + nc) * 32 + (h * 16 + p)) * 32 + k2] =
        (uint8_t)(c0 | (c1 << 4));
  }
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1)
    v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

__device__ __forceinline__ float int8_scale_of(float amax) {
  return (float)((double)amax / 127.0);
}
__device__ __forceinline__ float int8_inv_scale(float s) {
  return s != 0.0f ? __frcp_rn(s) : 0.0f;
}
__device__ __forceinline__ int int8_q(float v, float inv) {
  float r = rintf(__fmul_rn(v, inv));
  r = fminf(fmaxf(r, -127.0f), 127.0f);
  return (int)r;
}

// One wave per (output channel, K block of qbs).
template <typename T>
__global__ void __launch_bounds__(256)
quantize_qint8_kernel(const T* __restrict__ w, int64_t N, int64_t K, int64_t bk,
                      int64_t bc, int64_t vnni, int64_t qbs,
                      int8_t* __restrict__ q, float* __restrict__ scales) {
  int64_t nb = K / qbs;
  int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  int lane = threadIdx.x & 63;
  if (wave >= N * nb)
    return;
  // channel-in-16 fastest so neighbouring waves write neighbouring rows
  int64_t k2 = wave & 15;
  int64_t rest = wave >> 4;
  int64_t b = rest % nb, n1 = rest / nb;
  int64_t n = n1 * 16 + k2;
  float amax = 0.0f;
  for (int64_t j = lane; j < qbs; j += 64) {
    float a = fabsf(load_as_f32<T>(w, blocked_off(n, b * qbs + j, K, bk, bc, vnni)));
    amax = a > amax ? a : amax;
  }
  amax = wave_max(amax);
  float s = int8_scale_of(amax);
  float inv = int8_inv_scale(s);
  if (lane == 0)
    scales[(n1 * nb + b) * 16 + k2] = s;
  for (int64_t j = lane; j < qbs; j += 64) {
    float v = load_as_f32<T>(w, blocked_off(n, b * qbs + j, K, bk, bc, vnni));
    q[(((n1 * nb + b) * (qbs / 4) + (j >> 2)) * 16 + k2) * 4 + (j & 3)] =
        (int8_t)int8_q(v, inv);
  }
}

__constant__ float c_e2m1_tbl[16] = {0.0f,  0.5f,  1.0f,  1.5f, 2.0f,  3.0f,
                                     4.0f,  6.0f,  -0.0f, -0.5f, -1.0f, -1.5f,
                                     -2.0f, -3.0f, -4.0f, -6.0f};

// one thread per packed byte; out is [N/32][K/64][32][32][2] fp32
__global__ void __launch_bounds__(256)
dequantize_mxfp4_kernel(const uint8_t* __restrict__ qdata,
                        const uint8_t* __restrict__ scales, int64_t nbytes,
                        float* __restrict__ out) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= nbytes)
    return;
  int64_t k2 = t & 31, c2 = (t >> 5) & 31, tile = t >> 10;
  uint32_t b = qdata[t];
  float s = e8m0_to_f32(scales[(tile * 2 + (c2 >> 4)) * 32 + k2]);
  float2 r;
  r.x = c_e2m1_tbl[b & 0xf] * s;
  r.y = c_e2m1_tbl[b >> 4] * s;
  reinterpret_cast<float2*>(out)[t] = r;
}

// one thread per 4 int8; out [N/16][K/QBS][QBS/4][16][4] fp32
__global__ void __launch_bounds__(256)
dequantize_qint8_kernel(const int8_t* __restrict__ q,
                        const float* __restrict__ scales, int64_t ngroups,
                        int64_t qbs, float* __restrict__ out) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= ngroups)
    return;
  int64_t k2 = t & 15;
  int64_t blk = (t >> 4) / (qbs / 4); // (n1*nb + b)
  float s = scales[blk * 16 + k2];
  uint32_t v = reinterpret_cast<const uint32_t*>(q)[t];
  float4 r;
  r.x = (float)(int8_t)(v & 0xff) * s;
  r.y = (float)(int8_t)((v >> 8) & 0xff) * s;
  r.z = (float)(int8_t)((v >> 16) & 0xff) * s;
  r.w = (float)(int8_t)(v >> 24) * s;
  reinterpret_cast<float4*>(out)[t] = r;
}

// one thread per native 16-byte chunk (nt, kt, g, n)
__global__ void __launch_bounds__(256)
prepack_mxfp4_kernel(const uint8_t* __restrict__ qref,
                     const uint8_t* __restrict__ sref, int64_t N, int64_t K,
                     uint8_t* __restrict__ qnat, uint8_t* __restrict__ snat) {
  int64_t nchunks = N * (K / 32);
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= nchunks)
    return;
  int64_t n16 = t & 15, g = (t >> 4) & 3, rest = t >> 6;
  int64_t KT = K / 128, Nc = K / 64;
  int64_t kt = rest % KT, nt = rest / KT;
  int64_t n = nt * 16 + n16, k0 = kt * 128 + g * 32;
  int64_t nk = n >> 5, k2 = n & 31, nc = k0 >> 6, c2b = (k0 & 63) >> 1;
  const uint8_t* src = qref + ((nk * Nc + nc) * 32 + c2b) * 32 + k2;
  uint32_t wd[4];
#pragma unroll
  for (int d = 0; d < 4; d++) {
    uint32_t v = 0;
#pragma unroll
    for (int i = 0; i < 4; i++)
      v |= (uint32_t)src[(d * 4 + i) * 32] << (8 * i);
    wd[d] = v;
  }
  reinterpret_cast<uint4*>(qnat)[t] = make_uint4(wd[0], wd[1], wd[2], wd[3]);
  snat[t] = sref[((nk * Nc + nc) * 2 + ((k0 & 63) >> 5)) * 32 + k2];
}

__global__ void __launch_bounds__(256)
prepack_qint8_kernel(const int8_t* __restrict__ qref, int64_t N, int64_t K,
                     int64_t qbs, int8_t* __restrict__ qnat) {
  int64_t nchunks = N * (K / 16);
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= nchunks)
    return;
  int64_t n16 = t & 15, g = (t >> 4) & 3, rest = t >> 6;
  int64_t KT = K / 64, nb = K / qbs;
  int64_t kt = rest % KT, nt = rest / KT;
  int64_t k0 = kt * 64 + g * 16;
  int64_t b = k0 / qbs, a0 = (k0 % qbs) >> 2;
  const uint32_t* src = reinterpret_cast<const uint32_t*>(qref) +
      ((nt * nb + b) * (qbs / 4) + a0) * 16 + n16;
  reinterpret_cast<uint4*>(qnat)[t] =
      make_uint4(src[0], src[16], src[32], src[48]);
}

// bf16 weight in the reference's blocked layout [N/bk][K/bc][bc/v][bk][v] (v = 2: VNNI2 pairs; bk = 1, bc = K, v = 1:
// a plain [N][K] matrix) -> native bf16 tiles [N/16][K/128][4 j][4 g][16 n][8]: the 16 bytes lane (g, n) feeds to
// MFMA step j of K tile kt are W[nt*16 + n][kt*128 + (g*4 + j)*8 .. +7].
__global__ void __launch_bounds__(256)
prepack_bf16_kernel(const uint16_t* __restrict__ wref, int64_t N, int64_t K, int64_t bk, int64_t bc, int64_t v,
                    uint16_t* __restrict__ wnat) {
  const int64_t nchunks = N * (K / 8);
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= nchunks)
    return;
  const int64_t n16 = t & 15, g = (t >> 4) & 3, j = (t >> 6) & 3, rest = t >> 8;
  const int64_t KT = K / 128, kt = rest % KT, nt = rest / KT;
  const int64_t n = nt * 16 + n16, k0 = kt * 128 + (g * 4 + j) * 8;
  const int64_t n1 = n / bk, k2 = n % bk;
  uint16_t e[8];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const int64_t k = k0 + i, c1 = k / bc, kk = k % bc;
    e[i] = wref[(((n1 * (K / bc) + c1) * (bc / v) + kk / v) * bk + k2) * v + kk % v];
  }
  reinterpret_cast<uint4*>(wnat)[t] = make_uint4(e[0] | ((uint32_t)e[1] << 16), e[2] | ((uint32_t)e[3] << 16),
                                                 e[4] | ((uint32_t)e[5] << 16), e[6] | ((uint32_t)e[7] << 16));
}

// Activations for the block-scaled MFMA path: bf16 [M][K] -> MXFP8 (OCP E4M3 elements, one E8M0 scale per 32
// input channels, scale exponent = floor(log2 max|x|) - 8 as the OCP MX recipe has it), written in MFMA operand
// order: values [M/16][K/128][2 halves][64 lanes][16 B] -- an 8-bit operand of the 16x16x128 instruction is two
// 64-channel halves, so lane (g, m) of a 16-row x 128-channel tile holds channels g*16 .. g*16+15 of row m in half
// 0 and 64 + g*16 .. 64 + g*16+15 in half 1 -- and scale bytes [M/64][K/128][64 lanes][4 row tiles]: byte t of
// lane (b, m)'s word is the scale of channels b*32 .. b*32+31 of row m of the group's row tile t (the instruction
// scales by 32-channel block, whichever lanes hold the elements).  Rows are padded to a multiple of 64 with zeros
// (scale byte 0).
__device__ __forceinline__ uint32_t e4m3_encode_rne(float v) {
  const uint32_t sign = (__float_as_uint(v) >> 24) & 0x80u;
  const float a = fminf(fabsf(v), 448.0f);
  if (a < 0.015625f) // below the smallest normal 2^-6: multiples of 2^-9 (8 is the code of 2^-6 itself)
    return sign | (uint32_t)__float2int_rn(a * 512.0f);
  uint32_t u = __float_as_uint(a);
  u += 0x7ffffu + ((u >> 20) & 1u); // round to nearest even at 3 mantissa bits
  return sign | ((((u >> 23) - 120u) << 3) | ((u >> 20) & 7u));
}

__global__ void __launch_bounds__(256)
quant_act_mxfp8_kernel(const uint16_t* __restrict__ x, int64_t M, int64_t K, uint8_t* __restrict__ xq,
                       uint8_t* __restrict__ xs) {
  // One wave per half of a 16-row x 128-channel tile: lane (g, r) turns channels h*64 + g*16 .. +15 of row r into the
  // 16 bytes it holds as an operand, so a wave reads 16 pieces of 128 contiguous bytes and writes 1 KiB in lane order;
  // the two lanes that share a 32-channel block (g, g ^ 1) exchange their maxima.
  const int64_t KT = K / 128;
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t Mp = (M + 63) / 64 * 64;
  const int64_t tile = t >> 7;
  if (tile >= (Mp / 16) * KT) // wave-uniform
    return;
  const int lane = (int)(t & 63), h = (int)((t >> 6) & 1), g = lane >> 4, r = lane & 15;
  const int64_t mt = tile / KT, kt = tile % KT, m = mt * 16 + r;
  uint32_t w[8];
  if (m < M) {
    const uint4* src = reinterpret_cast<const uint4*>(x + m * K + kt * 128 + h * 64 + g * 16);
    const uint4 v0 = src[0], v1 = src[1];
    w[0] = v0.x; w[1] = v0.y; w[2] = v0.z; w[3] = v0.w;
    w[4] = v1.x; w[5] = v1.y; w[6] = v1.z; w[7] = v1.w;
  } else {
#pragma unroll
    for (int i = 0; i < 8; i++)
      w[i] = 0u;
  }
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; i++)
    amax = fmaxf(amax, fmaxf(fabsf(bf16_bits_to_f32(w[i] & 0xffffu)), fabsf(bf16_bits_to_f32(w[i] >> 16))));
  amax = fmaxf(amax, __shfl_xor(amax, 16));
  const int E = (int)((__float_as_uint(amax) >> 23) & 0xffu);
  const int X = min(max(E - 8, 0), 254);
  const float inv = __uint_as_float((uint32_t)(254 - X) << 23); // 2^(127 - X), X <= 246
  uint32_t out[4];
#pragma unroll
  for (int d = 0; d < 4; d++) {
    uint32_t v = 0;
#pragma unroll
    for (int e = 0; e < 2; e++) {
      const uint32_t pr = w[2 * d + e];
      v |= e4m3_encode_rne(bf16_bits_to_f32(pr & 0xffffu) * inv) << (16 * e);
      v |= e4m3_encode_rne(bf16_bits_to_f32(pr >> 16) * inv) << (16 * e + 8);
    }
    out[d] = v;
  }
  reinterpret_cast<uint4*>(xq)[((mt * KT + kt) * 2 + h) * 64 + lane] = make_uint4(out[0], out[1], out[2], out[3]);
  if ((g & 1) == 0) // block b = h*2 + g/2 of the tile: byte (mt & 3) of lane (b, r)'s word
    xs[(((mt >> 2) * KT + kt) * 64 + (h * 2 + (g >> 1)) * 16 + r) * 4 + (mt & 3)] = m < M ? (uint8_t)X : (uint8_t)0;
}

// Activation quantizer: one wave per (row, K block).  Each lane owns
// consecutive pairs so loads and stores stay contiguous.
__global__ void __launch_bounds__(256)
quant_act_int8_kernel(const uint16_t* __restrict__ x, int64_t M, int64_t K,
                      int64_t qbs, int8_t* __restrict__ xq,
                      float* __restrict__ sa, int mt) {
  int64_t nb = K / qbs;
  int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  int lane = threadIdx.x & 63;
  if (wave >= M * nb)
    return;
  int64_t m = wave / nb, b = wave % nb;
  const uint16_t* p = x + m * K + b * qbs;
  int8_t* o = xq + m * K + b * qbs;
  if (qbs == 256) {
    // 4 consecutive bf16 per lane
    uint2 raw = reinterpret_cast<const uint2*>(p)[lane];
    float v0 = bf16_bits_to_f32(raw.x & 0xffffu), v1 = bf16_bits_to_f32(raw.x >> 16);
    float v2 = bf16_bits_to_f32(raw.y & 0xffffu), v3 = bf16_bits_to_f32(raw.y >> 16);
    float amax = fmaxf(fmaxf(fabsf(v0), fabsf(v1)), fmaxf(fabsf(v2), fabsf(v3)));
    amax = wave_max(amax);
    float s = int8_scale_of(amax);
    float inv = int8_inv_scale(s);
    if (lane == 0)
      sa[mt > 0 ? b * (int64_t)mt * 16 + m : m * nb + b] = s;
    uint32_t packed = (uint32_t)(int8_q(v0, inv) & 0xff) |
        ((uint32_t)(int8_q(v1, inv) & 0xff) << 8) |
        ((uint32_t)(int8_q(v2, inv) & 0xff) << 16) |
        ((uint32_t)(int8_q(v3, inv) & 0xff) << 24);
    if (mt > 0) {
      // operand order: tile (k/64, m/16), lane slot (k%64)/16*16 + m%16, 16 B each
      const int64_t t = b * 4 + (lane >> 4);
      const int64_t slot = ((t * mt + (m >> 4)) * 64 + ((lane & 15) >> 2) * 16 + (m & 15));
      reinterpret_cast<uint32_t*>(xq)[slot * 4 + (lane & 3)] = packed;
    } else {
      reinterpret_cast<uint32_t*>(o)[lane] = packed;
    }
  } else {
    float amax = 0.0f;
    for (int64_t j = lane; j < qbs; j += 64)
      amax = fmaxf(amax, fabsf(bf16_bits_to_f32(p[j])));
    amax = wave_max(amax);
    float s = int8_scale_of(amax);
    float inv = int8_inv_scale(s);
    if (lane == 0)
      sa[mt > 0 ? b * (int64_t)mt * 16 + m : m * nb + b] = s;
    for (int64_t j = lane; j < qbs; j += 64) {
      const int8_t q = (int8_t)int8_q(bf16_bits_to_f32(p[j]), inv);
      if (mt > 0) {
        const int64_t k = b * qbs + j;
        xq[(((k >> 6) * mt + (m >> 4)) * 64 + ((k & 63) >> 4) * 16 + (m & 15)) * 16 + (k & 15)] = q;
      } else {
        o[j] = q;
      }
    }
  }
}

// Many rows, 256-wide blocks, row-major output (the large-M GEMM's input): 16 lanes per (row, block), 16 values per
// lane -- 32-byte reads, 16-byte writes, four blocks per wave -- and the maximum taken inside the 16-lane DPP row.
// Same arithmetic as the kernel above (the maximum does not depend on the order).
__global__ void __launch_bounds__(256)
quant_act_int8_rows_kernel(const uint16_t* __restrict__ x, int64_t M, int64_t K, int8_t* __restrict__ xq,
                           float* __restrict__ sa, int mt) {
  const int64_t nb = K >> 8;
  const int64_t blk = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 4;
  const int l = threadIdx.x & 15;
  if (blk >= M * nb) // whole DPP rows leave together
    return;
  const uint4* src = reinterpret_cast<const uint4*>(x + blk * 256 + l * 16); // (m, b) -> m*K + b*256 = blk*256
  const uint4 v0 = src[0], v1 = src[1];
  const uint32_t w[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
  float f[16];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    f[2 * i] = bf16_bits_to_f32(w[i] & 0xffffu);
    f[2 * i + 1] = bf16_bits_to_f32(w[i] >> 16);
  }
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < 16; i++)
    amax = fmaxf(amax, fabsf(f[i]));
  auto dpp = [](float v, auto CTRL) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), decltype(CTRL)::value, 0xf, 0xf, true));
  };
  amax = fmaxf(amax, dpp(amax, std::integral_constant<int, 0xB1>{}));  // quad_perm [1,0,3,2]
  amax = fmaxf(amax, dpp(amax, std::integral_constant<int, 0x4E>{}));  // quad_perm [2,3,0,1]
  amax = fmaxf(amax, dpp(amax, std::integral_constant<int, 0x141>{})); // row_half_mirror
  amax = fmaxf(amax, dpp(amax, std::integral_constant<int, 0x140>{})); // row_mirror
  const float s = int8_scale_of(amax);
  const float inv = int8_inv_scale(s);
  const int64_t m = blk / nb, b = blk - m * nb;
  if (l == 0)
    sa[mt > 0 ? b * (int64_t)mt * 16 + m : blk] = s; // [M][nb], or [nb][mt * 16] beside operand-order values
  uint32_t o[4];
#pragma unroll
  for (int d = 0; d < 4; d++)
    o[d] = (uint32_t)(int8_q(f[4 * d], inv) & 0xff) | ((uint32_t)(int8_q(f[4 * d + 1], inv) & 0xff) << 8) |
           ((uint32_t)(int8_q(f[4 * d + 2], inv) & 0xff) << 16) | ((uint32_t)(int8_q(f[4 * d + 3], inv) & 0xff) << 24);
  if (mt > 0) {
    // operand order: the lane's 16 values are K group l % 4 of tile b * 4 + l / 4 (64 K each), row m % 16 of row
    // tile m / 16: [tile][mt row tiles][4 K groups][16 rows][16 B]
    const int64_t t = b * 4 + (l >> 2);
    const int64_t slot = (t * mt + (m >> 4)) * 64 + (l & 3) * 16 + (m & 15);
    reinterpret_cast<uint4*>(xq)[slot] = make_uint4(o[0], o[1], o[2], o[3]);
  } else {
    reinterpret_cast<uint4*>(xq + blk * 256)[l] = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

// Scale blocks of several 256-wide runs (per-output-channel weights: one block = all of K): one workgroup per
// (row, block), 16 lanes per run as above; the runs' maxima meet in LDS.  A lane group's first run stays in registers
// between the two steps, further runs (blocks beyond 16 Ki channels) are read a second time.
__global__ void __launch_bounds__(1024)
quant_act_int8_bigblk_kernel(const uint16_t* __restrict__ x, int64_t M, int64_t K, int64_t qbs, int8_t* __restrict__ xq,
                             float* __restrict__ sa, int mt) {
  __shared__ float gmax[64];
  const int64_t nb = K / qbs, m = blockIdx.x / nb, b = blockIdx.x - m * nb;
  const int spb = (int)(qbs >> 8), groups = blockDim.x >> 4;
  const int l = threadIdx.x & 15, grp = threadIdx.x >> 4;
  const uint16_t* row = x + m * K + b * qbs;
  auto dpp = [](float v, auto CTRL) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), decltype(CTRL)::value, 0xf, 0xf, true));
  };
  auto load_run = [&](int r, uint32_t (&w)[8]) {
    const uint4* src = reinterpret_cast<const uint4*>(row + (int64_t)r * 256 + l * 16);
    const uint4 v0 = src[0], v1 = src[1];
    w[0] = v0.x; w[1] = v0.y; w[2] = v0.z; w[3] = v0.w;
    w[4] = v1.x; w[5] = v1.y; w[6] = v1.z; w[7] = v1.w;
  };
  auto amax_of = [&](const uint32_t (&w)[8]) {
    float a = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++)
      a = fmaxf(a, fmaxf(fabsf(bf16_bits_to_f32(w[i] & 0xffffu)), fabsf(bf16_bits_to_f32(w[i] >> 16))));
    return a;
  };
  uint32_t first[8] = {0, 0, 0, 0, 0, 0, 0, 0}, w[8];
  float amax = 0.0f;
  if (grp < spb) {
    load_run(grp, first);
    amax = amax_of(first);
  }
  for (int r = grp + groups; r < spb; r += groups) {
    load_run(r, w);
    amax = fmaxf(amax, amax_of(w));
  }
  amax = fmaxf(amax, dpp(amax, std::integral_constant<int, 0xB1>{}));
  amax = fmaxf(amax, dpp(amax, std::integral_constant<int, 0x4E>{}));
  amax = fmaxf(amax, dpp(amax, std::integral_constant<int, 0x141>{}));
  amax = fmaxf(amax, dpp(amax, std::integral_constant<int, 0x140>{}));
  if (l == 0)
    gmax[grp] = amax;
  __syncthreads();
  amax = 0.0f;
  for (int j = l; j < groups; j += 16)
    amax = fmaxf(amax, gmax[j]);
  amax = fmaxf(amax, dpp(amax, std::integral_constant<int, 0xB1>{}));
  amax = fmaxf(amax, dpp(amax, std::integral_constant<int, 0x4E>{}));
  amax = fmaxf(amax, dpp(amax, std::integral_constant<int, 0x141>{}));
  amax = fmaxf(amax, dpp(amax, std::integral_constant<int, 0x140>{}));
  const float s = int8_scale_of(amax);
  const float inv = int8_inv_scale(s);
  if (threadIdx.x == 0)
    sa[mt > 0 ? b * (int64_t)mt * 16 + m : m * nb + b] = s;
  auto emit = [&](int r, const uint32_t (&src)[8]) {
    uint32_t o[4];
#pragma unroll
    for (int d = 0; d < 4; d++) {
      const float f0 = bf16_bits_to_f32(src[2 * d] & 0xffffu), f1 = bf16_bits_to_f32(src[2 * d] >> 16);
      const float f2 = bf16_bits_to_f32(src[2 * d + 1] & 0xffffu), f3 = bf16_bits_to_f32(src[2 * d + 1] >> 16);
      o[d] = (uint32_t)(int8_q(f0, inv) & 0xff) | ((uint32_t)(int8_q(f1, inv) & 0xff) << 8) |
             ((uint32_t)(int8_q(f2, inv) & 0xff) << 16) | ((uint32_t)(int8_q(f3, inv) & 0xff) << 24);
    }
    const int64_t k0 = b * qbs + (int64_t)r * 256; // first channel of the run
    if (mt > 0) {
      const int64_t t = (k0 >> 6) + (l >> 2);
      const int64_t slot = (t * mt + (m >> 4)) * 64 + (l & 3) * 16 + (m & 15);
      reinterpret_cast<uint4*>(xq)[slot] = make_uint4(o[0], o[1], o[2], o[3]);
    } else {
      reinterpret_cast<uint4*>(xq + m * K + k0)[l] = make_uint4(o[0], o[1], o[2], o[3]);
    }
  };
  if (grp < spb)
    emit(grp, first);
  for (int r = grp + groups; r < spb; r += groups) {
    load_run(r, w);
    emit(r, w);
  }
}

// ---------------------------------------------------------------------------
// Generic per-block quantizers: any tensor viewed as in[pre][bs][post][vnni]
// (the geometry PerBlockQuantizer derives from sizes, block size, axis and the
// VNNI flag), one block = the bs * vnni elements that share (pre, post).  One
// thread per block; neighbouring threads own neighbouring `post` positions.
// The layouts the linears consume have their own, faster kernels above; these
// serve every other layout the helper functions accept.
// ---------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float block_amax(const T* base, int64_t bs, int64_t post, int64_t vnni) {
  // max = |first|, then std::max(max, |v|) as the CPU path has it
  float amax = fabsf(load_as_f32<T>(base, 0));
  for (int64_t k = 0; k < bs; k++)
    for (int64_t v = 0; v < vnni; v++) {
      const float a = fabsf(load_as_f32<T>(base, k * post * vnni + v));
      amax = a > amax ? a : amax;
    }
  return amax;
}

template <typename T, int FMT>
__global__ void __launch_bounds__(256)
quantize_per_block_kernel(const T* __restrict__ in, int64_t pre, int64_t bs, int64_t post, int64_t vnni,
                          uint8_t* __restrict__ out, void* __restrict__ scales) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= pre * post)
    return;
  const int64_t i = t / post, j = t - i * post;
  const T* base = in + (i * bs * post + j) * vnni;
  const float amax = block_amax<T>(base, bs, post, vnni);
  if (FMT == TPPX_Q_MXFP4) {
    const int e = (int)((__float_as_uint(amax) >> 23) & 0xffu);
    const bool flush = (e == 0);
    const int x = (e == 255) ? 255 : (e - 2 < 0 ? 0 : e - 2);
    reinterpret_cast<uint8_t*>(scales)[t] = (uint8_t)x;
    const int sh = 127 - x;
    const int64_t pv = vnni / 2;
    for (int64_t k = 0; k < bs; k++)
      for (int64_t v1 = 0; v1 < pv; v1++) {
        uint32_t c0 = 0, c1 = 0;
        if (!flush && x != 255) {
          c0 = e2m1_encode(ldexpf(load_as_f32<T>(base, k * post * vnni + 2 * v1), sh));
          c1 = e2m1_encode(ldexpf(load_as_f32<T>(base, k * post * vnni + 2 * v1 + 1), sh));
        }
        out[(i * bs * post + k * post + j) * pv + v1] = (uint8_t)(c0 | (c1 << 4));
      }
  } else if (FMT == TPPX_Q_INT8) {
    const float s = int8_scale_of(amax), inv = int8_inv_scale(s);
    reinterpret_cast<float*>(scales)[t] = s;
    for (int64_t k = 0; k < bs; k++)
      for (int64_t v = 0; v < vnni; v++)
        reinterpret_cast<int8_t*>(out)[(i * bs * post + k * post + j) * vnni + v] =
            (int8_t)int8_q(load_as_f32<T>(base, k * post * vnni + v), inv);
  } else { // INT4: scale = max / 7.0 in double, codes in [-8, 7], two per byte
    const float s = (float)((double)amax / 7.0), inv = int8_inv_scale(s);
    reinterpret_cast<float*>(scales)[t] = s;
    const int64_t pv = vnni / 2;
    for (int64_t k = 0; k < bs; k++)
      for (int64_t v1 = 0; v1 < pv; v1++) {
        uint32_t packed = 0;
#pragma unroll
        for (int v2 = 0; v2 < 2; v2++) {
          float r = rintf(__fmul_rn(load_as_f32<T>(base, k * post * vnni + 2 * v1 + v2), inv));
          r = fminf(fmaxf(r, -8.0f), 7.0f);
          packed |= ((uint32_t)(int)r & 0xfu) << (4 * v2);
        }
        out[(i * bs * post + k * post + j) * pv + v1] = (uint8_t)packed;
      }
  }
}

template <int FMT>
__global__ void __launch_bounds__(256)
dequantize_per_block_kernel(const uint8_t* __restrict__ q, const void* __restrict__ scales, int64_t pre, int64_t bs,
                            int64_t post, int64_t vnni, float* __restrict__ out) {
  // one thread per stored byte
  const int64_t pv = FMT == TPPX_Q_INT8 ? vnni : vnni / 2;
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= pre * bs * post * pv)
    return;
  const int64_t j = (t / pv) % post, i = t / (pv * post * bs);
  const uint32_t b = q[t];
  if (FMT == TPPX_Q_INT8) {
    out[t] = (float)(int8_t)b * reinterpret_cast<const float*>(scales)[i * post + j];
  } else if (FMT == TPPX_Q_MXFP4) {
    const float s = e8m0_to_f32(reinterpret_cast<const uint8_t*>(scales)[i * post + j]);
    out[2 * t] = c_e2m1_tbl[b & 0xf] * s;
    out[2 * t + 1] = c_e2m1_tbl[b >> 4] * s;
  } else {
    const float s = reinterpret_cast<const float*>(scales)[i * post + j];
    out[2 * t] = (float)(((int)(b & 0xf) ^ 8) - 8) * s; // two's complement nibbles
    out[2 * t + 1] = (float)(((int)(b >> 4) ^ 8) - 8) * s;
  }
}

// ---------------------------------------------------------------------------
// QINT2 interleaved (ternary) weights: one wave per (output channel, block of
// bs input channels).  scale = max(|w|, 1e-8) over the block, t = rne(w / scale)
// clamped to [-1, 1], code 0 / 1 / 2 for 0 / +1 / -1; byte [n1][b][c2][k2][c3]
// carries the codes of channels n1*32 + k3*8 + k2 (k3 = 0..3 at bits 2*k3) at
// input channel b*bs + c2*4 + c3.  The four channels of a byte belong to four
// different waves, so the bytes are assembled with atomic ORs on zeroed memory.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256) fill_zero_kernel(uint32_t* __restrict__ p, int64_t n) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n)
    p[t] = 0u;
}

template <typename T>
__global__ void __launch_bounds__(256)
quantize_qint2_kernel(const T* __restrict__ w, int64_t N, int64_t K, int64_t bk, int64_t bc, int64_t vnni, int64_t bs,
                      uint32_t* __restrict__ q32, float* __restrict__ scales) {
  const int64_t nb = K / bs;
  const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int lane = threadIdx.x & 63;
  if (wave >= N * nb)
    return;
  const int64_t r = wave & 31, rest = wave >> 5;
  const int64_t b = rest % nb, n1 = rest / nb;
  const int64_t n = n1 * 32 + r;
  float amax = 0.0f;
  for (int64_t c = lane; c < bs; c += 64)
    amax = fmaxf(amax, fabsf(load_as_f32<T>(w, blocked_off(n, b * bs + c, K, bk, bc, vnni))));
  amax = wave_max(amax);
  const float s = fmaxf(amax, 1.0e-8f);
  if (lane == 0)
    scales[(n1 * nb + b) * 32 + r] = s;
  const int k3 = (int)(r >> 3), k2 = (int)(r & 7);
  // a lane owns whole groups of 4 input channels = one byte position (c2, k2): 4 codes at bits 2*k3 of 4 bytes
  for (int64_t c2 = lane; c2 < bs / 4; c2 += 64) {
    uint32_t word = 0;
#pragma unroll
    for (int c3 = 0; c3 < 4; c3++) {
      const float t = rintf(__fdiv_rn(load_as_f32<T>(w, blocked_off(n, b * bs + c2 * 4 + c3, K, bk, bc, vnni)), s));
      const uint32_t code = t >= 1.0f ? 1u : (t <= -1.0f ? 2u : 0u);
      word |= (code << (2 * k3)) << (8 * c3);
    }
    if (word)
      atomicOr(&q32[((n1 * nb + b) * (bs / 4) + c2) * 8 + k2], word);
  }
}

// packed 2-bit (interleaved) -> native int8 tiles of the W8A8 kernels + scales [N/16][K/bs][16];
// one thread per native 16-byte chunk (nt, kt, g, n16): input channels kt*64 + g*16 .. +15 of channel nt*16 + n16
__global__ void __launch_bounds__(256)
prepack_qint2_kernel(const uint8_t* __restrict__ q2, const float* __restrict__ s2, int64_t N, int64_t K, int64_t bs,
                     int8_t* __restrict__ qnat, float* __restrict__ snat) {
  const int64_t nchunks = N * (K / 16);
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= nchunks)
    return;
  const int64_t n16 = t & 15, g = (t >> 4) & 3, rest = t >> 6;
  const int64_t KT = K / 64, nb = K / bs;
  const int64_t kt = rest % KT, nt = rest / KT;
  const int64_t n = nt * 16 + n16, k0 = kt * 64 + g * 16;
  const int64_t n1 = n >> 5, r = n & 31, k3 = r >> 3, k2 = r & 7;
  const int64_t b = k0 / bs, c2 = (k0 % bs) >> 2;
  const uint32_t* src = reinterpret_cast<const uint32_t*>(q2) + ((n1 * nb + b) * (bs / 4) + c2) * 8 + k2;
  uint32_t o[4];
#pragma unroll
  for (int d = 0; d < 4; d++) {
    const uint32_t codes = (src[d * 8] >> (2 * k3)) & 0x03030303u; // the four input channels c3 of group c2 + d
    // 0 -> 0x00, 1 -> 0x01, 2 -> 0xff (-1) per byte
    o[d] = __builtin_amdgcn_perm(0u, 0x00ff0100u, codes);
  }
  reinterpret_cast<uint4*>(qnat)[t] = make_uint4(o[0], o[1], o[2], o[3]);
  if (g == 0 && (kt * 64) % bs == 0)
    snat[(nt * nb + b) * 16 + n16] = s2[(n1 * nb + b) * 32 + r];
}

// packed 2-bit (interleaved) -> fp32 in the logical blocked shape [N/32][K/bs][bs/4][32][4]; one thread per output
__global__ void __launch_bounds__(256)
dequantize_qint2_kernel(const uint8_t* __restrict__ q2, const float* __restrict__ s2, int64_t total, int64_t bs,
                        float* __restrict__ out) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= total)
    return;
  const int64_t c3 = t & 3, r = (t >> 2) & 31, rest = t >> 7; // rest = (n1*nb + b) * (bs/4) + c2
  const int64_t blk = rest / (bs / 4);
  const uint32_t byte = q2[(rest * 8 + (r & 7)) * 4 + c3];
  const uint32_t code = (byte >> (2 * (r >> 3))) & 3u;
  out[t] = (code == 1 ? 1.0f : (code == 2 ? -1.0f : 0.0f)) * s2[blk * 32 + r];
}

// INT4 weight in the VNNI2 layout [N/16][K/bs][bs/2][16][2 codes per byte] -> native int8 tiles
__global__ void __launch_bounds__(256)
prepack_qint4_kernel(const uint8_t* __restrict__ q4, int64_t N, int64_t K, int64_t bs, int8_t* __restrict__ qnat) {
  const int64_t nchunks = N * (K / 16);
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= nchunks)
    return;
  const int64_t n16 = t & 15, g = (t >> 4) & 3, rest = t >> 6;
  const int64_t KT = K / 64, nb = K / bs;
  const int64_t kt = rest % KT, nt = rest / KT;
  const int64_t k0 = kt * 64 + g * 16;
  const int64_t b = k0 / bs, a0 = (k0 % bs) >> 1; // pair index inside the block
  const uint8_t* src = q4 + ((nt * nb + b) * (bs / 2) + a0) * 16 + n16;
  uint32_t o[4];
#pragma unroll
  for (int d = 0; d < 4; d++) {
    uint32_t word = 0;
#pragma unroll
    for (int pr = 0; pr < 2; pr++) {
      const uint32_t byte = src[(d * 2 + pr) * 16];
      const uint32_t lo = (uint32_t)((((int)(byte & 0xf) ^ 8) - 8) & 0xff), hi = (uint32_t)((((int)(byte >> 4) ^ 8) - 8) & 0xff);
      word |= (lo | (hi << 8)) << (16 * pr);
    }
    o[d] = word;
  }
  reinterpret_cast<uint4*>(qnat)[t] = make_uint4(o[0], o[1], o[2], o[3]);
}

// W4A8 weight (remap_and_quantize_mxfp4 under USE_MXFP4_INT8: q u8 [N/8][K/bc][bc/8][8][4], byte i of a group of 8
// K values = value i | value 4 + i << 4; scales u8 [N/8][K/bc][bc/32][8]) -> the decode kernel's tiles:
// q [N/16][K/128][64 lanes][4 dwords], lane = (channel c = lane & 15, K group kg = lane >> 4), dword j = the
// reference's dword of K group kg of MX block j of the tile; scales [N/16][K/128][16 c] dwords of the tile's four
// E8M0 bytes.  One thread per (tile, lane).
__global__ void __launch_bounds__(256)
prepack_w4a8_kernel(const uint32_t* __restrict__ qref, const uint8_t* __restrict__ sref, int64_t N, int64_t K, int64_t bc,
                    uint32_t* __restrict__ qnat, uint32_t* __restrict__ snat) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t KT = K / 128;
  if (t >= (N / 16) * KT * 64)
    return;
  const int lane = (int)(t & 63), c = lane & 15, kg = lane >> 4;
  const int64_t tile = t >> 6, kt = tile % KT, ntile = tile / KT;
  const int64_t n = ntile * 16 + c, n8b = n >> 3, n8 = n & 7;
  const int64_t C1 = K / bc, G = bc / 8, SB = bc / 32;
  uint32_t w[4], sc = 0;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int64_t k0 = (kt * 4 + j) * 32, c1 = k0 / bc, kb = k0 % bc;
    w[j] = qref[(((n8b * C1 + c1) * G + (kb >> 3) + kg) * 8 + n8)];
    sc |= (uint32_t)sref[((n8b * C1 + c1) * SB + (kb >> 5)) * 8 + n8] << (8 * j);
  }
  reinterpret_cast<uint4*>(qnat)[t] = make_uint4(w[0], w[1], w[2], w[3]);
  if (kg == 0)
    snat[tile * 16 + c] = sc;
}

// Native int8 tiles [N/16][K/64][64 lanes][16 B] of a QINT4 / QINT2 weight -> the codes at their own width, for the
// decode kernel that expands them in registers: [N/16][K/(64 G)][64 lanes][16 B], G = 8 / BITS tiles per 16 bytes.
//   BITS 4: byte b of dword d = (tile 0's byte d*4+b & 15) | (tile 1's byte d*4+b << 4)        (values -8..7)
//   BITS 2: byte i of dword kt = two's-complement 2-bit codes (0, 1, 3 = -1) of tile kt's bytes i, 4+i, 8+i, 12+i
//           (byte i of its four operand dwords) in bits 0-1, 2-3, 4-5, 6-7
template <int BITS>
__global__ void __launch_bounds__(256)
pack_qint_tiles_kernel(const int8_t* __restrict__ nat, int64_t groups, uint8_t* __restrict__ out) {
  constexpr int G = 8 / BITS;
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; // (tile group, lane)
  if (t >= groups * 64)
    return;
  const int64_t grp = t >> 6;
  const int lane = (int)(t & 63);
  int8_t v[G][16];
#pragma unroll
  for (int g = 0; g < G; g++) {
    const uint4 w = reinterpret_cast<const uint4*>(nat)[(grp * G + g) * 64 + lane];
    const uint32_t d[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 16; i++)
      v[g][i] = (int8_t)((d[i >> 2] >> (8 * (i & 3))) & 0xffu);
  }
  uint32_t o[4] = {0, 0, 0, 0};
  if (BITS == 4) {
#pragma unroll
    for (int i = 0; i < 16; i++)
      o[i >> 2] |= (((uint32_t)v[0][i] & 15u) | (((uint32_t)v[G - 1][i] & 15u) << 4)) << (8 * (i & 3));
  } else {
#pragma unroll
    for (int kt = 0; kt < G; kt++)
#pragma unroll
      for (int i = 0; i < 16; i++) // value i = byte i & 3 of operand dword i >> 2
        o[kt & 3] |= ((uint32_t)v[kt][i] & 3u) << (8 * (i & 3) + 2 * (i >> 2));
  }
  reinterpret_cast<uint4*>(out)[t] = make_uint4(o[0], o[1], o[2], o[3]);
}

static inline unsigned grid_for(int64_t n, int block) {
  return (unsigned)((n + block - 1) / block);
}

hipError_t launch_quant_act_int8(const void* x, int64_t M, int64_t K, int64_t qbs, void* xq, void* sa, int mt,
                                 hipStream_t stream) {
  // 16 lanes per (row, block) -- 32-byte reads, one 16-byte write per lane -- from 128 rows on, and for the operand-
  // order output of the decode kernels (17..64 rows) whatever the row count; a whole wave per (row, block) otherwise
  if (qbs == 256 && (M >= 128 || mt > 0) && env_int("TPPX_QUANT_ROWS16", 1) != 0) {
    const int64_t nt16 = M * (K / 256) * 16;
    TPPX_PLAN_ONLY(quant_act_int8_rows_kernel, dim3(grid_for(nt16, 256)), dim3(256), 0);
    quant_act_int8_rows_kernel<<<grid_for(nt16, 256), 256, 0, stream>>>((const uint16_t*)x, M, K, (int8_t*)xq, (float*)sa, mt);
    return hipGetLastError();
  }
  if (qbs > 256 && qbs % 256 == 0 && M * (K / qbs) < (1 << 30)) {
    const int64_t lanes = (qbs >> 8) * 16;
    const unsigned block = (unsigned)(lanes >= 1024 ? 1024 : (lanes + 63) / 64 * 64);
    const dim3 grid((unsigned)(M * (K / qbs)));
    TPPX_PLAN_ONLY(quant_act_int8_bigblk_kernel, grid, dim3(block), 0);
    quant_act_int8_bigblk_kernel<<<grid, block, 0, stream>>>((const uint16_t*)x, M, K, qbs, (int8_t*)xq, (float*)sa, mt);
    return hipGetLastError();
  }
  int64_t nthreads = M * (K / qbs) * 64;
  TPPX_PLAN_ONLY(quant_act_int8_kernel, dim3(grid_for(nthreads, 256)), dim3(256), 0);
  quant_act_int8_kernel<<<grid_for(nthreads, 256), 256, 0, stream>>>((const uint16_t*)x, M, K, qbs, (int8_t*)xq,
                                                                    (float*)sa, mt);
  return hipGetLastError();
}

hipError_t launch_quant_act_mxfp8(const void* x, int64_t M, int64_t K, void* xq, void* xs, hipStream_t stream) {
  const int64_t nthreads = (M + 63) / 64 * 4 * (K / 128) * 128; // a wave per half tile
  TPPX_PLAN_ONLY(quant_act_mxfp8_kernel, dim3(grid_for(nthreads, 256)), dim3(256), 0);
  quant_act_mxfp8_kernel<<<grid_for(nthreads, 256), 256, 0, stream>>>((const uint16_t*)x, M, K, (uint8_t*)xq, (uint8_t*)xs);
  return hipGetLastError();
}

} // namespace tppx

using namespace tppx;

extern "C" int tppx_quantize_mxfp4(const void* w, int w_dtype, int64_t N,
                                   int64_t K, int64_t bk, int64_t bc,
                                   int64_t vnni, void* qdata, void* scales,
                                   tppx_stream_t stream) {
  TPPX_REQUIRE(w && qdata && scales, TPPX_EINVAL, "tppx_quantize_mxfp4: null pointer");
  TPPX_REQUIRE(w_dtype == TPPX_DT_F32 || w_dtype == TPPX_DT_BF16, TPPX_EINVAL,
               "tppx_quantize_mxfp4: unknown weight dtype %d", w_dtype);
  TPPX_REQUIRE(N > 0 && K > 0 && N % 32 == 0 && K % 64 == 0, TPPX_ESHAPE,
               "tppx_quantize_mxfp4: shape not compatible for MXFP4 (N=%ld must be a multiple of 32, K=%ld of 64)",
               (long)N, (long)K);
  TPPX_REQUIRE(bk > 0 && bc > 0 && vnni > 0 && N % bk == 0 && K % bc == 0 && bc % vnni == 0,
               TPPX_ESHAPE, "tppx_quantize_mxfp4: blocking (bk=%ld, bc=%ld, vnni=%ld) does not divide [%ld,%ld]",
               (long)bk, (long)bc, (long)vnni, (long)N, (long)K);
  int64_t nblk = N * (K / 32);
  hipStream_t s = (hipStream_t)stream;
  if (w_dtype == TPPX_DT_F32)
    quantize_mxfp4_kernel<float><<<grid_for(nblk, 256), 256, 0, s>>>(
        (const float*)w, N, K, bk, bc, vnni, (uint8_t*)qdata, (uint8_t*)scales);
  else
    quantize_mxfp4_kernel<uint16_t><<<grid_for(nblk, 256), 256, 0, s>>>(
        (const uint16_t*)w, N, K, bk, bc, vnni, (uint8_t*)qdata, (uint8_t*)scales);
  return check_hip(hipGetLastError(), "tppx_quantize_mxfp4");
}

extern "C" int tppx_quantize_qint8(const void* w, int w_dtype, int64_t N,
                                   int64_t K, int64_t bk, int64_t bc,
                                   int64_t vnni, int64_t qbs, void* q,
                                   void* scales, tppx_stream_t stream) {
  TPPX_REQUIRE(w && q && scales, TPPX_EINVAL, "tppx_quantize_qint8: null pointer");
  TPPX_REQUIRE(w_dtype == TPPX_DT_F32 || w_dtype == TPPX_DT_BF16, TPPX_EINVAL,
               "tppx_quantize_qint8: unknown weight dtype %d", w_dtype);
  TPPX_REQUIRE(N > 0 && K > 0 && N % 16 == 0 && K % 64 == 0, TPPX_ESHAPE,
               "tppx_quantize_qint8: N=%ld must be a multiple of 16 and K=%ld of 64", (long)N, (long)K);
  TPPX_REQUIRE(qbs > 0 && qbs % 64 == 0 && K % qbs == 0, TPPX_ESHAPE,
               "tppx_quantize_qint8: block size %ld must be a multiple of 64 dividing K=%ld", (long)qbs, (long)K);
  TPPX_REQUIRE(bk > 0 && bc > 0 && vnni > 0 && N % bk == 0 && K % bc == 0 && bc % vnni == 0,
               TPPX_ESHAPE, "tppx_quantize_qint8: blocking (bk=%ld, bc=%ld, vnni=%ld) does not divide [%ld,%ld]",
               (long)bk, (long)bc, (long)vnni, (long)N, (long)K);
  int64_t nthreads = N * (K / qbs) * 64;
  hipStream_t s = (hipStream_t)stream;
  if (w_dtype == TPPX_DT_F32)
    quantize_qint8_kernel<float><<<grid_for(nthreads, 256), 256, 0, s>>>(
        (const float*)w, N, K, bk, bc, vnni, qbs, (int8_t*)q, (float*)scales);
  else
    quantize_qint8_kernel<uint16_t><<<grid_for(nthreads, 256), 256, 0, s>>>(
        (const uint16_t*)w, N, K, bk, bc, vnni, qbs, (int8_t*)q, (float*)scales);
  return check_hip(hipGetLastError(), "tppx_quantize_qint8");
}

extern "C" int tppx_dequantize_mxfp4(const void* qdata, const void* scales,
                                     int64_t N, int64_t K, void* out_f32,
                                     tppx_stream_t stream) {
  TPPX_REQUIRE(qdata && scales && out_f32, TPPX_EINVAL, "tppx_dequantize_mxfp4: null pointer");
  TPPX_REQUIRE(N > 0 && K > 0 && N % 32 == 0 && K % 64 == 0, TPPX_ESHAPE,
               "tppx_dequantize_mxfp4: N=%ld must be a multiple of 32 and K=%ld of 64", (long)N, (long)K);
  int64_t nbytes = N * K / 2;
  dequantize_mxfp4_kernel<<<grid_for(nbytes, 256), 256, 0, (hipStream_t)stream>>>(
      (const uint8_t*)qdata, (const uint8_t*)scales, nbytes, (float*)out_f32);
  return check_hip(hipGetLastError(), "tppx_dequantize_mxfp4");
}

extern "C" int tppx_dequantize_qint8(const void* q, const void* scales,
                                     int64_t N, int64_t K, int64_t qbs,
                                     void* out_f32, tppx_stream_t stream) {
  TPPX_REQUIRE(q && scales && out_f32, TPPX_EINVAL, "tppx_dequantize_qint8: null pointer");
  TPPX_REQUIRE(N > 0 && K > 0 && N % 16 == 0 && qbs > 0 && qbs % 4 == 0 && K % qbs == 0,
               TPPX_ESHAPE, "tppx_dequantize_qint8: bad shape N=%ld K=%ld qbs=%ld", (long)N, (long)K, (long)qbs);
  int64_t ngroups = N * K / 4;
  dequantize_qint8_kernel<<<grid_for(ngroups, 256), 256, 0, (hipStream_t)stream>>>(
      (const int8_t*)q, (const float*)scales, ngroups, qbs, (float*)out_f32);
  return check_hip(hipGetLastError(), "tppx_dequantize_qint8");
}

extern "C" int tppx_prepack_mxfp4(const void* qdata_ref, const void* scales_ref,
                                  int64_t N, int64_t K, void* qdata_nat,
                                  void* scales_nat, tppx_stream_t stream) {
  TPPX_REQUIRE(qdata_ref && scales_ref && qdata_nat && scales_nat, TPPX_EINVAL,
               "tppx_prepack_mxfp4: null pointer");
  TPPX_REQUIRE(aligned16(qdata_nat), TPPX_EINVAL, "tppx_prepack_mxfp4: output not 16-byte aligned");
  TPPX_REQUIRE(N > 0 && K > 0 && N % 32 == 0 && K % 128 == 0, TPPX_ESHAPE,
               "tppx_prepack_mxfp4: N=%ld must be a multiple of 32 and K=%ld of 128", (long)N, (long)K);
  int64_t nchunks = N * (K / 32);
  prepack_mxfp4_kernel<<<grid_for(nchunks, 256), 256, 0, (hipStream_t)stream>>>(
      (const uint8_t*)qdata_ref, (const uint8_t*)scales_ref, N, K,
      (uint8_t*)qdata_nat, (uint8_t*)scales_nat);
  return check_hip(hipGetLastError(), "tppx_prepack_mxfp4");
}

extern "C" int tppx_prepack_qint8(const void* q_ref, int64_t N, int64_t K,
                                  int64_t qbs, void* q_nat,
                                  tppx_stream_t stream) {
  TPPX_REQUIRE(q_ref && q_nat, TPPX_EINVAL, "tppx_prepack_qint8: null pointer");
  TPPX_REQUIRE(aligned16(q_nat) && aligned16(q_ref), TPPX_EINVAL, "tppx_prepack_qint8: pointer not 16-byte aligned");
  TPPX_REQUIRE(N > 0 && K > 0 && N % 16 == 0 && qbs > 0 && qbs % 64 == 0 && K % qbs == 0,
               TPPX_ESHAPE, "tppx_prepack_qint8: bad shape N=%ld K=%ld qbs=%ld", (long)N, (long)K, (long)qbs);
  int64_t nchunks = N * (K / 16);
  prepack_qint8_kernel<<<grid_for(nchunks, 256), 256, 0, (hipStream_t)stream>>>(
      (const int8_t*)q_ref, N, K, qbs, (int8_t*)q_nat);
  return check_hip(hipGetLastError(), "tppx_prepack_qint8");
}

extern "C" int tppx_prepack_mxfp4_int8(const void* q_ref, const void* sc_ref, int64_t N, int64_t K, int64_t bc,
                                       void* q_nat, void* s_nat, tppx_stream_t stream) {
  const char* who = "tppx_prepack_mxfp4_int8";
  TPPX_REQUIRE(q_ref && sc_ref && q_nat && s_nat, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(aligned16(q_nat) && ((uintptr_t)q_ref & 3) == 0 && ((uintptr_t)s_nat & 3) == 0, TPPX_EINVAL, "%s: pointer misaligned", who);
  TPPX_REQUIRE(N > 0 && N % 16 == 0 && K > 0 && K % 128 == 0 && bc >= 32 && bc % 32 == 0 && K % bc == 0, TPPX_ESHAPE,
               "%s: N=%ld must be a multiple of 16, K=%ld of 128 and of the block %ld (a multiple of 32)", who, (long)N, (long)K, (long)bc);
  const int64_t threads = (N / 16) * (K / 128) * 64;
  prepack_w4a8_kernel<<<grid_for(threads, 256), 256, 0, (hipStream_t)stream>>>((const uint32_t*)q_ref, (const uint8_t*)sc_ref,
                                                                              N, K, bc, (uint32_t*)q_nat, (uint32_t*)s_nat);
  return check_hip(hipGetLastError(), who);
}

extern "C" int tppx_pack_qint_tiles(const void* native_i8, int64_t N, int64_t K, int bits, void* packed,
                                    tppx_stream_t stream) {
  const char* who = "tppx_pack_qint_tiles";
  TPPX_REQUIRE(native_i8 && packed, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(aligned16(native_i8) && aligned16(packed), TPPX_EINVAL, "%s: pointer not 16-byte aligned", who);
  TPPX_REQUIRE(bits == 4 || bits == 2, TPPX_EINVAL, "%s: %d-bit codes are not built (4 or 2)", who, bits);
  TPPX_REQUIRE(N > 0 && N % 16 == 0 && K > 0 && K % 256 == 0, TPPX_ESHAPE, "%s: N=%ld must be a multiple of 16 and K=%ld of 256", who, (long)N, (long)K);
  const int64_t groups = (N / 16) * (K / 64) / (8 / bits);
  if (bits == 4)
    pack_qint_tiles_kernel<4><<<grid_for(groups * 64, 256), 256, 0, (hipStream_t)stream>>>((const int8_t*)native_i8, groups, (uint8_t*)packed);
  else
    pack_qint_tiles_kernel<2><<<grid_for(groups * 64, 256), 256, 0, (hipStream_t)stream>>>((const int8_t*)native_i8, groups, (uint8_t*)packed);
  return check_hip(hipGetLastError(), who);
}

extern "C" int tppx_prepack_bf16(const void* w_ref, int64_t N, int64_t K, int64_t bk, int64_t bc, int vnni,
                                 void* w_nat, tppx_stream_t stream) {
  TPPX_REQUIRE(w_ref && w_nat, TPPX_EINVAL, "tppx_prepack_bf16: null pointer");
  TPPX_REQUIRE(aligned16(w_nat), TPPX_EINVAL, "tppx_prepack_bf16: output not 16-byte aligned");
  TPPX_REQUIRE(N > 0 && K > 0 && N % 16 == 0 && K % 128 == 0, TPPX_ESHAPE,
               "tppx_prepack_bf16: N=%ld must be a multiple of 16 and K=%ld of 128", (long)N, (long)K);
  TPPX_REQUIRE(bk > 0 && bc > 0 && (vnni == 1 || vnni == 2) && N % bk == 0 && K % bc == 0 && bc % vnni == 0, TPPX_ESHAPE,
               "tppx_prepack_bf16: blocking bk=%ld bc=%ld vnni=%d does not divide N=%ld K=%ld", (long)bk, (long)bc, vnni,
               (long)N, (long)K);
  const int64_t nchunks = N * (K / 8);
  prepack_bf16_kernel<<<grid_for(nchunks, 256), 256, 0, (hipStream_t)stream>>>((const uint16_t*)w_ref, N, K, bk, bc, vnni,
                                                                                (uint16_t*)w_nat);
  return check_hip(hipGetLastError(), "tppx_prepack_bf16");
}

extern "C" int tppx_quant_act_mxfp8(const void* x, int64_t M, int64_t K, void* xq, void* xs, tppx_stream_t stream) {
  TPPX_REQUIRE(x && xq && xs, TPPX_EINVAL, "tppx_quant_act_mxfp8: null pointer");
  TPPX_REQUIRE(aligned16(x) && aligned16(xq), TPPX_EINVAL, "tppx_quant_act_mxfp8: pointer not 16-byte aligned");
  TPPX_REQUIRE(M > 0 && K > 0 && K % 128 == 0, TPPX_ESHAPE, "tppx_quant_act_mxfp8: bad shape M=%ld K=%ld (K in multiples of 128)", (long)M, (long)K);
  return check_hip(launch_quant_act_mxfp8(x, M, K, xq, xs, (hipStream_t)stream), "tppx_quant_act_mxfp8");
}

extern "C" int tppx_quant_act_int8(const void* x, int64_t M, int64_t K,
                                   int64_t qbs, void* xq, void* sa,
                                   tppx_stream_t stream) {
  TPPX_REQUIRE(x && xq && sa, TPPX_EINVAL, "tppx_quant_act_int8: null pointer");
  TPPX_REQUIRE(aligned16(x) && aligned16(xq), TPPX_EINVAL, "tppx_quant_act_int8: pointer not 16-byte aligned");
  TPPX_REQUIRE(M > 0 && K > 0 && qbs > 0 && qbs % 64 == 0 && K % qbs == 0, TPPX_ESHAPE,
               "tppx_quant_act_int8: bad shape M=%ld K=%ld qbs=%ld", (long)M, (long)K, (long)qbs);
  return check_hip(launch_quant_act_int8(x, M, K, qbs, xq, sa, 0, (hipStream_t)stream), "tppx_quant_act_int8");
}

// ---- generic helpers ---------------------------------------------------------
static int check_per_block(const char* who, int qfmt, int64_t pre, int64_t bs, int64_t post, int64_t vnni) {
  TPPX_REQUIRE(qfmt == TPPX_Q_MXFP4 || qfmt == TPPX_Q_INT8 || qfmt == TPPX_Q_INT4, TPPX_EINVAL, "%s: unknown format id %d", who, qfmt);
  TPPX_REQUIRE(pre > 0 && bs > 0 && post > 0 && vnni > 0, TPPX_ESHAPE, "%s: bad geometry pre=%ld bs=%ld post=%ld vnni=%ld", who,
               (long)pre, (long)bs, (long)post, (long)vnni);
  TPPX_REQUIRE(qfmt == TPPX_Q_INT8 || vnni % 2 == 0, TPPX_ESHAPE, "%s: 4-bit formats pack two codes per byte: vnni=%ld must be even", who, (long)vnni);
  TPPX_REQUIRE(pre * bs * post * vnni < ((int64_t)1 << 40), TPPX_ESHAPE, "%s: tensor too large", who);
  return TPPX_OK;
}

extern "C" int tppx_quantize_per_block(const void* in, int in_dtype, int qfmt, int64_t pre, int64_t bs, int64_t post,
                                       int64_t vnni, void* out, void* scales, tppx_stream_t stream) {
  const char* who = "tppx_quantize_per_block";
  TPPX_REQUIRE(in && out && scales, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(in_dtype == TPPX_DT_F32 || in_dtype == TPPX_DT_BF16, TPPX_EINVAL, "%s: unknown input dtype %d", who, in_dtype);
  if (int rc = check_per_block(who, qfmt, pre, bs, post, vnni))
    return rc;
  hipStream_t s = (hipStream_t)stream;
  const unsigned grid = grid_for(pre * post, 256);
#define TPPX_QPB(T, F) quantize_per_block_kernel<T, F><<<grid, 256, 0, s>>>((const T*)in, pre, bs, post, vnni, (uint8_t*)out, scales)
  if (in_dtype == TPPX_DT_F32) {
    if (qfmt == TPPX_Q_MXFP4) TPPX_QPB(float, TPPX_Q_MXFP4);
    else if (qfmt == TPPX_Q_INT8) TPPX_QPB(float, TPPX_Q_INT8);
    else TPPX_QPB(float, TPPX_Q_INT4);
  } else {
    if (qfmt == TPPX_Q_MXFP4) TPPX_QPB(uint16_t, TPPX_Q_MXFP4);
    else if (qfmt == TPPX_Q_INT8) TPPX_QPB(uint16_t, TPPX_Q_INT8);
    else TPPX_QPB(uint16_t, TPPX_Q_INT4);
  }
#undef TPPX_QPB
  return check_hip(hipGetLastError(), who);
}

extern "C" int tppx_dequantize_per_block(const void* q, const void* scales, int qfmt, int64_t pre, int64_t bs,
                                         int64_t post, int64_t vnni, void* out_f32, tppx_stream_t stream) {
  const char* who = "tppx_dequantize_per_block";
  TPPX_REQUIRE(q && scales && out_f32, TPPX_EINVAL, "%s: null pointer", who);
  if (int rc = check_per_block(who, qfmt, pre, bs, post, vnni))
    return rc;
  hipStream_t s = (hipStream_t)stream;
  const int64_t nbytes = pre * bs * post * (qfmt == TPPX_Q_INT8 ? vnni : vnni / 2);
  if (qfmt == TPPX_Q_MXFP4)
    dequantize_per_block_kernel<TPPX_Q_MXFP4><<<grid_for(nbytes, 256), 256, 0, s>>>((const uint8_t*)q, scales, pre, bs, post, vnni, (float*)out_f32);
  else if (qfmt == TPPX_Q_INT8)
    dequantize_per_block_kernel<TPPX_Q_INT8><<<grid_for(nbytes, 256), 256, 0, s>>>((const uint8_t*)q, scales, pre, bs, post, vnni, (float*)out_f32);
  else
    dequantize_per_block_kernel<TPPX_Q_INT4><<<grid_for(nbytes, 256), 256, 0, s>>>((const uint8_t*)q, scales, pre, bs, post, vnni, (float*)out_f32);
  return check_hip(hipGetLastError(), who);
}

static int check_qint2(const char* who, int64_t N, int64_t K, int64_t bs) {
  TPPX_REQUIRE(N > 0 && K > 0 && N % 32 == 0, TPPX_ESHAPE, "%s: N=%ld must be a positive multiple of 32", who, (long)N);
  TPPX_REQUIRE(bs > 0 && bs % 64 == 0 && K % bs == 0, TPPX_ESHAPE, "%s: block size %ld must be a multiple of 64 dividing K=%ld", who, (long)bs, (long)K);
  return TPPX_OK;
}

extern "C" int tppx_quantize_qint2_intlv(const void* w, int w_dtype, int64_t N, int64_t K, int64_t bk, int64_t bc,
                                         int64_t vnni, int64_t bs, void* q, void* scales, tppx_stream_t stream) {
  const char* who = "tppx_quantize_qint2_intlv";
  TPPX_REQUIRE(w && q && scales, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(w_dtype == TPPX_DT_F32 || w_dtype == TPPX_DT_BF16, TPPX_EINVAL, "%s: unknown weight dtype %d", who, w_dtype);
  TPPX_REQUIRE((reinterpret_cast<uintptr_t>(q) & 3u) == 0, TPPX_EINVAL, "%s: output not 4-byte aligned", who);
  if (int rc = check_qint2(who, N, K, bs))
    return rc;
  TPPX_REQUIRE(bk > 0 && bc > 0 && vnni > 0 && N % bk == 0 && K % bc == 0 && bc % vnni == 0, TPPX_ESHAPE,
               "%s: blocking (bk=%ld, bc=%ld, vnni=%ld) does not divide [%ld,%ld]", who, (long)bk, (long)bc, (long)vnni, (long)N, (long)K);
  hipStream_t s = (hipStream_t)stream;
  // the bytes are assembled with ORs: start from zeros (a fill kernel, so that the call can sit in a captured graph)
  const int64_t nwords = N * K / 16;
  fill_zero_kernel<<<grid_for(nwords, 256), 256, 0, s>>>((uint32_t*)q, nwords);
  const int64_t nthreads = N * (K / bs) * 64;
  if (w_dtype == TPPX_DT_F32)
    quantize_qint2_kernel<float><<<grid_for(nthreads, 256), 256, 0, s>>>((const float*)w, N, K, bk, bc, vnni, bs, (uint32_t*)q, (float*)scales);
  else
    quantize_qint2_kernel<uint16_t><<<grid_for(nthreads, 256), 256, 0, s>>>((const uint16_t*)w, N, K, bk, bc, vnni, bs, (uint32_t*)q, (float*)scales);
  return check_hip(hipGetLastError(), who);
}

extern "C" int tppx_dequantize_qint2_intlv(const void* q, const void* scales, int64_t N, int64_t K, int64_t bs,
                                           void* out_f32, tppx_stream_t stream) {
  const char* who = "tppx_dequantize_qint2_intlv";
  TPPX_REQUIRE(q && scales && out_f32, TPPX_EINVAL, "%s: null pointer", who);
  if (int rc = check_qint2(who, N, K, bs))
    return rc;
  dequantize_qint2_kernel<<<grid_for(N * K, 256), 256, 0, (hipStream_t)stream>>>((const uint8_t*)q, (const float*)scales, N * K, bs, (float*)out_f32);
  return check_hip(hipGetLastError(), who);
}

extern "C" int tppx_prepack_qint2(const void* q_ref, const void* scales_ref, int64_t N, int64_t K, int64_t bs,
                                  void* q_nat, void* scales_nat, tppx_stream_t stream) {
  const char* who = "tppx_prepack_qint2";
  TPPX_REQUIRE(q_ref && scales_ref && q_nat && scales_nat, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(aligned16(q_nat) && (reinterpret_cast<uintptr_t>(q_ref) & 3u) == 0, TPPX_EINVAL, "%s: pointer not aligned", who);
  if (int rc = check_qint2(who, N, K, bs))
    return rc;
  prepack_qint2_kernel<<<grid_for(N * (K / 16), 256), 256, 0, (hipStream_t)stream>>>((const uint8_t*)q_ref, (const float*)scales_ref, N, K, bs,
                                                                                      (int8_t*)q_nat, (float*)scales_nat);
  return check_hip(hipGetLastError(), who);
}

extern "C" int tppx_prepack_qint4(const void* q_ref, int64_t N, int64_t K, int64_t bs, void* q_nat, tppx_stream_t stream) {
  const char* who = "tppx_prepack_qint4";
  TPPX_REQUIRE(q_ref && q_nat, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(aligned16(q_nat), TPPX_EINVAL, "%s: output not 16-byte aligned", who);
  TPPX_REQUIRE(N > 0 && K > 0 && N % 16 == 0 && bs > 0 && bs % 64 == 0 && K % bs == 0, TPPX_ESHAPE, "%s: bad shape N=%ld K=%ld bs=%ld", who,
               (long)N, (long)K, (long)bs);
  prepack_qint4_kernel<<<grid_for(N * (K / 16), 256), 256, 0, (hipStream_t)stream>>>((const uint8_t*)q_ref, N, K, bs, (int8_t*)q_nat);
  return check_hip(hipGetLastError(), who);
}
