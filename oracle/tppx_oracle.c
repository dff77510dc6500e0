/*
 * CPU oracle for the weight-quantized LLM linear path (MXFP4 / QINT8).
 *
 * TEST INFRASTRUCTURE ONLY.  This file is a plain-C restatement of the
 * reference CPU algorithm.  It is compiled into libtppx_oracle.so and used by
 * the test-suite, the smoke check and the CPU-baseline leg of the benchmark as
 * the checker / the timed CPU path.  No product code path may call it.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the reference tree).
 *
 * Pinning status (what independent evidence fixes each function):
 *   orc_mx_scale_byte, orc_mx_quant_scale, orc_e2m1_encode, orc_mxfp4_quantize_generic
 *       -> pinned: golden vectors produced by compiling the reference's own
 *          src/csrc/mxfp_quant.h, OCP-MX known answers, exhaustive bf16 sweep
 *          against an independent nearest/ties-to-even table search.
 *   orc_int8_quantize_generic, orc_quant_act_int8
 *       -> pinned by closed form (max/127, nearbyintf, clamp), |w-q*s| <= s/2,
 *          brute force.
 *   orc_remap_quantize_* / orc_dequantize_*  (layouts)
 *       -> pinned: closed-form index formulas vs. an independent view/permute
 *          restatement with stock torch, byte equality.
 *   orc_linear_qint8_f32
 *       -> pinned: its bf16 rounding equals orc_linear_qint8 (ideal); fp64
 *          evaluation of the formula.
 *   orc_linear_mxfp4 / orc_linear_qint8 (mode ideal)
 *       -> pinned: reduces to torch.matmul in fp64 over the exactly
 *          dequantized weight; int32 partial sums bit-checked.
 *   orc_linear_* (mode faithful): the bf16 re-rounding points follow the
 *       reference source; the fp32 summation ORDER inside libxsmm's JIT
 *       BRGEMM and libxsmm's sigmoid/GELU polynomial are third-party and
 *       absent from the reference tree -> "parity unpinned" for those two
 *       aspects; covered by tolerance, not bit equality.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ */
/* bf16 <-> fp32 (round to nearest even; NaN kept quiet)              */
/* ------------------------------------------------------------------ */
static inline uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline float bf16_to_f32(uint16_t h) {
  return bits_f32((uint32_t)h << 16);
}
static inline uint16_t f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u)
    return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

ORC_API void orc_f32_to_bf16(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; i++)
    out[i] = f32_to_bf16(in[i]);
}
ORC_API void orc_bf16_to_f32(const uint16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; i++)
    out[i] = bf16_to_f32(in[i]);
}

/* ------------------------------------------------------------------ */
/* MXFP4 element / scale math                                          */
/* ------------------------------------------------------------------ */

/* E8M0 scale byte of a block whose largest magnitude is amax.
 * Follows MxFP4Quant(float max) (src/csrc/qtypes.cpp:69-77) ->
 * mx_get_shared_scale (src/csrc/mxfp_quant.h:141-161) with elem_max_norm 6.0
 * (unbiased exponent 2) and clamp_shared_exp (mxfp_quant.h:127-136, ebits 8):
 * X = biased_exp(amax) - 2, below -127 unbiased -> 0, Inf/NaN -> 255. */
ORC_API int orc_mx_scale_byte(float amax) {
  int e = (int)((f32_bits(amax) >> 23) & 0xffu);
  if (e == 255)
    return 255;
  int x = e - 2;
  return x < 0 ? 0 : x;
}

/* The float the elements are divided by during quantisation
 * (mxfp_quant.h:154-160: mantissa MSB set when the scale is subnormal or NaN,
 * so X == 0 means 2^-127 and X == 255 means NaN). */
ORC_API float orc_mx_quant_scale(int x) {
  if (x == 0)
    return bits_f32(0x00400000u);
  if (x == 255)
    return bits_f32(0x7fc00000u);
  return bits_f32((uint32_t)x << 23);
}

/* The float the codes are multiplied by during de-quantisation
 * (MxFP4Quant::set_scale -> get_fp_scale, qtypes.cpp:83-86,
 * mxfp_quant.h:78-83: the byte shifted into the exponent field, so X == 0
 * de-quantises with 0.0). */
ORC_API float orc_mx_dequant_scale(int x) {
  return bits_f32((uint32_t)(x & 0xff) << 23);
}

static const float e2m1_tbl[16] = {0.0f,  0.5f,  1.0f,  1.5f, 2.0f,  3.0f,
                                   4.0f,  6.0f,  -0.0f, -0.5f, -1.0f, -1.5f,
                                   -2.0f, -3.0f, -4.0f, -6.0f};

ORC_API float orc_e2m1_decode(int code) {
  return e2m1_tbl[code & 15];
}

/* E2M1 code of an (already scaled) value: round to nearest, ties to the even
 * mantissa, saturate to +-6, sub-normal step 0.5 kept; +-0 -> code 0.
 * Follows quantize_elemwise(v, 3, 2, 6.0, rd_even, true, true)
 * (mxfp_quant.h:240-300) plus the value->code chain of MxFP4Quant::quantize
 * (qtypes.cpp:87-131; "scaled_out == 0.0" catches -0 before the -0.0 branch;
 * a NaN matches no branch and leaves code 0, see below). */
ORC_API int orc_e2m1_encode(float v) {
  if (v != v) {
    /* A NaN whose mantissa rounds to zero at 2 bits turns into Inf inside
     * quantize_elemwise and saturates to +-6; every other NaN matches no
     * branch of the value->code chain and leaves 0.  (Only a signalling NaN
     * can get here with such a mantissa, and the division by the block scale
     * that precedes this step quiets it, so the quantiser itself always
     * yields 0 for a NaN element.) */
    uint32_t u = f32_bits(v);
    if ((u & 0x7fffffu) <= 0x200000u)
      return 7 | (int)((u >> 31) << 3);
    return 0;
  }
  float a = fabsf(v);
  int c;
  if (a <= 0.25f)
    c = 0;
  else if (a < 0.75f)
    c = 1;
  else if (a <= 1.25f)
    c = 2;
  else if (a < 1.75f)
    c = 3;
  else if (a <= 2.5f)
    c = 4;
  else if (a < 3.5f)
    c = 5;
  else if (a <= 5.0f)
    c = 6;
  else
    c = 7;
  if (c != 0 && (f32_bits(v) >> 31))
    c |= 8;
  return c;
}

/* array forms (bit patterns reach the scalar functions unchanged) */
ORC_API void orc_e2m1_encode_n(const float* v, int32_t* codes, int64_t n) {
  for (int64_t i = 0; i < n; i++)
    codes[i] = orc_e2m1_encode(v[i]);
}
ORC_API void orc_mx_quant_scale_of_amax_n(const float* amax, float* scale, int64_t n) {
  for (int64_t i = 0; i < n; i++)
    scale[i] = orc_mx_quant_scale(orc_mx_scale_byte(amax[i]));
}

/* Quantise one MX block given its amax: returns the scale byte, fills codes.
 * (qtypes.h:153-178 inner part; flush of fp32-subnormal blocks:
 * qtypes.cpp:71.) */
static inline int mx_quant_block_codes(const float* v, int n, int stride,
                                       float amax, uint8_t* codes) {
  int e = (int)((f32_bits(amax) >> 23) & 0xffu);
  int flush = (e == 0);
  int x = orc_mx_scale_byte(amax);
  float s = orc_mx_quant_scale(x);
  for (int i = 0; i < n; i++) {
    float scaled = flush ? 0.0f : v[(int64_t)i * stride] / s;
    codes[i] = (uint8_t)orc_e2m1_encode(scaled);
  }
  return x;
}

/* Generic symmetric per-block MXFP4 quantiser over a tensor viewed as
 * in[pre][bs][post][vnni] (fp32), out[pre][bs][post][vnni/2] (two codes per
 * byte, element v2 of a pair in bits 4*v2), scales[pre][post] (E8M0 bytes).
 * One block = the bs*vnni elements sharing (pre, post).
 * Follows PerBlockQuantizer::quantize_symetric<MxFP4Quant> with pack_size 2
 * (src/csrc/qtypes.h:133-178). */
ORC_API void orc_mxfp4_quantize_generic(const float* in, int64_t pre,
                                        int64_t bs, int64_t post, int64_t vnni,
                                        uint8_t* out, uint8_t* scales) {
  int64_t pv = vnni / 2;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t i = 0; i < pre; i++) {
    for (int64_t j = 0; j < post; j++) {
      const float* base = in + (i * bs * post + j) * vnni;
      float amax = fabsf(base[0]);
      for (int64_t k = 0; k < bs; k++)
        for (int64_t v = 0; v < vnni; v++) {
          float a = fabsf(base[k * post * vnni + v]);
          amax = a > amax ? a : amax; /* std::max(max, val) keeps max on NaN */
        }
      int e = (int)((f32_bits(amax) >> 23) & 0xffu);
      int flush = (e == 0);
      int x = orc_mx_scale_byte(amax);
      float s = orc_mx_quant_scale(x);
      scales[i * post + j] = (uint8_t)x;
      for (int64_t k = 0; k < bs; k++)
        for (int64_t v1 = 0; v1 < pv; v1++) {
          unsigned packed = 0;
          for (int v2 = 0; v2 < 2; v2++) {
            float w = base[k * post * vnni + v1 * 2 + v2];
            float scaled = flush ? 0.0f : w / s;
            packed |= ((unsigned)orc_e2m1_encode(scaled) & 0xf) << (4 * v2);
          }
          out[(i * bs * post + k * post + j) * pv + v1] = (uint8_t)packed;
        }
    }
  }
}

/* Inverse: PerBlockQuantizer::dequantize_symetric<MxFP4Quant>
 * (qtypes.h:196-243; value = table[code] * get_fp_scale(byte)). */
ORC_API void orc_mxfp4_dequantize_generic(const uint8_t* in,
                                          const uint8_t* scales, int64_t pre,
                                          int64_t bs, int64_t post,
                                          int64_t vnni, float* out) {
  int64_t pv = vnni / 2;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t i = 0; i < pre; i++)
    for (int64_t j = 0; j < post; j++) {
      float s = orc_mx_dequant_scale(scales[i * post + j]);
      for (int64_t k = 0; k < bs; k++)
        for (int64_t v1 = 0; v1 < pv; v1++) {
          unsigned b = in[(i * bs * post + k * post + j) * pv + v1];
          for (int v2 = 0; v2 < 2; v2++)
            out[(i * bs * post + k * post + j) * vnni + v1 * 2 + v2] =
                e2m1_tbl[(b >> (4 * v2)) & 0xf] * s;
        }
    }
}

/* ------------------------------------------------------------------ */
/* INT8 symmetric                                                      */
/* ------------------------------------------------------------------ */

/* Int8SymQuant(float max) (src/csrc/qtypes.cpp:163-166): the division is done
 * in double (127.0 literal) and narrowed; inverse in fp32. */
static inline float int8_scale(float amax) {
  return (float)((double)amax / 127.0);
}
static inline float int8_iscale(float s) {
  return s != 0.0f ? 1.0f / s : 0.0f;
}
/* Int8SymQuant::quantize (qtypes.cpp:177-182): nearbyintf (ties-to-even in
 * the default rounding mode) then clamp to +-127. */
static inline int int8_q(float w, float inv) {
  int q = (int)nearbyintf(w * inv);
  return q < -127 ? -127 : (q > 127 ? 127 : q);
}

/* Generic symmetric per-block INT8 quantiser over in[pre][bs][post][vnni]
 * (fp32) -> out same shape (int8), scales[pre][post] (fp32).
 * Follows PerBlockQuantizer::quantize_symetric<Int8SymQuant>
 * (src/csrc/qtypes.h:133-193). */
ORC_API void orc_int8_quantize_generic(const float* in, int64_t pre,
                                       int64_t bs, int64_t post, int64_t vnni,
                                       int8_t* out, float* scales) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t i = 0; i < pre; i++)
    for (int64_t j = 0; j < post; j++) {
      const float* base = in + (i * bs * post + j) * vnni;
      float amax = fabsf(base[0]);
      for (int64_t k = 0; k < bs; k++)
        for (int64_t v = 0; v < vnni; v++) {
          float a = fabsf(base[k * post * vnni + v]);
          amax = a > amax ? a : amax;
        }
      float s = int8_scale(amax);
      float inv = int8_iscale(s);
      scales[i * post + j] = s;
      for (int64_t k = 0; k < bs; k++)
        for (int64_t v = 0; v < vnni; v++)
          out[(i * bs * post + k * post + j) * vnni + v] =
              (int8_t)int8_q(base[k * post * vnni + v], inv);
    }
}

/* PerBlockQuantizer::dequantize_symetric<Int8SymQuant> (qtypes.h:196-243,
 * qtypes.cpp:193-196: value = q * scale). */
ORC_API void orc_int8_dequantize_generic(const int8_t* in, const float* scales,
                                         int64_t pre, int64_t bs, int64_t post,
                                         int64_t vnni, float* out) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t i = 0; i < pre; i++)
    for (int64_t j = 0; j < post; j++) {
      float s = scales[i * post + j];
      for (int64_t k = 0; k < bs; k++)
        for (int64_t v = 0; v < vnni; v++) {
          int64_t o = (i * bs * post + k * post + j) * vnni + v;
          out[o] = (float)in[o] * s;
        }
    }
}

/* Dynamic activation quantisation of the QINT8 linear: per (row, K-block of
 * qbs) scale = max|x|/127, xq = clamp(rne(x * (1/scale))).
 * Follows quantize_int8sym(t_in, block_size, -1, false)
 * (src/csrc/fused_gemm.h:1249 -> qtypes.cpp:613-624 -> qtypes.h:133-193 with
 * vnni 1, post 1; QuantTPP::ref, src/csrc/xsmm_functors.h:909-965).
 * x is bf16 (bit pattern), up-converted to fp32 first. */
ORC_API void orc_quant_act_int8(const uint16_t* x, int64_t M, int64_t K,
                                int64_t qbs, int8_t* xq, float* sa) {
  int64_t nb = K / qbs;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t m = 0; m < M; m++)
    for (int64_t b = 0; b < nb; b++) {
      const uint16_t* p = x + m * K + b * qbs;
      float amax = 0.0f;
      for (int64_t k = 0; k < qbs; k++) {
        float a = fabsf(bf16_to_f32(p[k]));
        amax = a > amax ? a : amax;
      }
      float s = int8_scale(amax);
      float inv = int8_iscale(s);
      sa[m * nb + b] = s;
      for (int64_t k = 0; k < qbs; k++)
        xq[m * K + b * qbs + k] = (int8_t)int8_q(bf16_to_f32(p[k]), inv);
    }
}

/* ------------------------------------------------------------------ */
/* Reference weight layouts (closed-form index maps)                   */
/* ------------------------------------------------------------------ */

/* MXFP4: plain W[N][K] fp32 -> reference layout
 *   qdata  [N/32][K/64][32 c2][32 k2]  byte = code(K even) | code(K odd) << 4
 *   scales [N/32][K/64][2 h][32 k2]    E8M0 byte of block K = nc*64+h*32..+31
 * element (nk,nc,c2,k2,c3) = W[nk*32+k2][nc*64+c2*2+c3].
 * Follows remap_and_quantize_mxfp4 (src/csrc/qtypes.cpp:783-864) followed by
 * quantize_mxfp4(t, 32, 2, true) (qtypes.cpp:602-611). */
ORC_API void orc_remap_quantize_mxfp4(const float* W, int64_t N, int64_t K,
                                      uint8_t* qdata, uint8_t* scales) {
  int64_t Nk = N / 32, Nc = K / 64;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t nk = 0; nk < Nk; nk++)
    for (int64_t nc = 0; nc < Nc; nc++)
      for (int h = 0; h < 2; h++)
        for (int k2 = 0; k2 < 32; k2++) {
          const float* row = W + (nk * 32 + k2) * K + nc * 64 + h * 32;
          /* max = |first|, then std::max(max, |v|) (qtypes.h:156-162): a NaN in the
           * first slot stays (byte 255), a NaN anywhere else never wins */
          float amax = fabsf(row[0]);
          for (int j = 1; j < 32; j++) {
            float a = fabsf(row[j]);
            amax = a > amax ? a : amax;
          }
          uint8_t codes[32];
          int x = mx_quant_block_codes(row, 32, 1, amax, codes);
          scales[((nk * Nc + nc) * 2 + h) * 32 + k2] = (uint8_t)x;
          for (int p = 0; p < 16; p++)
            qdata[((nk * Nc + nc) * 32 + (h * 16 + p)) * 32 + k2] =
                (uint8_t)(codes[2 * p] | (codes[2 * p + 1] << 4));
        }
}

static inline float mxfp4_ref_weight(const uint8_t* qdata,
                                     const uint8_t* scales, int64_t Nc,
                                     int64_t n, int64_t k) {
  int64_t nk = n >> 5, k2 = n & 31, nc = k >> 6, kk = k & 63;
  unsigned b = qdata[((nk * Nc + nc) * 32 + (kk >> 1)) * 32 + k2];
  unsigned code = (kk & 1) ? (b >> 4) : (b & 0xf);
  int x = scales[((nk * Nc + nc) * 2 + (kk >> 5)) * 32 + k2];
  return e2m1_tbl[code] * orc_mx_dequant_scale(x);
}

/* reference layout -> plain W[N][K] fp32 (exact) */
ORC_API void orc_dequantize_mxfp4(const uint8_t* qdata, const uint8_t* scales,
                                  int64_t N, int64_t K, float* W) {
  int64_t Nc = K / 64;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; n++)
    for (int64_t k = 0; k < K; k++)
      W[n * K + k] = mxfp4_ref_weight(qdata, scales, Nc, n, k);
}

/* QINT8: plain W[N][K] fp32 -> reference layout
 *   q      [N/16][K/qbs][qbs/4][16 k2][4 v]  element = W[n1*16+k2][b*qbs+a*4+v]
 *   scales [N/16][K/qbs][16]                 fp32
 * Follows remap_and_quantize_qint8 (src/csrc/qtypes.cpp:866-932) followed by
 * quantize_int8sym(t, qbs, 2, true). */
ORC_API void orc_remap_quantize_qint8(const float* W, int64_t N, int64_t K,
                                      int64_t qbs, int8_t* q, float* scales) {
  int64_t N1 = N / 16, nb = K / qbs;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t n1 = 0; n1 < N1; n1++)
    for (int64_t b = 0; b < nb; b++)
      for (int k2 = 0; k2 < 16; k2++) {
        const float* row = W + (n1 * 16 + k2) * K + b * qbs;
        float amax = 0.0f;
        for (int64_t j = 0; j < qbs; j++) {
          float a = fabsf(row[j]);
          amax = a > amax ? a : amax;
        }
        float s = int8_scale(amax);
        float inv = int8_iscale(s);
        scales[(n1 * nb + b) * 16 + k2] = s;
        for (int64_t j = 0; j < qbs; j++)
          q[(((n1 * nb + b) * (qbs / 4) + (j >> 2)) * 16 + k2) * 4 + (j & 3)] =
              (int8_t)int8_q(row[j], inv);
      }
}

ORC_API void orc_dequantize_qint8(const int8_t* q, const float* scales,
                                  int64_t N, int64_t K, int64_t qbs, float* W) {
  int64_t nb = K / qbs;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; n++)
    for (int64_t k = 0; k < K; k++) {
      int64_t n1 = n >> 4, k2 = n & 15, b = k / qbs, j = k % qbs;
      W[n * K + k] =
          (float)q[(((n1 * nb + b) * (qbs / 4) + (j >> 2)) * 16 + k2) * 4 +
                   (j & 3)] *
          scales[(n1 * nb + b) * 16 + k2];
    }
}

/* ------------------------------------------------------------------ */
/* INT4 symmetric (Int4SymQuant, src/csrc/qtypes.cpp:199-246)           */
/* ------------------------------------------------------------------ */
/* scale = (float)(max / 7.0) (double division, narrowed), inverse in fp32,
 * q = clamp(nearbyintf(w * iscale), -8, 7); two codes per byte, element v2
 * of a pair in bits 4*v2 (two's complement nibble), as
 * PerBlockQuantizer::quantize_symetric packs them (qtypes.h:166-178).
 * Geometry as for the other generic quantisers:
 * in[pre][bs][post][vnni] -> out[pre][bs][post][vnni/2], scales[pre][post]. */
static const int int4_tbl[16] = {0, 1, 2, 3, 4, 5, 6, 7, -8, -7, -6, -5, -4, -3, -2, -1};

ORC_API void orc_int4_quantize_generic(const float* in, int64_t pre, int64_t bs,
                                       int64_t post, int64_t vnni, uint8_t* out,
                                       float* scales) {
  int64_t pv = vnni / 2;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t i = 0; i < pre; i++)
    for (int64_t j = 0; j < post; j++) {
      const float* base = in + (i * bs * post + j) * vnni;
      float amax = fabsf(base[0]);
      for (int64_t k = 0; k < bs; k++)
        for (int64_t v = 0; v < vnni; v++) {
          float a = fabsf(base[k * post * vnni + v]);
          amax = a > amax ? a : amax;
        }
      float s = (float)((double)amax / 7.0);
      float inv = (s != 0.0f) ? (1.0f / s) : 0.0f;
      scales[i * post + j] = s;
      for (int64_t k = 0; k < bs; k++)
        for (int64_t v1 = 0; v1 < pv; v1++) {
          unsigned packed = 0;
          for (int v2 = 0; v2 < 2; v2++) {
            float r = nearbyintf(base[k * post * vnni + v1 * 2 + v2] * inv);
            int q = r < -8.0f ? -8 : (r > 7.0f ? 7 : (int)r);
            packed |= ((unsigned)q & 0xf) << (4 * v2);
          }
          out[(i * bs * post + k * post + j) * pv + v1] = (uint8_t)packed;
        }
    }
}

/* value = lkp_tbl[code] * scale (qtypes.cpp:241-244, qtypes.h:196-243) */
ORC_API void orc_int4_dequantize_generic(const uint8_t* in, const float* scales,
                                         int64_t pre, int64_t bs, int64_t post,
                                         int64_t vnni, float* out) {
  int64_t pv = vnni / 2;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t i = 0; i < pre; i++)
    for (int64_t j = 0; j < post; j++) {
      float s = scales[i * post + j];
      for (int64_t k = 0; k < bs; k++)
        for (int64_t v1 = 0; v1 < pv; v1++) {
          unsigned b = in[(i * bs * post + k * post + j) * pv + v1];
          for (int v2 = 0; v2 < 2; v2++)
            out[(i * bs * post + k * post + j) * vnni + v1 * 2 + v2] =
                (float)int4_tbl[(b >> (4 * v2)) & 0xf] * s;
        }
    }
}

/* ------------------------------------------------------------------ */
/* QINT2 interleaved (ternary weights)                                 */
/* ------------------------------------------------------------------ */
/* remap_and_quantize_qint2_intlv (src/csrc/qtypes.cpp:1004-1073) for N % 32
 * == 0 (K2 = 8, K3 = 4, C3 = 4) and a block of bs input channels:
 *   scale[n][b] = max(|W[n][b*bs ..]|, 1e-8)           (abs max, clamp_min)
 *   t = round_half_even(W / scale) clamped to [-1, 1]  (fp32 division)
 *   code: 0 -> 0, +1 -> 1, -1 -> 2   (uint8(-1) & 3 = 3, then 3 -> 2)
 *   byte[n1][b][c2][k2][c3] = code(n1*32 + 0*8 + k2) | code(.. 1*8 ..) << 2 |
 *                             code(.. 2*8 ..) << 4 | code(.. 3*8 ..) << 6
 *     at input channel b*bs + c2*4 + c3
 *   scales [N/32][K/bs][32]  (row r = k3*8 + k2 of the 32-channel group) */
ORC_API void orc_remap_quantize_qint2_intlv(const float* W, int64_t N, int64_t K,
                                            int64_t bs, uint8_t* q, float* scales) {
  int64_t N1 = N / 32, nb = K / bs, C2 = bs / 4;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t n1 = 0; n1 < N1; n1++)
    for (int64_t b = 0; b < nb; b++) {
      uint8_t* qb = q + (n1 * nb + b) * C2 * 32;
      memset(qb, 0, (size_t)(C2 * 32));
      for (int r = 0; r < 32; r++) {
        const float* row = W + (n1 * 32 + r) * K + b * bs;
        float amax = 0.0f;
        for (int64_t c = 0; c < bs; c++) {
          float a = fabsf(row[c]);
          amax = a > amax ? a : amax;
        }
        float s = amax < 1.0e-8f ? 1.0e-8f : amax;
        scales[(n1 * nb + b) * 32 + r] = s;
        int k3 = r >> 3, k2 = r & 7;
        for (int64_t c = 0; c < bs; c++) {
          float t = nearbyintf(row[c] / s);
          unsigned code = t >= 1.0f ? 1u : (t <= -1.0f ? 2u : 0u);
          qb[((c >> 2) * 8 + k2) * 4 + (c & 3)] |= (uint8_t)(code << (2 * k3));
        }
      }
    }
}

/* ------------------------------------------------------------------ */
/* Post-ops on the bf16 output tile                                    */
/* ------------------------------------------------------------------ */
enum {
  ORC_POST_NONE = 0,
  ORC_POST_SILU = 1,
  ORC_POST_MUL = 2,
  ORC_POST_ADD_SCALE = 3,
  ORC_POST_ADD2_SCALE = 4,
  ORC_POST_GELU = 5,
  ORC_POST_RELU = 6
};

/* y is the bf16-rounded GEMM(+bias) result; in1/in2 bf16 bit patterns.
 * SiluPostOp  (src/csrc/fused_gemm.h:1369; SiLUFwdTPP xsmm_functors.h:3279):
 *             s = bf16(sigmoid(y)); y = bf16(y*s)
 * MulPostOp   (fused_gemm.h:1409; MulTPP):        y = bf16(in*y)
 * AddScale    (fused_gemm.h:1434; ScaleAddTPP xsmm_functors.h:1858):
 *             y = bf16(y + in*scale)
 * Add2Scale   (fused_gemm.h:1460): y = bf16(y+in1); y = bf16(y + in2*scale)
 * Gelu        (fused_gemm.h:1349; scalar form xsmm_functors.h:2794):
 *             y = bf16(0.5*y*(1+erf(y/sqrt2)))
 * Relu        (fused_gemm.h:1389): y = max(y,0)
 * libxsmm evaluates sigmoid/GELU with its own polynomial; the exact libm
 * form is used here (tolerance-covered, parity unpinned for that detail). */
static inline uint16_t apply_post(uint16_t yb, int post, uint16_t in1,
                                  uint16_t in2, float scale) {
  float y = bf16_to_f32(yb);
  switch (post) {
    case ORC_POST_SILU: {
      float s = bf16_to_f32(f32_to_bf16(1.0f / (1.0f + expf(-y))));
      return f32_to_bf16(y * s);
    }
    case ORC_POST_MUL:
      return f32_to_bf16(bf16_to_f32(in1) * y);
    case ORC_POST_ADD_SCALE:
      return f32_to_bf16(fmaf(bf16_to_f32(in1), scale, y));
    case ORC_POST_ADD2_SCALE: {
      float t = bf16_to_f32(f32_to_bf16(y + bf16_to_f32(in1)));
      return f32_to_bf16(fmaf(bf16_to_f32(in2), scale, t));
    }
    case ORC_POST_GELU:
      return f32_to_bf16(0.5f * y * (1.0f + erff(y * 0.70710678118654752f)));
    case ORC_POST_RELU:
      return (yb & 0x8000u) ? (uint16_t)0 : yb;
    default:
      return yb;
  }
}

ORC_API void orc_post_op(uint16_t* y, int64_t n, int post, const uint16_t* in1,
                         const uint16_t* in2, float scale) {
  for (int64_t i = 0; i < n; i++)
    y[i] = apply_post(y[i], post, in1 ? in1[i] : 0, in2 ? in2[i] : 0, scale);
}

/* ------------------------------------------------------------------ */
/* Linear layers                                                       */
/* ------------------------------------------------------------------ */
enum { ORC_MODE_IDEAL = 0, ORC_MODE_FAITHFUL = 1, ORC_MODE_F64 = 2 };

/* MXFP4 weight-only linear on the reference layout.
 *   y[m][n] = post( bf16( bias[n] + sum_k x[m][k] * deq(W)[n][k] ) )
 * mode IDEAL   : one fp32 accumulation over all of K, one bf16 rounding.
 * mode FAITHFUL: the reference re-rounds the bf16 output tile after every
 *                K chunk of Ncb*64 (all of K when M/64 <= 4, else 4096)
 *                (src/csrc/fused_gemm.h:695-721 getBlockingParams,
 *                 :896-947 task body, beta = 1 BRGEMM into the bf16 tile).
 * mode F64     : fp64 accumulation, one rounding (error yard-stick).
 * Task grid as in the reference: one task per 32-wide output block nk,
 * parallel over nk (loop scheme "aCb", fused_gemm.h:33-37,982-998). */
ORC_API void orc_linear_mxfp4(const uint16_t* x, int64_t M, int64_t K,
                              const uint8_t* qdata, const uint8_t* scales,
                              int64_t N, const uint16_t* bias, int post,
                              const uint16_t* post_in, const uint16_t* post_in2,
                              float post_scale, int mode, uint16_t* y) {
  int64_t Nk = N / 32, Nc = K / 64;
  int64_t chunk = K;
  if (mode == ORC_MODE_FAITHFUL && (M / 64) > 4)
    chunk = 4096 < K ? 4096 : K;
#pragma omp parallel
  {
    float* wd = (float*)malloc(sizeof(float) * (size_t)K * 32); /* [K][32] */
    float* xf = (float*)malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(dynamic, 1)
    for (int64_t nk = 0; nk < Nk; nk++) {
      for (int64_t nc = 0; nc < Nc; nc++) {
        const uint8_t* qb = qdata + (nk * Nc + nc) * 1024;
        const uint8_t* sb = scales + (nk * Nc + nc) * 64;
        for (int c2 = 0; c2 < 32; c2++) {
          int h = c2 >> 4;
          float* w0 = wd + (nc * 64 + c2 * 2) * 32;
          for (int k2 = 0; k2 < 32; k2++) {
            unsigned b = qb[c2 * 32 + k2];
            float s = orc_mx_dequant_scale(sb[h * 32 + k2]);
            w0[k2] = e2m1_tbl[b & 0xf] * s;
            w0[32 + k2] = e2m1_tbl[b >> 4] * s;
          }
        }
      }
      for (int64_t m = 0; m < M; m++) {
        for (int64_t k = 0; k < K; k++)
          xf[k] = bf16_to_f32(x[m * K + k]);
        uint16_t yb[32];
        for (int j = 0; j < 32; j++)
          yb[j] = bias ? bias[nk * 32 + j] : 0;
        if (mode == ORC_MODE_F64) {
          double acc[32];
          for (int j = 0; j < 32; j++)
            acc[j] = (double)bf16_to_f32(yb[j]);
          for (int64_t k = 0; k < K; k++) {
            const float* w = wd + k * 32;
            double xv = (double)xf[k];
            for (int j = 0; j < 32; j++)
              acc[j] += xv * (double)w[j];
          }
          for (int j = 0; j < 32; j++)
            yb[j] = f32_to_bf16((float)acc[j]);
        } else {
          for (int64_t k0 = 0; k0 < K; k0 += chunk) {
            int64_t k1 = k0 + chunk < K ? k0 + chunk : K;
            float acc[32];
            for (int j = 0; j < 32; j++)
              acc[j] = 0.0f;
            for (int64_t k = k0; k < k1; k++) {
              const float* w = wd + k * 32;
              float xv = xf[k];
              for (int j = 0; j < 32; j++)
                acc[j] = fmaf(xv, w[j], acc[j]);
            }
            for (int j = 0; j < 32; j++)
              yb[j] = f32_to_bf16(bf16_to_f32(yb[j]) + acc[j]);
          }
        }
        for (int j = 0; j < 32; j++) {
          int64_t o = m * N + nk * 32 + j;
          y[o] = apply_post(yb[j], post, post_in ? post_in[o] : 0,
                            post_in2 ? post_in2[o] : 0, post_scale);
        }
      }
    }
    free(wd);
    free(xf);
  }
}

/* Exact int32 block sums of the QINT8 linear (test hook):
 * acc[m][n][b] = sum_{k in block b} xq[m][k]*wq[n][k]. */
ORC_API void orc_qint8_block_sums(const int8_t* xq, int64_t M, int64_t K,
                                  const int8_t* q, int64_t N, int64_t qbs,
                                  int32_t* acc) {
  int64_t nb = K / qbs;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; n++) {
    int64_t n1 = n >> 4, k2 = n & 15;
    for (int64_t m = 0; m < M; m++)
      for (int64_t b = 0; b < nb; b++) {
        int32_t s = 0;
        for (int64_t j = 0; j < qbs; j++)
          s += (int32_t)xq[m * K + b * qbs + j] *
               (int32_t)q[(((n1 * nb + b) * (qbs / 4) + (j >> 2)) * 16 + k2) * 4 +
                          (j & 3)];
        acc[(m * N + n) * nb + b] = s;
      }
  }
}

/* QINT8 (W8A8) linear on the reference layout.
 *   xq, sa = orc_quant_act_int8(x)
 * mode FAITHFUL (src/csrc/fused_gemm.h:1183-1233): the bf16 output tile is a
 *   running sum re-rounded after every group of G input channels,
 *   y = bf16( float(y) + float(acc_i32) * (sa*sw) ), G = qbs for rows inside
 *   a complete 64-row block and G = 64 for remainder rows
 *   (is_rem = s1 + 64 > M; DequantTPP fmadd xsmm_functors.h:987-1031).
 * mode IDEAL: fp32 running sum over the qbs blocks in K order
 *   (f = fma(float(acc_b), sa*sw, f)), bias added first, one bf16 rounding.
 * mode F64  : the same sum in fp64. */
ORC_API void orc_linear_qint8(const uint16_t* x, int64_t M, int64_t K,
                              const int8_t* q, const float* sw, int64_t N,
                              int64_t qbs, const uint16_t* bias, int post,
                              const uint16_t* post_in, const uint16_t* post_in2,
                              float post_scale, int mode, uint16_t* y) {
  int64_t N1 = N / 16, nb = K / qbs;
  int8_t* xq = (int8_t*)malloc((size_t)(M * K));
  float* sa = (float*)malloc(sizeof(float) * (size_t)(M * nb));
  orc_quant_act_int8(x, M, K, qbs, xq, sa);
  int64_t full_rows = (M / 64) * 64;
#pragma omp parallel
  {
    int8_t* wt = (int8_t*)malloc((size_t)K * 16); /* [16][K] plain */
#pragma omp for schedule(dynamic, 1)
    for (int64_t n1 = 0; n1 < N1; n1++) {
      for (int64_t b = 0; b < nb; b++)
        for (int64_t a = 0; a < qbs / 4; a++)
          for (int k2 = 0; k2 < 16; k2++)
            for (int v = 0; v < 4; v++)
              wt[k2 * K + b * qbs + a * 4 + v] =
                  q[(((n1 * nb + b) * (qbs / 4) + a) * 16 + k2) * 4 + v];
      for (int64_t m = 0; m < M; m++) {
        int64_t G = qbs;
        if (mode == ORC_MODE_FAITHFUL && m >= full_rows)
          G = 64;
        const int8_t* xr = xq + m * K;
        for (int k2 = 0; k2 < 16; k2++) {
          int64_t n = n1 * 16 + k2;
          const int8_t* wr = wt + k2 * K;
          uint16_t yb = bias ? bias[n] : 0;
          float f = bf16_to_f32(yb);
          double d = (double)f;
          for (int64_t g = 0; g < K; g += G) {
            int32_t acc = 0;
            for (int64_t k = g; k < g + G; k++)
              acc += (int32_t)xr[k] * (int32_t)wr[k];
            int64_t b = g / qbs;
            float s = sa[m * nb + b] * sw[(n1 * nb + b) * 16 + k2];
            if (mode == ORC_MODE_FAITHFUL) {
              yb = f32_to_bf16(fmaf((float)acc, s, bf16_to_f32(yb)));
            } else if (mode == ORC_MODE_F64) {
              d += (double)acc * (double)sa[m * nb + b] *
                   (double)sw[(n1 * nb + b) * 16 + k2];
            } else {
              f = fmaf((float)acc, s, f);
            }
          }
          if (mode == ORC_MODE_IDEAL)
            yb = f32_to_bf16(f);
          else if (mode == ORC_MODE_F64)
            yb = f32_to_bf16((float)d);
          int64_t o = m * N + n;
          y[o] = apply_post(yb, post, post_in ? post_in[o] : 0,
                            post_in2 ? post_in2[o] : 0, post_scale);
        }
      }
    }
    free(wt);
  }
  free(xq);
  free(sa);
}

/* The same GEMM on activations the caller has quantized (int8 [M][K] +
 * f32 [M][K/qbs]) with everything after the integer sums in fp32:
 * TppBlockedQInt8LinearW<float, uint8_t, float> (fused_gemm.h:1076-1341), the
 * path of float / half / pre-quantized inputs (fused_llm_infer.cpp:1526-1545).
 * y = bias + sum_b float(isum_b) * (sa*sw), one fused multiply-add per block in
 * ascending order (mode ideal of orc_linear_qint8 without the final rounding).
 * Pinned by: rounding y to bf16 reproduces orc_linear_qint8 (ideal) on bf16
 * inputs; fp64 evaluation of the formula (tests/test_oracle.py). */
ORC_API void orc_linear_qint8_f32(const int8_t* xq, const float* sa, int64_t M,
                                  int64_t K, const int8_t* q, const float* sw,
                                  int64_t N, int64_t qbs, const float* bias,
                                  float* y) {
  int64_t N1 = N / 16, nb = K / qbs;
#pragma omp parallel for schedule(dynamic, 1)
  for (int64_t n1 = 0; n1 < N1; n1++)
    for (int k2 = 0; k2 < 16; k2++) {
      int64_t n = n1 * 16 + k2;
      for (int64_t m = 0; m < M; m++) {
        float f = bias ? bias[n] : 0.0f;
        for (int64_t b = 0; b < nb; b++) {
          int32_t acc = 0;
          for (int64_t a = 0; a < qbs / 4; a++)
            for (int v = 0; v < 4; v++)
              acc += (int32_t)xq[m * K + b * qbs + a * 4 + v] *
                     (int32_t)q[(((n1 * nb + b) * (qbs / 4) + a) * 16 + k2) * 4 + v];
          f = fmaf((float)acc, sa[m * nb + b] * sw[(n1 * nb + b) * 16 + k2], f);
        }
        y[m * N + n] = f;
      }
    }
}

/* ------------------------------------------------------------------ */
/* W4A8: MXFP4 weights in the VNNI8-interleaved layout of               */
/* remap_and_quantize_mxfp4 under USE_MXFP4_INT8 (qtypes.cpp:787-790,    */
/* 840-861) with int8 activations (TppBlockedLinearW<int8_t, uint8_t,    */
/* Tout>, fused_gemm.h:965-978, 1523-1526).                              */
/* q u8 [N/8][K/bc][bc/8][8][4]: byte j of the group (n8, 8 K values)    */
/* holds K value j in its low and K value 4 + j in its high nibble;      */
/* sc u8 [N/8][K/bc][bc/32][8] E8M0.  Activations: int8 over blocks of   */
/* 32 along K with scale max/127 (quantize_int8sym), the scales then     */
/* multiplied by float(6.0/127.0) (fused_gemm.h:975-977).  The consumer  */
/* of that convention sits inside libxsmm (absent): it implies integer   */
/* weights w_i = e2m1 * 127/6.  RESTATED HERE AS round-to-nearest-even   */
/* of e2m1 * 127/6 -> {0, 11, 21, 32, 42, 64, 85, 127}: PARITY UNPINNED  */
/* for that table and for the summation order; pinned are the layout     */
/* (against the view/permute chain), the activation quantizer and the    */
/* identity w_i * 6/127 ~ e2m1 within the table's rounding.              */
/* y = post(bf16(bias + sum_b float(isum_b) * (sa'[m][b] * 2^(e-127)))). */
/* ------------------------------------------------------------------ */
static const int8_t w4a8_tbl[8] = {0, 11, 21, 32, 42, 64, 85, 127};
ORC_API int orc_w4a8_weight_int(int code) {
  int v = w4a8_tbl[code & 7];
  return (code & 8) ? -v : v;
}

ORC_API void orc_linear_w4a8(const int8_t* xq, const float* sa, int64_t M,
                             int64_t K, const uint8_t* q, const uint8_t* sc,
                             int64_t N, int64_t bc, const uint16_t* bias,
                             int post, const uint16_t* post_in,
                             const uint16_t* post_in2, float post_scale,
                             uint16_t* y) {
  int64_t C1 = K / bc, nb = K / 32;
#pragma omp parallel for schedule(dynamic, 8)
  for (int64_t n = 0; n < N; n++) {
    int64_t n8b = n / 8, n8 = n % 8;
    for (int64_t m = 0; m < M; m++) {
      float f = bias ? bf16_to_f32(bias[n]) : 0.0f;
      for (int64_t b = 0; b < nb; b++) {
        int64_t c1 = (b * 32) / bc, kb = (b * 32) % bc; /* K offset inside the bc block */
        int32_t acc = 0;
        for (int64_t k = 0; k < 32; k++) {
          int64_t kk = kb + k, g = kk / 8, j = kk % 8;
          uint8_t byte = q[(((n8b * C1 + c1) * (bc / 8) + g) * 8 + n8) * 4 + (j & 3)];
          int code = j < 4 ? (byte & 15) : (byte >> 4);
          acc += (int32_t)xq[m * K + b * 32 + k] * orc_w4a8_weight_int(code);
        }
        float ws = orc_mx_dequant_scale(sc[((n8b * C1 + c1) * (bc / 32) + kb / 32) * 8 + n8]);
        f = fmaf((float)acc, sa[m * nb + b] * ws, f);
      }
      int64_t o = m * N + n;
      y[o] = apply_post(f32_to_bf16(f), post, post_in ? post_in[o] : 0,
                        post_in2 ? post_in2[o] : 0, post_scale);
    }
  }
}

ORC_API int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
ORC_API void orc_set_num_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n);
#else
  (void)n;
#endif
}
