/*
 * tppx -- C ABI of the MI355X (gfx950) weight-quantized linear path.
 *
 * This is the drop-in boundary for the reference's quantized-linear path
 * (MXFP4 weight-only and QINT8 W8A8 linears with fused bias / SiLU / mul /
 * residual-add epilogues, fused QKV, and the quantize / remap helpers).
 *
 * Conventions
 *   - Every function returns 0 on success or a negative TPPX_E* code; nothing
 *     throws and nothing terminates the process (the reference's TPP_ASSERT
 *     printf+exit(1), src/csrc/utils.h:34-41, becomes an error code).
 *     tppx_last_error() returns a thread-local message for the last failure.
 *   - All data pointers are DEVICE pointers, 16-byte aligned, owned by the
 *     caller.  The library allocates no device memory.
 *   - Work is enqueued on `stream` (a hipStream_t passed as void*; NULL = the
 *     default stream) and the call returns without synchronising.
 *   - Arguments are validated before any HIP call, so the error paths can be
 *     exercised on a machine without a GPU.
 *   - bf16 = bfloat16 bit patterns; M = rows of the activation (tokens),
 *     K = in-features, N = out-features.
 *
 * Weight formats
 *   "reference layout" (what the quantize entry points emit, byte-identical to
 *   the reference's QTensor storage):
 *     MXFP4  qdata  u8 [N/32][K/64][32][32]  byte[nk][nc][c2][k2] holds
 *                      W[nk*32+k2][nc*64+2*c2] (low nibble) and [..+1] (high)
 *            scales u8 [N/32][K/64][2][32]   E8M0 of W[nk*32+k2][nc*64+h*32..+31]
 *     QINT8  q      i8 [N/16][K/QBS][QBS/4][16][4]  = W[n1*16+k2][b*QBS+a*4+v]
 *            scales f32[N/16][K/QBS][16]
 *   "native layout" (what the linear entry points consume; produced once by
 *   tppx_prepack_*; one 1 KiB tile = one wave-wide 128-bit load = one MFMA
 *   operand):
 *     MXFP4  qdata  u8 [N/16][K/128][4 g][16 n][16 B]  the 16 B are the 32
 *                      E2M1 codes of W[nt*16+n][kt*128+g*32 .. +31], even K in
 *                      the low nibble
 *            scales u8 [N/16][K/128][4 g][16 n]
 *     QINT8  q      i8 [N/16][K/64][4 g][16 n][16 B]   W[nt*16+n][kt*64+g*16..+15]
 *            scales: the reference array is used unchanged.
 */
#ifndef TPPX_H
#define TPPX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TPPX_VERSION 100

#define TPPX_OK 0
#define TPPX_EINVAL (-1)       /* null / misaligned pointer, bad enum value   */
#define TPPX_ESHAPE (-2)       /* a shape constraint of the path is violated  */
#define TPPX_EUNSUPPORTED (-3) /* legal in the reference, not built here      */
#define TPPX_EHIP (-4)         /* the HIP runtime reported an error           */

/* Post-ops, applied to the bf16-rounded GEMM(+bias) tile exactly where the
 * reference applies them (src/csrc/fused_gemm.h:1343-1488). */
#define TPPX_POST_NONE 0       /* NullPostOp      fused_gemm.h:1343 */
#define TPPX_POST_SILU 1       /* SiluPostOp      fused_gemm.h:1369 */
#define TPPX_POST_MUL 2        /* MulPostOp       fused_gemm.h:1409 */
#define TPPX_POST_ADD_SCALE 3  /* AddScalePostOp  fused_gemm.h:1434 */
#define TPPX_POST_ADD2_SCALE 4 /* Add2ScalePostOp fused_gemm.h:1460 */
#define TPPX_POST_GELU 5       /* GeluPostOp      fused_gemm.h:1349 */
#define TPPX_POST_RELU 6       /* ReluPostOp      fused_gemm.h:1389 */

/* Element type of a floating-point weight handed to the quantizers. */
#define TPPX_DT_F32 0
#define TPPX_DT_BF16 1
#define TPPX_DT_F16 2

/* Weight kinds of tppx_linear_wide. */
#define TPPX_W_MXFP4 0 /* native tiles + scale bytes of tppx_prepack_mxfp4 */
#define TPPX_W_BF16 1  /* native tiles of tppx_prepack_bf16 */

/* flags for the linear entry points */
#define TPPX_FLAG_NONE 0
#define TPPX_FLAG_FORCE_SKINNY 1 /* always take the decode (streaming) kernel */
#define TPPX_FLAG_FORCE_TILED 2  /* always take the prefill (LDS-tiled) kernel */
#define TPPX_FLAG_ACT_FP8 4      /* MXFP4 prefill: round activations to MXFP8
                                    (E4M3 + E8M0/32) and use the scaled
                                    f8f6f4 MFMA -- NOT the reference numerics */
#define TPPX_FLAG_XQ_REUSE 8     /* QINT8, x != NULL: xq / sa still hold this
                                    very x as an earlier call with the same
                                    M, K, qbs, flags left it (several GEMMs on
                                    one input): skip the re-quantization */

typedef void* tppx_stream_t;

int tppx_version(void);
const char* tppx_last_error(void);
/* The library reads its TPPX_* environment switches once per process, the
 * first time a launch asks for one, and keeps the answer (no getenv() per
 * launch; a kernel choice recorded in a captured graph cannot drift from the
 * eager one).  This drops what was kept, so the next launch reads the
 * environment again.  No counterpart in the reference (its switches are read
 * at static-initialisation time, e.g. src/csrc/fused_gemm.h:26-37). */
void tppx_reload_env(void);

/* ---- quantize / remap -------------------------------------------------- */

/* Replaces qtype.remap_and_quantize_mxfp4 (src/csrc/qtypes.cpp:783-864; bound
 * at qtypes.cpp:1089).  `w` is a blocked weight whose element (n,k) lives at
 *   ((n/bk)*(K/bc) + k/bc)*bk*bc + ((k%bc)/vnni)*bk*vnni + (n%bk)*vnni + k%vnni
 * (bk=1, bc=K, vnni=1 describes a plain row-major [N][K]); the 5-D bf16
 * tensors of the reference are bk=16, bc=64, vnni=2, the 4-D fp32 ones
 * vnni=1.  Needs N%32==0, K%64==0.  Output: reference layout. */
int tppx_quantize_mxfp4(const void* w, int w_dtype, int64_t N, int64_t K,
                        int64_t bk, int64_t bc, int64_t vnni, void* qdata,
                        void* scales, tppx_stream_t stream);

/* Replaces qtype.remap_and_quantize_qint8 (src/csrc/qtypes.cpp:866-932; bound
 * at qtypes.cpp:1091).  qbs is the K block the caller derived with the
 * reference rule (256 if it divides K, else the largest smaller power of two
 * >= 64 that does).  Needs N%16==0, K%qbs==0, qbs%64==0. */
int tppx_quantize_qint8(const void* w, int w_dtype, int64_t N, int64_t K,
                        int64_t bk, int64_t bc, int64_t vnni, int64_t qbs,
                        void* q, void* scales, tppx_stream_t stream);

/* Replaces at::Tensor::dequantize() of the two custom quantizers
 * (PerBlockMxFPQuantizer / PerBlockAffineQuantizer::dequantize,
 * src/csrc/qtypes.cpp:438-473,521-577).  Output fp32 in the blocked shape of
 * the quantized tensor: [N/32][K/64][32][32][2] resp. [N/16][K/QBS][QBS/4][16][4]. */
int tppx_dequantize_mxfp4(const void* qdata, const void* scales, int64_t N,
                          int64_t K, void* out_f32, tppx_stream_t stream);
int tppx_dequantize_qint8(const void* q, const void* scales, int64_t N,
                          int64_t K, int64_t qbs, void* out_f32,
                          tppx_stream_t stream);

/* Per-block formats of the generic helpers below. */
#define TPPX_Q_MXFP4 0 /* E2M1 codes, two per byte, E8M0 scale byte per block */
#define TPPX_Q_INT8 1  /* int8, fp32 scale = max/127                          */
#define TPPX_Q_INT4 2  /* two's complement nibbles, two per byte, fp32 scale = max/7 */

/* Replace quantize_mxfp4 / quantize_int8sym / quantize_int4sym on ANY layout
 * (src/csrc/qtypes.cpp:602-637 -> PerBlockQuantizer::quantize_symetric,
 * src/csrc/qtypes.h:30-68,133-193) and the matching dequantize
 * (qtypes.h:196-243).  The tensor is viewed as in[pre][bs][post][vnni] --
 * the geometry PerBlockQuantizer derives from (sizes, block_size, axis,
 * is_vnni): with is_vnni the last dimension is vnni and block_size / vnni
 * consecutive indices of `axis` form a block; without it the axis is the last
 * dimension, vnni = the format's pack size (2 for the 4-bit formats, 1 for
 * int8) -- and one block = the bs * vnni elements sharing (pre, post).
 * out: same order, 4-bit formats with two codes per byte (element 2*v1 in the
 * low nibble); scales[pre][post] (u8 for MXFP4, f32 otherwise). */
int tppx_quantize_per_block(const void* in, int in_dtype, int qfmt, int64_t pre,
                            int64_t bs, int64_t post, int64_t vnni, void* out,
                            void* scales, tppx_stream_t stream);
int tppx_dequantize_per_block(const void* q, const void* scales, int qfmt,
                              int64_t pre, int64_t bs, int64_t post,
                              int64_t vnni, void* out_f32, tppx_stream_t stream);

/* Replaces qtype.remap_and_quantize_qint2_intlv (src/csrc/qtypes.cpp:1004-1073;
 * bound at :1092; the "qint2" choice of FixLinear, llm_common.py:506-509) for
 * N % 32 == 0: ternary weights, scale = max(|w|, 1e-8) per (output channel,
 * block of bs input channels), code 0 / 1 / 2 for 0 / +1 / -1, four codes per
 * byte interleaved over output channels:
 *   q      u8  [N/32][K/bs][bs/4][8 k2][4 c3]: bits 2*k3 hold the code of
 *              W[n1*32 + k3*8 + k2][b*bs + c2*4 + c3]
 *   scales f32 [N/32][K/bs][32]
 * `w` is a blocked weight as for tppx_quantize_mxfp4.  The reference's own
 * dequantize() of such a tensor indexes a 4-entry table with whole bytes
 * (qtypes.h:232-239), so tppx_dequantize_qint2_intlv defines the meaningful
 * result instead: code value * scale in the logical blocked shape
 * [N/32][K/bs][bs/4][32][4]. */
int tppx_quantize_qint2_intlv(const void* w, int w_dtype, int64_t N, int64_t K,
                              int64_t bk, int64_t bc, int64_t vnni, int64_t bs,
                              void* q, void* scales, tppx_stream_t stream);
int tppx_dequantize_qint2_intlv(const void* q, const void* scales, int64_t N,
                                int64_t K, int64_t bs, void* out_f32,
                                tppx_stream_t stream);

/* Low-bit affine weights run on the W8A8 kernels (TppBlockedQInt8LinearW takes
 * kQUInt4x2 / kQUInt2x4 weights with int8 activations and int32 block sums,
 * src/csrc/fused_gemm.h:1112-1128): a one-time expansion of the packed codes
 * into the native int8 tiles tppx_linear_qint8 consumes (qbs = bs).
 * tppx_prepack_qint2: the interleaved layout above -> q_nat i8 (N*K bytes) and
 * scales_nat f32 [N/16][K/bs][16].  tppx_prepack_qint4: an INT4 weight in the
 * VNNI2 layout [N/16][K/bs][bs/2][16] bytes (two codes each) -> q_nat; its
 * scales [N/16][K/bs][1][16] are used unchanged. */
int tppx_prepack_qint2(const void* q_ref, const void* scales_ref, int64_t N,
                       int64_t K, int64_t bs, void* q_nat, void* scales_nat,
                       tppx_stream_t stream);
int tppx_prepack_qint4(const void* q_ref, int64_t N, int64_t K, int64_t bs,
                       void* q_nat, tppx_stream_t stream);

/* Reference layout -> native layout.  Plays the role of the reference's cached
 * first-token weight remap (wt_tensor_for_first_token,
 * src/csrc/llm/fused_llm_infer.cpp:366-420): a one-time re-layout kept next to
 * the weight.  MXFP4 needs K%128==0. */
int tppx_prepack_mxfp4(const void* qdata_ref, const void* scales_ref, int64_t N,
                       int64_t K, void* qdata_nat, void* scales_nat,
                       tppx_stream_t stream);
int tppx_prepack_qint8(const void* q_ref, int64_t N, int64_t K, int64_t qbs,
                       void* q_nat, tppx_stream_t stream);

/* Replaces quantize_int8sym(t_in, block_size, -1, false) on the activation
 * (src/csrc/fused_gemm.h:1249 -> src/csrc/qtypes.cpp:613-624): x bf16 [M][K]
 * -> xq i8 [M][K], sa f32 [M][K/qbs]. */
int tppx_quant_act_int8(const void* x, int64_t M, int64_t K, int64_t qbs,
                        void* xq, void* sa, tppx_stream_t stream);

/* ---- linears ----------------------------------------------------------- */

/* Workspace (`ws`, `ws_bytes`) of the linear entry points: optional device
 * scratch, 256-byte aligned, that lets decode-shape launches with more than 16
 * rows split K across workgroups (fp32 partial tiles, summed inside the same
 * launch by whichever workgroup of a tile finishes last, in a fixed order).
 * It needs no initialisation and carries no state between calls.
 * Launches that share a workspace must be ordered on one stream.  With
 * ws == NULL (or too small) the kernels simply do not split K.  32 MiB covers
 * every decode shape up to M=64, N=32768.  The arrival counters of such a
 * launch live in the library (16384 per device, handed out in rotation, at
 * most 256 per launch), so K-split launches on different streams may overlap
 * as long as fewer than 64 of them are in flight on one device. */

/* Replaces call_gemm_with_post_op -> TppBlockedLinearW<bf16,uint8_t,bf16>
 * (MXFP4 branch, src/csrc/fused_gemm.h:785-1073,1510-1522) i.e.
 * torch.ops.tpp_llm.fc_plain (src/csrc/llm/fused_llm_infer.cpp:1514,1589) and
 * the post-op GEMMs of the decoder layer (fused_llm_infer.cpp:1261-1273).
 *   y[M][N] = post( bf16( bias[n] + sum_k x[m][k]*deq(W)[n][k] ) )
 * x bf16 [M][K]; qw/sw native layout; bias bf16 [N] or NULL; post_in /
 * post_in2 bf16 [M][N] as the post-op needs; y bf16 [M][N]. */
int tppx_linear_mxfp4(const void* x, const void* qw, const void* sw,
                      const void* bias, const void* post_in,
                      const void* post_in2, void* y, int64_t M, int64_t N,
                      int64_t K, int post_op, float post_scale, int flags,
                      void* ws, int64_t ws_bytes, tppx_stream_t stream);

/* Activations for TPPX_FLAG_ACT_FP8 (no counterpart in the reference, whose
 * activations stay bf16; the closest is its W4A8 USE_MXFP4_INT8 variant,
 * src/csrc/fused_gemm.h:965-978): x bf16 [M][K] -> MXFP8, OCP E4M3 elements with
 * one E8M0 scale per 32 input channels (exponent floor(log2 max|x|) - 8, round
 * to nearest even, saturating at 448), in MFMA operand order:
 * with Mp = roundup(M, 64): xq [Mp/16][K/128][2][64][16] bytes (lane g*16 + m
 * of a 16-row tile holds channels h*64 + g*16 .. +15 of row m in half h) and
 * xs [Mp/64][K/128][64][4] bytes (byte t of lane g*16 + m: the scale of
 * channels g*32..g*32+31 of row m of the group's row tile t); rows past M are
 * zeros.  K%128==0.  tppx_linear_mxfp4 and its siblings call it themselves
 * when the flag is set (workspace: 33/32 * Mp * K bytes). */
int tppx_quant_act_mxfp8(const void* x, int64_t M, int64_t K, void* xq, void* xs,
                         tppx_stream_t stream);

/* Unquantized bf16 weights: TppBlockedLinearW<bf16,bf16>
 * (src/csrc/fused_gemm.h:785-1073 with the plain BRGEMM of :951-1064), the
 * class the reference's default bf16 lm_head runs through
 * (src/tpp_pytorch_extension/llm/fused_llama_infer.py:218-224).
 * tppx_prepack_bf16: blocked bf16 weight [N/bk][K/bc][bc/vnni][bk][vnni]
 * (vnni 2 = BlockedLinear's VNNI2 pairs, blocked_layout.py:75-80; bk=1,
 * bc=K, vnni=1 = a plain [N][K] matrix) -> native bf16 tiles
 * [N/16][K/128][4][64][8] (N*K*2 bytes).  N%16==0, K%128==0.
 * tppx_linear_bf16: y = post( bf16( bias[n] + sum_k x[m][k]*W[n][k] ) ) with
 * the row-group kernel at any M (beyond 64 rows every block of 64 rows
 * streams the weights again: meant for lm_head-sized M, not for prefill). */
int tppx_prepack_bf16(const void* w_ref, int64_t N, int64_t K, int64_t bk,
                      int64_t bc, int vnni, void* w_nat, tppx_stream_t stream);
int tppx_linear_bf16(const void* x, const void* w_nat, const void* bias,
                     const void* post_in, const void* post_in2, void* y,
                     int64_t M, int64_t N, int64_t K, int post_op,
                     float post_scale, int flags, tppx_stream_t stream);

/* Replaces TppBlockedQInt8LinearW<bf16,uint8_t,bf16>
 * (src/csrc/fused_gemm.h:1076-1341,1530-1534): activations are quantized into
 * the caller's scratch xq (room for roundup(M,64)*K bytes) / sa (room for
 * roundup(M,64)*(K/qbs) floats) and then
 *   y = post( bf16( bias + sum_b float(sum_{k in b} xq*wq) * sa[m][b]*sw[n][b] ) )
 * x == NULL means xq (i8 [M][K] row-major) / sa already hold the quantized
 * activations (the reference accepts a pre-quantized qint8 input,
 * fused_gemm.h:1244-1246).  With x != NULL the layout written into xq is
 * private to the library (the GEMM reads it in MFMA operand order). */
int tppx_linear_qint8(const void* x, void* xq, void* sa, const void* qw,
                      const void* sw, const void* bias, const void* post_in,
                      const void* post_in2, void* y, int64_t M, int64_t N,
                      int64_t K, int64_t qbs, int post_op, float post_scale,
                      int flags, void* ws, int64_t ws_bytes,
                      tppx_stream_t stream);

/* W4A8 decode calls (M <= 16) in one launch.  tppx_prepack_mxfp4_int8 turns the USE_MXFP4_INT8 weight
 * (src/csrc/qtypes.cpp:787-790, 840-861: q u8 [N/8][K/bc][bc/8][8][4], scales u8 [N/8][K/bc][bc/32][8]) into
 * tiles in MFMA operand order (q_nat N*K/2 bytes, s_nat N*K/32 bytes; N % 16 == 0, K % 128 == 0), once per weight;
 * tppx_linear_mxfp4_int8_rows is TppBlockedLinearW<int8_t, uint8_t, Tout> (src/csrc/fused_gemm.h:965-978) on them
 * for bf16 activations x [M][K]: the rows are quantized to int8 over blocks of 32 inside the launch
 * (quantize_int8sym, scales times 6/127), K is split over the waves of a workgroup.  Same arithmetic as
 * tppx_linear_mxfp4_int8 (exact int32 block sums, one fp32 multiply-add per block) in another summation order.
 * TPPX_EUNSUPPORTED for more than 16 rows or rows that do not fit the LDS: quantize the activations and call
 * tppx_linear_mxfp4_int8 then. */
int tppx_prepack_mxfp4_int8(const void* q_ref, const void* sc_ref, int64_t N,
                            int64_t K, int64_t bc, void* q_nat, void* s_nat,
                            tppx_stream_t stream);
int tppx_linear_mxfp4_int8_rows(const void* x, const void* q_nat,
                                const void* s_nat, const void* bias,
                                const void* post_in, const void* post_in2,
                                void* y, int64_t M, int64_t N, int64_t K,
                                int post_op, float post_scale,
                                tppx_stream_t stream);

/* W4A8 with many rows (prompt passes): the same arithmetic on the bf16 MFMA.  An int8 activation and a weight
 * integer times its block's power of two are exact in bf16 and so is the fp32 sum of one MX block's 32 products, so
 * one K = 32 MFMA per block gives float(int32 block sum) * 2^(e - 127) and the fold is one fp32 multiply-add with
 * sa[row][block] per output and block, in ascending block order from the bias: the same bits as
 * tppx_linear_mxfp4_int8's formula (src/csrc/fused_gemm.h:965-978).  tppx_prepack_mxfp4_int8_wide turns the
 * USE_MXFP4_INT8 weight (layout as for tppx_prepack_mxfp4_int8) into bf16 operand tiles, w_nat N*K*2 bytes,
 * N % 16 == 0, K % 128 == 0, once per weight.  tppx_linear_mxfp4_int8_wide takes bf16 rows x [M][K], quantizes
 * them over blocks of 32 (quantize_int8sym, scales times 6/127) into the workspace and runs the GEMM; ws must hold
 * Mp*K*2 + Mp*(K/32)*4 bytes with Mp = M rounded up to a multiple of 128, 16-byte aligned. */
int tppx_prepack_mxfp4_int8_wide(const void* q_ref, const void* sc_ref,
                                 int64_t N, int64_t K, int64_t bc, void* w_nat,
                                 tppx_stream_t stream);
int tppx_linear_mxfp4_int8_wide(const void* x, const void* w_nat,
                                const void* bias, const void* post_in,
                                const void* post_in2, void* y, int64_t M,
                                int64_t N, int64_t K, int post_op,
                                float post_scale, void* ws, int64_t ws_bytes,
                                tppx_stream_t stream);

/* QINT4 / ternary QINT2 weights at their own width for decode shapes.  The reference multiplies the packed codes as
 * they lie (TppBlockedQInt8LinearW on kQUInt4x2 / kQUInt2x4 weights, src/csrc/fused_gemm.h:1110-1126; BRGEMM with
 * b_vnni, src/csrc/xsmm_functors.h:2640-2666).  tppx_pack_qint_tiles turns the native int8 tiles of such a weight
 * (tppx_prepack_qint4 / tppx_prepack_qint2) into 4- or 2-bit codes in the kernel's order, N*K*bits/8 bytes;
 * tppx_linear_qintx is tppx_linear_qint8 on them for decode shapes and 256-wide scale blocks, the codes expanded
 * in registers in front of the int8 MFMA -- the same integer sums, scales and rounding as the expanded weight, so
 * the same bits.  Up to 16 rows the bf16 activations are quantized inside the launch (xq, sa may be NULL); more rows
 * run block rows of 32 / 64 behind the activation quantizer and need the xq / sa scratch of tppx_linear_qint8
 * (flags: 0 or TPPX_FLAG_XQ_REUSE).  sw: the f32 scales tppx_linear_qint8 takes.  TPPX_EUNSUPPORTED when at most
 * 16 rows do not fit the in-kernel quantisation (run the expanded tiles then). */
int tppx_pack_qint_tiles(const void* native_i8, int64_t N, int64_t K, int bits,
                         void* packed, tppx_stream_t stream);
int tppx_linear_qintx(const void* x, void* xq, void* sa, const void* qw_packed,
                      const void* sw, const void* bias, const void* post_in,
                      const void* post_in2, void* y, int64_t M, int64_t N,
                      int64_t K, int bits, int post_op, float post_scale,
                      int flags, tppx_stream_t stream);

/* No counterpart in the reference.  tppx_linear_qint8 for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the quantised activations, their
 * scales and the K-split workspace live in a static device array of the library (about 6.1 MiB per GPU, held
 * until the process ends) instead of caller buffers.  x must be given (bf16 [M][K]); limits: M <= 64 (decode
 * shapes), K <= 32768 -- larger sizes return TPPX_ESHAPE; flags: 0 or TPPX_FLAG_FORCE_SKINNY.  Same kernels and
 * the same bits as tppx_linear_qint8 with a 4 MiB workspace.  The call itself allocates nothing and frees nothing.
 * All calls on one GPU share the one array: calls that overlap on a GPU (different streams without ordering)
 * race; order them on one stream or with events.  Nothing in the array has to start at zero: every value that reaches
 * an output was written earlier in the same call (the padding rows of the last 16-row tile of quantised
 * activations are read as they lie, but the results of those rows are never stored).  The first call on a device
 * looks up the array's address (hipGetSymbolAddress, which may load the code object): make one eager call per
 * device before recording the entry point into a graph. */
int tppx_linear_qint8_noalloc(const void* x, const void* qw, const void* sw,
                              const void* bias, const void* post_in,
                              const void* post_in2, void* y, int64_t M,
                              int64_t N, int64_t K, int64_t qbs, int post_op,
                              float post_scale, int flags, tppx_stream_t stream);

/* One GEMM of a fused group sharing the activation. */
typedef struct tppx_seg {
  const void* qw;       /* native weight */
  const void* sw;       /* its scales    */
  const void* bias;     /* bf16 [N] or NULL */
  const void* post_in;  /* bf16 [M][N] or NULL */
  const void* post_in2; /* bf16 [M][N] or NULL */
  void* y;              /* bf16 [M][N] */
  int64_t N;
  int32_t post_op;
  float post_scale;
} tppx_seg;

/* Replaces fused_qkv_gemm -> TppBlockedLinearW::fused_gemm /
 * TppBlockedQInt8LinearW::fused_gemm (src/csrc/llm/fused_llm_infer.cpp:423-505,
 * src/csrc/fused_gemm.h:1001-1064,1273-1332): up to 4 GEMMs over one
 * activation in one launch, each with its own output tensor and post-op. */
int tppx_multi_linear_mxfp4(const void* x, const tppx_seg* segs, int n_segs,
                            int64_t M, int64_t K, int flags, void* ws,
                            int64_t ws_bytes, tppx_stream_t stream);
int tppx_multi_linear_qint8(const void* x, void* xq, void* sa,
                            const tppx_seg* segs, int n_segs, int64_t M,
                            int64_t K, int64_t qbs, int flags, void* ws,
                            int64_t ws_bytes, tppx_stream_t stream);

/* Replaces the gate/up pair of the Llama MLP
 * (src/csrc/llm/fused_llm_infer.cpp:1271-1272: i_gemm(SiluPostOp) then
 * i_gemm(MulPostOp)) in one launch with the same bf16 rounding points:
 *   g = silu(bf16(x Wg^T + bg));  y = bf16( g * bf16(x Wu^T + bu) )
 * Prefill shapes (M >= 192): with M * N * 2 bytes of workspace both GEMMs run
 * as one grid (the gate tile parked in the workspace) followed by an
 * elementwise pass; without it, as two launches.  Same bits either way. */
int tppx_swiglu_mxfp4(const void* x, const void* qw_gate, const void* sw_gate,
                      const void* bias_gate, const void* qw_up,
                      const void* sw_up, const void* bias_up, void* y,
                      int64_t M, int64_t N, int64_t K, int flags, void* ws,
                      int64_t ws_bytes, tppx_stream_t stream);

/* llama_rms_norm followed by the GEMMs that consume it, in ONE launch, for
 * decode steps (M <= 16): the two calls
 *   t_HS = llama_rms_norm(t_HS, gamma, eps); fused_qkv_gemm(t_HS, {Wq,Wk,Wv}, ...)
 * (src/csrc/llm/fused_llm_infer.cpp:1231,1247-1251) resp.
 *   t_HS = llama_rms_norm(t_SO, gamma, eps); i_gemm(Silu)...; i_gemm(Mul)...
 * (:1269-1272) with the same bf16 rounding of the normalised activations.
 * gamma f32 [K]; gamma == NULL skips the normalisation (same kernel, plain x).
 * TPPX_EUNSUPPORTED when M > 16 or K is too large for the LDS staging: run
 * tppx_rms_norm and the GEMM entry points separately then. */
int tppx_norm_multi_linear_mxfp4(const void* x, const void* gamma, float eps,
                                 const tppx_seg* segs, int n_segs, int64_t M,
                                 int64_t K, int flags, tppx_stream_t stream);
int tppx_norm_swiglu_mxfp4(const void* x, const void* gamma, float eps,
                           const void* qw_gate, const void* sw_gate,
                           const void* bias_gate, const void* qw_up,
                           const void* sw_up, const void* bias_up, void* y,
                           int64_t M, int64_t N, int64_t K, int flags,
                           tppx_stream_t stream);

/* The same two fusions without a pass over x for the normalisation: the launch
 * that WROTE x (the residual-add GEMM before the norm: o-projection,
 * down-projection of the previous layer) leaves, per row, the sums of squares
 * of its bf16 outputs in row_sumsq, f32 [16][256] ([row][workgroup], every call
 * overwrites the 256 slots of its M rows); the consuming launch adds a row's
 * 256 slots, takes 1/sqrt(sum/K + eps) and normalises the activations on
 * their way into LDS.  M <= 16, MXFP4 decode kernels only (TPPX_EUNSUPPORTED
 * otherwise: use the entry points above).  The table is plain device memory
 * owned by the caller; producer and consumer must be ordered on one stream.
 * No counterpart in the reference (its norm is a separate pass,
 * fused_llm_infer.cpp:1231,1269); results differ from that pass only through
 * the summation order of the squares (fp32). */
int tppx_linear_mxfp4_rowsq(const void* x, const void* qw, const void* sw,
                            const void* bias, const void* post_in,
                            const void* post_in2, void* y, int64_t M, int64_t N,
                            int64_t K, int post_op, float post_scale, int flags,
                            void* ws, int64_t ws_bytes, void* row_sumsq,
                            tppx_stream_t stream);
int tppx_normsq_multi_linear_mxfp4(const void* x, const void* row_sumsq,
                                   const void* gamma, float eps,
                                   const tppx_seg* segs, int n_segs, int64_t M,
                                   int64_t K, int flags, tppx_stream_t stream);
int tppx_normsq_swiglu_mxfp4(const void* x, const void* row_sumsq,
                             const void* gamma, float eps, const void* qw_gate,
                             const void* sw_gate, const void* bias_gate,
                             const void* qw_up, const void* sw_up,
                             const void* bias_up, void* y, int64_t M, int64_t N,
                             int64_t K, int flags, tppx_stream_t stream);

/* ---- decode-side operators of the decoder layer -------------------------- */

/* Replaces llama_rms_norm / RMSNormFwdTPP (src/csrc/llm/fused_llm_infer.cpp:309-363,
 * src/csrc/xsmm_functors.h:4575-4660): y = bf16((x * rsqrt(mean(x^2) + eps)) * gamma),
 * x, y bf16 [rows][K] (K % 8 == 0), gamma f32 or bf16 [K] (TPPX_DT_*). */
int tppx_rms_norm(const void* x, const void* gamma, int gamma_dtype, void* y,
                  int64_t rows, int64_t K, float eps, tppx_stream_t stream);

/* Replaces apply_rotary_pos_emb_llama (src/csrc/llm/fused_llm_infer.cpp:207-253):
 * in place on t bf16 [B][S][N][H]; emb_pos f32 [2][MP][HR] (cos, sin); pos i64
 * [B_pos][S] with B_pos 1 or B; positions >= MP are left untouched.  H a
 * multiple of 8 up to 512, HR a multiple of 16. */
int tppx_rotary_llama(void* t, const void* emb_pos, const void* pos, int64_t B,
                      int64_t S, int64_t N, int64_t H, int64_t MP, int64_t HR,
                      int64_t B_pos, tppx_stream_t stream);

/* The two rotary calls of LlamaDecoderLayer::_forward (fused_llm_infer.cpp:1252-1253)
 * and LayerCache::update (src/csrc/llm/attn.h:198-222) in one launch: rotates q
 * (may be NULL) and k in place and writes the rotated k and v rows into the
 * cache [B][Nkv][Smax][H] at position *offset_dev + s (offset_dev: device i32,
 * the cache length before the call, so the call can sit in a replayed graph;
 * emb_pos == NULL appends without rotation). */
int tppx_rotary_kv_append_llama(void* q, void* k, const void* v,
                                const void* emb_pos, const void* pos,
                                void* kcache, void* vcache,
                                const void* offset_dev, int64_t B, int64_t S,
                                int64_t Nq, int64_t Nkv, int64_t H, int64_t MP,
                                int64_t HR, int64_t B_pos, int64_t Smax,
                                tppx_stream_t stream);

/* Replaces lyr_norm / LayerNormFwdTPP (src/csrc/llm/fused_llm_infer.cpp:254-306,
 * src/csrc/xsmm_functors.h:4749-4786), the normalisation of GPTJBlock and
 * OPTDecoderLayer: m = mean(x), v = max(mean(x^2) - m^2, 0), s = 1/sqrt(v + eps),
 * y = bf16((x * s - s * m) * gamma + beta); x, y bf16 [rows][K] (K % 8 == 0),
 * gamma and beta both f32 or both bf16 [K] (TPPX_DT_*). */
int tppx_layer_norm(const void* x, const void* gamma, const void* beta,
                    int param_dtype, void* y, int64_t rows, int64_t K, float eps,
                    tppx_stream_t stream);

/* Replaces apply_rotary_pos_emb_gptj (src/csrc/llm/fused_llm_infer.cpp:150-205):
 * in place on t bf16 [B][S][N][H], pairs (h, h + 1) for h < HR; emb_pos f32
 * [MP][HR] = sin | cos (sin of pair h/2 at [p][h/2], cos at [p][HR/2 + h/2]);
 * pos i64 [B_pos][S]; positions >= MP are left untouched. */
int tppx_rotary_gptj(void* t, const void* emb_pos, const void* pos, int64_t B,
                     int64_t S, int64_t N, int64_t H, int64_t MP, int64_t HR,
                     int64_t B_pos, tppx_stream_t stream);

/* The two rotary calls of GPTJBlock::_forward (fused_llm_infer.cpp:784-785) and
 * LayerCache::update (src/csrc/llm/attn.h:198-222) in one launch: as
 * tppx_rotary_kv_append_llama with the GPT-J pairing and table. */
int tppx_rotary_kv_append_gptj(void* q, void* k, const void* v,
                               const void* emb_pos, const void* pos,
                               void* kcache, void* vcache,
                               const void* offset_dev, int64_t B, int64_t S,
                               int64_t Nq, int64_t Nkv, int64_t H, int64_t MP,
                               int64_t HR, int64_t B_pos, int64_t Smax,
                               tppx_stream_t stream);

/* Replaces attn<T> (src/csrc/llm/attn.cpp:781-955) for one query token per
 * sequence: q bf16 [B][Nq][128], cache bf16 [B][Nkv][Smax][128], additive mask
 * bf16 [B][mask_ld] or NULL; valid keys = *kv_len_dev (device i32) + kv_len_add
 * (the counter may still hold the length before this step's append); out bf16
 * [B][Nq][128].  ws: optional scratch for split-KV partial results.  Head sizes
 * H other than 128 (multiples of 8 up to 256, tensors [..][H]) run a kernel of
 * the same layout with 8, 16 or 32 lanes per key (not the rotary-fused form);
 * anything else returns TPPX_EUNSUPPORTED. */
int tppx_attn_decode(const void* q, const void* kcache, const void* vcache,
                     const void* mask, int64_t mask_ld, const void* kv_len_dev,
                     int64_t kv_len_add, void* out, int64_t B, int64_t Nq,
                     int64_t Nkv, int64_t H,
                     int64_t Smax, void* ws, int64_t ws_bytes,
                     tppx_stream_t stream);

/* The same with the launch in front of it folded in: tppx_rotary_kv_append_llama
 * for one token per sequence followed by tppx_attn_decode with kv_len_add = 1
 * (fused_llm_infer.cpp:1252-1253, attn.h:198-222, attn.cpp:781-955).  q bf16
 * [B][Nq][128], k / v bf16 [B][Nkv][128] as the q/k/v GEMMs leave them
 * (unrotated; they stay untouched), emb_pos f32 [2][MP][128] or NULL (append
 * without rotation), pos i64 [B_pos] with B_pos 1 or B; the rotated key and the
 * value are written to cache position *kv_len_dev (nothing is written when the
 * cache is full) and attended to together with the cached keys. */
int tppx_attn_decode_rotary(const void* q, const void* k, const void* v,
                            const void* emb_pos, const void* pos, int64_t B_pos,
                            int64_t MP, int64_t HR, void* kcache, void* vcache,
                            const void* mask, int64_t mask_ld,
                            const void* kv_len_dev, void* out, int64_t B,
                            int64_t Nq, int64_t Nkv, int64_t H, int64_t Smax,
                            void* ws, int64_t ws_bytes, tppx_stream_t stream);

/* The same attn<T> (src/csrc/llm/attn.cpp:781-955, isCausal) for S query tokens
 * per sequence (prompt processing, or several new tokens on a filled cache):
 * q / out bf16 [B][S][Nq][128]; the cache already holds the S new keys at
 * positions past_len .. past_len+S-1 (tppx_rotary_kv_append_llama before this
 * call); query i sees keys 0 .. past_len+i; additive mask bf16 [B][mask_ld]
 * over key positions or NULL.  Head sizes other than 128 (multiples of 8 up to
 * 256) run the same kernel over a head size padded to 64, 128 or 256. */
int tppx_attn_prefill(const void* q, const void* kcache, const void* vcache,
                      const void* mask, int64_t mask_ld, int64_t past_len,
                      void* out, int64_t B, int64_t S, int64_t Nq, int64_t Nkv,
                      int64_t H, int64_t Smax, tppx_stream_t stream);

/* The element-type switch of fc_plain_wrap (src/csrc/llm/fused_llm_infer.cpp:
 * 1526-1545) for QINT8-family weights and float / half activations, or a
 * pre-quantized qint8 input whose compute type is float
 * (TppBlockedQInt8LinearW<float,uint8_t,float>, src/csrc/fused_gemm.h:1076-1341):
 *   y[m][n] = bias[n] + sum_b float(sum_{k in b} xq*wq) * (sa[m][b]*sw[n][b])
 * in fp32, one fused multiply-add per K block in ascending order, no post-op.
 * xq i8 [M][K] row-major and sa f32 [M][K/qbs] come from
 * tppx_quantize_per_block on the activations (quantize_int8sym,
 * fused_gemm.h:1248); qw / sw are the native weight tiles / scales; bias f32
 * [N] or NULL; y f32 [M][N]. */
int tppx_linear_qint8_f32(const void* xq, const void* sa, const void* qw,
                          const void* sw, const void* bias_f32, void* y_f32,
                          int64_t M, int64_t N, int64_t K, int64_t qbs,
                          tppx_stream_t stream);

/* The same switch for MXFP4 and unquantized bf16 weights:
 * TppBlockedLinearW<Tin, uint8_t, Tout> / <Tin, bfloat16, Tout> with Tin =
 * float or half (src/csrc/fused_gemm.h:1519-1523, 1541-1550; 785-1073).  The
 * activations keep their own precision; every weight value is exact in fp32;
 *   y[m][n] = bias[n] + sum_k x[m][k] * w[n][k]      in fp32.
 * x fp32 or fp16 [M][K] (x_dtype = TPPX_DT_F32 / TPPX_DT_F16); w / sw native
 * tiles (w_kind = TPPX_W_MXFP4: tppx_prepack_mxfp4's tiles and scale bytes;
 * TPPX_W_BF16: tppx_prepack_bf16's tiles, sw ignored); bias f32 [N] or NULL;
 * y f32 [M][N].  K % 128 == 0.  The caller rounds to the activations' type
 * and applies the post-op with tppx_post_op_wide. */
int tppx_linear_wide(const void* x, int x_dtype, const void* w, const void* sw,
                     int w_kind, const void* bias_f32, void* y_f32, int64_t M,
                     int64_t N, int64_t K, tppx_stream_t stream);

/* Post-ops of call_gemm_with_post_op on a float or half output tile
 * (src/csrc/fused_gemm.h:1343-1488 with Tout = float / half): out[i] =
 * post(round_T(acc[i])) with a rounding to T (T = half; none for float) where
 * the CPU path stores its tile.  acc f32 [count] (bias + dot product);
 * post_in / post_in2 and out in T (out_dtype = TPPX_DT_F32 / TPPX_DT_F16). */
int tppx_post_op_wide(const void* acc_f32, int out_dtype, int post_op,
                      const void* post_in, const void* post_in2,
                      float post_scale, void* out, int64_t count,
                      tppx_stream_t stream);

/* W4A8, the reference's USE_MXFP4_INT8 mode: TppBlockedLinearW<int8_t, uint8_t,
 * Tout> (src/csrc/fused_gemm.h:965-978, 1523-1526) on the weight layout of
 * remap_and_quantize_mxfp4 under that flag (src/csrc/qtypes.cpp:787-790,
 * 840-861), read as the reference stores it:
 *   q  u8 [N/8][K/bc][bc/8][8][4]   byte j of a group of 8 K values =
 *                                   value j | value 4+j << 4 (E2M1 codes)
 *   sc u8 [N/8][K/bc][bc/32][8]     E8M0 scale per 32 K values and channel
 * xq i8 [M][K] + sa f32 [M][K/32]: activations quantized over blocks of 32
 * (tppx_quantize_per_block), the scales already multiplied by 6/127
 * (fused_gemm.h:975-977).
 *   y = post( bf16( bias + sum_b float(sum_k xq*wi) * (sa[m][b] * 2^(e-127)) ) )
 * wi = E2M1 value * 127/6 rounded to the nearest integer (0 11 21 32 42 64 85
 * 127): the table is the reference JIT library's and is restated, so results
 * match the reference within that rounding only.  bias / post_in / post_in2 /
 * y bf16; N%16==0, bc%32==0, K%bc==0. */
int tppx_linear_mxfp4_int8(const void* xq, const void* sa, const void* q,
                           const void* sc, const void* bias, const void* post_in,
                           const void* post_in2, void* y, int64_t M, int64_t N,
                           int64_t K, int64_t bc, int post_op, float post_scale,
                           tppx_stream_t stream);

/* fused_qkv_gemm (src/csrc/llm/fused_llm_infer.cpp:423-505) for decode steps
 * (M <= 16) as ONE GEMM over the concatenated native weights of up to three
 * projections (native tiles and scales are per 16-channel tile, so the
 * concatenation along N is the buffers one after the other): every workgroup
 * gets the same number of tiles whatever the projections' widths (three
 * separate segments of 256 tiles each do not divide into 256 groups of 3).
 * Output columns [0, n1) | [n1, n2) | [n2, N) go to three row-major bf16
 * matrices laid one after the other in y (M x n1, M x (n2-n1), M x (N-n2)).
 * gamma != NULL: llama_rms_norm on x inside the launch (row_sumsq != NULL: from
 * the row sums the launch that wrote x left, as tppx_normsq_multi_linear_mxfp4;
 * NULL: sums formed in the launch, as tppx_norm_multi_linear_mxfp4).  bias bf16
 * [N] over the concatenated channels or NULL.  TPPX_EUNSUPPORTED when the
 * LDS-staged kernel does not take the shape (callers fall back to
 * tppx_*multi_linear_mxfp4). */
int tppx_qkv_linear_mxfp4(const void* x, const void* row_sumsq, const void* gamma,
                          float eps, const void* qw, const void* sw,
                          const void* bias, void* y, int64_t M, int64_t N,
                          int64_t K, int64_t n1, int64_t n2, int flags,
                          tppx_stream_t stream);

/* Greedy step of a generation loop (what transformers' generate() does between
 * two forward passes when examples/llm/run_generation.py:420 runs with
 * --greedy: torch.argmax over the logits, the embedding lookup of the chosen
 * token) as one launch, so that a decode step replayed as a graph ends in a
 * single small kernel:
 *   tokens[b] (int64) = the first maximal index of logits[b][0..V) (bf16; a NaN
 *                       counts as maximal, like torch.argmax)
 *   pos[b] (int64)   += 1                       (pos != NULL)
 *   seq_len[0] (i32) += 1                       (seq_len != NULL)
 *   h_next[b][:]      = embed[tokens[b]][:]     (h_next != NULL; bf16 [*][hidden])
 * V % 8 == 0, hidden % 8 == 0. */
int tppx_greedy_next(const void* logits, int64_t B, int64_t V, const void* embed,
                     int64_t hidden, void* tokens, void* pos, void* seq_len,
                     void* h_next, tppx_stream_t stream);

/* ---- launch plans ------------------------------------------------------- */

/* No counterpart in the reference.  Writes into buf, one line per kernel, what
 * tppx_linear_mxfp4 / tppx_linear_qint8 would enqueue for this shape
 * ("<kernel name as a profiler prints it> grid=XxYxZ block=B lds=L"), and
 * launches nothing: for benchmarks and profilers that must name the kernel they
 * time.  x_given = 0 describes the pre-quantized (x == NULL) case. */
int tppx_plan_linear_mxfp4(int64_t M, int64_t N, int64_t K, int flags,
                           int64_t ws_bytes, char* buf, int64_t buf_len);
int tppx_plan_linear_qint8(int64_t M, int64_t N, int64_t K, int64_t qbs,
                           int x_given, int flags, int64_t ws_bytes, char* buf,
                           int64_t buf_len);

/* The same for a fused group: Ns[n_segs] output widths over one activation (tppx_multi_linear_*), or, with
 * dual = 1 and two equal widths, the gate/up pair of tppx_swiglu_mxfp4. */
int tppx_plan_multi_linear_mxfp4(const int64_t* Ns, int n_segs, int64_t M,
                                 int64_t K, int dual, int flags,
                                 int64_t ws_bytes, char* buf, int64_t buf_len);
int tppx_plan_multi_linear_qint8(const int64_t* Ns, int n_segs, int64_t M,
                                 int64_t K, int64_t qbs, int x_given, int flags,
                                 int64_t ws_bytes, char* buf, int64_t buf_len);

#ifdef __cplusplus
}
#endif
#endif /* TPPX_H */
