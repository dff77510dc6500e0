// C-ABI entry points of the linear path: argument validation (before any HIP
// call), kernel-family choice and launch.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "tppx_common.h"
#include "tppx_launch.h"

namespace tppx {

static thread_local char g_err[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess)
    return TPPX_OK;
  return set_error(TPPX_EHIP, "%s: HIP error %d (%s)", what, (int)e, hipGetErrorString(e));
}

int env_int(const char* name, int dflt) {
  const char* v = getenv(name);
  return (v && *v) ? atoi(v) : dflt;
}

static bool valid_post(int post) {
  return post >= TPPX_POST_NONE && post <= TPPX_POST_RELU;
}

// Checks one segment and fills the device descriptor.
static int fill_seg(const char* who, const tppx_seg& s, SkinnySeg& d, int n_mult) {
  TPPX_REQUIRE(s.qw && s.sw && s.y, TPPX_EINVAL, "%s: null weight/scale/output pointer", who);
  TPPX_REQUIRE(aligned16(s.qw) && aligned16(s.y), TPPX_EINVAL, "%s: weight/output pointer not 16-byte aligned", who);
  TPPX_REQUIRE(valid_post(s.post_op), TPPX_EINVAL, "%s: unknown post-op id %d", who, s.post_op);
  TPPX_REQUIRE(s.N > 0 && s.N % n_mult == 0, TPPX_ESHAPE, "%s: N=%ld must be a positive multiple of %d", who, (long)s.N, n_mult);
  TPPX_REQUIRE(s.N < (1 << 30), TPPX_ESHAPE, "%s: N=%ld too large", who, (long)s.N);
  bool need1 = s.post_op == TPPX_POST_MUL || s.post_op == TPPX_POST_ADD_SCALE || s.post_op == TPPX_POST_ADD2_SCALE;
  bool need2 = s.post_op == TPPX_POST_ADD2_SCALE;
  TPPX_REQUIRE(!need1 || s.post_in, TPPX_EINVAL, "%s: post-op %d needs post_in", who, s.post_op);
  TPPX_REQUIRE(!need2 || s.post_in2, TPPX_EINVAL, "%s: post-op %d needs post_in2", who, s.post_op);
  d.qw = s.qw;
  d.sw = s.sw;
  d.bias = (const uint16_t*)s.bias;
  d.post_in = need1 ? (const uint16_t*)s.post_in : nullptr;
  d.post_in2 = need2 ? (const uint16_t*)s.post_in2 : nullptr;
  d.y = (uint16_t*)s.y;
  d.N = (int)s.N;
  d.post_op = s.post_op;
  d.post_scale = s.post_scale;
  return TPPX_OK;
}

static int check_common(const char* who, const void* x, int64_t M, int64_t K, int n_segs, int flags) {
  TPPX_REQUIRE(x, TPPX_EINVAL, "%s: null activation pointer", who);
  TPPX_REQUIRE(aligned16(x), TPPX_EINVAL, "%s: activation pointer not 16-byte aligned", who);
  TPPX_REQUIRE(M > 0, TPPX_ESHAPE, "%s: M=%ld must be positive", who, (long)M);
  TPPX_REQUIRE(M < (1 << 24) && K < (1 << 24), TPPX_ESHAPE, "%s: M=%ld or K=%ld too large", who, (long)M, (long)K);
  TPPX_REQUIRE(n_segs >= 1 && n_segs <= TPPX_MAX_SEGS, TPPX_EINVAL, "%s: number of fused GEMMs %d not in 1..%d", who, n_segs, TPPX_MAX_SEGS);
  TPPX_REQUIRE((flags & ~(TPPX_FLAG_FORCE_SKINNY | TPPX_FLAG_FORCE_TILED | TPPX_FLAG_ACT_FP8)) == 0, TPPX_EINVAL, "%s: unknown flag bits 0x%x", who, flags);
  TPPX_REQUIRE(!((flags & TPPX_FLAG_FORCE_SKINNY) && (flags & TPPX_FLAG_FORCE_TILED)), TPPX_EINVAL, "%s: contradictory kernel-family flags", who);
  return TPPX_OK;
}

static int run_mxfp4(const char* who, const void* x, const tppx_seg* segs, int n_segs,
                     int64_t M, int64_t K, int flags, bool dual, hipStream_t stream) {
  int rc = check_common(who, x, M, K, n_segs, flags);
  if (rc)
    return rc;
  TPPX_REQUIRE(segs, TPPX_EINVAL, "%s: null segment table", who);
  TPPX_REQUIRE(K > 0 && K % 64 == 0, TPPX_ESHAPE, "%s: K=%ld must be a positive multiple of 64", who, (long)K);
  TPPX_REQUIRE(K % 128 == 0, TPPX_EUNSUPPORTED, "%s: K=%ld is not a multiple of 128 (native MXFP4 tiles span 128 input channels)", who, (long)K);
  SkinnyParams p;
  memset(&p, 0, sizeof(p));
  int tiles = 0;
  bool all_even = true;
  for (int i = 0; i < n_segs; i++) {
    rc = fill_seg(who, segs[i], p.seg[i], 32);
    if (rc)
      return rc;
    p.seg[i].tile0 = tiles;
    int t = (int)(segs[i].N / 16);
    all_even = all_even && (t % 2 == 0);
    tiles += t;
  }
  if (dual) {
    TPPX_REQUIRE(n_segs == 2 && segs[0].N == segs[1].N, TPPX_ESHAPE, "%s: gate and up projections must have equal N", who);
    tiles = (int)(segs[0].N / 16);
    p.seg[1].tile0 = 0;
  }
  TPPX_REQUIRE(!(flags & TPPX_FLAG_ACT_FP8), TPPX_EUNSUPPORTED, "%s: the FP8-activation path is not available", who);
  p.n_seg = n_segs;
  p.x = x;
  p.M = (int)M;
  p.K = (int)K;
  p.kunits = (int)(K / 128);
  SkinnyPlan pl = plan_skinny(M, tiles, p.kunits, all_even, dual);
  p.units_per_wave = pl.units_per_wave;
  return check_hip(launch_skinny_mxfp4(p, pl, dual, stream), who);
}

static int run_qint8(const char* who, const void* x, void* xq, void* sa, const tppx_seg* segs,
                     int n_segs, int64_t M, int64_t K, int64_t qbs, int flags, hipStream_t stream) {
  // x == NULL: xq / sa already hold quantized activations (the reference's
  // pre-quantized input case, src/csrc/fused_gemm.h:1244-1246)
  int rc = check_common(who, x ? x : xq, M, K, n_segs, flags);
  if (rc)
    return rc;
  TPPX_REQUIRE(segs, TPPX_EINVAL, "%s: null segment table", who);
  TPPX_REQUIRE(xq && sa, TPPX_EINVAL, "%s: null activation-quantization buffers", who);
  TPPX_REQUIRE(aligned16(xq), TPPX_EINVAL, "%s: scratch pointer not 16-byte aligned", who);
  TPPX_REQUIRE(K > 0 && K % 64 == 0, TPPX_ESHAPE, "%s: K=%ld must be a positive multiple of 64", who, (long)K);
  TPPX_REQUIRE(qbs > 0 && qbs % 64 == 0 && K % qbs == 0, TPPX_ESHAPE, "%s: block size mismatch (qbs=%ld, K=%ld)", who, (long)qbs, (long)K);
  SkinnyParams p;
  memset(&p, 0, sizeof(p));
  int tiles = 0;
  bool all_even = true;
  for (int i = 0; i < n_segs; i++) {
    rc = fill_seg(who, segs[i], p.seg[i], 16);
    if (rc)
      return rc;
    p.seg[i].tile0 = tiles;
    int t = (int)(segs[i].N / 16);
    all_even = all_even && (t % 2 == 0);
    tiles += t;
  }
  p.n_seg = n_segs;
  p.xq = xq;
  p.sa = (const float*)sa;
  p.M = (int)M;
  p.K = (int)K;
  p.qbs = (int)qbs;
  p.kunits = (int)(K / qbs);
  if (x) {
    rc = tppx_quant_act_int8(x, M, K, qbs, xq, sa, stream);
    if (rc)
      return rc;
  }
  SkinnyPlan pl = plan_skinny(M, tiles, p.kunits, all_even, false);
  p.units_per_wave = pl.units_per_wave;
  return check_hip(launch_skinny_qint8(p, pl, stream), who);
}

} // namespace tppx

using namespace tppx;

extern "C" int tppx_version(void) {
  return TPPX_VERSION;
}

extern "C" const char* tppx_last_error(void) {
  return g_err;
}

extern "C" int tppx_linear_mxfp4(const void* x, const void* qw, const void* sw,
                                 const void* bias, const void* post_in,
                                 const void* post_in2, void* y, int64_t M,
                                 int64_t N, int64_t K, int post_op,
                                 float post_scale, int flags,
                                 tppx_stream_t stream) {
  tppx_seg s = {qw, sw, bias, post_in, post_in2, y, N, post_op, post_scale};
  return run_mxfp4("tppx_linear_mxfp4", x, &s, 1, M, K, flags, false, (hipStream_t)stream);
}

extern "C" int tppx_multi_linear_mxfp4(const void* x, const tppx_seg* segs,
                                       int n_segs, int64_t M, int64_t K,
                                       int flags, tppx_stream_t stream) {
  return run_mxfp4("tppx_multi_linear_mxfp4", x, segs, n_segs, M, K, flags, false, (hipStream_t)stream);
}

extern "C" int tppx_swiglu_mxfp4(const void* x, const void* qw_gate,
                                 const void* sw_gate, const void* bias_gate,
                                 const void* qw_up, const void* sw_up,
                                 const void* bias_up, void* y, int64_t M,
                                 int64_t N, int64_t K, int flags,
                                 tppx_stream_t stream) {
  tppx_seg s[2] = {{qw_gate, sw_gate, bias_gate, nullptr, nullptr, y, N, TPPX_POST_NONE, 1.0f},
                   {qw_up, sw_up, bias_up, nullptr, nullptr, y, N, TPPX_POST_NONE, 1.0f}};
  return run_mxfp4("tppx_swiglu_mxfp4", x, s, 2, M, K, flags, true, (hipStream_t)stream);
}

extern "C" int tppx_linear_qint8(const void* x, void* xq, void* sa,
                                 const void* qw, const void* sw,
                                 const void* bias, const void* post_in,
                                 const void* post_in2, void* y, int64_t M,
                                 int64_t N, int64_t K, int64_t qbs, int post_op,
                                 float post_scale, int flags,
                                 tppx_stream_t stream) {
  tppx_seg s = {qw, sw, bias, post_in, post_in2, y, N, post_op, post_scale};
  return run_qint8("tppx_linear_qint8", x, xq, sa, &s, 1, M, K, qbs, flags, (hipStream_t)stream);
}

extern "C" int tppx_multi_linear_qint8(const void* x, void* xq, void* sa,
                                       const tppx_seg* segs, int n_segs,
                                       int64_t M, int64_t K, int64_t qbs,
                                       int flags, tppx_stream_t stream) {
  return run_qint8("tppx_multi_linear_qint8", x, xq, sa, segs, n_segs, M, K, qbs, flags, (hipStream_t)stream);
}
