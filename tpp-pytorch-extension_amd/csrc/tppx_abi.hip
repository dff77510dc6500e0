// C-ABI entry points of the linear path: argument validation (before any HIP
// call), kernel-family choice and launch.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <cxxabi.h>
#include <algorithm>
#include <map>
#include <mutex>
#include <string>
#include <utility>

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

static thread_local std::string* g_plan = nullptr;

bool plan_recording() {
  return g_plan != nullptr;
}

void plan_note(const void* kernel_fn, dim3 grid, dim3 block, size_t lds_bytes) {
  if (!g_plan)
    return;
  // name of the device function as a profiler prints it
  std::string name = "?";
  const char* mangled = hipKernelNameRefByPtr(kernel_fn, nullptr);
  if (mangled && *mangled) {
    int status = 0;
    char* dem = abi::__cxa_demangle(mangled, nullptr, nullptr, &status);
    name = (status == 0 && dem) ? dem : mangled;
    free(dem);
    const size_t paren = name.rfind('(');
    if (paren != std::string::npos)
      name.resize(paren);
  }
  char line[640];
  snprintf(line, sizeof(line), "%s grid=%ux%ux%u block=%u lds=%zu\n", name.c_str(), grid.x, grid.y, grid.z, block.x,
           lds_bytes);
  *g_plan += line;
}

// Raises the dynamic-LDS limit of `kern` on the current device once per (device, kernel, size) instead of on
// every launch; the record is per device because the attribute is.
hipError_t allow_dynamic_lds(const void* kern, size_t lds) {
  if (lds <= 48 * 1024)
    return hipSuccess;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return e;
  static std::mutex mu;
  static std::map<std::pair<int, const void*>, size_t> allowed;
  std::lock_guard<std::mutex> lock(mu);
  size_t& have = allowed[{dev, kern}];
  if (lds > have) {
    e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess)
      return e;
    have = lds;
  }
  return hipSuccess;
}

// TPPX_* switches are read from the environment ONCE per process (the first time a launch site asks) and kept, so
// that a launch costs no getenv() and a kernel choice recorded in a captured graph cannot drift from the eager
// one.  tppx_reload_env() drops what was kept (tests that flip a switch call it).  Keyed by the address of the
// name literal: every call site passes its own.
static std::mutex g_env_mu;
static std::map<const char*, std::pair<bool, int>> g_env_kept; // name -> (set in the environment, its value)

int env_int(const char* name, int dflt) {
  std::lock_guard<std::mutex> lock(g_env_mu);
  auto it = g_env_kept.find(name);
  if (it == g_env_kept.end()) {
    const char* v = getenv(name);
    const bool set = v && *v;
    it = g_env_kept.emplace(name, std::make_pair(set, set ? atoi(v) : 0)).first;
  }
  return it->second.first ? it->second.second : dflt;
}

static bool valid_post(int post) {
  return post >= TPPX_POST_NONE && post <= TPPX_POST_RELU;
}

// Checks one segment and fills the device descriptor.
static int fill_seg(const char* who, const tppx_seg& s, DecodeSeg& d, int n_mult) {
  TPPX_REQUIRE(s.qw && s.sw && s.y, TPPX_EINVAL, "%s: null weight/scale/output pointer", who);
  TPPX_REQUIRE(aligned16(s.qw) && aligned16(s.y), TPPX_EINVAL, "%s: weight/output pointer not 16-byte aligned", who);
  TPPX_REQUIRE(valid_post(s.post_op), TPPX_EINVAL, "%s: unknown post-op id %d", who, s.post_op);
  TPPX_REQUIRE(s.N > 0 && s.N % n_mult == 0, TPPX_ESHAPE, "%s: N=%ld must be a positive multiple of %d", who, (long)s.N, n_mult);
  TPPX_REQUIRE(s.N <= (1 << 25), TPPX_ESHAPE, "%s: N=%ld too large (at most 2^25 output channels)", who, (long)s.N);
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
  d.tiles = (int)(s.N / 16);
  d.post_op = s.post_op;
  d.post_scale = s.post_scale;
  return TPPX_OK;
}

static int check_common(const char* who, const void* x, int64_t M, int64_t K, int n_segs, int flags,
                        const void* ws, int64_t ws_bytes) {
  TPPX_REQUIRE(x, TPPX_EINVAL, "%s: null activation pointer", who);
  TPPX_REQUIRE(aligned16(x), TPPX_EINVAL, "%s: activation pointer not 16-byte aligned", who);
  TPPX_REQUIRE(M > 0, TPPX_ESHAPE, "%s: M=%ld must be positive", who, (long)M);
  TPPX_REQUIRE(M < (1 << 24) && K < (1 << 24), TPPX_ESHAPE, "%s: M=%ld or K=%ld too large", who, (long)M, (long)K);
  TPPX_REQUIRE(n_segs >= 1 && n_segs <= TPPX_MAX_SEGS, TPPX_EINVAL, "%s: number of fused GEMMs %d not in 1..%d", who, n_segs, TPPX_MAX_SEGS);
  TPPX_REQUIRE((flags & ~(TPPX_FLAG_FORCE_SKINNY | TPPX_FLAG_FORCE_TILED | TPPX_FLAG_ACT_FP8 | TPPX_FLAG_XQ_REUSE)) == 0, TPPX_EINVAL, "%s: unknown flag bits 0x%x", who, flags);
  TPPX_REQUIRE(!((flags & TPPX_FLAG_FORCE_SKINNY) && (flags & TPPX_FLAG_FORCE_TILED)), TPPX_EINVAL, "%s: contradictory kernel-family flags", who);
  TPPX_REQUIRE(ws_bytes >= 0 && (ws_bytes == 0 || ws), TPPX_EINVAL, "%s: workspace size %ld given with a null workspace", who, (long)ws_bytes);
  TPPX_REQUIRE(ws == nullptr || (reinterpret_cast<uintptr_t>(ws) & 255u) == 0, TPPX_EINVAL, "%s: workspace not 256-byte aligned", who);
  return TPPX_OK;
}

// Fills segments, group/tile offsets; returns total tiles through *tiles.
static void set_groups(DecodeParams& p, int tiles_per_group, bool dual) {
  int groups = 0;
  for (int i = 0; i < p.n_seg; i++) {
    p.seg[i].grp0 = groups;
    groups += (p.seg[i].tiles + tiles_per_group - 1) / tiles_per_group;
  }
  if (dual) {
    p.seg[1].grp0 = 0;
    groups = (p.seg[0].tiles + tiles_per_group - 1) / tiles_per_group;
  }
  p.groups = groups;
}

// LDS-staged decode kernel (M <= 16): channel tiles per workgroup = the fewest that keep the grid within one round of
// 256 workgroups (the kernel runs one workgroup per CU).  False when the K slice of a wave does not fit its staging.
static bool plan_xl(DecodeParams& p, bool dual, int* nt_out) {
  const int nt_max = dual ? 3 : 4;
  int nt = 1;
  for (; nt < nt_max; nt++) {
    set_groups(p, nt, dual);
    if (p.groups <= 256)
      break;
  }
  set_groups(p, nt, dual);
  *nt_out = nt;
  // staging per wave: 16 rows x 32 chunks of 16 bytes, so at most 2 K tiles per wave and slices of 16 or 32 chunks
  return p.units <= 32 && (p.units % 16 == 0 || p.units <= 16) && skinny_mxfp4_xl_lds(p.units, nt, dual) <= 160 * 1024;
}

// K split of the single-kernel decode paths for more than 16 rows: the largest S in {4, 2} (at most max_s) such that
// S channel tiles per workgroup still give at most 256 workgroups in all, every part keeps min_k input channels, and
// the partial tiles fit the workspace; 1 otherwise (also whenever there are enough channel tiles for three per
// workgroup, where the activations are the smaller stream anyway).
static int pick_split(const DecodeParams& p, int64_t M, int64_t K, int mg, int max_s, int64_t min_k, int64_t ws_bytes) {
  if (env_int("TPPX_SKINNY_SPLITK", 1) == 0 || p.n_seg != 1 || M > 64)
    return 1;
  for (int s = max_s; s >= 2; s >>= 1) {
    const int groups = (p.total_tiles + s - 1) / s;
    const int64_t need = (int64_t)s * p.total_tiles * mg * 256 * (int64_t)sizeof(float);
    if (p.total_tiles <= 256 && groups * s <= 256 && K / s >= min_k && need <= ws_bytes)
      return s;
  }
  return 1;
}

static int fill_all(const char* who, const tppx_seg* segs, int n_segs, int n_mult, bool dual,
                    DecodeParams& p) {
  int tiles = 0, groups = 0;
  for (int i = 0; i < n_segs; i++) {
    int rc = fill_seg(who, segs[i], p.seg[i], n_mult);
    if (rc)
      return rc;
    p.seg[i].tile0 = tiles;
    p.seg[i].grp0 = groups;
    tiles += p.seg[i].tiles;
    groups += p.seg[i].tiles; // one tile per workgroup until set_groups() says otherwise
  }
  if (dual) {
    TPPX_REQUIRE(n_segs == 2 && segs[0].N == segs[1].N, TPPX_ESHAPE, "%s: gate and up projections must have equal N", who);
    p.seg[1].tile0 = 0;
    p.seg[1].grp0 = 0;
    tiles = p.seg[0].tiles;
    groups = tiles;
  }
  p.n_seg = n_segs;
  p.total_tiles = tiles;
  p.groups = groups;
  return TPPX_OK;
}

static const int64_t TILED_MIN_M = 65; // more rows than the decode kernels cover in one block row

// More than 64 rows: the LDS-tiled kernels give every workgroup a whole output tile and all of K, so a launch with
// few tiles leaves most of the 256 CUs idle (7B shapes at 256 rows: 43 workgroups), while the decode kernels run one
// block row of 64 rows after the other over the full grid, streaming the weights once per block row.  Pick by a
// cost estimates fitted to measurements on MI355X (us).  MXFP4: a block row of 64 costs about 8 + weight bytes /
// 5.5 TB/s + 0.8 ns per input channel (its activations), a round of 256 x 256 tiles about 14.5 ns per input channel
// (128 x 128: 20; launches small enough for 64 x 128 workgroups: 10 us + 6 ns per input channel).  QINT8 (128 x 256
// tiles, one workgroup per CU) and unquantized bf16 weights (128 x 256 tiles, two workgroups per CU): their own fits
// below.  `wbytes` = weight bytes of
// the whole call, `n_tiles16` = its 16-channel tiles.  TPPX_TILED_MIN_M (when set) restores a plain row threshold.
enum { COST_MXFP4 = 0, COST_QINT8 = 1, COST_BF16 = 2 };
static bool want_tiled(int64_t M, int flags, int64_t K = 0, int64_t n_tiles16 = 0, double wbytes = 0.0,
                       int kind = COST_MXFP4) {
  if (flags & TPPX_FLAG_FORCE_SKINNY)
    return false;
  if (flags & TPPX_FLAG_FORCE_TILED)
    return true;
  if (M < TILED_MIN_M)
    return false;
  const int env_min = env_int("TPPX_TILED_MIN_M", -1);
  if (env_min >= 0)
    return M >= env_min;
  if (K <= 0 || n_tiles16 <= 0 || M > 1024)
    return true;
  const double rows64 = (double)((M + 63) / 64);
  if (kind == COST_QINT8) {
    const int64_t wgs = ((M + 127) / 128) * ((n_tiles16 + 15) / 16);
    // (launches of at most 128 such workgroups run as twice as many of 64 x 256)
    const bool small = wgs <= 128 && env_int("TPPX_TILED_SMALL", 1) != 0;
    const double tiled_us = small ? 8.0 + (double)K * 0.006 : (double)((wgs + 255) / 256) * (10.0 + (double)K * 0.0075);
    const double skinny_us = rows64 * (5.0 + wbytes / 5.5e6 + (double)K * 0.0004);
    return tiled_us <= skinny_us;
  }
  if (kind == COST_BF16 && M >= big_min_rows() && env_int("TPPX_BF16_BIG", 1) != 0) {
    const int64_t wgs = ((M + 127) / 128) * ((n_tiles16 + 15) / 16);
    const int64_t wgs2 = ((M + 63) / 64) * ((n_tiles16 + 7) / 8); // as 64 x 128 workgroups: the form up to 256 of them
    const bool small = wgs2 <= 256 && env_int("TPPX_TILED_SMALL", 1) != 0;
    const double tiled_us = small ? 12.0 + (double)K * 0.0045 : (17.0 + (double)K * 0.009) * std::max(1.0, (double)wgs / 200.0);
    const double skinny_us = rows64 * (6.5 + wbytes / 5.5e6 + (double)K * 0.0006);
    return tiled_us <= skinny_us;
  }
  const bool big = kind == COST_MXFP4 && M >= big_min_rows();
  if (big && env_int("TPPX_TILED_SMALL", 1) != 0) {
    // launches of at most 128 workgroups of 128 x 256 run as four times as many of 64 x 128
    const int64_t wgs1 = ((M + 127) / 128) * ((n_tiles16 + 15) / 16);
    if (wgs1 <= 128) {
      const int64_t wgs2 = ((M + 63) / 64) * ((n_tiles16 + 7) / 8);
      // (up to 128 of them: 26 us at K = 4096, 74 at K = 11008 whatever the rows)
      const double tiled_us = wgs2 <= 128 ? std::max(12.0, (double)K * 0.007 - 2.0)
                                          : 10.0 + (double)K * 0.006 * (wgs2 <= 384 ? 1.05 : 1.25);
      const double skinny_us = rows64 * (6.0 + wbytes / 5.5e6 + (double)K * 0.0007);
      return tiled_us <= skinny_us;
    }
  }
  const int64_t rows = big ? 256 : 128, cols16 = big ? 16 : 8;
  const int64_t wgs = ((M + rows - 1) / rows) * ((n_tiles16 + cols16 - 1) / cols16);
  const double tiled_us = (double)((wgs + 255) / 256) * (double)K * 0.0145 * (big ? 1.0 : 1.4);
  const double skinny_us = rows64 * (8.0 + wbytes / 5.5e6 + (double)K * 0.0008);
  return tiled_us <= skinny_us;
}

static TiledParams tiled_from_seg(const DecodeParams& p, int i) {
  TiledParams t;
  memset(&t, 0, sizeof(t));
  const DecodeSeg& s = p.seg[i];
  t.x = p.x;
  t.xq = p.xq;
  t.sa = p.sa;
  t.qw = s.qw;
  t.sw = s.sw;
  t.bias = s.bias;
  t.post_in = s.post_in;
  t.post_in2 = s.post_in2;
  t.y = s.y;
  t.M = p.M;
  t.N = s.N;
  t.K = p.K;
  t.tiles = s.tiles;
  t.post_op = s.post_op;
  t.post_scale = s.post_scale;
  return t;
}

static int run_mxfp4(const char* who, const void* x, const tppx_seg* segs, int n_segs,
                     int64_t M, int64_t K, int flags, bool dual, void* ws, int64_t ws_bytes,
                     hipStream_t stream, float* row_sumsq = nullptr) {
  int rc = check_common(who, x, M, K, n_segs, flags, ws, ws_bytes);
  if (rc)
    return rc;
  TPPX_REQUIRE(!row_sumsq || (M <= 16 && n_segs == 1 && !dual && ((uintptr_t)row_sumsq & 15) == 0), TPPX_EUNSUPPORTED,
               "%s: row sums of squares are produced for one GEMM of at most 16 rows (M=%ld) into a 16-byte aligned table",
               who, (long)M);
  TPPX_REQUIRE(segs, TPPX_EINVAL, "%s: null segment table", who);
  TPPX_REQUIRE(K > 0 && K % 64 == 0, TPPX_ESHAPE, "%s: K=%ld must be a positive multiple of 64", who, (long)K);
  TPPX_REQUIRE(K % 128 == 0, TPPX_EUNSUPPORTED, "%s: K=%ld is not a multiple of 128 (native MXFP4 tiles span 128 input channels)", who, (long)K);
  DecodeParams p;
  memset(&p, 0, sizeof(p));
  rc = fill_all(who, segs, n_segs, 32, dual, p);
  if (rc)
    return rc;
  p.x = x;
  p.M = (int)M;
  p.K = (int)K;
  p.units = (int)(K / 128);
  p.tpb = 1;
  p.S = 1;
  p.sumsq_out = row_sumsq;
  if (flags & TPPX_FLAG_ACT_FP8) {
    // opt-in, not the reference's arithmetic: activations quantised to MXFP8 (into the workspace), then the
    // block-scaled MFMA kernel on the weights' own codes and scales; any M, but built for prefill shapes
    TPPX_REQUIRE(!row_sumsq, TPPX_EUNSUPPORTED, "%s: row sums of squares are not produced by the FP8-activation kernel", who);
    const int64_t Mp = (M + 63) / 64 * 64, need = Mp * K + Mp * (K / 32);
    TPPX_REQUIRE(ws && ws_bytes >= need, TPPX_EINVAL, "%s: the FP8-activation path needs %ld bytes of workspace for the quantised activations (got %ld)", who, (long)need, (long)ws_bytes);
    uint8_t* xq = (uint8_t*)ws;
    uint8_t* xs = xq + Mp * K;
    rc = check_hip(launch_quant_act_mxfp8(x, M, K, xq, xs, stream), who);
    if (rc)
      return rc;
    TiledParams t[TPPX_MAX_SEGS];
    for (int i = 0; i < n_segs; i++) {
      t[i] = tiled_from_seg(p, i);
      t[i].xq = xq;
      t[i].sa = (const float*)xs;
    }
    if (!dual)
      return check_hip(launch_tiled_mxfp4_fp8_group(t, n_segs, stream), who);
    if (env_int("TPPX_TILED_DUAL_FUSED", 1) != 0) { // both projections per workgroup, silu(gate) * up in the epilogue
      t[0].post_op = t[1].post_op = TPPX_POST_NONE;
      return check_hip(launch_tiled_mxfp4_fp8_group(t, 2, stream, true), who);
    }
    {
      // gate and up as ONE grid when that fills the last round of workgroups better than two launches and the
      // workspace has room for the gate tile behind the quantised activations (as in the bf16-activation path below)
      const int64_t wgs = ((M + 255) / 256) * ((t[0].tiles + 15) / 16);
      const bool fewer_rounds = (2 * wgs + 255) / 256 < 2 * ((wgs + 255) / 256);
      const int64_t park = (need + 255) / 256 * 256;
      if (fewer_rounds && ws_bytes >= park + M * (int64_t)t[0].N * 2 && env_int("TPPX_TILED_DUAL_GROUP", 1) != 0) {
        uint16_t* gate = (uint16_t*)((uint8_t*)ws + park);
        t[0].y = gate;
        t[0].post_op = t[1].post_op = TPPX_POST_NONE;
        rc = check_hip(launch_tiled_mxfp4_fp8_group(t, 2, stream), who);
        if (rc)
          return rc;
        return check_hip(launch_silu_mul(gate, (uint16_t*)segs[1].y, M * (int64_t)t[0].N, stream), who);
      }
    }
    t[0].post_op = TPPX_POST_SILU; // silu(gate), then up * that: the rounding points of the two-GEMM form
    t[1].post_op = TPPX_POST_MUL;
    t[1].post_in = (const uint16_t*)segs[0].y;
    rc = check_hip(launch_tiled_mxfp4_fp8_group(&t[0], 1, stream), who);
    if (rc)
      return rc;
    return check_hip(launch_tiled_mxfp4_fp8_group(&t[1], 1, stream), who);
  }
  if (want_tiled(M, flags, K, dual ? 2 * p.total_tiles : p.total_tiles,
                 (dual ? 2.0 : 1.0) * (double)p.total_tiles * 16.0 * (double)K * (0.5 + 1.0 / 32))) {
    TPPX_REQUIRE(!row_sumsq, TPPX_EUNSUPPORTED, "%s: row sums of squares are not produced by the large-M kernels", who);
    // prefill shapes: one LDS-tiled launch per GEMM of the group; the fused
    // gate/up pair becomes silu(gate) followed by up * gate (same rounding)
    if (!dual && n_segs > 1) {
      TiledParams t[TPPX_MAX_SEGS];
      bool group = true;
      for (int i = 0; i < n_segs; i++) {
        t[i] = tiled_from_seg(p, i);
        group = group && tiled_mxfp4_takes_groups(t[i]);
      }
      if (group) // fused q/k/v: one grid over the channel blocks of all GEMMs
        return check_hip(launch_tiled_mxfp4_group(t, n_segs, stream), who);
    }
    if (dual && env_int("TPPX_TILED_DUAL_FUSED", 1) != 0) {
      // Gate and up in ONE launch whose workgroups own 128 output channels each and compute both projections for
      // them: silu(gate) * up is formed in the epilogue with the reference's rounding points and written once (no
      // parked gate tile, no elementwise pass, no workspace).
      TiledParams t[2] = {tiled_from_seg(p, 0), tiled_from_seg(p, 1)};
      if (tiled_mxfp4_takes_groups(t[0])) {
        t[0].post_op = t[1].post_op = TPPX_POST_NONE;
        return check_hip(launch_tiled_mxfp4_group(t, 2, stream, true), who);
      }
    }
    if (dual) {
      // Gate and up as ONE grid when that fills the last round of workgroups better than two launches (28672
      // channels at 2048 rows: 2 x 3.5 rounds of 256 CUs become 7): the gate GEMM leaves its bf16 tile (bias + dot,
      // the value the reference applies SiLU to) in the workspace, an elementwise pass then forms
      // silu(gate) * up with the reference's rounding points.  Needs M * N bf16 of workspace.
      TiledParams t[2] = {tiled_from_seg(p, 0), tiled_from_seg(p, 1)};
      const int64_t wgs = ((M + 255) / 256) * ((t[0].tiles + 15) / 16);
      const bool fewer_rounds = (2 * wgs + 255) / 256 < 2 * ((wgs + 255) / 256);
      if (fewer_rounds && ws && ws_bytes >= M * (int64_t)t[0].N * 2 && tiled_mxfp4_takes_groups(t[0]) &&
          env_int("TPPX_TILED_DUAL_GROUP", 1) != 0) {
        t[0].y = (uint16_t*)ws;
        t[0].post_op = t[1].post_op = TPPX_POST_NONE;
        rc = check_hip(launch_tiled_mxfp4_group(t, 2, stream), who);
        if (rc)
          return rc;
        return check_hip(launch_silu_mul((const uint16_t*)ws, (uint16_t*)segs[1].y, M * (int64_t)t[0].N, stream), who);
      }
    }
    for (int i = 0; i < n_segs; i++) {
      TiledParams t = tiled_from_seg(p, i);
      if (dual) {
        t.post_op = i == 0 ? TPPX_POST_SILU : TPPX_POST_MUL;
        t.post_in = i == 0 ? nullptr : (const uint16_t*)segs[0].y;
      }
      rc = check_hip(launch_tiled_mxfp4(t, stream), who);
      if (rc)
        return rc;
    }
    return TPPX_OK;
  }
  int nt_xl = 1;
  if (M <= 16 && env_int("TPPX_MXFP4_XL", 1) == 1 && plan_xl(p, dual, &nt_xl)) {
    TPPX_REQUIRE(!row_sumsq || p.groups <= 256, TPPX_EUNSUPPORTED, "%s: N=%ld needs more than 256 workgroups; the table of row sums has 256 slots", who, (long)segs[0].N);
    return check_hip(launch_skinny_mxfp4_xl(p, nt_xl, dual, stream), who);
  }
  if (M <= 16) {
    // K that the LDS-staged kernel above cannot hold.  Up to 4 rows (and K up to 16384): the same staging with only
    // the 4 rows kept; otherwise the tile-by-tile kernel with one row group (measured at K = 11008, N = 4096:
    // 1 row 8.8 -> 7.7 us, 16 rows 14.7 -> 11.7 us against operands read straight from global memory).
    const bool x4 = M <= 4 && p.units <= 128;
    // 5..16 rows, few channel tiles (N = 4096 at K = 11008, the Llama down-projection): the LDS-staged kernel with K
    // in 4 parts across workgroups that own 4 channel tiles each -- the same number of workgroups, every part short
    // enough for the staging, 16 KiB of partial sums per workgroup through the workspace.
    if (!x4 && !dual && n_segs == 1 && env_int("TPPX_MXFP4_XL_SPLIT", 1) == 1 && p.total_tiles % 4 == 0 &&
        p.total_tiles <= 256 && (p.units + 3) / 4 <= 32 && p.units >= 64 &&
        ws && ws_bytes >= (int64_t)4 * p.total_tiles * 256 * (int64_t)sizeof(float)) {
      set_groups(p, 4, false);
      p.S = 4;
      p.part = (float*)ws;
      return check_hip(launch_skinny_mxfp4_xl(p, 4, false, stream), who);
    }
    int nt = 1;
    for (; nt < 3; nt++) {
      set_groups(p, nt, dual);
      if (p.groups <= 256)
        break;
    }
    set_groups(p, nt, dual);
    TPPX_REQUIRE(!row_sumsq || p.groups <= 256, TPPX_EUNSUPPORTED, "%s: N=%ld needs more than 256 workgroups; the table of row sums has 256 slots", who, (long)segs[0].N);
    return check_hip(x4 ? launch_skinny_mxfp4_x4(p, nt, dual, stream) : launch_skinny_mxfp4_mg(p, 1, nt, dual, stream), who);
  }
  {
    // 17..64 rows: several MFMA row groups per workgroup, activations streamed through wave-private LDS
    const int mg = M <= 32 ? 2 : 4;
    // Few channel tiles and a long K: every workgroup would pull all of the activations (M x K) through its CU.
    // Split K across S workgroups that own S times the channel tiles each: the same number of workgroups, 1/S of
    // the activations per CU, fp32 partial tiles through the workspace, summed by whichever of the S workgroups
    // finishes last (measured: 26 -> 21 us for 64 rows at K = 11008 / N = 4096; no gain for 32 rows).
    // 33..64 rows, a single GEMM with few channel tiles and a long K: four tiles x four K parts per workgroup with
    // the activations of a K tile staged ONCE per workgroup, K in four slices across workgroups
    if (!dual && mg == 4 && n_segs == 1 && !row_sumsq && env_int("TPPX_MXFP4_NK", 1) != 0) {
      const int groups = (p.total_tiles + 3) / 4;
      if (groups * 4 <= 256 && groups * 4 >= 96 && p.units >= 64 && (p.units + 3) / 4 <= 32 &&
          (int64_t)4 * groups * 4 * mg * 256 * (int64_t)sizeof(float) * ((M + 63) / 64) <= ws_bytes) {
        p.S = 4;
        p.part = (float*)ws;
        return check_hip(launch_skinny_mxfp4_nk(p, stream), who);
      }
    }
    const int S = (dual || mg != 4) ? 1 : pick_split(p, M, K, mg, 4, 2048, ws_bytes);
    int nt = S;
    if (S == 1) {
      for (; nt < 3; nt++) {
        set_groups(p, nt, dual);
        if (p.groups <= 256)
          break;
      }
    }
    set_groups(p, nt, dual);
    p.S = S;
    p.part = (float*)ws;
    return check_hip(launch_skinny_mxfp4_mg(p, mg, nt, dual, stream), who);
  }
}

static int run_qint8(const char* who, const void* x, void* xq, void* sa, const tppx_seg* segs,
                     int n_segs, int64_t M, int64_t K, int64_t qbs, int flags, void* ws,
                     int64_t ws_bytes, hipStream_t stream) {
  // x == NULL: xq / sa already hold quantized activations (the reference's
  // pre-quantized input case, src/csrc/fused_gemm.h:1244-1246)
  int rc = check_common(who, x ? x : xq, M, K, n_segs, flags, ws, ws_bytes);
  if (rc)
    return rc;
  TPPX_REQUIRE(segs, TPPX_EINVAL, "%s: null segment table", who);
  TPPX_REQUIRE(xq && sa, TPPX_EINVAL, "%s: null activation-quantization buffers", who);
  TPPX_REQUIRE(aligned16(xq), TPPX_EINVAL, "%s: scratch pointer not 16-byte aligned", who);
  TPPX_REQUIRE(K > 0 && K % 64 == 0, TPPX_ESHAPE, "%s: K=%ld must be a positive multiple of 64", who, (long)K);
  TPPX_REQUIRE(qbs > 0 && qbs % 64 == 0 && K % qbs == 0, TPPX_ESHAPE, "%s: block size mismatch (qbs=%ld, K=%ld)", who, (long)qbs, (long)K);
  DecodeParams p;
  memset(&p, 0, sizeof(p));
  rc = fill_all(who, segs, n_segs, 16, false, p);
  if (rc)
    return rc;
  p.x = x;
  p.xq = xq;
  p.sa = (const float*)sa;
  p.M = (int)M;
  p.K = (int)K;
  p.tpb = (int)(qbs / 64);
  p.nblk = (int)(K / qbs);
  // what is dealt to waves and K parts: runs of 256 input channels inside larger blocks (per-output-channel scales,
  // qbs = K, keep every wave busy that way), whole blocks below 256, single tiles for other block sizes
  p.deal = p.tpb % 4 == 0 ? 4 : (p.tpb < 4 ? p.tpb : 1);
  p.units = (int)(K / (64 * p.deal));
  p.spb_magic = (p.deal == 4 && p.tpb > 4) ? (unsigned int)((((uint64_t)1 << 32) + (uint64_t)(p.tpb / 4) - 1) / (uint64_t)(p.tpb / 4)) : 0u;
  const bool reuse = (flags & TPPX_FLAG_XQ_REUSE) != 0; // xq / sa still hold this x, quantized by an earlier call
  if (qbs % 128 == 0 && want_tiled(M, flags, K, p.total_tiles, (double)p.total_tiles * 16.0 * (double)K, COST_QINT8)) {
    if (x && !reuse) {
      rc = check_hip(launch_quant_act_int8(x, M, K, qbs, xq, sa, 0, stream), who);
      if (rc)
        return rc;
    }
    if (n_segs > 1) { // fused q/k/v: one grid over the channel blocks of all GEMMs when the large-M kernel takes them
      TiledParams t[TPPX_MAX_SEGS];
      bool group = true;
      for (int i = 0; i < n_segs; i++) {
        t[i] = tiled_from_seg(p, i);
        t[i].qbs = (int)qbs;
        group = group && tiled_qint8_takes_groups(t[i]);
      }
      if (group)
        return check_hip(launch_tiled_qint8_group(t, n_segs, stream), who);
    }
    for (int i = 0; i < n_segs; i++) {
      TiledParams t = tiled_from_seg(p, i);
      t.qbs = (int)qbs;
      rc = check_hip(launch_tiled_qint8(t, stream), who);
      if (rc)
        return rc;
    }
    return TPPX_OK;
  }
  p.S = 1;
  SkinnyPlan sp = plan_skinny(M, p.total_tiles, p.units, p.tpb, p.deal, x != nullptr && qbs % 256 == 0);
  // 33..64 rows, few channel tiles and a long K: every workgroup would pull all of the int8 activations (M x K)
  // through its CU.  Two K parts of two channel tiles each halve that (measured at N = 4096, 64 rows: K = 11008
  // 20.4 -> 18.5 us, K = 14336 25.1 -> 21.6 us; K = 8192 and shorter lose to the extra pass over the partial sums).
  // The same shapes with bf16 activations at hand (so that they are quantised into operand order): four channel
  // tiles x four K parts per workgroup with the operands shared through LDS, K in 4 (or 2) slices across workgroups.
  // (measured at N = 4096: 64 rows K = 8192 19.2 -> 14.6 us, K = 11008 18.9 -> 17.1, K = 14336 21.7 -> 20.9; 32 rows
  // K = 11008 15.3 -> 14.1 and no gain at K = 8192, so 17..32 rows take it from K = 10240 on)
  if (x && sp.mg >= env_int("TPPX_QINT8_NK_MIN_MG", 2) && (sp.mg == 4 || p.units >= 40) && !sp.fused_quant && p.n_seg == 1 &&
      p.deal == 4 && M <= 64 && env_int("TPPX_QINT8_NK", 1) != 0) {
    const int groups = (p.total_tiles + 3) / 4;
    // four slices or nothing: with two, half the chip streams the weights (measured 25.8 us against 18.9 unsplit)
    int S = 0;
    if (groups * 4 <= 256 && groups * 4 >= 96 && p.units >= 32 && (p.units + 3) / 4 <= 32 &&
        (int64_t)4 * groups * 4 * sp.mg * 256 * (int64_t)sizeof(float) * sp.grid_y <= ws_bytes)
      S = 4;
    if (S > 0) {
      p.S = S;
      p.part = (float*)ws;
      p.mt = sp.grid_y * sp.mg;
      rc = reuse ? TPPX_OK : check_hip(launch_quant_act_int8(x, M, K, qbs, xq, sa, p.mt, stream), who);
      if (rc)
        return rc;
      return check_hip(launch_skinny_qint8_nk(p, sp.mg, stream), who);
    }
  }
  if (sp.mg == 4 && !sp.fused_quant && pick_split(p, M, K, sp.mg, 2, 5504, ws_bytes) == 2) {
    p.S = 2;
    p.part = (float*)ws;
    sp.ntw = 2;
    sp.waves = 8;
    sp.max_units = skinny_qint8_blocks_per_wave(((p.units + 1) / 2 + 7) / 8, p.tpb, p.deal, p.nblk);
  }
  if (x && !sp.fused_quant) {
    // quantise straight into MFMA operand order: the GEMM then reads one
    // contiguous 1 KiB per operand instead of 16 rows x 64 B
    p.mt = sp.grid_y * sp.mg;
    rc = reuse ? TPPX_OK : check_hip(launch_quant_act_int8(x, M, K, qbs, xq, sa, p.mt, stream), who);
    if (rc)
      return rc;
  }
  set_groups(p, sp.ntw, false);
  return check_hip(launch_skinny_qint8(p, sp, stream), who);
}

// LDS-staged MXFP4 decode kernel (M <= 16) with an optional RMSNorm in front
static int run_mxfp4_xl(const char* who, const void* x, const void* gamma, float eps, const tppx_seg* segs,
                        int n_segs, int64_t M, int64_t K, int flags, bool dual, hipStream_t stream,
                        const float* row_sumsq = nullptr, int64_t split1 = 0, int64_t split2 = 0) {
  int rc = check_common(who, x, M, K, n_segs, flags, nullptr, 0);
  if (rc)
    return rc;
  TPPX_REQUIRE(segs, TPPX_EINVAL, "%s: null segment table", who);
  TPPX_REQUIRE(K > 0 && K % 128 == 0, TPPX_ESHAPE, "%s: K=%ld must be a positive multiple of 128", who, (long)K);
  TPPX_REQUIRE(M <= 16, TPPX_EUNSUPPORTED, "%s: more than 16 rows (M=%ld): run the normalisation and the GEMM separately", who, (long)M);
  TPPX_REQUIRE(gamma == nullptr || aligned16(gamma), TPPX_EINVAL, "%s: gamma not 16-byte aligned", who);
  DecodeParams p;
  memset(&p, 0, sizeof(p));
  rc = fill_all(who, segs, n_segs, 32, dual, p);
  if (rc)
    return rc;
  if (split1 > 0) {
    TPPX_REQUIRE(n_segs == 1 && !dual && split1 % 16 == 0 && split2 % 16 == 0 && split1 <= split2 && split2 <= segs[0].N,
                 TPPX_ESHAPE, "%s: output split %ld / %ld must be multiples of 16 within N=%ld", who, (long)split1, (long)split2, (long)segs[0].N);
    TPPX_REQUIRE(M * segs[0].N < ((int64_t)1 << 31), TPPX_ESHAPE, "%s: M*N exceeds 2^31", who);
    p.seg[0].split1 = (int)split1;
    p.seg[0].split2 = (int)split2;
  }
  p.x = x;
  p.M = (int)M;
  p.K = (int)K;
  p.units = (int)(K / 128);
  p.tpb = 1;
  p.S = 1;
  p.norm_gamma = (const float*)gamma;
  p.norm_eps = eps;
  TPPX_REQUIRE(!row_sumsq || (gamma && ((uintptr_t)row_sumsq & 15) == 0), TPPX_EINVAL,
               "%s: the table of row sums needs gamma and 16-byte alignment", who);
  p.sumsq_in = row_sumsq;
  int nt = 1;
  TPPX_REQUIRE(plan_xl(p, dual, &nt), TPPX_EUNSUPPORTED,
               "%s: K=%ld does not split into 16 slices of 128 or 256 input channels (or fewer than 16 tiles) that fit the LDS staging; run the steps separately", who, (long)K);
  return check_hip(launch_skinny_mxfp4_xl(p, nt, dual, stream), who);
}

} // namespace tppx

using namespace tppx;

extern "C" int tppx_norm_multi_linear_mxfp4(const void* x, const void* gamma, float eps, const tppx_seg* segs,
                                            int n_segs, int64_t M, int64_t K, int flags, tppx_stream_t stream) {
  return run_mxfp4_xl("tppx_norm_multi_linear_mxfp4", x, gamma, eps, segs, n_segs, M, K, flags, false, (hipStream_t)stream);
}

extern "C" int tppx_norm_swiglu_mxfp4(const void* x, const void* gamma, float eps, const void* qw_gate,
                                      const void* sw_gate, const void* bias_gate, const void* qw_up,
                                      const void* sw_up, const void* bias_up, void* y, int64_t M, int64_t N,
                                      int64_t K, int flags, tppx_stream_t stream) {
  tppx_seg s[2] = {{qw_gate, sw_gate, bias_gate, nullptr, nullptr, y, N, TPPX_POST_NONE, 1.0f},
                   {qw_up, sw_up, bias_up, nullptr, nullptr, y, N, TPPX_POST_NONE, 1.0f}};
  return run_mxfp4_xl("tppx_norm_swiglu_mxfp4", x, gamma, eps, s, 2, M, K, flags, true, (hipStream_t)stream);
}

extern "C" int tppx_linear_mxfp4_rowsq(const void* x, const void* qw, const void* sw, const void* bias,
                                       const void* post_in, const void* post_in2, void* y, int64_t M, int64_t N,
                                       int64_t K, int post_op, float post_scale, int flags, void* ws,
                                       int64_t ws_bytes, void* row_sumsq, tppx_stream_t stream) {
  const char* who = "tppx_linear_mxfp4_rowsq";
  TPPX_REQUIRE(row_sumsq, TPPX_EINVAL, "%s: null table of row sums", who);
  tppx_seg s = {qw, sw, bias, post_in, post_in2, y, N, post_op, post_scale};
  return run_mxfp4(who, x, &s, 1, M, K, flags, false, ws, ws_bytes, (hipStream_t)stream, (float*)row_sumsq);
}

extern "C" int tppx_normsq_multi_linear_mxfp4(const void* x, const void* row_sumsq, const void* gamma, float eps,
                                              const tppx_seg* segs, int n_segs, int64_t M, int64_t K, int flags,
                                              tppx_stream_t stream) {
  const char* who = "tppx_normsq_multi_linear_mxfp4";
  TPPX_REQUIRE(row_sumsq && gamma, TPPX_EINVAL, "%s: null table of row sums or gamma", who);
  return run_mxfp4_xl(who, x, gamma, eps, segs, n_segs, M, K, flags, false, (hipStream_t)stream, (const float*)row_sumsq);
}

extern "C" int tppx_qkv_linear_mxfp4(const void* x, const void* row_sumsq, const void* gamma, float eps, const void* qw,
                                     const void* sw, const void* bias, void* y, int64_t M, int64_t N, int64_t K,
                                     int64_t n1, int64_t n2, int flags, tppx_stream_t stream) {
  const char* who = "tppx_qkv_linear_mxfp4";
  TPPX_REQUIRE(n1 > 0 && n2 >= n1, TPPX_ESHAPE, "%s: output widths must be positive", who);
  TPPX_REQUIRE(!row_sumsq || gamma, TPPX_EINVAL, "%s: row sums without gamma", who);
  tppx_seg s = {qw, sw, bias, nullptr, nullptr, y, N, TPPX_POST_NONE, 1.0f};
  return run_mxfp4_xl(who, x, gamma, eps, &s, 1, M, K, flags, false, (hipStream_t)stream, (const float*)row_sumsq, n1, n2);
}

extern "C" int tppx_normsq_swiglu_mxfp4(const void* x, const void* row_sumsq, const void* gamma, float eps,
                                        const void* qw_gate, const void* sw_gate, const void* bias_gate,
                                        const void* qw_up, const void* sw_up, const void* bias_up, void* y,
                                        int64_t M, int64_t N, int64_t K, int flags, tppx_stream_t stream) {
  const char* who = "tppx_normsq_swiglu_mxfp4";
  TPPX_REQUIRE(row_sumsq && gamma, TPPX_EINVAL, "%s: null table of row sums or gamma", who);
  tppx_seg s[2] = {{qw_gate, sw_gate, bias_gate, nullptr, nullptr, y, N, TPPX_POST_NONE, 1.0f},
                   {qw_up, sw_up, bias_up, nullptr, nullptr, y, N, TPPX_POST_NONE, 1.0f}};
  return run_mxfp4_xl(who, x, gamma, eps, s, 2, M, K, flags, true, (hipStream_t)stream, (const float*)row_sumsq);
}

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
                                 float post_scale, int flags, void* ws,
                                 int64_t ws_bytes, tppx_stream_t stream) {
  tppx_seg s = {qw, sw, bias, post_in, post_in2, y, N, post_op, post_scale};
  return run_mxfp4("tppx_linear_mxfp4", x, &s, 1, M, K, flags, false, ws, ws_bytes, (hipStream_t)stream);
}

extern "C" int tppx_linear_bf16(const void* x, const void* w, const void* bias, const void* post_in,
                                const void* post_in2, void* y, int64_t M, int64_t N, int64_t K, int post_op,
                                float post_scale, int flags, tppx_stream_t stream) {
  const char* who = "tppx_linear_bf16";
  int rc = check_common(who, x, M, K, 1, flags, nullptr, 0);
  if (rc)
    return rc;
  TPPX_REQUIRE(K > 0 && K % 128 == 0, TPPX_ESHAPE, "%s: K=%ld must be a positive multiple of 128 (native bf16 tiles span 128 input channels)", who, (long)K);
  TPPX_REQUIRE(!(flags & TPPX_FLAG_ACT_FP8), TPPX_EUNSUPPORTED, "%s: FP8 activations are built for MXFP4 weights only", who);
  TPPX_REQUIRE(M * N < ((int64_t)1 << 31), TPPX_ESHAPE, "%s: M*N=%ld outputs exceed 2^31", who, (long)(M * N));
  tppx_seg s = {w, w, bias, post_in, post_in2, y, N, post_op, post_scale}; // no scales: the slot repeats the weight
  DecodeParams p;
  memset(&p, 0, sizeof(p));
  rc = fill_all(who, &s, 1, 16, false, p);
  if (rc)
    return rc;
  p.x = x;
  p.M = (int)M;
  p.K = (int)K;
  p.units = (int)(K / 128);
  p.tpb = 1;
  p.S = 1;
  // more than 64 rows: the LDS-tiled kernel once it is the cheaper one (the estimate of the quantized formats with the
  // weight's real bytes: the row-group kernel streams the whole weight once per 64 rows)
  if (want_tiled(M, flags, K, p.total_tiles, (double)N * (double)K * 2.0, COST_BF16)) {
    TPPX_REQUIRE(aligned16(w), TPPX_EINVAL, "%s: weight not 16-byte aligned", who);
    return check_hip(launch_tiled_bf16(tiled_from_seg(p, 0), (hipStream_t)stream), who);
  }
  const int mg = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  const int nt = p.total_tiles > 512 ? 2 : 1; // two channel tiles per workgroup once one each still leaves two rounds
  set_groups(p, nt, false);
  return check_hip(launch_skinny_bf16(p, mg, nt, (hipStream_t)stream), who);
}

extern "C" int tppx_multi_linear_mxfp4(const void* x, const tppx_seg* segs,
                                       int n_segs, int64_t M, int64_t K,
                                       int flags, void* ws, int64_t ws_bytes,
                                       tppx_stream_t stream) {
  return run_mxfp4("tppx_multi_linear_mxfp4", x, segs, n_segs, M, K, flags, false, ws, ws_bytes, (hipStream_t)stream);
}

extern "C" int tppx_swiglu_mxfp4(const void* x, const void* qw_gate,
                                 const void* sw_gate, const void* bias_gate,
                                 const void* qw_up, const void* sw_up,
                                 const void* bias_up, void* y, int64_t M,
                                 int64_t N, int64_t K, int flags, void* ws,
                                 int64_t ws_bytes, tppx_stream_t stream) {
  tppx_seg s[2] = {{qw_gate, sw_gate, bias_gate, nullptr, nullptr, y, N, TPPX_POST_NONE, 1.0f},
                   {qw_up, sw_up, bias_up, nullptr, nullptr, y, N, TPPX_POST_NONE, 1.0f}};
  return run_mxfp4("tppx_swiglu_mxfp4", x, s, 2, M, K, flags, true, ws, ws_bytes, (hipStream_t)stream);
}

extern "C" int tppx_linear_qint8(const void* x, void* xq, void* sa,
                                 const void* qw, const void* sw,
                                 const void* bias, const void* post_in,
                                 const void* post_in2, void* y, int64_t M,
                                 int64_t N, int64_t K, int64_t qbs, int post_op,
                                 float post_scale, int flags, void* ws,
                                 int64_t ws_bytes, tppx_stream_t stream) {
  tppx_seg s = {qw, sw, bias, post_in, post_in2, y, N, post_op, post_scale};
  return run_qint8("tppx_linear_qint8", x, xq, sa, &s, 1, M, K, qbs, flags, ws, ws_bytes, (hipStream_t)stream);
}

extern "C" int tppx_multi_linear_qint8(const void* x, void* xq, void* sa,
                                       const tppx_seg* segs, int n_segs,
                                       int64_t M, int64_t K, int64_t qbs,
                                       int flags, void* ws, int64_t ws_bytes,
                                       tppx_stream_t stream) {
  return run_qint8("tppx_multi_linear_qint8", x, xq, sa, segs, n_segs, M, K, qbs, flags, ws, ws_bytes, (hipStream_t)stream);
}

// ---- the entry point that allocates nothing ----------------------------------
// Everything tppx_linear_qint8 takes from the caller as scratch -- the quantised activations xq, their scales sa and
// the K-split workspace -- lives in one file-scope device array instead.  The array's name is only a host-side
// handle: its device address is looked up once per device (hipGetSymbolAddress with that device current) and only
// that address is ever handed to kernels.
constexpr int64_t NA_MAX_M = 64, NA_MAX_K = 32768;
constexpr size_t NA_XQ_BYTES = (size_t)NA_MAX_M * NA_MAX_K;                        // int8 rows, 2 MiB
constexpr size_t NA_SA_BYTES = (size_t)NA_MAX_M * (NA_MAX_K / 64) * sizeof(float); // one scale per 64 channels at most
constexpr size_t NA_WS_BYTES = (size_t)4 * 256 * 4 * 256 * sizeof(float);          // 4 K slices x 256 tiles x 64 rows
static __device__ __align__(256) unsigned char scratch[NA_XQ_BYTES + NA_SA_BYTES + NA_WS_BYTES];

static int scratch_of_current_device(const char* who, unsigned char** out) {
  static std::mutex mu;
  static std::map<int, unsigned char*> per_device;
  int dev = 0;
  int rc = check_hip(hipGetDevice(&dev), who);
  if (rc)
    return rc;
  std::lock_guard<std::mutex> lock(mu);
  auto it = per_device.find(dev);
  if (it == per_device.end()) {
    void* ptr = nullptr;
    rc = check_hip(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), who);
    if (rc)
      return rc;
    TPPX_REQUIRE(ptr && (reinterpret_cast<uintptr_t>(ptr) & 255u) == 0, TPPX_EHIP, "%s: bad address of the static scratch", who);
    it = per_device.emplace(dev, (unsigned char*)ptr).first;
  }
  *out = it->second;
  return TPPX_OK;
}

extern "C" int tppx_linear_qint8_noalloc(const void* x, const void* qw, const void* sw, const void* bias,
                                         const void* post_in, const void* post_in2, void* y, int64_t M, int64_t N,
                                         int64_t K, int64_t qbs, int post_op, float post_scale, int flags,
                                         tppx_stream_t stream) {
  const char* who = "tppx_linear_qint8_noalloc";
  TPPX_REQUIRE(x, TPPX_EINVAL, "%s: null activation pointer (pre-quantized input needs no scratch: call tppx_linear_qint8)", who);
  TPPX_REQUIRE(M > 0 && M <= NA_MAX_M, TPPX_ESHAPE, "%s: M=%ld outside 1..%ld (the static scratch holds %ld quantised rows)", who, (long)M, (long)NA_MAX_M, (long)NA_MAX_M);
  TPPX_REQUIRE(K > 0 && K <= NA_MAX_K, TPPX_ESHAPE, "%s: K=%ld outside 1..%ld (the static scratch holds rows of %ld channels)", who, (long)K, (long)NA_MAX_K, (long)NA_MAX_K);
  TPPX_REQUIRE((flags & ~TPPX_FLAG_FORCE_SKINNY) == 0, TPPX_EINVAL, "%s: only TPPX_FLAG_FORCE_SKINNY is accepted here (flags 0x%x)", who, flags);
  // the remaining checks of tppx_linear_qint8, before the first HIP call, on placeholder scratch addresses
  void* a = reinterpret_cast<void*>(uintptr_t(1) << 20);
  tppx_seg s = {qw, sw, bias, post_in, post_in2, y, N, post_op, post_scale};
  {
    std::string text;
    g_plan = &text;
    const int rc = run_qint8(who, x, a, a, &s, 1, M, K, qbs, flags, a, (int64_t)NA_WS_BYTES, nullptr);
    g_plan = nullptr;
    if (rc)
      return rc;
  }
  unsigned char* base = nullptr;
  int rc = scratch_of_current_device(who, &base);
  if (rc)
    return rc;
  return run_qint8(who, x, base, base + NA_XQ_BYTES, &s, 1, M, K, qbs, flags, base + NA_XQ_BYTES + NA_SA_BYTES,
                   (int64_t)NA_WS_BYTES, (hipStream_t)stream);
}

extern "C" int tppx_linear_qintx(const void* x, void* xq, void* sa, const void* qw_packed, const void* sw,
                                 const void* bias, const void* post_in, const void* post_in2, void* y, int64_t M,
                                 int64_t N, int64_t K, int bits, int post_op, float post_scale, int flags,
                                 tppx_stream_t stream) {
  const char* who = "tppx_linear_qintx";
  int rc = check_common(who, x, M, K, 1, 0, nullptr, 0);
  if (rc)
    return rc;
  TPPX_REQUIRE(bits == 4 || bits == 2, TPPX_EINVAL, "%s: %d-bit codes are not built (4 or 2)", who, bits);
  TPPX_REQUIRE((flags & ~TPPX_FLAG_XQ_REUSE) == 0, TPPX_EINVAL, "%s: flags 0x%x not taken here (TPPX_FLAG_XQ_REUSE only)", who, flags);
  TPPX_REQUIRE(K > 0 && K % 256 == 0, TPPX_ESHAPE, "%s: K=%ld must be a positive multiple of the 256-wide scale block", who, (long)K);
  tppx_seg s = {qw_packed, sw, bias, post_in, post_in2, y, N, post_op, post_scale};
  DecodeParams p;
  memset(&p, 0, sizeof(p));
  rc = fill_all(who, &s, 1, 16, false, p);
  if (rc)
    return rc;
  p.x = x;
  p.M = (int)M;
  p.K = (int)K;
  p.tpb = 4;
  p.nblk = (int)(K / 256);
  p.deal = 4;
  p.units = p.nblk;
  p.spb_magic = 0;
  p.S = 1;
  p.wbits = bits;
  SkinnyPlan sp = plan_skinny(M, p.total_tiles, p.units, p.tpb, p.deal, true);
  if (sp.fused_quant) { // up to 16 rows whose quantised form fits the LDS: one launch
    set_groups(p, sp.ntw, false);
    return check_hip(launch_skinny_qint8(p, sp, (hipStream_t)stream), who);
  }
  // more rows: the activation quantiser in front (operand-order int8 rows), then the 17..64-row kernel on block
  // rows of 32 or 64
  TPPX_REQUIRE(M > 16, TPPX_EUNSUPPORTED, "%s: M=%ld rows of K=%ld channels do not fit the in-kernel quantisation's LDS; run the call on the expanded int8 tiles", who, (long)M, (long)K);
  TPPX_REQUIRE(xq && sa, TPPX_EINVAL, "%s: more than 16 rows need the xq / sa scratch of tppx_linear_qint8", who);
  TPPX_REQUIRE(aligned16(xq) && aligned16(sa), TPPX_EINVAL, "%s: scratch not 16-byte aligned", who);
  int ntw = 1;
  for (; ntw < 3; ntw++)
    if ((p.total_tiles + ntw - 1) / ntw <= 256)
      break;
  set_groups(p, ntw, false);
  p.xq = xq;
  p.sa = (const float*)sa;
  p.mt = sp.grid_y * sp.mg;
  if (!(flags & TPPX_FLAG_XQ_REUSE)) {
    rc = check_hip(launch_quant_act_int8(x, M, K, 256, xq, sa, p.mt, (hipStream_t)stream), who);
    if (rc)
      return rc;
  }
  return check_hip(launch_skinny_qintx(p, sp.mg, ntw, (hipStream_t)stream), who);
}

extern "C" int tppx_linear_mxfp4_int8_rows(const void* x, const void* q_nat, const void* s_nat, const void* bias,
                                           const void* post_in, const void* post_in2, void* y, int64_t M, int64_t N,
                                           int64_t K, int post_op, float post_scale, tppx_stream_t stream) {
  const char* who = "tppx_linear_mxfp4_int8_rows";
  int rc = check_common(who, x, M, K, 1, 0, nullptr, 0);
  if (rc)
    return rc;
  TPPX_REQUIRE(K > 0 && K % 128 == 0, TPPX_ESHAPE, "%s: K=%ld must be a positive multiple of 128", who, (long)K);
  tppx_seg s = {q_nat, s_nat, bias, post_in, post_in2, y, N, post_op, post_scale};
  DecodeParams p;
  memset(&p, 0, sizeof(p));
  rc = fill_all(who, &s, 1, 16, false, p);
  if (rc)
    return rc;
  int ntw = 1;
  TPPX_REQUIRE(skinny_w4a8_fits(M, p.total_tiles, (int)(K / 128), &ntw), TPPX_EUNSUPPORTED,
               "%s: M=%ld rows of K=%ld channels are not a decode shape of this kernel (at most 16 rows whose int8 form fits the LDS); quantize the activations and call tppx_linear_mxfp4_int8", who, (long)M, (long)K);
  p.x = x;
  p.M = (int)M;
  p.K = (int)K;
  p.units = (int)(K / 128);
  p.tpb = 1;
  p.S = 1;
  set_groups(p, ntw, false);
  return check_hip(launch_skinny_w4a8(p, ntw, (hipStream_t)stream), who);
}

extern "C" void tppx_reload_env(void) {
  std::lock_guard<std::mutex> lock(g_env_mu);
  g_env_kept.clear();
}

// ---- launch plans -----------------------------------------------------------
static int emit_plan(const char* who, int rc, std::string& text, char* buf, int64_t buf_len) {
  g_plan = nullptr;
  if (rc)
    return rc;
  TPPX_REQUIRE(buf && buf_len > 0, TPPX_EINVAL, "%s: null or empty text buffer", who);
  snprintf(buf, (size_t)buf_len, "%s", text.c_str());
  return TPPX_OK;
}

extern "C" int tppx_plan_linear_mxfp4(int64_t M, int64_t N, int64_t K, int flags, int64_t ws_bytes, char* buf,
                                      int64_t buf_len) {
  // placeholder addresses: validated for alignment, never dereferenced
  void* a = reinterpret_cast<void*>(uintptr_t(1) << 20);
  std::string text;
  g_plan = &text;
  tppx_seg s = {a, a, nullptr, nullptr, nullptr, a, N, TPPX_POST_NONE, 1.0f};
  int rc = run_mxfp4("tppx_plan_linear_mxfp4", a, &s, 1, M, K, flags, false, ws_bytes > 0 ? a : nullptr, ws_bytes, nullptr);
  return emit_plan("tppx_plan_linear_mxfp4", rc, text, buf, buf_len);
}

extern "C" int tppx_plan_linear_qint8(int64_t M, int64_t N, int64_t K, int64_t qbs, int x_given, int flags,
                                      int64_t ws_bytes, char* buf, int64_t buf_len) {
  void* a = reinterpret_cast<void*>(uintptr_t(1) << 20);
  std::string text;
  g_plan = &text;
  tppx_seg s = {a, a, nullptr, nullptr, nullptr, a, N, TPPX_POST_NONE, 1.0f};
  int rc = run_qint8("tppx_plan_linear_qint8", x_given ? a : nullptr, a, a, &s, 1, M, K, qbs, flags,
                     ws_bytes > 0 ? a : nullptr, ws_bytes, nullptr);
  return emit_plan("tppx_plan_linear_qint8", rc, text, buf, buf_len);
}

// the same for a fused group (q/k/v: dual = 0; the gate/up pair of tppx_swiglu_mxfp4: dual = 1, two equal Ns)
extern "C" int tppx_plan_multi_linear_mxfp4(const int64_t* Ns, int n_segs, int64_t M, int64_t K, int dual, int flags,
                                            int64_t ws_bytes, char* buf, int64_t buf_len) {
  const char* who = "tppx_plan_multi_linear_mxfp4";
  TPPX_REQUIRE(Ns && n_segs >= 1 && n_segs <= TPPX_MAX_SEGS && (!dual || n_segs == 2), TPPX_EINVAL,
               "%s: bad segment list", who);
  void* a = reinterpret_cast<void*>(uintptr_t(1) << 20);
  tppx_seg s[TPPX_MAX_SEGS];
  for (int i = 0; i < n_segs; i++)
    s[i] = {a, a, nullptr, nullptr, nullptr, a, Ns[i], TPPX_POST_NONE, 1.0f};
  std::string text;
  g_plan = &text;
  int rc = run_mxfp4(who, a, s, n_segs, M, K, flags, dual != 0, ws_bytes > 0 ? a : nullptr, ws_bytes, nullptr);
  return emit_plan(who, rc, text, buf, buf_len);
}

extern "C" int tppx_plan_multi_linear_qint8(const int64_t* Ns, int n_segs, int64_t M, int64_t K, int64_t qbs,
                                            int x_given, int flags, int64_t ws_bytes, char* buf, int64_t buf_len) {
  const char* who = "tppx_plan_multi_linear_qint8";
  TPPX_REQUIRE(Ns && n_segs >= 1 && n_segs <= TPPX_MAX_SEGS, TPPX_EINVAL, "%s: bad segment list", who);
  void* a = reinterpret_cast<void*>(uintptr_t(1) << 20);
  tppx_seg s[TPPX_MAX_SEGS];
  for (int i = 0; i < n_segs; i++)
    s[i] = {a, a, nullptr, nullptr, nullptr, a, Ns[i], TPPX_POST_NONE, 1.0f};
  std::string text;
  g_plan = &text;
  int rc = run_qint8(who, x_given ? a : nullptr, a, a, s, n_segs, M, K, qbs, flags, ws_bytes > 0 ? a : nullptr, ws_bytes,
                     nullptr);
  return emit_plan(who, rc, text, buf, buf_len);
}
