// Decode-shape ("skinny", M <= 64 per block row) weight-streaming kernels.
//
// Work decomposition: one workgroup owns NT consecutive 16-channel weight
// tiles and all of K; its waves split K into contiguous ranges, stream their
// 1 KiB native tiles straight from HBM into registers with one 128-bit load
// per lane (PF loads in flight per wave), feed them to the 16x16 MFMA with the
// activation rows as the other operand, and the per-wave fp32 partial tiles
// are summed through LDS in a fixed order (deterministic results) before the
// fused epilogue (bias, bf16 rounding, post-op) stores bf16.
//
// MFMA operand convention used throughout (A = activations, B = weights):
//   lane l supplies row/col (l & 15) and K group (l >> 4);
//   result register r of lane l is D[m = (l >> 4) * 4 + r][n = l & 15].
#include "tppx_common.h"
#include "tppx_launch.h"

namespace tppx {

__device__ __forceinline__ bf16x8 cvt_fp4x8(uint32_t codes, float scale) {
  bf16x2 c0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 0);
  bf16x2 c1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 1);
  bf16x2 c2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 2);
  bf16x2 c3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 3);
  bf16x8 w;
  w[0] = c0[0]; w[1] = c0[1]; w[2] = c1[0]; w[3] = c1[1];
  w[4] = c2[0]; w[5] = c2[1]; w[6] = c3[0]; w[7] = c3[1];
  return w;
}

__device__ __forceinline__ int find_seg(const SkinnyParams& p, int tile) {
  int s = 0;
#pragma unroll
  for (int i = 1; i < TPPX_MAX_SEGS; i++)
    if (i < p.n_seg && tile >= p.seg[i].tile0)
      s = i;
  return s;
}

// Sum the per-wave partial tiles through LDS and run the epilogue.
// red layout: [wave][(nt*MG + mg)*256 + r*64 + lane]
template <int MG, int NT, bool DUAL>
__device__ __forceinline__ void reduce_and_store(const SkinnyParams& p,
                                                 f32x4 (&acc)[NT][MG],
                                                 int seg_id, int local_tile,
                                                 int m0, float* red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int W = blockDim.x >> 6;
  constexpr int ELEMS = NT * MG * 256;
  {
    float* mine = red + wave * ELEMS;
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
      for (int mg = 0; mg < MG; mg++)
#pragma unroll
        for (int r = 0; r < 4; r++)
          mine[(nt * MG + mg) * 256 + r * 64 + lane] = acc[nt][mg][r];
    __syncthreads();
  }
  constexpr int OUT_ELEMS = DUAL ? ELEMS / 2 : ELEMS;
  for (int e = threadIdx.x; e < OUT_ELEMS; e += blockDim.x) {
    const int l = e & 63, r = (e >> 6) & 3, mg = (e >> 8) % MG;
    const int nt = (e >> 8) / MG;
    float v = 0.0f, v2 = 0.0f;
    for (int w = 0; w < W; w++)
      v += red[w * ELEMS + e];
    if (DUAL)
      for (int w = 0; w < W; w++)
        v2 += red[w * ELEMS + e + ELEMS / 2];
    const int m = m0 + mg * 16 + (l >> 4) * 4 + r;
    if (m >= p.M)
      continue;
    if (DUAL) {
      const SkinnySeg& g = p.seg[0];
      const SkinnySeg& u = p.seg[1];
      const int n = (local_tile + nt) * 16 + (l & 15);
      if (g.bias)
        v += bf16_bits_to_f32(g.bias[n]);
      if (u.bias)
        v2 += bf16_bits_to_f32(u.bias[n]);
      uint32_t gact = apply_post_bits(v, TPPX_POST_SILU, 0, 0, 1.0f);
      uint32_t out = apply_post_bits(v2, TPPX_POST_MUL, gact, 0, 1.0f);
      g.y[(int64_t)m * g.N + n] = (uint16_t)out;
    } else {
      const SkinnySeg& sg = p.seg[seg_id];
      const int n = (local_tile + nt) * 16 + (l & 15);
      const int64_t o = (int64_t)m * sg.N + n;
      if (sg.bias)
        v += bf16_bits_to_f32(sg.bias[n]);
      uint32_t in1 = sg.post_in ? sg.post_in[o] : 0u;
      uint32_t in2 = sg.post_in2 ? sg.post_in2[o] : 0u;
      sg.y[o] = (uint16_t)apply_post_bits(v, sg.post_op, in1, in2, sg.post_scale);
    }
  }
}

// ---------------------------------------------------------------------------
// MXFP4 weight-only: bf16 activations x (E2M1 * 2^e -> bf16, exact) weights,
// v_mfma_f32_16x16x32_bf16, fp32 accumulation over all of K.
// One native tile = 16 channels x 128 K = 4 MFMAs (one MX block per lane).
// ---------------------------------------------------------------------------
template <int MG, int NT, int PF, bool DUAL>
__global__ void __launch_bounds__(512)
skinny_mxfp4_kernel(const SkinnyParams p) {
  extern __shared__ float red[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int KT = p.kunits;
  constexpr int NTG = DUAL ? NT / 2 : NT; // distinct channel tiles per group
  const int tile = blockIdx.x * NTG;
  const int seg_id = DUAL ? 0 : find_seg(p, tile);
  const int local_tile = tile - p.seg[seg_id].tile0;
  const int m0 = blockIdx.y * (16 * MG);
  const int kbeg = wave * p.units_per_wave;
  const int kend = min(kbeg + p.units_per_wave, KT);

  const i32x4* wq[NT];
  const uint8_t* ws[NT];
#pragma unroll
  for (int nt = 0; nt < NT; nt++) {
    const SkinnySeg& sg = DUAL ? p.seg[nt / NTG] : p.seg[seg_id];
    const int64_t lt = local_tile + (DUAL ? nt % NTG : nt);
    wq[nt] = reinterpret_cast<const i32x4*>(sg.qw) + lt * KT * 64 + lane;
    ws[nt] = reinterpret_cast<const uint8_t*>(sg.sw) + lt * KT * 64 + lane;
  }
  const uint16_t* xrow[MG];
#pragma unroll
  for (int mg = 0; mg < MG; mg++) {
    int m = min(m0 + mg * 16 + (lane & 15), p.M - 1);
    xrow[mg] = reinterpret_cast<const uint16_t*>(p.x) + (int64_t)m * p.K + (lane >> 4) * 32;
  }

  f32x4 acc[NT][MG];
#pragma unroll
  for (int nt = 0; nt < NT; nt++)
#pragma unroll
    for (int mg = 0; mg < MG; mg++)
      acc[nt][mg] = f32x4{0.f, 0.f, 0.f, 0.f};

  i32x4 wreg[PF][NT];
  uint32_t sreg[PF][NT];
  bf16x8 xreg[PF][MG][4];

  auto load_stage = [&](int st, int kt) {
    kt = min(kt, kend - 1); // clamped: redundant but always in bounds
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      wreg[st][nt] = __builtin_nontemporal_load(wq[nt] + (int64_t)kt * 64);
      sreg[st][nt] = ws[nt][(int64_t)kt * 64];
    }
#pragma unroll
    for (int mg = 0; mg < MG; mg++)
#pragma unroll
      for (int j = 0; j < 4; j++)
        xreg[st][mg][j] = *reinterpret_cast<const bf16x8*>(xrow[mg] + kt * 128 + j * 8);
  };
  auto compute_stage = [&](int st) {
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      const float s = e8m0_to_f32(sreg[st][nt]);
      const uint32_t cw[4] = {(uint32_t)wreg[st][nt][0], (uint32_t)wreg[st][nt][1], (uint32_t)wreg[st][nt][2], (uint32_t)wreg[st][nt][3]};
#pragma unroll
      for (int j = 0; j < 4; j++) {
        bf16x8 wb = cvt_fp4x8(cw[j], s);
#pragma unroll
        for (int mg = 0; mg < MG; mg++)
          acc[nt][mg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              xreg[st][mg][j], wb, acc[nt][mg], 0, 0, 0);
      }
    }
  };

  if (kbeg < kend) {
#pragma unroll
    for (int i = 0; i < PF; i++)
      load_stage(i, kbeg + i);
    for (int kt = kbeg; kt < kend; kt += PF) {
#pragma unroll
      for (int i = 0; i < PF; i++) {
        if (kt + i < kend) {
          compute_stage(i);
          if (kt + i + PF < kend)
            load_stage(i, kt + i + PF);
        }
      }
    }
  }
  reduce_and_store<MG, NT, DUAL>(p, acc, seg_id, local_tile, m0, red);
}

// ---------------------------------------------------------------------------
// QINT8 (W8A8): int8 activations x int8 weights, v_mfma_i32_16x16x64_i8 with
// exact int32 sums per K block of qbs, then fp32 scale-and-accumulate
//   f = fma(float(acc), sa[m][b] * sw[n][b], f).
// One native tile = 16 channels x 64 K = 1 MFMA; a unit of work is one block
// of qbs/64 tiles.
// ---------------------------------------------------------------------------
template <int MG, int NT, int PF>
__global__ void __launch_bounds__(512)
skinny_qint8_kernel(const SkinnyParams p) {
  extern __shared__ float red[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int NB = p.kunits;       // K blocks of qbs
  const int TPB = p.qbs >> 6;    // tiles per block
  const int KT = NB * TPB;
  const int tile = blockIdx.x * NT;
  const int seg_id = find_seg(p, tile);
  const SkinnySeg& sg = p.seg[seg_id];
  const int local_tile = tile - sg.tile0;
  const int m0 = blockIdx.y * (16 * MG);
  const int bbeg = wave * p.units_per_wave;
  const int bend = min(bbeg + p.units_per_wave, NB);
  const int kbeg = bbeg * TPB, kend = bend * TPB;

  const i32x4* wq[NT];
  const float* ws[NT];
#pragma unroll
  for (int nt = 0; nt < NT; nt++) {
    const int64_t lt = local_tile + nt;
    wq[nt] = reinterpret_cast<const i32x4*>(sg.qw) + lt * KT * 64 + lane;
    ws[nt] = reinterpret_cast<const float*>(sg.sw) + lt * NB * 16 + (lane & 15);
  }
  const int8_t* xrow[MG];
  const float* sarow[MG][4];
#pragma unroll
  for (int mg = 0; mg < MG; mg++) {
    int m = min(m0 + mg * 16 + (lane & 15), p.M - 1);
    xrow[mg] = reinterpret_cast<const int8_t*>(p.xq) + (int64_t)m * p.K + (lane >> 4) * 16;
#pragma unroll
    for (int r = 0; r < 4; r++) {
      int mr = min(m0 + mg * 16 + (lane >> 4) * 4 + r, p.M - 1);
      sarow[mg][r] = p.sa + (int64_t)mr * NB;
    }
  }

  f32x4 facc[NT][MG];
  i32x4 iacc[NT][MG];
#pragma unroll
  for (int nt = 0; nt < NT; nt++)
#pragma unroll
    for (int mg = 0; mg < MG; mg++) {
      facc[nt][mg] = f32x4{0.f, 0.f, 0.f, 0.f};
      iacc[nt][mg] = i32x4{0, 0, 0, 0};
    }

  i32x4 wreg[PF][NT];
  i32x4 xreg[PF][MG];

  auto load_stage = [&](int st, int kt) {
    kt = min(kt, kend - 1);
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
      wreg[st][nt] = __builtin_nontemporal_load(wq[nt] + (int64_t)kt * 64);
#pragma unroll
    for (int mg = 0; mg < MG; mg++)
      xreg[st][mg] = *reinterpret_cast<const i32x4*>(xrow[mg] + kt * 64);
  };
  auto compute_stage = [&](int st, int kt) {
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
      for (int mg = 0; mg < MG; mg++)
        iacc[nt][mg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(
            xreg[st][mg], wreg[st][nt], iacc[nt][mg], 0, 0, 0);
    if ((kt + 1) % TPB == 0) { // block complete: scale and fold into fp32
      const int b = kt / TPB;
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        const float swv = ws[nt][b * 16];
#pragma unroll
        for (int mg = 0; mg < MG; mg++)
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const float s = sarow[mg][r][b] * swv;
            facc[nt][mg][r] = fmaf((float)iacc[nt][mg][r], s, facc[nt][mg][r]);
            iacc[nt][mg][r] = 0;
          }
      }
    }
  };

  if (kbeg < kend) {
#pragma unroll
    for (int i = 0; i < PF; i++)
      load_stage(i, kbeg + i);
    for (int kt = kbeg; kt < kend; kt += PF) {
#pragma unroll
      for (int i = 0; i < PF; i++) {
        if (kt + i < kend) {
          compute_stage(i, kt + i);
          if (kt + i + PF < kend)
            load_stage(i, kt + i + PF);
        }
      }
    }
  }
  reduce_and_store<MG, NT, false>(p, facc, seg_id, local_tile, m0, red);
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
template <int MG, int NT, int PF, bool DUAL>
static hipError_t launch_mxfp4_t(const SkinnyParams& p, dim3 grid, int waves,
                                 hipStream_t stream) {
  size_t lds = (size_t)waves * NT * MG * 256 * sizeof(float);
  auto kern = skinny_mxfp4_kernel<MG, NT, PF, DUAL>;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess)
      return e;
  }
  kern<<<grid, dim3(64 * waves), lds, stream>>>(p);
  return hipGetLastError();
}

template <int MG, int NT, int PF>
static hipError_t launch_qint8_t(const SkinnyParams& p, dim3 grid, int waves,
                                 hipStream_t stream) {
  size_t lds = (size_t)waves * NT * MG * 256 * sizeof(float);
  auto kern = skinny_qint8_kernel<MG, NT, PF>;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess)
      return e;
  }
  kern<<<grid, dim3(64 * waves), lds, stream>>>(p);
  return hipGetLastError();
}

// Pick (MG, NT, waves) for a problem.  total_tiles = sum of N/16 over the
// segments; kunits = K/128 (MXFP4) or K/qbs (QINT8).
SkinnyPlan plan_skinny(int64_t M, int total_tiles, int kunits, bool all_even,
                       bool dual) {
  SkinnyPlan pl;
  int mrows = (int)(M < 64 ? M : 64);
  pl.mg = mrows <= 16 ? 1 : (mrows <= 32 ? 2 : 4);
  pl.grid_y = (int)((M + 16 * pl.mg - 1) / (16 * pl.mg));
  pl.nt = 1;
  // Two channel tiles per wave halve the activation-operand traffic once the
  // activation block is as large as the weight tile it meets.
  if (!dual && all_even && pl.mg >= 2 && total_tiles >= 1024)
    pl.nt = 2;
  int env_nt = env_int("TPPX_SKINNY_NT", 0);
  if (!dual && env_nt == 1)
    pl.nt = 1;
  if (!dual && env_nt == 2 && all_even)
    pl.nt = 2;
  if (dual)
    pl.nt = 2;
  int groups = dual ? total_tiles : total_tiles / pl.nt;
  // aim for ~16 waves per CU over 256 CUs, at least 2 K units per wave
  int target_waves = 256 * 16;
  int w = (target_waves + groups * pl.grid_y - 1) / (groups * pl.grid_y);
  if (w > 8)
    w = 8;
  if (w > kunits / 2)
    w = kunits / 2;
  if (w < 1)
    w = 1;
  int env_w = env_int("TPPX_SKINNY_WAVES", 0);
  if (env_w > 0)
    w = env_w > 8 ? 8 : env_w;
  if (w > kunits)
    w = kunits;
  pl.units_per_wave = (kunits + w - 1) / w;
  pl.waves = (kunits + pl.units_per_wave - 1) / pl.units_per_wave;
  pl.grid_x = groups;
  return pl;
}

hipError_t launch_skinny_mxfp4(const SkinnyParams& p, const SkinnyPlan& pl,
                               bool dual, hipStream_t stream) {
  dim3 grid(pl.grid_x, pl.grid_y);
  if (dual) {
    switch (pl.mg) {
      case 1: return launch_mxfp4_t<1, 2, 4, true>(p, grid, pl.waves, stream);
      case 2: return launch_mxfp4_t<2, 2, 2, true>(p, grid, pl.waves, stream);
      default: return launch_mxfp4_t<4, 2, 1, true>(p, grid, pl.waves, stream);
    }
  }
  if (pl.nt == 2) {
    switch (pl.mg) {
      case 1: return launch_mxfp4_t<1, 2, 4, false>(p, grid, pl.waves, stream);
      case 2: return launch_mxfp4_t<2, 2, 2, false>(p, grid, pl.waves, stream);
      default: return launch_mxfp4_t<4, 2, 1, false>(p, grid, pl.waves, stream);
    }
  }
  switch (pl.mg) {
    case 1: return launch_mxfp4_t<1, 1, 4, false>(p, grid, pl.waves, stream);
    case 2: return launch_mxfp4_t<2, 1, 2, false>(p, grid, pl.waves, stream);
    default: return launch_mxfp4_t<4, 1, 1, false>(p, grid, pl.waves, stream);
  }
}

hipError_t launch_skinny_qint8(const SkinnyParams& p, const SkinnyPlan& pl,
                               hipStream_t stream) {
  dim3 grid(pl.grid_x, pl.grid_y);
  if (pl.nt == 2) {
    switch (pl.mg) {
      case 1: return launch_qint8_t<1, 2, 4>(p, grid, pl.waves, stream);
      case 2: return launch_qint8_t<2, 2, 4>(p, grid, pl.waves, stream);
      default: return launch_qint8_t<4, 2, 4>(p, grid, pl.waves, stream);
    }
  }
  switch (pl.mg) {
    case 1: return launch_qint8_t<1, 1, 4>(p, grid, pl.waves, stream);
    case 2: return launch_qint8_t<2, 1, 4>(p, grid, pl.waves, stream);
    default: return launch_qint8_t<4, 1, 4>(p, grid, pl.waves, stream);
  }
}

} // namespace tppx
