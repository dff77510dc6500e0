// Decode-shape (M <= 64 per block row) weight-streaming kernels.
//
// Decomposition
//   grid.x = groups * S.  A workgroup (8 waves) owns a group of 8 consecutive
//   16-channel weight tiles (one per wave) and one of S contiguous K ranges.
//   Every wave streams its own 1 KiB native tiles from HBM with one 128-bit
//   load per lane, PF loads in flight, first loads issued before anything
//   else.  The activation rows of the K range are staged once per workgroup
//   in LDS in MFMA operand order (a wave-wide ds_read_b128 is lane-contiguous,
//   conflict free) and shared by the 8 waves; for QINT8 with M <= 16 the
//   bf16 -> int8 activation quantisation happens during that staging (DPP max
//   reduction per row block), so the op is a single launch.
//   With S > 1 each wave stores its fp32 partial tile and a second, tiny
//   kernel sums the S partials in a fixed order (deterministic) and runs the
//   fused epilogue.
//   Workgroup id -> (K range = id % S, group = id / S): workgroups that share
//   an XCD (ids equal mod 8) share activation K ranges in that XCD's L2.
//
// MFMA operand convention (A = activations, B = weights):
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

__device__ __forceinline__ int find_seg(const DecodeParams& p, int grp) {
  int s = 0;
#pragma unroll
  for (int i = 1; i < TPPX_MAX_SEGS; i++)
    if (i < p.n_seg && grp >= p.seg[i].grp0)
      s = i;
  return s;
}

// max over the 64 lanes: DPP inside each row of 16, then the four row values
template <int CTRL>
__device__ __forceinline__ float dpp_max(float v) {
  int o = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true);
  return fmaxf(v, __int_as_float(o));
}
__device__ __forceinline__ float wave_absmax(float v) {
  v = dpp_max<0xB1>(v);  // quad_perm [1,0,3,2]
  v = dpp_max<0x4E>(v);  // quad_perm [2,3,0,1]
  v = dpp_max<0x141>(v); // row_half_mirror
  v = dpp_max<0x140>(v); // row_mirror
  float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

__device__ __forceinline__ int int8_rne(float v, float inv) {
  float r = rintf(__fmul_rn(v, inv));
  return (int)fminf(fmaxf(r, -127.0f), 127.0f);
}

// Cross-workgroup K reduction: with S > 1 every wave stores its fp32 partial
// tile (one 128-bit store per lane and row group, plain cached stores) and a
// second, tiny kernel sums the S partials in a fixed order (deterministic) and
// runs the fused epilogue.  The kernel boundary provides the cross-XCD
// visibility; no atomics, no fences, nobody waits.
// part layout: [ks][grid_y][tile][acc][mg][lane] x f32x4
template <int MG, int NACC>
__device__ __forceinline__ void store_partials(const DecodeParams& p, f32x4 (&acc)[NACC][MG],
                                               int gtile, int ks) {
  const int lane = threadIdx.x & 63;
  f32x4* dst = reinterpret_cast<f32x4*>(p.part) +
      ((((int64_t)ks * gridDim.y + blockIdx.y) * p.total_tiles + gtile) * NACC * MG) * 64 + lane;
#pragma unroll
  for (int a = 0; a < NACC; a++)
#pragma unroll
    for (int mg = 0; mg < MG; mg++)
      dst[(a * MG + mg) * 64] = acc[a][mg];
}

// Post-op inputs of a wave's output elements, fetched before the K reduction
// tail so that their latency overlaps it.
template <int MG>
struct PostIn {
  uint32_t in1[MG][4], in2[MG][4];
  float bias;
};

template <int MG>
__device__ __forceinline__ void prefetch_post(const DecodeParams& p, const DecodeSeg& sg, int ltile,
                                              int m0, PostIn<MG>& pi) {
  const int lane = threadIdx.x & 63;
  const int n = ltile * 16 + (lane & 15);
  pi.bias = sg.bias ? bf16_bits_to_f32(sg.bias[n]) : 0.0f;
#pragma unroll
  for (int mg = 0; mg < MG; mg++)
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int m = min(m0 + mg * 16 + (lane >> 4) * 4 + r, p.M - 1);
      const int64_t o = (int64_t)m * sg.N + n;
      pi.in1[mg][r] = sg.post_in ? sg.post_in[o] : 0u;
      pi.in2[mg][r] = sg.post_in2 ? sg.post_in2[o] : 0u;
    }
}

template <int MG>
__device__ __forceinline__ void epilogue_store(const DecodeParams& p, const DecodeSeg& sg,
                                               f32x4 (&acc)[MG], const PostIn<MG>& pi, int ltile, int m0) {
  const int lane = threadIdx.x & 63;
  const int n = ltile * 16 + (lane & 15);
#pragma unroll
  for (int mg = 0; mg < MG; mg++)
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int m = m0 + mg * 16 + (lane >> 4) * 4 + r;
      const uint32_t out = apply_post_bits(acc[mg][r] + pi.bias, sg.post_op, pi.in1[mg][r], pi.in2[mg][r],
                                           sg.post_scale);
      if (m < p.M)
        sg.y[(int64_t)m * sg.N + n] = (uint16_t)out;
    }
}

// ---------------------------------------------------------------------------
// QINT8 (W8A8): v_mfma_i32_16x16x64_i8, exact int32 sums per K block of qbs,
// then f = fma(float(acc), sa[m][b] * sw[n][b], f) in fp32.
// FUSEDQ: activations arrive as bf16 and are quantised while being staged
// (qbs == 256, one wave per (row, block): 4 values per lane).
// ---------------------------------------------------------------------------
template <int MG, bool FUSEDQ>
__global__ void __launch_bounds__(512)
decode_qint8_kernel(const DecodeParams p) {
  extern __shared__ __align__(16) uint8_t lds[];
  constexpr int PF = 8;
  constexpr int MPAD = MG * 16;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ks = blockIdx.x % p.S, grp = blockIdx.x / p.S;
  const DecodeSeg& sg = p.seg[find_seg(p, grp)];
  const int ltile = (grp - sg.grp0) * 8 + wave;
  const bool active = ltile < sg.tiles;
  const int m0 = blockIdx.y * MPAD;
  const int TPB = p.tpb;
  const int KT = p.units * TPB;
  const int u0 = (int)(((int64_t)ks * p.units) / p.S);
  const int u1 = (int)(((int64_t)(ks + 1) * p.units) / p.S);
  const int t0 = u0 * TPB, t1 = u1 * TPB;
  const int cht = p.cht;
  const int chu = cht / TPB; // whole units per chunk

  i32x4* xs = reinterpret_cast<i32x4*>(lds);                       // [cht][MG][64] x 16 B
  float* sa_s = reinterpret_cast<float*>(lds + (size_t)cht * MG * 1024); // [chu][MPAD]
  float* sw_s = sa_s + chu * MPAD;                                  // [chu][8][16]

  const i32x4* wq = reinterpret_cast<const i32x4*>(sg.qw) + (int64_t)(active ? ltile : 0) * KT * 64 + lane;
  i32x4 wreg[PF];
  auto load_w = [&](int slot, int t) {
    t = min(t, t1 - 1);
    wreg[slot] = __builtin_nontemporal_load(wq + (int64_t)t * 64);
  };
  if (active) {
#pragma unroll
    for (int i = 0; i < PF; i++)
      load_w(i, t0 + i);
  }

  f32x4 facc[1][MG];
  i32x4 iacc[MG];
#pragma unroll
  for (int mg = 0; mg < MG; mg++) {
    facc[0][mg] = f32x4{0.f, 0.f, 0.f, 0.f};
    iacc[mg] = i32x4{0, 0, 0, 0};
  }

  for (int tc = t0; tc < t1; tc += cht) {
    const int tce = min(tc + cht, t1);
    const int uc = tc / TPB, nu = (tce - tc) / TPB;
    __syncthreads();
    // ---- stage activations of tiles [tc, tce) ----
    if (FUSEDQ) {
      const int rows = min(p.M - m0, MPAD);
      const uint16_t* xb = reinterpret_cast<const uint16_t*>(p.x);
      const int nitems = rows * nu;
      for (int it0 = wave; it0 < nitems; it0 += 8 * 4) {
        uint2 raw[4];
#pragma unroll
        for (int u = 0; u < 4; u++) { // loads first: one round trip per 4 (row, block) items
          const int it = min(it0 + u * 8, nitems - 1);
          const int ul = it / rows, mr = it - ul * rows;
          raw[u] = *reinterpret_cast<const uint2*>(
              xb + (int64_t)(m0 + mr) * p.K + (int64_t)(uc + ul) * 256 + lane * 4);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
          const int it = it0 + u * 8;
          if (it < nitems) {
            const int ul = it / rows, mr = it - ul * rows;
            const float v0 = bf16_bits_to_f32(raw[u].x & 0xffffu), v1 = bf16_bits_to_f32(raw[u].x >> 16);
            const float v2 = bf16_bits_to_f32(raw[u].y & 0xffffu), v3 = bf16_bits_to_f32(raw[u].y >> 16);
            const float amax = wave_absmax(fmaxf(fmaxf(fabsf(v0), fabsf(v1)), fmaxf(fabsf(v2), fabsf(v3))));
            const float s = __fdiv_rn(amax, 127.0f); // == float(double(amax)/127.0) for bf16 amax
            const float inv = s != 0.0f ? __frcp_rn(s) : 0.0f;
            const uint32_t packed = (uint32_t)(int8_rne(v0, inv) & 0xff) | ((uint32_t)(int8_rne(v1, inv) & 0xff) << 8) |
                ((uint32_t)(int8_rne(v2, inv) & 0xff) << 16) | ((uint32_t)(int8_rne(v3, inv) & 0xff) << 24);
            // element k = lane*4.. of the block: tile lane/16, K group (lane%16)/4, byte (lane%4)*4
            const int tl = ul * 4 + (lane >> 4), mg = mr >> 4, g = (lane & 15) >> 2;
            reinterpret_cast<uint32_t*>(xs)[((tl * MG + mg) * 64 + g * 16 + (mr & 15)) * 4 + (lane & 3)] = packed;
            if (lane == 0)
              sa_s[ul * MPAD + mr] = s;
          }
        }
      }
    } else {
      const int8_t* xq = reinterpret_cast<const int8_t*>(p.xq);
      const int n16 = (tce - tc) * MG * 64;
      for (int i0 = tid; i0 < n16; i0 += 512 * 4) {
        i32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) { // loads first, LDS stores after: one round trip per 4
          const int i = min(i0 + u * 512, n16 - 1);
          const int m16 = i & 15, g = (i >> 4) & 3, mgt = i >> 6;
          const int tl = mgt / MG, mg = mgt - tl * MG;
          const int m = min(m0 + mg * 16 + m16, p.M - 1);
          v[u] = *reinterpret_cast<const i32x4*>(xq + (int64_t)m * p.K + (int64_t)(tc + tl) * 64 + g * 16);
        }
#pragma unroll
        for (int u = 0; u < 4; u++)
          if (i0 + u * 512 < n16)
            xs[i0 + u * 512] = v[u];
      }
      for (int i = tid; i < nu * MPAD; i += 512) {
        const int ul = i / MPAD, mr = i - ul * MPAD;
        sa_s[i] = p.sa[(int64_t)min(m0 + mr, p.M - 1) * p.units + uc + ul];
      }
    }
    for (int i = tid; i < nu * 128; i += 512) {
      const int ul = i >> 7, wv = (i >> 4) & 7, n = i & 15;
      const int tl = (grp - sg.grp0) * 8 + wv;
      if (tl < sg.tiles)
        sw_s[i] = reinterpret_cast<const float*>(sg.sw)[((int64_t)tl * p.units + uc + ul) * 16 + n];
    }
    __syncthreads();
    // ---- stream the weights of this chunk ----
    if (active) {
      // multiply ring slot i with tile tt; `last` = tt closes a K block
      auto consume = [&](int i, int tt, bool last, bool fast) {
        const int tl = tt - tc;
#pragma unroll
        for (int mg = 0; mg < MG; mg++)
          iacc[mg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xs[(tl * MG + mg) * 64 + lane], wreg[i], iacc[mg], 0, 0, 0);
        if (last) { // scale and fold into fp32
          const int ul = (fast ? (tt >> 2) : tt / TPB) - uc;
          const float swv = sw_s[(ul * 8 + wave) * 16 + (lane & 15)];
#pragma unroll
          for (int mg = 0; mg < MG; mg++) {
            const f32x4 sav = *reinterpret_cast<const f32x4*>(sa_s + ul * MPAD + mg * 16 + (lane >> 4) * 4);
#pragma unroll
            for (int r = 0; r < 4; r++) {
              facc[0][mg][r] = fmaf((float)iacc[mg][r], sav[r] * swv, facc[0][mg][r]);
              iacc[mg][r] = 0;
            }
          }
        }
      };
      int t = tc;
      if (TPB == 4) {
        // Full groups whose reloads are all real tiles: no branch and no load
        // other than the ring inside, so the wait counts stay exact and PF
        // tiles are really in flight (a branch in the body drains the ring).
        for (; t + PF <= tce && t + 2 * PF <= t1; t += PF) {
#pragma unroll
          for (int i = 0; i < PF; i++) {
            consume(i, t + i, (i & 3) == 3, true);
            load_w(i, t + i + PF);
          }
        }
      }
      for (; t < tce; t += PF) {
#pragma unroll
        for (int i = 0; i < PF; i++) {
          const int tt = t + i;
          if (tt < tce) {
            consume(i, tt, (tt + 1) % TPB == 0, false);
            if (tt + PF < t1)
              load_w(i, tt + PF);
          }
        }
      }
    }
  }
  if (!active)
    return;
  if (p.S > 1) {
    store_partials<MG, 1>(p, facc, sg.tile0 + ltile, ks);
    return;
  }
  PostIn<MG> pi;
  prefetch_post<MG>(p, sg, ltile, m0, pi);
  epilogue_store<MG>(p, sg, facc[0], pi, ltile, m0);
}

// ---------------------------------------------------------------------------
// MXFP4 weight-only: bf16 activations x (E2M1 * 2^e -> bf16, exact) weights,
// v_mfma_f32_16x16x32_bf16, fp32 accumulation over all of K.  One native tile
// = 16 channels x 128 K = 4 MFMAs (lane = one MX block and its scale byte).
// DUAL: the wave streams the gate tile and the up tile of the same channels
// and the epilogue is silu(gate) * up.
// ---------------------------------------------------------------------------
template <int MG, bool DUAL>
__global__ void __launch_bounds__(512)
decode_mxfp4_kernel(const DecodeParams p) {
  extern __shared__ __align__(16) uint8_t lds[];
  constexpr int PF = MG == 4 ? 4 : 8;
  constexpr int NW = DUAL ? 2 : 1;
  constexpr int MPAD = MG * 16;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ks = blockIdx.x % p.S, grp = blockIdx.x / p.S;
  const int seg_id = DUAL ? 0 : find_seg(p, grp);
  const DecodeSeg& sg = p.seg[seg_id];
  const int ltile = (grp - sg.grp0) * 8 + wave;
  const bool active = ltile < sg.tiles;
  const int m0 = blockIdx.y * MPAD;
  const int KT = p.units;
  const int t0 = (int)(((int64_t)ks * KT) / p.S);
  const int t1 = (int)(((int64_t)(ks + 1) * KT) / p.S);
  const int cht = p.cht;

  bf16x8* xs = reinterpret_cast<bf16x8*>(lds); // [cht][MG][4 j][64] x 16 B

  const i32x4* wq[NW];
  const uint8_t* wsc[NW];
#pragma unroll
  for (int s = 0; s < NW; s++) {
    const DecodeSeg& ss = p.seg[DUAL ? s : seg_id];
    const int64_t off = (int64_t)(active ? ltile : 0) * KT * 64 + lane;
    wq[s] = reinterpret_cast<const i32x4*>(ss.qw) + off;
    wsc[s] = reinterpret_cast<const uint8_t*>(ss.sw) + off;
  }
  i32x4 wreg[PF][NW];
  uint32_t sreg[PF][NW];
  auto load_w = [&](int slot, int t) {
    t = min(t, t1 - 1);
#pragma unroll
    for (int s = 0; s < NW; s++) {
      wreg[slot][s] = __builtin_nontemporal_load(wq[s] + (int64_t)t * 64);
      sreg[slot][s] = wsc[s][(int64_t)t * 64];
    }
  };
  if (active && t0 < t1) {
#pragma unroll
    for (int i = 0; i < PF; i++)
      load_w(i, t0 + i);
  }

  f32x4 acc[NW][MG];
#pragma unroll
  for (int s = 0; s < NW; s++)
#pragma unroll
    for (int mg = 0; mg < MG; mg++)
      acc[s][mg] = f32x4{0.f, 0.f, 0.f, 0.f};

  const uint16_t* xb = reinterpret_cast<const uint16_t*>(p.x);
  for (int tc = t0; tc < t1; tc += cht) {
    const int tce = min(tc + cht, t1);
    __syncthreads();
    const int n16 = (tce - tc) * MG * 256;
    for (int i0 = tid; i0 < n16; i0 += 512 * 4) {
      bf16x8 v[4];
#pragma unroll
      for (int u = 0; u < 4; u++) { // loads first, LDS stores after: one round trip per 4
        const int i = min(i0 + u * 512, n16 - 1);
        const int m16 = i & 15, g = (i >> 4) & 3, j = (i >> 6) & 3, mgt = i >> 8;
        const int tl = mgt / MG, mg = mgt - tl * MG;
        const int m = min(m0 + mg * 16 + m16, p.M - 1);
        v[u] = *reinterpret_cast<const bf16x8*>(xb + (int64_t)m * p.K + (int64_t)(tc + tl) * 128 + g * 32 + j * 8);
      }
#pragma unroll
      for (int u = 0; u < 4; u++)
        if (i0 + u * 512 < n16)
          xs[i0 + u * 512] = v[u];
    }
    __syncthreads();
    if (active) {
      auto consume = [&](int i, int tt) {
        const int tl = tt - tc;
        float sc[NW];
#pragma unroll
        for (int s = 0; s < NW; s++)
          sc[s] = e8m0_to_f32(sreg[i][s]);
#pragma unroll
        for (int j = 0; j < 4; j++) {
          bf16x8 wb[NW];
#pragma unroll
          for (int s = 0; s < NW; s++)
            wb[s] = cvt_fp4x8((uint32_t)wreg[i][s][j], sc[s]);
#pragma unroll
          for (int mg = 0; mg < MG; mg++) {
            const bf16x8 xa = xs[((tl * MG + mg) * 4 + j) * 64 + lane];
#pragma unroll
            for (int s = 0; s < NW; s++)
              acc[s][mg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa, wb[s], acc[s][mg], 0, 0, 0);
          }
        }
      };
      int t = tc;
      // Full groups whose reloads are all real tiles run without a branch in
      // the body, so the ring keeps PF tiles in flight with exact wait counts.
      for (; t + PF <= tce && t + 2 * PF <= t1; t += PF) {
#pragma unroll
        for (int i = 0; i < PF; i++) {
          consume(i, t + i);
          load_w(i, t + i + PF);
        }
      }
      for (; t < tce; t += PF) {
#pragma unroll
        for (int i = 0; i < PF; i++) {
          const int tt = t + i;
          if (tt < tce) {
            consume(i, tt);
            if (tt + PF < t1)
              load_w(i, tt + PF);
          }
        }
      }
    }
  }
  if (!active)
    return;
  if (p.S > 1) {
    store_partials<MG, NW>(p, acc, sg.tile0 + ltile, ks);
    return;
  }
  PostIn<MG> pi;
  if (!DUAL)
    prefetch_post<MG>(p, sg, ltile, m0, pi);
  if (DUAL) {
    const DecodeSeg& up = p.seg[1];
    const int n = ltile * 16 + (lane & 15);
    const float bg = sg.bias ? bf16_bits_to_f32(sg.bias[n]) : 0.0f;
    const float bu = up.bias ? bf16_bits_to_f32(up.bias[n]) : 0.0f;
#pragma unroll
    for (int mg = 0; mg < MG; mg++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int m = m0 + mg * 16 + (lane >> 4) * 4 + r;
        if (m < p.M) {
          uint32_t gact = apply_post_bits(acc[0][mg][r] + bg, TPPX_POST_SILU, 0, 0, 1.0f);
          sg.y[(int64_t)m * sg.N + n] =
              (uint16_t)apply_post_bits(acc[1][mg][r] + bu, TPPX_POST_MUL, gact, 0, 1.0f);
        }
      }
  } else {
    epilogue_store<MG>(p, sg, acc[0], pi, ltile, m0);
  }
}

// ---------------------------------------------------------------------------
// Second pass of a K-split launch: one wave per (row block, tile, row group).
// ---------------------------------------------------------------------------
template <int MG, bool DUAL>
__global__ void __launch_bounds__(256)
splitk_finish_kernel(const DecodeParams p) {
  constexpr int NACC = DUAL ? 2 : 1;
  const int lane = threadIdx.x & 63;
  const int64_t wid = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t per_y = (int64_t)p.total_tiles * MG;
  if (wid >= per_y * gridDim.y)
    return;
  const int by = (int)(wid / per_y);
  const int rem = (int)(wid - by * per_y);
  const int gtile = rem / MG, mg = rem - gtile * MG;
  int seg_id = 0;
  if (!DUAL) {
#pragma unroll
    for (int i = 1; i < TPPX_MAX_SEGS; i++)
      if (i < p.n_seg && gtile >= p.seg[i].tile0)
        seg_id = i;
  }
  const DecodeSeg& sg = p.seg[seg_id];
  const int ltile = gtile - sg.tile0;
  const int n = ltile * 16 + (lane & 15);
  const int mb = by * MG * 16 + mg * 16 + (lane >> 4) * 4;
  // post-op inputs first, so their latency overlaps the partial loads
  uint32_t in1[4] = {0, 0, 0, 0}, in2[4] = {0, 0, 0, 0};
  const float bias = sg.bias ? bf16_bits_to_f32(sg.bias[n]) : 0.0f;
  const float bias_up = (DUAL && p.seg[1].bias) ? bf16_bits_to_f32(p.seg[1].bias[n]) : 0.0f;
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const int64_t o = (int64_t)min(mb + r, p.M - 1) * sg.N + n;
    if (sg.post_in)
      in1[r] = sg.post_in[o];
    if (sg.post_in2)
      in2[r] = sg.post_in2[o];
  }
  f32x4 acc[NACC];
#pragma unroll
  for (int a = 0; a < NACC; a++)
    acc[a] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int64_t ks_stride = (int64_t)gridDim.y * p.total_tiles * NACC * MG * 64;
  const f32x4* src = reinterpret_cast<const f32x4*>(p.part) +
      (((int64_t)by * p.total_tiles + gtile) * NACC * MG + mg) * 64 + lane;
  for (int k = 0; k < p.S; k++) {
#pragma unroll
    for (int a = 0; a < NACC; a++)
      acc[a] += src[k * ks_stride + (int64_t)a * MG * 64];
  }
#pragma unroll
  for (int r = 0; r < 4; r++) {
    if (mb + r < p.M) {
      uint32_t out;
      if (DUAL) {
        uint32_t gact = apply_post_bits(acc[0][r] + bias, TPPX_POST_SILU, 0, 0, 1.0f);
        out = apply_post_bits(acc[1][r] + bias_up, TPPX_POST_MUL, gact, 0, 1.0f);
      } else {
        out = apply_post_bits(acc[0][r] + bias, sg.post_op, in1[r], in2[r], sg.post_scale);
      }
      sg.y[(int64_t)(mb + r) * sg.N + n] = (uint16_t)out;
    }
  }
}

template <int MG, bool DUAL>
static hipError_t launch_finish(const DecodeParams& p, const DecodePlan& pl, hipStream_t stream) {
  const int64_t waves = (int64_t)p.total_tiles * MG * pl.grid_y;
  TPPX_PLAN_ONLY((splitk_finish_kernel<MG, DUAL>), dim3((unsigned)((waves + 3) / 4)), dim3(256), 0);
  splitk_finish_kernel<MG, DUAL><<<dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, stream>>>(p);
  return hipGetLastError();
}

// second pass for the single-kernel paths that split K across workgroups (same partial layout, one GEMM per tile)
hipError_t launch_splitk_finish(const DecodeParams& p, int mg, int grid_y, hipStream_t stream) {
  DecodePlan pl = DecodePlan();
  pl.grid_y = grid_y;
  switch (mg) {
    case 1: return launch_finish<1, false>(p, pl, stream);
    case 2: return launch_finish<2, false>(p, pl, stream);
    default: return launch_finish<4, false>(p, pl, stream);
  }
}

// ---------------------------------------------------------------------------
// planning and launch
// ---------------------------------------------------------------------------
static const int LDS_BUDGET = 64 * 1024; // per workgroup, so that two fit on a CU

static int lcm_int(int a, int b) {
  int x = a, y = b;
  while (y) {
    int t = x % y;
    x = y;
    y = t;
  }
  return a / x * b;
}

// fmt 0 = MXFP4 (unit = one 128-K tile), 1 = QINT8 (unit = one qbs block).
DecodePlan plan_decode(int fmt, int64_t M, int groups, int total_tiles, int units, int tpb,
                       bool dual, size_t ws_bytes) {
  DecodePlan pl;
  const int mrows = (int)(M < 64 ? M : 64);
  pl.mg = mrows <= 16 ? 1 : (mrows <= 32 ? 2 : 4);
  pl.grid_y = (int)((M + 16 * pl.mg - 1) / (16 * pl.mg));
  const int pf = (fmt == 0 && pl.mg == 4) ? 4 : 8;
  const int step = fmt == 0 ? pf : lcm_int(pf, tpb);
  const int xbytes_per_tile = fmt == 0 ? pl.mg * 4096 : pl.mg * 1024;
  int cht = (LDS_BUDGET / xbytes_per_tile) / step * step;
  if (cht < step)
    cht = step;
  const int total_t = units * tpb;
  if (cht > total_t)
    cht = (total_t + step - 1) / step * step;
  pl.cht = cht;
  pl.fused_quant = (fmt == 1 && M <= 16 && tpb == 4);
  // K splits: enough workgroups to cover 256 CUs about twice
  const int nacc = dual ? 2 : 1;
  int target = env_int("TPPX_DECODE_TARGET_WGS", 512);
  int S = (target + groups * pl.grid_y - 1) / (groups * pl.grid_y);
  int env_s = env_int("TPPX_DECODE_SPLITK", 0);
  if (env_s > 0)
    S = env_s;
  if (S > units)
    S = units;
  if (S < 1)
    S = 1;
  // the workspace must hold the counters and S partial tiles per output tile
  auto need = [&](int s) {
    return (size_t)pl.grid_y * total_tiles * s * nacc * pl.mg * 256 * sizeof(float);
  };
  pl.counter_bytes = 0;
  while (S > 1 && need(S) > ws_bytes)
    S--;
  pl.S = S;
  pl.grid_x = groups * S;
  // no need to stage more than the longest K range of a split
  const int range_t = ((units + S - 1) / S) * tpb;
  if (cht > range_t)
    cht = (range_t + step - 1) / step * step;
  pl.cht = cht;
  size_t lds = (size_t)cht * xbytes_per_tile;
  if (fmt == 1) {
    int chu = cht / tpb;
    lds += (size_t)chu * pl.mg * 16 * sizeof(float) + (size_t)chu * 128 * sizeof(float);
  }
  pl.lds_bytes = lds;
  return pl;
}

template <typename K>
static hipError_t launch_k(K kern, const DecodeParams& p, const DecodePlan& pl, hipStream_t stream) {
  TPPX_PLAN_ONLY(kern, dim3(pl.grid_x, pl.grid_y), dim3(512), pl.lds_bytes);
  if (pl.lds_bytes > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)pl.lds_bytes);
    if (e != hipSuccess)
      return e;
  }
  kern<<<dim3(pl.grid_x, pl.grid_y), dim3(512), pl.lds_bytes, stream>>>(p);
  return hipGetLastError();
}

template <int MG, bool DUAL>
static hipError_t run_mxfp4_t(const DecodeParams& p, const DecodePlan& pl, hipStream_t stream) {
  hipError_t e = launch_k(decode_mxfp4_kernel<MG, DUAL>, p, pl, stream);
  if (e == hipSuccess && pl.S > 1)
    e = launch_finish<MG, DUAL>(p, pl, stream);
  return e;
}

hipError_t launch_decode_mxfp4(const DecodeParams& p, const DecodePlan& pl, bool dual, hipStream_t stream) {
  if (dual) {
    switch (pl.mg) {
      case 1: return run_mxfp4_t<1, true>(p, pl, stream);
      case 2: return run_mxfp4_t<2, true>(p, pl, stream);
      default: return run_mxfp4_t<4, true>(p, pl, stream);
    }
  }
  switch (pl.mg) {
    case 1: return run_mxfp4_t<1, false>(p, pl, stream);
    case 2: return run_mxfp4_t<2, false>(p, pl, stream);
    default: return run_mxfp4_t<4, false>(p, pl, stream);
  }
}

hipError_t launch_decode_qint8(const DecodeParams& p, const DecodePlan& pl, hipStream_t stream) {
  hipError_t e;
  if (pl.fused_quant && p.x) {
    e = launch_k(decode_qint8_kernel<1, true>, p, pl, stream);
  } else {
    switch (pl.mg) {
      case 1: e = launch_k(decode_qint8_kernel<1, false>, p, pl, stream); break;
      case 2: e = launch_k(decode_qint8_kernel<2, false>, p, pl, stream); break;
      default: e = launch_k(decode_qint8_kernel<4, false>, p, pl, stream); break;
    }
  }
  if (e == hipSuccess && pl.S > 1) {
    switch (pl.mg) {
      case 1: return launch_finish<1, false>(p, pl, stream);
      case 2: return launch_finish<2, false>(p, pl, stream);
      default: return launch_finish<4, false>(p, pl, stream);
    }
  }
  return e;
}

} // namespace tppx
